// Router prologue of the FlashMoE block for gfx950, fused with the product-key top-k:
//   q = BatchNorm1d(x)  (affine=False; batch statistics in training mode, running statistics otherwise)
//   logits = q Wr^T     [T, 2*nk]
//   log-softmax per half, top-k over the pair sums, exp / renormalise   (router_topk_kernel, logits-input mode)
//
// Launches, 16-bit activations (three in training mode, two in evaluation mode):
//   bn_block_stats_kernel  per (row block, 128-byte column strip): shifted sums -> (mean, M2) of the block   [training]
//   router_gate_kernel     MFMA GEMM.  Its prologue combines the (at most 16) row blocks per column (Chan's parallel
//                          formula) into mean and 1/sqrt(var+eps) - or takes the running statistics - for the columns
//                          it multiplies, and a few workgroups also store them and update the running statistics
//                          (momentum, unbiased variance) and the batch counter.  The A tile is normalised while it is
//                          staged: (x - mean) * rstd is rounded to the activation dtype exactly as a stand-alone
//                          batch-norm would emit it, then multiplied with the gate weights with fp32 accumulation;
//                          writes the logits in fp32 (for the routing) and in the activation dtype (the tensor the
//                          module returns).  With at most one tile per compute unit (4096 tokens) a workgroup is 16
//                          waves: four groups that each take every fourth k-tile and add their accumulators at the end
//   router_topk_kernel     (fmoe_router.hip)
// fp32 activations (a parity configuration, not tuned): bn_partial_kernel per (row block, 512-column strip),
// bn_finalize_kernel per column, router_gate_f32_kernel, router_topk_kernel.
#include <math.h>

#include <mutex>

#include "fmoe_common.h"
#include "fmoe_mfma.h"
#include "fmoe_vec.h"

// Scratch of fmoe_router_forward_noalloc: the batch-norm partials and the mean / 1/std vectors of one call, for hidden sizes
// up to kNoAllocMaxHidden.  Every GPU the library runs on holds its own copy at its own address for the life of the
// process; host code reaches it only through the address hipGetSymbolAddress returns for the current device.
#define FMOE_NOALLOC_MAX_HIDDEN 2048
#define FMOE_NOALLOC_SCRATCH_BYTES (256 * 3 * FMOE_NOALLOC_MAX_HIDDEN * 4 + 2 * FMOE_NOALLOC_MAX_HIDDEN * 4)
static __device__ __align__(256) unsigned char scratch[FMOE_NOALLOC_SCRATCH_BYTES];

namespace fmoe {
namespace {

constexpr int kStatsThreads = 256;
constexpr int kMaxRowBlocks = 256;
static_assert(kMaxRowBlocks * 3 * FMOE_NOALLOC_MAX_HIDDEN * 4 % 256 == 0, "the static scratch holds the largest plan exactly");

// Device address of `scratch` on the current device, looked up once per device.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

int static_scratch(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error("fmoe_router_forward_noalloc: no usable current device (%s)", hipGetErrorString(e));
        return e != hipSuccess ? (int)e : FMOE_ERR_UNSUPPORTED;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr) {
            set_error("fmoe_router_forward_noalloc: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
            return e != hipSuccess ? (int)e : FMOE_ERR_UNSUPPORTED;
        }
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return FMOE_OK;
}

// Block (rb, strip): rows [rb*rows_per_block, ...), columns strip*64*V + lane*V .. +V; the 4 waves take rows 4 apart.
// Sums are taken relative to the block's first row (pivot) so that var = E[d^2] - E[d]^2 does not cancel.
// partial: [row_blocks][3][H] = (mean, M2, n).
template <typename T>
__global__ __launch_bounds__(kStatsThreads) void bn_partial_kernel(const T* __restrict__ x, int64_t num_tokens, int hidden,
                                                                  int rows_per_block, float* __restrict__ partial) {
    constexpr int V = Elem<T>::kVec;
    __shared__ float red[3][2][kWave * V];   // waves 1..3 -> wave 0
    const int lane = lane_id(), wave = (int)(threadIdx.x >> 6);
    const int col = ((int)blockIdx.y * kWave + lane) * V;
    const bool col_ok = col < hidden;
    const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
    const int64_t r1 = r0 + rows_per_block < num_tokens ? r0 + rows_per_block : num_tokens;
    float pivot[V], s1[V], s2[V];
    {
        u32x4_t raw = {0u, 0u, 0u, 0u};
        if (col_ok) raw = *reinterpret_cast<const u32x4_t*>(x + r0 * hidden + col);
        unpack16<T>(raw, pivot);
    }
#pragma unroll
    for (int v = 0; v < V; ++v) s1[v] = s2[v] = 0.0f;
    if (col_ok) {
        // rows in batches of kBatch loads issued together (one memory round trip per batch); rows past the end are
        // read from the last row and left out of the sums
        constexpr int kBatch = 8;
        for (int64_t rb = r0 + wave; rb < r1; rb += 4 * kBatch) {
            u32x4_t raw[kBatch];
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                const int64_t r = rb + 4 * i;
                raw[i] = *reinterpret_cast<const u32x4_t*>(x + (r < r1 ? r : r1 - 1) * hidden + col);
            }
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                if (rb + 4 * i < r1) {
                    float xv[V];
                    unpack16<T>(raw[i], xv);
#pragma unroll
                    for (int v = 0; v < V; ++v) {
                        const float d = xv[v] - pivot[v];
                        s1[v] += d;
                        s2[v] = __builtin_fmaf(d, d, s2[v]);
                    }
                }
            }
        }
    }
    // waves 1..3 hand their sums (same pivot) to wave 0 through LDS
    if (wave > 0) {
#pragma unroll
        for (int v = 0; v < V; ++v) {
            red[wave - 1][0][lane * V + v] = s1[v];
            red[wave - 1][1][lane * V + v] = s2[v];
        }
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (int w = 0; w < 3; ++w)
#pragma unroll
            for (int v = 0; v < V; ++v) {
                s1[v] += red[w][0][lane * V + v];
                s2[v] += red[w][1][lane * V + v];
            }
    }
    if (wave == 0 && col_ok) {
        const float n = (float)(r1 - r0);
        float* out = partial + (int64_t)blockIdx.x * 3 * hidden;
#pragma unroll
        for (int v = 0; v < V; ++v) {
            const float m = s1[v] / n;
            out[col + v] = pivot[v] + m;
            out[hidden + col + v] = fmaxf(s2[v] - s1[v] * m, 0.0f);
            out[2 * hidden + col + v] = n;
        }
    }
}

// Statistics for the gate kernel's own prologue: few, tall row blocks, so that a gate workgroup can combine them itself.
// Block (rb, strip): rows [rb*rows_per_block, ...), 8*V columns (one 128-byte line per row for 16-bit elements).  A wave's
// load covers 8 rows (lanes 8 apart hold the same columns); the 4 waves take rows 8 apart.  Sums are relative to the
// block's first row, as in bn_partial_kernel.  partial: [row_blocks][2][H] = (mean, M2); the row count of a block follows
// from the geometry.
constexpr int kFoldMaxRowBlocks = 16;
template <typename T>
__global__ __launch_bounds__(kStatsThreads) void bn_block_stats_kernel(const T* __restrict__ x, int64_t num_tokens, int hidden,
                                                                      int rows_per_block, float* __restrict__ partial) {
    constexpr int V = Elem<T>::kVec;
    __shared__ float red[3][2][8 * V];
    const int lane = lane_id(), wave = (int)(threadIdx.x >> 6);
    const int sub = lane >> 3;                                   // which of the 8 rows of a load
    const int col = ((int)blockIdx.y * 8 + (lane & 7)) * V;
    const bool col_ok = col < hidden;
    const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
    const int64_t r1 = r0 + rows_per_block < num_tokens ? r0 + rows_per_block : num_tokens;
    float pivot[V], s1[V], s2[V];
    {
        u32x4_t raw = {0u, 0u, 0u, 0u};
        if (col_ok) raw = *reinterpret_cast<const u32x4_t*>(x + r0 * hidden + col);
        unpack16<T>(raw, pivot);
    }
#pragma unroll
    for (int v = 0; v < V; ++v) s1[v] = s2[v] = 0.0f;
    if (col_ok) {
        constexpr int kBatch = 8;                                // loads issued together: one memory round trip per batch
        for (int64_t rb = r0 + wave * 8 + sub; rb < r1; rb += 32 * kBatch) {
            u32x4_t raw[kBatch];
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                const int64_t r = rb + 32 * i;
                raw[i] = *reinterpret_cast<const u32x4_t*>(x + (r < r1 ? r : r1 - 1) * hidden + col);
            }
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                if (rb + 32 * i < r1) {
                    float xv[V];
                    unpack16<T>(raw[i], xv);
#pragma unroll
                    for (int v = 0; v < V; ++v) {
                        const float d = xv[v] - pivot[v];
                        s1[v] += d;
                        s2[v] = __builtin_fmaf(d, d, s2[v]);
                    }
                }
            }
        }
    }
    // the 8 row lanes of a wave (lane distance 8, 16, 32), then waves 1..3 -> wave 0 through LDS; fixed order
#pragma unroll
    for (int v = 0; v < V; ++v) {
#pragma unroll
        for (int m = 8; m < kWave; m <<= 1) {
            s1[v] += __shfl_xor(s1[v], m, kWave);
            s2[v] += __shfl_xor(s2[v], m, kWave);
        }
    }
    if (wave > 0 && lane < 8) {
#pragma unroll
        for (int v = 0; v < V; ++v) {
            red[wave - 1][0][lane * V + v] = s1[v];
            red[wave - 1][1][lane * V + v] = s2[v];
        }
    }
    __syncthreads();
    if (wave == 0 && lane < 8 && col_ok) {
#pragma unroll
        for (int w = 0; w < 3; ++w)
#pragma unroll
            for (int v = 0; v < V; ++v) {
                s1[v] += red[w][0][lane * V + v];
                s2[v] += red[w][1][lane * V + v];
            }
        const float n = (float)(r1 - r0);
        float* out = partial + (int64_t)blockIdx.x * 2 * hidden;
#pragma unroll
        for (int v = 0; v < V; ++v) {
            const float m = s1[v] / n;
            out[col + v] = pivot[v] + m;
            out[hidden + col + v] = fmaxf(s2[v] - s1[v] * m, 0.0f);
        }
    }
}

// Running statistics live in any of the three dtypes; the gate kernel is not instantiated per statistics dtype.
__device__ inline float load_stat_rt(const void* p, int i, int dtype) {
    switch (dtype) {
        case FMOE_F32: return ((const float*)p)[i];
        case FMOE_BF16: return Elem<bf16_t>::to_f32(((const bf16_t*)p)[i]);
        default: return Elem<f16_t>::to_f32(((const f16_t*)p)[i]);
    }
}
__device__ inline void store_stat_rt(void* p, int i, float v, int dtype) {
    switch (dtype) {
        case FMOE_F32: ((float*)p)[i] = v; break;
        case FMOE_BF16: ((bf16_t*)p)[i] = Elem<bf16_t>::from_f32(v); break;
        default: ((f16_t*)p)[i] = Elem<f16_t>::from_f32(v); break;
    }
}

// What the gate kernel's prologue needs to turn block statistics (or running statistics) into mean and 1/std.
struct GateStats {
    const float* partial;          // [row_blocks][2][H] from bn_block_stats_kernel (training)
    int row_blocks, rows_per_block;
    int64_t num_tokens;
    int training, stats_dtype;
    int ready;                     // mean_rstd already holds the statistics (a finalize launch ran): just stage them
    float momentum, eps;
    void* running_mean;
    void* running_var;
    int64_t* num_batches_tracked;
    float* mean_rstd;              // [2][H]: kept for a backward pass
};

template <typename TS> __device__ inline float load_stat(const void* p, int i) { return Elem<TS>::to_f32(((const TS*)p)[i]); }
template <typename TS> __device__ inline void store_stat(void* p, int i, float v) { ((TS*)p)[i] = Elem<TS>::from_f32(v); }

// 64 columns per block, 16 waves: wave w takes row-block partials w, w+16, ... (at most kMaxRowBlocks/16 = 16, all
// loaded before any is used so that one memory round trip covers them).  Two passes: N = sum n_b and
// mean = sum n_b*mean_b / N, then M2 = sum [M2_b + n_b*(mean_b - mean)^2].
// training: batch statistics; else the running statistics.  mean_rstd: [2][H] fp32.
constexpr int kFinalizeWaves = 16;
template <typename TS>
__global__ __launch_bounds__(kFinalizeWaves* kWave) void bn_finalize_kernel(
    const float* __restrict__ partial, int row_blocks, int hidden, int training, float momentum, float eps,
    void* running_mean, void* running_var, int64_t* num_batches_tracked, float* __restrict__ mean_rstd) {
    constexpr int PER = kMaxRowBlocks / kFinalizeWaves;
    __shared__ float red[kFinalizeWaves][2][kWave];
    const int lane = lane_id(), wave = (int)(threadIdx.x >> 6);
    const int h = (int)blockIdx.x * kWave + lane;
    if (blockIdx.x == 0 && threadIdx.x == 0 && training && num_batches_tracked != nullptr) *num_batches_tracked += 1;
    const bool h_ok = h < hidden;
    float mean = 0.0f, m2 = 0.0f, n = 0.0f;
    if (training) {
        float mb[PER], m2b[PER], nb[PER];
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int b = wave + i * kFinalizeWaves;
            const bool ok = h_ok && b < row_blocks;
            const float* p = partial + (int64_t)(ok ? b : 0) * 3 * hidden + (h_ok ? h : 0);
            mb[i] = ok ? p[0] : 0.0f;
            m2b[i] = ok ? p[hidden] : 0.0f;
            nb[i] = ok ? p[2 * hidden] : 0.0f;
        }
        float sn = 0.0f, snm = 0.0f;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            sn += nb[i];
            snm = __builtin_fmaf(nb[i], mb[i], snm);
        }
        red[wave][0][lane] = sn;
        red[wave][1][lane] = snm;
        __syncthreads();
        float tn = 0.0f, tnm = 0.0f;
#pragma unroll
        for (int w = 0; w < kFinalizeWaves; ++w) {
            tn += red[w][0][lane];
            tnm += red[w][1][lane];
        }
        n = tn;
        mean = tnm / fmaxf(tn, 1.0f);
        __syncthreads();
        float sm2 = 0.0f;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const float d = mb[i] - mean;
            sm2 += __builtin_fmaf(nb[i] * d, d, m2b[i]);
        }
        red[wave][0][lane] = sm2;
        __syncthreads();
#pragma unroll
        for (int w = 0; w < kFinalizeWaves; ++w) m2 += red[w][0][lane];
    }
    if (wave != 0 || !h_ok) return;
    float var;
    if (training) {
        var = m2 / n;                                   // biased: what normalises the batch
        if (running_mean != nullptr && running_var != nullptr) {
            const float unbiased = n > 1.0f ? m2 / (n - 1.0f) : var;
            store_stat<TS>(running_mean, h, (1.0f - momentum) * load_stat<TS>(running_mean, h) + momentum * mean);
            store_stat<TS>(running_var, h, (1.0f - momentum) * load_stat<TS>(running_var, h) + momentum * unbiased);
        }
    } else {
        mean = load_stat<TS>(running_mean, h);
        var = load_stat<TS>(running_var, h);
    }
    mean_rstd[h] = mean;
    mean_rstd[hidden + h] = 1.0f / sqrtf(var + eps);
}

// q = round_T((x - mean) * rstd) for one 16-byte packet
template <typename T> __device__ inline u32x4_t normalise16(u32x4_t raw, const float* mean, const float* rstd);
template <> __device__ inline u32x4_t normalise16<bf16_t>(u32x4_t raw, const float* mean, const float* rstd) {
    float v[8];
    unpack16<bf16_t>(raw, v);
    u32x4_t out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const bf16x2_t p = {(bf16_t)((v[2 * i] - mean[2 * i]) * rstd[2 * i]), (bf16_t)((v[2 * i + 1] - mean[2 * i + 1]) * rstd[2 * i + 1])};
        out[i] = __builtin_bit_cast(uint32_t, p);
    }
    return out;
}
template <> __device__ inline u32x4_t normalise16<f16_t>(u32x4_t raw, const float* mean, const float* rstd) {
    float v[8];
    unpack16<f16_t>(raw, v);
    u32x4_t out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const f16x2_t p = {(f16_t)((v[2 * i] - mean[2 * i]) * rstd[2 * i]), (f16_t)((v[2 * i + 1] - mean[2 * i + 1]) * rstd[2 * i + 1])};
        out[i] = __builtin_bit_cast(uint32_t, p);
    }
    return out;
}

// logits[M, N] = normalise(x)[M, K] * W[N, K]^T for 16-bit activations: 64x64 tiles (256 of them at T=4096, 2*nk=256),
// 4 waves of one 32x32 MFMA tile each, register-staged LDS tiles (the A tile is normalised between the global load and
// the LDS store).  With one such workgroup per CU nothing else hides the global-load latency, so the packets of the
// next kGatePrefetch k-tiles are kept in flight in registers.
constexpr int kGatePrefetch = 3;
constexpr int kGateMaxK = 8192;     // mean / rstd of all k are staged in LDS once: 2 * 4 * K bytes

// split != 0: half h of the outputs (columns [h*N/2, (h+1)*N/2)) scores only half h of the normalised activations,
// w is [N, K/2]: the product-key form in which each sub-key table sees its own half of the query (a block-diagonal gate).
// KG > 1: the k-tiles are dealt to KG groups of four waves (group g takes k-tiles g, g + KG, ...), each with LDS tiles
// and an accumulator of its own, and the groups' accumulators are added in group order through LDS at the end.  With
// 256 tiles for 256 compute units a tile's k loop is a chain of global-load latencies; KG = 4 runs four of them side by
// side on the same compute unit.  The result depends on KG (another summation order), not on anything else.
template <typename T, int KG>
__global__ __launch_bounds__(256 * KG) __attribute__((amdgpu_waves_per_eu(4, 4))) void router_gate_kernel(const T* __restrict__ x, const T* __restrict__ w, GateStats st,
                                                          float* __restrict__ logits32, T* __restrict__ logits, int M, int N,
                                                          int K_full, int tiles_m, int tiles_n, int split, int xcds) {
    using Frag = typename Mfma32<T>::Frag;
    constexpr int BM = 64, BN = 64, CH = 2;   // CH = 16-byte packets per thread per tile and operand
    constexpr int D = KG > 1 ? 4 : kGatePrefetch;
    constexpr int THREADS = 256 * KG;
    __shared__ __attribute__((aligned(16))) T tiles[KG][2][BM * kTileK];
    extern __shared__ __attribute__((aligned(16))) float stats[];   // [2][Kpad]: mean, rstd
    int tm, tn;
    tile_of_block(tiles_m, tiles_n, xcds, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int tid_all = (int)threadIdx.x;
    const int grp = __builtin_amdgcn_readfirstlane(tid_all / 256);
    const int tid = tid_all % 256, lane = tid & 63, wave = tid >> 6;
    T* As = tiles[grp][0];
    T* Bs = tiles[grp][1];
    const int wm = wave >> 1, wn = wave & 1;
    const int ch = tid % kTileChunks;          // this thread's packet column inside a k-tile: the same for all its packets
    const int row0 = tid / kTileChunks;        // rows row0 and row0 + 32
    const u32x4_t zero4 = {0u, 0u, 0u, 0u};
    // the k range of this tile: all of it, or the half of the activations its columns score (tiles do not straddle halves)
    const int K = split ? K_full / 2 : K_full;
    const int k_off = (split && n0 >= N / 2) ? K : 0;
    const int k_tiles = (K + kTileK - 1) / kTileK;
    const int kpad = k_tiles * kTileK;
    const int steps = (k_tiles + KG - 1) / KG;         // k-tile of step s in this group: grp + s * KG
    u32x4_t ra[D][CH], rb[D][CH];

    auto load_global = [&](int step, int slot) {
        const int kt = grp + step * KG;
        const int gk = kt * kTileK + ch * 8;
        const bool k_ok = kt < k_tiles && gk < K;
#pragma unroll
        for (int it = 0; it < CH; ++it) {
            const int gm = m0 + row0 + it * 32, gn = n0 + row0 + it * 32;
            ra[slot][it] = (gm < M && k_ok) ? *reinterpret_cast<const u32x4_t*>(x + (int64_t)gm * K_full + k_off + gk) : zero4;
            rb[slot][it] = (gn < N && k_ok) ? *reinterpret_cast<const u32x4_t*>(w + (int64_t)gn * K + gk) : zero4;
        }
    };
    auto store_lds = [&](int step, int slot) {
        const int kt = grp + step * KG;
        const float* mu = stats + (kt < k_tiles ? kt : 0) * kTileK + ch * 8;     // a step beyond the range multiplies zeros
        const float* rs = mu + kpad;
        float m8[8], r8[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            m8[i] = mu[i];
            r8[i] = rs[i];
        }
#pragma unroll
        for (int it = 0; it < CH; ++it) {
            *reinterpret_cast<u32x4_t*>(&As[swizzled_offset(row0 + it * 32, ch)]) =
                kt < k_tiles ? normalise16<T>(ra[slot][it], m8, r8) : zero4;
            *reinterpret_cast<u32x4_t*>(&Bs[swizzled_offset(row0 + it * 32, ch)]) = rb[slot][it];
        }
    };
    f32x16_t acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
    const int frow = lane & 31, fhalf = lane >> 5;
    // with k groups the operands of the first steps are requested before the statistics are combined: the two latencies overlap
    // (of the first two steps: the block statistics need the other registers)
    if (KG > 1) {
#pragma unroll
        for (int d = 0; d < 2; ++d) load_global(d, d);
    }
    // mean and 1/std of this tile's k range into LDS.  One column of tiles per k range also stores them (for a backward
    // pass) and updates the running statistics: tile row (i / 64) mod tiles_m takes column i, so every column is written
    // by exactly one workgroup.  CPT columns per thread and round: all their block statistics are loaded together (one
    // memory round trip per round), before the operand prefetch below claims its registers.
    {
        constexpr int CPT = KG > 1 ? 1 : 2;
        const bool keeper = tn == (k_off ? tiles_n / 2 : 0);
        if (blockIdx.x == 0 && tid_all == 0 && st.training && !st.ready && st.num_batches_tracked != nullptr) *st.num_batches_tracked += 1;
        const float n = (float)st.num_tokens;
        const float full = (float)st.rows_per_block;
        const float last = (float)(st.num_tokens - (int64_t)(st.row_blocks - 1) * st.rows_per_block);
        for (int i0 = tid_all; st.ready && i0 < kpad; i0 += THREADS) {
            stats[i0] = i0 < K ? st.mean_rstd[k_off + i0] : 0.0f;
            stats[kpad + i0] = i0 < K ? st.mean_rstd[K_full + k_off + i0] : 0.0f;
        }
        for (int i0 = tid_all; !st.ready && i0 < kpad; i0 += THREADS * CPT) {
            float mean[CPT], var[CPT], m2[CPT];
            if (st.training) {
                float mb[CPT][kFoldMaxRowBlocks], m2b[CPT][kFoldMaxRowBlocks];
#pragma unroll
                for (int u = 0; u < CPT; ++u) {
                    const int i = i0 + u * THREADS;
                    const float* pc = st.partial + k_off + (i < K ? i : 0);
#pragma unroll
                    for (int b = 0; b < kFoldMaxRowBlocks; ++b) {
                        const bool ok = b < st.row_blocks;
                        mb[u][b] = ok ? pc[(int64_t)b * 2 * K_full] : 0.0f;
                        m2b[u][b] = ok ? pc[(int64_t)b * 2 * K_full + K_full] : 0.0f;
                    }
                }
#pragma unroll
                for (int u = 0; u < CPT; ++u) {
                    float snm = 0.0f;
#pragma unroll
                    for (int b = 0; b < kFoldMaxRowBlocks; ++b) {
                        const float nb = b + 1 < st.row_blocks ? full : (b + 1 == st.row_blocks ? last : 0.0f);
                        snm = __builtin_fmaf(nb, mb[u][b], snm);
                    }
                    mean[u] = snm / n;
                    float acc2 = 0.0f;
#pragma unroll
                    for (int b = 0; b < kFoldMaxRowBlocks; ++b) {
                        const float nb = b + 1 < st.row_blocks ? full : (b + 1 == st.row_blocks ? last : 0.0f);
                        const float d = mb[u][b] - mean[u];
                        acc2 += __builtin_fmaf(nb * d, d, m2b[u][b]);
                    }
                    m2[u] = acc2;
                    var[u] = acc2 / n;                              // biased: what normalises the batch
                }
            } else {
#pragma unroll
                for (int u = 0; u < CPT; ++u) {
                    const int i = i0 + u * THREADS;
                    const int c = k_off + (i < K ? i : 0);
                    mean[u] = load_stat_rt(st.running_mean, c, st.stats_dtype);
                    var[u] = load_stat_rt(st.running_var, c, st.stats_dtype);
                    m2[u] = 0.0f;
                }
            }
#pragma unroll
            for (int u = 0; u < CPT; ++u) {
                const int i = i0 + u * THREADS;
                if (i >= kpad) continue;
                const int c = k_off + i;
                const float rstd = 1.0f / sqrtf(var[u] + st.eps);
                if (i < K && keeper && tm == (i / 64) % tiles_m) {
                    if (st.training && st.running_mean != nullptr && st.running_var != nullptr) {
                        const float unbiased = n > 1.0f ? m2[u] / (n - 1.0f) : var[u];
                        store_stat_rt(st.running_mean, c, (1.0f - st.momentum) * load_stat_rt(st.running_mean, c, st.stats_dtype) + st.momentum * mean[u], st.stats_dtype);
                        store_stat_rt(st.running_var, c, (1.0f - st.momentum) * load_stat_rt(st.running_var, c, st.stats_dtype) + st.momentum * unbiased, st.stats_dtype);
                    }
                    st.mean_rstd[c] = mean[u];
                    st.mean_rstd[K_full + c] = rstd;
                }
                stats[i] = i < K ? mean[u] : 0.0f;
                stats[kpad + i] = i < K ? rstd : 0.0f;
            }
        }
    }
#pragma unroll
    for (int d = KG > 1 ? 2 : 0; d < D; ++d) load_global(d, d);
    __syncthreads();               // stats[] visible
    // the step loop is unrolled by D so that the register slot of a tile is a compile-time index; every group runs every
    // step (a step beyond its k-tiles multiplies zeros), so the barriers are reached by all waves
    for (int s0 = 0; s0 < steps; s0 += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int step = s0 + d;
            if (step < steps) {
                store_lds(step, d);
                load_global(step + D, d);        // slot d is free again
                __syncthreads();
#pragma unroll
                for (int ks = 0; ks < kTileK / 16; ++ks) {
                    const int chunk = ks * 2 + fhalf;
                    const Frag fa = *reinterpret_cast<const Frag*>(&As[swizzled_offset(wm * 32 + frow, chunk)]);
                    const Frag fb = *reinterpret_cast<const Frag*>(&Bs[swizzled_offset(wn * 32 + frow, chunk)]);
                    acc = Mfma32<T>::run(fa, fb, acc);
                }
                __syncthreads();
            }
        }
    }
    if (KG > 1) {
        // groups 1 .. KG-1 hand their accumulators over through the tile memory; group 0 adds them in group order
        float* red = reinterpret_cast<float*>(&tiles[0][0][0]);
        static_assert(KG == 1 || (KG - 1) * BM * BN * sizeof(float) <= sizeof(tiles), "reduction fits the tile memory");
        if (grp > 0) {
#pragma unroll
            for (int v = 0; v < 16; ++v) red[(grp - 1) * BM * BN + (wave * 16 + v) * kWave + lane] = acc[v];
        }
        __syncthreads();
        if (grp > 0) return;
#pragma unroll
        for (int g = 1; g < KG; ++g)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[v] += red[(g - 1) * BM * BN + (wave * 16 + v) * kWave + lane];
    }
    const int col = n0 + wn * 32 + frow;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * 32 + 8 * (v / 4) + 4 * fhalf + (v % 4);
        if (row < M && col < N) {
            logits32[(int64_t)row * N + col] = acc[v];
            logits[(int64_t)row * N + col] = Elem<T>::from_f32(acc[v]);
        }
    }
}

// fp32 activations (the small parity configuration): plain FMA, 64x64 tile, 4x4 outputs per thread.
__global__ __launch_bounds__(256) void router_gate_f32_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                              const float* __restrict__ mean_rstd,
                                                              float* __restrict__ logits32, float* __restrict__ logits,
                                                              int M, int N, int K_full, int split) {
    constexpr int TS = 64, KS = 16;
    __shared__ float As[KS][TS + 1];
    __shared__ float Bs[KS][TS + 1];
    const int m0 = blockIdx.y * TS, n0 = blockIdx.x * TS;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    const int K = split ? K_full / 2 : K_full;              // split: the tile's columns score one half of the activations
    const int k_off = (split && n0 >= N / 2) ? K : 0;
    const float* mean = mean_rstd + k_off;
    const float* rstd = mean_rstd + K_full + k_off;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += KS) {
        for (int q = threadIdx.x; q < TS * KS; q += 256) {
            const int r = q / KS, kk = q % KS, gk = k0 + kk;
            As[kk][r] = (m0 + r < M && gk < K) ? (x[(int64_t)(m0 + r) * K_full + k_off + gk] - mean[gk]) * rstd[gk] : 0.0f;
            Bs[kk][r] = (n0 + r < N && gk < K) ? w[(int64_t)(n0 + r) * K + gk] : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                a[i] = As[kk][ty * 4 + i];
                b[i] = Bs[kk][tx * 4 + i];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = m0 + ty * 4 + i, col = n0 + tx * 4 + j;
            if (row < M && col < N) {
                logits32[(int64_t)row * N + col] = acc[i][j];
                logits[(int64_t)row * N + col] = acc[i][j];
            }
        }
}

// q = round_T((x - mean) * rstd), 16 bytes per thread: the normalised activations as a stand-alone batch-norm emits them,
// for the gate product on the shared MLP's tiled kernel (many tokens).  mean_rstd: [2][hidden].
template <typename T>
__global__ __launch_bounds__(256) void bn_apply_kernel(const u32x4_t* __restrict__ x, const float* __restrict__ mean_rstd,
                                                       u32x4_t* __restrict__ q, int64_t packets, int hidden) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= packets) return;
    const int col = (int)(i % (hidden / 8)) * 8;
    float m8[8], r8[8];
#pragma unroll
    for (int v = 0; v < 8; ++v) {
        m8[v] = mean_rstd[col + v];
        r8[v] = mean_rstd[hidden + col + v];
    }
    q[i] = normalise16<T>(x[i], m8, r8);
}

struct ProloguePlan {
    int row_blocks, rows_per_block;
    size_t off_partial, off_mean_rstd, off_q, base_bytes, bytes;
    bool tiled_gate;     // enough tokens for the gate product to run on 256 x 256 tiles from a normalised copy of x
};

ProloguePlan plan_prologue(int64_t T_, int H, int nk) {
    ProloguePlan p;
    int64_t rb = (T_ + 31) / 32;
    p.row_blocks = (int)(rb < 1 ? 1 : (rb > kMaxRowBlocks ? kMaxRowBlocks : rb));
    p.rows_per_block = (int)((T_ + p.row_blocks - 1) / p.row_blocks);
    p.row_blocks = (int)((T_ + p.rows_per_block - 1) / p.rows_per_block);
    p.off_partial = 0;
    p.off_mean_rstd = round_up((size_t)kMaxRowBlocks * 3 * (size_t)H * 4, 256);
    p.base_bytes = round_up(p.off_mean_rstd + 2 * (size_t)H * 4, 256);
    // the normalised copy (16-bit activations; callers whose workspace stops at base_bytes keep the 64 x 64 gate kernel)
    p.tiled_gate = gemm_nt_dual_usable(T_, 2 * nk, H);
    p.off_q = p.base_bytes;
    p.bytes = p.base_bytes + (p.tiled_gate ? round_up((size_t)T_ * (size_t)H * 2, 256) : 0);
    return p;
}

// Row blocks of the statistics the gate kernel combines itself: at most kFoldMaxRowBlocks, at least 128 rows each.
struct BlockStatsPlan { int row_blocks, rows_per_block; };
BlockStatsPlan plan_block_stats(int64_t T_) {
    BlockStatsPlan p;
    int64_t rb = (T_ + 127) / 128;
    rb = rb < 1 ? 1 : (rb > kFoldMaxRowBlocks ? kFoldMaxRowBlocks : rb);
    p.rows_per_block = (int)((T_ + rb - 1) / rb);
    p.row_blocks = (int)((T_ + p.rows_per_block - 1) / p.rows_per_block);
    return p;
}

template <typename T>
void launch_block_stats(const void* x, int64_t T_, int H, const BlockStatsPlan& p, float* partial, hipStream_t stream) {
    constexpr int V = Elem<T>::kVec;
    const int strips = (H + 8 * V - 1) / (8 * V);
    hipLaunchKernelGGL((bn_block_stats_kernel<T>), dim3((unsigned)p.row_blocks, (unsigned)strips), dim3(kStatsThreads), 0, stream,
                       (const T*)x, T_, H, p.rows_per_block, partial);
}

template <typename T>
void launch_stats(const void* x, int64_t T_, int H, const ProloguePlan& p, float* partial, hipStream_t stream) {
    constexpr int V = Elem<T>::kVec;
    const int strips = (H + kWave * V - 1) / (kWave * V);
    hipLaunchKernelGGL((bn_partial_kernel<T>), dim3((unsigned)p.row_blocks, (unsigned)strips), dim3(kStatsThreads), 0, stream,
                       (const T*)x, T_, H, p.rows_per_block, partial);
}

template <typename TS>
void launch_finalize(const float* partial, const ProloguePlan& p, int H, int training, float momentum, float eps,
                     void* rm, void* rv, int64_t* nbt, float* mean_rstd, hipStream_t stream) {
    hipLaunchKernelGGL((bn_finalize_kernel<TS>), dim3((unsigned)((H + kWave - 1) / kWave)), dim3(kFinalizeWaves * kWave), 0, stream, partial,
                       p.row_blocks, H, training, momentum, eps, rm, rv, nbt, mean_rstd);
}

// ------------------------------------------------------------------------------------------------------------
// Backward of the prologue (batch norm + gate product), for the differentiable composition of the block.
//   d   = dlogits (fp32) rounded to the activation dtype          q = round((x - mean) * rstd)     [recomputed]
//   dWr = d^T q,  dq = d Wr                                        (library GEMMs)
//   dx  = rstd * (dq - mean_t(dq) - xhat * mean_t(dq * xhat))      (training; xhat unrounded)   |   rstd * dq  (evaluation)
// ------------------------------------------------------------------------------------------------------------
// Workgroup b: row b / col_blocks of q (and of d), packets (b % col_blocks) * 256 + thread of that row.
template <typename T>
__global__ __launch_bounds__(256) void prologue_bwd_prepare_kernel(const float* __restrict__ dlogits, const T* __restrict__ x,
                                                                  const float* __restrict__ mean_rstd, T* __restrict__ d16,
                                                                  T* __restrict__ q, int hidden, int n_out, int col_blocks) {
    constexpr int V = Elem<T>::kVec;
    const uint32_t row = blockIdx.x / (uint32_t)col_blocks;
    const int pc = (int)(blockIdx.x % (uint32_t)col_blocks) * 256 + (int)threadIdx.x;
    const int col = pc * V;
    if (col < hidden) {
        const int64_t at = (int64_t)row * hidden + col;
        float xv[V], qv[V];
        unpack16<T>(*reinterpret_cast<const u32x4_t*>(x + at), xv);
#pragma unroll
        for (int h = 0; h < V / 4; ++h) {
            const f32x4_t m = *reinterpret_cast<const f32x4_t*>(mean_rstd + col + 4 * h);
            const f32x4_t r = *reinterpret_cast<const f32x4_t*>(mean_rstd + hidden + col + 4 * h);
#pragma unroll
            for (int j = 0; j < 4; ++j) qv[4 * h + j] = (xv[4 * h + j] - m[j]) * r[j];
        }
        *reinterpret_cast<u32x4_t*>(q + at) = pack16<T>(qv);
    }
    if (col < n_out) {
        const int64_t at = (int64_t)row * n_out + col;
        if (n_out % V == 0) {
            float dv[V];
#pragma unroll
            for (int h = 0; h < V / 4; ++h) {
                const f32x4_t g = *reinterpret_cast<const f32x4_t*>(dlogits + at + 4 * h);
#pragma unroll
                for (int j = 0; j < 4; ++j) dv[4 * h + j] = g[j];
            }
            *reinterpret_cast<u32x4_t*>(d16 + at) = pack16<T>(dv);
        } else {
            // rows of d that are not a whole number of 16-byte packets (2*nk not a multiple of V): element by element
            for (int j = 0; j < V && col + j < n_out; ++j) d16[at + j] = Elem<T>::from_f32(dlogits[at + j]);
        }
    }
}

// The same two tensors for the K-contiguous form of dWr = d^T q: d16 [T, N] as before (the A operand of dq = d Wr) plus the
// transposes dT [N, T] and qT [H, T], written through a 64 x 64 LDS tile so that both sides of the kernel move 16-byte
// packets.  Tile (tokens t0..t0+63) x (64 columns of q or of d); the column tiles of q come first.  Needs T, H and N to be
// multiples of 64 and 16-bit elements.
template <typename T>
__global__ __launch_bounds__(256) void prologue_bwd_prepare_transposed_kernel(
    const float* __restrict__ dlogits, const T* __restrict__ x, const float* __restrict__ mean_rstd, T* __restrict__ d16,
    T* __restrict__ dT, T* __restrict__ qT, int64_t num_tokens, int hidden, int n_out) {
    __shared__ T tile[64][64 + 2];          // [column][token], rows padded by one dword against bank conflicts
    const int q_tiles = hidden / 64;
    const int ct = (int)blockIdx.y;
    const bool is_q = ct < q_tiles;
    const int c0 = (is_q ? ct : ct - q_tiles) * 64;
    const int64_t t0 = (int64_t)blockIdx.x * 64;
    const int tid = (int)threadIdx.x;
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int idx = it * 256 + tid, r = idx >> 3, pk = idx & 7;      // token row r, packet pk (8 columns) of the tile
        const int col = c0 + pk * 8;
        float v[8];
        if (is_q) {
            float xv[8];
            unpack16<T>(*reinterpret_cast<const u32x4_t*>(x + (t0 + r) * hidden + col), xv);
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const f32x4_t m = *reinterpret_cast<const f32x4_t*>(mean_rstd + col + 4 * h);
                const f32x4_t rs = *reinterpret_cast<const f32x4_t*>(mean_rstd + hidden + col + 4 * h);
#pragma unroll
                for (int j = 0; j < 4; ++j) v[4 * h + j] = (xv[4 * h + j] - m[j]) * rs[j];
            }
        } else {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const f32x4_t g = *reinterpret_cast<const f32x4_t*>(dlogits + (t0 + r) * n_out + col + 4 * h);
#pragma unroll
                for (int j = 0; j < 4; ++j) v[4 * h + j] = g[j];
            }
            *reinterpret_cast<u32x4_t*>(d16 + (t0 + r) * n_out + col) = pack16<T>(v);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) tile[pk * 8 + j][r] = Elem<T>::from_f32(v[j]);
    }
    __syncthreads();
    T* out = is_q ? qT : dT;
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int idx = it * 256 + tid, c = idx >> 3, pk = idx & 7;      // column c of the tile, tokens pk*8 .. pk*8+7
        u32x4_t w;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t lo = __builtin_bit_cast(uint16_t, tile[c][pk * 8 + 2 * j]);
            const uint32_t hi = __builtin_bit_cast(uint16_t, tile[c][pk * 8 + 2 * j + 1]);
            w[j] = lo | (hi << 16);
        }
        *reinterpret_cast<u32x4_t*>(out + (int64_t)(c0 + c) * num_tokens + t0 + pk * 8) = w;
    }
}

// partial: [row_blocks][2][H] = (sum dq, sum dq * xhat) over the block's rows; same geometry as bn_partial_kernel.
template <typename T>
__global__ __launch_bounds__(kStatsThreads) void bn_bwd_partial_kernel(const T* __restrict__ x, const T* __restrict__ dq,
                                                                      const float* __restrict__ mean_rstd, int64_t num_tokens,
                                                                      int hidden, int rows_per_block, float* __restrict__ partial) {
    constexpr int V = Elem<T>::kVec;
    __shared__ float red[3][2][kWave * V];
    const int lane = lane_id(), wave = (int)(threadIdx.x >> 6);
    const int col = ((int)blockIdx.y * kWave + lane) * V;
    const bool col_ok = col < hidden;
    const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
    const int64_t r1 = r0 + rows_per_block < num_tokens ? r0 + rows_per_block : num_tokens;
    float mean[V], rstd[V], s1[V], s2[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        mean[v] = col_ok ? mean_rstd[col + v] : 0.0f;
        rstd[v] = col_ok ? mean_rstd[hidden + col + v] : 0.0f;
        s1[v] = s2[v] = 0.0f;
    }
    if (col_ok) {
        for (int64_t r = r0 + wave; r < r1; r += 4) {
            float xv[V], gv[V];
            unpack16<T>(*reinterpret_cast<const u32x4_t*>(x + r * hidden + col), xv);
            unpack16<T>(*reinterpret_cast<const u32x4_t*>(dq + r * hidden + col), gv);
#pragma unroll
            for (int v = 0; v < V; ++v) {
                s1[v] += gv[v];
                s2[v] = __builtin_fmaf(gv[v], (xv[v] - mean[v]) * rstd[v], s2[v]);
            }
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int v = 0; v < V; ++v) {
            red[wave - 1][0][lane * V + v] = s1[v];
            red[wave - 1][1][lane * V + v] = s2[v];
        }
    }
    __syncthreads();
    if (wave == 0 && col_ok) {
        float* out = partial + (int64_t)blockIdx.x * 2 * hidden;
#pragma unroll
        for (int v = 0; v < V; ++v) {
            float a = s1[v], b = s2[v];
#pragma unroll
            for (int w = 0; w < 3; ++w) {
                a += red[w][0][lane * V + v];
                b += red[w][1][lane * V + v];
            }
            out[col + v] = a;
            out[hidden + col + v] = b;
        }
    }
}

// sums[0][c] = sum over row blocks of partial[.][0][c] / T, sums[1][c] likewise: the two column means of the formula.
// The loads of 16 row blocks are issued together (independent accumulators), so a column costs a few memory round trips.
__global__ __launch_bounds__(256) void bn_bwd_finalize_kernel(const float* __restrict__ partial, int row_blocks, int hidden,
                                                              float inv_tokens, float* __restrict__ sums) {
    const int c = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (c >= 2 * hidden) return;
    float acc[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) acc[u] = 0.0f;
    for (int b0 = 0; b0 < row_blocks; b0 += 16) {
        float got[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const int b = b0 + u < row_blocks ? b0 + u : row_blocks - 1;      // clamped: every load is unconditional
            got[u] = partial[(int64_t)b * 2 * hidden + c];
        }
#pragma unroll
        for (int u = 0; u < 16; ++u) acc[u] += b0 + u < row_blocks ? got[u] : 0.0f;
    }
    float a = 0.0f;
#pragma unroll
    for (int u = 0; u < 16; ++u) a += acc[u];
    sums[c] = a * inv_tokens;
}

template <typename T>
__global__ __launch_bounds__(256) void bn_bwd_apply_kernel(const T* __restrict__ x, const T* __restrict__ dq,
                                                           const float* __restrict__ mean_rstd, const float* __restrict__ sums,
                                                           T* __restrict__ dx, int hidden, int col_blocks, int training) {
    constexpr int V = Elem<T>::kVec;
    const uint32_t row = blockIdx.x / (uint32_t)col_blocks;
    const int col = ((int)(blockIdx.x % (uint32_t)col_blocks) * 256 + (int)threadIdx.x) * V;
    if (col >= hidden) return;
    const int64_t at = (int64_t)row * hidden + col;
    float xv[V], gv[V], ov[V], mean[V], rstd[V], m1[V], m2[V];
    unpack16<T>(*reinterpret_cast<const u32x4_t*>(x + at), xv);
    unpack16<T>(*reinterpret_cast<const u32x4_t*>(dq + at), gv);
    // the four per-column vectors as 16-byte loads, all requested before any is used
#pragma unroll
    for (int h = 0; h < V / 4; ++h) {
        const f32x4_t a = *reinterpret_cast<const f32x4_t*>(mean_rstd + col + 4 * h);
        const f32x4_t b = *reinterpret_cast<const f32x4_t*>(mean_rstd + hidden + col + 4 * h);
        const f32x4_t c = training ? *reinterpret_cast<const f32x4_t*>(sums + col + 4 * h) : f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        const f32x4_t d = training ? *reinterpret_cast<const f32x4_t*>(sums + hidden + col + 4 * h) : f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            mean[4 * h + j] = a[j];
            rstd[4 * h + j] = b[j];
            m1[4 * h + j] = c[j];
            m2[4 * h + j] = d[j];
        }
    }
    // evaluation mode: m1 = m2 = 0 and the formula reduces to rstd * dq
#pragma unroll
    for (int v = 0; v < V; ++v) ov[v] = rstd[v] * (gv[v] - m1[v] - (xv[v] - mean[v]) * rstd[v] * m2[v]);
    *reinterpret_cast<u32x4_t*>(dx + at) = pack16<T>(ov);
}

struct PrologueBwdPlan {
    size_t off_d16, off_dT, off_q, off_dq, off_partial, off_sums, bytes;
};

PrologueBwdPlan plan_prologue_backward(int64_t T_, int H, int nk, int dtype) {
    PrologueBwdPlan p;
    const size_t elt = dtype_size(dtype);
    size_t o = 0;
    auto take = [&](size_t n) { const size_t at = o; o = round_up(o + n, 256); return at; };
    p.off_d16 = take((size_t)T_ * 2 * nk * elt);
    p.off_dT = take((size_t)T_ * 2 * nk * elt);
    p.off_q = take((size_t)T_ * H * elt);
    p.off_dq = take((size_t)T_ * H * elt);
    p.off_partial = take((size_t)kMaxRowBlocks * 2 * H * 4);
    p.off_sums = take((size_t)2 * H * 4);
    p.bytes = o;
    return p;
}

template <typename T>
int launch_prologue_backward(const float* dlogits, const void* x, const void* gate_w, const float* mean_rstd, int training,
                             int64_t T_, int H, int nk, int dtype, void* dx, void* dgate_w, void* workspace, hipStream_t s) {
    constexpr int V = Elem<T>::kVec;
    const PrologueBwdPlan p = plan_prologue_backward(T_, H, nk, dtype);
    const ProloguePlan rows = plan_prologue(T_, H, nk);
    char* ws = (char*)workspace;
    T *d16 = (T*)(ws + p.off_d16), *q = (T*)(ws + p.off_q), *dq = (T*)(ws + p.off_dq);
    float *partial = (float*)(ws + p.off_partial), *sums = (float*)(ws + p.off_sums);
    const int N = 2 * nk;
    const int widest = H > N ? H : N;
    const int col_blocks = ((widest + V - 1) / V + 255) / 256;
    bool transposed = false;
    if constexpr (sizeof(T) == 2) {
        if (T_ % 64 == 0 && H % 64 == 0 && N % 64 == 0) {
            // dWr[N, H] = dT[N, T] qT[H, T]^T: both operands K-contiguous, the forward's own GEMM ("down" form)
            T* dT = (T*)(ws + p.off_dT);
            hipLaunchKernelGGL((prologue_bwd_prepare_transposed_kernel<T>), dim3((unsigned)(T_ / 64), (unsigned)((H + N) / 64)),
                               dim3(256), 0, s, dlogits, (const T*)x, mean_rstd, d16, dT, q, T_, H, N);
            FMOE_CHECK_LAUNCH("fmoe_router_prologue_backward(prepare)");
            if (int rc = fmoe_mlp_down(dT, q, N, H, (int)T_, dtype, nullptr, dgate_w, s)) return rc;
            transposed = true;
        }
    }
    if (!transposed) {
        hipLaunchKernelGGL((prologue_bwd_prepare_kernel<T>), dim3((unsigned)(T_ * col_blocks)), dim3(256), 0, s, dlogits,
                           (const T*)x, mean_rstd, d16, q, H, N, col_blocks);
        FMOE_CHECK_LAUNCH("fmoe_router_prologue_backward(prepare)");
        if (int rc = blas_gemm(kBlasTN, N, H, (int)T_, d16, N, q, H, dgate_w, H, 0.0f, dtype, s)) return rc;      // dWr = d^T q
    }
    if (int rc = blas_gemm(kBlasNN, (int)T_, H, N, d16, N, gate_w, H, dq, H, 0.0f, dtype, s)) return rc;       // dq = d Wr
    if (training) {
        const int strips = (H + kWave * V - 1) / (kWave * V);
        hipLaunchKernelGGL((bn_bwd_partial_kernel<T>), dim3((unsigned)rows.row_blocks, (unsigned)strips), dim3(kStatsThreads), 0, s,
                           (const T*)x, (const T*)dq, mean_rstd, T_, H, rows.rows_per_block, partial);
        FMOE_CHECK_LAUNCH("fmoe_router_prologue_backward(column sums)");
        hipLaunchKernelGGL(bn_bwd_finalize_kernel, dim3((unsigned)((2 * H + 255) / 256)), dim3(256), 0, s, (const float*)partial,
                           rows.row_blocks, H, 1.0f / (float)T_, sums);
        FMOE_CHECK_LAUNCH("fmoe_router_prologue_backward(finalize)");
    }
    const int apply_blocks = (H / V + 255) / 256;
    hipLaunchKernelGGL((bn_bwd_apply_kernel<T>), dim3((unsigned)(T_ * apply_blocks)), dim3(256), 0, s, (const T*)x,
                       (const T*)dq, mean_rstd, (const float*)sums, (T*)dx, H, apply_blocks, training);
    FMOE_CHECK_LAUNCH("fmoe_router_prologue_backward(apply)");
    return FMOE_OK;
}

}  // namespace
}  // namespace fmoe

extern "C" size_t fmoe_router_workspace_bytes(int64_t num_tokens, int hidden, int num_keys) {
    if (num_tokens <= 0 || hidden <= 0 || num_keys <= 0) return 0;
    return fmoe::plan_prologue(num_tokens, hidden, num_keys).bytes;
}

extern "C" int fmoe_router_forward(const void* x, const void* gate_w, void* running_mean, void* running_var,
                                   int64_t* num_batches_tracked, int stats_dtype, int training, float momentum,
                                   float eps, int64_t num_tokens, int hidden, int num_keys, int top_k, int dtype,
                                   int norm_topk_prob, void* router_logits, float* logits_fp32, float* scores,
                                   int64_t* indices, void* gates, void* workspace, size_t workspace_bytes, void* stream) {
    fmoe::clear_error();
    return fmoe::router_forward_impl(x, gate_w, running_mean, running_var, num_batches_tracked, stats_dtype, training,
                                     momentum, eps, num_tokens, hidden, num_keys, top_k, dtype, norm_topk_prob,
                                     router_logits, logits_fp32, scores, indices, gates, nullptr, 0u, workspace,
                                     workspace_bytes, (hipStream_t)stream);
}

extern "C" int fmoe_router_forward_split(const void* x, const void* sub_keys, void* running_mean, void* running_var,
                                         int64_t* num_batches_tracked, int stats_dtype, int training, float momentum,
                                         float eps, int64_t num_tokens, int hidden, int num_keys, int top_k, int dtype,
                                         int norm_topk_prob, void* router_logits, float* logits_fp32, float* scores,
                                         int64_t* indices, void* gates, void* workspace, size_t workspace_bytes, void* stream) {
    fmoe::clear_error();
    return fmoe::router_forward_impl(x, sub_keys, running_mean, running_var, num_batches_tracked, stats_dtype, training,
                                     momentum, eps, num_tokens, hidden, num_keys, top_k, dtype, norm_topk_prob,
                                     router_logits, logits_fp32, scores, indices, gates, nullptr, 0u, workspace,
                                     workspace_bytes, (hipStream_t)stream, 1);
}

extern "C" int fmoe_router_forward_noalloc(const void* x, const void* gate_w, void* running_mean, void* running_var,
                                           int64_t* num_batches_tracked, int stats_dtype, int training, float momentum,
                                           float eps, int64_t num_tokens, int hidden, int num_keys, int top_k, int dtype,
                                           int norm_topk_prob, void* router_logits, float* logits_fp32, float* scores,
                                           int64_t* indices, void* gates, void* stream) {
    using namespace fmoe;
    clear_error();
    FMOE_REQUIRE(hidden <= FMOE_NOALLOC_MAX_HIDDEN, FMOE_ERR_UNSUPPORTED,
                 "fmoe_router_forward_noalloc: hidden=%d exceeds the %d columns its static scratch is sized for; use "
                 "fmoe_router_forward with a workspace", hidden, FMOE_NOALLOC_MAX_HIDDEN);
    if (num_tokens <= 0 || hidden <= 0 || num_keys <= 0)   // rejected (or empty) below, before any scratch is needed
        return router_forward_impl(x, gate_w, running_mean, running_var, num_batches_tracked, stats_dtype, training, momentum,
                                   eps, num_tokens, hidden, num_keys, top_k, dtype, norm_topk_prob, router_logits, logits_fp32,
                                   scores, indices, gates, nullptr, 0u, nullptr, 0, (hipStream_t)stream);
    void* ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    return router_forward_impl(x, gate_w, running_mean, running_var, num_batches_tracked, stats_dtype, training, momentum,
                               eps, num_tokens, hidden, num_keys, top_k, dtype, norm_topk_prob, router_logits, logits_fp32,
                               scores, indices, gates, nullptr, 0u, ws, (size_t)FMOE_NOALLOC_SCRATCH_BYTES, (hipStream_t)stream, 0, 1);
}

int fmoe::router_forward_impl(const void* x, const void* gate_w, void* running_mean, void* running_var,
                              int64_t* num_batches_tracked, int stats_dtype, int training, float momentum, float eps,
                              int64_t num_tokens, int hidden, int num_keys, int top_k, int dtype, int norm_topk_prob,
                              void* router_logits, float* logits_fp32, float* scores, int64_t* indices, void* gates,
                              uint32_t* row_offsets, uint32_t row_bytes, void* workspace, size_t workspace_bytes,
                              hipStream_t s, int split_query, int fixed_scratch) {
    using namespace fmoe;
    FMOE_REQUIRE(!split_query || (num_keys % 64 == 0 && hidden % 2 == 0), FMOE_ERR_UNSUPPORTED,
                 "fmoe_router_forward_split: num_keys=%d must be a multiple of 64 and hidden=%d even", num_keys, hidden);
    FMOE_REQUIRE(dtype_ok(dtype) && dtype_ok(stats_dtype), FMOE_ERR_BAD_DTYPE,
                 "fmoe_router_forward: unknown dtype %d / statistics dtype %d", dtype, stats_dtype);
    FMOE_REQUIRE(num_tokens >= 0 && hidden > 0 && num_keys > 0, FMOE_ERR_BAD_SHAPE,
                 "fmoe_router_forward: bad shape T=%lld H=%d nk=%d", (long long)num_tokens, hidden, num_keys);
    FMOE_REQUIRE(top_k >= 0 && top_k <= num_keys, FMOE_ERR_TOPK_RANGE,
                 "num_experts_per_tok should be in [0, %d], but got %d", num_keys, top_k);
    FMOE_REQUIRE(dtype == FMOE_F32 || hidden <= kGateMaxK, FMOE_ERR_UNSUPPORTED,
                 "fmoe_router_forward: hidden=%d > %d for 16-bit activations", hidden, kGateMaxK);
    FMOE_REQUIRE(num_keys <= 32767 && router_topk_supported(num_keys, top_k) && num_tokens < (1ll << 31), FMOE_ERR_UNSUPPORTED,
                 "fmoe_router_forward: nk=%d top_k=%d T=%lld beyond what the kernels are built for", num_keys, top_k,
                 (long long)num_tokens);
    if (num_tokens == 0) return FMOE_OK;
    FMOE_REQUIRE(!(training && num_tokens == 1), FMOE_ERR_BAD_SHAPE,
                 "Expected more than 1 value per channel when training, got input size [1, %d]", hidden);
    FMOE_REQUIRE(x && gate_w && router_logits && logits_fp32 && workspace, FMOE_ERR_NULL_POINTER,
                 "fmoe_router_forward: null tensor pointer");
    FMOE_REQUIRE(top_k == 0 || (scores && indices), FMOE_ERR_NULL_POINTER, "fmoe_router_forward: null scores/indices");
    FMOE_REQUIRE(training || (running_mean && running_var), FMOE_ERR_NULL_POINTER,
                 "fmoe_router_forward: evaluation mode needs running statistics");
    const int vec = (int)(16 / dtype_size(dtype));
    FMOE_REQUIRE(hidden % (split_query ? 2 * vec : vec) == 0 && aligned16(x) && aligned16(gate_w), FMOE_ERR_ALIGNMENT,
                 "fmoe_router_forward: hidden=%d must be a multiple of %d and tensors 16-byte aligned", hidden,
                 split_query ? 2 * vec : vec);
    const ProloguePlan p = plan_prologue(num_tokens, hidden, num_keys);
    // a workspace without room for the normalised copy (the fixed scratch of the no-allocation entry point) takes the
    // 64 x 64 gate kernel: the same sums in the same order
    const bool tiled_gate = p.tiled_gate && dtype != FMOE_F32 && !split_query && !fixed_scratch;
    const size_t need = fixed_scratch ? p.base_bytes : p.bytes;
    FMOE_REQUIRE(workspace_bytes >= need && aligned16(workspace), FMOE_ERR_WORKSPACE,
                 "fmoe_router_forward: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    char* ws = (char*)workspace;
    float* partial = (float*)(ws + p.off_partial);
    float* mean_rstd = (float*)(ws + p.off_mean_rstd);
    float* logits32 = logits_fp32;

    const int M = (int)num_tokens, N = 2 * num_keys;
    if (dtype == FMOE_F32) {
        if (training) {
            launch_stats<float>(x, num_tokens, hidden, p, partial, s);
            FMOE_CHECK_LAUNCH("fmoe_router_forward(batch statistics)");
        }
        switch (stats_dtype) {
            case FMOE_F32: launch_finalize<float>(partial, p, hidden, training, momentum, eps, running_mean, running_var, num_batches_tracked, mean_rstd, s); break;
            case FMOE_BF16: launch_finalize<bf16_t>(partial, p, hidden, training, momentum, eps, running_mean, running_var, num_batches_tracked, mean_rstd, s); break;
            default: launch_finalize<f16_t>(partial, p, hidden, training, momentum, eps, running_mean, running_var, num_batches_tracked, mean_rstd, s); break;
        }
        FMOE_CHECK_LAUNCH("fmoe_router_forward(finalize)");
        hipLaunchKernelGGL(router_gate_f32_kernel, dim3((N + 63) / 64, (M + 63) / 64), dim3(256), 0, s, (const float*)x,
                           (const float*)gate_w, (const float*)mean_rstd, logits32, (float*)router_logits, M, N, hidden, split_query);
    } else {
        const BlockStatsPlan bp = plan_block_stats(num_tokens);
        const int tiles_m = (M + 63) / 64, tiles_n = (N + 63) / 64;
        // Every gate workgroup combining the block statistics itself saves a launch, but repeats the combination per
        // tile: with more than a couple of tiles per CU one finalize launch is cheaper.
        const bool fold = (int64_t)tiles_m * tiles_n <= 2 * (int64_t)chip_info().cus;
        if (fold && training) {
            if (dtype == FMOE_BF16) launch_block_stats<bf16_t>(x, num_tokens, hidden, bp, partial, s);
            else launch_block_stats<f16_t>(x, num_tokens, hidden, bp, partial, s);
            FMOE_CHECK_LAUNCH("fmoe_router_forward(batch statistics)");
        }
        if (!fold) {
            if (training) {
                if (dtype == FMOE_BF16) launch_stats<bf16_t>(x, num_tokens, hidden, p, partial, s);
                else launch_stats<f16_t>(x, num_tokens, hidden, p, partial, s);
                FMOE_CHECK_LAUNCH("fmoe_router_forward(batch statistics)");
            }
            switch (stats_dtype) {
                case FMOE_F32: launch_finalize<float>(partial, p, hidden, training, momentum, eps, running_mean, running_var, num_batches_tracked, mean_rstd, s); break;
                case FMOE_BF16: launch_finalize<bf16_t>(partial, p, hidden, training, momentum, eps, running_mean, running_var, num_batches_tracked, mean_rstd, s); break;
                default: launch_finalize<f16_t>(partial, p, hidden, training, momentum, eps, running_mean, running_var, num_batches_tracked, mean_rstd, s); break;
            }
            FMOE_CHECK_LAUNCH("fmoe_router_forward(finalize)");
        }
        if (tiled_gate) {
            // fold is false here (at least one 256 x 256 tile per compute unit): mean and 1/std are in the workspace
            void* q = ws + p.off_q;
            const int64_t packets = num_tokens * (int64_t)(hidden / 8);
            if (dtype == FMOE_BF16)
                hipLaunchKernelGGL((bn_apply_kernel<bf16_t>), dim3((unsigned)((packets + 255) / 256)), dim3(256), 0, s,
                                   (const u32x4_t*)x, (const float*)mean_rstd, (u32x4_t*)q, packets, hidden);
            else
                hipLaunchKernelGGL((bn_apply_kernel<f16_t>), dim3((unsigned)((packets + 255) / 256)), dim3(256), 0, s,
                                   (const u32x4_t*)x, (const float*)mean_rstd, (u32x4_t*)q, packets, hidden);
            FMOE_CHECK_LAUNCH("fmoe_router_forward(normalise)");
            if (int rc = gemm_nt_dual(q, gate_w, router_logits, logits32, M, N, hidden, dtype, s)) return rc;
            if (top_k == 0) return FMOE_OK;
            return launch_router_from_logits(logits32, num_tokens, num_keys, top_k, scores, indices, gates, dtype, norm_topk_prob,
                                             row_offsets, row_bytes, s);
        }
        GateStats st;
        st.ready = fold ? 0 : 1;
        st.partial = partial;
        st.row_blocks = bp.row_blocks;
        st.rows_per_block = bp.rows_per_block;
        st.num_tokens = num_tokens;
        st.training = training;
        st.stats_dtype = stats_dtype;
        st.momentum = momentum;
        st.eps = eps;
        st.running_mean = running_mean;
        st.running_var = running_var;
        st.num_batches_tracked = num_batches_tracked;
        st.mean_rstd = mean_rstd;
        const size_t stats_bytes = (size_t)((hidden + kTileK - 1) / kTileK) * kTileK * 2 * sizeof(float);
        // few tiles with a long k loop: four k groups per workgroup, two for up to two tiles per compute unit; many tiles
        // already fill the chip
        const bool k_groups = (int64_t)tiles_m * tiles_n <= chip_info().cus && (split_query ? hidden / 2 : hidden) >= 8 * kTileK;
#define FMOE_LAUNCH_GATE(TT, KG)                                                                                            \
    hipLaunchKernelGGL((router_gate_kernel<TT, KG>), dim3((unsigned)(tiles_m * tiles_n)), dim3(256 * KG), stats_bytes, s,  \
                       (const TT*)x, (const TT*)gate_w, st, logits32, (TT*)router_logits, M, N, hidden, tiles_m, tiles_n,   \
                       split_query, chip_info().xcds)
        const bool k_pairs = !k_groups && (int64_t)tiles_m * tiles_n <= 2 * chip_info().cus && (split_query ? hidden / 2 : hidden) >= 8 * kTileK;
        if (dtype == FMOE_BF16) {
            if (k_groups) FMOE_LAUNCH_GATE(bf16_t, 4);
            else if (k_pairs) FMOE_LAUNCH_GATE(bf16_t, 2);
            else FMOE_LAUNCH_GATE(bf16_t, 1);
        } else {
            if (k_groups) FMOE_LAUNCH_GATE(f16_t, 4);
            else if (k_pairs) FMOE_LAUNCH_GATE(f16_t, 2);
            else FMOE_LAUNCH_GATE(f16_t, 1);
        }
#undef FMOE_LAUNCH_GATE
    }
    FMOE_CHECK_LAUNCH("fmoe_router_forward(gate)");
    if (top_k == 0) return FMOE_OK;
    return launch_router_from_logits(logits32, num_tokens, num_keys, top_k, scores, indices, gates, dtype, norm_topk_prob,
                                     row_offsets, row_bytes, s);
}

extern "C" size_t fmoe_router_workspace_stats_offset(int64_t num_tokens, int hidden, int num_keys) {
    if (num_tokens <= 0 || hidden <= 0 || num_keys <= 0) return 0;
    return fmoe::plan_prologue(num_tokens, hidden, num_keys).off_mean_rstd;
}

extern "C" size_t fmoe_router_prologue_backward_workspace_bytes(int64_t num_tokens, int hidden, int num_keys, int dtype) {
    if (num_tokens <= 0 || hidden <= 0 || num_keys <= 0 || !fmoe::dtype_ok(dtype)) return 0;
    return fmoe::plan_prologue_backward(num_tokens, hidden, num_keys, dtype).bytes;
}

extern "C" int fmoe_router_prologue_backward(const float* dlogits_fp32, const void* x, const void* gate_w, const float* mean_rstd,
                                             int training, int64_t num_tokens, int hidden, int num_keys, int dtype, void* dx,
                                             void* dgate_w, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace fmoe;
    clear_error();
    FMOE_REQUIRE(dtype_ok(dtype), FMOE_ERR_BAD_DTYPE, "fmoe_router_prologue_backward: unknown dtype %d", dtype);
    FMOE_REQUIRE(num_tokens > 0 && hidden > 0 && num_keys > 0 && num_tokens < (1ll << 24), FMOE_ERR_BAD_SHAPE,
                 "fmoe_router_prologue_backward: bad shape T=%lld H=%d nk=%d", (long long)num_tokens, hidden, num_keys);
    const int vec = (int)(16 / dtype_size(dtype));
    FMOE_REQUIRE(hidden % vec == 0, FMOE_ERR_ALIGNMENT,
                 "fmoe_router_prologue_backward: hidden=%d must be a multiple of %d", hidden, vec);
    FMOE_REQUIRE(dlogits_fp32 && x && gate_w && mean_rstd && dx && dgate_w, FMOE_ERR_NULL_POINTER,
                 "fmoe_router_prologue_backward: null tensor pointer");
    FMOE_REQUIRE(aligned16(x) && aligned16(dx) && aligned16(dlogits_fp32) && aligned16(mean_rstd), FMOE_ERR_ALIGNMENT,
                 "fmoe_router_prologue_backward: tensor pointers must be 16-byte aligned");
    const size_t need = plan_prologue_backward(num_tokens, hidden, num_keys, dtype).bytes;
    FMOE_REQUIRE(workspace && workspace_bytes >= need && aligned16(workspace), FMOE_ERR_WORKSPACE,
                 "fmoe_router_prologue_backward: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case FMOE_F32: return launch_prologue_backward<float>(dlogits_fp32, x, gate_w, mean_rstd, training, num_tokens, hidden, num_keys, dtype, dx, dgate_w, workspace, s);
        case FMOE_BF16: return launch_prologue_backward<bf16_t>(dlogits_fp32, x, gate_w, mean_rstd, training, num_tokens, hidden, num_keys, dtype, dx, dgate_w, workspace, s);
        default: return launch_prologue_backward<f16_t>(dlogits_fp32, x, gate_w, mean_rstd, training, num_tokens, hidden, num_keys, dtype, dx, dgate_w, workspace, s);
    }
}
