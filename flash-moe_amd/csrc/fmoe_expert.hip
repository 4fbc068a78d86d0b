// Routed-expert forward for gfx950:
//   out[t,:] = sum_k silu(<x[t,:], down[idx[t,k],:]>) * g[t,k] * up[idx[t,k],:]
//
// One wavefront owns one token.  The token's row of x stays in registers; for each of its K
// (expert, gate) pairs the wave streams the expert's `down` row (16 bytes per lane, 1 KiB per
// wave-wide load, fully coalesced), reduces the dot product across the 64 lanes, applies
// silu(.)*gate and streams the `up` row into fp32 accumulators.  The token's output row is
// written once at the end: no atomics, no zero-initialised output, deterministic summation order.
// Rows of several pairs are requested before any of them is consumed so that enough bytes are in
// flight to cover HBM / Infinity-Cache latency.
#include "fmoe_common.h"
#include "fmoe_vec.h"

namespace fmoe {
namespace {

// What is applied to the score <x, down[e]> before the gate: the routed experts of FlashMoE use SiLU, PEER uses the
// erf GELU, and a product-key memory has no score at all (its coefficient is the routing weight itself).
enum Activation { kActSilu = 0, kActGelu = 1, kActNone = 2 };
template <int ACT> __device__ inline float activate(float s) {
    if (ACT == kActSilu) return silu_f32(s);
    if (ACT == kActGelu) return 0.5f * s * (1.0f + erff(s * 0.70710678118654752440f));
    return 1.0f;
}

constexpr int kPairsInFlight = 4;   // (down,up) row pairs requested ahead per wave
constexpr int kWavesPerBlock = 4;

// NCH = number of 16-byte packets each lane holds per row: a row has at most NCH*64 packets.
// SPLIT = false: one wave per token, kWavesPerBlock tokens per workgroup.  SPLIT = true (few tokens): the workgroup's
// waves share one token, wave w taking pairs w*P .. w*P+P-1, (w+4)*P .. of it (P = pairs in flight), and their partial rows
// are added in wave order through LDS: four times shorter dependency chains when there are not enough tokens to fill the
// chip with one wave each.
template <typename T, int NCH, int ACT, bool SPLIT>
__global__ __launch_bounds__(kWavesPerBlock* kWave) void expert_token_kernel(
    const T* __restrict__ x, const T* __restrict__ down, const T* __restrict__ up,
    const int64_t* __restrict__ indices, const T* __restrict__ gates, T* __restrict__ out,
    int64_t num_tokens, int hidden, int64_t num_experts, int top_k) {
    constexpr int V = Elem<T>::kVec;
    const int lane = lane_id();
    const int wave = (int)(threadIdx.x >> 6);
    const int64_t token = SPLIT ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * kWavesPerBlock + wave;
    if (token >= num_tokens) return;   // whole wave leaves together (SPLIT: the whole workgroup)
    __shared__ float partial_rows[SPLIT ? (kWavesPerBlock - 1) * NCH * V * kWave : 1];

    const int packets = hidden / V;   // 16-byte packets per row (hidden % V == 0 is checked on the host)
    const u32x4_t zero4 = {0u, 0u, 0u, 0u};

    u32x4_t xr[NCH];
    bool live[NCH];
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int p = c * kWave + lane;
        live[c] = p < packets;
        xr[c] = (ACT != kActNone && live[c]) ? reinterpret_cast<const u32x4_t*>(x + token * hidden)[p] : zero4;
    }

    float acc[NCH][V];
#pragma unroll
    for (int c = 0; c < NCH; ++c)
#pragma unroll
        for (int v = 0; v < V; ++v) acc[c][v] = 0.0f;

    const int64_t* my_idx = indices + token * top_k;
    const T* my_gate = gates + token * top_k;

    const int k_first = SPLIT ? wave * kPairsInFlight : 0;
    const int k_step = SPLIT ? kWavesPerBlock * kPairsInFlight : kPairsInFlight;
    for (int k0 = k_first; k0 < top_k; k0 += k_step) {
        u32x4_t dn[kPairsInFlight][NCH];
        u32x4_t uq[kPairsInFlight][NCH];
        float gate[kPairsInFlight];
#pragma unroll
        for (int u = 0; u < kPairsInFlight; ++u) {
            const int k = k0 + u;
            int64_t e = -1;
            gate[u] = 0.0f;
            if (k < top_k) {
                e = my_idx[k];
                gate[u] = Elem<T>::to_f32(my_gate[k]);
            }
            // ids are uniform across the wave; make that visible so row addresses live in SGPRs
            const uint32_t elo = __builtin_amdgcn_readfirstlane((uint32_t)(e & 0xffffffff));
            const uint32_t ehi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)e >> 32));
            e = (int64_t)(((uint64_t)ehi << 32) | elo);
            const bool ok = e >= 0 && e < num_experts;
            if (!ok) gate[u] = 0.0f;
            const u32x4_t* drow = reinterpret_cast<const u32x4_t*>(down + (ok ? e : 0) * hidden);
            const u32x4_t* urow = reinterpret_cast<const u32x4_t*>(up + (ok ? e : 0) * hidden);
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                const int p = c * kWave + lane;
                dn[u][c] = (ACT != kActNone && ok && live[c]) ? drow[p] : zero4;
                uq[u][c] = (ok && live[c]) ? urow[p] : zero4;
            }
        }
        float s[kPairsInFlight];
#pragma unroll
        for (int u = 0; u < kPairsInFlight; ++u) {
            float part = 0.0f;
#pragma unroll
            for (int c = 0; c < NCH; ++c) part = dot16<T>(xr[c], dn[u][c], part);
            s[u] = part;
        }
        if (ACT != kActNone) {
#pragma unroll
            for (int u = 0; u < kPairsInFlight; ++u) s[u] = wave_sum(s[u]);
        }
#pragma unroll
        for (int u = 0; u < kPairsInFlight; ++u) {
            const float a = activate<ACT>(s[u]) * gate[u];
#pragma unroll
            for (int c = 0; c < NCH; ++c) axpy16<T>(a, uq[u][c], acc[c]);
        }
    }

    if (SPLIT) {
        if (wave > 0) {
#pragma unroll
            for (int c = 0; c < NCH; ++c)
#pragma unroll
                for (int v = 0; v < V; ++v) partial_rows[(((wave - 1) * NCH + c) * V + v) * kWave + lane] = acc[c][v];
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int w = 0; w < kWavesPerBlock - 1; ++w)
#pragma unroll
            for (int c = 0; c < NCH; ++c)
#pragma unroll
                for (int v = 0; v < V; ++v) acc[c][v] += partial_rows[((w * NCH + c) * V + v) * kWave + lane];
    }
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int p = c * kWave + lane;
        if (live[c]) reinterpret_cast<u32x4_t*>(out + token * hidden)[p] = pack16<T>(acc[c]);
    }
}

template <typename T>
int launch_expert_rows(int act, const void* x, const void* down, const void* up, const int64_t* indices, const void* gates,
                       int64_t T_, int H, int64_t E, int K, void* out, hipStream_t stream) {
    constexpr int V = Elem<T>::kVec;
    const int packets = H / V;
    const int nch = (packets + kWave - 1) / kWave;
    const dim3 block(kWavesPerBlock * kWave);
    // with at most 2048 tokens a workgroup per token still fits the chip at once
    const bool split = T_ <= 2048 && K > kPairsInFlight;
    const dim3 grid((unsigned)(split ? T_ : (T_ + kWavesPerBlock - 1) / kWavesPerBlock));
#define FMOE_LAUNCH_EXPERT_ACT(N, A)                                                                                  \
    do {                                                                                                              \
        if (split)                                                                                                    \
            hipLaunchKernelGGL((expert_token_kernel<T, N, A, true>), grid, block, 0, stream, (const T*)x, (const T*)down, \
                               (const T*)up, indices, (const T*)gates, (T*)out, T_, H, E, K);                         \
        else                                                                                                          \
            hipLaunchKernelGGL((expert_token_kernel<T, N, A, false>), grid, block, 0, stream, (const T*)x, (const T*)down, \
                               (const T*)up, indices, (const T*)gates, (T*)out, T_, H, E, K);                         \
    } while (0)
#define FMOE_LAUNCH_EXPERT(N)                                     \
    do {                                                          \
        if (act == kActSilu) FMOE_LAUNCH_EXPERT_ACT(N, kActSilu); \
        else if (act == kActGelu) FMOE_LAUNCH_EXPERT_ACT(N, kActGelu); \
        else FMOE_LAUNCH_EXPERT_ACT(N, kActNone);                 \
    } while (0)
    if (nch <= 1) FMOE_LAUNCH_EXPERT(1);
    else if (nch <= 2) FMOE_LAUNCH_EXPERT(2);
    else if (nch <= 4) FMOE_LAUNCH_EXPERT(4);
    else if (nch <= 8) FMOE_LAUNCH_EXPERT(8);
    else {
        set_error("fmoe_expert_forward: hidden=%d exceeds the %d elements per row this build supports", H,
                  8 * kWave * V);
        return FMOE_ERR_UNSUPPORTED;
    }
#undef FMOE_LAUNCH_EXPERT
#undef FMOE_LAUNCH_EXPERT_ACT
    FMOE_CHECK_LAUNCH("fmoe_expert_forward");
    return FMOE_OK;
}


// ------------------------------------------------------------------------------------------------
// Column-slice path.
//
// Random 2 KiB row gathers from tables of tens of MiB are served by the Infinity Cache / HBM through the
// fabric at ~7.6 TB/s on MI355X whatever the kernel does, while gathers from a working set that fits one
// XCD's 4 MiB L2 run at ~25 TB/s.  So the tables are processed in column slices of 256 bytes per row (128 for
// tables of more than 16384 rows): a slice of a 16384-row table is 4 MiB.  Workgroups are mapped so that XCD x
// works on slices x, x+8, ... one after the other (workgroup ids are dealt round-robin over the 8 XCDs), each
// slice streaming through all tokens while it stays resident in that XCD's L2; every table byte leaves HBM /
// Infinity Cache once.  A wave-wide load fetches the slice's pieces of 4 (or 8) different pairs, 16 bytes per
// lane; a round of 16 (or 8) such loads, all in flight together, covers 64 pairs.  The wider slice halves the
// passes over the offsets, coefficients and partial sums: measured 31.9 -> 27.7 us for the scores of 4096
// tokens x 64 pairs, 117 -> 102 us for 16384 tokens.
//
//   prepare : int64 ids -> int32 (-1 if outside [0,E))
//   scores  : spart[slice][pair] = <x[token, slice cols], down[expert, slice cols]>          (per slice)
//   gate    : a[pair] = silu(sum_slice spart[slice][pair]) * gate[pair]
//   states  : out[token, slice cols] = sum_k a[token,k] * up[expert_k, slice cols]           (per slice)
// `states` needs no cross-slice reduction, so the output is still written exactly once, without atomics.
// ------------------------------------------------------------------------------------------------
// A wave-wide 16-byte load covers 64 / CL rows when CL lanes share one row's chunk (CL = 8: 128-byte slices,
// CL = 16: 256-byte slices); a round of CL such loads handles 64 pairs.
constexpr uint32_t kBadOffset = kExpertBadOffset;

// Table rows are addressed through a raw buffer resource: 32-bit byte offsets (no 64-bit address arithmetic
// per load) and hardware bounds checking, so the row of an invalid id reads as zeros.
__device__ inline __amdgpu_buffer_rsrc_t table_resource(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ inline u32x4_t load_row_piece(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset) {
    return __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)byte_offset, 0, 0));
}

// ids -> byte offset of the row (kBadOffset if the id is outside [0,E))
__global__ __launch_bounds__(256) void expert_prepare_kernel(const int64_t* __restrict__ idx, uint32_t* __restrict__ off32,
                                                             int64_t n, int64_t num_experts, uint32_t row_bytes) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const int64_t e = idx[i];
        off32[i] = (e >= 0 && e < num_experts) ? (uint32_t)e * row_bytes : kBadOffset;
    }
}

__device__ inline bool slice_of_block(int num_slices, int blocks_per_slice, int& slice, int& tb) {
    const int b = (int)blockIdx.x;
    const int j = b >> 3;
    slice = (b & 7) + 8 * (j / blocks_per_slice);
    tb = j % blocks_per_slice;
    return slice < num_slices;
}

// p[u] holds, in each of the CL lanes of a chunk group, that lane's share of pair u's dot product.  Returns in
// lane c of the group the complete sum of pair u == c: a transposing butterfly (CL - 1 cross-lane adds instead of
// CL * log2(CL)).
template <int N, int STEP> __device__ inline float xor_step(float v) {
    if constexpr (STEP == 1) return dpp_move<0xB1>(v);
    else if constexpr (STEP == 2) return dpp_move<0x4E>(v);
    else if constexpr (STEP == 8) return dpp_move<0x128>(v);          // rotate the row of 16 by 8
    else return __shfl_xor(v, STEP, kWave);
}
template <int N, int STEP> __device__ inline float transpose_sum(const float (&p)[N], int c) {
    if constexpr (N == 1) {
        return p[0];
    } else {
        const bool up = c & STEP;
        float q[N / 2];
#pragma unroll
        for (int i = 0; i < N / 2; ++i) {
            const float keep = up ? p[2 * i + 1] : p[2 * i], send = up ? p[2 * i] : p[2 * i + 1];
            q[i] = keep + xor_step<N, STEP>(send);
        }
        return transpose_sum<N / 2, STEP * 2>(q, c);
    }
}

template <typename T, int CL>
__global__ __launch_bounds__(256) void expert_scores_slice_kernel(
    const T* __restrict__ x, const T* __restrict__ down, uint32_t table_bytes, const uint32_t* __restrict__ off32,
    float* __restrict__ spart, int64_t num_tokens, int hidden, int top_k, int num_slices, int blocks_per_slice,
    int tokens_per_block) {
    constexpr int V = Elem<T>::kVec;
    constexpr int PPL = kWave / CL;                         // pairs per wave-wide load
    int slice, tb;
    if (!slice_of_block(num_slices, blocks_per_slice, slice, tb)) return;
    const int lane = lane_id(), wave = (int)(threadIdx.x >> 6);
    const int c = lane & (CL - 1), pg = lane / CL;
    const int col = slice * (CL * V) + c * V;
    const bool col_ok = col < hidden;                       // false only in a partial last slice
    const uint32_t col_bytes = col_ok ? (uint32_t)col * sizeof(T) : 0u;
    const u32x4_t zero4 = {0u, 0u, 0u, 0u};
    const __amdgpu_buffer_rsrc_t rsrc = table_resource(down, table_bytes);
    const int64_t pairs = num_tokens * top_k;
    const int64_t t_begin = (int64_t)tb * tokens_per_block;
    const int64_t t_end = t_begin + tokens_per_block < num_tokens ? t_begin + tokens_per_block : num_tokens;
    float* my_spart = spart + (int64_t)slice * pairs;

    for (int64_t t = t_begin + wave; t < t_end; t += 4) {
        const u32x4_t xq = col_ok ? *reinterpret_cast<const u32x4_t*>(x + t * hidden + col) : zero4;
        const uint32_t* tok_off = off32 + t * top_k;
        for (int k0 = 0; k0 < top_k; k0 += kWave) {
            // one coalesced load brings the row offsets of 64 pairs; lane (pg, c) then needs those of pairs u*PPL+pg
            const uint32_t mine = k0 + lane < top_k ? tok_off[k0 + lane] : kBadOffset;
            u32x4_t w[CL];
#pragma unroll
            for (int u = 0; u < CL; ++u) {
                const uint32_t o = (uint32_t)__builtin_amdgcn_ds_bpermute((u * PPL + pg) * 4, (int)mine);
                w[u] = load_row_piece(rsrc, o + col_bytes);
            }
            float part[CL];
#pragma unroll
            for (int u = 0; u < CL; ++u) part[u] = dot16<T>(xq, w[u], 0.0f);
            const float total = transpose_sum<CL, 1>(part, c);      // pair k0 + c*PPL + pg
            const int kk = k0 + c * PPL + pg;
            if (kk < top_k) my_spart[t * top_k + kk] = total;
        }
    }
}

template <typename T, int ACT>
__global__ __launch_bounds__(256) void expert_gate_kernel(const float* __restrict__ spart, const T* __restrict__ gates,
                                                          const uint32_t* __restrict__ off32, float* __restrict__ a,
                                                          int64_t pairs, int num_slices) {
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= pairs) return;
    float s = 0.0f;
    for (int sl = 0; sl < num_slices; ++sl) s += spart[(int64_t)sl * pairs + p];
    a[p] = off32[p] != kBadOffset ? activate<ACT>(s) * Elem<T>::to_f32(gates[p]) : 0.0f;
}

// acc[0..kVec) += a0 * w0 + a1 * w1 for two 16-byte packets of two different rows
template <typename T> __device__ inline void axpy16_pair(float a0, float a1, u32x4_t w0, u32x4_t w1, float* acc) {
    axpy16<T>(a0, w0, acc);
    axpy16<T>(a1, w1, acc);
}
// bf16: interleave the two rows column by column and use the packed dot product, (w0[c], w1[c]) . (a0, a1);
// half the instructions of unpack + fma.  The two coefficients are rounded to bf16 for this (the reference
// forms silu(s)*g in the activation dtype as well, flash_expert.py:191).
template <> __device__ inline void axpy16_pair<bf16_t>(float a0, float a1, u32x4_t w0, u32x4_t w1, float* acc) {
    const bf16x2_t ap = {(bf16_t)a0, (bf16_t)a1};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t p0 = w0[i], p1 = w1[i];
        const uint32_t lo = __builtin_amdgcn_perm(p1, p0, 0x05040100u);   // (p0.lo16, p1.lo16)
        const uint32_t hi = __builtin_amdgcn_perm(p1, p0, 0x07060302u);   // (p0.hi16, p1.hi16)
        acc[2 * i] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, lo), ap, acc[2 * i], false);
        acc[2 * i + 1] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, hi), ap, acc[2 * i + 1], false);
    }
}

template <typename T, int CL>
__global__ __launch_bounds__(256) void expert_states_slice_kernel(
    const float* __restrict__ a, const T* __restrict__ up, uint32_t table_bytes, const uint32_t* __restrict__ off32,
    T* __restrict__ out, int64_t num_tokens, int hidden, int top_k, int num_slices, int blocks_per_slice,
    int tokens_per_block) {
    constexpr int V = Elem<T>::kVec;
    constexpr int PPL = kWave / CL;
    int slice, tb;
    if (!slice_of_block(num_slices, blocks_per_slice, slice, tb)) return;
    const int lane = lane_id(), wave = (int)(threadIdx.x >> 6);
    const int c = lane & (CL - 1), pg = lane / CL;
    const int col = slice * (CL * V) + c * V;
    const bool col_ok = col < hidden;
    const uint32_t col_bytes = col_ok ? (uint32_t)col * sizeof(T) : 0u;
    const __amdgpu_buffer_rsrc_t rsrc = table_resource(up, table_bytes);
    const int64_t t_begin = (int64_t)tb * tokens_per_block;
    const int64_t t_end = t_begin + tokens_per_block < num_tokens ? t_begin + tokens_per_block : num_tokens;

    for (int64_t t = t_begin + wave; t < t_end; t += 4) {
        const uint32_t* tok_off = off32 + t * top_k;
        const float* tok_a = a + t * top_k;
        float acc[V];
#pragma unroll
        for (int v = 0; v < V; ++v) acc[v] = 0.0f;
        for (int k0 = 0; k0 < top_k; k0 += kWave) {
            const bool live = k0 + lane < top_k;
            const uint32_t mine = live ? tok_off[k0 + lane] : kBadOffset;
            const float mine_a = live ? tok_a[k0 + lane] : 0.0f;
            u32x4_t w[CL];
            float av[CL];
#pragma unroll
            for (int u = 0; u < CL; ++u) {
                const int src = (u * PPL + pg) * 4;
                const uint32_t o = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)mine);
                av[u] = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(src, __builtin_bit_cast(int, mine_a)));
                w[u] = load_row_piece(rsrc, o + col_bytes);      // zeros for an invalid id (out of bounds)
            }
#pragma unroll
            for (int u = 0; u < CL; u += 2) axpy16_pair<T>(av[u], av[u + 1], w[u], w[u + 1], acc);
        }
        // sum the pair groups (lanes c, c+CL, c+2*CL, ... hold the same columns)
#pragma unroll
        for (int v = 0; v < V; ++v) {
            if constexpr (CL == 8) acc[v] += dpp_move<0x128>(acc[v]);             // lanes 8 apart
            acc[v] += __shfl_xor(acc[v], 16, kWave);
            acc[v] += __shfl_xor(acc[v], 32, kWave);
        }
        if (pg == 0 && col_ok) *reinterpret_cast<u32x4_t*>(out + t * hidden + col) = pack16<T>(acc);
    }
}

struct SlicePlan {
    int chunk_lanes, num_slices, blocks_per_slice, tokens_per_block;
    unsigned grid;
    size_t off_idx32, off_a, off_spart, bytes;
};

// A slice is as wide as one XCD's 4 MiB L2 can keep resident: 256 bytes per row up to 16384 rows (fewer passes over
// the offsets, coefficients and partial sums), 128 bytes beyond.
SlicePlan plan_slices(int64_t T_, int H, int64_t E, int K, size_t elt) {
    SlicePlan p;
    p.chunk_lanes = E * 256 <= (4ll << 20) ? 16 : 8;
    const size_t chunk_bytes = (size_t)p.chunk_lanes * 16;
    p.num_slices = (int)((H * elt + chunk_bytes - 1) / chunk_bytes);
    const int64_t want = (T_ + 3) / 4;                       // at least one token per wave
    p.blocks_per_slice = (int)(want < 1024 ? want : 1024);   // 256 blocks of 4 waves fill one XCD; a few rounds of them
    p.tokens_per_block = (int)((T_ + p.blocks_per_slice - 1) / p.blocks_per_slice);
    p.grid = (unsigned)(8 * p.blocks_per_slice * ((p.num_slices + 7) / 8));
    const size_t pairs = (size_t)T_ * (size_t)K;
    p.off_idx32 = 0;
    p.off_a = round_up(p.off_idx32 + pairs * 4, 256);
    p.off_spart = round_up(p.off_a + pairs * 4, 256);
    p.bytes = round_up(p.off_spart + (size_t)p.num_slices * pairs * 4, 256);
    return p;
}

template <typename T>
int launch_slice_scores(const void* x, const void* table, const uint32_t* off32, float* spart, int64_t T_, int H, int64_t E,
                        int K, hipStream_t stream) {
    const SlicePlan p = plan_slices(T_, H, E, K, sizeof(T));
    const uint32_t table_bytes = (uint32_t)(E * (int64_t)H * (int64_t)sizeof(T));
    if (p.chunk_lanes == 16)
        hipLaunchKernelGGL((expert_scores_slice_kernel<T, 16>), dim3(p.grid), dim3(256), 0, stream, (const T*)x,
                           (const T*)table, table_bytes, off32, spart, T_, H, K, p.num_slices, p.blocks_per_slice,
                           p.tokens_per_block);
    else
        hipLaunchKernelGGL((expert_scores_slice_kernel<T, 8>), dim3(p.grid), dim3(256), 0, stream, (const T*)x,
                           (const T*)table, table_bytes, off32, spart, T_, H, K, p.num_slices, p.blocks_per_slice,
                           p.tokens_per_block);
    FMOE_CHECK_LAUNCH("routed experts (slice scores)");
    return FMOE_OK;
}

template <typename T>
int launch_slice_states(const float* a, const void* table, const uint32_t* off32, void* out, int64_t T_, int H, int64_t E,
                        int K, hipStream_t stream) {
    const SlicePlan p = plan_slices(T_, H, E, K, sizeof(T));
    const uint32_t table_bytes = (uint32_t)(E * (int64_t)H * (int64_t)sizeof(T));
    if (p.chunk_lanes == 16)
        hipLaunchKernelGGL((expert_states_slice_kernel<T, 16>), dim3(p.grid), dim3(256), 0, stream, a, (const T*)table,
                           table_bytes, off32, (T*)out, T_, H, K, p.num_slices, p.blocks_per_slice, p.tokens_per_block);
    else
        hipLaunchKernelGGL((expert_states_slice_kernel<T, 8>), dim3(p.grid), dim3(256), 0, stream, a, (const T*)table,
                           table_bytes, off32, (T*)out, T_, H, K, p.num_slices, p.blocks_per_slice, p.tokens_per_block);
    FMOE_CHECK_LAUNCH("routed experts (slice states)");
    return FMOE_OK;
}

// Scores, gate and states launches on row offsets that already sit at the start of the workspace.
template <typename T>
int launch_expert_slices_prepared(int act, const void* x, const void* down, const void* up, const void* gates, int64_t T_,
                                  int H, int64_t E, int K, void* out, void* workspace, hipStream_t stream) {
    const SlicePlan p = plan_slices(T_, H, E, K, sizeof(T));
    char* ws = (char*)workspace;
    const uint32_t* off32 = (const uint32_t*)(ws + p.off_idx32);
    float* a = (float*)(ws + p.off_a);
    float* spart = (float*)(ws + p.off_spart);
    const int64_t pairs = T_ * K;
    const unsigned flat_grid = (unsigned)((pairs + 255) / 256);
    if (act != kActNone)
        if (int rc = launch_slice_scores<T>(x, down, off32, spart, T_, H, E, K, stream)) return rc;
    // without a score (product-key memory) the coefficient is the routing weight: no partial sums are read
    if (act == kActSilu)
        hipLaunchKernelGGL((expert_gate_kernel<T, kActSilu>), dim3(flat_grid), dim3(256), 0, stream, (const float*)spart,
                           (const T*)gates, off32, a, pairs, p.num_slices);
    else if (act == kActGelu)
        hipLaunchKernelGGL((expert_gate_kernel<T, kActGelu>), dim3(flat_grid), dim3(256), 0, stream, (const float*)spart,
                           (const T*)gates, off32, a, pairs, p.num_slices);
    else
        hipLaunchKernelGGL((expert_gate_kernel<T, kActNone>), dim3(flat_grid), dim3(256), 0, stream, (const float*)spart,
                           (const T*)gates, off32, a, pairs, 0);
    FMOE_CHECK_LAUNCH("fmoe_expert_forward(gate)");
    return launch_slice_states<T>(a, up, off32, out, T_, H, E, K, stream);
}

template <typename T>
int launch_expert_slices(int act, const void* x, const void* down, const void* up, const int64_t* indices, const void* gates,
                         int64_t T_, int H, int64_t E, int K, void* out, void* workspace, hipStream_t stream) {
    const SlicePlan p = plan_slices(T_, H, E, K, sizeof(T));
    uint32_t* off32 = (uint32_t*)((char*)workspace + p.off_idx32);
    const int64_t pairs = T_ * K;
    hipLaunchKernelGGL(expert_prepare_kernel, dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, stream, indices, off32,
                       pairs, E, (uint32_t)(H * sizeof(T)));
    FMOE_CHECK_LAUNCH("fmoe_expert_forward(prepare)");
    return launch_expert_slices_prepared<T>(act, x, down, up, gates, T_, H, E, K, out, workspace, stream);
}

// A slice of the table must stay resident in one XCD's 4 MiB L2 next to the streaming traffic; with 128-byte
// slices of up to 8 MiB the measured gather rate is still twice the fabric's.  Beyond that, and for problems with
// too few pairs to pay for four launches, whole rows are gathered by the one-wave-per-token kernel.
bool slices_pay(int64_t T_, int64_t E, int K) { return E * 128 <= (8ll << 20) && T_ * K >= (1ll << 16); }
// rows are addressed with 32-bit byte offsets below kBadOffset
bool slices_possible(int64_t E, int H, size_t elt) { return (uint64_t)E * (uint64_t)H * elt < (uint64_t)kBadOffset; }

}  // namespace

bool expert_slices_usable(int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype) {
    return top_k > 0 && slices_pay(num_tokens, num_experts, top_k) && slices_possible(num_experts, hidden, dtype_size(dtype));
}

uint32_t* expert_workspace_offsets(void* workspace) { return (uint32_t*)workspace; }   // SlicePlan::off_idx32 == 0

int expert_slices_prepared(const void* x, const void* down, const void* up, const void* gates, int64_t num_tokens,
                           int hidden, int64_t num_experts, int top_k, int dtype, void* out, void* workspace,
                           hipStream_t stream) {
    switch (dtype) {
        case FMOE_F32: return launch_expert_slices_prepared<float>(kActSilu, x, down, up, gates, num_tokens, hidden, num_experts, top_k, out, workspace, stream);
        case FMOE_BF16: return launch_expert_slices_prepared<bf16_t>(kActSilu, x, down, up, gates, num_tokens, hidden, num_experts, top_k, out, workspace, stream);
        default: return launch_expert_slices_prepared<f16_t>(kActSilu, x, down, up, gates, num_tokens, hidden, num_experts, top_k, out, workspace, stream);
    }
}

// The stages of the column-slice schedule one by one, for the backward pass (fmoe_backward.hip).
int expert_slice_count(int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype) {
    return plan_slices(num_tokens, hidden, num_experts, top_k, dtype_size(dtype)).num_slices;
}

int expert_slice_prepare(const int64_t* indices, uint32_t* off32, int64_t pairs, int hidden, int64_t num_experts, int dtype,
                         hipStream_t stream) {
    hipLaunchKernelGGL(expert_prepare_kernel, dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, stream, indices, off32,
                       pairs, num_experts, (uint32_t)(hidden * dtype_size(dtype)));
    FMOE_CHECK_LAUNCH("routed experts (slice offsets)");
    return FMOE_OK;
}

int expert_slice_scores(const void* x, const void* table, const uint32_t* off32, float* spart, int64_t num_tokens, int hidden,
                        int64_t num_experts, int top_k, int dtype, hipStream_t stream) {
    switch (dtype) {
        case FMOE_F32: return launch_slice_scores<float>(x, table, off32, spart, num_tokens, hidden, num_experts, top_k, stream);
        case FMOE_BF16: return launch_slice_scores<bf16_t>(x, table, off32, spart, num_tokens, hidden, num_experts, top_k, stream);
        default: return launch_slice_scores<f16_t>(x, table, off32, spart, num_tokens, hidden, num_experts, top_k, stream);
    }
}

int expert_slice_states(const float* coef, const void* table, const uint32_t* off32, void* out, int64_t num_tokens, int hidden,
                        int64_t num_experts, int top_k, int dtype, hipStream_t stream) {
    switch (dtype) {
        case FMOE_F32: return launch_slice_states<float>(coef, table, off32, out, num_tokens, hidden, num_experts, top_k, stream);
        case FMOE_BF16: return launch_slice_states<bf16_t>(coef, table, off32, out, num_tokens, hidden, num_experts, top_k, stream);
        default: return launch_slice_states<f16_t>(coef, table, off32, out, num_tokens, hidden, num_experts, top_k, stream);
    }
}

}  // namespace fmoe

extern "C" size_t fmoe_expert_workspace_bytes_algo(int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype,
                                                   int algo) {
    using namespace fmoe;
    if (num_tokens <= 0 || hidden <= 0 || num_experts <= 0 || top_k <= 0 || !dtype_ok(dtype)) return 0;
    const bool possible = slices_possible(num_experts, hidden, dtype_size(dtype));
    const bool slices = algo == FMOE_EXPERT_SLICES || (algo == FMOE_EXPERT_AUTO && possible && slices_pay(num_tokens, num_experts, top_k));
    return slices ? plan_slices(num_tokens, hidden, num_experts, top_k, dtype_size(dtype)).bytes : 0;   // the row schedule needs no scratch
}

extern "C" size_t fmoe_expert_workspace_bytes(int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype) {
    return fmoe_expert_workspace_bytes_algo(num_tokens, hidden, num_experts, top_k, dtype, FMOE_EXPERT_AUTO);
}

namespace fmoe {
namespace {

// Shared body of the three gather ops; `who` names the entry point in messages, `down` is unused for kActNone.
int expert_dispatch(const char* who, int act, const void* x, const void* down, const void* up, const int64_t* indices,
                    const void* gates, int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype, void* out,
                    void* workspace, size_t workspace_bytes, int algo, void* stream) {
    clear_error();
    FMOE_REQUIRE(dtype_ok(dtype), FMOE_ERR_BAD_DTYPE, "%s: unknown dtype %d", who, dtype);
    FMOE_REQUIRE(num_tokens >= 0 && hidden > 0 && num_experts > 0 && top_k >= 0, FMOE_ERR_BAD_SHAPE,
                 "%s: bad shape T=%lld H=%d E=%lld K=%d", who, (long long)num_tokens, hidden,
                 (long long)num_experts, top_k);
    FMOE_REQUIRE(algo >= FMOE_EXPERT_AUTO && algo <= FMOE_EXPERT_SLICES, FMOE_ERR_UNSUPPORTED,
                 "%s: unknown algo %d", who, algo);
    if (num_tokens == 0) return FMOE_OK;
    FMOE_REQUIRE((x || act == kActNone) && (down || act == kActNone) && up && out, FMOE_ERR_NULL_POINTER, "%s: null tensor pointer", who);
    FMOE_REQUIRE(top_k == 0 || (indices && gates), FMOE_ERR_NULL_POINTER,
                 "%s: null indices/gates with top_k=%d", who, top_k);
    const int vec = (int)(16 / dtype_size(dtype));
    FMOE_REQUIRE(hidden % vec == 0, FMOE_ERR_ALIGNMENT,
                 "%s: hidden=%d must be a multiple of %d (16-byte rows)", who, hidden, vec);
    FMOE_REQUIRE(aligned16(x) && aligned16(down) && aligned16(up) && aligned16(out), FMOE_ERR_ALIGNMENT,
                 "%s: tensor pointers must be 16-byte aligned", who);
    FMOE_REQUIRE(num_experts < (1ll << 31) && (int64_t)num_tokens * top_k < (1ll << 40), FMOE_ERR_UNSUPPORTED,
                 "%s: problem too large (E=%lld, pairs=%lld)", who, (long long)num_experts,
                 (long long)(num_tokens * top_k));
    hipStream_t s = (hipStream_t)stream;
    bool slices = algo == FMOE_EXPERT_SLICES || (algo == FMOE_EXPERT_AUTO && slices_pay(num_tokens, num_experts, top_k));
    if (top_k == 0) slices = false;
    if (slices && !slices_possible(num_experts, hidden, dtype_size(dtype))) {
        FMOE_REQUIRE(algo == FMOE_EXPERT_AUTO, FMOE_ERR_UNSUPPORTED,
                     "%s: tables of 4 GiB or more cannot use the column-slice schedule", who);
        slices = false;
    }
    if (slices) {
        const size_t need = fmoe_expert_workspace_bytes_algo(num_tokens, hidden, num_experts, top_k, dtype, FMOE_EXPERT_SLICES);
        FMOE_REQUIRE(workspace && workspace_bytes >= need && aligned16(workspace), FMOE_ERR_WORKSPACE,
                     "%s: workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
        switch (dtype) {
            case FMOE_F32: return launch_expert_slices<float>(act, x, down, up, indices, gates, num_tokens, hidden, num_experts, top_k, out, workspace, s);
            case FMOE_BF16: return launch_expert_slices<bf16_t>(act, x, down, up, indices, gates, num_tokens, hidden, num_experts, top_k, out, workspace, s);
            default: return launch_expert_slices<f16_t>(act, x, down, up, indices, gates, num_tokens, hidden, num_experts, top_k, out, workspace, s);
        }
    }
    switch (dtype) {
        case FMOE_F32: return launch_expert_rows<float>(act, x, down, up, indices, gates, num_tokens, hidden, num_experts, top_k, out, s);
        case FMOE_BF16: return launch_expert_rows<bf16_t>(act, x, down, up, indices, gates, num_tokens, hidden, num_experts, top_k, out, s);
        default: return launch_expert_rows<f16_t>(act, x, down, up, indices, gates, num_tokens, hidden, num_experts, top_k, out, s);
    }
}

}  // namespace
}  // namespace fmoe

extern "C" int fmoe_expert_forward_algo(const void* x, const void* down, const void* up, const int64_t* indices,
                                        const void* gates, int64_t num_tokens, int hidden, int64_t num_experts,
                                        int top_k, int dtype, void* out, void* workspace, size_t workspace_bytes,
                                        int algo, void* stream) {
    return fmoe::expert_dispatch("fmoe_expert_forward", fmoe::kActSilu, x, down, up, indices, gates, num_tokens, hidden,
                                 num_experts, top_k, dtype, out, workspace, workspace_bytes, algo, stream);
}

extern "C" int fmoe_peer_forward(const void* x, const void* down, const void* up, const void* routing_weights,
                                 const int64_t* indices, int64_t num_tokens, int hidden, int64_t num_experts, int top_k,
                                 int dtype, void* out, void* workspace, size_t workspace_bytes, void* stream) {
    return fmoe::expert_dispatch("fmoe_peer_forward", fmoe::kActGelu, x, down, up, indices, routing_weights, num_tokens, hidden,
                                 num_experts, top_k, dtype, out, workspace, workspace_bytes, FMOE_EXPERT_AUTO, stream);
}

extern "C" int fmoe_pkm_forward(const void* values, const void* routing_weights, const int64_t* indices, int64_t num_tokens,
                                int hidden, int64_t num_experts, int top_k, int dtype, void* out, void* workspace,
                                size_t workspace_bytes, void* stream) {
    return fmoe::expert_dispatch("fmoe_pkm_forward", fmoe::kActNone, values, values, values, indices, routing_weights, num_tokens,
                                 hidden, num_experts, top_k, dtype, out, workspace, workspace_bytes, FMOE_EXPERT_AUTO, stream);
}

extern "C" int fmoe_expert_forward(const void* x, const void* down, const void* up, const int64_t* indices,
                                   const void* gates, int64_t num_tokens, int hidden, int64_t num_experts,
                                   int top_k, int dtype, void* out, void* workspace, size_t workspace_bytes,
                                   void* stream) {
    return fmoe_expert_forward_algo(x, down, up, indices, gates, num_tokens, hidden, num_experts, top_k, dtype, out,
                                    workspace, workspace_bytes, FMOE_EXPERT_AUTO, stream);
}
