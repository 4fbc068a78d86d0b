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
#include <type_traits>

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
template <typename T, typename TG, int NCH, int ACT, bool SPLIT>
__global__ __launch_bounds__(kWavesPerBlock* kWave) void expert_token_kernel(
    const T* __restrict__ x, const T* __restrict__ down, const T* __restrict__ up,
    const int64_t* __restrict__ indices, const TG* __restrict__ gates, T* __restrict__ out,
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
    const TG* my_gate = gates + token * top_k;

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
                gate[u] = Elem<TG>::to_f32(my_gate[k]);
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
            hipLaunchKernelGGL((expert_token_kernel<T, T, N, A, true>), grid, block, 0, stream, (const T*)x, (const T*)down, \
                               (const T*)up, indices, (const T*)gates, (T*)out, T_, H, E, K);                         \
        else                                                                                                          \
            hipLaunchKernelGGL((expert_token_kernel<T, T, N, A, false>), grid, block, 0, stream, (const T*)x, (const T*)down, \
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

// out[t] = sum_k coef[t,k] * up[idx[t,k]] with fp32 coefficients that are already complete (the second phase of the
// bucketed schedule): the row kernel without its score phase.
template <typename T>
int launch_expert_rows_coef(const void* up, const int64_t* indices, const float* coef, int64_t T_, int H, int64_t E, int K,
                            void* out, hipStream_t stream) {
    constexpr int V = Elem<T>::kVec;
    const int nch = (H / V + kWave - 1) / kWave;
    const dim3 block(kWavesPerBlock * kWave);
    const dim3 grid((unsigned)((T_ + kWavesPerBlock - 1) / kWavesPerBlock));
#define FMOE_LAUNCH_COEF(N)                                                                                             \
    hipLaunchKernelGGL((expert_token_kernel<T, float, N, kActNone, false>), grid, block, 0, stream, (const T*)up, (const T*)up, \
                       (const T*)up, indices, coef, (T*)out, T_, H, E, K)
    if (nch <= 1) FMOE_LAUNCH_COEF(1);
    else if (nch <= 2) FMOE_LAUNCH_COEF(2);
    else if (nch <= 4) FMOE_LAUNCH_COEF(4);
    else if (nch <= 8) FMOE_LAUNCH_COEF(8);
    else {
        set_error("fmoe_expert_forward: hidden=%d exceeds the %d elements per row this build supports", H, 8 * kWave * V);
        return FMOE_ERR_UNSUPPORTED;
    }
#undef FMOE_LAUNCH_COEF
    FMOE_CHECK_LAUNCH("fmoe_expert_forward(states)");
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
// The same load marked non-temporal: data that is read once and should not displace what the L2 is meant to keep.
__device__ inline u32x4_t load_row_piece_streaming(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset) {
    return __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)byte_offset, 0, 2));
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

// Workgroup b runs on XCD b % xcds (ids are dealt round-robin): XCD x takes slices x, x + xcds, ... for whole rounds of
// xcds slices.  The slices left over after the last whole round (fewer than xcds) would leave XCDs idle: each of them is
// shared by xcds / left XCDs instead, which take interleaved token blocks of it.
__host__ __device__ inline int slice_parts(int num_slices, int xcds) {
    const int left = num_slices % xcds;
    return left ? xcds / left : 1;
}
__host__ __device__ inline int slice_grid_rows(int num_slices, int blocks_per_slice, int xcds) {   // grid = xcds * rows
    const int parts = slice_parts(num_slices, xcds);
    return (num_slices / xcds) * blocks_per_slice + (num_slices % xcds ? (blocks_per_slice + parts - 1) / parts : 0);
}
__device__ inline bool slice_of_block(int num_slices, int blocks_per_slice, int xcds, int& slice, int& tb) {
    const int b = (int)blockIdx.x;
    const int x = b % xcds, j = b / xcds;
    const int whole = num_slices / xcds;
    if (j < whole * blocks_per_slice) {
        slice = x + xcds * (j / blocks_per_slice);
        tb = j % blocks_per_slice;
        return true;
    }
    const int left = num_slices % xcds, parts = slice_parts(num_slices, xcds);
    if (left == 0 || x / left >= parts) return false;
    slice = whole * xcds + x % left;
    tb = (j - whole * blocks_per_slice) * parts + x / left;
    return tb < blocks_per_slice;
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

// IDS: the row offsets are not prepared yet: they are taken from the int64 ids (an id outside [0, num_experts) gives the
// out-of-bounds offset) and the workgroups of slice 0 also store them to off32 for the launches that follow.
template <typename T, int CL, bool IDS = false>
__global__ __launch_bounds__(256) void expert_scores_slice_kernel(
    const T* __restrict__ x, const T* __restrict__ down, uint32_t table_bytes, const uint32_t* __restrict__ off32,
    float* __restrict__ spart, int64_t num_tokens, int hidden, int top_k, int num_slices, int blocks_per_slice,
    int tokens_per_block, int xcds, const int64_t* __restrict__ ids = nullptr, int64_t num_experts = 0) {
    constexpr int V = Elem<T>::kVec;
    constexpr int PPL = kWave / CL;                         // pairs per wave-wide load
    int slice, tb;
    if (!slice_of_block(num_slices, blocks_per_slice, xcds, slice, tb)) return;
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
            uint32_t mine = kBadOffset;
            if constexpr (IDS) {
                if (k0 + lane < top_k) {
                    const int64_t e = ids[t * top_k + k0 + lane];
                    if (e >= 0 && e < num_experts) mine = (uint32_t)e * (uint32_t)(hidden * (int)sizeof(T));
                    if (slice == 0) const_cast<uint32_t*>(tok_off)[k0 + lane] = mine;
                }
            } else {
                if (k0 + lane < top_k) mine = tok_off[k0 + lane];
            }
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

// acc[0..8) += a * w for one 16-byte packet of a 16-bit row.  bf16: the coefficient is rounded to bf16 (the reference
// forms silu(s)*g in the activation dtype as well, flash_expert.py:191) and meets each element through the packed dot
// product, (w[2i], w[2i+1]) . (a, 0) and . (0, a): no unpacking, half the instructions of convert + fma.
template <typename T> __device__ inline void axpy16_coef(float a, u32x4_t w, float* acc) { axpy16<T>(a, w, acc); }
template <> __device__ inline void axpy16_coef<bf16_t>(float a, u32x4_t w, float* acc) {
    const bf16_t ab = (bf16_t)a, zero = (bf16_t)0.0f;
    const bf16x2_t lo = {ab, zero}, hi = {zero, ab};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t wi = w[i];
        acc[2 * i] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, wi), lo, acc[2 * i], false);
        acc[2 * i + 1] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, wi), hi, acc[2 * i + 1], false);
    }
}

template <typename T, int CL>
__global__ __launch_bounds__(256) void expert_states_slice_kernel(
    const float* __restrict__ a, const T* __restrict__ up, uint32_t table_bytes, const uint32_t* __restrict__ off32,
    T* __restrict__ out, int64_t num_tokens, int hidden, int top_k, int num_slices, int blocks_per_slice,
    int tokens_per_block, int xcds) {
    constexpr int V = Elem<T>::kVec;
    constexpr int PPL = kWave / CL;
    int slice, tb;
    if (!slice_of_block(num_slices, blocks_per_slice, xcds, slice, tb)) return;
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
    int chunk_lanes, num_slices, blocks_per_slice, tokens_per_block, xcds;
    unsigned grid;
    size_t off_idx32, off_a, off_spart, bytes;
};

// A slice is as wide as one XCD's 4 MiB L2 can keep resident: 256 bytes per row up to 16384 rows (fewer passes over
// the offsets, coefficients and partial sums), 128 bytes beyond.
SlicePlan plan_slices(int64_t T_, int H, int64_t E, int K, size_t elt) {
    SlicePlan p;
    const ChipInfo& chip = chip_info();
    p.xcds = chip.xcds;
    p.chunk_lanes = E * 256 <= chip.l2_bytes ? 16 : 8;
    const size_t chunk_bytes = (size_t)p.chunk_lanes * 16;
    p.num_slices = (int)((H * elt + chunk_bytes - 1) / chunk_bytes);
    const int64_t want = (T_ + 3) / 4;                       // at least one token per wave
    p.blocks_per_slice = (int)(want < 1024 ? want : 1024);   // 256 blocks of 4 waves fill one XCD; a few rounds of them
    p.tokens_per_block = (int)((T_ + p.blocks_per_slice - 1) / p.blocks_per_slice);
    p.grid = (unsigned)(p.xcds * slice_grid_rows(p.num_slices, p.blocks_per_slice, p.xcds));
    const size_t pairs = (size_t)T_ * (size_t)K;
    p.off_idx32 = 0;
    p.off_a = round_up(p.off_idx32 + pairs * 4, 256);
    p.off_spart = round_up(p.off_a + pairs * 4, 256);
    p.bytes = round_up(p.off_spart + (size_t)p.num_slices * pairs * 4, 256);
    return p;
}

// ids != nullptr: off32 is written by this launch (from the ids) instead of read
template <typename T>
int launch_slice_scores(const void* x, const void* table, const uint32_t* off32, float* spart, int64_t T_, int H, int64_t E,
                        int K, hipStream_t stream, const int64_t* ids = nullptr) {
    const SlicePlan p = plan_slices(T_, H, E, K, sizeof(T));
    const uint32_t table_bytes = (uint32_t)(E * (int64_t)H * (int64_t)sizeof(T));
    if (ids != nullptr) {
        if (p.chunk_lanes == 16)
            hipLaunchKernelGGL((expert_scores_slice_kernel<T, 16, true>), dim3(p.grid), dim3(256), 0, stream, (const T*)x,
                               (const T*)table, table_bytes, off32, spart, T_, H, K, p.num_slices, p.blocks_per_slice,
                               p.tokens_per_block, p.xcds, ids, E);
        else
            hipLaunchKernelGGL((expert_scores_slice_kernel<T, 8, true>), dim3(p.grid), dim3(256), 0, stream, (const T*)x,
                               (const T*)table, table_bytes, off32, spart, T_, H, K, p.num_slices, p.blocks_per_slice,
                               p.tokens_per_block, p.xcds, ids, E);
    } else if (p.chunk_lanes == 16)
        hipLaunchKernelGGL((expert_scores_slice_kernel<T, 16>), dim3(p.grid), dim3(256), 0, stream, (const T*)x,
                           (const T*)table, table_bytes, off32, spart, T_, H, K, p.num_slices, p.blocks_per_slice,
                           p.tokens_per_block, p.xcds, (const int64_t*)nullptr, (int64_t)0);
    else
        hipLaunchKernelGGL((expert_scores_slice_kernel<T, 8>), dim3(p.grid), dim3(256), 0, stream, (const T*)x,
                           (const T*)table, table_bytes, off32, spart, T_, H, K, p.num_slices, p.blocks_per_slice,
                           p.tokens_per_block, p.xcds, (const int64_t*)nullptr, (int64_t)0);
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
                           table_bytes, off32, (T*)out, T_, H, K, p.num_slices, p.blocks_per_slice, p.tokens_per_block, p.xcds);
    else
        hipLaunchKernelGGL((expert_states_slice_kernel<T, 8>), dim3(p.grid), dim3(256), 0, stream, a, (const T*)table,
                           table_bytes, off32, (T*)out, T_, H, K, p.num_slices, p.blocks_per_slice, p.tokens_per_block, p.xcds);
    FMOE_CHECK_LAUNCH("routed experts (slice states)");
    return FMOE_OK;
}

// Scores, gate and states launches on row offsets that already sit at the start of the workspace.
// ids != nullptr: the offsets are not in the workspace yet; the score launch writes them on its way
template <typename T>
int launch_expert_slices_prepared(int act, const void* x, const void* down, const void* up, const void* gates, int64_t T_,
                                  int H, int64_t E, int K, void* out, void* workspace, hipStream_t stream,
                                  const int64_t* ids = nullptr) {
    const SlicePlan p = plan_slices(T_, H, E, K, sizeof(T));
    char* ws = (char*)workspace;
    const uint32_t* off32 = (const uint32_t*)(ws + p.off_idx32);
    float* a = (float*)(ws + p.off_a);
    float* spart = (float*)(ws + p.off_spart);
    const int64_t pairs = T_ * K;
    const unsigned flat_grid = (unsigned)((pairs + 255) / 256);
    if (act != kActNone)
        if (int rc = launch_slice_scores<T>(x, down, off32, spart, T_, H, E, K, stream, ids)) return rc;
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
    // with a score phase the score launch turns the ids into row offsets itself (and stores them for the launches after it)
    if (act != kActNone) return launch_expert_slices_prepared<T>(act, x, down, up, gates, T_, H, E, K, out, workspace, stream, indices);
    const SlicePlan p = plan_slices(T_, H, E, K, sizeof(T));
    uint32_t* off32 = (uint32_t*)((char*)workspace + p.off_idx32);
    const int64_t pairs = T_ * K;
    hipLaunchKernelGGL(expert_prepare_kernel, dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, stream, indices, off32,
                       pairs, E, (uint32_t)(H * sizeof(T)));
    FMOE_CHECK_LAUNCH("fmoe_expert_forward(prepare)");
    return launch_expert_slices_prepared<T>(act, x, down, up, gates, T_, H, E, K, out, workspace, stream);
}

// ------------------------------------------------------------------------------------------------
// Bucketed (expert-centric) schedule, for tables too large for the column-slice schedule.
//
// The pairs are grouped by expert (fmoe_bucket.hip).  In that order consecutive pairs share their row of `down`, so a
// lane group keeps the row's piece in registers and only the pieces of x are gathered, one per pair; and it is x, not
// the table, that has to stay in L2: column bands of x (128 to 512 bytes per token, at most about 4 MiB for all tokens)
// are dealt to the XCDs like the slices above, while every table byte streams through once, in order.
//   bucket  : ids -> offsets[E+1], per slot of the grouped order: pair index, x row offset, table row offset
//   scores  : spart[band][slot] = <x[token, band cols], down[expert, band cols]>
//   gate    : a[pair] = act(sum_band spart[band][slot]) * gate[pair]        (back in (token, k) order)
//   states  : out[token] = sum_k a[token,k] * up[expert_k]                  (one wave per token, whole rows)
// ------------------------------------------------------------------------------------------------
constexpr int kBucketChunk = 64;     // consecutive slots one lane group works through
constexpr int kBucketBatch = 8;      // slots whose loads are in flight together

// xb[band][token][band bytes] = x[token][band * band bytes ...]: every band of x contiguous.  Pieces of one band that
// lie a whole row (a power of two, typically) apart compete for a few sets of the L2; contiguous, the band uses them all.
__global__ __launch_bounds__(256) void expert_band_copy_kernel(const u32x4_t* __restrict__ x, u32x4_t* __restrict__ xb,
                                                               int64_t num_tokens, int row_packets, int band_packets) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;       // packet index in x
    if (i >= num_tokens * row_packets) return;
    const int64_t t = i / row_packets;
    const int pk = (int)(i % row_packets), band = pk / band_packets, c = pk % band_packets;
    xb[((int64_t)band * num_tokens + t) * band_packets + c] = x[i];
}

// CL lanes share one pair: a band is CL * 16 bytes wide and a wave-wide load covers G = 64 / CL pairs.  A workgroup
// takes runs of 4 * G * kBucketChunk consecutive slots; each of its 4 * G lane groups works through kBucketChunk of them,
// kBucketBatch at a time.  The experts of such a run are consecutive rows of the table: their pieces of the band are
// staged in LDS with plain coalesced loads (every byte of the band leaves the table once; the loads are issued one run
// ahead and parked in registers), and a slot reads its piece from there, so that the only vector-memory instruction
// per slot is the gather of x: the kernel is bound by the rate at which a CU takes 64-lane loads (about 30 cycles
// each), not by bytes.  A run whose experts span more rows than fit (few pairs for many experts) loads the pieces per
// slot instead.
// entry[slot] = token | (expert & 255) << 24: with at most 256 staged rows the low byte of the id places the row.
constexpr int kBucketLdsBytes = 32768;     // staged rows per workgroup: 32 KiB / band width, at most 256
constexpr uint32_t kEntryTokenMask = 0x00FFFFFFu;

template <typename T, int CL>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void expert_scores_bucketed_kernel(
    const T* __restrict__ xb, uint32_t x_bytes, const T* __restrict__ down, uint32_t table_bytes,
    const uint32_t* __restrict__ entry, const uint32_t* __restrict__ expid, const int32_t* __restrict__ offsets,
    int64_t num_experts, float* __restrict__ spart, int64_t spart_stride, uint32_t row_bytes, int num_bands, int parts,
    int blocks_per_unit, int xcds) {
    constexpr int G = kWave / CL, U = kBucketBatch;
    constexpr int kRun = 4 * G * kBucketChunk;                          // slots per workgroup iteration
    constexpr int kBand = CL * 16;
    constexpr int kRows = kBucketLdsBytes / kBand;
    constexpr int kStage = kBucketLdsBytes / 16 / 256;                  // 16-byte pieces per thread that fill the LDS
    static_assert(kBucketChunk == 8 * U && CL >= 8 && kRows <= 256, "lane c < 8 holds the entries of batch c");
    __shared__ __attribute__((aligned(16))) unsigned char rows[kBucketLdsBytes];
    const int b = (int)blockIdx.x;
    const int unit = b % xcds + xcds * ((b / xcds) / blocks_per_unit);  // XCD b % xcds takes units x, x + xcds, ...
    const int tb = (b / xcds) % blocks_per_unit;
    if (unit >= num_bands * parts) return;
    const int band = unit % num_bands, part = unit / num_bands;
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane & (CL - 1), g = lane / CL;
    const int group_base = (lane & ~(CL - 1)) << 2;                     // byte address of the group's lane 0 for ds_bpermute
    const uint32_t col_bytes = (uint32_t)band * kBand + (uint32_t)c * 16;
    const uint32_t x_col_bytes = (uint32_t)band * (x_bytes / (uint32_t)num_bands) + (uint32_t)c * 16;   // x is band-major here
    const __amdgpu_buffer_rsrc_t xr = table_resource(xb, x_bytes), wr = table_resource(down, table_bytes);
    const __amdgpu_buffer_rsrc_t er = table_resource(entry, (uint32_t)spart_stride * 4u);
    const int n_valid = offsets[num_experts];
    const int runs = (n_valid + kRun - 1) / kRun;
    const int per_part = (runs + parts - 1) / parts;
    const int run_end = (part + 1) * per_part < runs ? (part + 1) * per_part : runs;
    float* my_spart = spart + (int64_t)band * spart_stride;

    // entries of the group's 64 slots: lanes 0..7 of the group hold 8 each (reads past the array give zeros; slots from
    // n_valid on are not stored)
    auto load_entries = [&](int run, u32x4_t (&t)[2]) {
        const uint32_t at = ((uint32_t)run * kRun + (uint32_t)(wave * G + g) * kBucketChunk + (uint32_t)(c & 7) * 8u) * 4u;
        t[0] = load_row_piece_streaming(er, at);
        t[1] = load_row_piece_streaming(er, at + 16u);
    };
    // first and last expert of a run (the slots are in ascending expert order)
    auto load_span = [&](int run, uint32_t& lo, uint32_t& hi) {
        const int q_lo = run * kRun, q_hi = (run + 1) * kRun < n_valid ? (run + 1) * kRun - 1 : n_valid - 1;
        lo = expid[q_lo];
        hi = expid[q_hi];
    };
    // piece k of thread i: row (i + 256 k) / CL of the run, packet (i + 256 k) % CL of the band
    auto load_rows = [&](uint32_t lo, uint32_t hi, u32x4_t (&st)[kStage]) {
        const uint32_t first = (uint32_t)__builtin_amdgcn_readfirstlane((int)lo);
        const uint32_t span = (uint32_t)__builtin_amdgcn_readfirstlane((int)hi) - first + 1u;
        if (span > (uint32_t)kRows) return;
#pragma unroll
        for (int k = 0; k < kStage; ++k) {
            const uint32_t i = (uint32_t)tid + 256u * k, r = i / CL;
            st[k] = load_row_piece_streaming(wr, r < span ? (first + r) * row_bytes + (uint32_t)band * kBand + (i % CL) * 16u : kBadOffset);
        }
    };
    int run = part * per_part + tb;
    u32x4_t ent[2], stage[kStage];
    uint32_t e_lo = 0, e_hi = 0, n_lo = 0, n_hi = 0;                    // expert span of this run and of the next one
    if (run < run_end) {
        load_entries(run, ent);
        load_span(run, e_lo, e_hi);
        load_span(run + blocks_per_unit < run_end ? run + blocks_per_unit : run, n_lo, n_hi);
        load_rows(e_lo, e_hi, stage);
    }
    for (; run < run_end; run += blocks_per_unit) {
        const int next = run + blocks_per_unit < run_end ? run + blocks_per_unit : run;
        const int next2 = next + blocks_per_unit < run_end ? next + blocks_per_unit : next;
        const uint32_t first = (uint32_t)__builtin_amdgcn_readfirstlane((int)e_lo);
        const uint32_t span = (uint32_t)__builtin_amdgcn_readfirstlane((int)e_hi) - first + 1u;
        const bool staged = span <= (uint32_t)kRows;
        if (staged) {
#pragma unroll
            for (int k = 0; k < kStage; ++k)
                *reinterpret_cast<u32x4_t*>(&rows[((uint32_t)tid + 256u * k) * 16u]) = stage[k];
        }
        __syncthreads();
        u32x4_t nxt[2];
        uint32_t f_lo, f_hi;
        load_entries(next, nxt);                                        // the next run's entries and rows, ahead of time
        load_span(next2, f_lo, f_hi);
        load_rows(n_lo, n_hi, stage);
        const int q_first = run * kRun + (wave * G + g) * kBucketChunk;
        if (staged) {
            const uint32_t lds_base = (uint32_t)c * 16u - (first & 255u) * kBand;     // + (entry >> 24) * kBand, modulo the LDS size
#pragma unroll 1
            for (int bt = 0; bt < kBucketChunk / U; ++bt) {
                const int q0 = q_first + bt * U;
                if (q0 >= n_valid) break;
                const int src = group_base + bt * 4;                    // lane bt of the group holds this batch's entries
                u32x4_t xg[U];
                uint32_t at[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const uint32_t en = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)ent[u / 4][u % 4]);
                    xg[u] = load_row_piece(xr, (en & kEntryTokenMask) * kBand + x_col_bytes);
                    at[u] = ((en >> 24) * kBand + lds_base) & (uint32_t)(kBucketLdsBytes - 1);
                }
                float partial[U];
#pragma unroll
                for (int u = 0; u < U; ++u)
                    partial[u] = dot16<T>(xg[u], *reinterpret_cast<const u32x4_t*>(&rows[at[u]]), 0.0f);
                float total = transpose_sum<U, 1>(partial, c);          // over each aligned 8 lanes: slot q0 + (c & 7)
                if constexpr (CL >= 16) total += xor_step<U, 8>(total);
                if constexpr (CL >= 32) total += xor_step<U, 16>(total);
                if (c < U && q0 + c < n_valid) __builtin_nontemporal_store(total, &my_spart[q0 + c]);
            }
        } else {
            // the experts of this run are too far apart to stage: each slot loads its own piece of the row
#pragma unroll 1
            for (int bt = 0; bt < kBucketChunk / U; ++bt) {
                const int q0 = q_first + bt * U;
                if (q0 >= n_valid) break;
                const int src = group_base + bt * 4;
                float partial[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const uint32_t en = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)ent[u / 4][u % 4]);
                    const uint32_t e = q0 + u < n_valid ? expid[q0 + u] : 0u;
                    const u32x4_t xg = load_row_piece(xr, (en & kEntryTokenMask) * kBand + x_col_bytes);
                    partial[u] = dot16<T>(xg, load_row_piece(wr, e * row_bytes + col_bytes), 0.0f);
                }
                float total = transpose_sum<U, 1>(partial, c);
                if constexpr (CL >= 16) total += xor_step<U, 8>(total);
                if constexpr (CL >= 32) total += xor_step<U, 16>(total);
                if (c < U && q0 + c < n_valid) __builtin_nontemporal_store(total, &my_spart[q0 + c]);
            }
        }
        __syncthreads();                                                // the rows are rewritten by the next run
        ent[0] = nxt[0];
        ent[1] = nxt[1];
        e_lo = n_lo;
        e_hi = n_hi;
        n_lo = f_lo;
        n_hi = f_hi;
    }
}

template <typename T, int ACT>
__global__ __launch_bounds__(256) void expert_gate_sorted_kernel(const float* __restrict__ spart, int64_t spart_stride,
                                                                 const T* __restrict__ gates, const int32_t* __restrict__ sorted_pairs,
                                                                 const int32_t* __restrict__ offsets, int64_t num_experts,
                                                                 float* __restrict__ a, int num_bands) {
    const int n_valid = offsets[num_experts];
    for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < n_valid; q += (int64_t)gridDim.x * blockDim.x) {
        const int32_t p = sorted_pairs[q];
        const float gate = Elem<T>::to_f32(gates[p]);
        float s = 0.0f;
        int bd = 0;
        for (; bd + 8 <= num_bands; bd += 8) {              // eight loads in flight at a time, summed in band order
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = __builtin_nontemporal_load(&spart[(int64_t)(bd + j) * spart_stride + q]);
#pragma unroll
            for (int j = 0; j < 8; ++j) s += v[j];
        }
        for (; bd < num_bands; ++bd) s += spart[(int64_t)bd * spart_stride + q];
        a[p] = activate<ACT>(s) * gate;
    }
}

// ---- second phase for large tables: a sweep over the experts with the output in LDS ----------------------------------
// out[t] = sum_k a[t,k] * up[e_k] needs one row of `up` per pair.  Token by token these rows come from all over a table
// far larger than the caches (the row schedule: bound by HBM).  Here every lane group owns kSweepTokens tokens and walks
// their pairs in ascending expert order; all lane groups of an XCD do so at the same pace on the same column band, so at
// any moment they gather from one narrow window of the band, which the L2 holds: the band leaves HBM once per pass over
// it.  The running sums of a workgroup's 512 tokens (64 fp32 columns each) live in LDS; a lane group is the only one to
// touch its tokens' rows, in list order, so the result is deterministic without atomics.
//   owner sort : per owner (kSweepTokens consecutive tokens) the keys expert << 10 | token_in_owner << 8 | k, sorted,
//                and the coefficients in that order
//   sweep      : out[token, band] for 512 tokens x one 128-byte band per workgroup
constexpr int kSweepTokens = 4;                          // tokens per lane group
constexpr int kSweepThreads = 1024;                      // 16 waves = 128 lane groups = 512 tokens per workgroup
constexpr int kSweepWgTokens = (kSweepThreads / 8) * kSweepTokens;
constexpr int kSweepMaxTopK = 256, kSweepMaxKeys = kSweepTokens * kSweepMaxTopK;

__global__ __launch_bounds__(256) void expert_owner_sort_kernel(const int64_t* __restrict__ indices, const float* __restrict__ a,
                                                                uint32_t* __restrict__ entries, float* __restrict__ coef,
                                                                int64_t num_tokens, int64_t num_experts, int top_k) {
    __shared__ uint32_t keys[kSweepMaxKeys];
    const int tid = (int)threadIdx.x;
    const int64_t owner = blockIdx.x;
    const int n = kSweepTokens * top_k;
    int m = 64;
    while (m < n) m <<= 1;
    for (int i = tid; i < m; i += 256) {
        uint32_t key = 0xFFFFFFFFu;
        if (i < n) {
            const int tl = i / top_k, k = i % top_k;
            const int64_t t = owner * kSweepTokens + tl;
            if (t < num_tokens) {
                const int64_t e = indices[t * top_k + k];
                if (e >= 0 && e < num_experts) key = (uint32_t)e << 10 | (uint32_t)tl << 8 | (uint32_t)k;
            }
        }
        keys[i] = key;
    }
    __syncthreads();
    for (int k = 2; k <= m; k <<= 1)
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int i = tid; i < m / 2; i += 256) {
                const int lo = ((i & ~(j - 1)) << 1) | (i & (j - 1)), hi = lo | j;
                const uint32_t x0 = keys[lo], x1 = keys[hi];
                if ((x0 > x1) == ((lo & k) == 0)) {
                    keys[lo] = x1;
                    keys[hi] = x0;
                }
            }
            __syncthreads();
        }
    for (int i = tid; i < n; i += 256) {
        const uint32_t key = keys[i];
        entries[owner * n + i] = key;
        float c = 0.0f;
        if (key != 0xFFFFFFFFu) c = a[(owner * kSweepTokens + ((key >> 8) & 3u)) * top_k + (key & 255u)];
        coef[owner * n + i] = c;
    }
}

template <typename T>
__global__ __launch_bounds__(kSweepThreads) void expert_states_sweep_kernel(
    const T* __restrict__ up, uint32_t table_bytes, const uint32_t* __restrict__ entries, const float* __restrict__ coef,
    T* __restrict__ out, int64_t num_tokens, int64_t num_experts, int top_k, uint32_t row_bytes, int num_bands,
    int token_blocks, int xcds) {
    constexpr int CL = 8;
    static_assert(sizeof(T) == 2, "eight 16-bit columns per lane: a 128-byte band is 64 columns");
    __shared__ __attribute__((aligned(16))) float sums[kSweepWgTokens * 64];   // [512 tokens][64 columns]: 128 KiB
    const int b = (int)blockIdx.x;
    const int band = b % xcds + xcds * ((b / xcds) / token_blocks);     // XCD b % xcds takes bands x, x + xcds, ...
    const int tb = (b / xcds) % token_blocks;
    if (band >= num_bands) return;
    const int tid = (int)threadIdx.x, lane = tid & 63;
    const int c = lane & (CL - 1), group = tid / CL;                    // lane group 0..127 of the workgroup
    const int group_base = (lane & ~(CL - 1)) << 2;
    const int64_t owner = (int64_t)tb * (kSweepThreads / CL) + group;
    const int n = kSweepTokens * top_k;
    const uint32_t col_bytes = (uint32_t)band * (CL * 16) + (uint32_t)c * 16;
    const __amdgpu_buffer_rsrc_t wr = table_resource(up, table_bytes);
    const uint64_t list_bytes = (uint64_t)((num_tokens + kSweepTokens - 1) / kSweepTokens) * (uint64_t)n * 4u;
    const __amdgpu_buffer_rsrc_t er = table_resource(entries, (uint32_t)list_bytes), cr = table_resource(coef, (uint32_t)list_bytes);
    // the group's rows of `sums`: token tl at (group * 4 + tl) * 64 floats; this lane's 8 columns are two 16-byte halves,
    // which odd groups keep in the opposite order so that two groups served together never meet in a bank
    float* my_rows = sums + group * kSweepTokens * 64 + c * 8;
    const int h0 = (group & 1) * 4, h1 = 4 - h0;
    const f32x4_t zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int tl = 0; tl < kSweepTokens; ++tl) {
        *reinterpret_cast<f32x4_t*>(my_rows + tl * 64) = zero4;
        *reinterpret_cast<f32x4_t*>(my_rows + tl * 64 + 4) = zero4;
    }
    const uint32_t list_at = (uint32_t)((uint64_t)owner * (uint64_t)n * 4u);
    auto load_entries = [&](int pos, u32x4_t (&en)[2], u32x4_t (&cf)[2]) {
        const uint32_t at = list_at + ((uint32_t)pos + (uint32_t)c * 8u) * 4u;
        const bool ok = pos + c * 8 < n;                                // whole 8-entry pieces: n is a multiple of 4, see below
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            en[h] = load_row_piece_streaming(er, ok ? at + 16u * h : kBadOffset);
            cf[h] = load_row_piece_streaming(cr, ok ? at + 16u * h : kBadOffset);
        }
    };
    // Four entries at a time, the gathers of the next four issued before the current four are added: the loads of a
    // wave never drain.  `fetch` turns four entries into their keys, coefficients and row pieces; `add` adds them.
    constexpr int Q = 4;
    struct Quad {
        u32x4_t w[Q];
        uint32_t key[Q];
        float cv[Q];
    };
    auto fetch = [&](Quad& q, const u32x4_t& e4, const u32x4_t& c4, int src, int at) {
#pragma unroll
        for (int u = 0; u < Q; ++u) {
            const bool live = at + u < n;                           // the last piece of a list may reach into the next one
            q.key[u] = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)e4[u]);
            const float cvu = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(src, (int)c4[u]));
            q.cv[u] = live ? cvu : 0.0f;
            const uint32_t e = q.key[u] >> 10;
            // a key that names no expert (an id outside the table sorts to the end with coefficient 0) takes an
            // address outside the table, which reads as zeros: 0 * row must not meet a non-finite row
            q.w[u] = load_row_piece(wr, (e < (uint32_t)num_experts && live) ? e * row_bytes + col_bytes : kBadOffset);
        }
    };
    auto add = [&](const Quad& q) {
#pragma unroll
        for (int u = 0; u < Q; ++u) {
            float* row = my_rows + ((q.key[u] >> 8) & 3u) * 64;
            f32x4_t s0 = *reinterpret_cast<f32x4_t*>(row + h0), s1 = *reinterpret_cast<f32x4_t*>(row + h1);
            float acc[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
            axpy16_coef<T>(q.cv[u], q.w[u], acc);
            s0 = f32x4_t{acc[0], acc[1], acc[2], acc[3]};
            s1 = f32x4_t{acc[4], acc[5], acc[6], acc[7]};
            *reinterpret_cast<f32x4_t*>(row + h0) = s0;
            *reinterpret_cast<f32x4_t*>(row + h1) = s1;
        }
    };
    u32x4_t en[2], cf[2];
    load_entries(0, en, cf);
    Quad qa, qb;
    fetch(qa, en[0], cf[0], group_base, 0);
    for (int pos = 0; pos < n; pos += kBucketChunk) {
        u32x4_t nen[2], ncf[2];
        load_entries(pos + kBucketChunk, nen, ncf);                     // the next 64 entries, ahead of time
#pragma unroll 1
        for (int bt = 0; bt < kBucketChunk / 8; ++bt) {
            const int at = pos + bt * 8;
            if (at >= n) break;
            const int src = group_base + bt * 4;                        // lane bt of the group holds entries at .. at + 7
            fetch(qb, en[1], cf[1], src, at + 4);
            add(qa);
            // the first four of the next eight: from lane bt + 1, or from lane 0 of the next 64
            if (bt + 1 < kBucketChunk / 8) fetch(qa, en[0], cf[0], src + 4, at + 8);
            else fetch(qa, nen[0], ncf[0], group_base, at + 8);
            add(qb);
            // every list has the same length, so equal positions mean (statistically) equal experts: keeping the
            // workgroup's waves within two batches of each other keeps their gathers inside one window of the band
            if (bt & 1) __syncthreads();
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            en[h] = nen[h];
            cf[h] = ncf[h];
        }
    }
    // the group's tokens: 8 columns per lane, rounded once
#pragma unroll
    for (int tl = 0; tl < kSweepTokens; ++tl) {
        const int64_t t = owner * kSweepTokens + tl;
        if (t < num_tokens) {
            const f32x4_t s0 = *reinterpret_cast<f32x4_t*>(my_rows + tl * 64 + h0), s1 = *reinterpret_cast<f32x4_t*>(my_rows + tl * 64 + h1);
            const float acc[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
            *reinterpret_cast<u32x4_t*>(reinterpret_cast<char*>(out) + t * (int64_t)row_bytes + col_bytes) = pack16<T>(acc);
        }
    }
}

struct BucketedPlan {
    int chunk_lanes, num_bands, parts, blocks_per_unit, xcds;
    unsigned grid;
    size_t off_bucket, off_part, off_offsets, off_pairs, off_tok, off_exp, off_a, off_spart, off_xb, off_sweep_keys, off_sweep_coef, bytes;
    bool sweep;
};

// the row kernels keep a whole row in the registers of one wavefront: at most 8 packets of 16 bytes per lane
bool rows_possible(int H, size_t elt) { return (size_t)H * elt <= (size_t)8 * kWave * 16; }

// The sweep needs 16-bit rows of whole 128-byte bands, at most 256 pairs per token, ids below 2^22 and lists below 4 GiB.
bool sweep_possible(int64_t T_, int H, int64_t E, int K, size_t elt) {
    const int64_t padded = (T_ + kSweepTokens - 1) / kSweepTokens * kSweepTokens;
    // keys are expert << 10 | token in owner << 8 | k with 0xFFFFFFFF for "no expert": E stays below 2^22 so that no pair
    // can encode to the sentinel and the sweep's `expert < E` test rejects it
    return elt == 2 && (H * elt) % 128 == 0 && K <= kSweepMaxTopK && E < (1ll << 22) && padded * K * 4 < (int64_t)kBadOffset;
}

// Band width: as wide as lets the band of all tokens stay in one XCD's L2 (about 2 MiB of its 4), at least 128 bytes.
BucketedPlan plan_bucketed(int64_t T_, int H, int64_t E, int K, size_t elt) {
    BucketedPlan p;
    const ChipInfo& chip = chip_info();
    p.xcds = chip.xcds;
    p.chunk_lanes = T_ * 512 <= chip.l2_bytes / 2 ? 32 : (T_ * 256 <= chip.l2_bytes / 2 ? 16 : 8);
    while (p.chunk_lanes > 8 && (H * elt) % ((size_t)p.chunk_lanes * 16) != 0) p.chunk_lanes /= 2;   // bands tile the row
    const size_t band_bytes = (size_t)p.chunk_lanes * 16;
    p.num_bands = (int)((H * elt + band_bytes - 1) / band_bytes);
    p.parts = (p.num_bands < p.xcds && p.xcds % p.num_bands == 0) ? p.xcds / p.num_bands : 1;      // several XCDs share a band
    const int64_t pairs = T_ * K;
    const int64_t run_slots = 4 * (kWave / p.chunk_lanes) * kBucketChunk;
    const int64_t want = ((pairs + run_slots - 1) / run_slots + p.parts - 1) / p.parts;      // runs per part
    p.blocks_per_unit = (int)(want < 1 ? 1 : (want > 256 ? 256 : want));
    const int units = p.num_bands * p.parts;
    p.grid = (unsigned)(p.xcds * p.blocks_per_unit * ((units + p.xcds - 1) / p.xcds));
    size_t o = 0;
    auto take = [&](size_t n) { const size_t at = o; o = round_up(o + n, 256); return at; };
    p.off_bucket = take(bucket_workspace_bytes(E));
    p.off_part = take(bucket_partition_workspace_bytes(pairs, E));
    p.off_offsets = take((size_t)(E + 1) * 4);
    p.off_pairs = take((size_t)pairs * 4);
    p.off_tok = take((size_t)pairs * 4);
    p.off_exp = take((size_t)pairs * 4);
    p.off_a = take((size_t)pairs * 4);
    p.off_spart = take((size_t)p.num_bands * pairs * 4);
    p.off_xb = take((size_t)T_ * H * elt);
    p.sweep = sweep_possible(T_, H, E, K, elt);
    const size_t padded_pairs = (size_t)((T_ + kSweepTokens - 1) / kSweepTokens * kSweepTokens) * (size_t)K;
    p.off_sweep_keys = take(p.sweep ? padded_pairs * 4 : 0);
    p.off_sweep_coef = take(p.sweep ? padded_pairs * 4 : 0);
    p.bytes = o;
    return p;
}

bool bucketed_possible(int64_t T_, int64_t E, int H, int K, size_t elt) {
    return (H * elt) % 128 == 0 &&      // whole 128-byte bands
           (uint64_t)E * (uint64_t)H * elt < (uint64_t)kBadOffset && (uint64_t)T_ * (uint64_t)H * elt < (uint64_t)kBadOffset &&
           T_ * (int64_t)K < (1ll << 31) - 4096 && E < (1ll << 31) - 1 && T_ <= (int64_t)kEntryTokenMask &&
           (sweep_possible(T_, H, E, K, elt) || rows_possible(H, elt));     // its second phase: the sweep, or the row kernel
}

template <typename T>
int launch_expert_bucketed(int act, const void* x, const void* down, const void* up, const int64_t* indices, const void* gates,
                           int64_t T_, int H, int64_t E, int K, void* out, void* workspace, hipStream_t stream) {
    const BucketedPlan p = plan_bucketed(T_, H, E, K, sizeof(T));
    char* ws = (char*)workspace;
    int32_t* offsets = (int32_t*)(ws + p.off_offsets);
    int32_t* sorted_pairs = (int32_t*)(ws + p.off_pairs);
    uint32_t* tokoff = (uint32_t*)(ws + p.off_tok);
    uint32_t* expoff = (uint32_t*)(ws + p.off_exp);
    float* a = (float*)(ws + p.off_a);
    float* spart = (float*)(ws + p.off_spart);
    const int64_t pairs = T_ * K;
    const uint32_t row_bytes = (uint32_t)(H * sizeof(T));
    if (act == kActNone) {
        // no score phase: the coefficient is the routing weight itself, nothing to group
        return launch_expert_rows<T>(act, x, down, up, indices, gates, T_, H, E, K, out, stream);
    }
    if (bucket_partition_pays(pairs, E)) {
        if (int rc = bucket_partition(indices, ws + p.off_part, pairs, E, K, offsets, sorted_pairs, tokoff, 1u, expoff, 1u, a, 24,
                                      stream))
            return rc;
    } else {
        if (int rc = bucket_clear(ws + p.off_bucket, E, stream)) return rc;
        if (int rc = bucket_histogram(indices, ws + p.off_bucket, pairs, E, stream)) return rc;
        if (int rc = bucket_scan_fill(indices, ws + p.off_bucket, pairs, E, K, offsets, sorted_pairs, tokoff, 1u, expoff, 1u, a,
                                      24, 0, stream))
            return rc;
    }
    void* xb = ws + p.off_xb;
    {
        const int64_t packets = T_ * (int64_t)(row_bytes / 16);
        hipLaunchKernelGGL(expert_band_copy_kernel, dim3((unsigned)((packets + 255) / 256)), dim3(256), 0, stream,
                           (const u32x4_t*)x, (u32x4_t*)xb, T_, (int)(row_bytes / 16), p.chunk_lanes);
        FMOE_CHECK_LAUNCH("fmoe_expert_forward(band copy)");
    }
    const uint32_t x_bytes = (uint32_t)(T_ * (int64_t)row_bytes), table_bytes = (uint32_t)(E * (int64_t)row_bytes);
#define FMOE_LAUNCH_BUCKETED(CLV)                                                                                          \
    hipLaunchKernelGGL((expert_scores_bucketed_kernel<T, CLV>), dim3(p.grid), dim3(256), 0, stream, (const T*)xb, x_bytes,  \
                       (const T*)down, table_bytes, (const uint32_t*)tokoff, (const uint32_t*)expoff, (const int32_t*)offsets, \
                       E, spart, pairs, row_bytes, p.num_bands, p.parts, p.blocks_per_unit, p.xcds)
    if (p.chunk_lanes == 32) FMOE_LAUNCH_BUCKETED(32);
    else if (p.chunk_lanes == 16) FMOE_LAUNCH_BUCKETED(16);
    else FMOE_LAUNCH_BUCKETED(8);
#undef FMOE_LAUNCH_BUCKETED
    FMOE_CHECK_LAUNCH("fmoe_expert_forward(bucketed scores)");
    const unsigned flat_grid = (unsigned)((pairs + 255) / 256 < 16384 ? (pairs + 255) / 256 : 16384);
    if (act == kActSilu)
        hipLaunchKernelGGL((expert_gate_sorted_kernel<T, kActSilu>), dim3(flat_grid), dim3(256), 0, stream, (const float*)spart,
                           pairs, (const T*)gates, (const int32_t*)sorted_pairs, (const int32_t*)offsets, E, a, p.num_bands);
    else
        hipLaunchKernelGGL((expert_gate_sorted_kernel<T, kActGelu>), dim3(flat_grid), dim3(256), 0, stream, (const float*)spart,
                           pairs, (const T*)gates, (const int32_t*)sorted_pairs, (const int32_t*)offsets, E, a, p.num_bands);
    FMOE_CHECK_LAUNCH("fmoe_expert_forward(bucketed gate)");
    if constexpr (sizeof(T) == 2) {
        if (p.sweep) {
            uint32_t* keys = (uint32_t*)(ws + p.off_sweep_keys);
            float* coef = (float*)(ws + p.off_sweep_coef);
            const int64_t owners = (T_ + kSweepTokens - 1) / kSweepTokens;
            hipLaunchKernelGGL(expert_owner_sort_kernel, dim3((unsigned)owners), dim3(256), 0, stream, indices, (const float*)a,
                               keys, coef, T_, E, K);
            FMOE_CHECK_LAUNCH("fmoe_expert_forward(owner sort)");
            const int bands = (int)(row_bytes / 128);
            const int token_blocks = (int)((T_ + kSweepWgTokens - 1) / kSweepWgTokens);
            const unsigned grid = (unsigned)(p.xcds * token_blocks * ((bands + p.xcds - 1) / p.xcds));
            hipLaunchKernelGGL((expert_states_sweep_kernel<T>), dim3(grid), dim3(kSweepThreads), 0, stream, (const T*)up,
                               table_bytes, (const uint32_t*)keys, (const float*)coef, (T*)out, T_, E, K, row_bytes, bands,
                               token_blocks, p.xcds);
            FMOE_CHECK_LAUNCH("fmoe_expert_forward(sweep)");
            return FMOE_OK;
        }
    }
    return launch_expert_rows_coef<T>(up, indices, a, T_, H, E, K, out, stream);
}

// A slice of the table must stay resident in one XCD's L2 (4 MiB) next to the streaming traffic; with 128-byte
// slices of up to twice the L2 the measured gather rate is still twice the fabric's.  Beyond that, and for problems with
// too few pairs to pay for four launches, whole rows are gathered by the one-wave-per-token kernel.
bool slices_pay(int64_t T_, int64_t E, int K) { return E * 128 <= 2 * chip_info().l2_bytes && T_ * K >= (1ll << 16); }
// rows are addressed with 32-bit byte offsets below kBadOffset
bool slices_possible(int64_t E, int H, size_t elt) { return (uint64_t)E * (uint64_t)H * elt < (uint64_t)kBadOffset; }

// column slices: when they pay, and for rows too long for the row kernels whatever the problem size
bool slices_chosen(int64_t T_, int H, int64_t E, int K, size_t elt) {
    return slices_possible(E, H, elt) && (slices_pay(T_, E, K) || !rows_possible(H, elt));
}

// Which schedule a call takes.  A forced schedule that cannot run these extents is reported by the dispatcher; AUTO
// falls back to whole rows.
// Grouping the pairs by expert pays once an expert's row serves about a dozen pairs (measured: 16 pairs per expert, bucketed
// 10-25 % ahead of whole-row gathers; 8 pairs per expert, 15 % behind): below that the rows are better gathered whole, straight
// from HBM.
bool buckets_pay(int64_t T_, int64_t E, int K) { return !slices_pay(T_, E, K) && T_ * K >= (1ll << 16) && T_ * K >= 12 * E; }
int choose_schedule(int algo, int64_t T_, int H, int64_t E, int K, size_t elt, bool scored = true) {
    if (K == 0) return FMOE_EXPERT_ROWS;
    if (algo != FMOE_EXPERT_AUTO) return algo;
    if (slices_chosen(T_, H, E, K, elt)) return FMOE_EXPERT_SLICES;
    // grouping by expert serves the score phase; an op without scores (product-key memory) has nothing to group
    if (scored && buckets_pay(T_, E, K) && bucketed_possible(T_, E, H, K, elt)) return FMOE_EXPERT_BUCKETS;
    return FMOE_EXPERT_ROWS;
}

}  // namespace

bool expert_slices_usable(int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype) {
    return top_k > 0 && slices_chosen(num_tokens, hidden, num_experts, top_k, dtype_size(dtype));
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
    const size_t elt = dtype_size(dtype);
    switch (choose_schedule(algo, num_tokens, hidden, num_experts, top_k, elt)) {
        case FMOE_EXPERT_SLICES: return plan_slices(num_tokens, hidden, num_experts, top_k, elt).bytes;
        case FMOE_EXPERT_BUCKETS: return plan_bucketed(num_tokens, hidden, num_experts, top_k, elt).bytes;
        default: return 0;   // the row schedule needs no scratch
    }
}

extern "C" size_t fmoe_expert_workspace_bytes(int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype) {
    return fmoe_expert_workspace_bytes_algo(num_tokens, hidden, num_experts, top_k, dtype, FMOE_EXPERT_AUTO);
}

extern "C" size_t fmoe_pkm_workspace_bytes(int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype) {
    using namespace fmoe;
    if (num_tokens <= 0 || hidden <= 0 || num_experts <= 0 || top_k <= 0 || !dtype_ok(dtype)) return 0;
    const size_t elt = dtype_size(dtype);
    return choose_schedule(FMOE_EXPERT_AUTO, num_tokens, hidden, num_experts, top_k, elt, false) == FMOE_EXPERT_SLICES
               ? plan_slices(num_tokens, hidden, num_experts, top_k, elt).bytes
               : 0;
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
    FMOE_REQUIRE(algo >= FMOE_EXPERT_AUTO && algo <= FMOE_EXPERT_BUCKETS, FMOE_ERR_UNSUPPORTED,
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
    const size_t elt = dtype_size(dtype);
    const int schedule = choose_schedule(algo, num_tokens, hidden, num_experts, top_k, elt, act != kActNone);
    FMOE_REQUIRE(schedule != FMOE_EXPERT_SLICES || slices_possible(num_experts, hidden, elt), FMOE_ERR_UNSUPPORTED,
                 "%s: tables of 4 GiB or more cannot use the column-slice schedule", who);
    FMOE_REQUIRE(schedule != FMOE_EXPERT_BUCKETS || bucketed_possible(num_tokens, num_experts, hidden, top_k, elt),
                 FMOE_ERR_UNSUPPORTED, "%s: the bucketed schedule needs rows that are multiples of 128 bytes (16-bit, or at most 8192 bytes), x and each table below 4 GiB and fewer than 2^31 pairs", who);
    if (schedule == FMOE_EXPERT_BUCKETS) {
        const size_t need = fmoe_expert_workspace_bytes_algo(num_tokens, hidden, num_experts, top_k, dtype, FMOE_EXPERT_BUCKETS);
        FMOE_REQUIRE(workspace && workspace_bytes >= need && aligned16(workspace), FMOE_ERR_WORKSPACE,
                     "%s: workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
        switch (dtype) {
            case FMOE_F32: return launch_expert_bucketed<float>(act, x, down, up, indices, gates, num_tokens, hidden, num_experts, top_k, out, workspace, s);
            case FMOE_BF16: return launch_expert_bucketed<bf16_t>(act, x, down, up, indices, gates, num_tokens, hidden, num_experts, top_k, out, workspace, s);
            default: return launch_expert_bucketed<f16_t>(act, x, down, up, indices, gates, num_tokens, hidden, num_experts, top_k, out, workspace, s);
        }
    }
    if (schedule == FMOE_EXPERT_SLICES) {
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
