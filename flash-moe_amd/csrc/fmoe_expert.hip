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

namespace fmoe {
namespace {

constexpr int kPairsInFlight = 4;   // (down,up) row pairs requested ahead per wave
constexpr int kWavesPerBlock = 4;

// dot of two 16-byte packets, accumulated into acc
template <typename T> __device__ inline float dot16(u32x4_t a, u32x4_t b, float acc);
template <> __device__ inline float dot16<float>(u32x4_t a, u32x4_t b, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_fmaf(__uint_as_float(a[i]), __uint_as_float(b[i]), acc);
    return acc;
}
template <> __device__ inline float dot16<bf16_t>(u32x4_t a, u32x4_t b, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        // element first into a scalar: bit-casting the subscript expression itself reads element 0
        const uint32_t ai = a[i], bi = b[i];
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, ai), __builtin_bit_cast(bf16x2_t, bi), acc, false);
    }
    return acc;
}
template <> __device__ inline float dot16<f16_t>(u32x4_t a, u32x4_t b, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t ai = a[i], bi = b[i];
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, ai), __builtin_bit_cast(f16x2_t, bi), acc, false);
    }
    return acc;
}

// acc[0..kVec) += s * packet
template <typename T> __device__ inline void axpy16(float s, u32x4_t w, float* acc);
template <> __device__ inline void axpy16<float>(float s, u32x4_t w, float* acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = __builtin_fmaf(s, __uint_as_float(w[i]), acc[i]);
}
template <> __device__ inline void axpy16<bf16_t>(float s, u32x4_t w, float* acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        acc[2 * i] = __builtin_fmaf(s, __uint_as_float(w[i] << 16), acc[2 * i]);
        acc[2 * i + 1] = __builtin_fmaf(s, __uint_as_float(w[i] & 0xffff0000u), acc[2 * i + 1]);
    }
}
template <> __device__ inline void axpy16<f16_t>(float s, u32x4_t w, float* acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t wi = w[i];
        f16x2_t p = __builtin_bit_cast(f16x2_t, wi);
        acc[2 * i] = __builtin_fmaf(s, (float)p[0], acc[2 * i]);
        acc[2 * i + 1] = __builtin_fmaf(s, (float)p[1], acc[2 * i + 1]);
    }
}

template <typename T> __device__ inline u32x4_t pack16(const float* v);
template <> __device__ inline u32x4_t pack16<float>(const float* v) {
    u32x4_t r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = __float_as_uint(v[i]);
    return r;
}
template <> __device__ inline u32x4_t pack16<bf16_t>(const float* v) {
    u32x4_t r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        bf16x2_t p = {(bf16_t)v[2 * i], (bf16_t)v[2 * i + 1]};
        r[i] = __builtin_bit_cast(uint32_t, p);
    }
    return r;
}
template <> __device__ inline u32x4_t pack16<f16_t>(const float* v) {
    u32x4_t r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f16x2_t p = {(f16_t)v[2 * i], (f16_t)v[2 * i + 1]};
        r[i] = __builtin_bit_cast(uint32_t, p);
    }
    return r;
}

// NCH = number of 16-byte packets each lane holds per row: a row has at most NCH*64 packets.
template <typename T, int NCH>
__global__ __launch_bounds__(kWavesPerBlock* kWave) void expert_token_kernel(
    const T* __restrict__ x, const T* __restrict__ down, const T* __restrict__ up,
    const int64_t* __restrict__ indices, const T* __restrict__ gates, T* __restrict__ out,
    int64_t num_tokens, int hidden, int64_t num_experts, int top_k) {
    constexpr int V = Elem<T>::kVec;
    const int lane = lane_id();
    const int64_t token = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (token >= num_tokens) return;   // whole wave leaves together

    const int packets = hidden / V;   // 16-byte packets per row (hidden % V == 0 is checked on the host)
    const u32x4_t zero4 = {0u, 0u, 0u, 0u};

    u32x4_t xr[NCH];
    bool live[NCH];
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int p = c * kWave + lane;
        live[c] = p < packets;
        xr[c] = live[c] ? reinterpret_cast<const u32x4_t*>(x + token * hidden)[p] : zero4;
    }

    float acc[NCH][V];
#pragma unroll
    for (int c = 0; c < NCH; ++c)
#pragma unroll
        for (int v = 0; v < V; ++v) acc[c][v] = 0.0f;

    const int64_t* my_idx = indices + token * top_k;
    const T* my_gate = gates + token * top_k;

    for (int k0 = 0; k0 < top_k; k0 += kPairsInFlight) {
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
                dn[u][c] = (ok && live[c]) ? drow[p] : zero4;
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
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1)
#pragma unroll
            for (int u = 0; u < kPairsInFlight; ++u) s[u] += __shfl_xor(s[u], m, kWave);
#pragma unroll
        for (int u = 0; u < kPairsInFlight; ++u) {
            const float a = silu_f32(s[u]) * gate[u];
#pragma unroll
            for (int c = 0; c < NCH; ++c) axpy16<T>(a, uq[u][c], acc[c]);
        }
    }

#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int p = c * kWave + lane;
        if (live[c]) reinterpret_cast<u32x4_t*>(out + token * hidden)[p] = pack16<T>(acc[c]);
    }
}

template <typename T>
int launch_expert(const void* x, const void* down, const void* up, const int64_t* indices, const void* gates,
                  int64_t T_, int H, int64_t E, int K, void* out, hipStream_t stream) {
    constexpr int V = Elem<T>::kVec;
    const int packets = H / V;
    const int nch = (packets + kWave - 1) / kWave;
    const dim3 block(kWavesPerBlock * kWave);
    const dim3 grid((unsigned)((T_ + kWavesPerBlock - 1) / kWavesPerBlock));
#define FMOE_LAUNCH_EXPERT(N)                                                                            \
    hipLaunchKernelGGL((expert_token_kernel<T, N>), grid, block, 0, stream, (const T*)x, (const T*)down, \
                       (const T*)up, indices, (const T*)gates, (T*)out, T_, H, E, K)
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
    FMOE_CHECK_LAUNCH("fmoe_expert_forward");
    return FMOE_OK;
}

}  // namespace
}  // namespace fmoe

extern "C" size_t fmoe_expert_workspace_bytes(int64_t, int, int64_t, int, int) { return 0; }

extern "C" int fmoe_expert_forward(const void* x, const void* down, const void* up, const int64_t* indices,
                                   const void* gates, int64_t num_tokens, int hidden, int64_t num_experts,
                                   int top_k, int dtype, void* out, void* workspace, size_t workspace_bytes,
                                   void* stream) {
    using namespace fmoe;
    (void)workspace;
    (void)workspace_bytes;
    clear_error();
    FMOE_REQUIRE(dtype_ok(dtype), FMOE_ERR_BAD_DTYPE, "fmoe_expert_forward: unknown dtype %d", dtype);
    FMOE_REQUIRE(num_tokens >= 0 && hidden > 0 && num_experts > 0 && top_k >= 0, FMOE_ERR_BAD_SHAPE,
                 "fmoe_expert_forward: bad shape T=%lld H=%d E=%lld K=%d", (long long)num_tokens, hidden,
                 (long long)num_experts, top_k);
    if (num_tokens == 0) return FMOE_OK;
    FMOE_REQUIRE(x && down && up && out, FMOE_ERR_NULL_POINTER, "fmoe_expert_forward: null tensor pointer");
    FMOE_REQUIRE(top_k == 0 || (indices && gates), FMOE_ERR_NULL_POINTER,
                 "fmoe_expert_forward: null indices/gates with top_k=%d", top_k);
    const int vec = (int)(16 / dtype_size(dtype));
    FMOE_REQUIRE(hidden % vec == 0, FMOE_ERR_ALIGNMENT,
                 "fmoe_expert_forward: hidden=%d must be a multiple of %d (16-byte rows)", hidden, vec);
    FMOE_REQUIRE(aligned16(x) && aligned16(down) && aligned16(up) && aligned16(out), FMOE_ERR_ALIGNMENT,
                 "fmoe_expert_forward: tensor pointers must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case FMOE_F32: return launch_expert<float>(x, down, up, indices, gates, num_tokens, hidden, num_experts, top_k, out, s);
        case FMOE_BF16: return launch_expert<bf16_t>(x, down, up, indices, gates, num_tokens, hidden, num_experts, top_k, out, s);
        default: return launch_expert<f16_t>(x, down, up, indices, gates, num_tokens, hidden, num_experts, top_k, out, s);
    }
}
