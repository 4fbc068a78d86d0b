// Backward passes of the router op, the SwiGLU gate and the routed-expert op for gfx950.
//
//   router  : drouter_logits[0,t,i] = sum_{k : idx[t,k] / nk == i} dscores[t,k],  [1,t,j] likewise with idx % nk
//   route   : gates = exp(top-k sums of the per-half log-softmax), renormalised or not -> gradient of the gate logits
//   swiglu  : c = silu(a) * b  ->  da = dc * (silu(a) * (1 - sigmoid(a)) + sigmoid(a)) * b,  db = dc * silu(a)
//   experts : out[t] = sum_k silu(s) * g * up[e],  s = <x[t], down[e]>,  e = idx[t,k]:
//               da_p   = <dout[t], up[e]>                 dg_p = da_p * silu(s)
//               ds_p   = da_p * g * sigmoid(s) * (1 + s * (1 - sigmoid(s)))
//               dx[t]  = sum_k ds_p * down[e]
//               ddown[e] = sum_{p -> e} ds_p * x[t_p]     dup[e] = sum_{p -> e} silu(s_p) * g_p * dout[t_p]
//
// No floating-point atomics on global memory: every output element is written once and sums run in a fixed order
// (pairs of an expert in ascending pair index), so gradients are reproducible bit for bit.  The per-token part of the
// expert backward is one wave per token with the token's rows of x and dout in registers (the layout of the forward
// row kernel).  The per-expert part needs the pairs grouped by expert: the bucketing stage (fmoe_bucket.hip: integer
// histogram taken by the per-token kernels, scan, fill, ordering pass) gives each expert one segment listing its pairs in
// ascending pair index, and the wave that owns the expert walks it in that order.
#include "fmoe_common.h"
#include "fmoe_vec.h"

namespace fmoe {
namespace {

constexpr int kBwdWaves = 4;

// ------------------------------------------------------------------------------------------------------------
// router
// ------------------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kBwdWaves* kWave) void router_backward_kernel(const T* __restrict__ dscores,
                                                                           const int64_t* __restrict__ indices,
                                                                           T* __restrict__ dlogits, int64_t num_tokens,
                                                                           int nk, int top_k, int waves_per_block, int chunk) {
    extern __shared__ float acc_all[];   // [waves_per_block][2 * chunk], one private row pair per wave
    const int lane = lane_id();
    const int wave = (int)(threadIdx.x >> 6);
    const int64_t token = (int64_t)blockIdx.x * waves_per_block + wave;
    if (wave >= waves_per_block || token >= num_tokens) return;   // whole waves leave; nobody waits on them
    float* acc = acc_all + (size_t)wave * 2 * chunk;
    const int64_t num_pairs = (int64_t)nk * nk;
    // The two gradient rows are built `chunk` keys at a time (chunk = nk when a row pair fits the LDS): per chunk the
    // pairs are scanned again and only the keys inside it are added.
    for (int c0 = 0; c0 < nk; c0 += chunk) {
        const int cn = nk - c0 < chunk ? nk - c0 : chunk;
        for (int p = lane; p < 2 * chunk; p += kWave) acc[p] = 0.0f;
        __builtin_amdgcn_wave_barrier();
        // LDS adds of one instruction that hit the same address are applied one after the other by the LDS unit, and the
        // instructions of a wave execute in order, so the sum has a fixed order for given inputs
        for (int k = lane; k < top_k; k += kWave) {
            const int64_t id = indices[token * top_k + k];
            if (id >= 0 && id < num_pairs) {
                const float d = Elem<T>::to_f32(dscores[token * top_k + k]);
                const int i = (int)(id / nk) - c0, j = (int)(id % nk) - c0;
                if (i >= 0 && i < cn) __hip_atomic_fetch_add(&acc[i], d, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
                if (j >= 0 && j < cn) __hip_atomic_fetch_add(&acc[chunk + j], d, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
            }
        }
        __builtin_amdgcn_wave_barrier();
        for (int p = lane; p < cn; p += kWave) {
            dlogits[token * nk + c0 + p] = Elem<T>::from_f32(acc[p]);
            dlogits[(num_tokens + token) * nk + c0 + p] = Elem<T>::from_f32(acc[chunk + p]);
        }
        __builtin_amdgcn_wave_barrier();
    }
}

// Keys of a half whose gradient row is held in LDS at a time: the whole half up to 8192 keys (64 KiB for the pair of
// rows), 4096 beyond.
inline int backward_key_chunk(int nk) { return nk <= 8192 ? nk : 4096; }

template <typename T>
int launch_router_backward(const void* dscores, const int64_t* indices, void* dlogits, int64_t T_, int nk, int K,
                           hipStream_t stream) {
    const int chunk = backward_key_chunk(nk);
    const size_t per_wave = (size_t)2 * chunk * sizeof(float);
    int waves = (int)((48 * 1024) / per_wave);
    waves = waves < 1 ? 1 : (waves > kBwdWaves ? kBwdWaves : waves);
    const unsigned grid = (unsigned)((T_ + waves - 1) / waves);
    hipLaunchKernelGGL((router_backward_kernel<T>), dim3(grid), dim3(kBwdWaves * kWave), waves * per_wave, stream,
                       (const T*)dscores, indices, (T*)dlogits, T_, nk, K, waves, chunk);
    FMOE_CHECK_LAUNCH("fmoe_router_topk_backward");
    return FMOE_OK;
}

// Routing stage between the gate logits and the gates, backward in one launch: exp / renormalisation, the scatter of the
// score gradients onto the two key rows, and the per-half log-softmax.  One wave per token; the log-probabilities are
// recomputed from the fp32 logits exactly as the forward computes them ((v - max) - log(sum exp(v - max))).
//   s_k = lp0[i_k] + lp1[j_k],  e_k = exp(s_k),  g_k = e_k  or  e_k / sum_m e_m
//   ds_k = dg_k * e_k                       (no renormalisation)
//   ds_k = g_k * (dg_k - sum_m dg_m g_m)    (renormalised)
//   dlp[h][i] = sum of ds_k over the pairs that use key i of half h
//   dlogits[h][i] = dlp[h][i] - softmax(logits[h])[i] * sum_i dlp[h][i]   (+ the gradient of the returned logits)
template <typename T>
__global__ __launch_bounds__(kBwdWaves* kWave) void route_backward_kernel(
    const T* __restrict__ dgates, const int64_t* __restrict__ indices, const float* __restrict__ logits,
    const T* __restrict__ dlogits_extra, float* __restrict__ dlogits, int64_t num_tokens, int nk, int top_k,
    int norm_topk_prob, int waves_per_block, int chunk) {
    extern __shared__ float acc_all[];   // [waves_per_block][2 * chunk], one private row pair per wave
    const int lane = lane_id();
    const int wave = (int)(threadIdx.x >> 6);
    const int64_t token = (int64_t)blockIdx.x * waves_per_block + wave;
    if (wave >= waves_per_block || token >= num_tokens) return;   // whole waves leave; nobody waits on them
    float* acc = acc_all + (size_t)wave * 2 * chunk;
    const float* row = logits + token * 2 * nk;
    float shift[2], lse[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        float mx = -INFINITY;
        for (int p = lane; p < nk; p += kWave) mx = fmaxf(mx, row[h * nk + p]);
        mx = wave_max(mx);
        float se = 0.0f;
        for (int p = lane; p < nk; p += kWave) se += expf(row[h * nk + p] - mx);
        shift[h] = mx;
        lse[h] = logf(wave_sum(se));
    }
    const int64_t num_pairs = (int64_t)nk * nk;
    // first pass (renormalised gates only): sum_m e_m and sum_m dg_m e_m
    float total = 1.0f, dot = 0.0f;
    if (norm_topk_prob) {
        float te = 0.0f, td = 0.0f;
        for (int k = lane; k < top_k; k += kWave) {
            const int64_t id = indices[token * top_k + k];
            if (id >= 0 && id < num_pairs) {
                const int i = (int)(id / nk), j = (int)(id % nk);
                const float e = expf(((row[i] - shift[0]) - lse[0]) + ((row[nk + j] - shift[1]) - lse[1]));
                te += e;
                td = __builtin_fmaf(Elem<T>::to_f32(dgates[token * top_k + k]), e, td);
            }
        }
        total = wave_sum(te);
        dot = wave_sum(td) / total;          // sum_m dg_m g_m
    }
    // The two gradient rows are built `chunk` keys at a time (chunk = nk when a row pair fits the LDS): per chunk the
    // pairs are scanned again and only the keys inside it are added.  With several chunks the row totals, which every
    // key's result needs, are the sum of the pair gradients themselves (each valid pair adds to one key of either half).
    const bool chunked = chunk < nk;
    float sum_all = 0.0f;
    if (chunked) {
        float part = 0.0f;
        for (int k = lane; k < top_k; k += kWave) {
            const int64_t id = indices[token * top_k + k];
            if (id >= 0 && id < num_pairs) {
                const int i = (int)(id / nk), j = (int)(id % nk);
                const float e = expf(((row[i] - shift[0]) - lse[0]) + ((row[nk + j] - shift[1]) - lse[1]));
                const float dg = Elem<T>::to_f32(dgates[token * top_k + k]);
                part += norm_topk_prob ? (e / total) * (dg - dot) : dg * e;
            }
        }
        sum_all = wave_sum(part);
    }
    for (int c0 = 0; c0 < nk; c0 += chunk) {
        const int cn = nk - c0 < chunk ? nk - c0 : chunk;
        for (int p = lane; p < 2 * chunk; p += kWave) acc[p] = 0.0f;
        __builtin_amdgcn_wave_barrier();
        // LDS adds of one instruction that hit the same address are applied one after the other by the LDS unit, and the
        // instructions of a wave execute in order, so the sum has a fixed order for given inputs
        for (int k = lane; k < top_k; k += kWave) {
            const int64_t id = indices[token * top_k + k];
            if (id >= 0 && id < num_pairs) {
                const int i = (int)(id / nk), j = (int)(id % nk);
                const float e = expf(((row[i] - shift[0]) - lse[0]) + ((row[nk + j] - shift[1]) - lse[1]));
                const float dg = Elem<T>::to_f32(dgates[token * top_k + k]);
                const float ds = norm_topk_prob ? (e / total) * (dg - dot) : dg * e;
                if (i >= c0 && i < c0 + cn) __hip_atomic_fetch_add(&acc[i - c0], ds, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
                if (j >= c0 && j < c0 + cn) __hip_atomic_fetch_add(&acc[chunk + j - c0], ds, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
            }
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            float sum = sum_all;
            if (!chunked) {
                sum = 0.0f;
                for (int p = lane; p < nk; p += kWave) sum += acc[h * chunk + p];
                sum = wave_sum(sum);
            }
            for (int p = lane; p < cn; p += kWave) {
                const int64_t at = token * 2 * nk + h * nk + c0 + p;
                float d = acc[h * chunk + p] - expf((row[h * nk + c0 + p] - shift[h]) - lse[h]) * sum;
                if (dlogits_extra != nullptr) d += Elem<T>::to_f32(dlogits_extra[at]);
                dlogits[at] = d;
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
}

template <typename T>
int launch_route_backward(const void* dgates, const int64_t* indices, const float* logits, const void* dlogits_extra,
                          float* dlogits, int64_t T_, int nk, int K, int norm, hipStream_t stream) {
    const int chunk = backward_key_chunk(nk);
    const size_t per_wave = (size_t)2 * chunk * sizeof(float);
    int waves = (int)((48 * 1024) / per_wave);
    waves = waves < 1 ? 1 : (waves > kBwdWaves ? kBwdWaves : waves);
    const unsigned grid = (unsigned)((T_ + waves - 1) / waves);
    hipLaunchKernelGGL((route_backward_kernel<T>), dim3(grid), dim3(kBwdWaves * kWave), waves * per_wave, stream,
                       (const T*)dgates, indices, logits, (const T*)dlogits_extra, dlogits, T_, nk, K, norm, waves, chunk);
    FMOE_CHECK_LAUNCH("fmoe_route_backward");
    return FMOE_OK;
}

// ------------------------------------------------------------------------------------------------------------
// SwiGLU
// ------------------------------------------------------------------------------------------------------------
// One 16-byte packet per thread; workgroup b works on row b / col_blocks.  Row strides (elements) let da / db / h live
// side by side in wider buffers.
template <typename T>
__global__ __launch_bounds__(256) void swiglu_backward_kernel(const T* __restrict__ dc, const T* __restrict__ a,
                                                              const T* __restrict__ b, T* __restrict__ da,
                                                              T* __restrict__ db, T* __restrict__ h, int col_blocks,
                                                              int cols, int64_t da_stride, int64_t db_stride) {
    constexpr int V = Elem<T>::kVec;
    const uint32_t row = blockIdx.x / (uint32_t)col_blocks;
    const int col = ((int)(blockIdx.x % (uint32_t)col_blocks) * 256 + (int)threadIdx.x) * V;
    if (col >= cols) return;
    const int64_t at = (int64_t)row * cols + col;
    float dcv[V], av[V], bv[V], dav[V], dbv[V], hv[V];
    unpack16<T>(*reinterpret_cast<const u32x4_t*>(dc + at), dcv);
    unpack16<T>(*reinterpret_cast<const u32x4_t*>(a + at), av);
    unpack16<T>(*reinterpret_cast<const u32x4_t*>(b + at), bv);
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const float sig = 1.0f / (1.0f + __expf(-av[v]));
        const float silu = av[v] * sig;
        dbv[v] = dcv[v] * silu;
        dav[v] = dcv[v] * (silu * (1.0f - sig) + sig) * bv[v];
        hv[v] = silu * bv[v];
    }
    *reinterpret_cast<u32x4_t*>(da + row * da_stride + col) = pack16<T>(dav);
    *reinterpret_cast<u32x4_t*>(db + row * db_stride + col) = pack16<T>(dbv);
    if (h != nullptr) *reinterpret_cast<u32x4_t*>(h + at) = pack16<T>(hv);
}

// ------------------------------------------------------------------------------------------------------------
// routed experts, per-token part: dx, dgates and the two coefficients of every pair
// ------------------------------------------------------------------------------------------------------------
template <typename T, int NCH>
__global__ __launch_bounds__(kBwdWaves* kWave) void expert_backward_token_kernel(
    const T* __restrict__ dout, const T* __restrict__ x, const T* __restrict__ down, const T* __restrict__ up,
    const int64_t* __restrict__ indices, const T* __restrict__ gates, T* __restrict__ dx, T* __restrict__ dgates,
    float* __restrict__ coef_up, float* __restrict__ coef_down, int32_t* __restrict__ counts, int64_t num_tokens,
    int hidden, int64_t num_experts, int top_k) {
    constexpr int V = Elem<T>::kVec;
    constexpr int PIF = NCH >= 8 ? 1 : (NCH >= 4 ? 2 : 4);   // (down, up) row pairs requested ahead
    const int lane = lane_id();
    const int64_t token = (int64_t)blockIdx.x * kBwdWaves + (threadIdx.x >> 6);
    if (token >= num_tokens) return;

    const int packets = hidden / V;
    const u32x4_t zero4 = {0u, 0u, 0u, 0u};
    u32x4_t xr[NCH], gr[NCH];
    bool live[NCH];
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int p = c * kWave + lane;
        live[c] = p < packets;
        xr[c] = live[c] ? reinterpret_cast<const u32x4_t*>(x + token * hidden)[p] : zero4;
        gr[c] = live[c] ? reinterpret_cast<const u32x4_t*>(dout + token * hidden)[p] : zero4;
    }
    float acc[NCH][V];
#pragma unroll
    for (int c = 0; c < NCH; ++c)
#pragma unroll
        for (int v = 0; v < V; ++v) acc[c][v] = 0.0f;

    for (int k0 = 0; k0 < top_k; k0 += PIF) {
        u32x4_t dn[PIF][NCH], uq[PIF][NCH];
        float gate[PIF];
        bool valid[PIF];
        int64_t expert[PIF];
#pragma unroll
        for (int u = 0; u < PIF; ++u) {
            const int k = k0 + u;
            int64_t e = -1;
            gate[u] = 0.0f;
            if (k < top_k) {
                e = indices[token * top_k + k];
                gate[u] = Elem<T>::to_f32(gates[token * top_k + k]);
            }
            const uint32_t elo = __builtin_amdgcn_readfirstlane((uint32_t)(e & 0xffffffff));
            const uint32_t ehi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)e >> 32));
            e = (int64_t)(((uint64_t)ehi << 32) | elo);
            valid[u] = e >= 0 && e < num_experts;
            expert[u] = e;
            const u32x4_t* drow = reinterpret_cast<const u32x4_t*>(down + (valid[u] ? e : 0) * hidden);
            const u32x4_t* urow = reinterpret_cast<const u32x4_t*>(up + (valid[u] ? e : 0) * hidden);
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                const int p = c * kWave + lane;
                dn[u][c] = (valid[u] && live[c]) ? drow[p] : zero4;
                uq[u][c] = (valid[u] && live[c]) ? urow[p] : zero4;
            }
        }
        float s[PIF], da[PIF];
#pragma unroll
        for (int u = 0; u < PIF; ++u) {
            float ps = 0.0f, pa = 0.0f;
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                ps = dot16<T>(xr[c], dn[u][c], ps);
                pa = dot16<T>(gr[c], uq[u][c], pa);
            }
            s[u] = ps;
            da[u] = pa;
        }
#pragma unroll
        for (int u = 0; u < PIF; ++u) {
            s[u] = wave_sum(s[u]);
            da[u] = wave_sum(da[u]);
        }
#pragma unroll
        for (int u = 0; u < PIF; ++u) {
            const int k = k0 + u;
            const float sig = 1.0f / (1.0f + __expf(-s[u]));
            const float act = s[u] * sig;
            const float ds = valid[u] ? da[u] * gate[u] * (sig * (1.0f + s[u] * (1.0f - sig))) : 0.0f;
#pragma unroll
            for (int c = 0; c < NCH; ++c) axpy16<T>(ds, dn[u][c], acc[c]);
            if (lane == 0 && k < top_k) {
                const int64_t p = token * top_k + k;
                coef_up[p] = valid[u] ? act * gate[u] : 0.0f;
                coef_down[p] = ds;
                dgates[p] = Elem<T>::from_f32(valid[u] ? da[u] * act : 0.0f);
                if (valid[u]) atomicAdd(&counts[expert[u]], 1);   // integer histogram: the result does not depend on order
            }
        }
    }
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int p = c * kWave + lane;
        if (live[c]) reinterpret_cast<u32x4_t*>(dx + token * hidden)[p] = pack16<T>(acc[c]);
    }
}

// Column-slice schedule of the per-token part (same kernels as the forward, fmoe_expert.hip): the partial dot products
// s = <x, down[e]> and u = <dout, up[e]> come per slice; this kernel sums them and forms every pair's coefficients,
// gate gradient and histogram entry; dx is then the forward's `states` pass over `down` with coef_down.
template <typename T>
__global__ __launch_bounds__(256) void expert_backward_gate_kernel(
    const float* __restrict__ spart_s, const float* __restrict__ spart_u, const T* __restrict__ gates,
    const uint32_t* __restrict__ off32, const int64_t* __restrict__ indices, T* __restrict__ dgates,
    float* __restrict__ coef_up, float* __restrict__ coef_down, int32_t* __restrict__ counts, int64_t pairs, int num_slices) {
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= pairs) return;
    float s = 0.0f, u = 0.0f;
    for (int sl = 0; sl < num_slices; ++sl) {
        s += spart_s[(int64_t)sl * pairs + p];
        u += spart_u[(int64_t)sl * pairs + p];
    }
    const bool valid = off32[p] != kExpertBadOffset;
    const float gate = Elem<T>::to_f32(gates[p]);
    const float sig = 1.0f / (1.0f + __expf(-s));
    const float act = s * sig;
    coef_up[p] = valid ? act * gate : 0.0f;
    coef_down[p] = valid ? u * gate * (sig * (1.0f + s * (1.0f - sig))) : 0.0f;
    dgates[p] = Elem<T>::from_f32(valid ? u * act : 0.0f);
    if (valid) atomicAdd(&counts[indices[p]], 1);   // integer histogram: the result does not depend on order
}

// One wave per expert and column chunk (blockIdx.y; NCH * 64 packets each): its rows of ddown and dup, summed over its
// pairs in ascending pair index.
template <typename T, int NCH>
__global__ __launch_bounds__(kBwdWaves* kWave) void expert_backward_weight_kernel(
    const T* __restrict__ dout, const T* __restrict__ x, const float* __restrict__ coef_up,
    const float* __restrict__ coef_down, const uint32_t* __restrict__ pairs, const int32_t* __restrict__ offsets,
    T* __restrict__ ddown, T* __restrict__ dup, int hidden, int64_t num_experts, int top_k) {
    constexpr int V = Elem<T>::kVec;
    constexpr int PIF = NCH >= 8 ? 1 : 2;
    const int lane = lane_id();
    const int64_t e = (int64_t)blockIdx.x * kBwdWaves + (threadIdx.x >> 6);
    if (e >= num_experts) return;
    const int packets = hidden / V;
    const int first = (int)blockIdx.y * NCH * kWave;          // first packet of this column chunk
    const u32x4_t zero4 = {0u, 0u, 0u, 0u};
    bool live[NCH];
#pragma unroll
    for (int c = 0; c < NCH; ++c) live[c] = first + c * kWave + lane < packets;
    float acc_d[NCH][V], acc_u[NCH][V];
#pragma unroll
    for (int c = 0; c < NCH; ++c)
#pragma unroll
        for (int v = 0; v < V; ++v) acc_d[c][v] = acc_u[c][v] = 0.0f;

    const int begin = offsets[e], end = offsets[e + 1];
    const int n_total = end - begin;
    // The segment lists the expert's pairs in ascending pair index (the bucketing stage orders it), kWave pairs per round.
    for (int done = 0; done < n_total; done += kWave) {
        const int n = n_total - done < kWave ? n_total - done : kWave;
        const uint32_t mine = lane < n ? pairs[begin + done + lane] : 0u;
        uint32_t tok = 0;
        float cu = 0.0f, cd = 0.0f;
        if (lane < n) {
            tok = mine / (uint32_t)top_k;
            cu = coef_up[mine];
            cd = coef_down[mine];
        }
        for (int j0 = 0; j0 < n; j0 += PIF) {
            u32x4_t xq[PIF][NCH], gq[PIF][NCH];
            float su[PIF], sd[PIF];
#pragma unroll
            for (int u = 0; u < PIF; ++u) {
                const int j = j0 + u < n ? j0 + u : n - 1;
                const bool on = j0 + u < n;
                const int64_t t = (int64_t)(uint32_t)__builtin_amdgcn_readlane((int)tok, j);
                su[u] = on ? __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, cu), j)) : 0.0f;
                sd[u] = on ? __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, cd), j)) : 0.0f;
#pragma unroll
                for (int c = 0; c < NCH; ++c) {
                    const int p = first + c * kWave + lane;
                    xq[u][c] = (on && live[c]) ? reinterpret_cast<const u32x4_t*>(x + t * hidden)[p] : zero4;
                    gq[u][c] = (on && live[c]) ? reinterpret_cast<const u32x4_t*>(dout + t * hidden)[p] : zero4;
                }
            }
#pragma unroll
            for (int u = 0; u < PIF; ++u)
#pragma unroll
                for (int c = 0; c < NCH; ++c) {
                    axpy16<T>(sd[u], xq[u][c], acc_d[c]);
                    axpy16<T>(su[u], gq[u][c], acc_u[c]);
                }
        }
    }
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int p = first + c * kWave + lane;
        if (live[c]) {
            reinterpret_cast<u32x4_t*>(ddown + e * hidden)[p] = pack16<T>(acc_d[c]);
            reinterpret_cast<u32x4_t*>(dup + e * hidden)[p] = pack16<T>(acc_u[c]);
        }
    }
}

struct ExpertBwdPlan {
    bool slices;
    int num_slices;
    size_t off_coef_up, off_coef_down, off_pairs, off_counts, off_cursor, off_offsets, off_off32, off_spart_s, off_spart_u, bytes;
};

ExpertBwdPlan plan_expert_backward(int64_t T_, int H, int64_t E, int K, int dtype) {
    ExpertBwdPlan p;
    const size_t pairs = (size_t)T_ * K;
    size_t o = 0;
    auto take = [&](size_t n) { const size_t at = o; o = round_up(o + n, 256); return at; };
    p.off_coef_up = take(pairs * 4);
    p.off_coef_down = take(pairs * 4);
    p.off_pairs = take(pairs * 4);
    p.off_counts = take(bucket_workspace_bytes(E));     // per-expert counts, then the fill's cursors, and the scan state
    p.off_cursor = p.off_counts;
    p.off_offsets = take((size_t)(E + 1) * 4);
    p.slices = expert_slices_usable(T_, H, E, K, dtype);
    p.num_slices = p.slices ? expert_slice_count(T_, H, E, K, dtype) : 0;
    p.off_off32 = p.off_spart_s = p.off_spart_u = o;
    if (p.slices) {
        p.off_off32 = take(pairs * 4);
        p.off_spart_s = take((size_t)p.num_slices * pairs * 4);
        p.off_spart_u = take((size_t)p.num_slices * pairs * 4);
    }
    p.bytes = o;
    return p;
}

template <typename T>
int launch_expert_backward(const void* dout, const void* x, const void* down, const void* up, const int64_t* indices,
                           const void* gates, int64_t T_, int H, int64_t E, int K, int dtype, void* dx, void* ddown, void* dup,
                           void* dgates, void* workspace, hipStream_t stream) {
    constexpr int V = Elem<T>::kVec;
    const ExpertBwdPlan p = plan_expert_backward(T_, H, E, K, dtype);
    char* ws = (char*)workspace;
    float* coef_up = (float*)(ws + p.off_coef_up);
    float* coef_down = (float*)(ws + p.off_coef_down);
    uint32_t* pairs_by_expert = (uint32_t*)(ws + p.off_pairs);
    void* bucket_ws = ws + p.off_counts;
    int32_t* counts = bucket_counts(bucket_ws);
    int32_t* offsets = (int32_t*)(ws + p.off_offsets);
    const int64_t pairs = T_ * K;
    const int nch = (H / V + kWave - 1) / kWave;
    const dim3 block(kBwdWaves * kWave);
    const dim3 token_grid((unsigned)((T_ + kBwdWaves - 1) / kBwdWaves));
    const dim3 expert_grid((unsigned)((E + kBwdWaves - 1) / kBwdWaves), (unsigned)((nch + 7) / 8));   // y: column chunks of long rows

    if (int rc = bucket_clear(bucket_ws, E, stream)) return rc;
    if (p.slices) {
        uint32_t* off32 = (uint32_t*)(ws + p.off_off32);
        float* spart_s = (float*)(ws + p.off_spart_s);
        float* spart_u = (float*)(ws + p.off_spart_u);
        if (int rc = expert_slice_prepare(indices, off32, pairs, H, E, dtype, stream)) return rc;
        if (int rc = expert_slice_scores(x, down, off32, spart_s, T_, H, E, K, dtype, stream)) return rc;
        if (int rc = expert_slice_scores(dout, up, off32, spart_u, T_, H, E, K, dtype, stream)) return rc;
        hipLaunchKernelGGL((expert_backward_gate_kernel<T>), dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, stream,
                           (const float*)spart_s, (const float*)spart_u, (const T*)gates, (const uint32_t*)off32, indices,
                           (T*)dgates, coef_up, coef_down, counts, pairs, p.num_slices);
        FMOE_CHECK_LAUNCH("fmoe_expert_backward(coefficients)");
        if (int rc = expert_slice_states(coef_down, down, off32, dx, T_, H, E, K, dtype, stream)) return rc;
    } else {
#define FMOE_LAUNCH_TOKEN(N)                                                                                          \
        hipLaunchKernelGGL((expert_backward_token_kernel<T, N>), token_grid, block, 0, stream, (const T*)dout, (const T*)x, \
                           (const T*)down, (const T*)up, indices, (const T*)gates, (T*)dx, (T*)dgates, coef_up, coef_down,  \
                           counts, T_, H, E, K)
        if (nch <= 1) FMOE_LAUNCH_TOKEN(1);
        else if (nch <= 2) FMOE_LAUNCH_TOKEN(2);
        else if (nch <= 4) FMOE_LAUNCH_TOKEN(4);
        else FMOE_LAUNCH_TOKEN(8);
#undef FMOE_LAUNCH_TOKEN
        FMOE_CHECK_LAUNCH("fmoe_expert_backward(tokens)");
    }

    // the per-token kernels above counted the pairs of every expert: offsets, segments, each in ascending pair index
    if (int rc = bucket_scan_fill(indices, bucket_ws, pairs, E, K, offsets, (int32_t*)pairs_by_expert, nullptr, 1u, nullptr, 1u,
                                  nullptr, 0, 1, stream))
        return rc;

#define FMOE_LAUNCH_WEIGHT(N)                                                                                            \
    hipLaunchKernelGGL((expert_backward_weight_kernel<T, N>), expert_grid, block, 0, stream, (const T*)dout, (const T*)x, \
                       (const float*)coef_up, (const float*)coef_down, (const uint32_t*)pairs_by_expert,                  \
                       (const int32_t*)offsets, (T*)ddown, (T*)dup, H, E, K)
    if (nch <= 1) FMOE_LAUNCH_WEIGHT(1);
    else if (nch <= 2) FMOE_LAUNCH_WEIGHT(2);
    else if (nch <= 4) FMOE_LAUNCH_WEIGHT(4);
    else FMOE_LAUNCH_WEIGHT(8);
#undef FMOE_LAUNCH_WEIGHT
    FMOE_CHECK_LAUNCH("fmoe_expert_backward(weights)");
    return FMOE_OK;
}

}  // namespace

__global__ void zero_fill_kernel(u32x4_t* __restrict__ p, size_t packets) {
    const u32x4_t zero4 = {0u, 0u, 0u, 0u};
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < packets; i += (size_t)gridDim.x * blockDim.x) p[i] = zero4;
}

// Used by the MLP backward (fmoe_mlp_backward.hip).
int launch_swiglu_backward(const void* dc, const void* a, const void* b, void* da, void* db, void* h, int64_t rows, int cols,
                           int64_t da_stride, int64_t db_stride, int dtype, hipStream_t stream) {
    const int vec = (int)(16 / dtype_size(dtype));
    if (rows == 0) return FMOE_OK;
    const int col_blocks = (cols / vec + 255) / 256;
    FMOE_REQUIRE(rows * col_blocks < (1ll << 31), FMOE_ERR_UNSUPPORTED, "fmoe_swiglu_backward: %lld rows of %d columns exceed the grid",
                 (long long)rows, cols);
    const dim3 grid((unsigned)(rows * col_blocks)), block(256);
    switch (dtype) {
        case FMOE_F32:
            hipLaunchKernelGGL((swiglu_backward_kernel<float>), grid, block, 0, stream, (const float*)dc, (const float*)a,
                               (const float*)b, (float*)da, (float*)db, (float*)h, col_blocks, cols, da_stride, db_stride);
            break;
        case FMOE_BF16:
            hipLaunchKernelGGL((swiglu_backward_kernel<bf16_t>), grid, block, 0, stream, (const bf16_t*)dc, (const bf16_t*)a,
                               (const bf16_t*)b, (bf16_t*)da, (bf16_t*)db, (bf16_t*)h, col_blocks, cols, da_stride, db_stride);
            break;
        default:
            hipLaunchKernelGGL((swiglu_backward_kernel<f16_t>), grid, block, 0, stream, (const f16_t*)dc, (const f16_t*)a,
                               (const f16_t*)b, (f16_t*)da, (f16_t*)db, (f16_t*)h, col_blocks, cols, da_stride, db_stride);
    }
    FMOE_CHECK_LAUNCH("fmoe_swiglu_backward");
    return FMOE_OK;
}

}  // namespace fmoe

extern "C" int fmoe_router_topk_backward(const void* dscores, const int64_t* indices, int64_t num_tokens, int num_keys,
                                         int top_k, int dtype, void* drouter_logits, void* stream) {
    using namespace fmoe;
    clear_error();
    FMOE_REQUIRE(dtype_ok(dtype), FMOE_ERR_BAD_DTYPE, "fmoe_router_topk_backward: unknown dtype %d", dtype);
    FMOE_REQUIRE(num_tokens >= 0 && num_keys > 0 && top_k >= 0, FMOE_ERR_BAD_SHAPE,
                 "fmoe_router_topk_backward: bad shape T=%lld nk=%d K=%d", (long long)num_tokens, num_keys, top_k);
    FMOE_REQUIRE(num_keys <= 65535, FMOE_ERR_UNSUPPORTED, "fmoe_router_topk_backward: num_keys=%d > 65535", num_keys);
    if (num_tokens == 0) return FMOE_OK;
    FMOE_REQUIRE(drouter_logits && (top_k == 0 || (dscores && indices)), FMOE_ERR_NULL_POINTER,
                 "fmoe_router_topk_backward: null tensor pointer");
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case FMOE_F32: return launch_router_backward<float>(dscores, indices, drouter_logits, num_tokens, num_keys, top_k, s);
        case FMOE_BF16: return launch_router_backward<bf16_t>(dscores, indices, drouter_logits, num_tokens, num_keys, top_k, s);
        default: return launch_router_backward<f16_t>(dscores, indices, drouter_logits, num_tokens, num_keys, top_k, s);
    }
}

extern "C" int fmoe_route_backward(const void* dgates, const int64_t* indices, const float* logits_fp32, const void* dlogits_extra,
                                   int64_t num_tokens, int num_keys, int top_k, int dtype, int norm_topk_prob,
                                   float* dlogits_fp32, void* stream) {
    using namespace fmoe;
    clear_error();
    FMOE_REQUIRE(dtype_ok(dtype), FMOE_ERR_BAD_DTYPE, "fmoe_route_backward: unknown dtype %d", dtype);
    FMOE_REQUIRE(num_tokens >= 0 && num_keys > 0 && top_k >= 0, FMOE_ERR_BAD_SHAPE,
                 "fmoe_route_backward: bad shape T=%lld nk=%d K=%d", (long long)num_tokens, num_keys, top_k);
    FMOE_REQUIRE(num_keys <= 32767, FMOE_ERR_UNSUPPORTED, "fmoe_route_backward: num_keys=%d > 32767", num_keys);
    if (num_tokens == 0) return FMOE_OK;
    FMOE_REQUIRE(logits_fp32 && dlogits_fp32 && (top_k == 0 || (dgates && indices)), FMOE_ERR_NULL_POINTER,
                 "fmoe_route_backward: null tensor pointer");
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case FMOE_F32: return launch_route_backward<float>(dgates, indices, logits_fp32, dlogits_extra, dlogits_fp32, num_tokens, num_keys, top_k, norm_topk_prob, s);
        case FMOE_BF16: return launch_route_backward<bf16_t>(dgates, indices, logits_fp32, dlogits_extra, dlogits_fp32, num_tokens, num_keys, top_k, norm_topk_prob, s);
        default: return launch_route_backward<f16_t>(dgates, indices, logits_fp32, dlogits_extra, dlogits_fp32, num_tokens, num_keys, top_k, norm_topk_prob, s);
    }
}

extern "C" int fmoe_swiglu_backward(const void* dc, const void* a, const void* b, int64_t rows, int cols, int dtype, void* da,
                                    void* db, void* stream) {
    using namespace fmoe;
    clear_error();
    FMOE_REQUIRE(dtype_ok(dtype), FMOE_ERR_BAD_DTYPE, "fmoe_swiglu_backward: unknown dtype %d", dtype);
    FMOE_REQUIRE(rows >= 0 && cols > 0, FMOE_ERR_BAD_SHAPE, "fmoe_swiglu_backward: bad shape rows=%lld cols=%d", (long long)rows, cols);
    if (rows == 0) return FMOE_OK;
    FMOE_REQUIRE(dc && a && b && da && db, FMOE_ERR_NULL_POINTER, "fmoe_swiglu_backward: null tensor pointer");
    const int vec = (int)(16 / dtype_size(dtype));
    FMOE_REQUIRE(cols % vec == 0 && aligned16(dc) && aligned16(a) && aligned16(b) && aligned16(da) && aligned16(db), FMOE_ERR_ALIGNMENT,
                 "fmoe_swiglu_backward: cols=%d must be a multiple of %d and tensors 16-byte aligned", cols, vec);
    return launch_swiglu_backward(dc, a, b, da, db, nullptr, rows, cols, cols, cols, dtype, (hipStream_t)stream);
}

extern "C" size_t fmoe_expert_backward_workspace_bytes(int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype) {
    if (num_tokens <= 0 || hidden <= 0 || num_experts <= 0 || top_k <= 0 || !fmoe::dtype_ok(dtype)) return 0;
    return fmoe::plan_expert_backward(num_tokens, hidden, num_experts, top_k, dtype).bytes;
}

extern "C" int fmoe_expert_backward(const void* dout, const void* x, const void* down, const void* up, const int64_t* indices,
                                    const void* gates, int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype,
                                    void* dx, void* ddown, void* dup, void* dgates, void* workspace, size_t workspace_bytes,
                                    void* stream) {
    using namespace fmoe;
    clear_error();
    FMOE_REQUIRE(dtype_ok(dtype), FMOE_ERR_BAD_DTYPE, "fmoe_expert_backward: unknown dtype %d", dtype);
    FMOE_REQUIRE(num_tokens >= 0 && hidden > 0 && num_experts > 0 && top_k >= 0, FMOE_ERR_BAD_SHAPE,
                 "fmoe_expert_backward: bad shape T=%lld H=%d E=%lld K=%d", (long long)num_tokens, hidden, (long long)num_experts, top_k);
    const int vec = (int)(16 / dtype_size(dtype));
    FMOE_REQUIRE(hidden % vec == 0, FMOE_ERR_ALIGNMENT, "fmoe_expert_backward: hidden=%d must be a multiple of %d (16-byte rows)", hidden, vec);
    // rows too long for the per-token row kernel take the column-slice kernels, which need 32-bit row offsets
    FMOE_REQUIRE(hidden <= 8 * kWave * vec || num_tokens == 0 || top_k == 0 || expert_slices_usable(num_tokens, hidden, num_experts, top_k, dtype),
                 FMOE_ERR_UNSUPPORTED, "fmoe_expert_backward: rows of more than %d elements need tables below 4 GiB (hidden=%d, E=%lld)",
                 8 * kWave * vec, hidden, (long long)num_experts);
    FMOE_REQUIRE(num_experts < (1ll << 31) - 1 && (int64_t)num_tokens * top_k < (1ll << 31), FMOE_ERR_UNSUPPORTED,
                 "fmoe_expert_backward: E=%lld or T*K=%lld >= 2^31", (long long)num_experts, (long long)num_tokens * top_k);
    FMOE_REQUIRE(ddown && dup && down && up && (num_tokens == 0 || (dx && x && dout)), FMOE_ERR_NULL_POINTER,
                 "fmoe_expert_backward: null tensor pointer");
    FMOE_REQUIRE(aligned16(dx) && aligned16(ddown) && aligned16(dup) && aligned16(x) && aligned16(dout) && aligned16(down) && aligned16(up),
                 FMOE_ERR_ALIGNMENT, "fmoe_expert_backward: tensor pointers must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const size_t elt = dtype_size(dtype);
    if (num_tokens == 0 || top_k == 0) {   // no pairs: every gradient is zero (a fill kernel, safe under graph capture)
        const size_t table_packets = (size_t)num_experts * hidden * elt / 16, x_packets = (size_t)num_tokens * hidden * elt / 16;
        hipLaunchKernelGGL(zero_fill_kernel, dim3(1024), dim3(256), 0, s, (u32x4_t*)ddown, table_packets);
        hipLaunchKernelGGL(zero_fill_kernel, dim3(1024), dim3(256), 0, s, (u32x4_t*)dup, table_packets);
        if (x_packets) hipLaunchKernelGGL(zero_fill_kernel, dim3(1024), dim3(256), 0, s, (u32x4_t*)dx, x_packets);
        FMOE_CHECK_LAUNCH("fmoe_expert_backward(clear)");
        return FMOE_OK;
    }
    FMOE_REQUIRE(indices && gates && dgates, FMOE_ERR_NULL_POINTER, "fmoe_expert_backward: null indices/gates with top_k=%d", top_k);
    const size_t need = plan_expert_backward(num_tokens, hidden, num_experts, top_k, dtype).bytes;
    FMOE_REQUIRE(workspace && workspace_bytes >= need && aligned16(workspace), FMOE_ERR_WORKSPACE,
                 "fmoe_expert_backward: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    switch (dtype) {
        case FMOE_F32: return launch_expert_backward<float>(dout, x, down, up, indices, gates, num_tokens, hidden, num_experts, top_k, dtype, dx, ddown, dup, dgates, workspace, s);
        case FMOE_BF16: return launch_expert_backward<bf16_t>(dout, x, down, up, indices, gates, num_tokens, hidden, num_experts, top_k, dtype, dx, ddown, dup, dgates, workspace, s);
        default: return launch_expert_backward<f16_t>(dout, x, down, up, indices, gates, num_tokens, hidden, num_experts, top_k, dtype, dx, ddown, dup, dgates, workspace, s);
    }
}
