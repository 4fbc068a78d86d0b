// Product-key router for gfx950: per token, the K largest sums a[i] + b[j] over two score vectors
// of nk entries each, without materialising the nk*nk sums.
//
// Exact pruning.  Order each half by (score descending, key index ascending) and call the rank of
// an entry in that order r.  A pair of ranks (ri, rj) is dominated by the (ri+1)*(rj+1)-1 pairs whose
// ranks are component-wise <=, because fp32 addition is monotone in each operand.  So only pairs with
// (ri+1)*(rj+1) <= K can be among the K best: sum_i floor(K/i) candidates (280 for K=64, 645 for
// K=128) instead of nk*nk (16384 / 262144).  The returned scores are therefore exactly the K largest
// sums; where sums tie exactly at the cut the chosen index may differ from an exhaustive scan.
//
// One wavefront handles one token.  All selection is done with 64-bit keys
//   (order-preserving bits of the fp32 score) << 32 | ~index
// so that "larger key" means "larger score, then smaller index".  top-K of a long list is computed in
// groups of KP = max(64, next_pow2(K)) keys: each group is bitonic-sorted across the wave (RK = KP/64
// keys per lane), odd groups in ascending order so that max(best[p], group[p]) is the bitonic sequence
// holding the K best of both, which one bitonic merge re-sorts.
#include <math.h>

#include "fmoe_common.h"

namespace fmoe {
namespace {

constexpr int kRouterWaves = 4;
constexpr int kMaxTopK = 256;
constexpr int kMaxCand = 2048;   // >= sum_{i=1..256} floor(256/i) = 1546

__device__ inline uint32_t order_bits(float f) {
    const uint32_t u = __float_as_uint(f);
    return u ^ ((u >> 31) ? 0xffffffffu : 0x80000000u);
}
__device__ inline float order_value(uint32_t o) {
    return __uint_as_float(o ^ ((o >> 31) ? 0x80000000u : 0xffffffffu));
}
__device__ inline uint64_t make_key(float score, uint32_t index) {
    return ((uint64_t)order_bits(score) << 32) | (uint64_t)(~index);
}
__device__ inline float key_score(uint64_t k) { return order_value((uint32_t)(k >> 32)); }
__device__ inline uint32_t key_index(uint64_t k) { return ~(uint32_t)(k & 0xffffffffu); }

// Value of lane (lane ^ mask) for mask in {1,2,4,8,16,32}; `mask` must be a compile-time constant after inlining.
// Distances 1, 2 and 8 are single DPP moves.  Distances 4, 16 and 32 would cost 2-4 vector instructions each on the
// DPP / permlane path; the kernel is bound by vector-ALU issue, so they go through the LDS crossbar instead
// (ds_swizzle / ds_bpermute: no LDS memory is touched, no vector-ALU slot is used, other waves cover the latency).
__device__ inline uint32_t xor_lane_u32(uint32_t v, int mask, int lane) {
    const int iv = (int)v;
    switch (mask) {
        case 1: return (uint32_t)__builtin_amdgcn_update_dpp(0, iv, 0xB1, 0xF, 0xF, true);    // quad_perm [1,0,3,2]
        case 2: return (uint32_t)__builtin_amdgcn_update_dpp(0, iv, 0x4E, 0xF, 0xF, true);    // quad_perm [2,3,0,1]
        case 4: return (uint32_t)__builtin_amdgcn_ds_swizzle(iv, (4 << 10) | 0x1F);          // bit mode: lane ^ 4
        case 8: return (uint32_t)__builtin_amdgcn_update_dpp(0, iv, 0x128, 0xF, 0xF, true);   // row_ror:8
        case 16: return (uint32_t)__builtin_amdgcn_ds_swizzle(iv, (16 << 10) | 0x1F);        // bit mode: lane ^ 16
        default: return (uint32_t)__builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, iv);
    }
}
__device__ inline uint64_t xor_lane_u64(uint64_t v, int mask, int lane) {
    const uint32_t lo = xor_lane_u32((uint32_t)v, mask, lane);
    const uint32_t hi = xor_lane_u32((uint32_t)(v >> 32), mask, lane);
    return ((uint64_t)hi << 32) | lo;
}

// Position of a key in the wave-wide sequence: p = lane*RK + r.
// One compare-exchange layer of a bitonic network: partner = p ^ J, blocks of size K alternate direction.
// Which lanes keep the larger key is a function of the lane number alone, so it is a 64-bit compile-time constant per
// (layer, register), handed to the selects as a lane mask (inverse ballot): no vector instruction and no live scalar
// register per layer, where lane-number compares hoisted out of the token loop would be spilled.
template <int RK> struct LaneMasks { uint64_t m[RK]; };
template <int RK, int K, bool DESC> constexpr LaneMasks<RK> descending_block_lanes() {
    LaneMasks<RK> out{};
    for (int r = 0; r < RK; ++r)
        for (int l = 0; l < kWave; ++l) out.m[r] |= (uint64_t)((((l * RK + r) & K) == 0) == DESC) << l;
    return out;
}
template <int RK, int K, int J, bool DESC> constexpr LaneMasks<RK> keep_max_lanes() {
    LaneMasks<RK> out{};
    for (int r = 0; r < RK; ++r)
        for (int l = 0; l < kWave; ++l) {
            const int p = l * RK + r;
            const bool desc_block = (((p & K) == 0) == DESC), first = (p & J) == 0;
            out.m[r] |= (uint64_t)(first == desc_block) << l;
        }
    return out;
}

template <int RK, bool DESC, int K, int J>
__device__ inline void bitonic_layer(uint64_t (&v)[RK], int lane) {
    if constexpr (J < RK) {
        constexpr LaneMasks<RK> desc = descending_block_lanes<RK, K, DESC>();
#pragma unroll
        for (int r = 0; r < RK; ++r) {
            if ((r & J) == 0) {
                const bool desc_block = __builtin_amdgcn_inverse_ballot_w64(desc.m[r]);
                const uint64_t a = v[r], b = v[r | J];
                const uint64_t hi = a > b ? a : b, lo = a > b ? b : a;
                v[r] = desc_block ? hi : lo;
                v[r | J] = desc_block ? lo : hi;
            }
        }
    } else {
        constexpr LaneMasks<RK> keep = keep_max_lanes<RK, K, J, DESC>();
#pragma unroll
        for (int r = 0; r < RK; ++r) {
            const uint64_t other = xor_lane_u64(v[r], J / RK, lane);
            const bool keep_max = __builtin_amdgcn_inverse_ballot_w64(keep.m[r]);
            // keep my key if it is the larger one and I keep the max, or the smaller one and I keep the min
            v[r] = ((v[r] > other) == keep_max) ? v[r] : other;
        }
    }
}

// layers J, J/2, ..., 1 of the stage with block size K
template <int RK, bool DESC, int K, int J>
__device__ inline void bitonic_stage(uint64_t (&v)[RK], int lane) {
    bitonic_layer<RK, DESC, K, J>(v, lane);
    if constexpr (J > 1) bitonic_stage<RK, DESC, K, J / 2>(v, lane);
}
// stages K, 2K, ..., N
template <int RK, bool DESC, int K>
__device__ inline void bitonic_stages_from(uint64_t (&v)[RK], int lane) {
    bitonic_stage<RK, DESC, K, K / 2>(v, lane);
    if constexpr (K < RK * kWave) bitonic_stages_from<RK, DESC, 2 * K>(v, lane);
}

template <int RK, bool DESC>
__device__ inline void bitonic_sort(uint64_t (&v)[RK], int lane) {
    bitonic_stages_from<RK, DESC, 2>(v, lane);
}

// v holds a bitonic sequence of N keys; sort it descending.
template <int RK>
__device__ inline void bitonic_merge_desc(uint64_t (&v)[RK], int lane) {
    constexpr int N = RK * kWave;
    bitonic_stage<RK, true, N, N / 2>(v, lane);
}

// Key at position `pos` of the wave-wide sequence (wave-uniform `pos`).
template <int RK>
__device__ inline uint64_t key_at(const uint64_t (&v)[RK], int pos) {
    uint64_t k = v[0];
#pragma unroll
    for (int r = 1; r < RK; ++r) k = (pos % RK == r) ? v[r] : k;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)k, pos / RK);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(k >> 32), pos / RK);
    return ((uint64_t)hi << 32) | lo;
}

// Fold groups of KP keys into the running sorted-descending top-KP.  can_stop(g, kth) may end the scan before group
// g >= 1 when no key of groups g, g+1, ... can exceed `kth`, the key now at position `cut` (the last one kept).
template <int RK, typename Gen, typename Stop>
__device__ inline void topk_groups(uint64_t (&best)[RK], int lane, int num_groups, Gen gen, int cut, Stop can_stop) {
    {
        uint64_t cur[RK];
#pragma unroll
        for (int r = 0; r < RK; ++r) cur[r] = gen(0, r);
        bitonic_sort<RK, true>(cur, lane);
#pragma unroll
        for (int r = 0; r < RK; ++r) best[r] = cur[r];
    }
    for (int g = 1; g < num_groups; ++g) {
        if (can_stop(g, key_at<RK>(best, cut))) break;
        uint64_t cur[RK];
#pragma unroll
        for (int r = 0; r < RK; ++r) cur[r] = gen(g, r);
        bitonic_sort<RK, false>(cur, lane);
#pragma unroll
        for (int r = 0; r < RK; ++r) best[r] = best[r] > cur[r] ? best[r] : cur[r];
        bitonic_merge_desc<RK>(best, lane);
    }
}

// T: element type of the input and of `scores`; TG: element type of `gates`.  FROM_LOGITS: the input is the raw gate
// output [num_tokens, 2*nk] (both halves of a token side by side) and the per-half log-softmax is computed here, as
// torch does it: (v - max) - log(sum(exp(v - max))) in fp32; otherwise the input is [2, num_tokens, nk] scores.
template <typename T, typename TG, int RK, bool FROM_LOGITS>
__global__ __launch_bounds__(kRouterWaves* kWave) __attribute__((amdgpu_waves_per_eu(1, RK >= 4 ? 5 : 8))) void router_topk_kernel(
    const T* __restrict__ lp, int64_t num_tokens, int nk, int top_k, int num_cand, T* __restrict__ scores,
    int64_t* __restrict__ indices, TG* __restrict__ gates, int norm_topk_prob, uint32_t* __restrict__ row_offsets,
    uint32_t row_bytes) {
    constexpr int KP = RK * kWave;
    __shared__ uint16_t cand[kMaxCand];
    __shared__ float half_score[kRouterWaves][2][KP];
    __shared__ uint32_t half_index[kRouterWaves][2][KP];

    // candidate table: all (i, j) with (i+1)*(j+1) <= K, packed i | j << 8, listed by i then j.  Row i has
    // K/(i+1) entries; the row starts are a running sum over the row lengths (kept in half_index until the table is
    // built: one division per thread, then additions only).
    {
        uint32_t* row_len = &half_index[0][0][0];
        for (int i = threadIdx.x; i < top_k; i += blockDim.x) row_len[i] = (uint32_t)(top_k / (i + 1));
        __syncthreads();
        for (int i = threadIdx.x; i < top_k; i += blockDim.x) {
            int off = 0;
            for (int q = 0; q < i; ++q) off += (int)row_len[q];
            const int n = (int)row_len[i];
            for (int j = 0; j < n; ++j) cand[off + j] = (uint16_t)(i | (j << 8));
        }
        __syncthreads();
    }

    const int lane = lane_id();
    const int wave = (int)(threadIdx.x >> 6);
    const int64_t waves_total = (int64_t)gridDim.x * kRouterWaves;
    const int64_t rounds = (num_tokens + waves_total - 1) / waves_total;
    const int half_groups = (nk + KP - 1) / KP;
    const int cand_groups = (num_cand + KP - 1) / KP;

    for (int64_t round = 0; round < rounds; ++round) {
        const int64_t token = round * waves_total + (int64_t)blockIdx.x * kRouterWaves + wave;
        const bool active = token < num_tokens;
        if (active) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const T* row = FROM_LOGITS ? lp + (token * 2 + h) * nk : lp + ((int64_t)h * num_tokens + token) * nk;
                float shift = 0.0f, lse = 0.0f;
                if (FROM_LOGITS) {
                    float mx = -INFINITY;
                    for (int p = lane; p < nk; p += kWave) mx = fmaxf(mx, Elem<T>::to_f32(row[p]));
                    mx = wave_max(mx);
                    float se = 0.0f;
                    for (int p = lane; p < nk; p += kWave) se += expf(Elem<T>::to_f32(row[p]) - mx);
                    shift = mx;
                    lse = logf(wave_sum(se));
                }
                uint64_t best[RK];
                topk_groups<RK>(best, lane, half_groups, [&](int g, int r) -> uint64_t {
                    const int p = g * KP + lane * RK + r;
                    if (p >= nk) return 0ull;
                    const float v = Elem<T>::to_f32(row[p]);
                    return make_key(FROM_LOGITS ? (v - shift) - lse : v, (uint32_t)p);
                }, KP - 1, [](int, uint64_t) { return false; });
#pragma unroll
                for (int r = 0; r < RK; ++r) {
                    half_score[wave][h][lane * RK + r] = key_score(best[r]);
                    half_index[wave][h][lane * RK + r] = key_index(best[r]);
                }
            }
        }
        __syncthreads();
        if (active) {
            uint64_t best[RK];
            topk_groups<RK>(best, lane, cand_groups, [&](int g, int r) -> uint64_t {
                const int c = g * KP + lane * RK + r;
                if (c >= num_cand) return 0ull;
                const int ij = cand[c];
                const int i = ij & 0xff, j = ij >> 8;
                const float s = round_through<T>(half_score[wave][0][i] + half_score[wave][1][j]);
                const uint32_t flat = half_index[wave][0][i] * (uint32_t)nk + half_index[wave][1][j];
                return make_key(s, flat);
            }, top_k - 1, [&](int g, uint64_t kth) {
                // candidates are listed by ascending rank i in half 0, so every sum from group g on is at most
                // half_score[0][i of the group's first entry] + half_score[1][0]; rounding to T is monotone
                const int i_first = cand[g * KP] & 0xff;
                const float bound = round_through<T>(half_score[wave][0][i_first] + half_score[wave][1][0]);
                return bound < key_score(kth);
            });
            float e[RK];
            float total = 0.0f;
#pragma unroll
            for (int r = 0; r < RK; ++r) {
                const int p = lane * RK + r;
                e[r] = p < top_k ? expf(key_score(best[r])) : 0.0f;
                total += e[r];
            }
            if (gates != nullptr && norm_topk_prob) total = wave_sum(total);
#pragma unroll
            for (int r = 0; r < RK; ++r) {
                const int p = lane * RK + r;
                if (p < top_k) {
                    const int64_t o = token * top_k + p;
                    scores[o] = Elem<T>::from_f32(key_score(best[r]));
                    indices[o] = (int64_t)key_index(best[r]);
                    if (row_offsets != nullptr) row_offsets[o] = key_index(best[r]) * row_bytes;
                    if (gates != nullptr) gates[o] = Elem<TG>::from_f32(norm_topk_prob ? e[r] / total : e[r]);
                }
            }
        }
        __syncthreads();
    }
}

// ------------------------------------------------------------------------------------------------------------
// Selection by threshold (num_keys <= 64*RH, candidates <= 64*RC): the same result as the group scan above, for the
// sizes where a whole list fits the wave's registers (R keys per lane).
//   1. tau = K-th largest score of the list, found bit by bit from the top: the largest value with at least K scores
//      >= it (per bit one compare per register, the counts come from the ballots on the scalar unit);
//   2. the keys above tau, then keys equal to tau in list order until K are taken, go to K slots in LDS (positions from
//      ballot prefix counts);
//   3. one bitonic sort of the KP slots on the 64-bit keys.
// List order is key index order for a half (position p = r*64 + lane), so ties at the cut go to the lowest index there;
// among candidate sums tied at the cut the earlier candidate (lower rank in half 0) is taken.
// ------------------------------------------------------------------------------------------------------------
__device__ inline uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
    for (int m = 1; m < kWave; m <<= 1) {
        const uint32_t o = (uint32_t)__shfl_xor((int)v, m, kWave);
        v = v > o ? v : o;
    }
    return (uint32_t)__builtin_amdgcn_readfirstlane((int)v);
}
// RK = registers whose 64 * RK entries cover at least k: their smallest score bounds tau from below (k entries are at
// least that large), the largest score of the list bounds it from above, and tau shares the leading bits the two bounds
// share - the search starts below them (log-probabilities of one token typically share the sign, the exponent and a
// few mantissa bits: about 22 of the 32 steps remain).  A padding entry (key 0) among those registers just gives the
// bound 0.
template <int R, int RK>
__device__ inline uint32_t kth_largest_score(const uint64_t (&key)[R], int k) {
    uint32_t hi = 0u, lo_inv = 0u;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint32_t s = (uint32_t)(key[r] >> 32);
        hi = hi > s ? hi : s;
        if (r < RK) lo_inv = lo_inv > ~s ? lo_inv : ~s;        // max of the complements = complement of the min
    }
    hi = wave_max_u32(hi);
    const uint32_t lo = ~wave_max_u32(lo_inv);
    const int bits = 32 - __builtin_clz((hi ^ lo) | 1u);         // low bits in which the bounds may differ
    uint32_t tau = bits >= 32 ? 0u : (hi >> bits) << bits;
    for (int bit = bits - 1; bit >= 0; --bit) {
        const uint32_t trial = tau | (1u << bit);
        int count = 0;
#pragma unroll
        for (int r = 0; r < R; ++r)
            count += __builtin_popcountll(__builtin_amdgcn_ballot_w64((uint32_t)(key[r] >> 32) >= trial));
        tau = count >= k ? trial : tau;
    }
    return tau;
}

__device__ inline int lanes_below(uint64_t mask) {
    return (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// slots: KP wave-private LDS entries.  Unused list entries hold key 0 (below every score).
template <int R, int RK>
__device__ inline void select_topk_sorted(const uint64_t (&key)[R], int k, uint64_t* slots, uint64_t (&best)[RK], int lane) {
    constexpr int KP = RK * kWave;
    const uint32_t tau = kth_largest_score<R, RK>(key, k);
    int base = 0;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const bool above = (uint32_t)(key[r] >> 32) > tau;
        const uint64_t m = __builtin_amdgcn_ballot_w64(above);
        if (above) slots[base + lanes_below(m)] = key[r];
        base += __builtin_popcountll(m);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const bool equal = (uint32_t)(key[r] >> 32) == tau;
        const uint64_t m = __builtin_amdgcn_ballot_w64(equal);
        const int pos = base + lanes_below(m);
        if (equal && pos < k) slots[pos] = key[r];
        base += __builtin_popcountll(m);
    }
    for (int p = k + lane; p < KP; p += kWave) slots[p] = 0ull;
    __builtin_amdgcn_wave_barrier();      // LDS operations of one wave complete in order; keep the compiler from moving them
#pragma unroll
    for (int r = 0; r < RK; ++r) best[r] = slots[lane * RK + r];
    __builtin_amdgcn_wave_barrier();
    bitonic_sort<RK, true>(best, lane);
}

// The candidate pairs (rank in half 0) | (rank in half 1) << 8, listed by rank in half 0: the list depends on top_k only,
// so the host writes it and it travels as a kernel argument (at most 64 * 11 entries for top_k <= 128).
constexpr int kSelectMaxCand = 11 * kWave;
struct CandidateTable { uint16_t pair[kSelectMaxCand]; };

// OCC: waves per SIMD the register allocation must leave room for.  With more than four tokens per SIMD eight resident
// waves (at most 64 registers, a few of them spilled for the larger lists) finish sooner than seven, whose eighth token
// per SIMD would wait for a second round; with at most four tokens per SIMD the unconstrained allocation is faster.
template <typename T, typename TG, int RK, int RH, int RC, bool FROM_LOGITS, int OCC>
__global__ __launch_bounds__(kRouterWaves* kWave, OCC) void router_select_kernel(
    const T* __restrict__ lp, int64_t num_tokens, int nk, int top_k, int num_cand, T* __restrict__ scores,
    int64_t* __restrict__ indices, TG* __restrict__ gates, int norm_topk_prob, uint32_t* __restrict__ row_offsets,
    uint32_t row_bytes, const CandidateTable table) {
    constexpr int KP = RK * kWave;
    static_assert(RC * kWave <= kSelectMaxCand, "candidate table");
    __shared__ uint16_t cand[RC * kWave];
    __shared__ float half_score[kRouterWaves][2][KP];
    __shared__ uint32_t half_index[kRouterWaves][2][KP];
    __shared__ uint64_t slot[kRouterWaves][KP];

    for (int i = (int)threadIdx.x; i < RC * kWave; i += (int)blockDim.x) cand[i] = table.pair[i];
    __syncthreads();
    const int lane = lane_id();
    const int wave = (int)(threadIdx.x >> 6);
    const int64_t waves_total = (int64_t)gridDim.x * kRouterWaves;
    const int64_t rounds = (num_tokens + waves_total - 1) / waves_total;

    for (int64_t round = 0; round < rounds; ++round) {
        const int64_t token = round * waves_total + (int64_t)blockIdx.x * kRouterWaves + wave;
        if (token >= num_tokens) continue;           // nothing below synchronises across waves
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const T* row = FROM_LOGITS ? lp + (token * 2 + h) * nk : lp + ((int64_t)h * num_tokens + token) * nk;
            float v[RH];
#pragma unroll
            for (int r = 0; r < RH; ++r) {
                const int p = r * kWave + lane;
                v[r] = p < nk ? Elem<T>::to_f32(row[p]) : 0.0f;
            }
            float shift = 0.0f, lse = 0.0f;
            if (FROM_LOGITS) {
                float mx = -INFINITY;
#pragma unroll
                for (int r = 0; r < RH; ++r)
                    if (r * kWave + lane < nk) mx = fmaxf(mx, v[r]);
                mx = wave_max(mx);
                float se = 0.0f;
#pragma unroll
                for (int r = 0; r < RH; ++r)
                    if (r * kWave + lane < nk) se += expf(v[r] - mx);
                shift = mx;
                lse = logf(wave_sum(se));
            }
            uint64_t key[RH];
#pragma unroll
            for (int r = 0; r < RH; ++r) {
                const int p = r * kWave + lane;
                key[r] = p < nk ? make_key(FROM_LOGITS ? (v[r] - shift) - lse : v[r], (uint32_t)p) : 0ull;
            }
            uint64_t best[RK];
            // every rank up to KP is looked up by the candidates (entries past nk stay key 0)
            select_topk_sorted<RH, RK>(key, nk < KP ? nk : KP, slot[wave], best, lane);
#pragma unroll
            for (int r = 0; r < RK; ++r) {
                half_score[wave][h][lane * RK + r] = key_score(best[r]);
                half_index[wave][h][lane * RK + r] = key_index(best[r]);
            }
        }
        __builtin_amdgcn_wave_barrier();
        uint64_t ckey[RC];
#pragma unroll
        for (int r = 0; r < RC; ++r) {
            const int c = r * kWave + lane;
            ckey[r] = 0ull;
            if (c < num_cand) {
                const int ij = cand[c];
                const int i = ij & 0xff, j = ij >> 8;
                const float s = round_through<T>(half_score[wave][0][i] + half_score[wave][1][j]);
                const uint32_t flat = half_index[wave][0][i] * (uint32_t)nk + half_index[wave][1][j];
                ckey[r] = make_key(s, flat);
            }
        }
        uint64_t best[RK];
        select_topk_sorted<RC, RK>(ckey, top_k, slot[wave], best, lane);
        float e[RK];
        float total = 0.0f;
#pragma unroll
        for (int r = 0; r < RK; ++r) {
            const int p = lane * RK + r;
            e[r] = p < top_k ? expf(key_score(best[r])) : 0.0f;
            total += e[r];
        }
        if (gates != nullptr && norm_topk_prob) total = wave_sum(total);
#pragma unroll
        for (int r = 0; r < RK; ++r) {
            const int p = lane * RK + r;
            if (p < top_k) {
                const int64_t o = token * top_k + p;
                scores[o] = Elem<T>::from_f32(key_score(best[r]));
                indices[o] = (int64_t)key_index(best[r]);
                if (row_offsets != nullptr) row_offsets[o] = key_index(best[r]) * row_bytes;
                if (gates != nullptr) gates[o] = Elem<TG>::from_f32(norm_topk_prob ? e[r] / total : e[r]);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------------------
// top_k beyond 256 (up to 1024, with num_keys up to 8192): one workgroup per token, every ordering is a bitonic sort of
// the 64-bit keys in LDS.  Same pruning, same keys and therefore the same result as the kernels above; an order of
// magnitude slower per token, for shapes none of the reference's configurations use.
// ------------------------------------------------------------------------------------------------------------
constexpr int kBigThreads = 1024;
constexpr int kBigMaxKeys = 8192;      // 64 KiB of keys
constexpr int kBigMaxTopK = 1024;      // sum_{i<=1024} floor(1024/i) = 7689 candidates <= kBigMaxKeys

// descending bitonic sort of keys[0..m), m a power of two, by the whole workgroup
__device__ inline void block_sort_desc(uint64_t* keys, int m) {
    for (int k = 2; k <= m; k <<= 1)
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int i = (int)threadIdx.x; i < m / 2; i += (int)blockDim.x) {
                const int lo = ((i & ~(j - 1)) << 1) | (i & (j - 1)), hi = lo | j;
                const uint64_t a = keys[lo], b = keys[hi];
                if ((a < b) == ((lo & k) == 0)) {
                    keys[lo] = b;
                    keys[hi] = a;
                }
            }
            __syncthreads();
        }
}

template <typename T, typename TG, bool FROM_LOGITS>
__global__ __launch_bounds__(kBigThreads) void router_topk_big_kernel(
    const T* __restrict__ lp, int64_t num_tokens, int nk, int top_k, int num_cand, T* __restrict__ scores,
    int64_t* __restrict__ indices, TG* __restrict__ gates, int norm_topk_prob, uint32_t* __restrict__ row_offsets,
    uint32_t row_bytes) {
    __shared__ uint64_t keys[kBigMaxKeys];
    __shared__ float half_score[2][kBigMaxTopK];
    __shared__ uint32_t half_index[2][kBigMaxTopK];
    __shared__ uint32_t row_start[kBigMaxTopK + 1];    // candidates of rank i in half 0 start here; row i has top_k/(i+1)
    __shared__ float stat[2];
    const int tid = (int)threadIdx.x, lane = lane_id();
    for (int i = tid; i <= top_k; i += kBigThreads) {
        uint32_t off = 0;
        for (int q = 0; q < i; ++q) off += (uint32_t)(top_k / (q + 1));
        row_start[i] = off;
    }
    int m_half = 64, m_cand = 64;
    while (m_half < nk) m_half <<= 1;
    while (m_cand < num_cand) m_cand <<= 1;
    const int kept = top_k < nk ? top_k : nk;           // ranks of a half the candidates can name
    __syncthreads();

    for (int64_t token = blockIdx.x; token < num_tokens; token += gridDim.x) {
        for (int h = 0; h < 2; ++h) {
            const T* row = FROM_LOGITS ? lp + (token * 2 + h) * nk : lp + ((int64_t)h * num_tokens + token) * nk;
            if (FROM_LOGITS) {
                // by one wave, in the order the one-wave-per-token kernels use: identical log-probabilities
                if (tid < kWave) {
                    float mx = -INFINITY;
                    for (int p = lane; p < nk; p += kWave) mx = fmaxf(mx, Elem<T>::to_f32(row[p]));
                    mx = wave_max(mx);
                    float se = 0.0f;
                    for (int p = lane; p < nk; p += kWave) se += expf(Elem<T>::to_f32(row[p]) - mx);
                    const float lse = logf(wave_sum(se));
                    if (lane == 0) {
                        stat[0] = mx;
                        stat[1] = lse;
                    }
                }
                __syncthreads();
            }
            const float shift = FROM_LOGITS ? stat[0] : 0.0f, lse = FROM_LOGITS ? stat[1] : 0.0f;
            for (int p = tid; p < m_half; p += kBigThreads) {
                uint64_t key = 0ull;
                if (p < nk) {
                    const float v = Elem<T>::to_f32(row[p]);
                    key = make_key(FROM_LOGITS ? (v - shift) - lse : v, (uint32_t)p);
                }
                keys[p] = key;
            }
            __syncthreads();
            block_sort_desc(keys, m_half);
            for (int r = tid; r < kept; r += kBigThreads) {
                half_score[h][r] = key_score(keys[r]);
                half_index[h][r] = key_index(keys[r]);
            }
            __syncthreads();
        }
        for (int c = tid; c < m_cand; c += kBigThreads) keys[c] = 0ull;
        __syncthreads();
        for (int i = tid; i < kept; i += kBigThreads) {
            const uint32_t at = row_start[i];
            int n = (int)(row_start[i + 1] - at);
            n = n < kept ? n : kept;                                    // half 1 has only `kept` ranks
            const float si = half_score[0][i];
            const uint32_t base = half_index[0][i] * (uint32_t)nk;
            for (int j = 0; j < n; ++j)
                keys[at + j] = make_key(round_through<T>(si + half_score[1][j]), base + half_index[1][j]);
        }
        __syncthreads();
        block_sort_desc(keys, m_cand);
        if (tid < kWave) {
            float total = 0.0f;
            if (gates != nullptr && norm_topk_prob) {
                for (int p = lane; p < top_k; p += kWave) total += expf(key_score(keys[p]));
                total = wave_sum(total);
            }
            stat[0] = total;
        }
        __syncthreads();
        const float total = stat[0];
        for (int p = tid; p < top_k; p += kBigThreads) {
            const uint64_t key = keys[p];
            const int64_t o = token * top_k + p;
            scores[o] = Elem<T>::from_f32(key_score(key));
            indices[o] = (int64_t)key_index(key);
            if (row_offsets != nullptr) row_offsets[o] = key_index(key) * row_bytes;
            if (gates != nullptr) {
                const float e = expf(key_score(key));
                gates[o] = Elem<TG>::from_f32(norm_topk_prob ? e / total : e);
            }
        }
        __syncthreads();
    }
}

// ------------------------------------------------------------------------------------------------------------
// top_k up to 4096 with any num_keys (what the kernel above cannot hold in LDS): one workgroup per token.  Neither a half
// (up to 65535 keys) nor the candidate list (sum_i floor(K/i), 35 000 for K = 4096) is stored: the K-th largest 64-bit key of
// a list is found by radix selection (eight passes over the list, a 256-bin histogram in LDS per pass; the list is
// regenerated from global memory or from the sorted halves each time), the K keys at or above it are collected and
// bitonic-sorted in LDS.  Same pruning, same keys (unique: they carry the index), so the same result as the other
// kernels, ties to the lowest flat index.  A completeness path: milliseconds for thousands of tokens.
// ------------------------------------------------------------------------------------------------------------
constexpr int kRadixMaxTopK = 4096;

// K-th largest of the keys `each(f)` feeds to f (every thread its share; the same keys on every call), by the whole
// workgroup.  hist: 256 counters; pick: two words.
template <typename Each>
__device__ inline uint64_t block_kth_largest(Each each, int want, uint32_t* hist, uint64_t* pick) {
    uint64_t prefix = 0ull;
    int remaining = want;
    for (int d = 7; d >= 0; --d) {
        for (int i = (int)threadIdx.x; i < 256; i += (int)blockDim.x) hist[i] = 0u;
        __syncthreads();
        each([&](uint64_t key) {
            if (d == 7 || (key >> (8 * (d + 1))) == prefix) atomicAdd(&hist[(uint32_t)(key >> (8 * d)) & 255u], 1u);
        });
        __syncthreads();
        if (threadIdx.x == 0) {
            int above = 0, digit = 0;
            for (int bin = 255; bin >= 0; --bin) {
                const int n = (int)hist[bin];
                if (above + n >= remaining) {
                    digit = bin;
                    break;
                }
                above += n;
            }
            pick[0] = prefix << 8 | (uint64_t)digit;
            pick[1] = (uint64_t)(remaining - above);
        }
        __syncthreads();
        prefix = pick[0];
        remaining = (int)pick[1];
    }
    return prefix;
}

template <typename T, typename TG, bool FROM_LOGITS>
__global__ __launch_bounds__(kBigThreads) void router_topk_radix_kernel(
    const T* __restrict__ lp, int64_t num_tokens, int nk, int top_k, T* __restrict__ scores, int64_t* __restrict__ indices,
    TG* __restrict__ gates, int norm_topk_prob, uint32_t* __restrict__ row_offsets, uint32_t row_bytes) {
    __shared__ uint64_t keys[kRadixMaxTopK];
    __shared__ float half_score[2][kRadixMaxTopK];
    __shared__ uint32_t half_index[2][kRadixMaxTopK];
    __shared__ uint32_t hist[256];
    __shared__ uint64_t pick[2];
    __shared__ float stat[2];
    __shared__ int filled;
    const int tid = (int)threadIdx.x, lane = lane_id(), wave = tid >> 6;
    int m = 64;
    while (m < top_k) m <<= 1;
    // keys at or above `tau` into keys[0..top_k), the rest of keys[0..m) zero, sorted descending
    auto collect_and_sort = [&](auto each, uint64_t tau) {
        for (int i = tid; i < m; i += kBigThreads) keys[i] = 0ull;
        if (tid == 0) filled = 0;
        __syncthreads();
        each([&](uint64_t key) {
            if (key >= tau) {
                const int at = atomicAdd(&filled, 1);
                if (at < top_k) keys[at] = key;
            }
        });
        __syncthreads();
        block_sort_desc(keys, m);
    };
    for (int64_t token = blockIdx.x; token < num_tokens; token += gridDim.x) {
        for (int h = 0; h < 2; ++h) {
            const T* row = FROM_LOGITS ? lp + (token * 2 + h) * nk : lp + ((int64_t)h * num_tokens + token) * nk;
            if (FROM_LOGITS) {
                // by one wave, in the order the one-wave-per-token kernels use: identical log-probabilities
                if (tid < kWave) {
                    float mx = -INFINITY;
                    for (int p = lane; p < nk; p += kWave) mx = fmaxf(mx, Elem<T>::to_f32(row[p]));
                    mx = wave_max(mx);
                    float se = 0.0f;
                    for (int p = lane; p < nk; p += kWave) se += expf(Elem<T>::to_f32(row[p]) - mx);
                    const float lse = logf(wave_sum(se));
                    if (lane == 0) {
                        stat[0] = mx;
                        stat[1] = lse;
                    }
                }
                __syncthreads();
            }
            const float shift = FROM_LOGITS ? stat[0] : 0.0f, lse = FROM_LOGITS ? stat[1] : 0.0f;
            auto each_key = [&](auto f) {
                for (int p = tid; p < nk; p += kBigThreads) {
                    const float v = Elem<T>::to_f32(row[p]);
                    f(make_key(FROM_LOGITS ? (v - shift) - lse : v, (uint32_t)p));
                }
            };
            const uint64_t tau = block_kth_largest(each_key, top_k, hist, pick);
            collect_and_sort(each_key, tau);
            for (int r = tid; r < top_k; r += kBigThreads) {
                half_score[h][r] = key_score(keys[r]);
                half_index[h][r] = key_index(keys[r]);
            }
            __syncthreads();
        }
        // candidates: rank i of half 0 with ranks 0 .. top_k/(i+1)-1 of half 1; a wave per row, lanes along the row
        auto each_candidate = [&](auto f) {
            for (int i = wave; i < top_k; i += kBigThreads / kWave) {
                const int n = top_k / (i + 1);
                const float si = half_score[0][i];
                const uint32_t base = half_index[0][i] * (uint32_t)nk;
                for (int j = lane; j < n; j += kWave) f(make_key(round_through<T>(si + half_score[1][j]), base + half_index[1][j]));
            }
        };
        const uint64_t tau = block_kth_largest(each_candidate, top_k, hist, pick);
        collect_and_sort(each_candidate, tau);
        if (tid < kWave) {
            float total = 0.0f;
            if (gates != nullptr && norm_topk_prob) {
                for (int p = lane; p < top_k; p += kWave) total += expf(key_score(keys[p]));
                total = wave_sum(total);
            }
            stat[0] = total;
        }
        __syncthreads();
        const float total = stat[0];
        for (int p = tid; p < top_k; p += kBigThreads) {
            const uint64_t key = keys[p];
            const int64_t o = token * top_k + p;
            scores[o] = Elem<T>::from_f32(key_score(key));
            indices[o] = (int64_t)key_index(key);
            if (row_offsets != nullptr) row_offsets[o] = key_index(key) * row_bytes;
            if (gates != nullptr) {
                const float e = expf(key_score(key));
                gates[o] = Elem<TG>::from_f32(norm_topk_prob ? e / total : e);
            }
        }
        __syncthreads();
    }
}

int count_candidates(int top_k) {
    int n = 0;
    for (int i = 1; i <= top_k; ++i) n += top_k / i;
    return n;
}

template <typename T, typename TG, bool FROM_LOGITS>
int launch_router(const void* lp, int64_t T_, int nk, int K, void* scores, int64_t* indices, void* gates,
                  int norm, uint32_t* row_offsets, uint32_t row_bytes, hipStream_t stream) {
    const int num_cand = count_candidates(K);
    const int64_t blocks_needed = (T_ + kRouterWaves - 1) / kRouterWaves;
    const int64_t max_blocks = (int64_t)chip_info().cus * 8;   // a few resident blocks per CU; the kernel loops over tokens
    const dim3 grid((unsigned)(blocks_needed < max_blocks ? blocks_needed : max_blocks));
    const dim3 block(kRouterWaves * kWave);
    if (K > kMaxTopK) {      // the workgroup-per-token kernels; their limits are checked by the callers
        const int64_t big_blocks = T_ < (int64_t)chip_info().cus * 2 ? T_ : (int64_t)chip_info().cus * 2;
        if (K > kBigMaxTopK || nk > kBigMaxKeys) {
            const int64_t radix_blocks = T_ < (int64_t)chip_info().cus ? T_ : (int64_t)chip_info().cus;
            hipLaunchKernelGGL((router_topk_radix_kernel<T, TG, FROM_LOGITS>), dim3((unsigned)radix_blocks), dim3(kBigThreads), 0,
                               stream, (const T*)lp, T_, nk, K, (T*)scores, indices, (TG*)gates, norm, row_offsets, row_bytes);
            FMOE_CHECK_LAUNCH("fmoe_router_topk");
            return FMOE_OK;
        }
        hipLaunchKernelGGL((router_topk_big_kernel<T, TG, FROM_LOGITS>), dim3((unsigned)big_blocks), dim3(kBigThreads), 0, stream,
                           (const T*)lp, T_, nk, K, num_cand, (T*)scores, indices, (TG*)gates, norm, row_offsets, row_bytes);
        FMOE_CHECK_LAUNCH("fmoe_router_topk");
        return FMOE_OK;
    }
    // lists that fit the registers of a wave take the threshold selection
    const bool crowded = T_ > (int64_t)chip_info().cus * 4 * kRouterWaves;      // more than four tokens per SIMD
#define FMOE_LAUNCH_SELECT(RK_, RH_, RC_)                                                                                    \
    do {                                                                                                                     \
        if (crowded)                                                                                                         \
            hipLaunchKernelGGL((router_select_kernel<T, TG, RK_, RH_, RC_, FROM_LOGITS, 8>), grid, block, 0, stream,         \
                               (const T*)lp, T_, nk, K, num_cand, (T*)scores, indices, (TG*)gates, norm, row_offsets,        \
                               row_bytes, table);                                                                            \
        else                                                                                                                 \
            hipLaunchKernelGGL((router_select_kernel<T, TG, RK_, RH_, RC_, FROM_LOGITS, 1>), grid, block, 0, stream,         \
                               (const T*)lp, T_, nk, K, num_cand, (T*)scores, indices, (TG*)gates, norm, row_offsets,        \
                               row_bytes, table);                                                                            \
    } while (0)
    CandidateTable table;
    if (K <= 128 && nk <= 512) {
        int c = 0;
        for (int i = 0; i < K; ++i)
            for (int j = 0; j < K / (i + 1); ++j) table.pair[c++] = (uint16_t)(i | (j << 8));
        for (; c < kSelectMaxCand; ++c) table.pair[c] = 0;
    }
    if (K <= 64 && nk <= 512) {
        if (nk <= 128) FMOE_LAUNCH_SELECT(1, 2, 5);
        else FMOE_LAUNCH_SELECT(1, 8, 5);
        FMOE_CHECK_LAUNCH("fmoe_router_topk");
        return FMOE_OK;
    }
    if (K <= 128 && nk <= 512) {
        if (nk <= 128) FMOE_LAUNCH_SELECT(2, 2, 11);
        else FMOE_LAUNCH_SELECT(2, 8, 11);
        FMOE_CHECK_LAUNCH("fmoe_router_topk");
        return FMOE_OK;
    }
#undef FMOE_LAUNCH_SELECT
#define FMOE_LAUNCH_ROUTER(R)                                                                                      \
    hipLaunchKernelGGL((router_topk_kernel<T, TG, R, FROM_LOGITS>), grid, block, 0, stream, (const T*)lp, T_, nk, K, \
                       num_cand, (T*)scores, indices, (TG*)gates, norm, row_offsets, row_bytes)
    if (K <= 64) FMOE_LAUNCH_ROUTER(1);
    else if (K <= 128) FMOE_LAUNCH_ROUTER(2);
    else FMOE_LAUNCH_ROUTER(4);
#undef FMOE_LAUNCH_ROUTER
    FMOE_CHECK_LAUNCH("fmoe_router_topk");
    return FMOE_OK;
}

}  // namespace

bool router_topk_supported(int num_keys, int top_k) {
    return top_k <= kRadixMaxTopK;       // <= 256: a wave per token; beyond: a workgroup per token
}

int launch_router_from_logits(const float* logits, int64_t num_tokens, int num_keys, int top_k, float* scores,
                              int64_t* indices, void* gates, int gate_dtype, int norm_topk_prob, uint32_t* row_offsets,
                              uint32_t row_bytes, hipStream_t stream) {
    switch (gate_dtype) {
        case FMOE_F32: return launch_router<float, float, true>(logits, num_tokens, num_keys, top_k, scores, indices, gates, norm_topk_prob, row_offsets, row_bytes, stream);
        case FMOE_BF16: return launch_router<float, bf16_t, true>(logits, num_tokens, num_keys, top_k, scores, indices, gates, norm_topk_prob, row_offsets, row_bytes, stream);
        default: return launch_router<float, f16_t, true>(logits, num_tokens, num_keys, top_k, scores, indices, gates, norm_topk_prob, row_offsets, row_bytes, stream);
    }
}

}  // namespace fmoe

extern "C" int fmoe_router_topk(const void* log_probs, int64_t num_tokens, int num_keys, int top_k, int dtype,
                                void* scores, int64_t* indices, void* gates, int norm_topk_prob, void* stream) {
    using namespace fmoe;
    clear_error();
    FMOE_REQUIRE(dtype_ok(dtype), FMOE_ERR_BAD_DTYPE, "fmoe_router_topk: unknown dtype %d", dtype);
    FMOE_REQUIRE(num_tokens >= 0 && num_keys > 0, FMOE_ERR_BAD_SHAPE, "fmoe_router_topk: bad shape T=%lld nk=%d",
                 (long long)num_tokens, num_keys);
    FMOE_REQUIRE(top_k >= 0 && top_k <= num_keys, FMOE_ERR_TOPK_RANGE,
                 "num_experts_per_tok should be in [0, %d], but got %d", num_keys, top_k);
    FMOE_REQUIRE(num_keys <= 65535, FMOE_ERR_UNSUPPORTED, "fmoe_router_topk: num_keys=%d > 65535", num_keys);
    FMOE_REQUIRE(router_topk_supported(num_keys, top_k), FMOE_ERR_UNSUPPORTED,
                 "fmoe_router_topk: top_k=%d > %d (num_keys=%d)", top_k, kRadixMaxTopK, num_keys);
    if (num_tokens == 0 || top_k == 0) return FMOE_OK;
    FMOE_REQUIRE(log_probs && scores && indices, FMOE_ERR_NULL_POINTER, "fmoe_router_topk: null tensor pointer");
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case FMOE_F32: return launch_router<float, float, false>(log_probs, num_tokens, num_keys, top_k, scores, indices, gates, norm_topk_prob, nullptr, 0u, s);
        case FMOE_BF16: return launch_router<bf16_t, bf16_t, false>(log_probs, num_tokens, num_keys, top_k, scores, indices, gates, norm_topk_prob, nullptr, 0u, s);
        default: return launch_router<f16_t, f16_t, false>(log_probs, num_tokens, num_keys, top_k, scores, indices, gates, norm_topk_prob, nullptr, 0u, s);
    }
}
