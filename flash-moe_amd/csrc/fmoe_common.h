// Shared host/device helpers of the FlashMoE gfx950 kernels: status + error text, element-type
// traits, wave64 reductions.  Everything here targets CDNA4 only (64-lane wavefronts).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/flashmoe_hip.h"

namespace fmoe {

constexpr int kWave = 64;

// ---- error reporting -------------------------------------------------------------------------
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
void clear_error();

#define FMOE_REQUIRE(cond, status, ...)          \
    do {                                         \
        if (!(cond)) {                           \
            ::fmoe::set_error(__VA_ARGS__);      \
            return (status);                     \
        }                                        \
    } while (0)

// Launch check: hipGetLastError after a launch; returns the positive hipError_t on failure.
#define FMOE_CHECK_LAUNCH(what)                                                        \
    do {                                                                               \
        hipError_t e__ = hipGetLastError();                                            \
        if (e__ != hipSuccess) {                                                       \
            ::fmoe::set_error("%s: launch failed: %s", what, hipGetErrorString(e__));  \
            return (int)e__;                                                           \
        }                                                                              \
    } while (0)

// What the launch geometry depends on: compute units, XCDs (workgroup ids are dealt round-robin over them, each has its
// own L2) and the size of one L2, of the current device (fmoe_core.hip).
struct ChipInfo {
    int cus, xcds;
    int64_t l2_bytes;
};
const ChipInfo& chip_info();

// Top-k of the router taking raw fp32 gate outputs [T, 2*nk] (log-softmax per half is done inside); defined in
// fmoe_router.hip, used by the fused router entry point.  gates has element type `gate_dtype`.  When `row_offsets`
// is given, the byte offset id*row_bytes of each selected expert's table row is written next to its id.
int launch_router_from_logits(const float* logits, int64_t num_tokens, int num_keys, int top_k, float* scores,
                              int64_t* indices, void* gates, int gate_dtype, int norm_topk_prob, uint32_t* row_offsets,
                              uint32_t row_bytes, hipStream_t stream);
// Whether a top-k kernel exists for these extents: top_k <= 256 with any num_keys, or top_k <= 1024 with num_keys <= 8192.
bool router_topk_supported(int num_keys, int top_k);

// The fused router (fmoe_router_forward) with the optional row-offset output; defined in fmoe_router_prologue.hip.
// fixed_scratch: the workspace is the fixed scratch of the no-allocation entry point, which has no room for the normalised
// copy of x that many tokens would otherwise use.
int router_forward_impl(const void* x, const void* gate_w, void* running_mean, void* running_var,
                        int64_t* num_batches_tracked, int stats_dtype, int training, float momentum, float eps,
                        int64_t num_tokens, int hidden, int num_keys, int top_k, int dtype, int norm_topk_prob,
                        void* router_logits, float* logits_fp32, float* scores, int64_t* indices, void* gates,
                        uint32_t* row_offsets, uint32_t row_bytes, void* workspace, size_t workspace_bytes,
                        hipStream_t stream, int split_query = 0, int fixed_scratch = 0);

// Column-slice schedule of the routed experts on row offsets that are already in place at the start of `workspace`
// (the layout fmoe_expert_workspace_bytes describes); defined in fmoe_expert.hip.
bool expert_slices_usable(int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype);
uint32_t* expert_workspace_offsets(void* workspace);
int expert_slices_prepared(const void* x, const void* down, const void* up, const void* gates, int64_t num_tokens,
                           int hidden, int64_t num_experts, int top_k, int dtype, void* out, void* workspace,
                           hipStream_t stream);
// The same schedule stage by stage (for the backward pass): row byte offsets of the ids (kExpertBadOffset for an id
// outside [0,E)), per-slice partial dot products spart[slice][pair] = <x[token, slice], table[expert, slice]>, and
// out[token, :] = sum_k coef[token,k] * table[expert_k, :].  expert_slice_count is the number of slices.
constexpr uint32_t kExpertBadOffset = 0xFFF00000u;   // beyond any table the slice schedule accepts
int expert_slice_count(int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype);
int expert_slice_prepare(const int64_t* indices, uint32_t* off32, int64_t pairs, int hidden, int64_t num_experts, int dtype,
                         hipStream_t stream);
int expert_slice_scores(const void* x, const void* table, const uint32_t* off32, float* spart, int64_t num_tokens, int hidden,
                        int64_t num_experts, int top_k, int dtype, hipStream_t stream);
int expert_slice_states(const float* coef, const void* table, const uint32_t* off32, void* out, int64_t num_tokens, int hidden,
                        int64_t num_experts, int top_k, int dtype, hipStream_t stream);

// C[M,N] = A[M,K] * B[N,K]^T written in the 16-bit dtype and in fp32, on the shared MLP's tiled kernel (fmoe_mlp.hip);
// usable when the extents are whole tiles and there are enough of them.
bool gemm_nt_dual_usable(int64_t M, int N, int K);
int gemm_nt_dual(const void* A, const void* B, void* C, float* C32, int M, int N, int K, int dtype, hipStream_t stream);

// Expert-centric bucketing (fmoe_bucket.hip): pairs grouped by expert id.  The workspace holds the per-expert counts
// (bucket_counts; cleared by bucket_clear, filled by bucket_histogram or by a caller's own kernel) and the scan state.
// bucket_scan_fill turns the counts into offsets [E+1] and writes, per slot of the grouped order, the pair index, and
// optionally token * tok_scale and expert * exp_scale; `coef_clear` [num_pairs] gets a zero for every pair whose id is
// outside [0,E); with `pack_shift` the token word also carries the id, shifted left by that many bits (truncated to 32
// bits); `ordered` puts every segment in ascending pair index (and rewrites the token words without packing).
size_t bucket_workspace_bytes(int64_t num_experts);
int32_t* bucket_counts(void* workspace);
int bucket_clear(void* workspace, int64_t num_experts, hipStream_t stream);
int bucket_histogram(const int64_t* indices, void* workspace, int64_t num_pairs, int64_t num_experts, hipStream_t stream);
int bucket_scan_fill(const int64_t* indices, void* workspace, int64_t num_pairs, int64_t num_experts, int top_k,
                     int32_t* offsets, int32_t* sorted_pairs, uint32_t* tok, uint32_t tok_scale, uint32_t* exp,
                     uint32_t exp_scale, float* coef_clear, int pack_shift, int ordered, hipStream_t stream);

// The same grouping without global atomics, by two partition passes (fmoe_bucket.hip), for large numbers of pairs: own
// workspace, no clear / histogram needed, segments in no particular pair order.  bucket_partition_pays says when to take it.
bool bucket_partition_pays(int64_t num_pairs, int64_t num_experts);
size_t bucket_partition_workspace_bytes(int64_t num_pairs, int64_t num_experts);
int bucket_partition(const int64_t* indices, void* workspace, int64_t num_pairs, int64_t num_experts, int top_k,
                     int32_t* offsets, int32_t* sorted_pairs, uint32_t* tok, uint32_t tok_scale, uint32_t* exp,
                     uint32_t exp_scale, float* coef_clear, int pack_shift, hipStream_t stream);

// Plain library GEMM (rocBLAS, loaded on first use) for the operand layouts of the backward passes; row-major
// C[M,N] = A[M,K] B[K,N] (kBlasNN) or A[K,M]^T B[K,N] (kBlasTN), C = product + beta * C.  Defined in fmoe_mlp_backward.hip.
enum { kBlasNN = 0, kBlasTN = 1 };
int blas_gemm(int layout, int M, int N, int K, const void* A, int lda, const void* B, int ldb, void* C, int ldc, float beta,
              int dtype, hipStream_t stream);

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline size_t dtype_size(int dtype) { return dtype == FMOE_F32 ? 4 : 2; }
inline bool dtype_ok(int dtype) { return dtype == FMOE_F32 || dtype == FMOE_BF16 || dtype == FMOE_F16; }
inline size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// ---- element types ---------------------------------------------------------------------------
using bf16_t = __bf16;
using f16_t = _Float16;

typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int kVec = 4;   // elements per 16-byte load
    __device__ static float to_f32(float v) { return v; }
    __device__ static float from_f32(float v) { return v; }
};
template <> struct Elem<bf16_t> {
    static constexpr int kVec = 8;
    __device__ static float to_f32(bf16_t v) { return (float)v; }
    __device__ static bf16_t from_f32(float v) { return (bf16_t)v; }
};
template <> struct Elem<f16_t> {
    static constexpr int kVec = 8;
    __device__ static float to_f32(f16_t v) { return (float)v; }
    __device__ static f16_t from_f32(float v) { return (f16_t)v; }
};

// Round an fp32 value to T and back (what "computed in the input dtype" means for one add).
template <typename T> __device__ inline float round_through(float v) { return Elem<T>::to_f32(Elem<T>::from_f32(v)); }

// ---- wave64 helpers --------------------------------------------------------------------------
__device__ inline int lane_id() { return (int)(threadIdx.x & (kWave - 1)); }

// Cross-lane moves through the DPP path (no LDS traffic).  CTRL: 0xB1 / 0x4E = swap lanes 1 / 2 apart inside
// a quad, 0x141 = mirror inside 8 lanes, 0x140 = mirror inside a row of 16 lanes, 0x128 = rotate a row by 8
// (= swap lanes 8 apart), 0x142 / 0x143 = broadcast lane 15 / 31 to the following row(s).
template <int CTRL, int ROW_MASK = 0xF, bool BOUND = true>
__device__ inline float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, BOUND));
}
// Sum over each aligned group of 8 lanes, result in all 8.
__device__ inline float group8_sum(float v) {
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    v += dpp_move<0x141>(v);
    return v;
}
// Sum over the 64 lanes, result in all lanes (it comes back through an SGPR, so it is wave-uniform).
__device__ inline float wave_sum(float v) {
    v = group8_sum(v);
    v += dpp_move<0x140>(v);
    v += dpp_move<0x142, 0xA, false>(v);   // row_bcast15: lane 15 of rows 0 and 2 into rows 1 and 3
    v += dpp_move<0x143, 0xC, false>(v);   // row_bcast31: lane 31 into rows 2 and 3
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Max over the 64 lanes, result in all lanes.
__device__ inline float wave_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));
    v = fmaxf(v, dpp_move<0x4E>(v));
    v = fmaxf(v, dpp_move<0x141>(v));
    v = fmaxf(v, dpp_move<0x140>(v));
    v = fmaxf(v, __shfl_xor(v, 16, kWave));
    v = fmaxf(v, __shfl_xor(v, 32, kWave));
    return v;
}

__device__ inline float silu_f32(float v) { return v / (1.0f + __expf(-v)); }
// Same function with the hardware reciprocal (1 ulp) instead of an IEEE division: for results rounded to 16 bits.
__device__ inline float silu_fast_f32(float v) {
    return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(v * -1.44269504088896340736f));
}

}  // namespace fmoe
