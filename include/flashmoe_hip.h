/*
 * flashmoe_hip.h -- C ABI of the MI355X (gfx950) FlashMoE forward path.
 *
 * The reference (flash-algo/flash-moe) has no C ABI: its hot path is three Python entry points
 * that launch Triton kernels on the caller's current stream.  Each function below is what a
 * binding for one of those entry points calls instead; the comment on each names the reference
 * interface it replaces.  All tensors are dense row-major device buffers owned by the caller
 * (torch); the library never allocates or frees device memory, never synchronises the host, and
 * launches only on the stream it is given (a hipStream_t passed as void*; NULL = default stream).
 *
 * Return value: 0 on success, a negative fmoe_status_t for a rejected argument, or a positive
 * hipError_t if a launch failed.  fmoe_last_error() returns a thread-local description.
 */
#ifndef FLASHMOE_HIP_H
#define FLASHMOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FMOE_ABI_VERSION 1

/* element type of activations / weights / scores */
typedef enum {
    FMOE_F32 = 0,
    FMOE_BF16 = 1,
    FMOE_F16 = 2
} fmoe_dtype_t;

typedef enum {
    FMOE_OK = 0,
    FMOE_ERR_NULL_POINTER = -1,   /* a required pointer is NULL */
    FMOE_ERR_BAD_SHAPE = -2,      /* negative / zero / inconsistent extent */
    FMOE_ERR_TOPK_RANGE = -3,     /* top_k outside [0, num_keys]            (flash_router.py:261-263) */
    FMOE_ERR_BAD_DTYPE = -4,      /* dtype not one of fmoe_dtype_t */
    FMOE_ERR_UNSUPPORTED = -5,    /* extent beyond what the kernels are built for (message says which) */
    FMOE_ERR_ALIGNMENT = -6,      /* pointer not 16-byte aligned or row length not a multiple of 16 bytes */
    FMOE_ERR_WORKSPACE = -7,      /* workspace NULL or smaller than the *_workspace_bytes() figure */
    FMOE_ERR_LIBRARY = -8         /* rocBLAS (backward GEMMs only) could not be loaded or reported a failure */
} fmoe_status_t;

/* ABI version of the loaded library (== FMOE_ABI_VERSION it was built with). */
int fmoe_abi_version(void);

/* Thread-local text of the last error returned on this thread ("" if none). */
const char* fmoe_last_error(void);

/* ------------------------------------------------------------------------------------------------
 * Product-key router.
 * Replaces triton_flash_router_func / FlashRouterFunc.forward / _flash_router_forward
 * (flash_moe/ops/triton/flash_router.py:381-382, 347-368, 252-314; contract docs/flash_router.md:16-40),
 * and, when `gates` is given, the two statements after it in FlashMoE.forward
 * (flash_moe/modules/flash_moe.py:80-85: exp, optional renormalisation).
 *
 *   log_probs  [2, num_tokens, num_keys]  dtype      per-half scores (log-probabilities in the module)
 *   scores     [num_tokens, top_k]        dtype      K largest sums lp[0,t,i]+lp[1,t,j], descending;
 *                                                    16-bit dtypes: each sum rounded to dtype, as the
 *                                                    reference adds in the input dtype (flash_router.py:51-53)
 *   indices    [num_tokens, top_k]        int64      i*num_keys + j.  Equal sums at the cut: with num_keys <= 512 and
 *                                                    top_k <= 128 (the register-resident selection) the entries equal to
 *                                                    the K-th sum are taken in candidate order (rank in half 0, then
 *                                                    rank in half 1); otherwise the lower flat index wins (tl.argmax
 *                                                    rule).  The scores are the same either way.
 *   gates      [num_tokens, top_k]        dtype      optional (NULL to skip): exp(score), divided by the
 *                                                    per-token sum when norm_topk_prob != 0
 * Requires 0 <= top_k <= num_keys (same rule as the reference's assert).
 * Limits of this build (FMOE_ERR_UNSUPPORTED beyond): num_keys <= 65535; top_k <= 4096 (beyond 256 a workgroup per
 * token: in-LDS sorts up to top_k 1024 with num_keys <= 8192, radix selection otherwise - milliseconds for thousands of
 * tokens).  The reference accepts any top_k <= num_keys (flash_router.py:261-263); its own benchmarks stop at 4096.
 */
int fmoe_router_topk(const void* log_probs, int64_t num_tokens, int num_keys, int top_k, int dtype,
                     void* scores, int64_t* indices, void* gates, int norm_topk_prob, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Router of the block, from the block's input to gates: everything FlashMoE.forward does before it calls the
 * expert op (flash_moe/modules/flash_moe.py:62-85): BatchNorm1d(affine=False) -> router_gate (Linear, no bias) ->
 * per-half log-softmax -> triton_flash_router_func -> exp -> optional renormalisation.
 *
 *   x              [T, H]        dtype   block input
 *   gate_w         [2*nk, H]     dtype   router_gate.weight (rows [0,nk) score half 0, rows [nk,2nk) half 1)
 *   running_mean / running_var [H], num_batches_tracked [1] int64: router_norm's buffers, element type stats_dtype.
 *                  training != 0: batch statistics normalise x and the buffers are updated as nn.BatchNorm1d does
 *                  (momentum, unbiased variance; the counter is incremented); they may be NULL to skip the update.
 *                  training == 0: the running statistics normalise x.
 *   router_logits  [T, 2*nk]     dtype   out: the gate output the module returns (as a [2,T,nk] view)
 *   logits_fp32    [T, 2*nk]     fp32    out: the same before rounding; the routing is computed from these
 *   scores         [T, top_k]    fp32    out: log-probability sums, descending
 *   indices        [T, top_k]    int64   out: expert ids i*nk + j
 *   gates          [T, top_k]    dtype   out: routing weights (NULL to skip)
 * The normalised activations are rounded to dtype as a stand-alone batch-norm emits them; the product with gate_w,
 * the log-softmax and the pair sums are fp32.  With T == 1 in training mode the call is rejected like
 * nn.BatchNorm1d rejects it.  workspace: fmoe_router_workspace_bytes() bytes, 256-byte aligned (batch statistics, mean and
 * 1/std, and - when the logits give every compute unit a 256 x 256 tile - T*H*2 bytes for the normalised activations, from
 * which the gate product then runs on the shared MLP's tiled kernel; the logits are the same bit for bit either way).
 * Limits of this build: num_keys <= 32767, top_k as in fmoe_router_topk, num_tokens < 2^31 (FMOE_ERR_UNSUPPORTED beyond); hidden a whole
 * number of 16-byte packets (FMOE_ERR_ALIGNMENT) and, for the 16-bit dtypes, hidden <= 8192.
 */
size_t fmoe_router_workspace_bytes(int64_t num_tokens, int hidden, int num_keys);

int fmoe_router_forward(const void* x, const void* gate_w, void* running_mean, void* running_var,
                        int64_t* num_batches_tracked, int stats_dtype, int training, float momentum, float eps,
                        int64_t num_tokens, int hidden, int num_keys, int top_k, int dtype, int norm_topk_prob,
                        void* router_logits, float* logits_fp32, float* scores, int64_t* indices, void* gates,
                        void* workspace, size_t workspace_bytes, void* stream);

/* The same routing stage with a split query: half h of the gate (sub_keys rows [h*nk, (h+1)*nk), each of hidden/2
 * columns) scores only columns [h*hidden/2, (h+1)*hidden/2) of the normalised activations, i.e. fmoe_router_forward with a
 * block-diagonal router_gate.weight, at half the multiply-adds.  This is the product-key form in which each sub-key
 * table sees its own half of the query (two 128 x 512 tables against a 1024-wide query in the router benchmark
 * configuration); FlashMoE.forward itself scores the full query against both halves (flash_moe/modules/flash_moe.py:65-66),
 * so the module never takes this entry point.
 *   sub_keys [2*nk, H/2] dtype; everything else as in fmoe_router_forward.  Requires nk % 64 == 0 and H/2 a whole number
 *   of 16-byte packets. */
int fmoe_router_forward_split(const void* x, const void* sub_keys, void* running_mean, void* running_var,
                              int64_t* num_batches_tracked, int stats_dtype, int training, float momentum, float eps,
                              int64_t num_tokens, int hidden, int num_keys, int top_k, int dtype, int norm_topk_prob,
                              void* router_logits, float* logits_fp32, float* scores, int64_t* indices, void* gates,
                              void* workspace, size_t workspace_bytes, void* stream);

/* fmoe_router_forward for callers that cannot allocate device memory (code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc): same arguments without the workspace, same kernels, same results.  It has no
 * counterpart in the reference.  The scratch the call needs (batch-norm partials, mean and 1/std: about 6 MiB) is a
 * static array in device memory, one copy per GPU for the life of the process, so hidden is limited to 2048
 * (FMOE_ERR_UNSUPPORTED beyond) and two calls that overlap on one GPU (different streams or threads) race on it.
 * The call itself allocates and frees nothing; the device the stream belongs to must be the current device.  The first call
 * on a device asks the runtime for the scratch's address and the device geometry (host-side queries, no stream work):
 * make one call outside any capture before capturing the entry point into a graph. */
int fmoe_router_forward_noalloc(const void* x, const void* gate_w, void* running_mean, void* running_var,
                                int64_t* num_batches_tracked, int stats_dtype, int training, float momentum, float eps,
                                int64_t num_tokens, int hidden, int num_keys, int top_k, int dtype, int norm_topk_prob,
                                void* router_logits, float* logits_fp32, float* scores, int64_t* indices, void* gates,
                                void* stream);

/* ------------------------------------------------------------------------------------------------
 * Routed experts.
 * Replaces triton_flash_expert_func / FlashExpertFunc.forward / _flash_expert_forward and its host-side
 * preprocessing (flash_moe/ops/triton/flash_expert.py:831-836, 748-796, 580-651, 528-577; contract
 * docs/flash_expert.md:17-58):
 *   out[t,:] = sum_k silu(<x[t,:], down[idx[t,k],:]>) * gates[t,k] * up[idx[t,k],:]
 *
 *   x [T,H], down [E,H], up [E,H], gates [T,K], out [T,H]: dtype;  indices [T,K]: int64 in [0,E).
 * Duplicate ids in a row add, as in the reference.  An id outside [0,E) contributes nothing (the
 * reference reads out of bounds).  Accumulation is fp32 and deterministic (no atomics); `out` is
 * written once, it need not be zeroed.
 * fmoe_expert_workspace_bytes() gives the scratch fmoe_expert_forward needs for these extents (0 when it takes the
 * row schedule); pass a 256-byte aligned buffer of at least that size.  fmoe_expert_workspace_bytes_algo() gives it
 * for a schedule forced through fmoe_expert_forward_algo().
 * Limits of this build: hidden a whole number of 16-byte packets (FMOE_ERR_ALIGNMENT); E < 2^31 and T*K < 2^40; and per
 * schedule (FMOE_ERR_UNSUPPORTED when a call can take none of them, or when the forced one does not apply):
 *   rows     rows of at most 8192 bytes (hidden <= 4096 for the 16-bit dtypes, 2048 for fp32)
 *   slices   each table below 4 GiB (rows are addressed with 32-bit byte offsets)
 *   buckets  rows a multiple of 128 bytes; x and each table below 4 GiB; T*K < 2^31 - 4096; T < 2^24 (its second
 *            phase sweeps the experts when the dtype is 16-bit, K <= 256 and E < 2^22; else it gathers whole rows)
 * fmoe_expert_forward picks slices when E*128 bytes fit twice the L2 of one XCD and there are at least 65536 pairs, or
 * when the rows are too long for the row schedule; else buckets when there are at least 65536 pairs and 12 pairs per
 * expert (each table row then serves enough pairs to pay for the grouping) and its limits hold; else rows.  So any
 * hidden size works as long as each table stays below 4 GiB.
 */
size_t fmoe_expert_workspace_bytes(int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype);
size_t fmoe_expert_workspace_bytes_algo(int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype, int algo);

int fmoe_expert_forward(const void* x, const void* down, const void* up, const int64_t* indices,
                        const void* gates, int64_t num_tokens, int hidden, int64_t num_experts, int top_k,
                        int dtype, void* out, void* workspace, size_t workspace_bytes, void* stream);

/* Expert-centric preprocessing on its own.
 * Replaces _preprocess_expert_centric_indices_pytorch (flash_moe/ops/triton/flash_expert.py:528-577: flatten the pairs,
 * sort by expert id, bincount + cumsum), on the GPU and without its host synchronisation:
 *   expert_offsets    [E+1]   int32   out: pairs of expert e occupy slots [offsets[e], offsets[e+1]); offsets[E] = number
 *                                     of pairs with an id in [0,E) (ids outside belong to no segment)
 *   sorted_pair_ids   [T*K]   int32   out: flattened position t*K + k of the pair in each slot; inside a segment in
 *                                     ascending order (the order of a stable sort; torch.sort in the reference is not
 *                                     stable, so its order there is unspecified); entries from offsets[E] on are not written
 *   sorted_token_ids  [T*K]   int32   out, optional (NULL to skip): token of each slot, sorted_pair_ids / K
 *   sorted_expert_ids [T*K]   int32   out, optional: expert id of each slot
 * workspace: fmoe_expert_bucket_workspace_bytes(E) bytes, 256-byte aligned.  Requires E and T*K below 2^31. */
size_t fmoe_expert_bucket_workspace_bytes(int64_t num_experts);

int fmoe_expert_bucket(const int64_t* indices, int64_t num_tokens, int top_k, int64_t num_experts, int32_t* expert_offsets,
                       int32_t* sorted_pair_ids, int32_t* sorted_token_ids, int32_t* sorted_expert_ids, void* workspace,
                       size_t workspace_bytes, void* stream);

/* Same operation with the schedule chosen by the caller instead of by problem size (fmoe_expert_forward
 * passes FMOE_EXPERT_AUTO).  All schedules compute the formula above; they differ in how the table rows
 * travel: whole rows per (token, expert) pair; 128- or 256-byte column slices of the tables, each worked through by
 * one XCD (one L2) at a time; or, for tables far larger than the L2s, pairs grouped by expert so that the scores
 * stream each down row once against column bands of x.
 * The reference has one schedule (expert-centric Triton kernels, flash_expert.py:580-651). */
typedef enum {
    FMOE_EXPERT_AUTO = 0,
    FMOE_EXPERT_ROWS = 1,     /* one wavefront per token, whole rows; no workspace needed */
    FMOE_EXPERT_SLICES = 2,   /* column slices of the tables resident in L2; needs the workspace */
    FMOE_EXPERT_BUCKETS = 3   /* pairs grouped by expert (the fmoe_expert_bucket stage), column bands of x resident in
                                 L2, each down row streamed once; needs the workspace */
} fmoe_expert_algo_t;

int fmoe_expert_forward_algo(const void* x, const void* down, const void* up, const int64_t* indices,
                             const void* gates, int64_t num_tokens, int hidden, int64_t num_experts, int top_k,
                             int dtype, void* out, void* workspace, size_t workspace_bytes, int algo, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Shared SwiGLU MLP.
 * Replaces triton_flash_mlp_func / TritonSwiGLUFunc.forward / swiglu_forward
 * (flash_moe/ops/triton/flash_mlp.py:169-181, 153-159, 105-123) and, when `residual` is given, the add
 * that follows it in FlashMoE.forward (flash_moe/modules/flash_moe.py:101):
 *   out = (silu(x gate_w^T) * (x up_w^T)) down_w^T  [+ residual]
 *
 *   x [T,H], gate_w [I,H], up_w [I,H], down_w [H,I], residual [T,H] or NULL, out [T,H]: dtype.
 * The gate/up products are kept in fp32 until after silu(.)*(.), then rounded once to dtype.
 * workspace: fmoe_mlp_workspace_bytes() bytes (the [T,I] activation), 256-byte aligned.
 */
size_t fmoe_mlp_workspace_bytes(int64_t num_tokens, int hidden, int intermediate, int dtype);

int fmoe_mlp_forward(const void* x, const void* gate_w, const void* up_w, const void* down_w,
                     int64_t num_tokens, int hidden, int intermediate, int dtype, const void* residual,
                     void* out, void* workspace, size_t workspace_bytes, void* stream);

/* The two launches of fmoe_mlp_forward, individually (same argument rules; `act` is the [T,I] activation
 * that fmoe_mlp_forward keeps in its workspace).  A caller that wants the activation, or that times
 * the two GEMMs separately, calls these instead.
 *   fmoe_mlp_gate_up: act = silu(x gate_w^T) * (x up_w^T)     -- the two matmuls and the SwiGLU kernel of
 *                     triton_flash_mlp_func (flash_moe/ops/triton/flash_mlp.py:175-179, 25-49)
 *   fmoe_mlp_down:    out = act down_w^T [+ residual]          -- its last matmul (flash_mlp.py:173-181) */
int fmoe_mlp_gate_up(const void* x, const void* gate_w, const void* up_w, int64_t num_tokens, int hidden,
                     int intermediate, int dtype, void* act, void* stream);
/* fmoe_mlp_gate_up that also keeps the two products for a backward pass, as TritonSwiGLUFunc.forward saves a and b
 * (flash_moe/ops/triton/flash_mlp.py:153-159): saved [2,T,I] dtype, plane 0 = x gate_w^T, plane 1 = x up_w^T. */
int fmoe_mlp_gate_up_save(const void* x, const void* gate_w, const void* up_w, int64_t num_tokens, int hidden,
                          int intermediate, int dtype, void* act, void* saved, void* stream);

int fmoe_mlp_down(const void* act, const void* down_w, int64_t num_tokens, int hidden, int intermediate, int dtype,
                  const void* residual, void* out, void* stream);

/* ------------------------------------------------------------------------------------------------
 * The whole block: FlashMoE.forward (flash_moe/modules/flash_moe.py:55-105) in one call, on the flattened tokens.
 *   out = mlp(x) + experts(x, route(x)),   router_logits = router_gate(router_norm(x))
 * Same stages and numerics as fmoe_router_forward -> fmoe_expert_forward -> fmoe_mlp_forward(residual = experts);
 * intermediates live in `workspace` (fmoe_block_workspace_bytes(), 256-byte aligned).
 *
 *   x [T,H]; gate_proj_w, up_proj_w [I,H]; down_proj_w [H,I]; router_gate_w [2*nk,H]; down_embed, up_embed [E,H]: dtype
 *   running_mean / running_var / num_batches_tracked, stats_dtype, training, momentum, eps: as in fmoe_router_forward
 *   out [T,H] dtype; router_logits [T,2*nk] dtype
 *   indices_out [T,K] int64 and gates_out [T,K] dtype: optional (NULL keeps them in the workspace)
 * Requires nk*nk <= E and 0 <= top_k <= nk.  The limits of the three stages apply (top_k <= 4096, nk <= 32767, the expert
 * schedules' limits above; hidden and intermediate multiples of 8 for the 16-bit dtypes), and T, E < 2^31.
 */
size_t fmoe_block_workspace_bytes(int64_t num_tokens, int hidden, int intermediate, int num_keys, int64_t num_experts,
                                  int top_k, int dtype);

int fmoe_block_forward(const void* x, const void* gate_proj_w, const void* up_proj_w, const void* down_proj_w,
                       const void* router_gate_w, const void* down_embed, const void* up_embed, void* running_mean,
                       void* running_var, int64_t* num_batches_tracked, int stats_dtype, int training, float momentum,
                       float eps, int64_t num_tokens, int hidden, int intermediate, int64_t num_experts, int num_keys,
                       int top_k, int dtype, int norm_topk_prob, void* out, void* router_logits, int64_t* indices_out,
                       void* gates_out, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------------
 * The two other gather ops of the reference that share the routed-expert kernels (forward only there too).
 *
 * PEER, triton_peer_func / peer_forward (flash_moe/ops/triton/peer.py:246-255, 151-219; eager form tests/test_peer.py:9-24):
 *   out[t] = sum_k gelu(<x[t], down[idx[t,k]]>) * w[t,k] * up[idx[t,k]]     (erf GELU)
 * i.e. fmoe_expert_forward with GELU in place of SiLU; note the reference's argument order (weights before indices).
 *
 * PKM, triton_pkm_func / pkm_forward (flash_moe/ops/triton/pkm.py:195-200, 123-174; eager form tests/test_pkm.py:9-20):
 *   out[t] = sum_k w[t,k] * values[idx[t,k]]
 * PEER takes a workspace of fmoe_expert_workspace_bytes(num_tokens, hidden, num_experts, top_k, dtype) bytes.  PKM has no
 * score phase, so it never groups pairs by expert: it takes fmoe_pkm_workspace_bytes(...) bytes (the column-slice
 * workspace when the slices are chosen, else nothing).
 */
size_t fmoe_pkm_workspace_bytes(int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype);

int fmoe_peer_forward(const void* x, const void* down, const void* up, const void* routing_weights, const int64_t* indices,
                      int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype, void* out, void* workspace,
                      size_t workspace_bytes, void* stream);

int fmoe_pkm_forward(const void* values, const void* routing_weights, const int64_t* indices, int64_t num_tokens, int hidden,
                     int64_t num_experts, int top_k, int dtype, void* out, void* workspace, size_t workspace_bytes,
                     void* stream);

/* ================================================================================================
 * Backward passes.  Deterministic: no global atomics, every gradient element is written once.
 * ================================================================================================ */

/* FlashRouterFunc.backward / _flash_router_backward / _bwd_kernel (flash_moe/ops/triton/flash_router.py:317-344,
 * 205-249): drouter_logits [2, T, nk] (dtype), fully written:
 *   [0,t,i] = sum of dscores[t,k] over k with indices[t,k] / nk == i;  [1,t,j] likewise with indices[t,k] % nk.
 * dscores [T, K] dtype, indices [T, K] int64 (ids outside [0, nk*nk) contribute nothing).
 * Limit of this build: num_keys <= 65535, as fmoe_router_topk. */
int fmoe_router_topk_backward(const void* dscores, const int64_t* indices, int64_t num_tokens, int num_keys, int top_k,
                              int dtype, void* drouter_logits, void* stream);

/* Backward of the routing stage between the gate logits and the gates (flash_moe/modules/flash_moe.py:69-85: per-half
 * log_softmax, flash_router_func, exp, optional renormalisation; autograd of torch ops around
 * flash_moe/ops/triton/flash_router.py:317-344 in the reference), in one launch.
 *   dgates [T, K] dtype: gradient of the gates; indices [T, K] int64 as returned by the forward (ids outside
 *   [0, nk*nk) contribute nothing); logits_fp32 [T, 2*nk]: the fp32 gate logits the forward routed from
 *   (router_logits_fp32 of fmoe_router_forward); dlogits_extra [T, 2*nk] dtype or NULL: gradient of the returned
 *   router logits, added to the result; dlogits_fp32 [T, 2*nk] fp32, fully written: what
 *   fmoe_router_prologue_backward takes.  Limit of this build: num_keys <= 32767, as fmoe_router_forward. */
int fmoe_route_backward(const void* dgates, const int64_t* indices, const float* logits_fp32, const void* dlogits_extra,
                        int64_t num_tokens, int num_keys, int top_k, int dtype, int norm_topk_prob, float* dlogits_fp32,
                        void* stream);

/* Backward of the router prologue q = BatchNorm1d(x), logits = q gate_w^T (flash_moe/modules/flash_moe.py:62-67; autograd of
 * torch ops in the reference).  The forward is fmoe_router_forward with top_k = 0: it leaves mean and 1/sqrt(var+eps), [2,H]
 * fp32, at byte offset fmoe_router_workspace_stats_offset() of its workspace; pass that as mean_rstd.
 *   dlogits_fp32 [T, 2*nk] fp32 (rounded to dtype for the two GEMMs); dx [T,H], dgate_w [2*nk,H]: dtype.
 * training != 0: batch statistics were used (the gradient flows through mean and variance); else running statistics
 * (constants).  The two GEMMs are rocBLAS calls.
 * Limits of this build: num_tokens < 2^24; hidden a whole number of 16-byte packets; any num_keys the forward accepts. */
size_t fmoe_router_workspace_stats_offset(int64_t num_tokens, int hidden, int num_keys);
size_t fmoe_router_prologue_backward_workspace_bytes(int64_t num_tokens, int hidden, int num_keys, int dtype);
int fmoe_router_prologue_backward(const float* dlogits_fp32, const void* x, const void* gate_w, const float* mean_rstd,
                                  int training, int64_t num_tokens, int hidden, int num_keys, int dtype, void* dx,
                                  void* dgate_w, void* workspace, size_t workspace_bytes, void* stream);

/* swiglu_backward / _swiglu_backward_kernel (flash_moe/ops/triton/flash_mlp.py:64-102, 126-150): for c = silu(a) * b,
 *   da = dc * (silu(a) * (1 - sigmoid(a)) + sigmoid(a)) * b,   db = dc * silu(a),   all [rows, cols] dtype. */
int fmoe_swiglu_backward(const void* dc, const void* a, const void* b, int64_t rows, int cols, int dtype, void* da,
                         void* db, void* stream);

/* Backward of triton_flash_mlp_func (flash_moe/ops/triton/flash_mlp.py:169-181: two matmuls, TritonSwiGLUFunc, one
 * matmul, differentiated by autograd in the reference): from dy [T,H] the gradients dx [T,H], dgate_w, dup_w [I,H],
 * ddown_w [H,I].  saved_products: the [2,T,I] buffer fmoe_mlp_gate_up_save() filled in the forward, or NULL to
 * recompute the gate and up products here.  The transposed-operand GEMMs are rocBLAS calls (loaded on first use;
 * FMOE_ERR_LIBRARY if unavailable).  When dup_w starts where dgate_w ends (one [2I,H] buffer) the two weight gradients
 * are formed as one product (faster; the sums may differ in the last bit from two products); separate buffers work as well. */
size_t fmoe_mlp_backward_workspace_bytes(int64_t num_tokens, int hidden, int intermediate, int dtype);

int fmoe_mlp_backward(const void* dy, const void* x, const void* gate_w, const void* up_w, const void* down_w,
                      const void* saved_products, int64_t num_tokens, int hidden, int intermediate, int dtype, void* dx, void* dgate_w, void* dup_w,
                      void* ddown_w, void* workspace, size_t workspace_bytes, void* stream);

/* FlashExpertFunc.backward / _flash_expert_backward (flash_moe/ops/triton/flash_expert.py:654-745, kernels :234-525):
 * from dout [T,H] the gradients dx [T,H], ddown, dup [E,H] (rows of experts no pair selects are zero) and
 * dgates [T,K]; indices get none.  Scores are recomputed, not saved.
 * Limits of this build: T*K < 2^31, E < 2^31 - 1, hidden a whole number of 16-byte packets; rows of more than 8192 bytes
 * (hidden > 4096 for the 16-bit dtypes, 2048 for fp32) need tables below 4 GiB. */
size_t fmoe_expert_backward_workspace_bytes(int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype);

int fmoe_expert_backward(const void* dout, const void* x, const void* down, const void* up, const int64_t* indices,
                         const void* gates, int64_t num_tokens, int hidden, int64_t num_experts, int top_k, int dtype,
                         void* dx, void* ddown, void* dup, void* dgates, void* workspace, size_t workspace_bytes,
                         void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASHMOE_HIP_H */
