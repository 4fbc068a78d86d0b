// The whole FlashMoE block forward in one call: router -> routed experts -> shared SwiGLU MLP (+ add).
// The stages are the same launches as the per-op entry points; what the single call adds is that intermediates never
// leave the caller's one workspace, the router writes the experts' table-row offsets directly (no int64 -> offset
// pass), and the host does one FFI call instead of three plus their allocations.
#include "fmoe_common.h"

namespace fmoe {
namespace {

struct BlockPlan {
    size_t off_router, off_logits32, off_scores, off_indices, off_gates, off_expert, off_act, off_experts_out, bytes;
};

BlockPlan plan_block(int64_t T_, int H, int I, int nk, int64_t E, int K, int dtype) {
    BlockPlan p;
    const size_t elt = dtype_size(dtype);
    size_t o = 0;
    auto take = [&](size_t n) { const size_t at = o; o = round_up(o + n, 256); return at; };
    p.off_router = take(fmoe_router_workspace_bytes(T_, H, nk));
    p.off_logits32 = take((size_t)T_ * 2 * nk * 4);
    p.off_scores = take((size_t)T_ * K * 4);
    p.off_indices = take((size_t)T_ * K * 8);
    p.off_gates = take((size_t)T_ * K * elt);
    p.off_expert = take(fmoe_expert_workspace_bytes(T_, H, E, K, dtype));
    p.off_act = take(fmoe_mlp_workspace_bytes(T_, H, I, dtype));
    p.off_experts_out = take((size_t)T_ * H * elt);
    p.bytes = o;
    return p;
}

}  // namespace
}  // namespace fmoe

extern "C" size_t fmoe_block_workspace_bytes(int64_t num_tokens, int hidden, int intermediate, int num_keys,
                                             int64_t num_experts, int top_k, int dtype) {
    if (num_tokens <= 0 || hidden <= 0 || intermediate <= 0 || num_keys <= 0 || num_experts <= 0 || top_k < 0 ||
        !fmoe::dtype_ok(dtype))
        return 0;
    return fmoe::plan_block(num_tokens, hidden, intermediate, num_keys, num_experts, top_k, dtype).bytes;
}

extern "C" int fmoe_block_forward(const void* x, const void* gate_proj_w, const void* up_proj_w, const void* down_proj_w,
                                  const void* router_gate_w, const void* down_embed, const void* up_embed,
                                  void* running_mean, void* running_var, int64_t* num_batches_tracked, int stats_dtype,
                                  int training, float momentum, float eps, int64_t num_tokens, int hidden,
                                  int intermediate, int64_t num_experts, int num_keys, int top_k, int dtype,
                                  int norm_topk_prob, void* out, void* router_logits, int64_t* indices_out,
                                  void* gates_out, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace fmoe;
    clear_error();
    FMOE_REQUIRE(dtype_ok(dtype), FMOE_ERR_BAD_DTYPE, "fmoe_block_forward: unknown dtype %d", dtype);
    FMOE_REQUIRE(num_tokens >= 0 && hidden > 0 && intermediate > 0 && num_experts > 0 && num_keys > 0, FMOE_ERR_BAD_SHAPE,
                 "fmoe_block_forward: bad shape T=%lld H=%d I=%d E=%lld nk=%d", (long long)num_tokens, hidden, intermediate,
                 (long long)num_experts, num_keys);
    FMOE_REQUIRE((int64_t)num_keys * num_keys <= num_experts, FMOE_ERR_BAD_SHAPE,
                 "fmoe_block_forward: num_keys^2 = %lld exceeds num_experts = %lld", (long long)num_keys * num_keys,
                 (long long)num_experts);
    FMOE_REQUIRE(top_k >= 0 && top_k <= num_keys, FMOE_ERR_TOPK_RANGE, "num_experts_per_tok should be in [0, %d], but got %d",
                 num_keys, top_k);
    if (num_tokens == 0) return FMOE_OK;
    FMOE_REQUIRE(x && gate_proj_w && up_proj_w && down_proj_w && router_gate_w && down_embed && up_embed && out && router_logits,
                 FMOE_ERR_NULL_POINTER, "fmoe_block_forward: null tensor pointer");
    // what the stages would refuse is refused here, before the first launch
    const int vec = (int)(16 / dtype_size(dtype));
    FMOE_REQUIRE(hidden % vec == 0 && (dtype == FMOE_F32 || intermediate % 8 == 0), FMOE_ERR_ALIGNMENT,
                 "fmoe_block_forward: hidden=%d and intermediate=%d must give 16-byte rows", hidden, intermediate);
    FMOE_REQUIRE(aligned16(x) && aligned16(gate_proj_w) && aligned16(up_proj_w) && aligned16(down_proj_w) &&
                     aligned16(router_gate_w) && aligned16(down_embed) && aligned16(up_embed) && aligned16(out),
                 FMOE_ERR_ALIGNMENT, "fmoe_block_forward: tensor pointers must be 16-byte aligned");
    FMOE_REQUIRE(num_tokens < (1ll << 31) && num_experts < (1ll << 31), FMOE_ERR_UNSUPPORTED,
                 "fmoe_block_forward: T=%lld or E=%lld >= 2^31", (long long)num_tokens, (long long)num_experts);
    const BlockPlan p = plan_block(num_tokens, hidden, intermediate, num_keys, num_experts, top_k, dtype);
    FMOE_REQUIRE(workspace && workspace_bytes >= p.bytes && aligned16(workspace), FMOE_ERR_WORKSPACE,
                 "fmoe_block_forward: workspace of %zu bytes needed, %zu given", p.bytes, workspace_bytes);
    hipStream_t s = (hipStream_t)stream;
    char* ws = (char*)workspace;
    float* logits32 = (float*)(ws + p.off_logits32);
    float* scores = (float*)(ws + p.off_scores);
    int64_t* indices = indices_out ? indices_out : (int64_t*)(ws + p.off_indices);
    void* gates = gates_out ? gates_out : (void*)(ws + p.off_gates);
    void* expert_ws = ws + p.off_expert;
    void* act = ws + p.off_act;
    void* experts = ws + p.off_experts_out;
    const size_t elt = dtype_size(dtype);

    const bool slices = expert_slices_usable(num_tokens, hidden, num_experts, top_k, dtype);
    int rc = router_forward_impl(x, router_gate_w, running_mean, running_var, num_batches_tracked, stats_dtype, training,
                                 momentum, eps, num_tokens, hidden, num_keys, top_k, dtype, norm_topk_prob, router_logits,
                                 logits32, scores, indices, gates, slices ? expert_workspace_offsets(expert_ws) : nullptr,
                                 (uint32_t)(hidden * elt), ws + p.off_router, p.off_logits32 - p.off_router, s);
    if (rc) return rc;
    const void* residual = nullptr;
    if (top_k > 0) {
        if (slices)
            rc = expert_slices_prepared(x, down_embed, up_embed, gates, num_tokens, hidden, num_experts, top_k, dtype, experts,
                                        expert_ws, s);
        else
            rc = fmoe_expert_forward(x, down_embed, up_embed, indices, gates, num_tokens, hidden, num_experts, top_k, dtype,
                                     experts, expert_ws, p.off_act - p.off_expert, stream);
        if (rc) return rc;
        residual = experts;
    }
    rc = fmoe_mlp_gate_up(x, gate_proj_w, up_proj_w, num_tokens, hidden, intermediate, dtype, act, stream);
    if (rc) return rc;
    return fmoe_mlp_down(act, down_proj_w, num_tokens, hidden, intermediate, dtype, residual, out, stream);
}
