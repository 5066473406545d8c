// The whole OmniMoE forward (reference omni_moe/modules/omni_moe.py:60-106) as one call:
// router -> fused experts on one branch, gate/up projection -> down projection on the other,
// joined by the final add.  With a second stream the two branches are enqueued side by side
// (the expert kernel lives on cache bandwidth and no LDS, the down projection on LDS and the
// matrix cores, so they share CUs); the fork and the join are two events the caller owns.
#include "common.h"
#include "omni_moe_hip.h"

namespace omni {
static inline size_t up256(size_t v) { return (v + 255) / 256 * 256; }
static inline size_t elem_bytes(int dtype) { return dtype == OMNI_F32 ? 4 : 2; }
// defined beside the expert kernels: OMNI_OK when omni_expert_fwd takes `algo` at this shape (decided from the sizes alone)
int expert_algo_check(int algo, int64_t num_tokens, int hidden_size, int64_t num_experts, int top_k, int dtype);
// defined beside the select kernels: whether they take num_expert_sqrt keys per half with top_k and this dtype
bool select_covers(int r, int k, int dtype);
// defined beside the GEMM kernels: omni_linear_fwd with the caller's word on whether the launch has the GPU to itself
// (then a GEMM of whole 256-tile rounds may take the form that holds every CU until it ends)
int linear_fwd_impl(const void* x, const void* weight, const void* residual, void* y, int64_t num_tokens, int32_t in_features,
                    int32_t out_features, int32_t dtype, void* stream, bool exclusive);
}  // namespace omni

// workspace: router workspace | gates [T,k] | ids [T,k] | expert output [T,H] | expert workspace | SwiGLU activations [T,I]
extern "C" OMNI_API size_t omni_moe_workspace_bytes(int64_t num_tokens, int32_t hidden_size, int32_t intermediate_size,
                                                    int64_t num_experts, int32_t num_expert_sqrt, int32_t num_experts_per_token,
                                                    int32_t dtype) {
  return omni_moe_workspace_bytes_algo(num_tokens, hidden_size, intermediate_size, num_experts, num_expert_sqrt, num_experts_per_token,
                                       dtype, OMNI_EXPERT_ALGO_AUTO);
}

extern "C" OMNI_API size_t omni_moe_workspace_bytes_algo(int64_t num_tokens, int32_t hidden_size, int32_t intermediate_size,
                                                         int64_t num_experts, int32_t num_expert_sqrt, int32_t num_experts_per_token,
                                                         int32_t dtype, int32_t expert_algo) {
  using namespace omni;
  if (num_tokens < 0 || hidden_size <= 0 || intermediate_size <= 0 || num_expert_sqrt <= 0 || num_experts_per_token < 0) return 0;
  const size_t es = elem_bytes(dtype), T = (size_t)num_tokens, k = (size_t)num_experts_per_token;
  return up256(omni_router_workspace_bytes(num_tokens, num_expert_sqrt, dtype)) + up256(T * k * es) + up256(T * k * 4) +
         up256(T * (size_t)hidden_size * es) +
         up256(omni_expert_workspace_bytes(num_tokens, hidden_size, num_experts, num_experts_per_token, dtype, expert_algo)) +
         up256(omni_mlp_workspace_bytes(num_tokens, hidden_size, intermediate_size, dtype));
}

extern "C" OMNI_API int32_t omni_moe_fwd(const void* x, const void* gate_weight, const void* up_weight, const void* down_weight,
                                         const void* router_weight_x, const void* router_weight_y,
                                         void* running_mean_x, void* running_var_x, int64_t* num_batches_tracked_x,
                                         void* running_mean_y, void* running_var_y, int64_t* num_batches_tracked_y,
                                         const void* up_embed, const void* down_embed, void* y,
                                         int64_t num_tokens, int32_t hidden_size, int32_t intermediate_size, int64_t num_experts,
                                         int32_t num_expert_sqrt, int32_t num_experts_per_token, int32_t dtype, int32_t stats_dtype,
                                         int32_t training, float momentum, float eps, void* workspace, void* stream,
                                         void* side_stream, void* fork_event, void* join_event) {
  return omni_moe_fwd_algo(x, gate_weight, up_weight, down_weight, router_weight_x, router_weight_y, running_mean_x, running_var_x,
                           num_batches_tracked_x, running_mean_y, running_var_y, num_batches_tracked_y, up_embed, down_embed, y,
                           num_tokens, hidden_size, intermediate_size, num_experts, num_expert_sqrt, num_experts_per_token, dtype,
                           stats_dtype, training, momentum, eps, workspace, stream, side_stream, fork_event, join_event,
                           OMNI_EXPERT_ALGO_AUTO);
}

extern "C" OMNI_API int32_t omni_moe_fwd_algo(const void* x, const void* gate_weight, const void* up_weight, const void* down_weight,
                                              const void* router_weight_x, const void* router_weight_y,
                                              void* running_mean_x, void* running_var_x, int64_t* num_batches_tracked_x,
                                              void* running_mean_y, void* running_var_y, int64_t* num_batches_tracked_y,
                                              const void* up_embed, const void* down_embed, void* y,
                                              int64_t num_tokens, int32_t hidden_size, int32_t intermediate_size, int64_t num_experts,
                                              int32_t num_expert_sqrt, int32_t num_experts_per_token, int32_t dtype, int32_t stats_dtype,
                                              int32_t training, float momentum, float eps, void* workspace, void* stream,
                                              void* side_stream, void* fork_event, void* join_event, int32_t expert_algo) {
  using namespace omni;
  if (num_tokens < 0 || hidden_size <= 0 || intermediate_size <= 0 || num_experts <= 0 || num_expert_sqrt <= 0) return OMNI_ERR_SHAPE;
  if (dtype != OMNI_BF16 && dtype != OMNI_F16 && dtype != OMNI_F32) return OMNI_ERR_DTYPE;
  // every stage's shape rule, before the first kernel is enqueued
  {
    const int64_t esz = (int64_t)elem_bytes(dtype), r = num_expert_sqrt, k = num_experts_per_token;
    if ((hidden_size * esz) % 16 != 0 || (intermediate_size * esz) % 16 != 0) return OMNI_ERR_SHAPE;   // rows are fetched 16 bytes at a time
    if (k < 0 || k > r * r || k > 128 || k % 2 != 0) return OMNI_ERR_TOPK;
    if (!select_covers((int)r, (int)k, dtype)) return OMNI_ERR_UNSUPPORTED;
    if (r * r > num_experts) return OMNI_ERR_SHAPE;                                                   // ids reach r*r - 1
    if (int e = expert_algo_check(expert_algo, num_tokens, hidden_size, num_experts, num_experts_per_token, dtype)) return e;
  }
  if (num_tokens == 0) return OMNI_OK;
  if (training && num_tokens == 1) return OMNI_ERR_SHAPE;   // batch statistics of one sample: nn.BatchNorm1d raises
  if (!x || !y || !up_embed || !down_embed) return OMNI_ERR_NULL;
  if (!workspace) return OMNI_ERR_WORKSPACE;
  if (side_stream && (!fork_event || !join_event)) return OMNI_ERR_NULL;
  const size_t es = elem_bytes(dtype), T = (size_t)num_tokens, k = (size_t)num_experts_per_token;
  char* w = (char*)workspace;
  void* router_ws = w;  w += up256(omni_router_workspace_bytes(num_tokens, num_expert_sqrt, dtype));
  void* gates = w;      w += up256(T * k * es);
  int32_t* ids = (int32_t*)w;  w += up256(T * k * 4);
  void* experts = w;    w += up256(T * (size_t)hidden_size * es);
  void* expert_ws = w;
  w += up256(omni_expert_workspace_bytes(num_tokens, hidden_size, num_experts, num_experts_per_token, dtype, expert_algo));
  void* h = w;

  hipStream_t main_s = (hipStream_t)stream;
  hipStream_t branch = side_stream ? (hipStream_t)side_stream : main_s;
  hipError_t he;
  if (side_stream) {
    if ((he = hipEventRecord((hipEvent_t)fork_event, main_s)) != hipSuccess) return OMNI_ERR_HIP_BASE + (int)he;
    if ((he = hipStreamWaitEvent(branch, (hipEvent_t)fork_event, 0)) != hipSuccess) return OMNI_ERR_HIP_BASE + (int)he;
  }
  // From here on the side stream may hold work: whatever happens, the caller's stream is made to wait
  // for it before this call returns, so that an error leaves no work behind that the caller cannot order.
  int e = omni_router_fwd(x, router_weight_x, router_weight_y, running_mean_x, running_var_x, num_batches_tracked_x,
                          running_mean_y, running_var_y, num_batches_tracked_y, training, momentum, eps, gates, ids, nullptr,
                          num_tokens, hidden_size, num_expert_sqrt, num_experts_per_token, dtype, stats_dtype, router_ws, branch);
  const bool alone = side_stream == nullptr;            // one stream: every kernel runs by itself
  // Beside the side branch the gate/up projection keeps its one-block-per-tile grid while that is at most two rounds of 256 tiles
  // (CUs come free between the rounds); with more tiles the streaming form wins although it holds every CU (hidden 1024 x
  // intermediate 4096, two streams: 4096 tokens 125.7 against 128.0 us, 6144 tokens 188.9 against 178.5, 8192 tokens 243.5 against 228.7)
  const int64_t gate_up_tiles = ((num_tokens + 255) / 256) * (((int64_t)intermediate_size + 127) / 128);
  if (!e) e = (alone || gate_up_tiles > 512)
                  ? omni_swiglu_linear_fwd(x, gate_weight, up_weight, h, num_tokens, hidden_size, intermediate_size, dtype, main_s)
                  : omni_swiglu_linear_fwd_shared(x, gate_weight, up_weight, h, num_tokens, hidden_size, intermediate_size, dtype, main_s);
  if (!e) e = omni_expert_fwd(x, up_embed, down_embed, gates, ids, experts, num_tokens, hidden_size, num_experts,
                              num_experts_per_token, dtype, expert_algo, expert_ws, branch);
  if (!side_stream) {   // one stream: the add is the down projection's epilogue
    if (!e) e = linear_fwd_impl(h, down_weight, experts, y, num_tokens, intermediate_size, hidden_size, dtype, main_s, true);
    return e;
  }
  if (!e) e = linear_fwd_impl(h, down_weight, nullptr, y, num_tokens, intermediate_size, hidden_size, dtype, main_s, false);
  if ((he = hipEventRecord((hipEvent_t)join_event, branch)) != hipSuccess) return e ? e : OMNI_ERR_HIP_BASE + (int)he;
  if ((he = hipStreamWaitEvent(main_s, (hipEvent_t)join_event, 0)) != hipSuccess) return e ? e : OMNI_ERR_HIP_BASE + (int)he;
  if (e) return e;
  return omni_add_inplace(y, experts, (int64_t)T * hidden_size, dtype, main_s);
}
