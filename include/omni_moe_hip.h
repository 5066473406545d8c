/* C ABI of libomni_moe_hip.so: the OmniMoE layer (forward path, plus the backward of its three operators) on AMD Instinct MI355X (gfx950).
 *
 * Plain pointers and sizes only.  Every pointer named "device" is a device address
 * of a densely packed row-major array.  Every call enqueues its kernels on `stream`
 * (a hipStream_t passed as void*, NULL = the default stream) and returns without
 * waiting for the device.  The library allocates no memory: outputs and workspaces
 * come from the caller (the *_workspace_bytes calls give the sizes).  Inputs are
 * never written.  Its global state is set-up that is done once per device: a per-kernel
 * note of the devices whose shared-memory limit has been raised (atomic) and the device
 * address of the scratch array of omni_schedule_noalloc.  Calls are re-entrant as long as
 * their outputs and workspaces are distinct (omni_schedule_noalloc: see there).
 *
 * Return value: OMNI_OK (0); a negative OMNI_ERR_* for a rejected argument (nothing
 * was enqueued); OMNI_ERR_HIP_BASE + hipError_t when the HIP runtime refused a launch.
 *
 * Citations are file:line in the reference tree (HKUSTDial/omni-moe).
 */
#ifndef OMNI_MOE_HIP_H_
#define OMNI_MOE_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OMNI_ABI_VERSION 1

#if defined(__GNUC__)
#define OMNI_API __attribute__((visibility("default")))
#else
#define OMNI_API
#endif

/* storage dtype of activations / weights / scores */
#define OMNI_BF16 0
#define OMNI_F16 1
#define OMNI_F32 2

#define OMNI_OK 0
#define OMNI_ERR_NULL (-1)        /* a required pointer is NULL */
#define OMNI_ERR_SHAPE (-2)       /* a size is negative, misaligned or out of range */
#define OMNI_ERR_DTYPE (-3)       /* unknown dtype code */
#define OMNI_ERR_TOPK (-4)        /* num_experts_per_token violates the router contract */
#define OMNI_ERR_UNSUPPORTED (-5) /* valid request that no kernel here covers */
#define OMNI_ERR_WORKSPACE (-6)   /* workspace NULL or too small */
#define OMNI_ERR_SCRATCH (-7)     /* request exceeds the fixed device scratch of omni_schedule_noalloc */
#define OMNI_ERR_HIP_BASE 1000    /* + hipError_t */

/* expert algorithms */
#define OMNI_EXPERT_ALGO_AUTO 0
#define OMNI_EXPERT_ALGO_GATHER 1   /* token-resident gather, no schedule needed */
#define OMNI_EXPERT_ALGO_SEGMENT 2  /* expert-centric segments from omni_schedule */
#define OMNI_EXPERT_ALGO_SPLIT 3    /* hidden dimension cut into 8 slices, one per XCD: table slices stay in that XCD's L2 */
#define OMNI_EXPERT_ALGO_DENSE 4    /* few experts, hundreds of tokens each: two MFMA GEMMs over all experts (the reference's group regime) */

OMNI_API int32_t omni_abi_version(void);
OMNI_API const char* omni_error_string(int32_t code);

/* Optional one-time set-up of the CURRENT device: raises the dynamic-LDS limit of every kernel that needs more
 * than the 64 KiB default and resolves the device scratch of omni_schedule_noalloc.  Every entry point does its
 * share of this on first use, so calling omni_init() is only needed by callers that must not meet a
 * non-stream HIP call later -- e.g. before the first HIP-graph capture of a shape that has not run eagerly.
 * Needs a GPU; idempotent; call once per device, with that device current.  No counterpart in the reference
 * (Triton compiles and configures its kernels on first launch). */
OMNI_API int32_t omni_init(void);

/* Cartesian-product router selection.
 * Replaces triton_omni_router_func / _omni_router_forward
 * (omni_moe/ops/triton/interface.py:32-51, omni_router.py:167-232, kernel :8-95)
 * including its two torch.topk pre-steps (:186-189).
 *   logits_x, logits_y : device [num_tokens, num_expert_sqrt], dtype `dtype`
 *   scores             : device [num_tokens, k], dtype `dtype`, descending
 *   indices            : device [num_tokens, k] int32, ix*num_expert_sqrt+iy
 * Contract of utils.py:81-104: 0 <= k <= r*r, k <= 128, k even (else OMNI_ERR_TOPK).
 * Ties: the lower key index wins inside a half; the lower candidate position
 * a*k'+b (a, b = ranks in the two halves, k' = min(r,k)) wins among equal sums.
 * num_expert_sqrt <= 1024; with bf16/f16 scores and k <= 64 up to 16384 (else OMNI_ERR_UNSUPPORTED). */
OMNI_API int32_t omni_router_select(const void* logits_x, const void* logits_y, void* scores, int32_t* indices,
                           int64_t num_tokens, int32_t num_expert_sqrt, int32_t num_experts_per_token,
                           int32_t dtype, void* stream);

/* Expert-centric schedule: counting sort of the (token, expert) pairs by expert id.
 * Replaces get_scheduling_info's tail part (omni_moe/ops/triton/omni_scheduler.py:48-101).
 *   indices          : device [num_tokens, k] int32, each in [0, num_experts)
 *   offsets          : device [num_experts+1] int32; pairs of expert e occupy
 *                      [offsets[e], offsets[e+1]) of the sorted arrays
 *   sorted_pair_ids  : device [num_tokens*k] int32, pair id = token*k + slot;
 *                      inside a segment ascending (a stable sort; the reference's
 *                      torch.sort, :71, leaves that order open); pairs whose id is
 *                      outside [0, N) follow at positions >= offsets[N]
 *   sorted_token_ids : device [num_tokens*k] int32 (= sorted_pair_ids / k), may be NULL
 *   workspace        : device, omni_schedule_workspace_bytes() bytes
 * At most 2^30 - 1 pairs (else OMNI_ERR_SHAPE). */
OMNI_API size_t omni_schedule_workspace_bytes(int64_t num_tokens, int32_t num_experts_per_token, int64_t num_experts);
OMNI_API int32_t omni_schedule(const int32_t* indices, int32_t* offsets, int32_t* sorted_pair_ids,
                      int32_t* sorted_token_ids, int64_t num_tokens, int32_t num_experts_per_token,
                      int64_t num_experts, void* workspace, void* stream);

/* omni_schedule for callers that cannot allocate: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments and results as
 * omni_schedule, without the workspace: the sort's scratch is a fixed array of
 * OMNI_SCHEDULE_NOALLOC_SCRATCH_BYTES that every GPU the library runs on holds until the process ends.
 * The call allocates and frees nothing.  Requests whose omni_schedule_workspace_bytes() exceeds the
 * array return OMNI_ERR_SCRATCH (nothing enqueued); about 64 million pairs fit when num_experts <= 4096 (one counting pass: only the histograms live there), about 690 000 pairs above that (two passes keep three arrays of pairs).
 * All calls on one GPU share that GPU's array: calls that may overlap on the device (different
 * streams without an ordering between them) race; calls on one stream are safe. */
#define OMNI_SCHEDULE_NOALLOC_SCRATCH_BYTES (8u << 20)
OMNI_API int32_t omni_schedule_noalloc(const int32_t* indices, int32_t* offsets, int32_t* sorted_pair_ids,
                              int32_t* sorted_token_ids, int64_t num_tokens, int32_t num_experts_per_token,
                              int64_t num_experts, void* stream);

/* Fused atomic-expert forward  y[t] = sum_j silu(<x[t],U[id_tj]>) * g_tj * V[id_tj].
 * Replaces triton_omni_expert_func / omni_expert_forward
 * (interface.py:54-72, omni_expert.py:920-992 with kernels :8-87 and :90-168).
 *   x [T,H], up_weight [N,H], down_weight [N,H], routing_weights [T,k] : dtype `dtype`
 *   indices [T,k] int32 in [0,N) (duplicates inside a token add; not range-checked,
 *   as in the reference); y [T,H] dtype `dtype`, fully overwritten.
 * H*sizeof(elem) must be a multiple of 16.  Sums are fp32, one rounding at the end.
 *   algo      : OMNI_EXPERT_ALGO_*.  GATHER: one wave per token fetches whole rows.  SPLIT: the hidden
 *               dimension in 8 slices, slice s handled by the blocks that run on XCD s, so that
 *               each XCD's L2 holds its eighth of both tables; two launches and [8][T][k] floats
 *               of partial dot products (H*sizeof(elem)/8 must be 64..1024 bytes, a power of two; wider rows are
 *               taken in up to 64 column blocks of that form, one pair of launches per block, [8 * blocks][T][k] floats).
 *               Rows beyond 8 KiB exist for SPLIT only, and AUTO is SPLIT for them.
 *               AUTO chooses between GATHER and SPLIT from a measured grid, by the length of the row slice
 *               each lane group streams (H*sizeof(elem)/8), the bytes of both tables and the pair count
 *               T*k: GATHER below 32768 pairs, for tables of at most 3 MiB, for slices under 128 bytes
 *               and for k > 128; SPLIT for 128-byte slices up to 32 MiB of tables from 131072 pairs, for
 *               256-byte slices up to 128 MiB (from 65536 pairs, or from 16 MiB of tables), for longer
 *               slices up to 256 MiB of tables or from 262144 pairs (and 2k >= lanes per row), and for
 *               rows beyond 8 KiB.  SEGMENT is the expert-centric organisation:
 *               omni_schedule, a pass over the sorted pairs for the coefficients, a token pass
 *               for the sum; kept so that the organisations can be measured side by side.
 *               GATHER and SEGMENT agree bit for bit, SPLIT to fp32 rounding of the dot products.
 *               DENSE is for the regime of the reference's group path (omni_scheduler.py:58,103-226,
 *               omni_expert.py:171-372: T*k/N > 256): a gate matrix G[T,N], C = silu(x U^T) * G on the matrix
 *               cores (kept with 16 significant bits), y = C V on the matrix cores; bf16/f16, N % 32 == 0,
 *               N <= 2048, H % 64 == 0.  AUTO never takes it, for two differences from every other algorithm
 *               and from the reference: it multiplies each token by EVERY table row, so a non-finite value
 *               in a row that no token selected reaches all tokens (0 * Inf = NaN in the second GEMM), and
 *               with f16 storage a coefficient silu(s) * g beyond 65504 becomes Inf where the others keep
 *               it in fp32.  Where it wins (T*k/N > 256 and N <= 16 * num_experts_per_token) it wins
 *               little; ask for it by name on finite tables.
 *   workspace : omni_expert_workspace_bytes() bytes for the same arguments (0 = may be NULL) */
OMNI_API size_t omni_expert_workspace_bytes(int64_t num_tokens, int32_t hidden_size, int64_t num_experts,
                                   int32_t num_experts_per_token, int32_t dtype, int32_t algo);
OMNI_API int32_t omni_expert_fwd(const void* x, const void* up_weight, const void* down_weight,
                        const void* routing_weights, const int32_t* indices, void* y,
                        int64_t num_tokens, int32_t hidden_size, int64_t num_experts,
                        int32_t num_experts_per_token, int32_t dtype, int32_t algo,
                        void* workspace, void* stream);

/* Shared SwiGLU MLP  y = (silu(x Wg^T) * (x Wu^T)) Wd^T  [+ residual].
 * Replaces triton_omni_mlp_func (interface.py:7-29: three torch.matmul around the SwiGLU
 * kernel omni_mlp.py:102-177).  Two MFMA GEMMs: gate/up with the SwiGLU product formed in
 * the epilogue (gate and up are rounded to the storage dtype, the product is fp32, rounded
 * once, as omni_mlp.py:53-61), then the down projection.
 *   x [T,H]; gate_weight, up_weight [I,H]; down_weight [H,I]; y [T,H]  (bf16, f16 or f32)
 *   residual : NULL, or [T,H] added to the rounded down projection and rounded again
 *              (the layer's final  mlp + experts , omni_moe.py:102)
 *   workspace: omni_mlp_workspace_bytes() bytes (the [T,I] SwiGLU activations)
 * H and I must be multiples of 8 (of 4 for f32): rows are fetched 16 bytes at a time. */
OMNI_API size_t omni_mlp_workspace_bytes(int64_t num_tokens, int32_t hidden_size, int32_t intermediate_size, int32_t dtype);
OMNI_API int32_t omni_mlp_fwd(const void* x, const void* gate_weight, const void* up_weight, const void* down_weight,
                              const void* residual, void* y, int64_t num_tokens, int32_t hidden_size,
                              int32_t intermediate_size, int32_t dtype, void* workspace, void* stream);

/* The two halves of omni_mlp_fwd as separate calls.
 * omni_swiglu_linear_fwd: h[T,I] = silu(x Wg^T) * (x Wu^T)   (interface.py:23-27 + omni_mlp.py:102-177)
 * omni_linear_fwd:        y[T,out] = x[T,in] weight[out,in]^T [+ residual[T,out]]
 *                         (a bias-free nn.Linear / torch.matmul(., W.t()): interface.py:23-29,
 *                          omni_moe/modules/omni_moe.py:47-52,70-71)
 * in_features / hidden_size multiples of 8 (4 for f32); out_features / intermediate_size of any size
 * (multiples of 8 take the widest stores). */
OMNI_API int32_t omni_swiglu_linear_fwd(const void* x, const void* gate_weight, const void* up_weight, void* h,
                                        int64_t num_tokens, int32_t hidden_size, int32_t intermediate_size,
                                        int32_t dtype, void* stream);
OMNI_API int32_t omni_linear_fwd(const void* x, const void* weight, const void* residual, void* y, int64_t num_tokens,
                                 int32_t in_features, int32_t out_features, int32_t dtype, void* stream);

/* omni_swiglu_linear_fwd for callers that run other kernels beside it (another stream).  Where the product has at least 256
 * tiles of 256 x 256, omni_swiglu_linear_fwd / omni_linear_fwd / omni_mlp_fwd launch one block per CU that walks its share
 * of the tiles -- faster alone, but it holds every CU until it ends, so a concurrent kernel waits.  This entry launches one
 * block per tile instead (omni_moe_fwd with a side stream uses it for a gate/up projection of at most two rounds of tiles).
 * Same results bit for bit.  No counterpart in the reference. */
OMNI_API int32_t omni_swiglu_linear_fwd_shared(const void* x, const void* gate_weight, const void* up_weight, void* h,
                                               int64_t num_tokens, int32_t hidden_size, int32_t intermediate_size,
                                               int32_t dtype, void* stream);

/* omni_swiglu_linear_fwd that also keeps the two projections a backward pass needs (the reference materialises them:
 * interface.py:23-27 calls torch.matmul twice before the SwiGLU function saves gate and up, omni_mlp.py:359-371):
 *   gate_out, up_out [T,I]: x Wg^T and x Wu^T rounded to the storage dtype; h [T,I] their SwiGLU product.
 * bf16 / f16 only, intermediate_size % 8 == 0, hidden_size % 64 == 0, 16-byte aligned outputs; anything else
 * returns OMNI_ERR_UNSUPPORTED (use omni_linear_fwd twice and omni_swiglu_fwd). */
OMNI_API int32_t omni_swiglu_linear_save_fwd(const void* x, const void* gate_weight, const void* up_weight, void* h,
                                             void* gate_out, void* up_out, int64_t num_tokens, int32_t hidden_size,
                                             int32_t intermediate_size, int32_t dtype, void* stream);

/* Diagnostic, no counterpart in the reference: the device's matrix-core rate with nothing else going on.
 * num_blocks blocks of 4 waves each issue iters x 16 v_mfma_f32_32x32x16_bf16 (iters * 16 * 32768 flop per
 * wave) on register operands read once from `operands` (8 KiB; the bits matter: the clock the board sustains
 * under its power limit depends on how many of them toggle).  sink: num_blocks * 256 floats, overwritten.
 * The caller times the launch; the benchmark prints the result beside the published peak. */
OMNI_API int32_t omni_probe_mfma(const void* operands, float* sink, int32_t num_blocks, int32_t iters, void* stream);
/* The same for v_mfma_f32_16x16x32_bf16, the instruction of the 256 x 256 GEMM kernel: num_blocks blocks of 8 waves each
 * issue iters x 32 of them (iters * 32 * 16384 flop per wave).  sink: num_blocks * 512 floats, overwritten.  Under the
 * board's power limit this instruction sustains more than the 32x32x16 one on the same operand bits. */
OMNI_API int32_t omni_probe_mfma16(const void* operands, float* sink, int32_t num_blocks, int32_t iters, void* stream);

/* y[i] = round(y[i] + addend[i]) in place: the layer's final  mlp + experts  (omni_moe.py:102) as a
 * call of its own, for callers that run the two branches on different streams.  num_elements a
 * multiple of 8 (4 for f32); both pointers 16-byte aligned. */
OMNI_API int32_t omni_add_inplace(void* y, const void* addend, int64_t num_elements, int32_t dtype, void* stream);

/* ---- backward of the three operators (the training path) ----------------------------------- */

/* Router backward: the gradient of the selected scores scatters to the two half-logit rows,
 * dlogits_x[t, ix] += dscores[t, j], dlogits_y[t, iy] += dscores[t, j] for id = ix*r + iy.
 * Replaces _omni_router_backward (omni_moe/ops/triton/omni_router.py:235-274, kernel :98-164).
 *   dscores [T,k] dtype `dtype`; indices [T,k] int32 as returned by omni_router_select (ids outside
 *   [0, r*r) are skipped); dlogits_x, dlogits_y [T,r] dtype `dtype`, fully overwritten.
 * fp32 sums in slot order (the reference uses fp32 atomics), one rounding.  r <= 1024, k <= 128. */
OMNI_API int32_t omni_router_bwd(const void* dscores, const int32_t* indices, void* dlogits_x, void* dlogits_y,
                                 int64_t num_tokens, int32_t num_expert_sqrt, int32_t num_experts_per_token,
                                 int32_t dtype, void* stream);

/* The rest of the router stage in reverse: from d(gates) back to d(z), z = x [Wx;Wy]^T being the
 * raw projections that omni_router_fwd leaves in its workspace.  Covers what autograd does in the
 * reference for torch.exp, the router op, F.log_softmax and nn.BatchNorm1d (omni_moe.py:70-86):
 *   d(score) = d(gate) gate;  d(l) by omni_router_bwd's scatter;  d(n) = d(l) - exp(l) sum(d(l));
 *   eval: d(z) = rstd d(n);   train: d(z) = rstd (d(n) - mean_T d(n) - nhat mean_T(d(n) nhat)).
 *   dgates, gates [T,k] dtype `dtype`; indices [T,k] int32; z [T,2r] dtype `dtype` and stats [4r] f32
 *   (mean_x | rstd_x | mean_y | rstd_y) as left by omni_router_fwd at workspace offset 0 and
 *   omni_router_workspace_stats_offset(); dz [T,2r] dtype `dtype`, fully overwritten.
 * The two GEMMs around it (dW = dz^T x, dx = dz [Wx;Wy]) are the caller's. */
OMNI_API size_t omni_router_workspace_stats_offset(int64_t num_tokens, int32_t num_expert_sqrt, int32_t dtype);
OMNI_API size_t omni_router_norm_bwd_workspace_bytes(int64_t num_tokens, int32_t num_expert_sqrt);
OMNI_API int32_t omni_router_norm_bwd(const void* dgates, const void* gates, const int32_t* indices, const void* z,
                                      const float* stats, void* dz, int64_t num_tokens, int32_t num_expert_sqrt,
                                      int32_t num_experts_per_token, int32_t dtype, int32_t training, void* workspace,
                                      void* stream);

/* Fused atomic-expert backward.  For pair (t, e = indices[t,j]) with s = <x_t, U_e>, a = <dy_t, V_e>,
 * g = routing_weights[t,j]:  drouting_weights[t,j] = a silu(s);  dx_t += a g silu'(s) U_e;
 * dup_weight[e] += a g silu'(s) x_t;  ddown_weight[e] += silu(s) g dy_t.
 * Replaces omni_expert_backward (omni_expert.py:1067-1277, kernels :375-618).  s is recomputed (the
 * forward saves nothing); every output is fully overwritten (rows of experts nobody selected are
 * zero); sums are fp32 in a fixed order with one rounding, no atomics.
 *   dy, x, dx [T,H]; up_weight, down_weight, dup_weight, ddown_weight [N,H]; routing_weights,
 *   drouting_weights [T,k] : dtype `dtype`; indices [T,k] int32 (ids outside [0,N) contribute nothing)
 *   workspace : omni_expert_bwd_workspace_bytes() bytes */
OMNI_API size_t omni_expert_bwd_workspace_bytes(int64_t num_tokens, int32_t hidden_size, int64_t num_experts,
                                                int32_t num_experts_per_token, int32_t dtype);
OMNI_API int32_t omni_expert_bwd(const void* dy, const void* x, const void* up_weight, const void* down_weight,
                                 const void* routing_weights, const int32_t* indices, void* dx, void* dup_weight,
                                 void* ddown_weight, void* drouting_weights, int64_t num_tokens, int32_t hidden_size,
                                 int64_t num_experts, int32_t num_experts_per_token, int32_t dtype, void* workspace,
                                 void* stream);

/* Element-wise SwiGLU for the training path, which keeps gate and up:
 *   omni_swiglu_fwd: out = silu(gate) * up, fp32 product, one rounding
 *                    (TritonSwiGLUFunc.forward, omni_mlp.py:252-303, kernel :102-177, math :53-61)
 *   omni_swiglu_bwd: dup = dout * silu(gate);  dgate = dout * (silu(gate) (1 - sig) + sig) * up
 *                    (TritonSwiGLUFunc.backward, omni_mlp.py:306-356, kernel :180-249)
 * num_elements a multiple of 8 (4 for f32); pointers 16-byte aligned. */
OMNI_API int32_t omni_swiglu_fwd(const void* gate, const void* up, void* out, int64_t num_elements, int32_t dtype,
                                 void* stream);
OMNI_API int32_t omni_swiglu_bwd(const void* dout, const void* gate, const void* up, void* dgate, void* dup,
                                 int64_t num_elements, int32_t dtype, void* stream);


/* Two bias-free linear layers sharing their input, written side by side:
 * y[T, 2*out] = [x weight_lo^T | x weight_hi^T].  One GEMM for the router's x and y
 * projections (omni_moe.py:70-71).  out_features_each a multiple of 2. */
OMNI_API int32_t omni_linear2_fwd(const void* x, const void* weight_lo, const void* weight_hi, void* y,
                                  int64_t num_tokens, int32_t in_features, int32_t out_features_each,
                                  int32_t dtype, void* stream);

/* Router of the layer, from hidden states to gates and expert ids:
 * projection -> BatchNorm1d(affine=False) -> log_softmax -> Cartesian top-k -> exp.
 * Replaces omni_moe/modules/omni_moe.py:70-86 (two nn.Linear, two nn.BatchNorm1d, two
 * F.log_softmax, triton_omni_router_func, torch.exp).  Every stage rounds to the storage
 * dtype where the torch ops do.
 *   x [T,H]; weight_x, weight_y [r,H]                                     (bf16, f16 or f32)
 *   running_mean_*, running_var_* [r] of dtype stats_dtype; num_batches_tracked_* int64
 *     scalars (may be NULL).  training != 0: batch statistics normalise (biased variance)
 *     and the buffers are UPDATED in place with `momentum` (unbiased variance), as
 *     nn.BatchNorm1d in train mode; momentum < 0 stands for momentum=None, the cumulative
 *     average with factor 1 / num_batches_tracked (the counters are then required); one token in
 *     training is OMNI_ERR_SHAPE (nn.BatchNorm1d raises).  training == 0: the buffers
 *     normalise, nothing is written.
 *   Limits (OMNI_ERR_UNSUPPORTED, nothing enqueued): num_expert_sqrt > 1024 with fp32 scores or k > 64, and
 *     num_expert_sqrt > 16384 (up to 1024 keys per half the selection holds the row in registers; beyond that it
 *     walks the row in chunks, with 16-bit scores and at most 64 candidates per half); and training with
 *     momentum < 0 and k == 0 (no selection follows the statistics, and the cumulative average's
 *     counter is advanced by the selection kernel).
 *   gates [T,k] dtype = exp(score); indices [T,k] int32; scores [T,k] dtype or NULL
 *   workspace: omni_router_workspace_bytes() bytes */
OMNI_API size_t omni_router_workspace_bytes(int64_t num_tokens, int32_t num_expert_sqrt, int32_t dtype);
OMNI_API int32_t omni_router_fwd(const void* x, const void* weight_x, const void* weight_y,
                                 void* running_mean_x, void* running_var_x, int64_t* num_batches_tracked_x,
                                 void* running_mean_y, void* running_var_y, int64_t* num_batches_tracked_y,
                                 int32_t training, float momentum, float eps, void* gates, int32_t* indices,
                                 void* scores, int64_t num_tokens, int32_t hidden_size, int32_t num_expert_sqrt,
                                 int32_t num_experts_per_token, int32_t dtype, int32_t stats_dtype,
                                 void* workspace, void* stream);

/* The whole layer forward in one call: replaces OmniMoE.forward (omni_moe/modules/omni_moe.py:60-106),
 * i.e. omni_router_fwd + omni_expert_fwd + omni_mlp_fwd with the final add (:102).
 *   x, y [T,H]; gate_weight, up_weight [I,H]; down_weight [H,I]; router_weight_x/y [r,H];
 *   up_embed, down_embed [N,H]; BatchNorm buffers as in omni_router_fwd.
 *   stream      : every kernel is ordered on it
 *   side_stream : NULL, or a second stream on which the router + expert branch is enqueued while the
 *                 MLP branch runs on `stream`; then fork_event and join_event must be two events of
 *                 the caller (hipEvent_t, timing disabled is fine); `stream` waits for the branch before
 *                 the final add, so after the call `stream` alone orders all later work.
 *   workspace   : omni_moe_workspace_bytes() bytes; must stay untouched until the work has run. */
OMNI_API size_t omni_moe_workspace_bytes(int64_t num_tokens, int32_t hidden_size, int32_t intermediate_size,
                                         int64_t num_experts, int32_t num_expert_sqrt, int32_t num_experts_per_token,
                                         int32_t dtype);
OMNI_API int32_t omni_moe_fwd(const void* x, const void* gate_weight, const void* up_weight, const void* down_weight,
                              const void* router_weight_x, const void* router_weight_y,
                              void* running_mean_x, void* running_var_x, int64_t* num_batches_tracked_x,
                              void* running_mean_y, void* running_var_y, int64_t* num_batches_tracked_y,
                              const void* up_embed, const void* down_embed, void* y,
                              int64_t num_tokens, int32_t hidden_size, int32_t intermediate_size, int64_t num_experts,
                              int32_t num_expert_sqrt, int32_t num_experts_per_token, int32_t dtype, int32_t stats_dtype,
                              int32_t training, float momentum, float eps, void* workspace, void* stream,
                              void* side_stream, void* fork_event, void* join_event);

/* omni_moe_fwd with the expert algorithm named by the caller (OMNI_EXPERT_ALGO_*; omni_moe_fwd is this call with
 * OMNI_EXPERT_ALGO_AUTO).  AUTO decides from sizes alone, without a device-to-host read; which algorithm is faster
 * also depends on how many DISTINCT experts the router picks, which only the caller can know: AUTO's rule is fitted
 * to ids spread evenly over the tables, and a router that concentrates on few experts moves the crossover (what is
 * live then fits the caches whatever the table size), so a caller who knows the skew may name the algorithm.
 * An algorithm that does not cover the
 * shape is OMNI_ERR_UNSUPPORTED before anything is enqueued.  The workspace size depends on the algorithm.
 * No counterpart in the reference (its scheduler reads the id statistics back to the host, omni_scheduler.py:82,90). */
OMNI_API size_t omni_moe_workspace_bytes_algo(int64_t num_tokens, int32_t hidden_size, int32_t intermediate_size,
                                              int64_t num_experts, int32_t num_expert_sqrt, int32_t num_experts_per_token,
                                              int32_t dtype, int32_t expert_algo);
OMNI_API int32_t omni_moe_fwd_algo(const void* x, const void* gate_weight, const void* up_weight, const void* down_weight,
                                   const void* router_weight_x, const void* router_weight_y,
                                   void* running_mean_x, void* running_var_x, int64_t* num_batches_tracked_x,
                                   void* running_mean_y, void* running_var_y, int64_t* num_batches_tracked_y,
                                   const void* up_embed, const void* down_embed, void* y,
                                   int64_t num_tokens, int32_t hidden_size, int32_t intermediate_size, int64_t num_experts,
                                   int32_t num_expert_sqrt, int32_t num_experts_per_token, int32_t dtype, int32_t stats_dtype,
                                   int32_t training, float momentum, float eps, void* workspace, void* stream,
                                   void* side_stream, void* fork_event, void* join_event, int32_t expert_algo);

#ifdef __cplusplus
}
#endif
#endif /* OMNI_MOE_HIP_H_ */
