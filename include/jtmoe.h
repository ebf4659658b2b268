/*
 * jtmoe.h -- C ABI of libjtmoe.so: the MoE expert-layer forward of Jaxtitan
 * (vpareek2/research, src/jaxtitan/models/components/moe.py) on AMD gfx950.
 *
 * Conventions (they follow the reference's native-kernel boundary,
 * src/jaxtitan/kernels/cuda/rmsnorm/rmsnorm_ffi.cu:24-74):
 *   - every pointer is a DEVICE pointer to a dense row-major array; the caller
 *     owns every buffer, results and workspace are pre-allocated by the caller;
 *   - a launcher validates its arguments, enqueues kernels on `stream` only and
 *     returns; it never allocates, frees, synchronises or retains a pointer;
 *   - return value 0 (JTMOE_OK) or a negative JTMOE_E* code; the message of the
 *     last failure on the calling thread is `jtmoe_last_error()`;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *   - `dtype` selects the compute dtype of activations and weights:
 *     JTMOE_BF16 (2-byte elements) or JTMOE_F32 (4-byte elements).
 *
 * Index conventions: T tokens, H hidden size, E experts, K = top_k,
 * I = expert intermediate size, A = T*K assignments; assignment a = t*K + s
 * (moe.py:583-586).
 */
#ifndef JTMOE_H_
#define JTMOE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define JTMOE_VERSION 1

enum {
  JTMOE_BF16 = 0,
  JTMOE_F32 = 1
};

enum {
  JTMOE_OK = 0,
  JTMOE_EINVAL = -1,       /* bad pointer, shape or attribute                    */
  JTMOE_EUNSUPPORTED = -2, /* valid request outside the implemented envelope     */
  JTMOE_EWORKSPACE = -3,   /* workspace too small                                */
  JTMOE_ELAUNCH = -4       /* hipGetLastError() after a launch reported an error */
};

/*
 * Score function of the router.  JTMOE_SCORE_SIGMOID is the reference's (moe.py:133) and what every
 * entry point without the _sf suffix computes.  JTMOE_SCORE_SOFTMAX has no counterpart in the
 * reference: the benchmark's second configuration names a softmax router, so it is offered as an
 * attribute of the same router: scores = softmax over the experts of the fp32 logits, everything
 * after the scores (biased top-k, renormalised weights, statistics) unchanged.  The _sf entry points
 * take it right after route_scale and are otherwise their namesakes.
 */
enum {
  JTMOE_SCORE_SIGMOID = 0,
  JTMOE_SCORE_SOFTMAX = 1
};

/* Limits of the implementation. */
#define JTMOE_MAX_EXPERTS 256
#define JTMOE_MAX_TOP_K 16

int jtmoe_version(void);

/* Message of the last error returned on this thread ("" if none). */
const char* jtmoe_last_error(void);

/*
 * Router.  Replaces SigmoidTopKRouter.__call__ (moe.py:131-147):
 *   logits = f32(round_dtype(x @ w_router)); scores = sigmoid(logits);
 *   ids = top_k(scores + expert_bias, K)  (descending; equal values -> lower index);
 *   weights = scores[ids] / (sum_k scores[ids] + 1e-20) * route_scale, cast to dtype.
 * and the two vectors of _router_stats (moe.py:802-805):
 *   expert_counts[e] = #{(t,s): ids[t,s]==e},  importance[e] = sum of their weights.
 *
 *   x [T,H] dtype; w_router [H,E] dtype; expert_bias [E] f32 or NULL (= zeros).
 *   out: expert_ids [T,K] i32; weights [T,K] dtype; scores [T,E] f32;
 *        expert_counts [E] f32; importance [E] f32; logits [T,E] f32 or NULL.
 *   workspace: jtmoe_router_workspace_bytes(E) bytes.
 */
size_t jtmoe_router_workspace_bytes(int64_t E);
int jtmoe_router(const void* x, const void* w_router, const float* expert_bias,
                 int64_t T, int64_t H, int64_t E, int64_t K, double route_scale, int dtype,
                 int32_t* expert_ids, void* weights, float* scores,
                 float* expert_counts, float* importance, float* logits,
                 void* workspace, size_t workspace_bytes, void* stream);

int jtmoe_router_sf(const void* x, const void* w_router, const float* expert_bias,
                    int64_t T, int64_t H, int64_t E, int64_t K, double route_scale, int score_func, int dtype,
                    int32_t* expert_ids, void* weights, float* scores,
                    float* expert_counts, float* importance, float* logits,
                    void* workspace, size_t workspace_bytes, void* stream);

/*
 * The same router, starting from given fp32 logits [T,E] (moe.py:133-147 only).
 * The routing decision is a pure function of the logits, identical bit for bit
 * to what jtmoe_router derives from its own logits.
 */
int jtmoe_router_from_logits(const float* logits, const float* expert_bias,
                             int64_t T, int64_t E, int64_t K, double route_scale, int dtype,
                             int32_t* expert_ids, void* weights, float* scores,
                             float* expert_counts, float* importance,
                             void* workspace, size_t workspace_bytes, void* stream);
int jtmoe_router_from_logits_sf(const float* logits, const float* expert_bias,
                                int64_t T, int64_t E, int64_t K, double route_scale, int score_func, int dtype,
                                int32_t* expert_ids, void* weights, float* scores,
                                float* expert_counts, float* importance,
                                void* workspace, size_t workspace_bytes, void* stream);

/*
 * Token dispatch.  Replaces the single-device part of local_dispatch
 * (moe.py:583-602): per-expert histogram, exclusive prefix sum, the stable
 * permutation of assignments into expert-contiguous order and its inverse, and
 * the row gather packed_x[j] = x[source_order[j] / K].
 *
 *   expert_ids [A] i32, each in [0,E) (duplicates within a token are legal);
 *   x [T,H] dtype, or NULL to skip the row gather (then packed_x is ignored).
 *   out: group_sizes [E] i32; offsets [E] i32; source_order [A] i32;
 *        inverse [A] i32; packed_x [A,H] dtype.
 *   workspace: jtmoe_dispatch_workspace_bytes(T*K, E) bytes.
 * An id outside [0,E) is not detected on the host (ids live on the device); such
 * an assignment is dropped from the permutation.
 */
size_t jtmoe_dispatch_workspace_bytes(int64_t A, int64_t E);
int jtmoe_dispatch(const int32_t* expert_ids, const void* x,
                   int64_t T, int64_t H, int64_t E, int64_t K, int dtype,
                   int32_t* group_sizes, int32_t* offsets,
                   int32_t* source_order, int32_t* inverse, void* packed_x,
                   void* workspace, size_t workspace_bytes, void* stream);

/*
 * jtmoe_dispatch without a workspace argument and without any allocation.  It has no counterpart in
 * the reference (XLA owns every buffer there and hands the handler its scratch as a result buffer,
 * rmsnorm_ffi.cu:59-68); it is for callers that cannot allocate device memory at all: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same arguments, results and
 * errors as jtmoe_dispatch; the partial histograms live in a buffer of
 * JTMOE_DISPATCH_STATIC_MAX_BYTES that is part of the library's device image (each GPU the library
 * runs on holds its own copy until the process ends).
 *   Limit: jtmoe_dispatch_workspace_bytes(T*K, E) <= JTMOE_DISPATCH_STATIC_MAX_BYTES, i.e.
 *   ceil(T*K / 1024) * E <= 262144 (1 048 576 assignments at 256 experts, 4 194 304 at 64);
 *   beyond it JTMOE_EUNSUPPORTED and nothing is launched.
 *   All calls on one GPU share that buffer: calls that may overlap on one GPU (two streams, two
 *   threads) race and must be ordered by the caller.  Nothing in it has to be cleared between
 *   calls.  The buffer's device address is looked up on the first call per GPU (not a stream
 *   operation; make that first call outside graph capture).
 */
#define JTMOE_DISPATCH_STATIC_MAX_BYTES ((size_t)1 << 20)
int jtmoe_dispatch_static(const int32_t* expert_ids, const void* x,
                          int64_t T, int64_t H, int64_t E, int64_t K, int dtype,
                          int32_t* group_sizes, int32_t* offsets,
                          int32_t* source_order, int32_t* inverse, void* packed_x,
                          void* stream);

/*
 * Grouped SwiGLU expert FFN.  Replaces the three jax.lax.ragged_dot calls and
 * the SwiGLU between them (moe.py:638-641):
 *   rows offsets[e] .. offsets[e]+group_sizes[e]-1 of packed_x use expert e;
 *   act = silu(packed_x @ gate[e]) * (packed_x @ up[e]);  packed_y = act @ down[e].
 *
 *   packed_x [A,H] dtype; gate, up [E,H,I] dtype; down [E,I,H] dtype;
 *   group_sizes, offsets [E] i32 (device); act [A,I] dtype (workspace, overwritten);
 *   out: packed_y [A,H] dtype.  Groups of size 0 cost nothing.
 */
int jtmoe_grouped_swiglu(const void* packed_x, const void* gate, const void* up, const void* down,
                         const int32_t* group_sizes, const int32_t* offsets,
                         int64_t A, int64_t H, int64_t I, int64_t E, int dtype,
                         void* act, void* packed_y, void* stream);

/*
 * Grouped SwiGLU with the row gather fused in.  Replaces sorted_x = flat_x[source_order]
 * (moe.py:583, 595) together with the three ragged_dot calls (moe.py:638-641): packed row j is
 * fetched from x[source_order[j] / K] while the GEMM loads its tiles, so packed_x is never
 * materialised.  Same results as jtmoe_dispatch(..., x, packed_x) followed by
 * jtmoe_grouped_swiglu.  Only for shapes jtmoe_grouped_swiglu_gather_supported() accepts
 * (bf16, H and I multiples of 64); otherwise JTMOE_EUNSUPPORTED.
 *   x [T,H] dtype; source_order [T*K] i32; others as jtmoe_grouped_swiglu.
 */
int jtmoe_grouped_swiglu_gather_supported(int64_t T, int64_t H, int64_t I, int dtype);
int jtmoe_grouped_swiglu_gather(const void* x, const int32_t* source_order,
                                const void* gate, const void* up, const void* down,
                                const int32_t* group_sizes, const int32_t* offsets,
                                int64_t T, int64_t K, int64_t H, int64_t I, int64_t E, int dtype,
                                void* act, void* packed_y, void* stream);

/*
 * Shared experts.  Replaces SharedSwiGLU.__call__ (moe.py:361-364) on one device
 * (execution.py:186-187, 199-200): one dense SwiGLU of width Is = I*num_shared.
 *   x [T,H]; gate, up [H,Is]; down [Is,H]; act [T,Is] workspace; out shared_y [T,H].
 */
int jtmoe_shared_swiglu(const void* x, const void* gate, const void* up, const void* down,
                        int64_t T, int64_t H, int64_t Is, int dtype,
                        void* act, void* shared_y, void* stream);

/*
 * Combine.  Replaces the unpermute / weight / reduce of moe.py:663-671 and the
 * unweighted shared-expert add of moe.py:415, 429:
 *   y[t] = round_dtype( sum_s round_dtype(packed_y[inverse[t*K+s]] * weights[t,s]) )
 *   (fp32 accumulation in slot order), then y[t] = round_dtype(y[t] + shared_y[t]).
 *   packed_y [A,H]; inverse [A] i32; weights [T,K] dtype; shared_y [T,H] or NULL.
 */
int jtmoe_combine(const void* packed_y, const int32_t* inverse, const void* weights,
                  const void* shared_y, int64_t T, int64_t H, int64_t K, int dtype,
                  void* y, void* stream);

/*
 * Scalar router statistics.  Replaces the scalar fields of _router_stats
 * (moe.py:806-813) derived from expert_counts [E] f32:
 *   stats6 = {total_assignments, load_min, load_max, load_mean, max_vio, load_entropy}
 *   max_vio = (load_max - mean) / max(mean, 1e-6);  entropy = -sum_{p>0} p ln p, p = counts / max(total, 1e-6).
 */
int jtmoe_router_stats(const float* expert_counts, int64_t E, float* stats6, void* stream);

/*
 * Sequence balance loss.  Replaces _sequence_balance_loss (moe.py:828-840):
 *   f[b,e] = E/(K*S) * #{(s,k): ids[b,s,k]==e};  p[b,e] = mean_s scores[b,s,e]/max(sum_e scores, 1e-20);
 *   loss = sum_{b,e} f*p / B.
 *   expert_ids [B,S,K] i32; scores [B,S,E] f32; out loss [1] f32.
 *   workspace: jtmoe_balance_workspace_bytes(B, E) bytes.
 */
size_t jtmoe_balance_workspace_bytes(int64_t B, int64_t E);
int jtmoe_sequence_balance_loss(const int32_t* expert_ids, const float* scores,
                                int64_t B, int64_t S, int64_t E, int64_t K,
                                float* loss, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Gradient of jtmoe_sequence_balance_loss with respect to the scores: what jax.grad yields for
 * _sequence_balance_loss (moe.py:828-840) when the loss takes part in the training objective.  The
 * per-sequence counts come from one_hot(expert_ids) (moe.py:832) and carry no gradient.
 *   d_scores[b,s,e] = g / (B*S) * ( f[b,e] / D - (sum_i f[b,i] * scores[b,s,i]) / D^2 ),
 *   D = sum_e scores[b,s,e],  f[b,e] = E/(K*S) * #{(s,k): ids[b,s,k]==e},  g = *d_loss (1 if NULL).
 *   expert_ids [B,S,K] i32; scores [B,S,E] f32; d_loss [1] f32 (device) or NULL; out d_scores [B,S,E] f32.
 */
int jtmoe_sequence_balance_loss_backward(const int32_t* expert_ids, const float* scores, const float* d_loss,
                                         int64_t B, int64_t S, int64_t E, int64_t K,
                                         float* d_scores, void* stream);

/*
 * SMEBU balancing update: the consumer of expert_counts.  Replaces apply_moe_balance_update
 * (steps/moe_balance.py:97-162) and the bias write of _update_expert_biases (:174-184) for L MoE
 * layers of E experts, on device buffers (hand the layer calls rows of one [L,E] counts buffer as
 * their expert_counts output and nothing passes through the host):
 *   mean = sum(counts)/E; violation = (mean - counts)/max(mean, 1e-6);
 *   delta = load_lr * tanh(clamp * violation); delta -= mean(delta);
 *   momentum = momentum_factor * momentum + (1 - momentum_factor) * delta;  expert_bias += momentum.
 *   router_counts [L,E] f32; momentum, expert_bias [L,E] f32, updated in place;
 *   metrics6 = {max_vio (max over layers), load_min, load_max, load_entropy (mean over layers),
 *               bias_norm, momentum_norm}  (MoeBalanceMetrics, :32-41).
 *   load_lr, momentum_factor, clamp > 0 (MoeBalanceSpec, specs/model.py:18-36).
 */
int jtmoe_smebu_update(const float* router_counts, float* momentum, float* expert_bias,
                       int64_t L, int64_t E, float load_lr, float momentum_factor, float clamp,
                       float* metrics6, void* stream);

/*
 * The whole layer.  Replaces SparseMoE.__call__ / forward_with_output
 * (moe.py:411-446): router -> dispatch -> grouped SwiGLU -> (shared experts) ->
 * combine, enqueued back to back on `stream`.
 *
 *   shared_gate/up [H,Is], shared_down [Is,H], or all NULL with Is == 0.
 *   out: y [T,H]; expert_ids [T,K]; weights [T,K]; scores [T,E];
 *        expert_counts, importance [E] f32; group_sizes, offsets [E] i32;
 *        source_order, inverse [A] i32.
 *   workspace: jtmoe_workspace_bytes(...) bytes, 256-byte aligned.  Where
 *        jtmoe_grouped_swiglu_gather_supported(T, H, I, dtype) holds, the grouped
 *        GEMM fetches its rows through the permutation, the workspace holds no
 *        permuted copy of x ([A,H]: a third of it at 64 experts, top-8, H = 2048),
 *        and x, gate, up and down must be 16-byte aligned (JTMOE_EINVAL otherwise).
 *   decode sizes: where jtmoe_moe_forward_takes_decode_path(T, H, E, K, I, dtype) holds (bf16, at
 *        most 64 tokens, T*K >= 2*E, 16 / 32 / 64 experts, H a multiple of 128: a decode
 *        step), one launch runs every token through every expert's gate and up matrices --
 *        which needs nothing of the routing -- while a few of its workgroups are the
 *        router and write the dispatch plan; the down launch then takes the routed rows.
 *        The workspace then holds the activations [E,T,I]; results are bit for bit those
 *        of the other path.  That launch counts its router workgroups in a word of the
 *        workspace (tagged per launch, so the workspace needs no clearing): like every
 *        call, it shares no state with calls that use other workspaces.  No counterpart
 *        in the reference (XLA decides its own fusions).
 */
int jtmoe_moe_forward_takes_decode_path(int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int dtype);
size_t jtmoe_workspace_bytes(int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is, int dtype);
int jtmoe_moe_forward(const void* x, const void* w_router, const float* expert_bias,
                      const void* gate, const void* up, const void* down,
                      const void* shared_gate, const void* shared_up, const void* shared_down,
                      int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is,
                      double route_scale, int dtype,
                      void* y, int32_t* expert_ids, void* weights, float* scores,
                      float* expert_counts, float* importance,
                      int32_t* group_sizes, int32_t* offsets,
                      int32_t* source_order, int32_t* inverse,
                      void* workspace, size_t workspace_bytes, void* stream);
int jtmoe_moe_forward_sf(const void* x, const void* w_router, const float* expert_bias,
                         const void* gate, const void* up, const void* down,
                         const void* shared_gate, const void* shared_up, const void* shared_down,
                         int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is,
                         double route_scale, int score_func, int dtype,
                         void* y, int32_t* expert_ids, void* weights, float* scores,
                         float* expert_counts, float* importance,
                         int32_t* group_sizes, int32_t* offsets,
                         int32_t* source_order, int32_t* inverse,
                         void* workspace, size_t workspace_bytes, void* stream);

/*
 * Measurement aid with no counterpart in the reference (its benchmarks time
 * whole calls, src/jaxtitan/runtime/profile_bench.py:232-270): one
 * jtmoe_moe_forward with a hipEvent recorded on `stream` after every stage.
 * Unlike every other entry point it creates events and SYNCHRONISES the stream.
 * stage_ms is a HOST array of JTMOE_NUM_STAGES floats, milliseconds per stage:
 *   {router, dispatch (histogram+scan+rank), dispatch (row scatter),
 *    routed gate/up GEMM + SwiGLU, routed down GEMM,
 *    shared gate/up GEMM + SwiGLU, shared down GEMM, combine}.
 */
#define JTMOE_NUM_STAGES 8
int jtmoe_moe_forward_timed(const void* x, const void* w_router, const float* expert_bias,
                            const void* gate, const void* up, const void* down,
                            const void* shared_gate, const void* shared_up, const void* shared_down,
                            int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is,
                            double route_scale, int dtype,
                            void* y, int32_t* expert_ids, void* weights, float* scores,
                            float* expert_counts, float* importance,
                            int32_t* group_sizes, int32_t* offsets,
                            int32_t* source_order, int32_t* inverse,
                            void* workspace, size_t workspace_bytes, void* stream,
                            float* stage_ms);

/* ------------------------------------------------------------------------------------------
 * The decoder block around the layer (blocks.py:224-230):
 *     x = x + ffn_post_norm(mlp(ffn_pre_norm(x)))
 * ------------------------------------------------------------------------------------------ */

/*
 * RMSNorm over the last axis.  Replaces the modules of build_rms_norm
 * (models/components/norm.py:12-31: flax nnx.RMSNorm, float32 scale) and the reference's
 * forward-only kernel boundary rmsnorm_reference / rmsnorm_tk_forward
 * (kernels/rmsnorm.py:14-52, kernels/cuda/rmsnorm/rmsnorm_ffi.cu):
 *   y = round_dtype( f32(x) * (1/sqrt(mean(f32(x)^2) + eps) * scale) ),  scale float32 [H].
 */
int jtmoe_rmsnorm(const void* x, const float* scale, int64_t T, int64_t H, double eps, int dtype,
                  void* y, void* stream);

/*
 * jtmoe_combine followed, inside the same kernel, by the block's tail:
 *   out[t] = round( residual[t] + rmsnorm(y[t]; post_scale, eps) ),  y = the plain combine result.
 */
int jtmoe_combine_norm_residual(const void* packed_y, const int32_t* inverse, const void* weights,
                                const void* shared_y, const void* residual, const float* post_scale,
                                double eps, int64_t T, int64_t H, int64_t K, int dtype,
                                void* out, void* stream);

/*
 * The block's second half in one call: out = x + rmsnorm(moe(rmsnorm(x; pre_scale)); post_scale).
 * Router outputs and dispatch plan as in jtmoe_moe_forward (they refer to the normalised x).
 */
size_t jtmoe_ffn_block_workspace_bytes(int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is,
                                       int dtype);
int jtmoe_ffn_block_forward(const void* x, const float* pre_scale, const float* post_scale, double eps,
                            const void* w_router, const float* expert_bias,
                            const void* gate, const void* up, const void* down,
                            const void* shared_gate, const void* shared_up, const void* shared_down,
                            int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is,
                            double route_scale, int dtype,
                            void* out, int32_t* expert_ids, void* weights, float* scores,
                            float* expert_counts, float* importance,
                            int32_t* group_sizes, int32_t* offsets,
                            int32_t* source_order, int32_t* inverse,
                            void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * Training: forward passes that keep residuals, and the vector-Jacobian products.
 *
 * The reference trains SparseMoE through JAX automatic differentiation and requires a
 * forward-only kernel to bring its own VJP before it may replace a training component
 * (docs/kernel_backend_design.md:120-128).  These entry points are that VJP, operator by
 * operator; the gradient tests of the reference's expert dispatcher are the specification
 * (tests/jaxtitan/test_model.py:549-691: gradients with respect to x, route weights, gate,
 * up and down; repeated calls must return identical bits).
 *
 * Residuals: gate_pre = round(Xp Wg[e]) and up_pre = round(Xp Wu[e]), both [A, I] in the
 * compute dtype (packed row order), and the same two for the shared experts, [T, Is].
 * Gradients of rounding steps are passed straight through.  Gradient outputs have the
 * compute dtype and the shape of what they differentiate.
 * ------------------------------------------------------------------------------------------ */

/*
 * jtmoe_grouped_swiglu / jtmoe_grouped_swiglu_gather that also store gate_pre and up_pre.
 * source_order != NULL: x is [T, H] token-major and packed row j reads token
 * source_order[j] / K (A = T*K); source_order == NULL: x is already packed, A = T rows.
 */
int jtmoe_grouped_swiglu_train(const void* x, const int32_t* source_order,
                               const void* gate, const void* up, const void* down,
                               const int32_t* group_sizes, const int32_t* offsets,
                               int64_t T, int64_t K, int64_t H, int64_t I, int64_t E, int dtype,
                               void* gate_pre, void* up_pre, void* act, void* packed_y, void* stream);

/* jtmoe_shared_swiglu that also stores gate_pre and up_pre ([T, Is]). */
int jtmoe_shared_swiglu_train(const void* x, const void* gate, const void* up, const void* down,
                              int64_t T, int64_t H, int64_t Is, int dtype,
                              void* gate_pre, void* up_pre, void* act, void* shared_y, void* stream);

/*
 * VJP of dispatch -> grouped SwiGLU -> combine (moe.py:583-671) for the cotangent dy [T, H]:
 *   dx [T, H]        = sum_s dXp[inverse[t,s]]  (+ dx_extra, if given: e.g. the shared experts'
 *                      and the router's contribution to the gradient of x)
 *   d_weights [T, K] = <dy[t], Yp[inverse[t,s]]>
 *   d_gate, d_up [E, H, I], d_down [E, I, H]; experts without rows get zeros.
 * weights are the route weights [T, K] of the forward pass.
 */
size_t jtmoe_experts_backward_workspace_bytes(int64_t T, int64_t K, int64_t H, int64_t I, int dtype);
int jtmoe_experts_backward(const void* x, const void* dy,
                           const int32_t* source_order, const int32_t* inverse, const void* weights,
                           const int32_t* group_sizes, const int32_t* offsets,
                           const void* gate, const void* up, const void* down,
                           const void* gate_pre, const void* up_pre,
                           int64_t T, int64_t K, int64_t H, int64_t I, int64_t E, int dtype,
                           const void* dx_extra,
                           void* dx, void* d_weights, void* d_gate, void* d_up, void* d_down,
                           void* workspace, size_t workspace_bytes, void* stream);

/* VJP of SharedSwiGLU.__call__ (moe.py:361-364): dx [T, H], d_gate, d_up [H, Is], d_down [Is, H]. */
size_t jtmoe_shared_backward_workspace_bytes(int64_t T, int64_t H, int64_t Is, int dtype);
int jtmoe_shared_backward(const void* x, const void* dy,
                          const void* gate, const void* up, const void* down,
                          const void* gate_pre, const void* up_pre,
                          int64_t T, int64_t H, int64_t Is, int dtype,
                          void* dx, void* d_gate, void* d_up, void* d_down,
                          void* workspace, size_t workspace_bytes, void* stream);

/*
 * VJP of SigmoidTopKRouter.__call__ (moe.py:131-147) for the cotangents d_weights [T, K]
 * (compute dtype) and, optionally, d_scores [T, E] (fp32; NULL = zeros), e.g. from an
 * auxiliary loss on the scores.  scores and expert_ids are the forward's outputs.  The
 * selection itself and the expert bias carry no gradient (moe.py:139-140).
 *   dx [T, H], d_w_router [H, E].
 */
size_t jtmoe_router_backward_workspace_bytes(int64_t T, int64_t H, int64_t E, int dtype);
int jtmoe_router_backward(const void* x, const void* w_router,
                          const float* scores, const int32_t* expert_ids,
                          const void* d_weights, const float* d_scores, double route_scale,
                          int64_t T, int64_t H, int64_t E, int64_t K, int dtype,
                          void* dx, void* d_w_router,
                          void* workspace, size_t workspace_bytes, void* stream);
int jtmoe_router_backward_sf(const void* x, const void* w_router,
                             const float* scores, const int32_t* expert_ids,
                             const void* d_weights, const float* d_scores, double route_scale, int score_func,
                             int64_t T, int64_t H, int64_t E, int64_t K, int dtype,
                             void* dx, void* d_w_router,
                             void* workspace, size_t workspace_bytes, void* stream);

/*
 * The layer: jtmoe_moe_forward that also stores the residuals, and the VJP of
 * SparseMoE.forward_with_output (moe.py:409-430) for the cotangents dy [T, H] and
 * d_scores [T, E] (NULL = zeros).  Is == 0: pass NULL for every shared-expert argument.
 */
int jtmoe_moe_forward_train(const void* x, const void* w_router, const float* expert_bias,
                            const void* gate, const void* up, const void* down,
                            const void* shared_gate, const void* shared_up, const void* shared_down,
                            int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is,
                            double route_scale, int dtype,
                            void* y, int32_t* expert_ids, void* weights, float* scores,
                            float* expert_counts, float* importance,
                            int32_t* group_sizes, int32_t* offsets,
                            int32_t* source_order, int32_t* inverse,
                            void* gate_pre, void* up_pre, void* shared_gate_pre, void* shared_up_pre,
                            void* workspace, size_t workspace_bytes, void* stream);
int jtmoe_moe_forward_train_sf(const void* x, const void* w_router, const float* expert_bias,
                               const void* gate, const void* up, const void* down,
                               const void* shared_gate, const void* shared_up, const void* shared_down,
                               int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is,
                               double route_scale, int score_func, int dtype,
                               void* y, int32_t* expert_ids, void* weights, float* scores,
                               float* expert_counts, float* importance,
                               int32_t* group_sizes, int32_t* offsets,
                               int32_t* source_order, int32_t* inverse,
                               void* gate_pre, void* up_pre, void* shared_gate_pre, void* shared_up_pre,
                               void* workspace, size_t workspace_bytes, void* stream);

size_t jtmoe_moe_backward_workspace_bytes(int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is,
                                          int dtype);
int jtmoe_moe_backward(const void* x, const void* dy, const float* d_scores,
                       const void* w_router, const void* gate, const void* up, const void* down,
                       const void* shared_gate, const void* shared_up, const void* shared_down,
                       const float* scores, const int32_t* expert_ids, const void* weights,
                       const int32_t* source_order, const int32_t* inverse,
                       const int32_t* group_sizes, const int32_t* offsets,
                       const void* gate_pre, const void* up_pre,
                       const void* shared_gate_pre, const void* shared_up_pre,
                       double route_scale,
                       int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is, int dtype,
                       void* dx, void* d_w_router, void* d_gate, void* d_up, void* d_down,
                       void* d_shared_gate, void* d_shared_up, void* d_shared_down,
                       void* workspace, size_t workspace_bytes, void* stream);
int jtmoe_moe_backward_sf(const void* x, const void* dy, const float* d_scores,
                          const void* w_router, const void* gate, const void* up, const void* down,
                          const void* shared_gate, const void* shared_up, const void* shared_down,
                          const float* scores, const int32_t* expert_ids, const void* weights,
                          const int32_t* source_order, const int32_t* inverse,
                          const int32_t* group_sizes, const int32_t* offsets,
                          const void* gate_pre, const void* up_pre,
                          const void* shared_gate_pre, const void* shared_up_pre,
                          double route_scale, int score_func,
                          int64_t T, int64_t H, int64_t E, int64_t K, int64_t I, int64_t Is, int dtype,
                          void* dx, void* d_w_router, void* d_gate, void* d_up, void* d_down,
                          void* d_shared_gate, void* d_shared_up, void* d_shared_down,
                          void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* JTMOE_H_ */
