// XLA FFI handlers for libjtmoe: thin shims that unpack XLA buffers and forward to the
// extern "C" launchers of include/jtmoe.h.  They follow the reference's handler
// (src/jaxtitan/kernels/cuda/rmsnorm/rmsnorm_ffi.cu:24-85): validate rank / shape / dtype and
// return InvalidArgument, launch on the stream XLA supplies, never allocate (scratch is an
// extra result buffer that XLA allocates), map a launch failure to Internal.
//
// Built only where xla/ffi/api/ffi.h exists (it ships inside jaxlib and is located with
// jax.ffi.include_dir(), cf. src/jaxtitan/kernels/build.py:280-283):
//     make ffi XLA_FFI_INCLUDE=$(python -c "import jax; print(jax.ffi.include_dir())")
#include "xla/ffi/api/ffi.h"

#include <hip/hip_runtime.h>

#include <cstdint>

#include "jtmoe.h"

namespace ffi = xla::ffi;

namespace {

int dtype_code(ffi::DataType t) {
  if (t == ffi::DataType::BF16) return JTMOE_BF16;
  if (t == ffi::DataType::F32) return JTMOE_F32;
  return -1;
}

ffi::Error status_to_error(int rc) {
  if (rc == JTMOE_OK) return ffi::Error::Success();
  if (rc == JTMOE_ELAUNCH) return ffi::Error::Internal(jtmoe_last_error());
  return ffi::Error::InvalidArgument(jtmoe_last_error());
}

int64_t leading(ffi::Span<const int64_t> dims) {  // product of all but the last dimension
  int64_t n = 1;
  for (size_t i = 0; i + 1 < dims.size(); ++i) n *= dims[i];
  return n;
}

// x [..., H], w_router [H, E], expert_bias [E] f32, gate/up [E, H, I], down [E, I, H],
// shared_gate/up [H, Is], shared_down [Is, H] (Is may be 0: pass [H,0] / [0,H] arrays)
ffi::Error MoeForward(hipStream_t stream, ffi::AnyBuffer x, ffi::AnyBuffer w_router,
                      ffi::Buffer<ffi::DataType::F32> expert_bias, ffi::AnyBuffer gate, ffi::AnyBuffer up,
                      ffi::AnyBuffer down, ffi::AnyBuffer shared_gate, ffi::AnyBuffer shared_up,
                      ffi::AnyBuffer shared_down, ffi::Result<ffi::AnyBuffer> y,
                      ffi::Result<ffi::Buffer<ffi::DataType::S32>> expert_ids, ffi::Result<ffi::AnyBuffer> weights,
                      ffi::Result<ffi::Buffer<ffi::DataType::F32>> scores,
                      ffi::Result<ffi::Buffer<ffi::DataType::F32>> expert_counts,
                      ffi::Result<ffi::Buffer<ffi::DataType::F32>> importance,
                      ffi::Result<ffi::Buffer<ffi::DataType::S32>> group_sizes,
                      ffi::Result<ffi::Buffer<ffi::DataType::S32>> offsets,
                      ffi::Result<ffi::Buffer<ffi::DataType::S32>> source_order,
                      ffi::Result<ffi::Buffer<ffi::DataType::S32>> inverse,
                      ffi::Result<ffi::Buffer<ffi::DataType::U8>> workspace, int64_t top_k, double route_scale) {
  const auto xd = x.dimensions();
  const auto gd = gate.dimensions();
  if (xd.size() < 2) return ffi::Error::InvalidArgument("moe input rank must be at least 2");
  if (gd.size() != 3) return ffi::Error::InvalidArgument("expert gate matrix must be rank 3");
  const int dtype = dtype_code(x.element_type());
  if (dtype < 0) return ffi::Error::InvalidArgument("moe compute dtype must be bfloat16 or float32");
  for (const ffi::AnyBuffer* b : {&w_router, &gate, &up, &down, &shared_gate, &shared_up, &shared_down})
    if (b->element_type() != x.element_type())
      return ffi::Error::InvalidArgument("moe weights must have the dtype of the input");
  const int64_t H = xd.back(), T = leading(xd), E = gd[0], I = gd[2];
  const int64_t Is = shared_gate.dimensions().size() == 2 ? shared_gate.dimensions()[1] : 0;
  if (gd[1] != H) return ffi::Error::InvalidArgument("expert gate matrix must be [E, H, I]");
  const auto wd = w_router.dimensions();
  if (wd.size() != 2 || wd[0] != H || wd[1] != E) return ffi::Error::InvalidArgument("router kernel must be [H, E]");
  if (expert_bias.element_count() != static_cast<size_t>(E))
    return ffi::Error::InvalidArgument("expert_bias must have shape [E]");
  if (workspace->element_count() < jtmoe_workspace_bytes(T, H, E, top_k, I, Is, dtype))
    return ffi::Error::InvalidArgument("moe workspace result buffer is too small");
  const int rc = jtmoe_moe_forward(
      x.untyped_data(), w_router.untyped_data(), expert_bias.typed_data(), gate.untyped_data(), up.untyped_data(),
      down.untyped_data(), Is ? shared_gate.untyped_data() : nullptr, Is ? shared_up.untyped_data() : nullptr,
      Is ? shared_down.untyped_data() : nullptr, T, H, E, top_k, I, Is, route_scale, dtype, y->untyped_data(),
      expert_ids->typed_data(), weights->untyped_data(), scores->typed_data(), expert_counts->typed_data(),
      importance->typed_data(), group_sizes->typed_data(), offsets->typed_data(), source_order->typed_data(),
      inverse->typed_data(), workspace->typed_data(), workspace->element_count(), stream);
  return status_to_error(rc);
}

ffi::Error MoeRouter(hipStream_t stream, ffi::AnyBuffer x, ffi::AnyBuffer w_router,
                     ffi::Buffer<ffi::DataType::F32> expert_bias,
                     ffi::Result<ffi::Buffer<ffi::DataType::S32>> expert_ids, ffi::Result<ffi::AnyBuffer> weights,
                     ffi::Result<ffi::Buffer<ffi::DataType::F32>> scores,
                     ffi::Result<ffi::Buffer<ffi::DataType::F32>> expert_counts,
                     ffi::Result<ffi::Buffer<ffi::DataType::F32>> importance,
                     ffi::Result<ffi::Buffer<ffi::DataType::U8>> workspace, int64_t top_k, double route_scale) {
  const auto xd = x.dimensions();
  const auto wd = w_router.dimensions();
  if (xd.size() < 2 || wd.size() != 2 || wd[0] != xd.back())
    return ffi::Error::InvalidArgument("router expects x [..., H] and kernel [H, E]");
  const int dtype = dtype_code(x.element_type());
  if (dtype < 0 || w_router.element_type() != x.element_type())
    return ffi::Error::InvalidArgument("router dtype must be bfloat16 or float32 for x and kernel alike");
  const int rc = jtmoe_router(x.untyped_data(), w_router.untyped_data(), expert_bias.typed_data(), leading(xd),
                              xd.back(), wd[1], top_k, route_scale, dtype, expert_ids->typed_data(),
                              weights->untyped_data(), scores->typed_data(), expert_counts->typed_data(),
                              importance->typed_data(), nullptr, workspace->typed_data(),
                              workspace->element_count(), stream);
  return status_to_error(rc);
}

ffi::Error MoeDispatch(hipStream_t stream, ffi::Buffer<ffi::DataType::S32> expert_ids, ffi::AnyBuffer x,
                       ffi::Result<ffi::Buffer<ffi::DataType::S32>> group_sizes,
                       ffi::Result<ffi::Buffer<ffi::DataType::S32>> offsets,
                       ffi::Result<ffi::Buffer<ffi::DataType::S32>> source_order,
                       ffi::Result<ffi::Buffer<ffi::DataType::S32>> inverse, ffi::Result<ffi::AnyBuffer> packed_x,
                       ffi::Result<ffi::Buffer<ffi::DataType::U8>> workspace) {
  const auto id = expert_ids.dimensions();
  const auto xd = x.dimensions();
  if (id.size() < 1 || xd.size() < 2) return ffi::Error::InvalidArgument("dispatch expects ids [..., K] and x [..., H]");
  const int dtype = dtype_code(x.element_type());
  if (dtype < 0) return ffi::Error::InvalidArgument("dispatch dtype must be bfloat16 or float32");
  const int64_t K = id.back(), T = leading(xd);
  if (leading(id) != T) return ffi::Error::InvalidArgument("dispatch ids and x disagree on the token count");
  const int rc = jtmoe_dispatch(expert_ids.typed_data(), x.untyped_data(), T, xd.back(),
                                static_cast<int64_t>(group_sizes->element_count()), K, dtype,
                                group_sizes->typed_data(), offsets->typed_data(), source_order->typed_data(),
                                inverse->typed_data(), packed_x->untyped_data(), workspace->typed_data(),
                                workspace->element_count(), stream);
  return status_to_error(rc);
}

ffi::Error MoeGroupedSwiglu(hipStream_t stream, ffi::AnyBuffer packed_x, ffi::AnyBuffer gate, ffi::AnyBuffer up,
                            ffi::AnyBuffer down, ffi::Buffer<ffi::DataType::S32> group_sizes,
                            ffi::Buffer<ffi::DataType::S32> offsets, ffi::Result<ffi::AnyBuffer> packed_y,
                            ffi::Result<ffi::AnyBuffer> act) {
  const auto pd = packed_x.dimensions();
  const auto gd = gate.dimensions();
  if (pd.size() != 2 || gd.size() != 3 || gd[1] != pd[1])
    return ffi::Error::InvalidArgument("grouped_swiglu expects packed_x [A, H] and gate [E, H, I]");
  const int dtype = dtype_code(packed_x.element_type());
  if (dtype < 0) return ffi::Error::InvalidArgument("grouped_swiglu dtype must be bfloat16 or float32");
  const int rc = jtmoe_grouped_swiglu(packed_x.untyped_data(), gate.untyped_data(), up.untyped_data(),
                                      down.untyped_data(), group_sizes.typed_data(), offsets.typed_data(), pd[0],
                                      pd[1], gd[2], gd[0], dtype, act->untyped_data(), packed_y->untyped_data(),
                                      stream);
  return status_to_error(rc);
}

ffi::Error MoeCombine(hipStream_t stream, ffi::AnyBuffer packed_y, ffi::Buffer<ffi::DataType::S32> inverse,
                      ffi::AnyBuffer weights, ffi::Result<ffi::AnyBuffer> y) {
  const auto pd = packed_y.dimensions();
  const auto wd = weights.dimensions();
  if (pd.size() != 2 || wd.size() < 1) return ffi::Error::InvalidArgument("combine expects packed_y [A, H], weights [..., K]");
  const int dtype = dtype_code(packed_y.element_type());
  if (dtype < 0 || weights.element_type() != packed_y.element_type())
    return ffi::Error::InvalidArgument("combine dtype must be bfloat16 or float32 for packed_y and weights alike");
  const int rc = jtmoe_combine(packed_y.untyped_data(), inverse.typed_data(), weights.untyped_data(), nullptr,
                               leading(wd), pd[1], wd.back(), dtype, y->untyped_data(), stream);
  return status_to_error(rc);
}

// Forward that keeps the residuals of the backward pass.  Same operands as MoeForward; four more
// results: gate_pre, up_pre [A, I] and shared_gate_pre, shared_up_pre [T, Is].
ffi::Error MoeForwardTrain(hipStream_t stream, ffi::AnyBuffer x, ffi::AnyBuffer w_router,
                           ffi::Buffer<ffi::DataType::F32> expert_bias, ffi::AnyBuffer gate, ffi::AnyBuffer up,
                           ffi::AnyBuffer down, ffi::AnyBuffer shared_gate, ffi::AnyBuffer shared_up,
                           ffi::AnyBuffer shared_down, ffi::Result<ffi::AnyBuffer> y,
                           ffi::Result<ffi::Buffer<ffi::DataType::S32>> expert_ids,
                           ffi::Result<ffi::AnyBuffer> weights, ffi::Result<ffi::Buffer<ffi::DataType::F32>> scores,
                           ffi::Result<ffi::Buffer<ffi::DataType::F32>> expert_counts,
                           ffi::Result<ffi::Buffer<ffi::DataType::F32>> importance,
                           ffi::Result<ffi::Buffer<ffi::DataType::S32>> group_sizes,
                           ffi::Result<ffi::Buffer<ffi::DataType::S32>> offsets,
                           ffi::Result<ffi::Buffer<ffi::DataType::S32>> source_order,
                           ffi::Result<ffi::Buffer<ffi::DataType::S32>> inverse, ffi::Result<ffi::AnyBuffer> gate_pre,
                           ffi::Result<ffi::AnyBuffer> up_pre, ffi::Result<ffi::AnyBuffer> shared_gate_pre,
                           ffi::Result<ffi::AnyBuffer> shared_up_pre,
                           ffi::Result<ffi::Buffer<ffi::DataType::U8>> workspace, int64_t top_k, double route_scale) {
  const auto xd = x.dimensions();
  const auto gd = gate.dimensions();
  if (xd.size() < 2 || gd.size() != 3) return ffi::Error::InvalidArgument("moe expects x [..., H] and gate [E, H, I]");
  const int dtype = dtype_code(x.element_type());
  if (dtype < 0) return ffi::Error::InvalidArgument("moe compute dtype must be bfloat16 or float32");
  const int64_t H = xd.back(), T = leading(xd), E = gd[0], I = gd[2];
  const int64_t Is = shared_gate.dimensions().size() == 2 ? shared_gate.dimensions()[1] : 0;
  if (gd[1] != H) return ffi::Error::InvalidArgument("expert gate matrix must be [E, H, I]");
  if (workspace->element_count() < jtmoe_workspace_bytes(T, H, E, top_k, I, Is, dtype))
    return ffi::Error::InvalidArgument("moe workspace result buffer is too small");
  const int rc = jtmoe_moe_forward_train(
      x.untyped_data(), w_router.untyped_data(), expert_bias.typed_data(), gate.untyped_data(), up.untyped_data(),
      down.untyped_data(), Is ? shared_gate.untyped_data() : nullptr, Is ? shared_up.untyped_data() : nullptr,
      Is ? shared_down.untyped_data() : nullptr, T, H, E, top_k, I, Is, route_scale, dtype, y->untyped_data(),
      expert_ids->typed_data(), weights->untyped_data(), scores->typed_data(), expert_counts->typed_data(),
      importance->typed_data(), group_sizes->typed_data(), offsets->typed_data(), source_order->typed_data(),
      inverse->typed_data(), gate_pre->untyped_data(), up_pre->untyped_data(),
      Is ? shared_gate_pre->untyped_data() : nullptr, Is ? shared_up_pre->untyped_data() : nullptr,
      workspace->typed_data(), workspace->element_count(), stream);
  return status_to_error(rc);
}

// Vector-Jacobian product of the layer for the cotangents dy [..., H] and d_scores [..., E].
ffi::Error MoeBackward(hipStream_t stream, ffi::AnyBuffer x, ffi::AnyBuffer dy,
                       ffi::Buffer<ffi::DataType::F32> d_scores, ffi::AnyBuffer w_router, ffi::AnyBuffer gate,
                       ffi::AnyBuffer up, ffi::AnyBuffer down, ffi::AnyBuffer shared_gate, ffi::AnyBuffer shared_up,
                       ffi::AnyBuffer shared_down, ffi::Buffer<ffi::DataType::F32> scores,
                       ffi::Buffer<ffi::DataType::S32> expert_ids, ffi::AnyBuffer weights,
                       ffi::Buffer<ffi::DataType::S32> source_order, ffi::Buffer<ffi::DataType::S32> inverse,
                       ffi::Buffer<ffi::DataType::S32> group_sizes, ffi::Buffer<ffi::DataType::S32> offsets,
                       ffi::AnyBuffer gate_pre, ffi::AnyBuffer up_pre, ffi::AnyBuffer shared_gate_pre,
                       ffi::AnyBuffer shared_up_pre, ffi::Result<ffi::AnyBuffer> dx,
                       ffi::Result<ffi::AnyBuffer> d_w_router, ffi::Result<ffi::AnyBuffer> d_gate,
                       ffi::Result<ffi::AnyBuffer> d_up, ffi::Result<ffi::AnyBuffer> d_down,
                       ffi::Result<ffi::AnyBuffer> d_shared_gate, ffi::Result<ffi::AnyBuffer> d_shared_up,
                       ffi::Result<ffi::AnyBuffer> d_shared_down,
                       ffi::Result<ffi::Buffer<ffi::DataType::U8>> workspace, double route_scale) {
  const auto xd = x.dimensions();
  const auto gd = gate.dimensions();
  const auto id = expert_ids.dimensions();
  if (xd.size() < 2 || gd.size() != 3 || id.size() < 1)
    return ffi::Error::InvalidArgument("moe backward expects x [..., H], gate [E, H, I] and ids [..., K]");
  const int dtype = dtype_code(x.element_type());
  if (dtype < 0 || dy.element_type() != x.element_type())
    return ffi::Error::InvalidArgument("moe backward: x and dy must both be bfloat16 or float32");
  const int64_t H = xd.back(), T = leading(xd), E = gd[0], I = gd[2], K = id.back();
  const int64_t Is = shared_gate.dimensions().size() == 2 ? shared_gate.dimensions()[1] : 0;
  if (workspace->element_count() < jtmoe_moe_backward_workspace_bytes(T, H, E, K, I, Is, dtype))
    return ffi::Error::InvalidArgument("moe backward workspace result buffer is too small");
  const int rc = jtmoe_moe_backward(
      x.untyped_data(), dy.untyped_data(), d_scores.typed_data(), w_router.untyped_data(), gate.untyped_data(),
      up.untyped_data(), down.untyped_data(), Is ? shared_gate.untyped_data() : nullptr,
      Is ? shared_up.untyped_data() : nullptr, Is ? shared_down.untyped_data() : nullptr, scores.typed_data(),
      expert_ids.typed_data(), weights.untyped_data(), source_order.typed_data(), inverse.typed_data(),
      group_sizes.typed_data(), offsets.typed_data(), gate_pre.untyped_data(), up_pre.untyped_data(),
      Is ? shared_gate_pre.untyped_data() : nullptr, Is ? shared_up_pre.untyped_data() : nullptr, route_scale, T, H,
      E, K, I, Is, dtype, dx->untyped_data(), d_w_router->untyped_data(), d_gate->untyped_data(),
      d_up->untyped_data(), d_down->untyped_data(), Is ? d_shared_gate->untyped_data() : nullptr,
      Is ? d_shared_up->untyped_data() : nullptr, Is ? d_shared_down->untyped_data() : nullptr,
      workspace->typed_data(), workspace->element_count(), stream);
  return status_to_error(rc);
}

// RMSNorm with a float32 scale, the operands of the reference's own handler
// (rmsnorm_ffi.cu:24-74) for any hidden size and both dtypes.
ffi::Error Rmsnorm(hipStream_t stream, ffi::AnyBuffer x, ffi::Buffer<ffi::DataType::F32> scale,
                   ffi::Result<ffi::AnyBuffer> y, double eps) {
  const auto xd = x.dimensions();
  if (xd.size() < 2) return ffi::Error::InvalidArgument("rmsnorm input rank must be at least 2");
  if (scale.element_count() != static_cast<size_t>(xd.back()))
    return ffi::Error::InvalidArgument("rmsnorm scale must have shape [H]");
  const int dtype = dtype_code(x.element_type());
  if (dtype < 0) return ffi::Error::InvalidArgument("rmsnorm dtype must be bfloat16 or float32");
  return status_to_error(
      jtmoe_rmsnorm(x.untyped_data(), scale.typed_data(), leading(xd), xd.back(), eps, dtype, y->untyped_data(), stream));
}

// x + post_norm(moe(pre_norm(x))): operands of MoeForward preceded by x's two norm scales.
ffi::Error FfnBlockForward(hipStream_t stream, ffi::AnyBuffer x, ffi::Buffer<ffi::DataType::F32> pre_scale,
                           ffi::Buffer<ffi::DataType::F32> post_scale, ffi::AnyBuffer w_router,
                           ffi::Buffer<ffi::DataType::F32> expert_bias, ffi::AnyBuffer gate, ffi::AnyBuffer up,
                           ffi::AnyBuffer down, ffi::AnyBuffer shared_gate, ffi::AnyBuffer shared_up,
                           ffi::AnyBuffer shared_down, ffi::Result<ffi::AnyBuffer> out,
                           ffi::Result<ffi::Buffer<ffi::DataType::S32>> expert_ids,
                           ffi::Result<ffi::AnyBuffer> weights, ffi::Result<ffi::Buffer<ffi::DataType::F32>> scores,
                           ffi::Result<ffi::Buffer<ffi::DataType::F32>> expert_counts,
                           ffi::Result<ffi::Buffer<ffi::DataType::F32>> importance,
                           ffi::Result<ffi::Buffer<ffi::DataType::S32>> group_sizes,
                           ffi::Result<ffi::Buffer<ffi::DataType::S32>> offsets,
                           ffi::Result<ffi::Buffer<ffi::DataType::S32>> source_order,
                           ffi::Result<ffi::Buffer<ffi::DataType::S32>> inverse,
                           ffi::Result<ffi::Buffer<ffi::DataType::U8>> workspace, int64_t top_k, double route_scale,
                           double eps) {
  const auto xd = x.dimensions();
  const auto gd = gate.dimensions();
  if (xd.size() < 2 || gd.size() != 3) return ffi::Error::InvalidArgument("block expects x [..., H] and gate [E, H, I]");
  const int dtype = dtype_code(x.element_type());
  if (dtype < 0) return ffi::Error::InvalidArgument("block compute dtype must be bfloat16 or float32");
  const int64_t H = xd.back(), T = leading(xd), E = gd[0], I = gd[2];
  const int64_t Is = shared_gate.dimensions().size() == 2 ? shared_gate.dimensions()[1] : 0;
  if (pre_scale.element_count() != static_cast<size_t>(H) || post_scale.element_count() != static_cast<size_t>(H))
    return ffi::Error::InvalidArgument("norm scales must have shape [H]");
  if (workspace->element_count() < jtmoe_ffn_block_workspace_bytes(T, H, E, top_k, I, Is, dtype))
    return ffi::Error::InvalidArgument("block workspace result buffer is too small");
  const int rc = jtmoe_ffn_block_forward(
      x.untyped_data(), pre_scale.typed_data(), post_scale.typed_data(), eps, w_router.untyped_data(),
      expert_bias.typed_data(), gate.untyped_data(), up.untyped_data(), down.untyped_data(),
      Is ? shared_gate.untyped_data() : nullptr, Is ? shared_up.untyped_data() : nullptr,
      Is ? shared_down.untyped_data() : nullptr, T, H, E, top_k, I, Is, route_scale, dtype, out->untyped_data(),
      expert_ids->typed_data(), weights->untyped_data(), scores->typed_data(), expert_counts->typed_data(),
      importance->typed_data(), group_sizes->typed_data(), offsets->typed_data(), source_order->typed_data(),
      inverse->typed_data(), workspace->typed_data(), workspace->element_count(), stream);
  return status_to_error(rc);
}

// SMEBU balancing update (steps/moe_balance.py:97-162).  The C entry point works in place; XLA hands
// over separate result buffers unless the caller aliases operands 1 and 2 to results 0 and 1
// (input_output_aliases), so the state is copied across first when the pointers differ.
ffi::Error MoeSmebuUpdate(hipStream_t stream, ffi::Buffer<ffi::DataType::F32> router_counts,
                          ffi::Buffer<ffi::DataType::F32> momentum, ffi::Buffer<ffi::DataType::F32> expert_bias,
                          ffi::Result<ffi::Buffer<ffi::DataType::F32>> next_momentum,
                          ffi::Result<ffi::Buffer<ffi::DataType::F32>> next_bias,
                          ffi::Result<ffi::Buffer<ffi::DataType::F32>> metrics, double load_lr, double momentum_factor,
                          double clamp) {
  const auto cd = router_counts.dimensions();
  if (cd.size() != 2) return ffi::Error::InvalidArgument("router counts must have shape [layers, experts]");
  const size_t n = router_counts.element_count();
  if (momentum.element_count() != n || expert_bias.element_count() != n || next_momentum->element_count() != n ||
      next_bias->element_count() != n)
    return ffi::Error::InvalidArgument("router count shape must match MoE balance state");
  if (metrics->element_count() != 6) return ffi::Error::InvalidArgument("metrics must have shape [6]");
  if (next_momentum->typed_data() != momentum.typed_data() &&
      hipMemcpyAsync(next_momentum->typed_data(), momentum.typed_data(), n * sizeof(float), hipMemcpyDeviceToDevice,
                     stream) != hipSuccess)
    return ffi::Error::Internal("smebu update: copy of the momentum failed");
  if (next_bias->typed_data() != expert_bias.typed_data() &&
      hipMemcpyAsync(next_bias->typed_data(), expert_bias.typed_data(), n * sizeof(float), hipMemcpyDeviceToDevice,
                     stream) != hipSuccess)
    return ffi::Error::Internal("smebu update: copy of the expert bias failed");
  return status_to_error(jtmoe_smebu_update(router_counts.typed_data(), next_momentum->typed_data(),
                                            next_bias->typed_data(), cd[0], cd[1], (float)load_lr,
                                            (float)momentum_factor, (float)clamp, metrics->typed_data(), stream));
}

}  // namespace

XLA_FFI_DEFINE_HANDLER_SYMBOL(JaxtitanMoeForward, MoeForward,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()                      // x
                                  .Arg<ffi::AnyBuffer>()                      // router kernel
                                  .Arg<ffi::Buffer<ffi::DataType::F32>>()     // expert_bias
                                  .Arg<ffi::AnyBuffer>()                      // gate
                                  .Arg<ffi::AnyBuffer>()                      // up
                                  .Arg<ffi::AnyBuffer>()                      // down
                                  .Arg<ffi::AnyBuffer>()                      // shared gate
                                  .Arg<ffi::AnyBuffer>()                      // shared up
                                  .Arg<ffi::AnyBuffer>()                      // shared down
                                  .Ret<ffi::AnyBuffer>()                      // y
                                  .Ret<ffi::Buffer<ffi::DataType::S32>>()     // expert_ids
                                  .Ret<ffi::AnyBuffer>()                      // weights
                                  .Ret<ffi::Buffer<ffi::DataType::F32>>()     // scores
                                  .Ret<ffi::Buffer<ffi::DataType::F32>>()     // expert_counts
                                  .Ret<ffi::Buffer<ffi::DataType::F32>>()     // importance
                                  .Ret<ffi::Buffer<ffi::DataType::S32>>()     // group_sizes
                                  .Ret<ffi::Buffer<ffi::DataType::S32>>()     // offsets
                                  .Ret<ffi::Buffer<ffi::DataType::S32>>()     // source_order
                                  .Ret<ffi::Buffer<ffi::DataType::S32>>()     // inverse
                                  .Ret<ffi::Buffer<ffi::DataType::U8>>()      // workspace
                                  .Attr<int64_t>("top_k")
                                  .Attr<double>("route_scale"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(JaxtitanMoeRouter, MoeRouter,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::DataType::F32>>()
                                  .Ret<ffi::Buffer<ffi::DataType::S32>>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::Buffer<ffi::DataType::F32>>()
                                  .Ret<ffi::Buffer<ffi::DataType::F32>>()
                                  .Ret<ffi::Buffer<ffi::DataType::F32>>()
                                  .Ret<ffi::Buffer<ffi::DataType::U8>>()
                                  .Attr<int64_t>("top_k")
                                  .Attr<double>("route_scale"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(JaxtitanMoeDispatch, MoeDispatch,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::DataType::S32>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::Buffer<ffi::DataType::S32>>()
                                  .Ret<ffi::Buffer<ffi::DataType::S32>>()
                                  .Ret<ffi::Buffer<ffi::DataType::S32>>()
                                  .Ret<ffi::Buffer<ffi::DataType::S32>>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::Buffer<ffi::DataType::U8>>());

XLA_FFI_DEFINE_HANDLER_SYMBOL(JaxtitanMoeGroupedSwiglu, MoeGroupedSwiglu,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::DataType::S32>>()
                                  .Arg<ffi::Buffer<ffi::DataType::S32>>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>());

XLA_FFI_DEFINE_HANDLER_SYMBOL(JaxtitanMoeCombine, MoeCombine,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::DataType::S32>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>());

#define JT_ANY .Arg<ffi::AnyBuffer>()
#define JT_F32 .Arg<ffi::Buffer<ffi::DataType::F32>>()
#define JT_S32 .Arg<ffi::Buffer<ffi::DataType::S32>>()
#define JT_RANY .Ret<ffi::AnyBuffer>()
#define JT_RF32 .Ret<ffi::Buffer<ffi::DataType::F32>>()
#define JT_RS32 .Ret<ffi::Buffer<ffi::DataType::S32>>()
#define JT_RU8 .Ret<ffi::Buffer<ffi::DataType::U8>>()

XLA_FFI_DEFINE_HANDLER_SYMBOL(JaxtitanMoeForwardTrain, MoeForwardTrain,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  JT_ANY JT_ANY JT_F32 JT_ANY JT_ANY JT_ANY JT_ANY JT_ANY JT_ANY  // as MoeForward
                                  JT_RANY JT_RS32 JT_RANY JT_RF32 JT_RF32 JT_RF32 JT_RS32 JT_RS32 JT_RS32 JT_RS32
                                  JT_RANY JT_RANY JT_RANY JT_RANY  // gate_pre, up_pre, shared_gate_pre, shared_up_pre
                                  JT_RU8
                                  .Attr<int64_t>("top_k")
                                  .Attr<double>("route_scale"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(JaxtitanMoeBackward, MoeBackward,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  JT_ANY JT_ANY JT_F32                             // x, dy, d_scores
                                  JT_ANY JT_ANY JT_ANY JT_ANY JT_ANY JT_ANY JT_ANY  // router, gate, up, down, shared x3
                                  JT_F32 JT_S32 JT_ANY                             // scores, expert_ids, weights
                                  JT_S32 JT_S32 JT_S32 JT_S32                      // source_order, inverse, sizes, offsets
                                  JT_ANY JT_ANY JT_ANY JT_ANY                      // the four residuals
                                  JT_RANY JT_RANY JT_RANY JT_RANY JT_RANY JT_RANY JT_RANY JT_RANY  // the eight gradients
                                  JT_RU8
                                  .Attr<double>("route_scale"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(JaxtitanRmsnorm, Rmsnorm,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  JT_ANY JT_F32 JT_RANY
                                  .Attr<double>("eps"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(JaxtitanFfnBlockForward, FfnBlockForward,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  JT_ANY JT_F32 JT_F32                                              // x, pre, post scale
                                  JT_ANY JT_F32 JT_ANY JT_ANY JT_ANY JT_ANY JT_ANY JT_ANY            // as MoeForward after x
                                  JT_RANY JT_RS32 JT_RANY JT_RF32 JT_RF32 JT_RF32 JT_RS32 JT_RS32 JT_RS32 JT_RS32
                                  JT_RU8
                                  .Attr<int64_t>("top_k")
                                  .Attr<double>("route_scale")
                                  .Attr<double>("eps"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(JaxtitanMoeSmebuUpdate, MoeSmebuUpdate,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  JT_F32 JT_F32 JT_F32    // router counts, momentum, expert bias
                                  JT_RF32 JT_RF32 JT_RF32  // next momentum, next bias, metrics
                                  .Attr<double>("load_lr")
                                  .Attr<double>("momentum_factor")
                                  .Attr<double>("clamp"));

#undef JT_ANY
#undef JT_F32
#undef JT_S32
#undef JT_RANY
#undef JT_RF32
#undef JT_RS32
#undef JT_RU8
