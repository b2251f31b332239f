// XLA FFI (jax.ffi) custom-call targets forwarding to the C ABI of libvmoe_hip.so.
//
// NOT BUILT in this repository's default build: it needs the XLA FFI headers
// that ship with jaxlib (`jax.ffi.include_dir()`), which are not installed
// here.  Build, where jaxlib is available, with
//   hipcc -shared -fPIC -std=c++17 -I$(python -c "import jax; print(jax.ffi.include_dir())") \
//         -Iinclude vmoe_amd/csrc/ffi/vmoe_xla_ffi.cc -Lvmoe_amd/_lib -lvmoe_hip -o libvmoe_xla_ffi.so
// and register each symbol with
//   jax.ffi.register_ffi_target("vmoe_route_assign", jax.ffi.pycapsule(lib.VmoeRouteAssign), platform="ROCM")
#if __has_include("xla/ffi/api/ffi.h")
#include <hip/hip_runtime.h>

#include "vmoe_hip.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

static ffi::Error Status(int rc, const char* what) {
  if (rc == 0) return ffi::Error::Success();
  return ffi::Error(rc < 0 ? ffi::ErrorCode::kInvalidArgument : ffi::ErrorCode::kInternal,
                    std::string(what) + ": " + vmoe_error_string(rc));
}

static int DType(ffi::DataType t) { return t == ffi::DataType::BF16 ? VMOE_BF16 : VMOE_F32; }

// gate_topk: x (G,S,D), w (D,E) -> gates (G,S,E), topk_val (G,S,K) f32, topk_idx (G,S,K) s32
static ffi::Error GateTopkImpl(hipStream_t stream, ffi::AnyBuffer x, ffi::AnyBuffer w,
                               ffi::Result<ffi::AnyBuffer> gates,
                               ffi::Result<ffi::Buffer<ffi::F32>> topk_val,
                               ffi::Result<ffi::Buffer<ffi::S32>> topk_idx) {
  auto xd = x.dimensions();
  VmoeGateTopkParams p{};
  p.x = x.untyped_data();
  p.w = w.untyped_data();
  p.gates = gates->untyped_data();
  p.topk_val = topk_val->typed_data();
  p.topk_idx = topk_idx->typed_data();
  p.num_items = (int32_t)(xd[0] * xd[1]);
  p.D = (int32_t)xd[2];
  p.E = (int32_t)w.dimensions()[1];
  p.K = (int32_t)topk_idx->dimensions()[2];
  p.dtype = DType(x.element_type());
  return Status(vmoe_gate_topk(&p, stream), "vmoe_gate_topk");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeGateTopk, GateTopkImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::S32>>());

// route_assign: topk_val, topk_idx -> indices (G,S,K,2), token_slot (G,S,K), slot_token (E*G*C), fill (G,E)
static ffi::Error RouteAssignImpl(hipStream_t stream, ffi::Buffer<ffi::F32> topk_val,
                                  ffi::Buffer<ffi::S32> topk_idx,
                                  ffi::Result<ffi::Buffer<ffi::S32>> indices,
                                  ffi::Result<ffi::Buffer<ffi::S32>> token_slot,
                                  ffi::Result<ffi::Buffer<ffi::S32>> slot_token,
                                  ffi::Result<ffi::Buffer<ffi::S32>> fill, int32_t num_experts,
                                  int32_t capacity, bool batch_priority) {
  auto d = topk_idx.dimensions();
  VmoeRouteAssignParams p{};
  p.topk_val = topk_val.typed_data();
  p.topk_idx = topk_idx.typed_data();
  p.indices = indices->typed_data();
  p.token_slot = token_slot->typed_data();
  p.slot_token = slot_token->typed_data();
  p.fill = fill->typed_data();
  p.G = (int32_t)d[0]; p.S = (int32_t)d[1]; p.K = (int32_t)d[2];
  p.E = num_experts; p.C = capacity; p.batch_priority = batch_priority;
  return Status(vmoe_route_assign(&p, stream), "vmoe_route_assign");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeRouteAssign, RouteAssignImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::S32>>()
                                  .Attr<int32_t>("num_experts")
                                  .Attr<int32_t>("capacity")
                                  .Attr<bool>("batch_priority"));

// dispatch / combine
static ffi::Error DispatchImpl(hipStream_t stream, ffi::AnyBuffer x, ffi::Buffer<ffi::S32> token_slot,
                               ffi::Buffer<ffi::S32> slot_token, ffi::Result<ffi::AnyBuffer> out) {
  auto xd = x.dimensions();
  VmoeDispatchParams p{};
  p.x = x.untyped_data();
  p.token_slot = token_slot.typed_data();
  p.slot_token = slot_token.typed_data();
  p.out = out->untyped_data();
  p.num_items = (int32_t)(xd[0] * xd[1]);
  p.num_slots = (int32_t)slot_token.element_count();
  p.K = (int32_t)token_slot.dimensions()[2];
  p.D = (int32_t)xd[2];
  p.dtype = DType(x.element_type());
  return Status(vmoe_dispatch(&p, stream), "vmoe_dispatch");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeDispatch, DispatchImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::AnyBuffer>());

static ffi::Error CombineImpl(hipStream_t stream, ffi::AnyBuffer y, ffi::Buffer<ffi::S32> token_slot,
                              ffi::Buffer<ffi::F32> weights, ffi::Result<ffi::AnyBuffer> out) {
  auto td = token_slot.dimensions();
  VmoeCombineParams p{};
  p.y = y.untyped_data();
  p.token_slot = token_slot.typed_data();
  p.weights = weights.typed_data();
  p.out = out->untyped_data();
  p.num_items = (int32_t)(td[0] * td[1]);
  p.K = (int32_t)td[2];
  p.D = (int32_t)y.dimensions().back();
  p.num_slots = (int32_t)(y.element_count() / p.D);
  p.dtype = DType(y.element_type());
  return Status(vmoe_combine(&p, stream), "vmoe_combine");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeCombine, CombineImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::AnyBuffer>());

// expert_mlp: x (E,R,D), w0t (E,M,D), b0 (E,M), w1t (E,D,M), b1 (E,D), workspace -> out (E,R,D)
static ffi::Error ExpertMlpImpl(hipStream_t stream, ffi::AnyBuffer x, ffi::AnyBuffer w0t,
                                ffi::AnyBuffer b0, ffi::AnyBuffer w1t, ffi::AnyBuffer b1,
                                ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> workspace) {
  auto xd = x.dimensions();
  VmoeExpertMlpParams p{};
  p.x = x.untyped_data();
  p.w0t = w0t.untyped_data(); p.b0 = b0.untyped_data();
  p.w1t = w1t.untyped_data(); p.b1 = b1.untyped_data();
  p.out = out->untyped_data();
  p.workspace = workspace->untyped_data();
  p.workspace_bytes = workspace->size_bytes();
  p.E = (int32_t)xd[0]; p.R = (int32_t)xd[1]; p.D = (int32_t)xd[2];
  p.M = (int32_t)w0t.dimensions()[1];
  p.dtype = DType(x.element_type());
  p.gelu = VMOE_GELU_TANH;
  return Status(vmoe_expert_mlp(&p, stream), "vmoe_expert_mlp");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeExpertMlp, ExpertMlpImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>());
#endif  // __has_include("xla/ffi/api/ffi.h")
