// XLA FFI (jax.ffi) custom-call targets forwarding to the C ABI of libvmoe_hip.so: one
// handler per entry point of include/vmoe_hip.h that takes a parameter block (the three
// measurement aids vmoe_copy_bytes, vmoe_mfma_probe and vmoe_operand_delivery_probe have
// none).  Handler symbol = the entry point's name in CamelCase (vmoe_gate_topk ->
// VmoeGateTopk); register it under the entry point's name:
//   jax.ffi.register_ffi_target("vmoe_gate_topk", jax.ffi.pycapsule(lib.VmoeGateTopk), platform="ROCM")
//
// NOT BUILT, NOT RUN in this repository: it needs the XLA FFI headers that ship with
// jaxlib (`jax.ffi.include_dir()`), which are not installed here; the file compiles to
// nothing without them.  Build, where jaxlib is available, with
//   hipcc -shared -fPIC -std=c++17 -I$(python -c "import jax; print(jax.ffi.include_dir())") \
//         -Iinclude vmoe_amd/csrc/ffi/vmoe_xla_ffi.cc -Lvmoe_amd/_lib -lvmoe_hip -o libvmoe_xla_ffi.so
//
// Conventions.  Shapes come from the buffers, scalars are attributes.  XLA has no optional
// operands: an optional pointer of the C ABI is an ordinary operand plus a bool attribute
// (has_...) that says whether it is used (pass any one-element array when it is not).
// Workspaces and scratch arrays are extra results, so XLA owns them.  Results that the C
// ABI wants zeroed are cleared here with hipMemsetAsync on the call's stream (the handlers
// are not marked command-buffer compatible, so XLA does not capture them into graphs).
#if __has_include("xla/ffi/api/ffi.h")
#include <hip/hip_runtime.h>

#include <string>

#include "vmoe_hip.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

using Any = ffi::AnyBuffer;
using AnyOut = ffi::Result<ffi::AnyBuffer>;
using F32 = ffi::Buffer<ffi::F32>;
using S32 = ffi::Buffer<ffi::S32>;
using F32Out = ffi::Result<ffi::Buffer<ffi::F32>>;
using S32Out = ffi::Result<ffi::Buffer<ffi::S32>>;
using Stream = ffi::PlatformStream<hipStream_t>;

static ffi::Error Status(int rc, const char* what) {
  if (rc == 0) return ffi::Error::Success();
  return ffi::Error(rc < 0 ? ffi::ErrorCode::kInvalidArgument : ffi::ErrorCode::kInternal,
                    std::string(what) + ": " + vmoe_error_string(rc));
}
static ffi::Error Cleared(hipStream_t stream, void* p, size_t bytes) {
  hipError_t e = hipMemsetAsync(p, 0, bytes, stream);
  return e == hipSuccess ? ffi::Error::Success()
                         : ffi::Error(ffi::ErrorCode::kInternal, hipGetErrorString(e));
}
static int DType(ffi::DataType t) { return t == ffi::DataType::BF16 ? VMOE_BF16 : VMOE_F32; }
static int WDType(ffi::DataType t) {
  return t == ffi::DataType::PRED ? VMOE_W_BOOL : t == ffi::DataType::BF16 ? VMOE_W_BF16 : VMOE_W_F32;
}
template <typename B> static int32_t Dim(const B& b, size_t i) { return (int32_t)b.dimensions()[i]; }

// ---------------------------------------------------------------- gating
// x (G,S,D), w (D,E), logit_bias (E,) f32 -> gates (G,S,E), topk_val (G,S,K) f32,
// topk_idx (G,S,K) s32, logits (G,S,E) f32.  has_logit_bias / want_gates / want_logits.
static ffi::Error GateTopkImpl(hipStream_t stream, Any x, Any w, F32 logit_bias, AnyOut gates,
                               F32Out topk_val, S32Out topk_idx, F32Out logits, bool has_logit_bias,
                               bool want_gates, bool want_logits) {
  VmoeGateTopkParams p{};
  p.x = x.untyped_data();
  p.w = w.untyped_data();
  p.logit_bias = has_logit_bias ? logit_bias.typed_data() : nullptr;
  p.gates = want_gates ? gates->untyped_data() : nullptr;
  p.topk_val = topk_val->typed_data();
  p.topk_idx = topk_idx->typed_data();
  p.logits = want_logits ? logits->typed_data() : nullptr;
  p.num_items = Dim(x, 0) * Dim(x, 1);
  p.D = Dim(x, 2);
  p.E = Dim(w, 1);
  p.K = (int32_t)topk_idx->dimensions()[2];
  p.dtype = DType(x.element_type());
  return Status(vmoe_gate_topk(&p, stream), "vmoe_gate_topk");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeGateTopk, GateTopkImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Arg<Any>().Arg<F32>()
                                  .Ret<Any>().Ret<F32>().Ret<S32>().Ret<F32>()
                                  .Attr<bool>("has_logit_bias").Attr<bool>("want_gates")
                                  .Attr<bool>("want_logits"));

// logits, noise (G,S,E) f32 -> gates_noisy (G,S,E) f32, load_loss (G,) f32
static ffi::Error NoisyGatesImpl(hipStream_t stream, F32 logits, F32 noise, F32Out gates_noisy,
                                 F32Out load_loss, int32_t num_selected_experts, float noise_std) {
  VmoeNoisyGatesParams p{};
  p.logits = logits.typed_data();
  p.noise = noise.typed_data();
  p.gates_noisy = gates_noisy->typed_data();
  p.load_loss = load_loss->typed_data();
  p.G = Dim(logits, 0); p.S = Dim(logits, 1); p.E = Dim(logits, 2);
  p.K = num_selected_experts;
  p.noise_std = noise_std;
  return Status(vmoe_noisy_gates(&p, stream), "vmoe_noisy_gates");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeNoisyGates, NoisyGatesImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<F32>().Arg<F32>().Ret<F32>().Ret<F32>()
                                  .Attr<int32_t>("num_selected_experts").Attr<float>("noise_std"));

// gates (..., E) f32 -> topk_val, topk_idx (..., K)
static ffi::Error TopkImpl(hipStream_t stream, F32 gates, F32Out topk_val, S32Out topk_idx) {
  VmoeTopkParams p{};
  p.gates = gates.typed_data();
  p.topk_val = topk_val->typed_data();
  p.topk_idx = topk_idx->typed_data();
  p.E = (int32_t)gates.dimensions().back();
  p.K = (int32_t)topk_idx->dimensions().back();
  p.num_items = (int32_t)(gates.element_count() / p.E);
  return Status(vmoe_topk(&p, stream), "vmoe_topk");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeTopk, TopkImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<F32>().Ret<F32>().Ret<S32>());

// ---------------------------------------------------------------- router losses
static void FillMetrics(VmoeRouterMetricsParams* m, const Any& gates, const S32& topk_idx,
                        F32Out& importance, F32Out& gshard, F32Out& auxiliary, float gshard_weight,
                        float importance_weight) {
  m->gates = gates.untyped_data();
  m->top1_idx = topk_idx.typed_data();
  m->importance_loss = importance->typed_data();
  m->gshard_loss = gshard->typed_data();
  m->auxiliary_loss = auxiliary->typed_data();
  m->gshard_loss_weight = gshard_weight;
  m->importance_loss_weight = importance_weight;
  m->G = Dim(gates, 0); m->S = Dim(gates, 1); m->E = Dim(gates, 2);
  m->top1_stride = (int32_t)topk_idx.dimensions().back();
  m->dtype = DType(gates.element_type());
}
// gates (G,S,E), topk_idx (G,S,K) -> importance_loss, gshard_loss, auxiliary_loss (G,) f32
static ffi::Error RouterMetricsImpl(hipStream_t stream, Any gates, S32 topk_idx, F32Out importance,
                                    F32Out gshard, F32Out auxiliary, float gshard_loss_weight,
                                    float importance_loss_weight) {
  VmoeRouterMetricsParams m{};
  FillMetrics(&m, gates, topk_idx, importance, gshard, auxiliary, gshard_loss_weight,
              importance_loss_weight);
  return Status(vmoe_router_metrics(&m, stream), "vmoe_router_metrics");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeRouterMetrics, RouterMetricsImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Arg<S32>().Ret<F32>().Ret<F32>()
                                  .Ret<F32>().Attr<float>("gshard_loss_weight")
                                  .Attr<float>("importance_loss_weight"));

// ---------------------------------------------------------------- slot assignment
static void FillRoute(VmoeRouteAssignParams* p, const F32& topk_val, const S32& topk_idx,
                      S32Out& indices, S32Out& token_slot, S32Out& slot_token, S32Out& fill,
                      int32_t num_experts, int32_t capacity, bool batch_priority) {
  p->topk_val = topk_val.typed_data();
  p->topk_idx = topk_idx.typed_data();
  p->indices = indices->typed_data();
  p->token_slot = token_slot->typed_data();
  p->slot_token = slot_token->typed_data();
  p->fill = fill->typed_data();
  p->G = Dim(topk_idx, 0); p->S = Dim(topk_idx, 1); p->K = Dim(topk_idx, 2);
  p->E = num_experts; p->C = capacity; p->batch_priority = batch_priority;
}
// topk_val, topk_idx (G,S,K) -> indices (G,S,K,2), token_slot (G,S,K), slot_token (E*G*C,), fill (G,E)
static ffi::Error RouteAssignImpl(hipStream_t stream, F32 topk_val, S32 topk_idx, S32Out indices,
                                  S32Out token_slot, S32Out slot_token, S32Out fill,
                                  int32_t num_experts, int32_t capacity, bool batch_priority) {
  VmoeRouteAssignParams p{};
  FillRoute(&p, topk_val, topk_idx, indices, token_slot, slot_token, fill, num_experts, capacity,
            batch_priority);
  return Status(vmoe_route_assign(&p, stream), "vmoe_route_assign");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeRouteAssign, RouteAssignImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<F32>().Arg<S32>().Ret<S32>().Ret<S32>()
                                  .Ret<S32>().Ret<S32>().Attr<int32_t>("num_experts")
                                  .Attr<int32_t>("capacity").Attr<bool>("batch_priority"));

// The deterministic branch of NoisyTopExpertsPerItemRouter after vmoe_gate_topk: slot
// assignment and the three losses in one launch.
static ffi::Error RouteAssignMetricsImpl(hipStream_t stream, Any gates, F32 topk_val, S32 topk_idx,
                                         S32Out indices, S32Out token_slot, S32Out slot_token,
                                         S32Out fill, F32Out importance, F32Out gshard,
                                         F32Out auxiliary, int32_t num_experts, int32_t capacity,
                                         bool batch_priority, float gshard_loss_weight,
                                         float importance_loss_weight) {
  VmoeRouteAssignParams p{};
  FillRoute(&p, topk_val, topk_idx, indices, token_slot, slot_token, fill, num_experts, capacity,
            batch_priority);
  VmoeRouterMetricsParams m{};
  FillMetrics(&m, gates, topk_idx, importance, gshard, auxiliary, gshard_loss_weight,
              importance_loss_weight);
  return Status(vmoe_route_assign_metrics(&p, &m, stream), "vmoe_route_assign_metrics");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeRouteAssignMetrics, RouteAssignMetricsImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Arg<F32>().Arg<S32>().Ret<S32>()
                                  .Ret<S32>().Ret<S32>().Ret<S32>().Ret<F32>().Ret<F32>().Ret<F32>()
                                  .Attr<int32_t>("num_experts").Attr<int32_t>("capacity")
                                  .Attr<bool>("batch_priority").Attr<float>("gshard_loss_weight")
                                  .Attr<float>("importance_loss_weight"));

// gates (G,S,E) -> indices (G,S,E,2), token_slot (G,S,E), slot_token (E*G*C,), weights (G,S,E) f32,
// sel_minmax (G,E,2) f32
static ffi::Error TopItemsPerExpertImpl(hipStream_t stream, Any gates, S32Out indices,
                                        S32Out token_slot, S32Out slot_token, F32Out weights,
                                        F32Out sel_minmax, int32_t capacity) {
  VmoeTopItemsParams p{};
  p.gates = gates.untyped_data();
  p.indices = indices->typed_data();
  p.token_slot = token_slot->typed_data();
  p.slot_token = slot_token->typed_data();
  p.weights = weights->typed_data();
  p.sel_minmax = sel_minmax->typed_data();
  p.G = Dim(gates, 0); p.S = Dim(gates, 1); p.E = Dim(gates, 2);
  p.C = capacity;
  p.dtype = DType(gates.element_type());
  return Status(vmoe_top_items_per_expert(&p, stream), "vmoe_top_items_per_expert");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeTopItemsPerExpert, TopItemsPerExpertImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Ret<S32>().Ret<S32>().Ret<S32>()
                                  .Ret<F32>().Ret<F32>().Attr<int32_t>("capacity"));

// indices (G,S,K,2) -> token_slot (G,S,K), slot_token (E*G*C,), num_duplicates (1,), num_invalid (1,)
static ffi::Error IndicesToSlotsImpl(hipStream_t stream, S32 indices, S32Out token_slot,
                                     S32Out slot_token, S32Out num_duplicates, S32Out num_invalid,
                                     int32_t num_experts, int32_t capacity) {
  ffi::Error e = Cleared(stream, num_duplicates->typed_data(), sizeof(int32_t));
  if (e.failure()) return e;
  e = Cleared(stream, num_invalid->typed_data(), sizeof(int32_t));
  if (e.failure()) return e;
  VmoeIndicesToSlotsParams p{};
  p.indices = indices.typed_data();
  p.token_slot = token_slot->typed_data();
  p.slot_token = slot_token->typed_data();
  p.num_duplicates = num_duplicates->typed_data();
  p.num_invalid = num_invalid->typed_data();
  p.G = Dim(indices, 0); p.S = Dim(indices, 1); p.K = Dim(indices, 2);
  p.E = num_experts; p.C = capacity;
  return Status(vmoe_indices_to_slots(&p, stream), "vmoe_indices_to_slots");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeIndicesToSlots, IndicesToSlotsImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<S32>().Ret<S32>().Ret<S32>().Ret<S32>()
                                  .Ret<S32>().Attr<int32_t>("num_experts").Attr<int32_t>("capacity"));

// fill (G,E), token_slot (G,S,K) -> token_row (G,S,K), rows_per_expert (E,), row_token (E,G*C),
// prefix (G,E) scratch
static void FillCompact(VmoeCompactRowsParams* p, const S32& fill, const S32& token_slot,
                        S32Out& token_row, S32Out& rows_per_expert, S32Out& row_token,
                        int32_t capacity) {
  p->fill = fill.typed_data();
  p->token_slot = token_slot.typed_data();
  p->token_row = token_row->typed_data();
  p->rows_per_expert = rows_per_expert->typed_data();
  p->row_token = row_token->typed_data();
  p->G = Dim(fill, 0); p->E = Dim(fill, 1);
  p->S = Dim(token_slot, 1); p->K = Dim(token_slot, 2);
  p->C = capacity;
}
static ffi::Error CompactRowsImpl(hipStream_t stream, S32 fill, S32 token_slot, S32Out token_row,
                                  S32Out rows_per_expert, S32Out row_token, S32Out prefix,
                                  int32_t capacity) {
  VmoeCompactRowsParams p{};
  FillCompact(&p, fill, token_slot, token_row, rows_per_expert, row_token, capacity);
  p.prefix = prefix->typed_data();
  return Status(vmoe_compact_rows(&p, stream), "vmoe_compact_rows");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeCompactRows, CompactRowsImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<S32>().Arg<S32>().Ret<S32>().Ret<S32>()
                                  .Ret<S32>().Ret<S32>().Attr<int32_t>("capacity"));
// The same without the scratch result (it lives in a static device array of the library).
static ffi::Error CompactRowsStaticImpl(hipStream_t stream, S32 fill, S32 token_slot,
                                        S32Out token_row, S32Out rows_per_expert, S32Out row_token,
                                        int32_t capacity) {
  VmoeCompactRowsParams p{};
  FillCompact(&p, fill, token_slot, token_row, rows_per_expert, row_token, capacity);
  return Status(vmoe_compact_rows_static(&p, stream), "vmoe_compact_rows_static");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeCompactRowsStatic, CompactRowsStaticImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<S32>().Arg<S32>().Ret<S32>().Ret<S32>()
                                  .Ret<S32>().Attr<int32_t>("capacity"));

// ---------------------------------------------------------------- dispatch / combine
// x (G,S,D), token_slot (G,S,K) [slot rows, or packed rows with zero_fill false],
// slot_token (E*G*C,) -> out (E, G*C, D).  zero_fill false leaves unclaimed rows untouched.
static ffi::Error DispatchImpl(hipStream_t stream, Any x, S32 token_slot, S32 slot_token, AnyOut out,
                               bool zero_fill) {
  VmoeDispatchParams p{};
  p.x = x.untyped_data();
  p.token_slot = token_slot.typed_data();
  p.slot_token = zero_fill ? slot_token.typed_data() : nullptr;
  p.out = out->untyped_data();
  p.D = (int32_t)x.dimensions().back();
  p.num_items = (int32_t)(x.element_count() / p.D);
  p.num_slots = (int32_t)(out->element_count() / p.D);
  p.K = (int32_t)token_slot.dimensions().back();
  p.dtype = DType(x.element_type());
  return Status(vmoe_dispatch(&p, stream), "vmoe_dispatch");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeDispatch, DispatchImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Arg<S32>().Arg<S32>().Ret<Any>()
                                  .Attr<bool>("zero_fill"));

// y (E, G*C, D), token_slot (G,S,K), weights (G,S,K) f32 -> out (G,S,D)
static ffi::Error CombineImpl(hipStream_t stream, Any y, S32 token_slot, F32 weights, AnyOut out) {
  VmoeCombineParams p{};
  p.y = y.untyped_data();
  p.token_slot = token_slot.typed_data();
  p.weights = weights.typed_data();
  p.out = out->untyped_data();
  p.K = (int32_t)token_slot.dimensions().back();
  p.num_items = (int32_t)(token_slot.element_count() / p.K);
  p.D = (int32_t)y.dimensions().back();
  p.num_slots = (int32_t)(y.element_count() / p.D);
  p.dtype = DType(y.element_type());
  return Status(vmoe_combine(&p, stream), "vmoe_combine");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeCombine, CombineImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Arg<S32>().Arg<F32>().Ret<Any>());

// dout (G,S,D), token_slot, weights (G,S,K), slot_token (E*G*C,) -> dy (E, G*C, D)
static ffi::Error CombineBackwardDataImpl(hipStream_t stream, Any dout, S32 token_slot, F32 weights,
                                          S32 slot_token, AnyOut dy, bool zero_fill) {
  VmoeCombineBackwardParams p{};
  p.dout = dout.untyped_data();
  p.token_slot = token_slot.typed_data();
  p.weights = weights.typed_data();
  p.slot_token = zero_fill ? slot_token.typed_data() : nullptr;
  p.dy = dy->untyped_data();
  p.K = (int32_t)token_slot.dimensions().back();
  p.num_items = (int32_t)(token_slot.element_count() / p.K);
  p.D = (int32_t)dout.dimensions().back();
  p.num_slots = (int32_t)(dy->element_count() / p.D);
  p.dtype = DType(dout.element_type());
  return Status(vmoe_combine_backward_data(&p, stream), "vmoe_combine_backward_data");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeCombineBackwardData, CombineBackwardDataImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Arg<S32>().Arg<F32>().Arg<S32>()
                                  .Ret<Any>().Attr<bool>("zero_fill"));

// dout (G,S,D), y (E, G*C, D), token_slot (G,S,K) -> dweights (G,S,K) f32
static ffi::Error CombineBackwardWeightsImpl(hipStream_t stream, Any dout, Any y, S32 token_slot,
                                             F32Out dweights) {
  VmoeCombineBackwardParams p{};
  p.dout = dout.untyped_data();
  p.y = y.untyped_data();
  p.token_slot = token_slot.typed_data();
  p.dweights = dweights->typed_data();
  p.K = (int32_t)token_slot.dimensions().back();
  p.num_items = (int32_t)(token_slot.element_count() / p.K);
  p.D = (int32_t)dout.dimensions().back();
  p.num_slots = (int32_t)(y.element_count() / p.D);
  p.dtype = DType(dout.element_type());
  return Status(vmoe_combine_backward_weights(&p, stream), "vmoe_combine_backward_weights");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeCombineBackwardWeights, CombineBackwardWeightsImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Arg<Any>().Arg<S32>().Ret<F32>());

// indices (G,S,K,2), weights (G,S,K) -> combine (G,S,E,C) f32, dispatch (G,S,E,C) bool
static ffi::Error DensifyImpl(hipStream_t stream, S32 indices, F32 weights, F32Out combine,
                              ffi::Result<ffi::Buffer<ffi::PRED>> dispatch) {
  ffi::Error e = Cleared(stream, combine->typed_data(), combine->size_bytes());
  if (e.failure()) return e;
  e = Cleared(stream, dispatch->typed_data(), dispatch->size_bytes());
  if (e.failure()) return e;
  VmoeDensifyParams p{};
  p.indices = indices.typed_data();
  p.weights = weights.typed_data();
  p.combine = combine->typed_data();
  p.dispatch = reinterpret_cast<uint8_t*>(dispatch->typed_data());
  p.G = Dim(indices, 0); p.S = Dim(indices, 1); p.K = Dim(indices, 2);
  p.E = (int32_t)combine->dimensions()[2];
  p.C = (int32_t)combine->dimensions()[3];
  return Status(vmoe_densify(&p, stream), "vmoe_densify");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeDensify, DensifyImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<S32>().Arg<F32>().Ret<F32>()
                                  .Ret<ffi::Buffer<ffi::PRED>>());

// ---------------------------------------------------------------- expert MLP
// Copies the status words of the MLP call just issued (vmoe_expert_mlp_status: abandoned
// waits, plan mismatches) from its workspace into the call's `status` result, behind the
// kernels on the stream: XLA hands out a fresh workspace per call, so the words must leave
// with the call.  Zeros where the call keeps none (float32).
static ffi::Error CopyStatus(hipStream_t stream, const VmoeExpertMlpParams& p, S32Out& status) {
  const int32_t* words = nullptr;
  ffi::Error e = Status(vmoe_expert_mlp_status(&p, &words), "vmoe_expert_mlp_status");
  if (e.failure()) return e;
  const size_t bytes = VMOE_MLP_STATUS_WORDS * sizeof(int32_t);
  hipError_t h = words != nullptr
                     ? hipMemcpyAsync(status->typed_data(), words, bytes, hipMemcpyDeviceToDevice, stream)
                     : hipMemsetAsync(status->typed_data(), 0, bytes, stream);
  return h == hipSuccess ? ffi::Error::Success()
                         : ffi::Error(ffi::ErrorCode::kInternal, hipGetErrorString(h));
}

// x (E,R,D) -- or, with gather, the items (T,D) --, w0, b0 (E,M), w1, b1 (E,D),
// rows_per_expert (E,), x_rows (E,R) -> out (E,R,D), workspace (bytes; size it with
// vmoe_expert_mlp_workspace_bytes through ctypes when building the call), status (2,) s32.  packed: w0 / w1
// are the transposed copies made by vmoe_pack_expert_weights, (E,M,D) / (E,D,M); else the
// reference's (E,D,M) / (E,M,D) kernels (bfloat16: repacked into the workspace every call).
static ffi::Error ExpertMlpImpl(hipStream_t stream, Any x, Any w0, Any b0, Any w1, Any b1,
                                S32 rows_per_expert, S32 x_rows, AnyOut out, AnyOut workspace,
                                S32Out status, bool packed, bool has_bias, bool ragged, bool gather,
                                int32_t gelu) {
  VmoeExpertMlpParams p{};
  p.x = x.untyped_data();
  if (packed) {
    p.w0t = w0.untyped_data();
    p.w1t = w1.untyped_data();
  } else {
    p.w0 = w0.untyped_data();
    p.w1 = w1.untyped_data();
  }
  p.b0 = has_bias ? b0.untyped_data() : nullptr;
  p.b1 = has_bias ? b1.untyped_data() : nullptr;
  p.out = out->untyped_data();
  p.workspace = workspace->untyped_data();
  p.workspace_bytes = workspace->size_bytes();
  p.E = (int32_t)out->dimensions()[0];
  p.R = (int32_t)out->dimensions()[1];
  p.D = (int32_t)out->dimensions()[2];
  p.M = packed ? Dim(w0, 1) : Dim(w0, 2);
  p.dtype = DType(x.element_type());
  p.gelu = gelu;
  p.rows_per_expert = (ragged || gather) ? rows_per_expert.typed_data() : nullptr;
  p.x_rows = gather ? x_rows.typed_data() : nullptr;
  p.num_items = gather ? (int32_t)(x.element_count() / p.D) : 0;
  ffi::Error e = Status(vmoe_expert_mlp(&p, stream), "vmoe_expert_mlp");
  if (e.failure()) return e;
  return CopyStatus(stream, p, status);
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeExpertMlp, ExpertMlpImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Arg<Any>().Arg<Any>().Arg<Any>()
                                  .Arg<Any>().Arg<S32>().Arg<S32>().Ret<Any>().Ret<Any>().Ret<S32>()
                                  .Attr<bool>("packed").Attr<bool>("has_bias").Attr<bool>("ragged")
                                  .Attr<bool>("gather").Attr<int32_t>("gelu"));

// The MLP with its launch plans already in `workspace` (written by vmoe_compact_rows_planned
// for the same shapes): bind `workspace` as a result that aliases the operand holding them
// (input_output_aliases).  Operands and attributes as VmoeExpertMlp with ragged = gather = true.
static ffi::Error ExpertMlpPlannedImpl(hipStream_t stream, Any x, Any w0, Any b0, Any w1, Any b1,
                                       S32 rows_per_expert, S32 x_rows, AnyOut out, AnyOut workspace,
                                       S32Out status, bool packed, bool has_bias, int32_t gelu) {
  VmoeExpertMlpParams p{};
  p.x = x.untyped_data();
  if (packed) {
    p.w0t = w0.untyped_data();
    p.w1t = w1.untyped_data();
  } else {
    p.w0 = w0.untyped_data();
    p.w1 = w1.untyped_data();
  }
  p.b0 = has_bias ? b0.untyped_data() : nullptr;
  p.b1 = has_bias ? b1.untyped_data() : nullptr;
  p.out = out->untyped_data();
  p.workspace = workspace->untyped_data();
  p.workspace_bytes = workspace->size_bytes();
  p.E = (int32_t)out->dimensions()[0];
  p.R = (int32_t)out->dimensions()[1];
  p.D = (int32_t)out->dimensions()[2];
  p.M = packed ? Dim(w0, 1) : Dim(w0, 2);
  p.dtype = DType(x.element_type());
  p.gelu = gelu;
  p.rows_per_expert = rows_per_expert.typed_data();
  p.x_rows = x_rows.typed_data();
  p.num_items = (int32_t)(x.element_count() / p.D);
  ffi::Error e = Status(vmoe_expert_mlp_planned(&p, stream), "vmoe_expert_mlp_planned");
  if (e.failure()) return e;
  return CopyStatus(stream, p, status);
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeExpertMlpPlanned, ExpertMlpPlannedImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Arg<Any>().Arg<Any>().Arg<Any>()
                                  .Arg<Any>().Arg<S32>().Arg<S32>().Ret<Any>().Ret<Any>().Ret<S32>()
                                  .Attr<bool>("packed").Attr<bool>("has_bias").Attr<int32_t>("gelu"));

// Row compaction, launch plans and the MLP of the gathered rows as one custom call (the form
// in which XLA would use the pair vmoe_compact_rows_planned / vmoe_expert_mlp_planned):
// fill (G,E), token_slot (G,S,K), items (T,D), weights as VmoeExpertMlp -> token_row (G,S,K),
// rows_per_expert (E,), row_token (E, G*C), out (E, G*C, D), workspace, status (2,) s32,
// prefix (G,E) s32 scratch.  Shapes for which the one-launch form does not exist (more than
// 256 experts, fewer than 256 assignments per group, very many groups of few experts,
// float32: vmoe_compact_rows_planned returns VMOE_E_UNSUPPORTED) take vmoe_compact_rows with
// the `prefix` scratch followed by vmoe_expert_mlp, as the Python host does: same results.
static ffi::Error CompactRowsPlannedImpl(hipStream_t stream, S32 fill, S32 token_slot, Any x, Any w0,
                                         Any b0, Any w1, Any b1, S32Out token_row,
                                         S32Out rows_per_expert, S32Out row_token, AnyOut out,
                                         AnyOut workspace, S32Out status, S32Out prefix,
                                         int32_t capacity, bool packed, bool has_bias, int32_t gelu) {
  VmoeCompactRowsParams c{};
  FillCompact(&c, fill, token_slot, token_row, rows_per_expert, row_token, capacity);
  VmoeExpertMlpParams p{};
  p.x = x.untyped_data();
  if (packed) {
    p.w0t = w0.untyped_data();
    p.w1t = w1.untyped_data();
  } else {
    p.w0 = w0.untyped_data();
    p.w1 = w1.untyped_data();
  }
  p.b0 = has_bias ? b0.untyped_data() : nullptr;
  p.b1 = has_bias ? b1.untyped_data() : nullptr;
  p.out = out->untyped_data();
  p.workspace = workspace->untyped_data();
  p.workspace_bytes = workspace->size_bytes();
  p.E = (int32_t)out->dimensions()[0];
  p.R = (int32_t)out->dimensions()[1];
  p.D = (int32_t)out->dimensions()[2];
  p.M = packed ? Dim(w0, 1) : Dim(w0, 2);
  p.dtype = DType(x.element_type());
  p.gelu = gelu;
  p.rows_per_expert = rows_per_expert->typed_data();
  p.x_rows = row_token->typed_data();
  p.num_items = (int32_t)(x.element_count() / p.D);
  const int rc = vmoe_compact_rows_planned(&c, &p, stream);
  ffi::Error e = ffi::Error::Success();
  if (rc == VMOE_E_UNSUPPORTED) {
    c.prefix = prefix->typed_data();
    e = Status(vmoe_compact_rows(&c, stream), "vmoe_compact_rows");
    if (e.failure()) return e;
    if (p.dtype != VMOE_BF16 || p.D % 32 != 0) {
      // (only the bfloat16 first product gathers its rows: other callers dispatch first and
      // use VmoeExpertMlp; this custom call is defined for the gathering form)
      return ffi::Error(ffi::ErrorCode::kInvalidArgument,
                        "vmoe_compact_rows_planned: the gathering expert MLP needs bfloat16 and D % 32 == 0");
    }
    e = Status(vmoe_expert_mlp(&p, stream), "vmoe_expert_mlp");
  } else {
    e = Status(rc, "vmoe_compact_rows_planned");
    if (e.failure()) return e;
    e = Status(vmoe_expert_mlp_planned(&p, stream), "vmoe_expert_mlp_planned");
  }
  if (e.failure()) return e;
  return CopyStatus(stream, p, status);
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeCompactRowsPlanned, CompactRowsPlannedImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<S32>().Arg<S32>().Arg<Any>().Arg<Any>()
                                  .Arg<Any>().Arg<Any>().Arg<Any>().Ret<S32>().Ret<S32>().Ret<S32>()
                                  .Ret<Any>().Ret<Any>().Ret<S32>().Ret<S32>().Attr<int32_t>("capacity").Attr<bool>("packed")
                                  .Attr<bool>("has_bias").Attr<int32_t>("gelu"));

// in (batch, rows, cols) -> out (batch, cols, rows)
static ffi::Error PackExpertWeightsImpl(hipStream_t stream, Any in, AnyOut out) {
  VmoeTransposeParams p{};
  p.in = in.untyped_data();
  p.out = out->untyped_data();
  p.batch = Dim(in, 0); p.rows = Dim(in, 1); p.cols = Dim(in, 2);
  p.dtype = DType(in.element_type());
  return Status(vmoe_pack_expert_weights(&p, stream), "vmoe_pack_expert_weights");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoePackExpertWeights, PackExpertWeightsImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Ret<Any>());

// ---------------------------------------------------------------- Soft MoE
// x (G,S,D), mu (D,N) -> dispatch_w, combine_w, logits (G,S,N), workspace (vmoe_soft_route_workspace_bytes)
static ffi::Error SoftRouteImpl(hipStream_t stream, Any x, Any mu, AnyOut dispatch_w, AnyOut combine_w,
                                AnyOut logits, AnyOut workspace, float scale, bool want_logits) {
  VmoeSoftRouteParams p{};
  p.x = x.untyped_data();
  p.mu = mu.untyped_data();
  p.scale = scale;
  p.dispatch_w = dispatch_w->untyped_data();
  p.combine_w = combine_w->untyped_data();
  p.logits = want_logits ? logits->untyped_data() : nullptr;
  p.workspace = workspace->untyped_data();
  p.workspace_bytes = workspace->size_bytes();
  p.G = Dim(x, 0); p.S = Dim(x, 1); p.D = Dim(x, 2);
  p.N = Dim(mu, 1);
  p.dtype = DType(x.element_type());
  p.workspace_prepared = 0;     // XLA hands out a fresh workspace per call
  return Status(vmoe_soft_route(&p, stream), "vmoe_soft_route");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeSoftRoute, SoftRouteImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Arg<Any>().Ret<Any>().Ret<Any>()
                                  .Ret<Any>().Ret<Any>().Attr<float>("scale").Attr<bool>("want_logits"));

// combine_w, dispatch_w (G,S,N) -> stats (5,) f32, partial (G,4) f32 scratch
static ffi::Error SoftRouterStatsImpl(hipStream_t stream, Any combine_w, Any dispatch_w, F32Out stats,
                                      F32Out partial) {
  VmoeSoftStatsParams p{};
  p.combine_w = combine_w.untyped_data();
  p.dispatch_w = dispatch_w.untyped_data();
  p.stats = stats->typed_data();
  p.partial = partial->typed_data();
  p.G = Dim(combine_w, 0); p.S = Dim(combine_w, 1); p.N = Dim(combine_w, 2);
  p.dtype = DType(combine_w.element_type());
  return Status(vmoe_soft_router_stats(&p, stream), "vmoe_soft_router_stats");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeSoftRouterStats, SoftRouterStatsImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Arg<Any>().Ret<F32>().Ret<F32>());

// x (G,S,D), mu (D,N) -> dispatch_w, combine_w, logits (G,S,N), workspace, stats (5,) f32, partial (G,4) f32
static ffi::Error SoftRouteStatsImpl(hipStream_t stream, Any x, Any mu, AnyOut dispatch_w, AnyOut combine_w,
                                     AnyOut logits, AnyOut workspace, F32Out stats, F32Out partial, float scale,
                                     bool want_logits) {
  VmoeSoftRouteParams p{};
  p.x = x.untyped_data();
  p.mu = mu.untyped_data();
  p.scale = scale;
  p.dispatch_w = dispatch_w->untyped_data();
  p.combine_w = combine_w->untyped_data();
  p.logits = want_logits ? logits->untyped_data() : nullptr;
  p.workspace = workspace->untyped_data();
  p.workspace_bytes = workspace->size_bytes();
  p.G = Dim(x, 0); p.S = Dim(x, 1); p.D = Dim(x, 2);
  p.N = Dim(mu, 1);
  p.dtype = DType(x.element_type());
  p.workspace_prepared = 0;
  VmoeSoftStatsParams st{};
  st.combine_w = p.combine_w;
  st.dispatch_w = p.dispatch_w;
  st.stats = stats->typed_data();
  st.partial = partial->typed_data();
  st.G = p.G; st.S = p.S; st.N = p.N;
  st.dtype = p.dtype;
  return Status(vmoe_soft_route_stats(&p, &st, stream), "vmoe_soft_route_stats");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeSoftRouteStats, SoftRouteStatsImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Arg<Any>().Ret<Any>().Ret<Any>()
                                  .Ret<Any>().Ret<Any>().Ret<F32>().Ret<F32>().Attr<float>("scale")
                                  .Attr<bool>("want_logits"));

// w (G,S,E,C), data -> out; dispatch: data (G,S,D) -> (E, G*C, D); combine: data (E, G*C, D) -> (G,S,D)
static void FillEinsum(VmoeEinsumParams* p, const Any& w, const Any& data, AnyOut& out) {
  p->w = w.untyped_data();
  p->data = data.untyped_data();
  p->out = out->untyped_data();
  p->G = Dim(w, 0); p->S = Dim(w, 1); p->E = Dim(w, 2); p->C = Dim(w, 3);
  p->D = (int32_t)data.dimensions().back();
  p->w_dtype = WDType(w.element_type());
  p->data_dtype = DType(data.element_type());
  p->out_dtype = DType(out->element_type());
}
static ffi::Error EinsumDispatchImpl(hipStream_t stream, Any w, Any data, AnyOut out) {
  VmoeEinsumParams p{};
  FillEinsum(&p, w, data, out);
  return Status(vmoe_einsum_dispatch(&p, stream), "vmoe_einsum_dispatch");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeEinsumDispatch, EinsumDispatchImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Arg<Any>().Ret<Any>());
static ffi::Error EinsumCombineImpl(hipStream_t stream, Any w, Any data, AnyOut out) {
  VmoeEinsumParams p{};
  FillEinsum(&p, w, data, out);
  return Status(vmoe_einsum_combine(&p, stream), "vmoe_einsum_combine");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeEinsumCombine, EinsumCombineImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Arg<Any>().Ret<Any>());

// float32 <-> bfloat16, any shape
static ffi::Error CastImpl(hipStream_t stream, Any in, AnyOut out) {
  VmoeCastParams p{};
  p.in = in.untyped_data();
  p.out = out->untyped_data();
  p.n = in.element_count();
  p.in_dtype = DType(in.element_type());
  p.out_dtype = DType(out->element_type());
  return Status(vmoe_cast(&p, stream), "vmoe_cast");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeCast, CastImpl, ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Ret<Any>());

// ---------------------------------------------------------------- the transformer around the layer
// residual (rows, D) f32, branch (rows, D), scale, bias (D,) f32 -> residual_out f32, norm_out
static ffi::Error AddLayerNormImpl(hipStream_t stream, F32 residual, Any branch, F32 scale, F32 bias,
                                   F32Out residual_out, AnyOut norm_out, bool has_branch,
                                   bool has_affine, bool want_residual, bool want_norm, float eps) {
  VmoeAddLayerNormParams p{};
  p.residual = residual.typed_data();
  p.branch = has_branch ? branch.untyped_data() : nullptr;
  p.scale = has_affine ? scale.typed_data() : nullptr;
  p.bias = has_affine ? bias.typed_data() : nullptr;
  p.residual_out = want_residual ? residual_out->typed_data() : nullptr;
  p.norm_out = want_norm ? norm_out->untyped_data() : nullptr;
  p.D = (int32_t)residual.dimensions().back();
  p.rows = residual.element_count() / p.D;
  p.eps = eps;
  p.branch_dtype = DType(branch.element_type());
  p.out_dtype = DType(norm_out->element_type());
  return Status(vmoe_add_layer_norm(&p, stream), "vmoe_add_layer_norm");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeAddLayerNorm, AddLayerNormImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<F32>().Arg<Any>().Arg<F32>().Arg<F32>()
                                  .Ret<F32>().Ret<Any>().Attr<bool>("has_branch").Attr<bool>("has_affine")
                                  .Attr<bool>("want_residual").Attr<bool>("want_norm").Attr<float>("eps"));

// q (B,Sq,H,hd), k, v (B,Sk,H,hd), contiguous -> out (B,Sq,H*hd)
static ffi::Error AttentionImpl(hipStream_t stream, Any q, Any k, Any v, AnyOut out, float scale) {
  VmoeAttentionParams p{};
  p.q = q.untyped_data();
  p.k = k.untyped_data();
  p.v = v.untyped_data();
  p.out = out->untyped_data();
  p.B = Dim(q, 0); p.Sq = Dim(q, 1); p.H = Dim(q, 2); p.head_dim = Dim(q, 3);
  p.Sk = Dim(k, 1);
  const int64_t row = (int64_t)p.H * p.head_dim;
  p.q_stride_s = p.k_stride_s = p.v_stride_s = row;
  p.q_stride_b = row * p.Sq;
  p.k_stride_b = p.v_stride_b = row * p.Sk;
  p.scale = scale;
  p.dtype = DType(q.element_type());
  return Status(vmoe_attention(&p, stream), "vmoe_attention");
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeAttention, AttentionImpl,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Any>().Arg<Any>().Arg<Any>().Ret<Any>()
                                  .Attr<float>("scale"));
#endif  // __has_include("xla/ffi/api/ffi.h")
