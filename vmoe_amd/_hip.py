"""ctypes binding of libvmoe_hip.so (the C ABI declared in include/vmoe_hip.h).

The library is loaded from ``vmoe_amd/_lib``; there is no CPU fallback: every
op raises if the library is missing or if a tensor is not on a ROCm device.
PyTorch is used for device memory and streams only.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_float, c_int32, c_size_t, c_void_p

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_lib", "libvmoe_hip.so")
_lib = None

F32, BF16 = 0, 1
GELU_TANH, GELU_ERF = 0, 1
MLP_STATUS_ABANDONED_WAITS, MLP_STATUS_PLAN_MISMATCHES, MLP_STATUS_WORDS = 0, 1, 2
W_F32, W_BF16, W_BOOL = 0, 1, 2

EXPORTS = [
    "vmoe_abi_version", "vmoe_error_string", "vmoe_gate_topk", "vmoe_topk", "vmoe_router_metrics",
    "vmoe_route_assign", "vmoe_route_assign_metrics", "vmoe_top_items_per_expert", "vmoe_indices_to_slots", "vmoe_dispatch", "vmoe_combine", "vmoe_densify",
    "vmoe_expert_mlp_workspace_bytes", "vmoe_expert_mlp", "vmoe_expert_mlp_planned", "vmoe_expert_mlp_status", "vmoe_compact_rows_planned", "vmoe_pack_expert_weights",
    "vmoe_soft_route_workspace_bytes", "vmoe_soft_route", "vmoe_einsum_dispatch",
    "vmoe_einsum_combine", "vmoe_cast", "vmoe_copy_bytes", "vmoe_mfma_probe", "vmoe_operand_delivery_probe", "vmoe_operand_delivery_probe_k64", "vmoe_resident_delivery_probe",
    "vmoe_add_layer_norm", "vmoe_attention", "vmoe_noisy_gates", "vmoe_compact_rows", "vmoe_compact_rows_static",
    "vmoe_combine_backward_data", "vmoe_combine_backward_weights", "vmoe_soft_router_stats",
    "vmoe_soft_route_stats",
]


class VmoeError(RuntimeError):
  pass


def lib_path() -> str:
  return _LIB_PATH


def lib() -> ctypes.CDLL:
  """Loads the HIP library, failing loudly if it has not been built."""
  global _lib
  if _lib is None:
    if not os.path.exists(_LIB_PATH):
      raise VmoeError(
          f"{_LIB_PATH} is missing: build it with `python -m vmoe_amd.csrc.build` "
          "(hipcc, gfx950). There is no CPU fallback.")
    _lib = ctypes.CDLL(_LIB_PATH)
    _lib.vmoe_error_string.restype = ctypes.c_char_p
    _lib.vmoe_expert_mlp_workspace_bytes.restype = c_size_t
    _lib.vmoe_soft_route_workspace_bytes.restype = c_size_t
    if _lib.vmoe_abi_version() != 1:
      raise VmoeError("libvmoe_hip.so ABI version mismatch")
  return _lib


def check(code: int, what: str) -> None:
  if code != 0:
    msg = lib().vmoe_error_string(code).decode()
    raise VmoeError(f"{what} failed: {msg} (code {code})")


def dtype_code(dtype: torch.dtype) -> int:
  if dtype == torch.float32:
    return F32
  if dtype == torch.bfloat16:
    return BF16
  raise TypeError(f"Unsupported dtype {dtype}; the kernels cover float32 and bfloat16.")


def ptr(t) -> c_void_p:
  if t is None:
    return c_void_p(None)
  if not t.is_cuda:
    raise VmoeError("tensor is not on a ROCm device; there is no CPU fallback")
  if not t.is_contiguous():
    raise VmoeError("tensor must be contiguous")
  return c_void_p(t.data_ptr())


def stream() -> c_void_p:
  return c_void_p(torch.cuda.current_stream().cuda_stream)


class GateTopkParams(ctypes.Structure):
  _fields_ = [("x", c_void_p), ("w", c_void_p), ("logit_bias", c_void_p), ("gates", c_void_p),
              ("topk_val", c_void_p), ("topk_idx", c_void_p), ("num_items", c_int32),
              ("D", c_int32), ("E", c_int32), ("K", c_int32), ("dtype", c_int32),
              ("logits", c_void_p)]


class NoisyGatesParams(ctypes.Structure):
  _fields_ = [("logits", c_void_p), ("noise", c_void_p), ("gates_noisy", c_void_p),
              ("load_loss", c_void_p), ("G", c_int32), ("S", c_int32), ("E", c_int32),
              ("K", c_int32), ("noise_std", ctypes.c_float)]


class TopkParams(ctypes.Structure):
  _fields_ = [("gates", c_void_p), ("topk_val", c_void_p), ("topk_idx", c_void_p),
              ("num_items", c_int32), ("E", c_int32), ("K", c_int32)]


class RouterMetricsParams(ctypes.Structure):
  _fields_ = [("gates", c_void_p), ("top1_idx", c_void_p), ("importance_loss", c_void_p),
              ("gshard_loss", c_void_p), ("auxiliary_loss", c_void_p),
              ("gshard_loss_weight", c_float), ("importance_loss_weight", c_float),
              ("G", c_int32), ("S", c_int32), ("E", c_int32), ("top1_stride", c_int32),
              ("dtype", c_int32)]


class RouteAssignParams(ctypes.Structure):
  _fields_ = [("topk_val", c_void_p), ("topk_idx", c_void_p), ("indices", c_void_p),
              ("token_slot", c_void_p), ("slot_token", c_void_p), ("fill", c_void_p),
              ("G", c_int32), ("S", c_int32), ("E", c_int32), ("K", c_int32), ("C", c_int32),
              ("batch_priority", c_int32)]


class TopItemsParams(ctypes.Structure):
  _fields_ = [("gates", c_void_p), ("indices", c_void_p), ("token_slot", c_void_p),
              ("slot_token", c_void_p), ("weights", c_void_p), ("sel_minmax", c_void_p),
              ("G", c_int32), ("S", c_int32), ("E", c_int32), ("C", c_int32), ("dtype", c_int32)]


class IndicesToSlotsParams(ctypes.Structure):
  _fields_ = [("indices", c_void_p), ("token_slot", c_void_p), ("slot_token", c_void_p),
              ("num_duplicates", c_void_p), ("num_invalid", c_void_p),
              ("G", c_int32), ("S", c_int32), ("E", c_int32), ("K", c_int32), ("C", c_int32)]


class DispatchParams(ctypes.Structure):
  _fields_ = [("x", c_void_p), ("token_slot", c_void_p), ("slot_token", c_void_p),
              ("out", c_void_p), ("num_items", c_int32), ("num_slots", c_int32),
              ("K", c_int32), ("D", c_int32), ("dtype", c_int32)]


class CombineParams(ctypes.Structure):
  _fields_ = [("y", c_void_p), ("token_slot", c_void_p), ("weights", c_void_p),
              ("out", c_void_p), ("num_items", c_int32), ("num_slots", c_int32),
              ("K", c_int32), ("D", c_int32), ("dtype", c_int32)]


class DensifyParams(ctypes.Structure):
  _fields_ = [("indices", c_void_p), ("weights", c_void_p), ("combine", c_void_p),
              ("dispatch", c_void_p), ("G", c_int32), ("S", c_int32), ("E", c_int32),
              ("K", c_int32), ("C", c_int32)]


class ExpertMlpParams(ctypes.Structure):
  _fields_ = [("x", c_void_p), ("w0", c_void_p), ("b0", c_void_p), ("w1", c_void_p),
              ("b1", c_void_p), ("w0t", c_void_p), ("w1t", c_void_p), ("out", c_void_p),
              ("workspace", c_void_p), ("workspace_bytes", c_size_t),
              ("E", c_int32), ("R", c_int32), ("D", c_int32), ("M", c_int32),
              ("dtype", c_int32), ("gelu", c_int32), ("rows_per_expert", c_void_p),
              ("x_rows", c_void_p), ("num_items", c_int32)]


class CompactRowsParams(ctypes.Structure):
  _fields_ = [("fill", c_void_p), ("token_slot", c_void_p), ("token_row", c_void_p),
              ("rows_per_expert", c_void_p), ("prefix", c_void_p), ("row_token", c_void_p),
              ("G", c_int32), ("S", c_int32), ("E", c_int32), ("K", c_int32), ("C", c_int32)]


class TransposeParams(ctypes.Structure):
  _fields_ = [("in_", c_void_p), ("out", c_void_p), ("batch", c_int32), ("rows", c_int32),
              ("cols", c_int32), ("dtype", c_int32)]


class SoftRouteParams(ctypes.Structure):
  _fields_ = [("x", c_void_p), ("mu", c_void_p), ("scale", c_float), ("dispatch_w", c_void_p),
              ("combine_w", c_void_p), ("logits", c_void_p), ("workspace", c_void_p),
              ("workspace_bytes", c_size_t), ("G", c_int32), ("S", c_int32), ("D", c_int32),
              ("N", c_int32), ("dtype", c_int32), ("workspace_prepared", c_int32)]


class EinsumParams(ctypes.Structure):
  _fields_ = [("w", c_void_p), ("data", c_void_p), ("out", c_void_p),
              ("G", c_int32), ("S", c_int32), ("E", c_int32), ("C", c_int32), ("D", c_int32),
              ("w_dtype", c_int32), ("data_dtype", c_int32), ("out_dtype", c_int32)]


class CastParams(ctypes.Structure):
  _fields_ = [("in_", c_void_p), ("out", c_void_p), ("n", c_size_t),
              ("in_dtype", c_int32), ("out_dtype", c_int32)]


class SoftStatsParams(ctypes.Structure):
  _fields_ = [("combine_w", c_void_p), ("dispatch_w", c_void_p), ("partial", c_void_p),
              ("stats", c_void_p), ("G", c_int32), ("S", c_int32), ("N", c_int32), ("dtype", c_int32)]


class CombineBackwardParams(ctypes.Structure):
  _fields_ = [("dout", c_void_p), ("y", c_void_p), ("token_slot", c_void_p), ("weights", c_void_p),
              ("slot_token", c_void_p), ("dy", c_void_p), ("dweights", c_void_p),
              ("num_items", c_int32), ("num_slots", c_int32), ("K", c_int32), ("D", c_int32),
              ("dtype", c_int32)]


class AddLayerNormParams(ctypes.Structure):
  _fields_ = [("residual", c_void_p), ("branch", c_void_p), ("scale", c_void_p),
              ("bias", c_void_p), ("residual_out", c_void_p), ("norm_out", c_void_p),
              ("rows", c_size_t), ("D", c_int32), ("eps", ctypes.c_float),
              ("branch_dtype", c_int32), ("out_dtype", c_int32)]


class AttentionParams(ctypes.Structure):
  _fields_ = [("q", c_void_p), ("k", c_void_p), ("v", c_void_p), ("out", c_void_p),
              ("q_stride_b", ctypes.c_int64), ("q_stride_s", ctypes.c_int64),
              ("k_stride_b", ctypes.c_int64), ("k_stride_s", ctypes.c_int64),
              ("v_stride_b", ctypes.c_int64), ("v_stride_s", ctypes.c_int64),
              ("B", c_int32), ("H", c_int32), ("Sq", c_int32), ("Sk", c_int32),
              ("head_dim", c_int32), ("scale", ctypes.c_float), ("dtype", c_int32)]


_timing_sink = None


class TimingSink(dict):
  """``sink[name]`` -> list of (start, stop) event pairs, one per call of entry point
  ``name``.  Creating a timing event costs the host far more than recording one, so
  ``pairs`` of them are created (and recorded once, which is when the runtime really
  allocates them) up front; a measured loop then only records.  An event between two
  kernels also keeps the second from being set up while the first still runs, so a
  loop whose total time matters passes ``only`` = the entry points it needs timed."""

  def __init__(self, pairs: int = 0, only=None):
    super().__init__()
    self.only = None if only is None else frozenset(only)   # entry points to time; None = all
    self._pool = []
    for _ in range(pairs):
      pair = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
      pair[0].record()
      pair[1].record()
      self._pool.append(pair)
    if pairs:
      torch.cuda.synchronize()

  def take(self):
    if self._pool:
      return self._pool.pop()
    return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)


def set_timing_sink(sink) -> None:
  """With a dict (or a TimingSink) as sink, every entry point is bracketed by a pair
  of timing events on the stream it is launched on; the pairs are appended to
  ``sink[name]`` for the caller to read after synchronising.  None disables."""
  global _timing_sink
  _timing_sink = sink


def call2(name: str, first: ctypes.Structure, second: ctypes.Structure) -> None:
  """An entry point that takes two parameter blocks; timed like call()."""
  fn = getattr(lib(), name)
  sink = _timing_sink
  if sink is None or (getattr(sink, "only", None) is not None and name not in sink.only):
    check(fn(ctypes.byref(first), ctypes.byref(second), stream()), name)
    return
  take = getattr(sink, "take", None)
  start, stop = take() if take is not None else (
      torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
  start.record()
  code = fn(ctypes.byref(first), ctypes.byref(second), stream())
  stop.record()
  sink.setdefault(name, []).append((start, stop))
  check(code, name)


def call_blocks(name: str, *args, accept=()) -> int:
  """An entry point that takes several parameter blocks before the stream (passed by
  reference).  Timed like call().  Return codes listed in `accept` are returned, not raised."""
  fn = getattr(lib(), name)
  cargs = [ctypes.byref(a) if isinstance(a, ctypes.Structure) else a for a in args]
  sink = _timing_sink
  if sink is None or (getattr(sink, "only", None) is not None and name not in sink.only):
    code = fn(*cargs, stream())
  else:
    take = getattr(sink, "take", None)
    start, stop = take() if take is not None else (
        torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
    start.record()
    code = fn(*cargs, stream())
    stop.record()
    sink.setdefault(name, []).append((start, stop))
  if code in accept:
    return code
  check(code, name)
  return code


def call(name: str, params: ctypes.Structure) -> None:
  fn = getattr(lib(), name)
  sink = _timing_sink
  if sink is None or (getattr(sink, "only", None) is not None and name not in sink.only):
    check(fn(ctypes.byref(params), stream()), name)
    return
  take = getattr(sink, "take", None)
  start, stop = take() if take is not None else (
      torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
  start.record()
  code = fn(ctypes.byref(params), stream())
  stop.record()
  sink.setdefault(name, []).append((start, stop))
  check(code, name)
