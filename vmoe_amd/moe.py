"""Dispatchers and routing algorithms of the MoE layer, on HIP kernels.

Host-side mirror of vmoe/moe.py: same class names, argument names, shapes and
error messages, with torch tensors on a ROCm device in place of jax arrays.
All arithmetic runs in the HIP kernels of libvmoe_hip.so (vmoe_amd.kernels);
there is no CPU path.

In all cases dispatch takes (G, S, ...) and returns (E, G*C, ...) in the row
order of the reference's _dispatch (vmoe/moe.py:488-500); combine takes
(E, G*C, ...) and returns (G, S, ...).
"""
from __future__ import annotations

import abc
import functools
import logging
import math
from typing import Any, Callable, Dict, Mapping, Optional, Tuple

import torch

from vmoe_amd import kernels as K

Array = torch.Tensor
_FLOAT_DTYPES = (torch.float32, torch.bfloat16)


class BaseDispatcher(abc.ABC):
  """Interface of vmoe/moe.py:50-90."""

  @abc.abstractmethod
  def dispatch(self, data: Array) -> Array:
    """(G, S, ...) -> (E, G * C, ...)."""

  @abc.abstractmethod
  def combine(self, data: Array) -> Array:
    """(E, G * C, ...) -> (G, S, ...)."""


def _as_rows(data: Array, lead: int) -> Tuple[Array, Tuple[int, ...], int]:
  """Flattens trailing item dims to one and pads rows to a multiple of 16 bytes."""
  if data.dtype not in _FLOAT_DTYPES:
    raise TypeError(f"Unsupported data dtype {data.dtype}: the kernels move float32 and bfloat16.")
  item_shape = tuple(data.shape[lead:])
  width = int(math.prod(item_shape)) if item_shape else 1
  rows = data.reshape(-1, width)
  per16 = 16 // data.element_size()
  pad = (-width) % per16
  if pad:
    rows = torch.nn.functional.pad(rows, (0, pad))
  return rows.contiguous(), item_shape, width


def _from_rows(rows: Array, lead_shape, item_shape, width: int) -> Array:
  if rows.shape[-1] != width:
    rows = rows[:, :width]
  return rows.reshape(*lead_shape, *item_shape)


class _DispatchFn(torch.autograd.Function):
  """dispatch with its gradient: dx[t] = sum_k dbuf[slot(t, k)] (combine with unit weights)."""

  @staticmethod
  def forward(ctx, rows, token_slot, slot_token, num_slots):
    ctx.save_for_backward(token_slot)
    return K.dispatch(rows, token_slot, slot_token, num_slots=num_slots)

  @staticmethod
  def backward(ctx, grad):
    (token_slot,) = ctx.saved_tensors
    ones = torch.ones(token_slot.shape, dtype=torch.float32, device=grad.device)
    return K.combine(grad.contiguous(), token_slot, ones), None, None, None


class _CombineFn(torch.autograd.Function):
  """combine with its gradients: dy[slot(t, k)] = w[t, k] * dout[t] and
  dw[t, k] = <dout[t], y[slot(t, k)]>."""

  @staticmethod
  def forward(ctx, rows, token_slot, weights, slot_token):
    ctx.save_for_backward(rows, token_slot, weights, slot_token)
    return K.combine(rows, token_slot, weights)

  @staticmethod
  def backward(ctx, grad):
    rows, token_slot, weights, slot_token = ctx.saved_tensors
    grad = grad.contiguous()
    d_rows = d_w = None
    if ctx.needs_input_grad[0]:
      d_rows = K.combine_backward_data(grad, token_slot, weights, slot_token, rows.shape[0])
    if ctx.needs_input_grad[2]:
      d_w = K.combine_backward_weights(grad, rows, token_slot).to(weights.dtype)
    return d_rows, None, d_w, None


def _wants_grad(*tensors) -> bool:
  return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


class ExpertIndicesDispatcher(BaseDispatcher):
  """Dispatcher using (expert, buffer position) indices; vmoe/moe.py:164-209.

  Attributes:
    indices: (G, S, K, 2) int32 (expert, position) per item and choice; entries
      with expert >= num_experts or position >= capacity are dropped.
    combine_weights: (G, S, K).
    num_experts, capacity: static sizes of the expert buffer.

  Routers give every slot at most one item.  Hand-made indices that send several items
  to one slot are accumulated as the reference's scatter-add does (vmoe/moe.py:190-197,
  :522-544): dispatch then runs once per "occurrence" (the r-th item of every slot) and
  the passes are added in float32, in item order.
  """

  def __init__(self, indices: Array, combine_weights: Array, num_experts: int, capacity: int,
               partition_spec=None, einsum_precision=None, _slots=None):
    self.indices = indices
    self._combine_weights = combine_weights       # a tensor, or (float32 tensor, dtype) cast on first read
    self.num_experts = int(num_experts)
    self.capacity = int(capacity)
    self.partition_spec = partition_spec          # accepted for API parity; one GPU, no mesh
    self.einsum_precision = einsum_precision      # combine always accumulates in float32
    self._slots = _slots                          # (token_slot (G,S,K), slot_token (E*G*C,))
    self._weights_f32 = None                      # float32 copy of combine_weights, if on hand
    self.fill = None                              # (G, E) kept items per (group, expert), if known
    self._packed_maps = None                      # (token_row (G,S,K), rows_per_expert (E,))
    self._rounds = None                           # per-occurrence slot maps when slots are shared

  @property
  def combine_weights(self) -> Array:
    cw = self._combine_weights
    if isinstance(cw, tuple):                     # made by a router: the cast is only for readers
      cw = self._combine_weights = K.cast(cw[0], cw[1])
    return cw

  @combine_weights.setter
  def combine_weights(self, value: Array):
    self._combine_weights = value

  def _maps(self):
    if self._slots is None:
      if self.indices.ndim != 4 or self.indices.shape[-1] != 2:
        raise ValueError(f"indices must have shape (G, S, K, 2), got {tuple(self.indices.shape)}")
      token_slot, slot_token, counters = K.indices_to_slots(
          self.indices, self.num_experts, self.capacity)
      dups, invalid = counters.tolist()
      if invalid:
        raise ValueError("ExpertIndicesDispatcher: negative indices are not supported.")
      if dups:
        self._rounds = self._occurrence_rounds(token_slot, slot_token.numel())
      self._slots = (token_slot, slot_token)
    return self._slots

  @staticmethod
  def _occurrence_rounds(token_slot: Array, num_slots: int):
    """Splits the assignments so that no slot appears twice in a part: part r holds, for
    every slot, its r-th assignment in item order.  Returns [(token_slot_r, slot_token_r)]."""
    flat = token_slot.reshape(-1).to(torch.int64)
    K_ = token_slot.shape[-1]
    order = torch.argsort(flat, stable=True)
    sorted_slots = flat[order]
    first = torch.ones_like(sorted_slots, dtype=torch.bool)
    first[1:] = sorted_slots[1:] != sorted_slots[:-1]
    pos = torch.arange(flat.numel(), device=flat.device)
    start = torch.where(first, pos, torch.zeros_like(pos)).cummax(0).values
    occurrence = torch.empty_like(flat)
    occurrence[order] = pos - start
    occurrence[flat < 0] = -1
    rounds = []
    for r in range(int(occurrence.max().item()) + 1):
      mine = occurrence == r
      ts_r = torch.where(mine, flat, torch.full_like(flat, -1)).to(torch.int32)
      st_r = torch.full((num_slots,), -1, dtype=torch.int32, device=flat.device)
      st_r[flat[mine]] = (pos[mine] // K_).to(torch.int32)
      rounds.append((ts_r.view(-1, K_).contiguous(), st_r))
    return rounds

  def dispatch(self, data: Array) -> Array:
    G, S, Kk, _ = self.indices.shape
    token_slot, slot_token = self._maps()
    rows, item_shape, width = _as_rows(data, 2)
    if self._rounds is not None:
      if _wants_grad(rows):
        raise NotImplementedError("gradients through a dispatch with shared slots")
      acc = None
      for ts_r, st_r in self._rounds:
        part = K.dispatch(rows, ts_r, st_r).to(torch.float32)
        acc = part if acc is None else acc + part
      out = acc.to(rows.dtype)
    elif _wants_grad(rows):
      out = _DispatchFn.apply(rows, token_slot.view(G * S, Kk), slot_token, slot_token.numel())
    else:
      out = K.dispatch(rows, token_slot.view(G * S, Kk), slot_token)
    return _from_rows(out, (self.num_experts, G * self.capacity), item_shape, width)

  def combine(self, data: Array) -> Array:
    G, S, Kk, _ = self.indices.shape
    token_slot, slot_token = self._maps()
    rows, item_shape, width = _as_rows(data, 2)
    cw = self._combine_weights
    if _wants_grad(rows, cw if isinstance(cw, torch.Tensor) else None):
      # differentiable in the data and in combine_weights
      w = self.combine_weights.to(torch.float32)
      out = _CombineFn.apply(rows, token_slot.view(G * S, Kk), w.reshape(G * S, Kk), slot_token)
      return _from_rows(out, (G, S), item_shape, width)
    w = self._weights_f32 if self._weights_f32 is not None else K.cast(
        self.combine_weights.contiguous(), torch.float32)
    out = K.combine(rows, token_slot.view(G * S, Kk), w.view(G * S, Kk))
    return _from_rows(out, (G, S), item_shape, width)

  # Packed rows.  The reference's buffer gives every (group, expert) pair `capacity`
  # rows, filled or not, and the experts run over all of them.  When the fill counts
  # are known (dispatchers made by the routers), the same buffer can hold each
  # expert's items in its first rows instead; experts that accept a row count per
  # expert then skip the rest.  dispatch_packed / combine_packed are the pair used
  # by sparse_moe_spmd for that; dispatch / combine keep the reference layout.
  def supports_packed(self) -> bool:
    return self.fill is not None

  def _packed(self):
    if self._packed_maps is None:
      token_slot, _ = self._maps()
      self._packed_maps = K.compact_rows(self.fill, token_slot, self.capacity)
    return self._packed_maps

  def pending_compaction(self):
    """-> (fill, token_slot, capacity) while the packed rows have not been computed (an
    expert that computes them itself hands them back with set_packed_maps), else None."""
    if self._packed_maps is not None or self.fill is None:
      return None
    token_slot, _ = self._maps()
    return self.fill, token_slot, self.capacity

  def set_packed_maps(self, maps) -> None:
    self._packed_maps = tuple(maps)

  def packed_rows(self):
    """-> (row_token (E, G * capacity) int32: the item (g * S + s) in every packed row,
    rows_per_expert (E,) int32): what an expert needs to gather its rows itself."""
    _, rows_per_expert, row_token = self._packed()
    return row_token, rows_per_expert

  def dispatch_packed(self, data: Array):
    """-> (buffer (E, G * capacity, ...) whose expert e holds items in rows
    0 .. rows_per_expert[e] - 1 and arbitrary values after them, rows_per_expert (E,) int32)."""
    G, S, Kk, _ = self.indices.shape
    token_row, rows_per_expert, _ = self._packed()
    rows, item_shape, width = _as_rows(data, 2)
    out = K.dispatch(rows, token_row.view(G * S, Kk), None,
                     num_slots=self.num_experts * G * self.capacity)
    return (_from_rows(out, (self.num_experts, G * self.capacity), item_shape, width),
            rows_per_expert)

  def combine_packed(self, data: Array) -> Array:
    G, S, Kk, _ = self.indices.shape
    token_row = self._packed()[0]
    rows, item_shape, width = _as_rows(data, 2)
    w = self._weights_f32 if self._weights_f32 is not None else K.cast(
        self.combine_weights.contiguous(), torch.float32)
    out = K.combine(rows, token_row.view(G * S, Kk), w.view(G * S, Kk))
    return _from_rows(out, (G, S), item_shape, width)


class EinsumDispatcher(BaseDispatcher):
  """Dispatcher using dense (G, S, E, C) weights; vmoe/moe.py:127-161."""

  def __init__(self, combine_weights: Array, dispatch_weights: Optional[Array] = None,
               partition_spec=None, einsum_precision=None):
    self.combine_weights = combine_weights
    self.dispatch_weights = dispatch_weights
    self.partition_spec = partition_spec
    self.einsum_precision = einsum_precision

  @staticmethod
  def _result_dtype(w: Array, data: Array) -> torch.dtype:
    if w.dtype == torch.bool:
      return data.dtype
    return torch.promote_types(w.dtype, data.dtype)

  def dispatch(self, data: Array) -> Array:
    w = self.combine_weights > 0 if self.dispatch_weights is None else self.dispatch_weights
    G, S, E, C = w.shape
    rows, item_shape, width = _as_rows(data, 2)
    out = K.einsum_dispatch(w, rows.view(G, S, -1), self._result_dtype(w, data))
    return _from_rows(out, (E, G * C), item_shape, width)

  def combine(self, data: Array) -> Array:
    w = self.combine_weights
    G, S, E, C = w.shape
    rows, item_shape, width = _as_rows(data, 2)
    out = K.einsum_combine(w, rows, self._result_dtype(w, data))
    return _from_rows(out.view(G * S, -1), (G, S), item_shape, width)


class DenseEinsumDispatcher(BaseDispatcher):
  """Dispatcher sending every item to every expert (C = S); vmoe/moe.py:93-124.

  Attributes:
    combine_weights: (G, S, E).
  """

  def __init__(self, combine_weights: Array, partition_spec=None, einsum_precision=None):
    self.combine_weights = combine_weights
    self.partition_spec = partition_spec
    self.einsum_precision = einsum_precision

  def dispatch(self, data: Array) -> Array:
    # every expert receives a copy of every item: (E, G*S, ...) in the buffer row order
    G, S, E = self.combine_weights.shape
    dev = data.device
    slot = torch.arange(S, dtype=torch.int32, device=dev)
    indices = torch.stack(torch.meshgrid(torch.arange(E, dtype=torch.int32, device=dev), slot,
                                         indexing="ij"), dim=-1)      # (E, S, 2): (e, s)
    indices = indices.permute(1, 0, 2)[None].expand(G, S, E, 2).contiguous()
    ones = torch.ones((G, S, E), dtype=torch.float32, device=dev)
    return ExpertIndicesDispatcher(indices, ones, E, S).dispatch(data)

  def combine(self, data: Array) -> Array:
    G, S, E = self.combine_weights.shape
    dev = data.device
    slot = torch.arange(S, dtype=torch.int32, device=dev)
    indices = torch.stack(torch.meshgrid(torch.arange(E, dtype=torch.int32, device=dev), slot,
                                         indexing="ij"), dim=-1).permute(1, 0, 2)
    indices = indices[None].expand(G, S, E, 2).contiguous()
    return ExpertIndicesDispatcher(indices, self.combine_weights, E, S).combine(data)


class _SparseEinsumDispatcher(EinsumDispatcher):
  """EinsumDispatcher produced by top-experts-per-item routing.

  The (G, S, E, C) one-hot weights (vmoe/moe.py:609-619) are only materialised
  when ``combine_weights`` / ``dispatch_weights`` are read; dispatch and combine
  use the item <-> slot maps, which give the same results as the one-hot
  einsums (each slot has at most one contributor).
  """

  def __init__(self, inner: ExpertIndicesDispatcher, gates_dtype: torch.dtype, **kwargs):
    self._inner = inner
    self._gates_dtype = gates_dtype
    self._dense = None
    self.partition_spec = kwargs.get("partition_spec")
    self.einsum_precision = kwargs.get("einsum_precision")

  def _densify(self):
    if self._dense is None:
      cw, dw = K.densify(self._inner.indices, self._inner.combine_weights,
                         self._inner.num_experts, self._inner.capacity)
      self._dense = (K.cast(cw, self._gates_dtype), dw)
    return self._dense

  @property
  def combine_weights(self) -> Array:
    return self._densify()[0]

  @property
  def dispatch_weights(self) -> Array:
    return self._densify()[1]

  def dispatch(self, data: Array) -> Array:
    return self._inner.dispatch(data)

  def combine(self, data: Array) -> Array:
    return self._inner.combine(data)

  def supports_packed(self) -> bool:
    return self._inner.supports_packed()

  def dispatch_packed(self, data: Array):
    return self._inner.dispatch_packed(data)

  def packed_rows(self):
    return self._inner.packed_rows()

  def pending_compaction(self):
    return self._inner.pending_compaction()

  def set_packed_maps(self, maps) -> None:
    self._inner.set_packed_maps(maps)

  def combine_packed(self, data: Array) -> Array:
    return self._inner.combine_packed(data)


class Bfloat16Dispatcher(BaseDispatcher):
  """Wrapper converting data to bfloat16 around the inner dispatcher; vmoe/moe.py:212-227."""

  def __init__(self, dispatcher: BaseDispatcher):
    self.dispatcher = dispatcher

  def dispatch(self, data: Array) -> Array:
    dtype = data.dtype
    data = _cast_to_bfloat16(data)
    data = self.dispatcher.dispatch(data)
    return K.cast(data, dtype) if data.is_floating_point() else data

  def combine(self, data: Array) -> Array:
    dtype = data.dtype
    data = _cast_to_bfloat16(data)
    data = self.dispatcher.combine(data)
    return K.cast(data, dtype) if data.is_floating_point() else data

  def supports_packed(self) -> bool:
    fn = getattr(self.dispatcher, "supports_packed", None)
    return bool(fn and fn())

  def dispatch_packed(self, data: Array):
    dtype = data.dtype
    out, rows = self.dispatcher.dispatch_packed(_cast_to_bfloat16(data))
    return (K.cast(out, dtype) if out.is_floating_point() else out), rows

  def combine_packed(self, data: Array) -> Array:
    dtype = data.dtype
    out = self.dispatcher.combine_packed(_cast_to_bfloat16(data))
    return K.cast(out, dtype) if out.is_floating_point() else out


def _cast_to_bfloat16(x: Array) -> Array:
  """vmoe/moe.py:477-478."""
  return K.cast(x, torch.bfloat16) if x.is_floating_point() else x


@functools.lru_cache(maxsize=256)   # a layer asks on every call; compute (and warn) once per shape
def compute_capacity(num_tokens: int, num_experts: int, capacity_factor: float,
                     ceil_or_round: str = "ceil", multiple_of: Optional[int] = 4) -> int:
  """Capacity per expert needed to distribute num_tokens among num_experts; vmoe/moe.py:230-257."""
  if ceil_or_round == "ceil":
    capacity = int(math.ceil(num_tokens * capacity_factor / num_experts))
  elif ceil_or_round == "round":
    capacity = int(round(num_tokens * capacity_factor / num_experts))
  else:
    raise ValueError(f"Unsupported {ceil_or_round=}")
  if capacity < 1:
    raise ValueError(f"The values num_tokens = f{num_tokens}, num_experts = "
                     f"{num_experts} and capacity_factor = {capacity_factor} "
                     f"lead to capacity = {capacity}, but it must be greater "
                     "than or equal to 1.")
  if multiple_of and multiple_of > 0:
    capacity += (-capacity) % multiple_of
  actual_capacity_factor = capacity * num_experts / num_tokens
  if abs(actual_capacity_factor - capacity_factor) > 1e-6:
    logging.warning(
        "The target capacity_factor is %f, but with num_tokens=%d and "
        "num_experts=%d the actual capacity_factor is %f.",
        capacity_factor, num_tokens, num_experts, actual_capacity_factor)
  return capacity


def get_dense_einsum_dispatcher(gates: Array, **dispatcher_kwargs) -> DenseEinsumDispatcher:
  """Every item goes to every expert: nothing to route, the gates (G, S, E) are the
  combine weights; vmoe/moe.py:260-264."""
  return DenseEinsumDispatcher(combine_weights=gates, **dispatcher_kwargs)


def get_top_experts_per_item_dispatcher(
    gates: Array, name: str, num_selected_experts: int, batch_priority: bool,
    capacity: Optional[int] = None, capacity_factor: Optional[float] = None,
    capacity_ceil_or_round: str = "ceil", capacity_multiple_of: Optional[int] = 4,
    **dispatcher_kwargs) -> BaseDispatcher:
  """Top-Experts-Per-Item routing; vmoe/moe.py:267-327.

  gates is (S, E) as in the reference, or (G, S, E) for all groups at once (what
  the reference obtains with jax.vmap, vmoe/nn/routing.py:123-128).
  """
  if (capacity is None) == (capacity_factor is None):
    raise ValueError(
        "You must specify either 'capacity' or 'capacity_factor', and not both."
        f" Current values are capacity = {capacity!r}, "
        f"capacity_factor = {capacity_factor!r}")
  if not capacity:
    group_size, num_experts = gates.shape[-2:]
    capacity = compute_capacity(
        num_tokens=group_size * num_selected_experts,
        num_experts=num_experts,
        capacity_factor=capacity_factor,
        ceil_or_round=capacity_ceil_or_round,
        multiple_of=capacity_multiple_of)
  fn_map = {
      "einsum": _get_top_experts_per_item_einsum_dispatcher,
      "indices": _get_top_experts_per_item_expert_indices_dispatcher,
  }
  if name not in fn_map:
    raise ValueError(f"Unknown dispatcher type: {name!r}")
  return fn_map[name](gates, num_selected_experts, capacity, batch_priority,
                      **dispatcher_kwargs)


def _route(gates: Array, num_selected_experts: int, capacity: int, batch_priority: bool,
           topk: Optional[Tuple[Array, Array]] = None, _metrics=None, **dispatcher_kwargs):
  """Shared core of vmoe/moe.py:547-590: top-k, priority order, slot positions.

  ``_metrics=(gshard_loss_weight, importance_loss_weight, out)`` (used by the routers)
  computes the auxiliary losses of vmoe/nn/routing.py:133-157 in the same launch and
  stores them in the dict ``out``."""
  if gates.ndim not in (2, 3):
    raise ValueError(f"gates must be (S, E) or (G, S, E), got {tuple(gates.shape)}")
  batched = gates.ndim == 3
  g3 = gates if batched else gates[None]
  num_experts = g3.shape[-1]
  if topk is None:
    val, idx = K.topk(g3, num_selected_experts)
  else:
    val, idx = topk
  if _metrics is not None and batched:
    w_gshard, w_importance, out = _metrics
    indices, token_slot, slot_token, fill, losses = K.route_assign(
        val, idx, num_experts, capacity, batch_priority, metrics=(g3, w_gshard, w_importance))
    out["importance_loss"], out["gshard_loss"], out["auxiliary_loss"] = losses
  else:
    indices, token_slot, slot_token, fill = K.route_assign(
        val, idx, num_experts, capacity, batch_priority)
  inner = ExpertIndicesDispatcher(
      indices=indices, combine_weights=(val, gates.dtype) if gates.dtype != val.dtype else val,
      num_experts=num_experts, capacity=capacity, _slots=(token_slot, slot_token),
      **dispatcher_kwargs)
  inner.fill = fill
  inner._weights_f32 = val
  return inner, batched


def _get_top_experts_per_item_expert_indices_dispatcher(
    gates: Array, num_selected_experts: int, capacity: int, batch_priority: bool,
    _topk=None, _metrics=None, **dispatcher_kwargs) -> ExpertIndicesDispatcher:
  """vmoe/moe.py:626-652."""
  inner, batched = _route(gates, num_selected_experts, capacity, batch_priority, _topk,
                          _metrics=_metrics, **dispatcher_kwargs)
  if not batched:   # reference shapes for a single group: (S, K, 2) and (S, K)
    return _SingleGroupView(inner)
  return inner


def _get_top_experts_per_item_einsum_dispatcher(
    gates: Array, num_selected_experts: int, capacity: int, batch_priority: bool,
    _topk=None, _metrics=None, **dispatcher_kwargs) -> EinsumDispatcher:
  """vmoe/moe.py:593-623."""
  inner, batched = _route(gates, num_selected_experts, capacity, batch_priority, _topk,
                          _metrics=_metrics)
  d = _SparseEinsumDispatcher(inner, gates.dtype, **dispatcher_kwargs)
  if not batched:
    return _SingleGroupView(d)
  return d


class _SingleGroupView:
  """Presents a one-group dispatcher with the reference's un-vmapped leaf shapes."""

  def __init__(self, dispatcher):
    self._d = dispatcher

  def __getattr__(self, name):
    v = getattr(self._d, name)
    if isinstance(v, torch.Tensor) and name in ("indices", "combine_weights", "dispatch_weights"):
      return v[0]
    return v

  @property
  def __class__(self):   # isinstance(view, EinsumDispatcher) holds, as in the reference tests
    return self._d.__class__


def get_top_items_per_expert_dispatcher(gates: Array, name: str, capacity: Optional[int] = None,
                                        capacity_factor: Optional[float] = None,
                                        capacity_ceil_or_round: str = "ceil",
                                        capacity_multiple_of: Optional[int] = 4,
                                        **dispatcher_kwargs):
  """Top-Items-Per-Expert ("experts choice") routing; vmoe/moe.py:330-385.

  gates is (S, E) as in the reference, or (G, S, E) for all groups at once (what
  the reference obtains with jax.vmap, vmoe/nn/routing.py:236-241; the metrics
  then have a leading group axis, as under vmap).  Returns (dispatcher, metrics).
  """
  if (capacity is None) == (capacity_factor is None):
    raise ValueError(
        "You must specify either 'capacity' or 'capacity_factor', and not both."
        f" Current values are capacity = {capacity!r}, "
        f"capacity_factor = {capacity_factor!r}")
  if not capacity:
    group_size, num_experts = gates.shape[-2:]
    capacity = compute_capacity(
        num_tokens=group_size, num_experts=num_experts, capacity_factor=capacity_factor,
        ceil_or_round=capacity_ceil_or_round, multiple_of=capacity_multiple_of)
  fn_map = {"einsum": _get_top_items_per_expert_einsum_dispatcher}
  if name not in fn_map:
    raise ValueError(f"Unknown dispatcher type: {name!r}")
  return fn_map[name](gates, capacity, **dispatcher_kwargs)


def _get_top_items_per_expert_einsum_dispatcher(gates: Array, capacity: int, **dispatcher_kwargs):
  """vmoe/moe.py:655-694: every expert takes the `capacity` items with its largest gates.

  The dispatcher is an EinsumDispatcher whose (G, S, E, C) one-hot weights are
  only materialised when read; dispatch and combine move rows through the
  item <-> slot maps (every slot has exactly one contributor), which gives the
  results of the reference's einsums.
  """
  if gates.ndim not in (2, 3):
    raise ValueError(f"gates must be (S, E) or (G, S, E), got {tuple(gates.shape)}")
  batched = gates.ndim == 3
  g3 = gates if batched else gates[None]
  G, S, E = g3.shape
  if capacity > S:   # jax.lax.top_k(operand, k) requires k <= the operand's last dimension
    raise ValueError(f"capacity = {capacity} exceeds the group size {S}")
  indices, token_slot, slot_token, weights, sel = K.top_items_per_expert(g3, capacity)
  inner = ExpertIndicesDispatcher(
      indices=indices, combine_weights=weights, num_experts=E, capacity=capacity,
      _slots=(token_slot, slot_token))
  inner._weights_f32 = weights
  dispatcher = _SparseEinsumDispatcher(inner, gates.dtype, **dispatcher_kwargs)
  # Metrics useful for monitoring training (moe.py:681-692).
  per_item = (token_slot >= 0).sum(dim=2, dtype=torch.int32)            # (G, S)
  metrics = {
      "num_experts_per_item_min": per_item.amin(dim=1),
      "num_experts_per_item_max": per_item.amax(dim=1),
      "min_selected_gate": sel[:, :, 0].amin(dim=1).to(gates.dtype),
      "max_selected_gate": sel[:, :, 1].amax(dim=1).to(gates.dtype),
  }
  log2_num_experts = int(math.log2(E))
  for t in [2**i for i in range(log2_num_experts + 1)] + [E]:
    metrics[f"ratio_processed_items_by_at_least_{t}_experts"] = (
        (per_item >= t).sum(dim=1).to(torch.float32) / S)
  if not batched:
    return _SingleGroupView(dispatcher), {k: v[0] for k, v in metrics.items()}
  return dispatcher, metrics


def sparse_moe_spmd(target, variable_axes: Optional[Mapping[str, Any]] = None,
                    split_rngs: Optional[Mapping[str, bool]] = None, has_aux: bool = False,
                    methods=None):
  """Wraps an expert module class into a sparse MoE of it; vmoe/moe.py:388-448.

  The returned class is constructed like ``target``; its instances are called as
  ``layer.apply(variables, dispatcher, *inputs)``: inputs are dispatched, the
  expert is applied to every slice along the leading (expert) axis with the
  matching slice of the parameters, and outputs are combined.

  Parameters live stacked on axis 0 (``variable_axes={'params': 0}``).  If the
  target defines ``apply_experts(variables, *inputs)`` it receives all experts
  at once (this is how MlpBlock reaches the grouped GEMM kernel); otherwise
  ``target.apply`` runs once per expert.
  """
  del methods
  variable_axes = dict(variable_axes or {"params": 0})
  split_rngs = dict(split_rngs or {})

  class SparseMoe:
    expert_cls = target

    def __init__(self, *args, name: Optional[str] = None, **kwargs):
      self.name = name
      self.expert = target(*args, **kwargs)

    def init(self, rng, dispatcher: BaseDispatcher, *inputs):
      dispatched = [dispatcher.dispatch(x) for x in inputs]
      num_experts = dispatched[0].shape[0]
      split = bool(split_rngs.get("params", False))
      per_expert = []
      for e in range(num_experts):
        seed = _fold_seed(rng, e if split else 0)
        per_expert.append(self.expert.init(seed, *[d[e] for d in dispatched]))
      return _tree_stack(per_expert)

    def apply(self, variables, dispatcher: BaseDispatcher, *inputs):
      supports = getattr(dispatcher, "supports_packed", None)
      if (not has_aux and len(inputs) == 1 and supports is not None and supports()
          and getattr(self.expert, "supports_packed_rows", False)
          and not _wants_grad(inputs[0])):
        # Each expert's items in its first rows; the expert skips the empty ones.
        gather = getattr(self.expert, "apply_experts_gathered", None)
        packed_rows = getattr(dispatcher, "packed_rows", None)
        x = inputs[0]
        if (gather is not None and packed_rows is not None and x.ndim == 3
            and self.expert.can_gather(x)):
          # ... and fetches them from the items itself: no dispatched buffer at all.
          routed = getattr(self.expert, "apply_experts_routed", None)
          pending = getattr(dispatcher, "pending_compaction", None)
          todo = pending() if (routed is not None and pending is not None) else None
          if todo is not None:    # the packed rows come out of the expert's planning launch
            outputs, maps = routed(variables, x.reshape(-1, x.shape[-1]), *todo)
            dispatcher.set_packed_maps(maps)
          else:
            row_token, rows_per_expert = packed_rows()
            outputs = gather(variables, x.reshape(-1, x.shape[-1]), row_token, rows_per_expert)
        else:
          dispatched, rows_per_expert = dispatcher.dispatch_packed(x)
          outputs = self.expert.apply_experts(variables, dispatched,
                                              rows_per_expert=rows_per_expert)
        return _tree_map(dispatcher.combine_packed, outputs)
      dispatched = [dispatcher.dispatch(x) for x in inputs]
      if hasattr(self.expert, "apply_experts"):
        outputs = self.expert.apply_experts(variables, *dispatched)
      else:
        num_experts = dispatched[0].shape[0]
        outs = [self.expert.apply(_tree_index(variables, e), *[d[e] for d in dispatched])
                for e in range(num_experts)]
        outputs = _tree_stack(outs)
      aux = None
      if has_aux:
        outputs, aux = outputs
      outputs = _tree_map(dispatcher.combine, outputs)
      return (outputs, aux) if has_aux else outputs

    __call__ = apply

  SparseMoe.__name__ = f"SparseMoe{getattr(target, '__name__', 'Target')}"
  return SparseMoe


def sparse_moe_spmd_with_axes(target, variable_axes, split_rngs, partitioning_axis_names,
                              has_aux: bool = False, methods=None):
  """vmoe/moe.py:451-474; the axis-name metadata has no effect on one GPU."""
  del partitioning_axis_names
  return sparse_moe_spmd(target, variable_axes, split_rngs, has_aux, methods)


# ----------------------------------------------------------------------------- tree helpers
def _fold_seed(rng, i: int) -> int:
  base = int(rng) if not isinstance(rng, torch.Generator) else rng.initial_seed()
  return (base * 1000003 + i) % (2**63 - 1)


def _tree_map(fn: Callable, tree):
  if isinstance(tree, Mapping):
    return {k: _tree_map(fn, v) for k, v in tree.items()}
  if isinstance(tree, (tuple, list)):
    return type(tree)(_tree_map(fn, v) for v in tree)
  return fn(tree)


def _tree_index(tree, e: int):
  return _tree_map(lambda t: t[e], tree)


def _tree_stack(trees):
  first = trees[0]
  if isinstance(first, Mapping):
    return {k: _tree_stack([t[k] for t in trees]) for k in first}
  if isinstance(first, (tuple, list)):
    return type(first)(_tree_stack([t[i] for t in trees]) for i in range(len(first)))
  return torch.stack(list(trees), dim=0)
