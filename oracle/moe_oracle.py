"""NumPy restatement of the reference MoE layer (TEST INFRASTRUCTURE ONLY).

Every function cites the reference lines it follows (paths are relative to the
reference checkout).  Arrays are NumPy ``float32``/``int32``; a "bfloat16"
array is a float32 array whose values are all exactly representable in
bfloat16 (see :func:`bf16_round`), which makes "bf16 operands, fp32
accumulate" a plain float32 matmul of rounded operands.

Pinning status (what fixes each function besides its own text):

* ``compute_capacity``, ``top_experts_per_item_*``, ``ExpertIndicesDispatcher``,
  ``EinsumDispatcher``, ``dispatch_layout``/``receive_layout``,
  ``Bfloat16Dispatcher``, ``gshard_auxiliary_loss``,
  ``importance_auxiliary_loss``, ``load_auxiliary_loss``,
  ``soft_router_metrics``, ``cosine_psim``, ``top_items_per_expert_einsum``:
  pinned by the golden vectors the reference's own tests hold
  (tests/golden/*.json) plus brute-force and invariant checks in tests/.
* ``dispatch_layout`` for ``G/E > 1``: pinned by an einops-based independent
  statement of the reshape/swapaxes at moe.py:493-495 and by round trips.
* tie-breaking in ``top_k``/BPR order: the reference goldens hold no ties;
  pinned only to the documented stable semantics of ``lax.top_k`` /
  ``jnp.argsort`` (lower index first) and cross-checked against the
  sequential greedy simulator (``route_greedy``, also in C).
* ``softmax``, ``dense``, ``soft_router`` numerics: textbook definitions,
  checked against float64 closed forms; the exact bfloat16 rounding points of
  XLA are a library property and are PARITY UNPINNED (tolerance-checked only).
* ``mlp_block`` (expert MLP): arithmetic lives in the third-party module
  ``vit_jax.models_vit.MlpBlock`` (github.com/google-research/vision_transformer,
  un-pinned HEAD; call sites vmoe/nn/vit_moe.py:20,38-45), absent from the
  reference checkout.  Restated from its published definition
  (Dense -> tanh-GELU -> Dense).  PARITY UNPINNED beyond parameter shapes
  (vmoe/nn/vit_moe_test.py:66-73).
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Tuple

import numpy as np

F32 = "float32"
BF16 = "bfloat16"


# --------------------------------------------------------------------------- dtypes
def bf16_round(x) -> np.ndarray:
  """Rounds float32 values to the nearest bfloat16 (ties to even), kept as float32.

  Large arrays go through torch's CPU conversion, which is the same rounding
  (tests/test_oracle_golden.py::test_bf16_round_vs_torch) on all cores.
  """
  x = np.ascontiguousarray(x, dtype=np.float32)
  if x.size >= (1 << 20):
    import torch
    return torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
  return _bf16_round_numpy(x)


def _bf16_round_numpy(x: np.ndarray) -> np.ndarray:
  u = x.view(np.uint32)
  bias = ((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)
  r = ((u + bias) & np.uint32(0xFFFF0000)).view(np.float32)
  return np.where(np.isnan(x), x, r).astype(np.float32)


def cast(x, dtype: str) -> np.ndarray:
  """``x.astype(dtype)`` for the two dtypes of the path."""
  if dtype == BF16:
    return bf16_round(x)
  if dtype == F32:
    return np.asarray(x, dtype=np.float32)
  raise ValueError(f"Unsupported dtype {dtype!r}")


# --------------------------------------------------------------------------- capacity
def compute_capacity(num_tokens: int, num_experts: int, capacity_factor: float,
                     ceil_or_round: str = "ceil",
                     multiple_of: Optional[int] = 4) -> int:
  """vmoe/moe.py:230-257."""
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
  return capacity


# --------------------------------------------------------------------------- routing
def top_k(x: np.ndarray, k: int) -> Tuple[np.ndarray, np.ndarray]:
  """``jax.lax.top_k`` along the last axis: descending, ties -> lower index."""
  idx = np.argsort(-x, axis=-1, kind="stable")[..., :k]
  return np.take_along_axis(x, idx, axis=-1), idx.astype(np.int32)


def one_hot(idx: np.ndarray, n: int, dtype=np.int32) -> np.ndarray:
  """``jax.nn.one_hot``: indices outside [0, n) give an all-zero row."""
  return (np.asarray(idx)[..., None] == np.arange(n)).astype(dtype)


def top_experts_per_item_common(gates: np.ndarray, num_selected_experts: int,
                                batch_priority: bool):
  """vmoe/moe.py:547-590, literal one-hot / cumsum formulation, one group.

  Returns combine_weights (S,K), expert_index (S,K), buffer_index (S,K,E).
  """
  group_size, num_experts = gates.shape
  combine_weights, expert_index = top_k(gates, num_selected_experts)   # :567
  if batch_priority:
    perm = np.argsort(-combine_weights[:, 0], kind="stable")            # :571
    expert_index = expert_index[perm]                                   # :572
  expert_index = np.swapaxes(expert_index, 0, 1).ravel()                # :575
  expert_one_hot = one_hot(expert_index, num_experts, np.int32)         # :577
  buffer_index = np.cumsum(expert_one_hot, axis=0) * expert_one_hot - 1  # :580
  buffer_index = buffer_index.reshape(-1, group_size, num_experts)      # :581
  buffer_index = np.swapaxes(buffer_index, 0, 1)                        # :582
  expert_index = np.swapaxes(expert_index.reshape(-1, group_size), 0, 1)  # :584
  if batch_priority:
    inv_perm = np.argsort(perm, kind="stable")                          # :587
    expert_index = expert_index[inv_perm]
    buffer_index = buffer_index[inv_perm]
  return combine_weights, expert_index.astype(np.int32), buffer_index.astype(np.int32)


def top_experts_per_item_indices(gates: np.ndarray, num_selected_experts: int,
                                 batch_priority: bool):
  """vmoe/moe.py:626-652 for one group: indices (S,K,2) int32 (raw, unclipped
  positions) and combine weights (S,K)."""
  cw, expert_idx, buffer_idx = top_experts_per_item_common(
      gates, num_selected_experts, batch_priority)
  buffer_idx = buffer_idx.max(axis=2)                                   # :646
  return np.stack([expert_idx, buffer_idx], axis=-1).astype(np.int32), cw


def top_experts_per_item_einsum(gates: np.ndarray, num_selected_experts: int,
                                capacity: int, batch_priority: bool):
  """vmoe/moe.py:593-623 for one group: combine (S,E,C) and dispatch (S,E,C) bool."""
  _, _, buffer_idx = top_experts_per_item_common(
      gates, num_selected_experts, batch_priority)
  buffer_idx = buffer_idx.max(axis=1)                                   # :612
  dispatch_weights = one_hot(buffer_idx, capacity, np.bool_)            # :615
  combine_weights = gates[:, :, None] * dispatch_weights                # :618-619
  return combine_weights.astype(gates.dtype), dispatch_weights


def top_items_per_expert_einsum(gates: np.ndarray, capacity: int):
  """vmoe/moe.py:655-694 for one group (experts-choice routing)."""
  group_size, num_experts = gates.shape
  top_items_gates, top_items_index = top_k(gates.T, capacity)           # :671 (E,C)
  # one_hot(..., group_size, axis=0): (S, E, C)
  dispatch_weights = (np.arange(group_size)[:, None, None] ==
                      top_items_index[None, :, :])                      # :672
  combine_weights = gates[:, :, None] * dispatch_weights                # :676
  num_experts_per_item = dispatch_weights.sum(axis=(1, 2)).astype(np.int32)  # :682
  metrics = {
      "num_experts_per_item_min": num_experts_per_item.min(),
      "num_experts_per_item_max": num_experts_per_item.max(),
      "min_selected_gate": top_items_gates.min(),
      "max_selected_gate": top_items_gates.max(),
  }
  log2_num_experts = int(math.log2(num_experts))
  for t in [2**i for i in range(log2_num_experts + 1)] + [num_experts]:  # :690
    metrics[f"ratio_processed_items_by_at_least_{t}_experts"] = (
        np.sum(num_experts_per_item >= t) / group_size)
  return combine_weights.astype(gates.dtype), dispatch_weights, metrics


def route_greedy(expert_idx: np.ndarray, top1_gate: Optional[np.ndarray],
                 num_experts: int) -> np.ndarray:
  """Independent statement of the slot assignment: walk the K choice levels in
  order, inside each level walk items by priority (index order, or descending
  top-1 gate with index as tie break) and hand out per-expert counters.

  expert_idx (S,K) -> positions (S,K), raw (not clipped to capacity).  This is
  what the one-hot/cumsum of vmoe/moe.py:575-589 evaluates to; it shares no
  code with :func:`top_experts_per_item_common`.
  """
  S, K = expert_idx.shape
  if top1_gate is None:
    order = list(range(S))
  else:
    order = sorted(range(S), key=lambda s: (-float(top1_gate[s]), s))
  count = [0] * num_experts
  pos = np.zeros((S, K), np.int32)
  for k in range(K):
    for s in order:
      e = int(expert_idx[s, k])
      pos[s, k] = count[e]
      count[e] += 1
  return pos


# --------------------------------------------------------------------------- layout
def dispatch_layout(data: np.ndarray) -> np.ndarray:
  """vmoe/moe.py:488-500 without a mesh: (G,E,C,...) -> (E, G*C, ...)."""
  num_groups, num_experts, capacity, *item_shape = data.shape
  if num_groups % num_experts == 0:
    data = data.reshape(num_experts, -1, num_experts, capacity, *item_shape)
    data = np.swapaxes(data, 0, 2)
  else:
    data = np.swapaxes(data, 0, 1)
  data = data.reshape(-1, *item_shape)
  return data.reshape(num_experts, num_groups * capacity, *item_shape)


def receive_layout(data: np.ndarray, num_groups: int) -> np.ndarray:
  """vmoe/moe.py:503-519 without a mesh: (E, G*C, ...) -> (G,E,C,...)."""
  num_experts, gc, *item_shape = data.shape
  capacity = gc // num_groups
  data = data.reshape(num_experts * num_groups, capacity, *item_shape)
  if num_groups % num_experts == 0:
    data = data.reshape(num_experts, -1, num_experts, capacity, *item_shape)
    data = np.swapaxes(data, 0, 2)
    data = data.reshape(num_groups, num_experts, capacity, *item_shape)
  else:
    data = data.reshape(num_experts, num_groups, capacity, *item_shape)
    data = np.swapaxes(data, 0, 1)
  return data


def buffer_row(g: int, c: int, G: int, E: int, C: int) -> int:
  """Closed form of the row that slot (g, c) takes inside an expert's (G*C)
  buffer after :func:`dispatch_layout`."""
  if G % E == 0:
    q = G // E
    return ((g % q) * E + g // q) * C + c
  return g * C + c


def scatter_nd(indices: np.ndarray, updates: np.ndarray, shape) -> np.ndarray:
  """vmoe/moe.py:522-544: cumulative scatter, out-of-range rows dropped.

  Negative indices would wrap NumPy-style under JAX; routers never produce
  them and the oracle rejects them.
  """
  out = np.zeros(shape, updates.dtype)
  nd = len(shape)
  for row, upd in zip(indices.reshape(-1, nd), updates.reshape(-1, *updates.shape[1:])):
    if np.any(row < 0):
      raise ValueError("negative scatter index")
    if all(int(row[d]) < shape[d] for d in range(nd)):
      out[tuple(int(v) for v in row)] += upd
  return out


# --------------------------------------------------------------------------- dispatchers
class ExpertIndicesDispatcher:
  """vmoe/moe.py:164-209."""

  def __init__(self, indices, combine_weights, num_experts, capacity):
    self.indices = np.asarray(indices, np.int32)            # (G,S,K,2)
    self.combine_weights = np.asarray(combine_weights, np.float32)  # (G,S,K)
    self.num_experts = num_experts
    self.capacity = capacity

  def dispatch(self, data: np.ndarray) -> np.ndarray:
    G, S, K, _ = self.indices.shape
    item_shape = data.shape[2:]
    out = np.zeros((G, self.num_experts, self.capacity, *item_shape), data.dtype)
    e = self.indices[..., 0]
    c = self.indices[..., 1]
    if np.any(e < 0) or np.any(c < 0):
      raise ValueError("negative index")
    ok = (e < self.num_experts) & (c < self.capacity)
    g_i, s_i, k_i = np.nonzero(ok)
    # np.add.at accumulates duplicates, as .at[].add does (moe.py:526-527, :544).
    np.add.at(out, (g_i, e[g_i, s_i, k_i], c[g_i, s_i, k_i]), data[g_i, s_i])
    return dispatch_layout(out)

  def combine(self, data: np.ndarray) -> np.ndarray:
    G, S, K, _ = self.indices.shape
    data = receive_layout(data, G)                                       # :201
    e = self.indices[..., 0]
    c = self.indices[..., 1]
    mask = (e < self.num_experts) & (c < self.capacity)                  # :204-205
    e_c = np.clip(e, 0, self.num_experts - 1)   # gather clamps out-of-range
    c_c = np.clip(c, 0, self.capacity - 1)
    g_i = np.arange(G)[:, None, None]
    gathered = data[g_i, e_c, c_c]                                       # (G,S,K,...)
    extra = (1,) * (gathered.ndim - 3)
    gathered = gathered * mask.reshape(mask.shape + extra)               # :206
    w = self.combine_weights.reshape(self.combine_weights.shape + extra)
    # Precision.HIGHEST einsum (:208-209): float32 products and sums.
    return (gathered.astype(np.float32) * w).sum(axis=2).astype(np.float32)


class EinsumDispatcher:
  """vmoe/moe.py:127-161."""

  def __init__(self, combine_weights, dispatch_weights=None):
    self.combine_weights = np.asarray(combine_weights)      # (G,S,E,C)
    self.dispatch_weights = dispatch_weights

  def dispatch(self, data: np.ndarray) -> np.ndarray:
    dw = (self.combine_weights > 0 if self.dispatch_weights is None
          else self.dispatch_weights)                                    # :149-151
    G, S, E, C = dw.shape
    item_shape = data.shape[2:]
    flat = data.reshape(G, S, -1).astype(np.float32)
    out = np.matmul(np.asarray(dw, np.float32).reshape(G, S, E * C).transpose(0, 2, 1), flat)
    return dispatch_layout(out.reshape(G, E, C, *item_shape))            # :152-154

  def combine(self, data: np.ndarray) -> np.ndarray:
    G, S, E, C = self.combine_weights.shape
    data = receive_layout(data, G)                                       # :159
    item_shape = data.shape[3:]
    flat = data.reshape(G, E * C, -1).astype(np.float32)
    out = np.matmul(self.combine_weights.astype(np.float32).reshape(G, S, E * C), flat)
    return out.reshape(G, S, *item_shape)                                # :160


class DenseEinsumDispatcher:
  """vmoe/moe.py:93-124 (every item to every expert, C = S)."""

  def __init__(self, combine_weights):
    self.combine_weights = np.asarray(combine_weights)      # (G,S,E)

  def dispatch(self, data):
    G, S, E = self.combine_weights.shape
    out = np.broadcast_to(data[:, None], (G, E, *data.shape[1:])).astype(data.dtype)
    return dispatch_layout(out)

  def combine(self, data):
    G, S, E = self.combine_weights.shape
    data = receive_layout(data, G)       # (G,E,S,...)
    return np.einsum("GSE,GES...->GS...", self.combine_weights.astype(np.float32),
                     data.astype(np.float32))


class Bfloat16Dispatcher:
  """vmoe/moe.py:212-227: data is rounded to bfloat16 on the way in, the inner
  dispatcher sees bfloat16 data, and the result is cast back to the caller's
  dtype.  ``result_dtype`` models the dtype of the inner result *before* the
  cast back (bfloat16 when the weights are bfloat16 too, float32 otherwise)."""

  def __init__(self, dispatcher, inner_result_dtype: str = F32):
    self.dispatcher = dispatcher
    self.inner_result_dtype = inner_result_dtype

  def dispatch(self, data):
    return cast(self.dispatcher.dispatch(bf16_round(data)), self.inner_result_dtype)

  def combine(self, data):
    return cast(self.dispatcher.combine(bf16_round(data)), self.inner_result_dtype)


def get_top_experts_per_item_dispatcher(
    gates: np.ndarray, name: str, num_selected_experts: int, batch_priority: bool,
    capacity: Optional[int] = None, capacity_factor: Optional[float] = None,
    capacity_ceil_or_round: str = "ceil", capacity_multiple_of: Optional[int] = 4):
  """vmoe/moe.py:267-327 vmapped over the leading group axis, as
  vmoe/nn/routing.py:123-128 does.  gates: (G,S,E)."""
  if (capacity is None) == (capacity_factor is None):
    raise ValueError(
        "You must specify either 'capacity' or 'capacity_factor', and not both."
        f" Current values are capacity = {capacity!r}, "
        f"capacity_factor = {capacity_factor!r}")
  G, S, E = gates.shape
  if not capacity:
    capacity = compute_capacity(S * num_selected_experts, E, capacity_factor,
                                capacity_ceil_or_round, capacity_multiple_of)
  if name == "indices":
    res = [top_experts_per_item_indices(g, num_selected_experts, batch_priority)
           for g in gates]
    return ExpertIndicesDispatcher(np.stack([r[0] for r in res]),
                                   np.stack([r[1] for r in res]), E, capacity)
  if name == "einsum":
    res = [top_experts_per_item_einsum(g, num_selected_experts, capacity, batch_priority)
           for g in gates]
    return EinsumDispatcher(np.stack([r[0] for r in res]), np.stack([r[1] for r in res]))
  raise ValueError(f"Unknown dispatcher type: {name!r}")


# --------------------------------------------------------------------------- router
def softmax(x: np.ndarray, axis=-1) -> np.ndarray:
  """``jax.nn.softmax``: exp(x - max) / sum, float32 internals."""
  x = np.asarray(x, np.float32)
  u = np.exp(x - x.max(axis=axis, keepdims=True))
  return (u / u.sum(axis=axis, keepdims=True)).astype(np.float32)


def dense(x, kernel, bias, dtype: str) -> np.ndarray:
  """``flax.linen.Dense(dtype=dtype)``: operands cast to dtype, float32
  accumulation, result in dtype; bias added in dtype."""
  y = cast(np.matmul(cast(x, dtype), cast(kernel, dtype)), dtype)
  if bias is not None:
    y = cast(y + cast(bias, dtype), dtype)
  return y


def router_gates(x: np.ndarray, kernel: np.ndarray, dtype: str,
                 logit_bias: Optional[np.ndarray] = None) -> np.ndarray:
  """vmoe/nn/routing.py:71-80, deterministic branch: softmax(Dense(x)) in dtype.

  ``logit_bias`` is not part of the reference router (it has ``use_bias=False``);
  it exists for the benchmark configuration that skews the logits and is added
  in float32 before the softmax.
  """
  logits = dense(x, kernel, None, dtype)
  if logit_bias is not None:
    logits = cast(logits + np.asarray(logit_bias, np.float32), dtype)
  return cast(softmax(logits), dtype)


def importance_auxiliary_loss(gates: np.ndarray) -> np.float32:
  """vmoe/nn/routing.py:150-157, one group."""
  importance = gates.reshape(-1, gates.shape[-1]).astype(np.float32).sum(axis=0)
  return np.float32((importance.std() / importance.mean()) ** 2)


def gshard_auxiliary_loss(gates: np.ndarray) -> np.float32:
  """vmoe/nn/routing.py:133-148, one group."""
  _, num_experts = gates.shape
  mean_gates = gates.astype(np.float32).mean(axis=0)
  top1 = one_hot(np.argmax(gates, axis=1), num_experts, np.int32).mean(axis=0)
  return np.float32(np.mean(top1 * mean_gates) * num_experts ** 2)


def load_auxiliary_loss(logits, logits_noisy, noise_std, num_selected_experts):
  """vmoe/nn/routing.py:159-183 (training-time branch; kept for its golden)."""
  from scipy.stats import norm
  num_experts = logits_noisy.shape[-1]
  thr_idx = top_k(logits_noisy, num_selected_experts)[1][..., -1]
  thr = np.sum(one_hot(thr_idx, num_experts, np.float32) * logits_noisy, axis=-1)
  noise_required = (thr[..., None] - logits) / noise_std
  p = 1.0 - norm.cdf(noise_required)
  p_mean = p.mean(axis=0)
  return (p_mean.std() / p_mean.mean()) ** 2


def router_metrics(gates: np.ndarray, gshard_loss_weight: float = 0.0,
                   importance_loss_weight: float = 1.0) -> Dict[str, np.ndarray]:
  """vmoe/nn/routing.py:81-91 (+ _weighted_sum :247-252).  gates (G,S,E)."""
  imp = np.stack([importance_auxiliary_loss(g) for g in gates])
  gsh = np.stack([gshard_auxiliary_loss(g) for g in gates])
  aux = sum(x * w for w, x in ((gshard_loss_weight, gsh),
                               (importance_loss_weight, imp)) if w > 0)
  return {"auxiliary_loss": aux, "gshard_loss": gsh, "importance_loss": imp}


def noisy_top_experts_per_item_router(
    x, kernel, num_selected_experts, dispatcher_kwargs, dtype=F32,
    gshard_loss_weight=0.0, importance_loss_weight=1.0, logit_bias=None,
    noise=None, noise_std=1.0, load_loss_weight=1.0):
  """vmoe/nn/routing.py:55-60 + :62-131.  With ``noise`` None the deterministic
  branch; otherwise ``noise`` is the standard normal sample (G,S,E) that
  ``jax.random.normal`` would supply and the noisy branch (:92-114) runs."""
  if x.ndim != 3:
    raise ValueError(f"inputs.ndim must be 3, but it is {x.ndim}")
  num_experts = kernel.shape[-1]
  if not num_experts >= num_selected_experts >= 1:
    raise ValueError(f"num_experts >= num_selected_experts >= 1, but got "
                     f"num_experts = {num_experts} and "
                     f"num_selected_experts = {num_selected_experts}.")
  kw = dict(dispatcher_kwargs or {})
  use_bfloat16 = kw.pop("bfloat16", False)
  if noise is None:
    gates = router_gates(x, kernel, dtype, logit_bias)
    metrics = router_metrics(gates, gshard_loss_weight, importance_loss_weight)
  else:
    logits = dense(x, kernel, None, dtype)                                    # :73-74
    if logit_bias is not None:
      logits = cast(logits + np.asarray(logit_bias, np.float32), dtype)
    gates_clean = cast(softmax(logits), dtype)                                # :80
    imp = np.stack([importance_auxiliary_loss(g) for g in gates_clean])       # :81
    std = np.float32((1.0 / num_experts) * noise_std)                         # :93
    logits_noisy = (logits + std * np.asarray(noise, np.float32)).astype(np.float32)   # :94-96
    gates = softmax(logits_noisy)                                             # :97
    load = np.stack([load_auxiliary_loss(l, ln, std, num_selected_experts)
                     for l, ln in zip(logits, logits_noisy)]).astype(np.float32)  # :98-102
    gsh = np.stack([gshard_auxiliary_loss(g) for g in gates])                 # :103
    aux = sum(v * w for w, v in ((gshard_loss_weight, gsh), (importance_loss_weight, imp),
                                 (load_loss_weight, load)) if w > 0)
    metrics = {"auxiliary_loss": aux, "gshard_loss": gsh, "importance_loss": imp,
               "load_loss": load}
  dispatcher = get_top_experts_per_item_dispatcher(
      gates, num_selected_experts=num_selected_experts, **kw)
  if use_bfloat16:
    dispatcher = Bfloat16Dispatcher(dispatcher, inner_result_dtype=dtype)
  return dispatcher, metrics, gates


def ensemble_router(x, kernel, ensemble_size, num_selected_experts, dispatcher_kwargs,
                    dtype=F32, gshard_loss_weight=0.0, importance_loss_weight=1.0,
                    noises=None, noise_std=1.0, load_loss_weight=1.0):
  """vmoe/nn/ensemble_routing.py:73-134: x (G,S,D) with items ordered (S/M, M), kernel
  (D, M, E/M).  Member m routes items i*M+m inside experts m*E/M .. (m+1)*E/M - 1; the
  gating matrix is block diagonal and the losses have shape (G, M).  ``noises`` is a
  list of M standard normal samples (G, S/M, E/M) for the noisy branch."""
  if x.ndim != 3:
    raise ValueError(f"inputs.ndim must be 3, but it is {x.ndim}")
  G, S, D = x.shape
  M = ensemble_size
  _, m2, e_m = kernel.shape
  E = M * e_m
  if m2 != M or S % M != 0:
    raise ValueError("kernel / group size do not match the ensemble size")
  x4 = x.reshape(G, S // M, M, D)
  full = None
  per_member = []
  for m in range(M):
    _, metrics_m, gates_m = noisy_top_experts_per_item_router(
        x4[:, :, m, :], kernel[:, m, :], min(num_selected_experts, e_m),
        dict(name="indices", capacity=1, batch_priority=False), dtype, gshard_loss_weight,
        importance_loss_weight,
        noise=None if noises is None else noises[m], noise_std=noise_std,
        load_loss_weight=load_loss_weight)
    if full is None:
      full = np.zeros((G, S // M, M, M, e_m), gates_m.dtype)
    full[:, :, m, m, :] = gates_m
    per_member.append(metrics_m)
  gates = full.reshape(G, S, E)
  metrics = {k: np.stack([pm[k] for pm in per_member], axis=1) for k in per_member[0]}
  kw = dict(dispatcher_kwargs or {})
  use_bfloat16 = kw.pop("bfloat16", False)
  dispatcher = get_top_experts_per_item_dispatcher(
      gates, num_selected_experts=num_selected_experts, **kw)
  if use_bfloat16:
    dispatcher = Bfloat16Dispatcher(dispatcher, inner_result_dtype=dtype)
  return dispatcher, metrics, gates


# --------------------------------------------------------------------------- experts
def gelu(x: np.ndarray, approximate: bool = True) -> np.ndarray:
  """``flax.linen.gelu``: tanh form by default, erf form otherwise (float32)."""
  x = np.asarray(x, np.float32)
  if approximate:
    c = np.float32(math.sqrt(2.0 / math.pi))
    inner = c * (x + np.float32(0.044715) * (x * x * x))
    return (np.float32(0.5) * x * (np.float32(1.0) + np.tanh(inner))).astype(np.float32)
  from scipy.special import erf
  return (0.5 * x * (1.0 + erf(x / math.sqrt(2.0)))).astype(np.float32)


def mlp_block(x, w0, b0, w1, b1, dtype: str, approximate_gelu: bool = True):
  """vit_jax.models_vit.MlpBlock at inference (dropout off), applied per expert:
  x (E,R,D), w0 (E,D,M), b0 (E,M), w1 (E,M,D), b1 (E,D) -> (E,R,D).

  Call site: vmoe/nn/vit_moe.py:38-45 under the expert vmap of
  vmoe/moe.py:434-439.
  """
  h = dense(x, w0, None if b0 is None else b0[:, None, :], dtype)
  h = cast(gelu(h, approximate_gelu), dtype)
  return dense(h, w1, None if b1 is None else b1[:, None, :], dtype)


def sparse_moe(dispatcher, expert_fn, x):
  """vmoe/moe.py:429-444: dispatch -> experts over axis 0 -> combine."""
  return dispatcher.combine(expert_fn(dispatcher.dispatch(x)))


def mlp_moe_block(inputs, params, *, group_size, num_selected_experts,
                  dispatcher_kwargs, dtype=F32, logit_bias=None,
                  approximate_gelu=True, gshard_loss_weight=0.0,
                  importance_loss_weight=1.0):
  """vmoe/nn/vit_moe.py:101-124 with NoisyTopExpertsPerItemRouter (deterministic).

  params = {"Router": {"dense": {"kernel"}}, "Mlp": {"Dense_0": {"kernel","bias"},
  "Dense_1": {"kernel","bias"}}} with the expert axis leading in Mlp/*.
  Returns (outputs, metrics).
  """
  assert inputs.ndim == 3, f"Expected ndim = 3, but got shape {inputs.shape}"
  shape = inputs.shape
  x = cast(inputs, dtype).reshape(-1, group_size, shape[-1])             # :107
  dispatcher, metrics, _ = noisy_top_experts_per_item_router(
      x, params["Router"]["dense"]["kernel"], num_selected_experts,
      dispatcher_kwargs, dtype, gshard_loss_weight=gshard_loss_weight,
      importance_loss_weight=importance_loss_weight, logit_bias=logit_bias)
  mlp = params["Mlp"]
  fn = lambda buf: mlp_block(buf, mlp["Dense_0"]["kernel"], mlp["Dense_0"]["bias"],
                             mlp["Dense_1"]["kernel"], mlp["Dense_1"]["bias"], dtype,
                             approximate_gelu)
  out = cast(sparse_moe(dispatcher, fn, x), dtype)
  return out.reshape(*shape[:-1], out.shape[-1]), metrics                # :123


# --------------------------------------------------------------------------- Soft MoE
def normalize(x: np.ndarray, axis: int = -1, eps: float = 1e-6) -> np.ndarray:
  """vmoe/projects/soft_moe/router.py:36-38 (float32 internals)."""
  x = np.asarray(x, np.float32)
  m = 1.0 / np.sqrt(np.square(x).sum(axis=axis, keepdims=True, dtype=np.float32)
                    + np.float32(eps))
  return (x * m).astype(np.float32)


def soft_router_weights(inputs, mu, scale, dtype: str = F32):
  """vmoe/projects/soft_moe/router.py:56-96 without noise.

  inputs (G,m,D), mu (D,n,p), scale () -> logits, dispatch_weights, combine_weights,
  each (G,m,n,p), and the unit-norm mu.
  """
  x = cast(normalize(cast(inputs, dtype), axis=-1), dtype)               # :59
  mu_unit = cast(normalize(cast(mu, dtype), axis=0), dtype)              # :75
  s = cast(np.float32(scale), dtype)                                     # :78
  mu_s = mu_unit
  if x.size < mu_unit.size:                                              # :79-82
    x = cast(x * s, dtype)
  else:
    mu_s = cast(mu_unit * s, dtype)
  G, m, D = x.shape
  _, n, p = mu_s.shape
  logits = cast(np.matmul(x, mu_s.reshape(D, n * p)), dtype).reshape(G, m, n, p)  # :91
  dispatch_w = cast(softmax(logits, axis=1), dtype)                      # :94
  combine_w = cast(softmax(logits.reshape(G, m, n * p), axis=-1), dtype).reshape(G, m, n, p)  # :96
  return logits, dispatch_w, combine_w, mu_unit


def cosine_psim(x, batch_axes, contract_axes, eps: float = 1e-9):
  """vmoe/projects/soft_moe/router.py:170-182 (pairwise cosine similarity)."""
  x = np.asarray(x, np.float32)
  m = 1.0 / np.sqrt(np.square(x).sum(axis=tuple(contract_axes), keepdims=True) + eps)
  x = x * m
  nd = x.ndim
  batch_axes = tuple(a % nd for a in batch_axes)
  contract_axes = tuple(a % nd for a in contract_axes)
  free = tuple(a for a in range(nd) if a not in batch_axes and a not in contract_axes)
  xt = np.transpose(x, batch_axes + free + contract_axes)
  bshape = tuple(x.shape[a] for a in batch_axes)
  fshape = tuple(x.shape[a] for a in free)
  nb = int(np.prod(bshape)) if bshape else 1
  nf = int(np.prod(fshape)) if fshape else 1
  xm = xt.reshape(nb, nf, -1)
  out = np.matmul(xm, xm.transpose(0, 2, 1))
  return out.reshape(*bshape, *fshape, *fshape)


def soft_router_metrics(combine_weights, dispatch_weights, mu,
                        compute_similarity_metrics: bool = True):
  """vmoe/projects/soft_moe/router.py:112-167."""
  g, m, n, p = combine_weights.shape
  metrics = {
      "auxiliary_loss": np.float32(0.0),
      "combine_weights_min_mean": combine_weights.min(axis=(2, 3)).mean(),
      "combine_weights_max_mean": combine_weights.max(axis=(2, 3)).mean(),
      "dispatch_weights_min_mean": dispatch_weights.min(axis=1).mean(),
      "dispatch_weights_max_mean": dispatch_weights.max(axis=1).mean(),
  }
  if compute_similarity_metrics:
    cw_sim = cosine_psim(combine_weights, (0,), (2, 3))
    cw_id = np.eye(m)[None]
    cw_sim_masked = (1 - cw_id) * cw_sim
    cw_sim_masked = cw_sim_masked + cw_id * cw_sim_masked.max()
    metrics["combine_weights_similarity_min"] = cw_sim_masked.min()
    metrics["combine_weights_similarity_max"] = cw_sim_masked.max()
    metrics["combine_weights_similarity_mean"] = (cw_sim.sum() - g * m) / (g * m * (m - 1))
    dw_sim = cosine_psim(dispatch_weights, (0,), (1,))
    dw_id = np.eye(n * p)[None].reshape(1, n, p, n, p)
    dw_sim_masked = (1 - dw_id) * dw_sim
    dw_sim_masked = dw_sim_masked + dw_id * dw_sim_masked.max()
    metrics["dispatch_weights_similarity_min"] = dw_sim_masked.min()
    metrics["dispatch_weights_similarity_max"] = dw_sim_masked.max()
    metrics["dispatch_weights_similarity_mean"] = (
        (dw_sim.sum() - g * n * p) / (g * n * p * (n * p - 1)))
    mu_sim = cosine_psim(mu, (), (0,))
    mu_id = np.eye(n * p).reshape(n, p, n, p)
    mu_sim_masked = (1 - mu_id) * mu_sim
    mu_sim_masked = mu_sim_masked + mu_id * mu_sim_masked.max()
    metrics["mu_similarity_min"] = mu_sim_masked.min()
    metrics["mu_similarity_max"] = mu_sim_masked.max()
    metrics["mu_similarity_mean"] = (mu_sim.sum() - n * p) / (n * p * (n * p - 1))
  return metrics


def soft_router(inputs, mu, scale, dtype: str = F32,
                compute_similarity_metrics: bool = True):
  """vmoe/projects/soft_moe/router.py:56-102: (Bfloat16Dispatcher(EinsumDispatcher), metrics)."""
  _, dw, cw, mu_unit = soft_router_weights(inputs, mu, scale, dtype)
  dispatcher = Bfloat16Dispatcher(EinsumDispatcher(cw, dw), inner_result_dtype=dtype)
  return dispatcher, soft_router_metrics(cw, dw, mu_unit, compute_similarity_metrics)


def soft_num_slots(group_size: int, num_experts: int, num_slots: Optional[int],
                   capacity_factor: Optional[float]) -> int:
  """vmoe/projects/soft_moe/router.py:62-67."""
  if num_slots is None:
    return compute_capacity(group_size, num_experts, capacity_factor,
                            ceil_or_round="round", multiple_of=1)
  return num_slots
