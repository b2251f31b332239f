"""Functional wrappers of the C ABI: allocate outputs with torch, call the HIP kernels.

Each function maps to one entry point of include/vmoe_hip.h.  Tensors must live
on a ROCm device and are used as raw device pointers on torch's current stream.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional, Tuple

import torch

from vmoe_amd import _hip as H


def _i32(*shape, device):
  return torch.empty(shape, dtype=torch.int32, device=device)


def _f32(*shape, device):
  return torch.empty(shape, dtype=torch.float32, device=device)


def gate_topk(x: torch.Tensor, w: torch.Tensor, num_selected_experts: int,
              logit_bias: Optional[torch.Tensor] = None, return_gates: bool = True,
              return_logits: bool = False):
  """x (G,S,D), w (D,E) -> gates (G,S,E) or None, topk_val (G,S,K) f32, topk_idx (G,S,K) i32
  [, logits (G,S,E) f32 with return_logits]."""
  G, S, D = x.shape
  E = w.shape[1]
  K = num_selected_experts
  x = x.contiguous()
  w = w.to(x.dtype).contiguous()
  vec = 8 if x.dtype == torch.bfloat16 else 4
  if D % vec != 0:   # the kernel reads rows in 16-byte pieces: zero columns change nothing
    pad = vec - D % vec
    x = torch.nn.functional.pad(x, (0, pad))
    w = torch.nn.functional.pad(w, (0, 0, 0, pad))
    D += pad
  gates = torch.empty((G, S, E), dtype=x.dtype, device=x.device) if return_gates else None
  val = _f32(G, S, K, device=x.device)
  idx = _i32(G, S, K, device=x.device)
  if logit_bias is not None:
    logit_bias = logit_bias.to(torch.float32).contiguous()
  logits = _f32(G, S, E, device=x.device) if return_logits else None
  p = H.GateTopkParams(H.ptr(x), H.ptr(w), H.ptr(logit_bias), H.ptr(gates), H.ptr(val), H.ptr(idx),
                       G * S, D, E, K, H.dtype_code(x.dtype), H.ptr(logits))
  H.call("vmoe_gate_topk", p)
  if return_logits:
    return gates, val, idx, logits
  return gates, val, idx


def noisy_gates(logits: torch.Tensor, noise: torch.Tensor, noise_std: float,
                num_selected_experts: int, return_load_loss: bool = True):
  """logits, noise (G,S,E) f32 -> softmax(logits + noise_std * noise) (G,S,E) f32 and the
  load loss per group (G,) f32 (None if not asked for)."""
  G, S, E = logits.shape
  logits = logits.to(torch.float32).contiguous()
  noise = noise.to(torch.float32).contiguous()
  if noise.shape != logits.shape:
    raise ValueError(f"noise {tuple(noise.shape)} != logits {tuple(logits.shape)}")
  gates = torch.empty_like(logits)
  loss = _f32(G, device=logits.device) if return_load_loss else None
  p = H.NoisyGatesParams(H.ptr(logits), H.ptr(noise), H.ptr(gates), H.ptr(loss), G, S, E,
                         num_selected_experts, float(noise_std))
  H.call("vmoe_noisy_gates", p)
  return gates, loss


def topk(gates: torch.Tensor, k: int):
  """gates (..., E) float32 -> values (..., K) f32, indices (..., K) i32; ties -> lower index."""
  E = gates.shape[-1]
  g = gates.to(torch.float32).contiguous()
  n = g.numel() // E
  val = _f32(*gates.shape[:-1], k, device=g.device)
  idx = _i32(*gates.shape[:-1], k, device=g.device)
  H.call("vmoe_topk", H.TopkParams(H.ptr(g), H.ptr(val), H.ptr(idx), n, E, k))
  return val, idx


def router_metrics(gates: torch.Tensor, topk_idx: torch.Tensor, gshard_loss_weight: float,
                   importance_loss_weight: float):
  """gates (G,S,E), topk_idx (G,S,K) -> importance_loss, gshard_loss, auxiliary_loss, each (G,) f32."""
  G, S, E = gates.shape
  gates = gates.contiguous()
  topk_idx = topk_idx.contiguous()
  imp, gsh, aux = (_f32(G, device=gates.device) for _ in range(3))
  p = H.RouterMetricsParams(H.ptr(gates), H.ptr(topk_idx), H.ptr(imp), H.ptr(gsh), H.ptr(aux),
                            float(gshard_loss_weight), float(importance_loss_weight), G, S, E,
                            topk_idx.shape[-1], H.dtype_code(gates.dtype))
  H.call("vmoe_router_metrics", p)
  return imp, gsh, aux


_E_UNSUPPORTED = -6


def route_assign(topk_val: Optional[torch.Tensor], topk_idx: torch.Tensor, num_experts: int,
                 capacity: int, batch_priority: bool, metrics=None):
  """topk_idx (G,S,K) -> indices (G,S,K,2), token_slot (G,S,K), slot_token (E*G*C,), fill (G,E).

  With ``metrics=(gates (G,S,E), gshard_loss_weight, importance_loss_weight)`` the router's
  losses are computed in the same launch and a fifth result
  ``(importance_loss, gshard_loss, auxiliary_loss)`` is returned (what router_metrics gives)."""
  G, S, K = topk_idx.shape
  dev = topk_idx.device
  topk_idx = topk_idx.contiguous()
  if topk_val is not None:
    topk_val = topk_val.to(torch.float32).contiguous()
  indices = _i32(G, S, K, 2, device=dev)
  token_slot = _i32(G, S, K, device=dev)
  slot_token = _i32(num_experts * G * capacity, device=dev)
  fill = _i32(G, num_experts, device=dev)
  p = H.RouteAssignParams(H.ptr(topk_val), H.ptr(topk_idx), H.ptr(indices), H.ptr(token_slot),
                          H.ptr(slot_token), H.ptr(fill), G, S, num_experts, K, capacity,
                          int(bool(batch_priority)))
  if metrics is None:
    H.call("vmoe_route_assign", p)
    return indices, token_slot, slot_token, fill
  gates, gshard_loss_weight, importance_loss_weight = metrics
  if tuple(gates.shape) != (G, S, num_experts):
    raise ValueError(f"gates have shape {tuple(gates.shape)}, expected {(G, S, num_experts)}")
  gates = gates.contiguous()
  imp, gsh, aux = (_f32(G, device=dev) for _ in range(3))
  m = H.RouterMetricsParams(H.ptr(gates), H.ptr(topk_idx), H.ptr(imp), H.ptr(gsh), H.ptr(aux),
                            float(gshard_loss_weight), float(importance_loss_weight), G, S,
                            num_experts, K, H.dtype_code(gates.dtype))
  H.call2("vmoe_route_assign_metrics", p, m)
  return indices, token_slot, slot_token, fill, (imp, gsh, aux)


def top_items_per_expert(gates: torch.Tensor, capacity: int):
  """gates (G,S,E) -> indices (G,S,E,2), token_slot (G,S,E), slot_token (E*G*C,),
  weights (G,S,E) float32, sel_minmax (G,E,2) float32."""
  G, S, E = gates.shape
  dev = gates.device
  gates = gates.contiguous()
  indices = _i32(G, S, E, 2, device=dev)
  token_slot = _i32(G, S, E, device=dev)
  slot_token = _i32(E * G * capacity, device=dev)
  weights = torch.empty((G, S, E), dtype=torch.float32, device=dev)
  sel = torch.empty((G, E, 2), dtype=torch.float32, device=dev)
  p = H.TopItemsParams(H.ptr(gates), H.ptr(indices), H.ptr(token_slot), H.ptr(slot_token),
                       H.ptr(weights), H.ptr(sel), G, S, E, capacity, H.dtype_code(gates.dtype))
  H.call("vmoe_top_items_per_expert", p)
  return indices, token_slot, slot_token, weights, sel


def indices_to_slots(indices: torch.Tensor, num_experts: int, capacity: int):
  """indices (G,S,K,2) -> token_slot (G,S,K), slot_token (E*G*C,), counters (2,) [dups, invalid]."""
  G, S, K, _ = indices.shape
  dev = indices.device
  indices = indices.to(torch.int32).contiguous()
  token_slot = _i32(G, S, K, device=dev)
  slot_token = _i32(num_experts * G * capacity, device=dev)
  counters = torch.zeros(2, dtype=torch.int32, device=dev)
  p = H.IndicesToSlotsParams(H.ptr(indices), H.ptr(token_slot), H.ptr(slot_token),
                             H.c_void_p(counters.data_ptr()), H.c_void_p(counters.data_ptr() + 4),
                             G, S, num_experts, K, capacity)
  H.call("vmoe_indices_to_slots", p)
  return token_slot, slot_token, counters


def compact_rows(fill: torch.Tensor, token_slot: torch.Tensor, capacity: int):
  """fill (G,E), token_slot (G,S,K) -> token_row (G,S,K): the kept assignments of every
  expert renumbered into the first rows of its block; rows_per_expert (E,); row_token
  (E, G*C): the item in every packed row (rows past an expert's count are unset)."""
  G, E = fill.shape
  _, S, K = token_slot.shape
  token_row = _i32(G, S, K, device=fill.device)
  rows = _i32(E, device=fill.device)
  prefix = _i32(G, E, device=fill.device)
  row_token = _i32(E, G * capacity, device=fill.device)
  p = H.CompactRowsParams(H.ptr(fill), H.ptr(token_slot), H.ptr(token_row), H.ptr(rows),
                          H.ptr(prefix), H.ptr(row_token), G, S, E, K, capacity)
  H.call("vmoe_compact_rows", p)
  return token_row, rows, row_token


def dispatch(x: torch.Tensor, token_slot: torch.Tensor, slot_token: Optional[torch.Tensor],
             out: Optional[torch.Tensor] = None, num_slots: Optional[int] = None) -> torch.Tensor:
  """x (T,D), token_slot (T,K), slot_token (NS,) -> (NS, D).  With slot_token None (and
  num_slots given) unclaimed rows are left as allocated instead of zeroed."""
  T, D = x.shape
  K = token_slot.shape[-1]
  NS = slot_token.numel() if slot_token is not None else int(num_slots)
  x = x.contiguous()
  if out is None:
    out = torch.empty((NS, D), dtype=x.dtype, device=x.device)
  p = H.DispatchParams(H.ptr(x), H.ptr(token_slot), H.ptr(slot_token), H.ptr(out), T, NS, K, D,
                       H.dtype_code(x.dtype))
  H.call("vmoe_dispatch", p)
  return out


def combine(y: torch.Tensor, token_slot: torch.Tensor, weights: torch.Tensor,
            out: Optional[torch.Tensor] = None) -> torch.Tensor:
  """y (NS,D), token_slot (T,K), weights (T,K) f32 -> (T, D)."""
  NS, D = y.shape
  T, K = token_slot.shape
  y = y.contiguous()
  weights = weights.to(torch.float32).contiguous()
  if out is None:
    out = torch.empty((T, D), dtype=y.dtype, device=y.device)
  p = H.CombineParams(H.ptr(y), H.ptr(token_slot), H.ptr(weights), H.ptr(out), T, NS, K, D,
                      H.dtype_code(y.dtype))
  H.call("vmoe_combine", p)
  return out


def combine_backward_data(dout: torch.Tensor, token_slot: torch.Tensor, weights: torch.Tensor,
                          slot_token: Optional[torch.Tensor], num_slots: int) -> torch.Tensor:
  """dout (T,D) -> dy (NS,D): dy[slot(t,k)] = w[t,k] * dout[t]; unclaimed slots are zero when
  slot_token is given, unwritten otherwise."""
  T, D = dout.shape
  Kk = token_slot.shape[-1]
  dout = dout.contiguous()
  weights = weights.to(torch.float32).contiguous()
  dy = torch.empty((num_slots, D), dtype=dout.dtype, device=dout.device)
  p = H.CombineBackwardParams(H.ptr(dout), None, H.ptr(token_slot), H.ptr(weights),
                              H.ptr(slot_token), H.ptr(dy), None, T, num_slots, Kk, D,
                              H.dtype_code(dout.dtype))
  H.call("vmoe_combine_backward_data", p)
  return dy


def combine_backward_weights(dout: torch.Tensor, y: torch.Tensor,
                             token_slot: torch.Tensor) -> torch.Tensor:
  """dout (T,D), y (NS,D) -> dweights (T,K) f32: <dout[t], y[slot(t,k)]>, 0 where dropped."""
  T, D = dout.shape
  Kk = token_slot.shape[-1]
  dout, y = dout.contiguous(), y.contiguous()
  dw = _f32(T, Kk, device=dout.device)
  p = H.CombineBackwardParams(H.ptr(dout), H.ptr(y), H.ptr(token_slot), None, None, None,
                              H.ptr(dw), T, y.shape[0], Kk, D, H.dtype_code(dout.dtype))
  H.call("vmoe_combine_backward_weights", p)
  return dw


def densify(indices: torch.Tensor, weights: torch.Tensor, num_experts: int, capacity: int):
  """indices (G,S,K,2), weights (G,S,K) -> combine (G,S,E,C) f32, dispatch (G,S,E,C) bool."""
  G, S, K, _ = indices.shape
  dev = indices.device
  cw = torch.zeros((G, S, num_experts, capacity), dtype=torch.float32, device=dev)
  dw = torch.zeros((G, S, num_experts, capacity), dtype=torch.uint8, device=dev)
  weights = weights.to(torch.float32).contiguous()
  p = H.DensifyParams(H.ptr(indices.contiguous()), H.ptr(weights), H.ptr(cw), H.ptr(dw), G, S,
                      num_experts, K, capacity)
  H.call("vmoe_densify", p)
  return cw, dw.view(torch.bool)


def pack_expert_weights(w: torch.Tensor) -> torch.Tensor:
  """(E, rows, cols) -> (E, cols, rows), contiguous."""
  E, rows, cols = w.shape
  w = w.contiguous()
  out = torch.empty((E, cols, rows), dtype=w.dtype, device=w.device)
  p = H.TransposeParams(H.ptr(w), H.ptr(out), E, rows, cols, H.dtype_code(w.dtype))
  H.call("vmoe_pack_expert_weights", p)
  return out


def expert_mlp(x: torch.Tensor, w0, b0, w1, b1, w0t=None, w1t=None, approximate_gelu: bool = True,
               workspace: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
               rows_per_expert: Optional[torch.Tensor] = None,
               x_rows: Optional[torch.Tensor] = None, compact=None):
  """x (E,R,D) -> (E,R,D): gelu(x @ w0 + b0) @ w1 + b1 per expert; with rows_per_expert (E,)
  int32 only that many leading rows of every expert are computed.  With x_rows (E,R) int32,
  x is the (T,D) matrix of items and x_rows names the item of every row (gathered by the
  first product; see expert_mlp_can_gather).

  With ``compact=(fill (G,E), token_slot (G,S,K), capacity)`` x is the (T,D) matrix of items
  and the packed rows are computed here, in the launch that plans the products (what
  compact_rows gives is returned as well): -> (out, (token_row, rows_per_expert, row_token))."""
  maps = None
  if compact is not None:
    fill, token_slot, capacity = compact
    G, E = fill.shape
    _, S, K = token_slot.shape
    token_row = _i32(G, S, K, device=fill.device)
    rows_per_expert = _i32(E, device=fill.device)
    x_rows = _i32(E, G * capacity, device=fill.device)
    maps = (token_row, rows_per_expert, x_rows)
  num_items = 0
  if x_rows is not None:
    E, R = x_rows.shape
    num_items, D = x.shape
  else:
    E, R, D = x.shape
  M = (w0.shape[2] if w0 is not None else w0t.shape[1])
  x = x.contiguous()
  if out is None:
    out = torch.empty((E, R, D), dtype=x.dtype, device=x.device)
  p = H.ExpertMlpParams(H.ptr(x), H.ptr(w0), H.ptr(b0), H.ptr(w1), H.ptr(b1), H.ptr(w0t),
                        H.ptr(w1t), H.ptr(out), None, 0, E, R, D, M, H.dtype_code(x.dtype),
                        H.GELU_TANH if approximate_gelu else H.GELU_ERF, H.ptr(rows_per_expert),
                        H.ptr(x_rows), num_items)
  need = H.lib().vmoe_expert_mlp_workspace_bytes(H.ctypes.byref(p))
  if workspace is None or workspace.numel() * workspace.element_size() < need:
    workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
  p.workspace = H.ptr(workspace)
  p.workspace_bytes = workspace.numel() * workspace.element_size()
  _note_status_words(p, workspace)
  if compact is None:
    H.call("vmoe_expert_mlp", p)
    return out
  c = H.CompactRowsParams(H.ptr(fill), H.ptr(token_slot), H.ptr(maps[0]), H.ptr(maps[1]),
                          H.ptr(None), H.ptr(maps[2]), G, S, E, K, capacity)
  # (VMOE_PLAN_SEPARATE_LAUNCH=1 in the environment keeps the planning launch apart: the
  # switch behind the before / after figures)
  rc = _E_UNSUPPORTED
  if x.dtype == torch.bfloat16 and not os.environ.get("VMOE_PLAN_SEPARATE_LAUNCH"):   # float32 products keep no plan
    rc = H.call_blocks("vmoe_compact_rows_planned", c, p, accept=(_E_UNSUPPORTED,))
  if rc == 0:
    H.call("vmoe_expert_mlp_planned", p)
    global _last_planned
    _last_planned = (p, (x, w0, b0, w1, b1, w0t, w1t, out, workspace) + maps)
  else:
    c.prefix = H.ptr(_i32(G, E, device=fill.device))
    H.call("vmoe_compact_rows", c)
    H.call("vmoe_expert_mlp", p)
  return out, maps


_last_planned = None


def expert_mlp_replay_planned() -> torch.Tensor:
  """Issues vmoe_expert_mlp_planned again with the parameter block of the most recent
  expert_mlp(compact=...) call that planned its launches (same routing, same buffers: what a
  serving loop or a graph of the experts alone does) and returns that call's output tensor."""
  if _last_planned is None:
    raise RuntimeError("no planned expert_mlp call to repeat")
  p, keep = _last_planned
  H.call("vmoe_expert_mlp_planned", p)
  return keep[7]


_last_status_words: Optional[torch.Tensor] = None


def _note_status_words(p, workspace: torch.Tensor) -> None:
  """Remembers where the status words of this call's workspace are (vmoe_expert_mlp_status)."""
  global _last_status_words
  addr = ctypes.c_void_p()
  H.check(H.lib().vmoe_expert_mlp_status(ctypes.byref(p), ctypes.byref(addr)), "vmoe_expert_mlp_status")
  if not addr.value:
    _last_status_words = None
    return
  off = addr.value - workspace.data_ptr()
  flat = workspace.view(torch.uint8).reshape(-1)
  _last_status_words = flat[off:off + 4 * H.MLP_STATUS_WORDS].view(torch.int32)


def expert_mlp_status() -> Optional[Tuple[int, int]]:
  """(abandoned waits, plan mismatches) counted so far on the workspace of the most recent
  expert_mlp call (synchronises); None for float32.  Anything but (0, 0) means that some
  call on that workspace did not produce the product it should have."""
  if _last_status_words is None:
    return None
  words = _last_status_words.cpu()
  return int(words[H.MLP_STATUS_ABANDONED_WAITS]), int(words[H.MLP_STATUS_PLAN_MISMATCHES])


def expert_mlp_can_gather(dtype: torch.dtype, D: int, num_items: int) -> bool:
  """Whether expert_mlp can take the items themselves plus x_rows (no dispatched buffer)."""
  if dtype == torch.float32:
    return D % 32 == 0 and num_items * D * 4 < (1 << 31)
  return dtype == torch.bfloat16 and D % 32 == 0 and num_items * D * 2 < (1 << 32)


def expert_mlp_workspace_bytes(E, R, D, M, dtype, prepacked: bool) -> int:
  one = H.c_void_p(16)
  p = H.ExpertMlpParams(one, one, None, one, None, one if prepacked else None,
                        one if prepacked else None, one, None, 0, E, R, D, M,
                        H.dtype_code(dtype), 0)
  return int(H.lib().vmoe_expert_mlp_workspace_bytes(H.ctypes.byref(p)))


def soft_route(x: torch.Tensor, mu: torch.Tensor, scale: float, return_logits: bool = False,
               prepared: Optional[dict] = None, with_stats: bool = False):
  """x (G,S,D), mu (D,N) -> dispatch_w (G,S,N), combine_w (G,S,N) [, logits] [, stats].

  ``prepared``: a dict the caller keeps for as long as mu, scale, dtype and the shapes stay
  the same; the unit-norm, scaled slot parameters are computed on the first call, kept in
  it, and reused by the later ones.

  ``with_stats``: also the five scalars of soft_router_stats (a tuple of 0-dim float32
  tensors, last in the result), from the same call."""
  G, S, D = x.shape
  N = mu.shape[1]
  x = x.contiguous()
  mu = mu.to(x.dtype).contiguous()
  dw = torch.empty((G, S, N), dtype=x.dtype, device=x.device)
  cw = torch.empty_like(dw)
  logits = torch.empty_like(dw) if return_logits else None
  p = H.SoftRouteParams(H.ptr(x), H.ptr(mu), float(scale), H.ptr(dw), H.ptr(cw), H.ptr(logits),
                        None, 0, G, S, D, N, H.dtype_code(x.dtype), 0)
  key = (G, S, D, N, x.dtype, float(scale), str(x.device))
  ws = prepared.get(key) if prepared is not None else None
  if ws is None:
    need = H.lib().vmoe_soft_route_workspace_bytes(H.ctypes.byref(p))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=x.device)
    if prepared is not None:
      prepared.clear()
      prepared[key] = ws
  else:
    p.workspace_prepared = 1
  p.workspace = H.ptr(ws)
  p.workspace_bytes = ws.numel()
  out = (dw, cw, logits) if return_logits else (dw, cw)
  if not with_stats:
    H.call("vmoe_soft_route", p)
    return out
  buf = _f32(G * 4 + 8, device=x.device)
  stats = buf[G * 4:G * 4 + 5]
  H.call_blocks("vmoe_soft_route_stats", p, H.SoftStatsParams(
      H.ptr(cw), H.ptr(dw), H.ptr(buf), H.ptr(stats), G, S, N, H.dtype_code(x.dtype)))
  return out + ((stats[0], stats[1], stats[2], stats[3], stats[4]),)


def soft_router_stats(combine_w: torch.Tensor, dispatch_w: torch.Tensor):
  """combine_w, dispatch_w (G,S,N) -> the scalars of SoftRouter.get_metrics as 0-dim
  float32 tensors: (combine min-mean, combine max-mean, dispatch min-mean, dispatch
  max-mean, auxiliary loss = 0)."""
  G, S, N = combine_w.shape
  combine_w, dispatch_w = combine_w.contiguous(), dispatch_w.contiguous()
  buf = _f32(G * 4 + 8, device=combine_w.device)
  stats = buf[G * 4:G * 4 + 5]
  H.call("vmoe_soft_router_stats", H.SoftStatsParams(
      H.ptr(combine_w), H.ptr(dispatch_w), H.ptr(buf), H.ptr(stats), G, S, N,
      H.dtype_code(combine_w.dtype)))
  return stats[0], stats[1], stats[2], stats[3], stats[4]


def _w_code(w: torch.Tensor) -> int:
  if w.dtype == torch.float32:
    return H.W_F32
  if w.dtype == torch.bfloat16:
    return H.W_BF16
  if w.dtype == torch.bool:
    return H.W_BOOL
  raise TypeError(f"Unsupported weight dtype {w.dtype}")


def einsum_dispatch(w: torch.Tensor, data: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
  """w (G,S,E,C), data (G,S,D) -> (E*G*C, D) in the expert buffer's row order."""
  G, S, E, C = w.shape
  D = data.shape[-1]
  w = w.contiguous()
  data = data.contiguous()
  out = torch.empty((E * G * C, D), dtype=out_dtype, device=data.device)
  wv = w.view(torch.uint8) if w.dtype == torch.bool else w
  p = H.EinsumParams(H.ptr(wv), H.ptr(data), H.ptr(out), G, S, E, C, D, _w_code(w),
                     H.dtype_code(data.dtype), H.dtype_code(out_dtype))
  H.call("vmoe_einsum_dispatch", p)
  return out


def einsum_combine(w: torch.Tensor, data: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
  """w (G,S,E,C), data (E*G*C, D) -> (G,S,D)."""
  G, S, E, C = w.shape
  D = data.shape[-1]
  w = w.contiguous()
  data = data.contiguous()
  out = torch.empty((G, S, D), dtype=out_dtype, device=data.device)
  p = H.EinsumParams(H.ptr(w), H.ptr(data), H.ptr(out), G, S, E, C, D, _w_code(w),
                     H.dtype_code(data.dtype), H.dtype_code(out_dtype))
  H.call("vmoe_einsum_combine", p)
  return out


def cast(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
  """float32 <-> bfloat16 with the library's conversion kernel."""
  if x.dtype == dtype:
    return x
  x = x.contiguous()
  out = torch.empty(x.shape, dtype=dtype, device=x.device)
  if x.numel():
    p = H.CastParams(H.ptr(x), H.ptr(out), x.numel(), H.dtype_code(x.dtype), H.dtype_code(dtype))
    H.call("vmoe_cast", p)
  return out


def add_layer_norm(residual: torch.Tensor, branch: Optional[torch.Tensor],
                   scale: Optional[torch.Tensor], bias: Optional[torch.Tensor], eps: float,
                   out_dtype: Optional[torch.dtype], write_residual: bool = True):
  """x = residual (+ branch); returns (x as float32 or None, layer_norm(x) in out_dtype or None).

  residual (..., D) float32; branch the same shape, float32 or bfloat16, or None;
  out_dtype None skips the norm (add only).  Without a branch the residual itself
  is returned as x.
  """
  if residual.dtype != torch.float32:
    raise TypeError(f"residual must be float32, got {residual.dtype}")
  residual = residual.contiguous()
  D = residual.shape[-1]
  rows = residual.numel() // D
  dev = residual.device
  if branch is not None:
    if branch.shape != residual.shape:
      raise ValueError(f"branch {tuple(branch.shape)} != residual {tuple(residual.shape)}")
    branch = branch.contiguous()
  f32 = lambda t: None if t is None else t.to(torch.float32).contiguous()
  scale, bias = f32(scale), f32(bias)
  res_out = torch.empty_like(residual) if (branch is not None and write_residual) else None
  norm_out = None if out_dtype is None else torch.empty(residual.shape, dtype=out_dtype, device=dev)
  if res_out is None and norm_out is None:
    return residual, None
  optr = lambda t: None if t is None else H.ptr(t)
  p = H.AddLayerNormParams(
      H.ptr(residual), optr(branch), optr(scale), optr(bias), optr(res_out), optr(norm_out),
      rows, D, float(eps), H.dtype_code(branch.dtype) if branch is not None else 0,
      H.dtype_code(out_dtype) if out_dtype is not None else 0)
  H.call("vmoe_add_layer_norm", p)
  return (res_out if res_out is not None else residual), norm_out


ATTENTION_HEAD_DIM = 64


def attention_supported(q: torch.Tensor, k: torch.Tensor) -> bool:
  """Shapes the attention kernel covers: bfloat16, head size 64, keys and values
  of one head resident in LDS; (B, S, H, hd) views whose last two axes are contiguous."""
  if q.dtype != torch.bfloat16 or q.shape[-1] != ATTENTION_HEAD_DIM:
    return False
  sk_pad = (k.shape[1] + 31) // 32 * 32
  waves = min(8, (q.shape[1] + 31) // 32)
  lds = sk_pad * 144 + 64 * (sk_pad + 8) * 2 + waves * 32 * 80
  return lds <= 160 * 1024


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float) -> torch.Tensor:
  """softmax(q k^T * scale) v per (image, head).  q (B, Sq, H, hd), k, v (B, Sk, H, hd):
  views are fine as long as heads and head columns are contiguous (e.g. slices of a
  packed projection output).  Returns (B, Sq, H * hd)."""
  B, Sq, heads, hd = q.shape
  Sk = k.shape[1]
  for t in (q, k, v):
    if t.stride(3) != 1 or t.stride(2) != hd:
      raise H.VmoeError("attention operands need contiguous (H, hd) trailing axes")
  out = torch.empty((B, Sq, heads * hd), dtype=q.dtype, device=q.device)
  p = H.AttentionParams(
      ctypes.c_void_p(q.data_ptr()), ctypes.c_void_p(k.data_ptr()), ctypes.c_void_p(v.data_ptr()),
      H.ptr(out), q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1),
      B, heads, Sq, Sk, hd, float(scale), H.dtype_code(q.dtype))
  H.call("vmoe_attention", p)
  return out


def copy_bytes(src: torch.Tensor, dst: torch.Tensor) -> None:
  n = src.numel() * src.element_size()
  H.check(H.lib().vmoe_copy_bytes(H.ptr(src), H.ptr(dst), H.c_size_t(n), H.stream()),
          "vmoe_copy_bytes")


def operand_delivery_probe(a: torch.Tensor, bt: torch.Tensor, k_tile: int = 32) -> float:
  """Launches the load-only counterpart of the 256 x 256 product a (B, R, K) . bt (B, N, K)^T
  (bfloat16, contiguous); returns the operand bytes it moves (time it with events).
  k_tile = 32: 64-byte row segments per request (first product, plain second product);
  k_tile = 64: 128-byte segments (tile-walking second product)."""
  if k_tile not in (32, 64):
    raise ValueError("operand_delivery_probe: k_tile is 32 or 64")
  if a.dim() == 2:
    a, bt = a[None], bt[None]
  if a.dtype != torch.bfloat16 or bt.dtype != torch.bfloat16 or not (a.is_contiguous() and bt.is_contiguous()):
    raise ValueError("operand_delivery_probe: contiguous bfloat16 operands")
  if a.shape[0] != bt.shape[0] or a.shape[2] != bt.shape[2]:
    raise ValueError("operand_delivery_probe: a (B, R, K) and bt (B, N, K)")
  moved = H.ctypes.c_double(0.0)
  fn = H.lib().vmoe_operand_delivery_probe if k_tile == 32 else H.lib().vmoe_operand_delivery_probe_k64
  H.check(fn(H.ptr(a), H.ptr(bt), a.shape[0], a.shape[1], bt.shape[1], a.shape[2],
             H.ctypes.byref(moved), H.stream()), "vmoe_operand_delivery_probe")
  return float(moved.value)


def resident_delivery_probe(buf: torch.Tensor, row_bytes: int, k_tiles: int,
                            tiles_per_workgroup: int = 4, segment_bytes: int = 128) -> float:
  """Launches the load-only kernel whose 256 workgroups share the few tiles of 512 rows x
  row_bytes that `buf` (contiguous, any dtype) holds (few tiles: hardly a request waits for HBM);
  returns the bytes it moves into LDS (time it with events)."""
  moved = H.ctypes.c_double(0.0)
  n = buf.numel() * buf.element_size()
  H.check(H.lib().vmoe_resident_delivery_probe(H.ptr(buf), H.c_size_t(n), row_bytes, k_tiles,
                                               tiles_per_workgroup, segment_bytes,
                                               H.ctypes.byref(moved), H.stream()),
          "vmoe_resident_delivery_probe")
  return float(moved.value)


def mfma_probe(seed: torch.Tensor, blocks: int = 256, iters: int = 2000) -> float:
  """Launches the register-resident MFMA loop on operands read from `seed`;
  returns the floating-point operations it issues (time it with events)."""
  sink = torch.empty(blocks * 256, dtype=torch.float32, device=seed.device)
  flops = H.ctypes.c_double(0.0)
  n = seed.numel() * seed.element_size()
  H.check(H.lib().vmoe_mfma_probe(H.ptr(seed), H.c_size_t(n), H.ptr(sink), blocks, iters,
                                  H.ctypes.byref(flops), H.stream()), "vmoe_mfma_probe")
  return float(flops.value)
