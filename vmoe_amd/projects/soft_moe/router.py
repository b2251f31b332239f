"""Soft MoE router on HIP kernels; host-side mirror of vmoe/projects/soft_moe/router.py."""
from __future__ import annotations

import logging
from typing import Dict, Optional, Tuple

import torch

from vmoe_amd import kernels as K
from vmoe_amd import moe
from vmoe_amd.nn import module

Array = torch.Tensor
BaseDispatcher = moe.BaseDispatcher
Bfloat16Dispatcher = moe.Bfloat16Dispatcher
EinsumDispatcher = moe.EinsumDispatcher


class SoftRouter(module.Module):
  """Soft router merging tokens as inputs/outputs of the experts; router.py:41-167.

  Parameters: ``{'mu': (D, num_experts, num_slots), 'scale': ()}``.  Noise is a
  training-time feature and is not implemented (noise_std must be 0 or
  deterministic=True).  The pairwise-similarity metrics
  (``compute_similarity_metrics``) are monitoring values computed with torch ops.
  """
  _fields = dict(num_experts=module._REQUIRED, num_slots=None, capacity_factor=1.0,
                 noise_std=0.0, deterministic=False, dtype=None, precision=None,
                 partition_spec=None, compute_similarity_metrics=True)

  def _num_slots(self, group_size: int) -> int:
    if self.num_slots is None:
      return moe.compute_capacity(group_size, self.num_experts, self.capacity_factor,
                                  ceil_or_round="round", multiple_of=1)
    actual_capacity_factor = self.num_experts * self.num_slots / group_size
    pre = f"{self.capacity_factor=} ignored. " if self.capacity_factor else ""
    logging.info("%sWith num_tokens=%d, num_experts=%d and num_slots=%d, the actual "
                 "capacity_factor is %f.", pre, group_size, self.num_experts, self.num_slots,
                 actual_capacity_factor)
    return self.num_slots

  def init(self, rng, inputs: Array):
    _, group_size, dim = inputs.shape
    num_slots = self._num_slots(group_size)
    gen = module.generator(rng)
    # lecun_normal on (dim, n, p): fan_in is the product of all but the last axis.
    mu = module.lecun_normal(gen, (dim, self.num_experts, num_slots),
                             fan_in=dim * self.num_experts, device=inputs.device)
    scale = torch.ones((), dtype=torch.float32, device=inputs.device)
    return {"params": {"mu": mu, "scale": scale}}

  def apply(self, variables, inputs: Array) -> Tuple[BaseDispatcher, Dict[str, Array]]:
    if not self.deterministic and self.noise_std > 0:
      raise NotImplementedError("Router noise is a training-time feature and is not implemented.")
    p = variables["params"]
    module.require_no_grad("SoftRouter", inputs, p["mu"], p["scale"])
    dtype = self.dtype or inputs.dtype
    x = K.cast(inputs, dtype)
    G, m, dim = x.shape
    num_slots = self._num_slots(m)
    mu = p["mu"]
    if tuple(mu.shape) != (dim, self.num_experts, num_slots):
      raise ValueError(f"mu has shape {tuple(mu.shape)}, expected {(dim, self.num_experts, num_slots)}")
    n, s = self.num_experts, num_slots
    mu_c = self._cast_mu(mu, dtype)
    # (the routing call also returns the scalars of get_metrics that come from the weights)
    dw, cw, scalars = K.soft_route(x, mu_c.reshape(dim, n * s), self._scale_value(p["scale"]),
                                   prepared=self._prepared_mu(mu_c, p["scale"]), with_stats=True)
    dispatch_weights = dw.view(G, m, n, s)
    combine_weights = cw.view(G, m, n, s)
    dispatcher = EinsumDispatcher(combine_weights, dispatch_weights,
                                  partition_spec=self.partition_spec,
                                  einsum_precision=self.precision)
    dispatcher = Bfloat16Dispatcher(dispatcher)
    metrics = self.get_metrics(combine_weights, dispatch_weights, mu_c, scalars=scalars)
    return dispatcher, metrics

  def _cast_mu(self, mu: Array, dtype) -> Array:
    """The slot parameters in the compute dtype, cast once per parameter tensor."""
    if mu.dtype == dtype:
      return mu
    cache = self.__dict__.setdefault("_mu_cache", module.ParamCache())
    return cache.get((mu,), dtype, lambda: K.cast(mu, dtype))

  def _prepared_mu(self, mu_c: Array, scale) -> dict:
    """Holder of the normalised, scaled slot parameters of this (mu, scale) pair: they are
    computed by the first call and reused until either tensor changes."""
    cache = self.__dict__.setdefault("_prepared_cache", module.ParamCache())
    tensors = (mu_c, scale) if isinstance(scale, torch.Tensor) else (mu_c,)
    return cache.get(tensors, "prepared", dict)

  def _scale_value(self, scale) -> float:
    """The scalar parameter as a host float.  Reading a device scalar waits for the
    stream, so it is read once per parameter tensor (and again if it is modified)."""
    if not isinstance(scale, torch.Tensor):
      return float(scale)
    cache = self.__dict__.setdefault("_scale_cache", module.ParamCache())
    return cache.get((scale,), "scale", lambda: float(scale))

  def get_metrics(self, combine_weights: Array, dispatch_weights: Array, mu: Array, scalars=None):
    """router.py:112-167.  Monitoring scalars; mu is normalised inside cosine_psim.
    ``scalars``: the five scalars of the weights where the routing call already took them."""
    g, m, n, p = combine_weights.shape
    if scalars is not None:
      cmin, cmax, dmin, dmax, aux = scalars
    elif combine_weights.is_cuda and combine_weights.dtype in (torch.float32, torch.bfloat16):
      cmin, cmax, dmin, dmax, aux = K.soft_router_stats(
          combine_weights.reshape(g, m, n * p), dispatch_weights.reshape(g, m, n * p))
    else:
      aux = torch.zeros((), dtype=torch.float32, device=combine_weights.device)
      cwf, dwf = combine_weights.float(), dispatch_weights.float()
      cmin, cmax = cwf.amin(dim=(2, 3)).mean(), cwf.amax(dim=(2, 3)).mean()
      dmin, dmax = dwf.amin(dim=1).mean(), dwf.amax(dim=1).mean()
    metrics = {
        "auxiliary_loss": aux,
        "combine_weights_min_mean": cmin,
        "combine_weights_max_mean": cmax,
        "dispatch_weights_min_mean": dmin,
        "dispatch_weights_max_mean": dmax,
    }
    if self.compute_similarity_metrics:
      cwf, dwf = combine_weights.float(), dispatch_weights.float()
      def masked(sim, eye):
        mk = (1 - eye) * sim
        return mk + eye * mk.max()
      cw_sim = cosine_psim(cwf, (0,), (2, 3))
      cw_m = masked(cw_sim, torch.eye(m, device=cwf.device)[None])
      metrics["combine_weights_similarity_min"] = cw_m.min()
      metrics["combine_weights_similarity_max"] = cw_m.max()
      metrics["combine_weights_similarity_mean"] = (cw_sim.sum() - g * m) / (g * m * (m - 1))
      dw_sim = cosine_psim(dwf, (0,), (1,))
      dw_m = masked(dw_sim, torch.eye(n * p, device=cwf.device).reshape(1, n, p, n, p))
      metrics["dispatch_weights_similarity_min"] = dw_m.min()
      metrics["dispatch_weights_similarity_max"] = dw_m.max()
      metrics["dispatch_weights_similarity_mean"] = (
          (dw_sim.sum() - g * n * p) / (g * n * p * (n * p - 1)))
      assert mu.ndim == 3 and tuple(mu.shape[1:]) == (n, p)
      mu_sim = cosine_psim(mu.float(), (), (0,))
      mu_m = masked(mu_sim, torch.eye(n * p, device=cwf.device).reshape(n, p, n, p))
      metrics["mu_similarity_min"] = mu_m.min()
      metrics["mu_similarity_max"] = mu_m.max()
      metrics["mu_similarity_mean"] = (mu_sim.sum() - n * p) / (n * p * (n * p - 1))
    return metrics


def normalize(x: Array, axis: int = -1, eps: float = 1e-6) -> Array:
  """router.py:36-38 (host-side helper; the router itself normalises in the kernel)."""
  m = torch.rsqrt(torch.square(x).sum(dim=axis, keepdim=True) + eps)
  return x * m


def cosine_psim(x: Array, batch_axes, contract_axes, precision=None, eps: float = 1e-9) -> Array:
  """Pairwise cosine similarity over arbitrary axes; router.py:170-182."""
  del precision
  nd = x.ndim
  batch_axes = tuple(a % nd for a in batch_axes)
  contract_axes = tuple(a % nd for a in contract_axes)
  m = torch.rsqrt(torch.square(x).sum(dim=contract_axes, keepdim=True) + eps)
  x = x * m
  free = tuple(a for a in range(nd) if a not in batch_axes and a not in contract_axes)
  xt = x.permute(*batch_axes, *free, *contract_axes)
  bshape = tuple(x.shape[a] for a in batch_axes)
  fshape = tuple(x.shape[a] for a in free)
  xm = xt.reshape(max(1, int(torch.tensor(bshape).prod()) if bshape else 1), -1,
                  int(torch.tensor([x.shape[a] for a in contract_axes]).prod()))
  out = torch.matmul(xm, xm.transpose(1, 2).contiguous())
  return out.reshape(*bshape, *fshape, *fshape)
