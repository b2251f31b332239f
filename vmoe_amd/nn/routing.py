"""Routers of the MoE layer on HIP kernels; host-side mirror of vmoe/nn/routing.py.

A router is called on (G, S, D) inputs and returns ``(dispatcher, metrics)``.
"""
from __future__ import annotations

from typing import Any, Dict, Mapping, Optional, Tuple

import torch

import vmoe_amd.moe
from vmoe_amd import kernels as K
from vmoe_amd.nn import module

Array = torch.Tensor
BaseDispatcher = vmoe_amd.moe.BaseDispatcher
KwArgs = Mapping[str, Any]
Metrics = Mapping[str, Array]


class NoisyTopExpertsPerItemRouter(module.Module):
  """Top-K experts per item with optional Batch Priority Routing; vmoe/nn/routing.py:31-183.

  Parameters: ``{'dense': {'kernel': (D, E)}}``.  With ``deterministic=True`` or
  ``noise_std == 0`` the gates are the softmax of the logits; otherwise
  ``apply(variables, inputs, rngs={'gating': seed or torch.Generator})`` adds
  normal noise of standard deviation ``noise_std / num_experts`` to the logits and
  reports the load loss as well (forward only: there is no backward pass here).

  ``logit_bias`` (not in the reference, whose gating layer has no bias) adds a
  fixed float32 (E,) vector to the logits before the softmax; it exists for the
  benchmark configuration that skews the expert load.
  """
  _fields = dict(num_experts=module._REQUIRED, num_selected_experts=1, noise_std=1.0,
                 gshard_loss_weight=0.0, importance_loss_weight=1.0, load_loss_weight=1.0,
                 dispatcher=None, deterministic=False, dtype=None, logit_bias=None)

  def init(self, rng, inputs: Array):
    gen = module.generator(rng)
    D = inputs.shape[-1]
    kernel = module.lecun_normal(gen, (D, self.num_experts), fan_in=D, device=inputs.device)
    return {"params": {"dense": {"kernel": kernel}}}

  def apply(self, variables, inputs: Array, rngs=None) -> Tuple[BaseDispatcher, Metrics]:
    kernel = variables["params"]["dense"]["kernel"]
    if self.deterministic or self.noise_std == 0.0:
      # The losses run as extra workgroups of the slot-assignment launch.
      gates, _, topk = self._compute_gates_softmax_and_metrics(inputs, kernel, rngs,
                                                               with_metrics=False)
      metrics = {}
      dispatcher = self._create_dispatcher(
          gates, topk, _metrics=(self.gshard_loss_weight, self.importance_loss_weight, metrics))
      if not metrics:   # a dispatcher that does not come from the slot-assignment kernel
        metrics["importance_loss"], metrics["gshard_loss"], metrics["auxiliary_loss"] = (
            K.router_metrics(gates, topk[1], self.gshard_loss_weight, self.importance_loss_weight))
      return dispatcher, {k: metrics[k] for k in ("auxiliary_loss", "gshard_loss", "importance_loss")}
    gates, metrics, topk = self._compute_gates_softmax_and_metrics(inputs, kernel, rngs)
    dispatcher = self._create_dispatcher(gates, topk)
    return dispatcher, metrics

  def _compute_gates_softmax_and_metrics(self, inputs: Array, kernel: Array, rngs=None,
                                         num_experts: Optional[int] = None,
                                         with_metrics: bool = True):
    num_experts = self.num_experts if num_experts is None else num_experts
    if inputs.ndim != 3:
      raise ValueError(f"inputs.ndim must be 3, but it is {inputs.ndim}")
    if not num_experts >= self.num_selected_experts >= 1:
      raise ValueError(f"num_experts >= num_selected_experts >= 1, but got "
                       f"num_experts = {num_experts} and "
                       f"num_selected_experts = {self.num_selected_experts}.")
    if kernel.shape != (inputs.shape[-1], num_experts):
      raise ValueError(f"Router kernel has shape {tuple(kernel.shape)}, expected "
                       f"{(inputs.shape[-1], num_experts)}")
    module.require_no_grad(type(self).__name__, inputs, kernel)
    dtype = self.dtype or inputs.dtype
    x = K.cast(inputs, dtype)
    w = self._cast_kernel(kernel, dtype)
    if self.deterministic or self.noise_std == 0.0:
      gates, val, idx = K.gate_topk(x, w, self.num_selected_experts, logit_bias=self.logit_bias)
      if not with_metrics:
        return gates, None, (val, idx)
      importance_loss, gshard_loss, auxiliary_loss = K.router_metrics(
          gates, idx, self.gshard_loss_weight, self.importance_loss_weight)
      metrics = {
          "auxiliary_loss": auxiliary_loss,
          "gshard_loss": gshard_loss,
          "importance_loss": importance_loss,
      }
      return gates, metrics, (val, idx)
    # Noisy branch, vmoe/nn/routing.py:92-114: the importance loss comes from the
    # clean gates, everything else from the gates of the noisy logits.
    noise_std = (1.0 / num_experts) * self.noise_std
    gates, _, top1, logits = K.gate_topk(x, w, 1, logit_bias=self.logit_bias, return_logits=True)
    noise = _gating_noise(rngs, logits.shape, logits.device)
    gates_noisy, load_loss = K.noisy_gates(logits, noise, noise_std, self.num_selected_experts)
    val, idx = K.topk(gates_noisy, self.num_selected_experts)
    importance_loss, _, _ = K.router_metrics(gates, top1, 0.0, 1.0)
    _, gshard_loss, _ = K.router_metrics(gates_noisy, idx, 1.0, 0.0)
    metrics = {
        "auxiliary_loss": _weighted_sum((self.gshard_loss_weight, gshard_loss),
                                        (self.importance_loss_weight, importance_loss),
                                        (self.load_loss_weight, load_loss)),
        "gshard_loss": gshard_loss,
        "importance_loss": importance_loss,
        "load_loss": load_loss,
    }
    return gates_noisy, metrics, (val, idx)

  def _cast_kernel(self, kernel: Array, dtype) -> Array:
    """The router kernel in the compute dtype; the cast of a parameter tensor is
    done once and reused until the tensor changes."""
    if kernel.dtype == dtype:
      return kernel
    cache = self.__dict__.setdefault("_kernel_cache", module.ParamCache())
    return cache.get((kernel,), dtype, lambda: K.cast(kernel, dtype))

  def _create_dispatcher(self, gates_dispatch: Array, topk=None, _metrics=None):
    dispatcher_kwargs = dict(**(self.dispatcher or {}))
    use_bfloat16 = dispatcher_kwargs.pop("bfloat16", False)
    dispatcher = vmoe_amd.moe.get_top_experts_per_item_dispatcher(
        gates_dispatch, num_selected_experts=self.num_selected_experts, _topk=topk,
        _metrics=_metrics, **dispatcher_kwargs)
    if use_bfloat16:
      dispatcher = vmoe_amd.moe.Bfloat16Dispatcher(dispatcher)
    return dispatcher


class NoisyTopItemsPerExpertRouter(module.Module):
  """Experts-choice router: every expert picks its top-C items; vmoe/nn/routing.py:186-244.

  Parameters: ``{'dense': {'kernel': (D, E)}}``.  The noisy branch takes
  ``rngs={'gating': seed or torch.Generator}`` like the top-experts router.
  """
  _fields = dict(num_experts=module._REQUIRED, noise_std=1.0, dispatcher=None,
                 deterministic=False, dtype=None)

  def init(self, rng, inputs: Array):
    gen = module.generator(rng)
    D = inputs.shape[-1]
    kernel = module.lecun_normal(gen, (D, self.num_experts), fan_in=D, device=inputs.device)
    return {"params": {"dense": {"kernel": kernel}}}

  def apply(self, variables, inputs: Array, rngs=None) -> Tuple[BaseDispatcher, Metrics]:
    kernel = variables["params"]["dense"]["kernel"]
    gates_softmax = self._compute_gates_softmax(inputs, kernel, rngs)
    dispatcher, metrics = self._create_dispatcher_and_metrics(gates_softmax)
    metrics["auxiliary_loss"] = 0.
    return dispatcher, metrics

  def _compute_gates_softmax(self, inputs: Array, kernel: Array, rngs=None) -> Array:
    if inputs.ndim != 3:
      raise ValueError(f"inputs.ndim must be 3, but it is {inputs.ndim}")
    if kernel.shape != (inputs.shape[-1], self.num_experts):
      raise ValueError(f"Router kernel has shape {tuple(kernel.shape)}, expected "
                       f"{(inputs.shape[-1], self.num_experts)}")
    module.require_no_grad(type(self).__name__, inputs, kernel)
    dtype = self.dtype or inputs.dtype
    if self.deterministic or self.noise_std == 0.0:
      gates, _, _ = K.gate_topk(K.cast(inputs, dtype), K.cast(kernel, dtype), 1)
      return gates
    # vmoe/nn/routing.py:226-232
    noise_std = (1.0 / self.num_experts) * self.noise_std
    _, _, _, logits = K.gate_topk(K.cast(inputs, dtype), K.cast(kernel, dtype), 1,
                                  return_gates=False, return_logits=True)
    noise = _gating_noise(rngs, logits.shape, logits.device)
    gates_noisy, _ = K.noisy_gates(logits, noise, noise_std, 1, return_load_loss=False)
    return gates_noisy

  def _create_dispatcher_and_metrics(self, gates_dispatch: Array):
    dispatcher_kwargs = dict(**(self.dispatcher or {}))
    use_bfloat16 = dispatcher_kwargs.pop("bfloat16", False)
    dispatcher, metrics = vmoe_amd.moe.get_top_items_per_expert_dispatcher(
        gates_dispatch, **dispatcher_kwargs)
    if use_bfloat16:
      dispatcher = vmoe_amd.moe.Bfloat16Dispatcher(dispatcher)
    return dispatcher, metrics


def _gating_noise(rngs, shape, device) -> Array:
  """Standard normal noise from ``rngs['gating']`` (a seed or a torch.Generator on the
  device): what ``jax.random.normal(self.make_rng('gating'), shape)`` is in the
  reference.  The distribution is the same, the random stream is torch's."""
  rng = (rngs or {}).get("gating")
  if rng is None:
    raise ValueError("The noisy branch of the router needs rngs={'gating': seed or "
                     "torch.Generator}; use deterministic=True or noise_std=0 for inference.")
  gen = module.make_rngs({"gating": rng}, device)["gating"]
  return torch.randn(tuple(shape), generator=gen, device=device, dtype=torch.float32)


def _weighted_sum(*args):
  """Weighted sum of [(weight, element), ...] for weights > 0; vmoe/nn/routing.py:247-252."""
  return sum(x * w for w, x in args if w > 0)
