"""Router for ensembles of experts; host-side mirror of vmoe/nn/ensemble_routing.py.

The batch is assumed to be repeated M times (``ensemble_size``) and the E experts
are split into M subsets: the m-th copy of an input can only be routed inside the
m-th subset, i.e. the gating matrix is block diagonal."""
from __future__ import annotations

from typing import Mapping, Tuple

import torch

from vmoe_amd.nn import module
from vmoe_amd.nn import routing

Array = torch.Tensor
BaseDispatcher = routing.BaseDispatcher
Metrics = Mapping[str, Array]


def reshape_to_group_size_representation(x: Array, group_size: int, ensemble_size: int) -> Array:
  """Keeps the repeat-ensemble structure in each of the G groups; ensemble_routing.py:43-53."""
  batch_size_with_repeat, num_tokens_per_image, hidden_size = x.shape
  batch_size = batch_size_with_repeat // ensemble_size
  # (B * M, T, H) -> (B, M, T, H) -> (B, T, M, H) -> (G, S, H).
  x = x.reshape(batch_size, ensemble_size, num_tokens_per_image, hidden_size)
  x = x.transpose(1, 2)
  return x.reshape(-1, group_size, hidden_size)


def reshape_from_group_size_representation(x: Array, num_tokens_per_image: int,
                                           ensemble_size: int) -> Array:
  """Back to the repeat-ensemble structure at the image level; ensemble_routing.py:56-65."""
  hidden_size = x.shape[2]
  # (G, S, H) -> (B, T, M, H) -> (B, M, T, H) -> (B * M, T, H).
  x = x.reshape(-1, num_tokens_per_image, ensemble_size, hidden_size)
  x = x.transpose(1, 2)
  return x.reshape(-1, num_tokens_per_image, hidden_size)


def reshape_from_diag_blocks(diagonal_blocks: Array) -> Array:
  """(G, M, R, C) blocks -> (G, M * R, M * C) block-diagonal matrices; ensemble_routing.py:68-70."""
  G, M, R, C = diagonal_blocks.shape
  out = diagonal_blocks.new_zeros((G, M, R, M, C))
  for m in range(M):
    out[:, m, :, m, :] = diagonal_blocks[:, m]
  return out.reshape(G, M * R, M * C)


class NoisyTopExpertsPerItemEnsembleRouter(routing.NoisyTopExpertsPerItemRouter):
  """vmoe/nn/ensemble_routing.py:73-134.

  Parameters: ``{'dense': {'kernel': (D, M, E / M)}}`` (the members' gating layers stacked
  on axis 1).  Group items are ordered (S / M, M): item ``i * M + m`` belongs to member m.
  The losses in the metrics have shape (G, M).
  """
  _fields = dict(ensemble_size=1)

  def init(self, rng, inputs: Array):
    gen = module.generator(rng)
    D, M = inputs.shape[-1], self.ensemble_size
    kernel = module.lecun_normal(gen, (D, M, self.num_experts // M), fan_in=D,
                                 device=inputs.device)
    return {"params": {"dense": {"kernel": kernel}}}

  def apply(self, variables, inputs: Array, rngs=None) -> Tuple[BaseDispatcher, Metrics]:
    kernel = variables["params"]["dense"]["kernel"]
    gates_softmax, metrics = self._compute_ensemble_gates_softmax_and_metrics(inputs, kernel, rngs)
    dispatcher = self._create_dispatcher(gates_softmax)
    return dispatcher, metrics

  def _compute_ensemble_gates_softmax_and_metrics(self, inputs: Array, kernel: Array, rngs=None):
    if inputs.ndim != 3:
      raise ValueError(f"inputs.ndim must be 3, but it is {inputs.ndim}")
    M, E = self.ensemble_size, self.num_experts
    if M <= 0:
      raise ValueError(f"Ensemble size must be >= 1; got {M}.")
    if E % M != 0:
      raise ValueError(f"num_experts must be multiple of ensemble_size, but got {E} and {M}.")
    num_groups, group_size, hidden_size = inputs.shape
    if group_size % M != 0:
      raise ValueError(f"group_size must be multiple of ensemble_size, but "
                       f"got {group_size} and {M}.")
    if tuple(kernel.shape) != (hidden_size, M, E // M):
      raise ValueError(f"Router kernel has shape {tuple(kernel.shape)}, expected "
                       f"{(hidden_size, M, E // M)}")
    kernel = self._cast_kernel(kernel, self.dtype or inputs.dtype)   # once for all members
    rngs = module.make_rngs(rngs, inputs.device)   # one stream, split over the members in order
    x = inputs.reshape(num_groups, group_size // M, M, hidden_size)
    gates_full, per_member = None, []
    for m in range(M):
      gates_m, metrics_m, _ = self._compute_gates_softmax_and_metrics(
          x[:, :, m, :].contiguous(), kernel[:, m, :].contiguous(), rngs, num_experts=E // M)
      if gates_full is None:
        gates_full = gates_m.new_zeros((num_groups, group_size // M, M, M, E // M))
      gates_full[:, :, m, m, :] = gates_m
      per_member.append(metrics_m)
    metrics = {k: torch.stack([pm[k] for pm in per_member], dim=1) for k in per_member[0]}
    return gates_full.reshape(num_groups, group_size, E), metrics
