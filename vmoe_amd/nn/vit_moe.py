"""The sparse MoE layer of MLPs on HIP kernels; host-side mirror of the MoE parts
of vmoe/nn/vit_moe.py (MlpBlock :38-45, MlpMoeBlock :48-124)."""
from __future__ import annotations

from typing import Any, Iterable, Mapping, Optional, Union

import torch

import vmoe_amd.moe
import vmoe_amd.utils
from vmoe_amd import kernels as K
from vmoe_amd.nn import module
from vmoe_amd.nn import routing

Array = torch.Tensor
KwArgs = Mapping[str, Any]


class MlpBlock(module.Module):
  """Dense -> GELU -> Dense, the expert of the MoE layer.

  Follows vit_jax.models_vit.MlpBlock as subclassed at vmoe/nn/vit_moe.py:38-45
  (dropout is inactive at inference).  Parameters:
  ``{'Dense_0': {'kernel': (D, M), 'bias': (M,)}, 'Dense_1': {'kernel': (M, D), 'bias': (D,)}}``;
  under sparse_moe_spmd every leaf gains a leading expert axis.

  The bf16 kernels read the weights K-contiguous; the transposed copies are made
  once per parameter tensor and cached.
  """
  _fields = dict(mlp_dim=module._REQUIRED, dtype=None, out_dim=None, dropout_rate=0.0,
                 deterministic=False, approximate_gelu=True)

  def __init__(self, **kwargs):
    super().__init__(**kwargs)
    self._packed = {}

  def init(self, rng, inputs: Array):
    gen = module.generator(rng)
    D = inputs.shape[-1]
    out_dim = self.out_dim or D
    M = self.mlp_dim
    dev = inputs.device
    # xavier_uniform kernels, normal(1e-6) biases, as vit_jax does.
    lim0, lim1 = (6.0 / (D + M)) ** 0.5, (6.0 / (M + out_dim)) ** 0.5
    k0 = (torch.rand((D, M), generator=gen) * 2 - 1) * lim0
    k1 = (torch.rand((M, out_dim), generator=gen) * 2 - 1) * lim1
    b0 = torch.randn((M,), generator=gen) * 1e-6
    b1 = torch.randn((out_dim,), generator=gen) * 1e-6
    return {"params": {"Dense_0": {"kernel": k0.to(dev), "bias": b0.to(dev)},
                       "Dense_1": {"kernel": k1.to(dev), "bias": b1.to(dev)}}}

  def _pack(self, w: Array, dtype) -> Array:
    key = (w.data_ptr(), w._version, tuple(w.shape), dtype)
    hit = self._packed.get(key)
    if hit is None:
      if len(self._packed) > 8:
        self._packed.clear()
      hit = K.pack_expert_weights(K.cast(w, dtype))
      self._packed[key] = hit
    return hit

  def apply_experts(self, variables, inputs: Array) -> Array:
    """inputs (E, R, D) with parameters stacked on axis 0 -> (E, R, D)."""
    p = variables["params"]
    dtype = self.dtype or inputs.dtype
    x = K.cast(inputs, dtype)
    w0, b0 = p["Dense_0"]["kernel"], p["Dense_0"].get("bias")
    w1, b1 = p["Dense_1"]["kernel"], p["Dense_1"].get("bias")
    cast = lambda t: None if t is None else K.cast(t, dtype)
    if dtype == torch.bfloat16:
      return K.expert_mlp(x, None, cast(b0), None, cast(b1), w0t=self._pack(w0, dtype),
                          w1t=self._pack(w1, dtype), approximate_gelu=self.approximate_gelu)
    return K.expert_mlp(x, cast(w0), cast(b0), cast(w1), cast(b1),
                        approximate_gelu=self.approximate_gelu)

  def apply(self, variables, inputs: Array) -> Array:
    """Single MLP: inputs (..., D)."""
    stacked = vmoe_amd.moe._tree_map(lambda t: t[None], variables)
    lead = inputs.shape[:-1]
    out = self.apply_experts(stacked, inputs.reshape(1, -1, inputs.shape[-1]))
    return out.reshape(*lead, out.shape[-1])


class MlpMoeBlock(module.Module):
  """Sparse MoE layer of MLPs; vmoe/nn/vit_moe.py:48-124.

  Parameters: ``{'Router': {...}, 'Mlp': {'Dense_0': {'kernel': (E, D, M), 'bias': (E, M)},
  'Dense_1': {'kernel': (E, M, D), 'bias': (E, D)}}}``.
  ``apply(variables, inputs)`` with inputs (num_seqs, seq_len, D) returns
  ``(outputs, metrics)``.
  """
  _fields = dict(mlp_dim=module._REQUIRED, num_experts=module._REQUIRED,
                 group_size=module._REQUIRED, dropout_rate=0.0, deterministic=False,
                 router=None, dtype=None, split_rngs=False)

  def __init__(self, **kwargs):
    super().__init__(**kwargs)
    self._router = None
    self._mlp = None

  def create_router(self):
    router_kwargs = dict(num_experts=self.num_experts, **(self.router or {}))
    router_kwargs["deterministic"] = router_kwargs.get("deterministic", self.deterministic)
    router_cls = router_kwargs.pop("name", "NoisyTopExpertsPerItemRouter")
    router_cls, router_args, router_kwargs2 = vmoe_amd.utils.parse_call(
        router_cls, default_module=routing)
    return router_cls(*router_args, dtype=self.dtype, name="Router",
                      **{**router_kwargs2, **router_kwargs})

  def create_split_rngs(self) -> Mapping[str, bool]:
    if isinstance(self.split_rngs, bool):
      return {"params": self.split_rngs, "dropout": self.split_rngs}
    split_rngs = set(self.split_rngs)
    return {"params": "params" in split_rngs, "dropout": "dropout" in split_rngs}

  def _modules(self):
    if self._router is None:
      self._router = self.create_router()
      self._mlp = vmoe_amd.moe.sparse_moe_spmd(
          MlpBlock, has_aux=False, variable_axes={"params": 0, "intermediates": 0},
          split_rngs=self.create_split_rngs())(
              mlp_dim=self.mlp_dim, dropout_rate=self.dropout_rate, dtype=self.dtype,
              deterministic=self.deterministic, name="Mlp")
    return self._router, self._mlp

  def init(self, rng, inputs: Array):
    assert inputs.ndim == 3, f"Expected ndim = 3, but got shape {inputs.shape}"
    router, mlp = self._modules()
    x = inputs.reshape(-1, self.group_size, inputs.shape[-1])
    seed = vmoe_amd.moe._fold_seed(rng, 17)
    router_vars = router.init(seed, x)
    dispatcher, _ = router.apply(router_vars, x)
    mlp_vars = mlp.init(vmoe_amd.moe._fold_seed(rng, 23), dispatcher, x)
    return {"params": {"Router": router_vars["params"], "Mlp": mlp_vars["params"]}}

  def apply(self, variables, inputs: Array):
    assert inputs.ndim == 3, f"Expected ndim = 3, but got shape {inputs.shape}"
    router, mlp = self._modules()
    inputs_shape = inputs.shape
    x = inputs.reshape(-1, self.group_size, inputs.shape[-1])
    params = variables["params"]
    dispatcher, metrics = router.apply({"params": params["Router"]}, x)
    outputs = mlp.apply({"params": params["Mlp"]}, dispatcher, x)
    outputs = outputs.reshape(*inputs_shape[:-1], outputs.shape[-1])
    return outputs, metrics
