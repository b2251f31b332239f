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
    self._packed = module.ParamCache()

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
    return self._packed.get((w,), dtype, lambda: K.pack_expert_weights(K.cast(w, dtype)))

  supports_packed_rows = True

  def apply_experts(self, variables, inputs: Array, rows_per_expert: Optional[Array] = None) -> Array:
    """inputs (E, R, D) with parameters stacked on axis 0 -> (E, R, D).  With
    rows_per_expert (E,) int32 only that many leading rows of each expert are
    computed; the other rows of the result are not written."""
    p = variables["params"]
    dtype = self.dtype or inputs.dtype
    w0, b0 = p["Dense_0"]["kernel"], p["Dense_0"].get("bias")
    w1, b1 = p["Dense_1"]["kernel"], p["Dense_1"].get("bias")
    module.require_no_grad("MlpBlock", inputs, w0, b0, w1, b1)
    x = K.cast(inputs, dtype)
    cast = lambda t: None if t is None else K.cast(t, dtype)
    if dtype == torch.bfloat16:
      return K.expert_mlp(x, None, cast(b0), None, cast(b1), w0t=self._pack(w0, dtype),
                          w1t=self._pack(w1, dtype), approximate_gelu=self.approximate_gelu,
                          rows_per_expert=rows_per_expert)
    return K.expert_mlp(x, cast(w0), cast(b0), cast(w1), cast(b1),
                        approximate_gelu=self.approximate_gelu, rows_per_expert=rows_per_expert)

  def can_gather(self, items: Array) -> bool:
    """Whether apply_experts_gathered covers these items (dtype and width of the kernel)."""
    dtype = self.dtype or items.dtype
    return (items.is_cuda and dtype in (torch.bfloat16, torch.float32) and items.dtype == dtype
            and K.expert_mlp_can_gather(dtype, items.shape[-1], items.numel() // items.shape[-1]))

  def apply_experts_gathered(self, variables, items: Array, row_token: Array,
                             rows_per_expert: Array) -> Array:
    """items (T, D); row_token (E, R) int32 names the item in row r of expert e,
    rows_per_expert (E,) how many rows each expert has -> (E, R, D).  The first product
    reads its rows straight from ``items``: the dispatched buffer is never built."""
    p = variables["params"]
    dtype = self.dtype or items.dtype
    w0, b0 = p["Dense_0"]["kernel"], p["Dense_0"].get("bias")
    w1, b1 = p["Dense_1"]["kernel"], p["Dense_1"].get("bias")
    module.require_no_grad("MlpBlock", items, w0, b0, w1, b1)
    cast = lambda t: None if t is None else K.cast(t, dtype)
    if dtype != torch.bfloat16:      # float32 reads the kernels in the reference's layout
      return K.expert_mlp(K.cast(items, dtype), cast(w0), cast(b0), cast(w1), cast(b1),
                          approximate_gelu=self.approximate_gelu, rows_per_expert=rows_per_expert,
                          x_rows=row_token)
    return K.expert_mlp(K.cast(items, dtype), None, cast(b0), None, cast(b1),
                        w0t=self._pack(w0, dtype), w1t=self._pack(w1, dtype),
                        approximate_gelu=self.approximate_gelu, rows_per_expert=rows_per_expert,
                        x_rows=row_token)

  def apply_experts_routed(self, variables, items: Array, fill: Array, token_slot: Array,
                           capacity: int):
    """apply_experts_gathered for a dispatcher whose packed rows are still to be computed:
    items (T, D), fill (G, E) and token_slot (G, S, K) of the slot assignment -> (outputs
    (E, G * capacity, D), (token_row, rows_per_expert, row_token)).  The renumbering of the
    assignments shares a launch with the planning of the two products."""
    p = variables["params"]
    dtype = self.dtype or items.dtype
    w0, b0 = p["Dense_0"]["kernel"], p["Dense_0"].get("bias")
    w1, b1 = p["Dense_1"]["kernel"], p["Dense_1"].get("bias")
    module.require_no_grad("MlpBlock", items, w0, b0, w1, b1)
    cast = lambda t: None if t is None else K.cast(t, dtype)
    if dtype != torch.bfloat16:
      return K.expert_mlp(K.cast(items, dtype), cast(w0), cast(b0), cast(w1), cast(b1),
                          approximate_gelu=self.approximate_gelu,
                          compact=(fill, token_slot, capacity))
    return K.expert_mlp(K.cast(items, dtype), None, cast(b0), None, cast(b1),
                        w0t=self._pack(w0, dtype), w1t=self._pack(w1, dtype),
                        approximate_gelu=self.approximate_gelu,
                        compact=(fill, token_slot, capacity))

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

  @staticmethod
  def _route(router, variables, x: Array, rngs):
    """Routers that draw random numbers take them as ``rngs=``; the others are
    called without (their apply has no such argument)."""
    if isinstance(router, (routing.NoisyTopExpertsPerItemRouter,
                           routing.NoisyTopItemsPerExpertRouter)):
      return router.apply(variables, x, rngs=module.make_rngs(rngs, x.device))
    return router.apply(variables, x)

  def init(self, rng, inputs: Array):
    assert inputs.ndim == 3, f"Expected ndim = 3, but got shape {inputs.shape}"
    router, mlp = self._modules()
    x = inputs.reshape(-1, self.group_size, inputs.shape[-1])
    seed = vmoe_amd.moe._fold_seed(rng, 17)
    router_vars = router.init(seed, x)
    dispatcher, _ = self._route(router, router_vars, x,
                                {"gating": vmoe_amd.moe._fold_seed(rng, 29)})
    mlp_vars = mlp.init(vmoe_amd.moe._fold_seed(rng, 23), dispatcher, x)
    return {"params": {"Router": router_vars["params"], "Mlp": mlp_vars["params"]}}

  def apply(self, variables, inputs: Array, rngs=None):
    assert inputs.ndim == 3, f"Expected ndim = 3, but got shape {inputs.shape}"
    router, mlp = self._modules()
    inputs_shape = inputs.shape
    x = inputs.reshape(-1, self.group_size, inputs.shape[-1])
    params = variables["params"]
    dispatcher, metrics = self._route(router, {"params": params["Router"]}, x, rngs)
    outputs = mlp.apply({"params": params["Mlp"]}, dispatcher, x)
    outputs = outputs.reshape(*inputs_shape[:-1], outputs.shape[-1])
    return outputs, metrics


# --------------------------------------------------------------------------- the transformer
# The layers below surround the MoE layer in the full model (vmoe/nn/vit_moe.py:127-383).
# They are library calls of torch-ROCm (layer norm, GEMMs, attention); the dense and
# sparse MLPs run on this package's own kernels.

def _layer_norm(x: Array, p: Mapping[str, Array], dtype: Optional[torch.dtype],
                eps: float = 1e-6) -> Array:
  """flax.linen.LayerNorm: float32 statistics, result in ``dtype`` (float32 if None)."""
  n = x.shape[-1]
  scale, bias = p.get("scale"), p.get("bias")
  y = torch.nn.functional.layer_norm(
      x.float(), (n,), None if scale is None else scale.float(),
      None if bias is None else bias.float(), eps)
  return y if dtype in (None, torch.float32) else y.to(dtype)


def _add_layer_norm(residual: Array, branch: Optional[Array], p: Mapping[str, Array],
                    dtype: Optional[torch.dtype], eps: float = 1e-6):
  """``x = residual + branch; y = LayerNorm(dtype)(x)`` (vmoe/nn/vit_moe.py:162-179) ->
  (x, y).  A float32 residual takes the fused kernel; anything else keeps the
  promotion rules of the separate operations."""
  if residual.dtype == torch.float32 and (
      branch is None or branch.dtype in (torch.float32, torch.bfloat16)):
    return K.add_layer_norm(residual, branch, p.get("scale"), p.get("bias"), eps,
                            dtype or torch.float32)
  x = residual if branch is None else residual + branch
  return x, _layer_norm(x, p, dtype, eps)


class IdentityLayer(module.Module):
  """vit_jax.models_vit.IdentityLayer (exists to name the pre-logits activation)."""

  def apply(self, variables, x):
    return x


class AddPositionEmbs(module.Module):
  """vit_jax.models_vit.AddPositionEmbs: learned (1, n, D) embedding added to the tokens."""
  _fields = dict(posemb_std=0.02)

  def init(self, rng, inputs: Array):
    gen = module.generator(rng)
    emb = torch.randn((1, inputs.shape[1], inputs.shape[2]), generator=gen) * self.posemb_std
    return {"params": {"pos_embedding": emb.to(inputs.device)}}

  def apply(self, variables, inputs: Array) -> Array:
    assert inputs.ndim == 3, f"Number of dimensions should be 3, but it is: {inputs.ndim}"
    return inputs + variables["params"]["pos_embedding"]


class MultiHeadDotProductAttention(module.Module):
  """flax.linen.MultiHeadDotProductAttention at inference, as used at
  vmoe/nn/vit_moe.py:139-144 and :166-174.

  Parameters: query/key/value ``{'kernel': (D, H, hd), 'bias': (H, hd)}``,
  out ``{'kernel': (H, hd, D), 'bias': (D,)}``; with ``normalize_qk`` also
  query_ln / key_ln ``{'scale': (hd,)}``.  The three input projections of
  self-attention run as one GEMM on a packed (3·D, D) weight that is built once
  per parameter tensor.
  """
  _fields = dict(num_heads=module._REQUIRED, dtype=None, normalize_qk=False, deterministic=True,
                 dropout_rate=0.0, broadcast_dropout=False, kernel_init=None)

  def __init__(self, **kwargs):
    super().__init__(**kwargs)
    self._packed = module.ParamCache()

  def init(self, rng, inputs_q: Array, inputs_kv: Optional[Array] = None):
    gen = module.generator(rng)
    D = inputs_q.shape[-1]
    H = self.num_heads
    hd = D // H
    dev = inputs_q.device
    lim = (6.0 / (D + D)) ** 0.5       # xavier_uniform on the (D, H*hd) matrix
    u = lambda *s: ((torch.rand(s, generator=gen) * 2 - 1) * lim).to(dev)
    p = {k: {"kernel": u(D, H, hd), "bias": torch.zeros((H, hd), device=dev)}
         for k in ("query", "key", "value")}
    p["out"] = {"kernel": u(H, hd, D), "bias": torch.zeros((D,), device=dev)}
    if self.normalize_qk:
      p["query_ln"] = {"scale": torch.ones((hd,), device=dev)}
      p["key_ln"] = {"scale": torch.ones((hd,), device=dev)}
    return {"params": p}

  def _proj_weights(self, p, names, dtype):
    """(sum of H * hd, D) weight and bias of the named input projections, packed once."""
    def build():
      w = torch.cat([p[n]["kernel"].reshape(p[n]["kernel"].shape[0], -1).t() for n in names])
      b = torch.cat([p[n]["bias"].reshape(-1) for n in names])
      return w.to(dtype).contiguous(), b.to(dtype).contiguous()
    tensors = [p[n][leaf] for n in names for leaf in ("kernel", "bias")]
    return self._packed.get(tensors, (dtype, names), build)

  def apply(self, variables, inputs_q: Array, inputs_kv: Optional[Array] = None) -> Array:
    p = variables["params"]
    if inputs_kv is None:
      inputs_kv = inputs_q
    dtype = self.dtype or torch.float32
    H = self.num_heads
    B, Sq, D = inputs_q.shape
    Sk = inputs_kv.shape[1]
    hd = p["query"]["kernel"].shape[-1]
    xq = inputs_q.to(dtype)
    linear = torch.nn.functional.linear
    if inputs_kv is inputs_q:
      w, b = self._proj_weights(p, ("query", "key", "value"), dtype)
      qkv = linear(xq, w, b).view(B, Sq, 3, H, hd)
      q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    else:
      wq, bq = self._proj_weights(p, ("query",), dtype)
      wkv, bkv = self._proj_weights(p, ("key", "value"), dtype)
      q = linear(xq, wq, bq).view(B, Sq, H, hd)
      kv = linear(inputs_kv.to(dtype), wkv, bkv).view(B, Sk, 2, H, hd)
      k, v = kv[:, :, 0], kv[:, :, 1]
    if self.normalize_qk:
      q = _layer_norm(q, p["query_ln"], dtype)
      k = _layer_norm(k, p["key_ln"], dtype)
    if q.is_cuda and K.attention_supported(q, k):
      ctx = K.attention(q, k, v, hd ** -0.5)                            # (B, Sq, H * hd)
    else:
      ctx = torch.nn.functional.scaled_dot_product_attention(
          q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2))     # (B, H, Sq, hd)
      ctx = ctx.transpose(1, 2).reshape(B, Sq, H * hd)
    wo, bo = self._packed.get(
        (p["out"]["kernel"], p["out"]["bias"]), (dtype, "out"),
        lambda: (p["out"]["kernel"].reshape(H * hd, -1).t().to(dtype).contiguous(),
                 p["out"]["bias"].to(dtype)))
    return linear(ctx, wo, bo)


class MapHead(module.Module):
  """Multihead attention pooling; vmoe/nn/vit_moe.py:127-148."""
  _fields = dict(mlp_dim=module._REQUIRED, num_heads=module._REQUIRED, qk_norm=False)

  def _modules(self):
    if not hasattr(self, "_attn"):
      self._attn = MultiHeadDotProductAttention(num_heads=self.num_heads, deterministic=True,
                                                normalize_qk=self.qk_norm,
                                                name="MultiHeadDotProductAttention")
      self._mlp = MlpBlock(mlp_dim=self.mlp_dim, deterministic=True, name="Mlp")
    return self._attn, self._mlp

  def init(self, rng, x: Array):
    attn, mlp = self._modules()
    gen = module.generator(rng)
    D = x.shape[-1]
    lim = (6.0 / (D + D)) ** 0.5
    probe = ((torch.rand((1, 1, D), generator=gen) * 2 - 1) * lim).to(x.device)
    fold = vmoe_amd.moe._fold_seed
    return {"params": {
        "probe": probe,
        "MultiHeadDotProductAttention": attn.init(fold(rng, 1), probe, x)["params"],
        "LayerNorm": {"scale": torch.ones((D,), device=x.device),
                      "bias": torch.zeros((D,), device=x.device)},
        "Mlp": mlp.init(fold(rng, 2), probe)["params"]}}

  def apply(self, variables, x: Array) -> Array:
    assert x.ndim == 3, f"Unexpected ndim = {x.ndim}, it must be 3"
    attn, mlp = self._modules()
    p = variables["params"]
    probe = p["probe"].to(x.dtype).expand(x.shape[0], 1, x.shape[-1])
    x = attn.apply({"params": p["MultiHeadDotProductAttention"]}, probe, x)
    y = _layer_norm(x, p["LayerNorm"], None)
    y = mlp.apply({"params": p["Mlp"]}, y)
    return (x + y)[:, 0, :]


class EncoderBlock(module.Module):
  """Encoder block with a dense MLP or a sparse MoE of MLPs; vmoe/nn/vit_moe.py:151-184.

  ``mlp_block`` is a callable returning the MLP module when called with
  ``dtype=`` and ``deterministic=`` (a class or a functools.partial of one).
  Parameters: LayerNorm_0, SelfAttention, LayerNorm_1 and 'Mlp' or 'Moe'
  (the name the MLP module was created with).
  """
  _fields = dict(mlp_block=module._REQUIRED, num_heads=module._REQUIRED, dtype=None,
                 dropout_rate=0.0, attention_dropout_rate=0.0, attention_qk_norm=False,
                 deterministic=False)

  def _modules(self):
    if not hasattr(self, "_attn"):
      self._attn = MultiHeadDotProductAttention(
          dtype=self.dtype, deterministic=self.deterministic, normalize_qk=self.attention_qk_norm,
          dropout_rate=self.attention_dropout_rate, num_heads=self.num_heads, name="SelfAttention")
      self._mlp = self.mlp_block(dtype=self.dtype, deterministic=self.deterministic)
    return self._attn, self._mlp

  def _check_inference(self):
    if not self.deterministic and (self.dropout_rate > 0 or self.attention_dropout_rate > 0):
      raise NotImplementedError("Dropout (training) is not implemented; use deterministic=True.")

  def init(self, rng, inputs: Array):
    attn, mlp = self._modules()
    D = inputs.shape[-1]
    dev = inputs.device
    fold = vmoe_amd.moe._fold_seed
    ln = lambda: {"scale": torch.ones((D,), device=dev), "bias": torch.zeros((D,), device=dev)}
    x = inputs if self.dtype is None else inputs.to(self.dtype)
    return {"params": {"LayerNorm_0": ln(), "LayerNorm_1": ln(),
                       "SelfAttention": attn.init(fold(rng, 1), x)["params"],
                       mlp.name: mlp.init(fold(rng, 2), x)["params"]}}

  def apply(self, variables, inputs: Array, rngs=None):
    x, y, metrics = self._forward(variables["params"], inputs, None,
                                  module.make_rngs(rngs, inputs.device))
    return x + y if metrics is None else (x + y, metrics)

  def _forward(self, p, residual: Array, pending: Optional[Array], rngs=None):
    """The block on ``residual + pending``, the last add left to the caller:
    returns (residual, mlp output not yet added, metrics or None).  Leaving the
    add pending lets it run inside the kernel of the layer norm that follows."""
    self._check_inference()
    attn, mlp = self._modules()
    x, a = _add_layer_norm(residual, pending, p["LayerNorm_0"], self.dtype)
    h = attn.apply({"params": p["SelfAttention"]}, a)
    x, y = _add_layer_norm(x, h, p["LayerNorm_1"], self.dtype)
    if isinstance(mlp, MlpMoeBlock):
      y, metrics = mlp.apply({"params": p[mlp.name]}, y, rngs=rngs)
      return x, y, metrics
    y = mlp.apply({"params": p[mlp.name]}, y)
    if isinstance(y, torch.Tensor):
      return x, y, None
    y, metrics = y
    return x, y, metrics


class EncoderMoe(module.Module):
  """Transformer encoder with optional blocks of sparse MoE of MLPs;
  vmoe/nn/vit_moe.py:187-309.  ``moe={'layers': (...), ...MlpMoeBlock options}``."""
  _fields = dict(num_layers=module._REQUIRED, mlp_dim=module._REQUIRED,
                 num_heads=module._REQUIRED, dropout_rate=0.0, attention_dropout_rate=0.0,
                 attention_qk_norm=False, moe=None, deterministic=False, dtype=None,
                 position_emb=None)
  DEFAULT_SINCOS2D_TEMPERATURE = 10_000.

  def _blocks(self):
    if not hasattr(self, "_block_list"):
      import functools
      dense_mlp_params = dict(mlp_dim=self.mlp_dim, dropout_rate=self.dropout_rate)
      moe_mlp_params = {**dense_mlp_params, **(self.moe or {})}
      self._moe_layers = tuple(moe_mlp_params.pop("layers", ()))
      dense_mlp_cls = functools.partial(MlpBlock, **dense_mlp_params, name="Mlp")
      moe_mlp_cls = functools.partial(MlpMoeBlock, **moe_mlp_params, name="Moe")
      self._block_list = [
          EncoderBlock(
              name=f"encoderblock_{b}", num_heads=self.num_heads, dropout_rate=self.dropout_rate,
              attention_dropout_rate=self.attention_dropout_rate,
              attention_qk_norm=self.attention_qk_norm, deterministic=self.deterministic,
              dtype=self.dtype,
              mlp_block=moe_mlp_cls if b in self._moe_layers else dense_mlp_cls)
          for b in range(self.num_layers)]
    return self._block_list

  def init(self, rng, inputs: Array):
    assert inputs.ndim == 3, f"Expected ndim = 3, but got shape {inputs.shape}"
    fold = vmoe_amd.moe._fold_seed
    D = inputs.shape[-1]
    dev = inputs.device
    params = {"encoder_norm": {"scale": torch.ones((D,), device=dev),
                               "bias": torch.zeros((D,), device=dev)}}
    if (self.position_emb or {}).get("name", "learned") == "learned":
      params["posembed_input"] = AddPositionEmbs(name="posembed_input").init(
          fold(rng, 1000), inputs)["params"]
    x = self.add_position_emb({"params": params}, inputs)
    for b, block in enumerate(self._blocks()):
      params[block.name] = block.init(fold(rng, b), x)["params"]
    return {"params": params}

  def apply(self, variables, inputs: Array, rngs=None):
    assert inputs.ndim == 3, f"Expected ndim = 3, but got shape {inputs.shape}"
    rngs = module.make_rngs(rngs, inputs.device)
    if not self.deterministic and self.dropout_rate > 0:
      raise NotImplementedError("Dropout (training) is not implemented; use deterministic=True.")
    params = variables["params"]
    x = self.add_position_emb(variables, inputs)
    metrics = {}
    pending = None          # output of the previous block's MLP, added by the next layer norm
    for b, block in enumerate(self._blocks()):
      x, pending, m = block._forward(params[block.name], x, pending, rngs)
      if b in self._moe_layers:
        metrics[block.name] = m
    _, encoded = _add_layer_norm(x, pending, params["encoder_norm"], None)
    metrics["auxiliary_loss"] = sum(m["auxiliary_loss"] for m in metrics.values())
    return encoded, metrics

  def add_position_emb(self, variables, inputs: Array) -> Array:
    position_emb = self.position_emb or {}
    name = position_emb.get("name", "learned")
    if name == "none":
      return inputs
    if name == "learned":
      return AddPositionEmbs(name="posembed_input").apply(
          {"params": variables["params"]["posembed_input"]}, inputs)
    if name == "sincos2d":
      _, n, c = inputs.shape
      h, w = position_emb["h"], position_emb["w"]
      if c % 4 != 0 or c < 8:
        raise ValueError(f"The hidden_size={c} must be multiple of 4 and >= 8.")
      temperature = position_emb.get("temperature", self.DEFAULT_SINCOS2D_TEMPERATURE)
      dev, dt = inputs.device, inputs.dtype
      y, x = torch.meshgrid(torch.arange(h, device=dev, dtype=dt),
                            torch.arange(w, device=dev, dtype=dt), indexing="ij")
      y, x = y.flatten(), x.flatten()
      omega = torch.arange(c // 4, device=dev, dtype=dt) / (c // 4 - 1)
      omega = 1. / (temperature ** omega)
      x = x[:, None] * omega[None, :]
      y = y[:, None] * omega[None, :]
      posembed = torch.cat([torch.sin(x), torch.cos(x), torch.sin(y), torch.cos(y)], dim=-1)[None]
      if n == h * w:
        return inputs + posembed
      if n == h * w + 1:
        return torch.cat([inputs[:, :1, :], inputs[:, 1:, :] + posembed], dim=1)
      raise ValueError(f"Unsupported sequence length {n=} for the given {h=} and {w=}.")
    raise ValueError(f"Unsupported position embedding: {self.position_emb}")


class VisionTransformerMoe(module.Module):
  """Vision Transformer with sparse MoE layers; vmoe/nn/vit_moe.py:312-383.

  ``apply(variables, images)`` with images (B, H, W, 3) returns (logits, metrics).
  Parameter tree as in vmoe/nn/vit_moe_test.py:159-187: embedding/{kernel (ph, pw, 3, D), bias},
  Encoder/..., head/{kernel, bias}, and cls / pre_logits / MapHead when configured.
  """
  _fields = dict(num_classes=module._REQUIRED, patch_size=module._REQUIRED,
                 hidden_size=module._REQUIRED, encoder=module._REQUIRED, classifier="token",
                 representation_size=None, deterministic=False, head_bias_init=0.0,
                 head_kernel_zero_init=True, encoder_cls=None)

  def _patches(self, inputs: Array) -> Array:
    """(B, H, W, Cin) -> (B, gh, gw, ph*pw*Cin): the rows the 'VALID' strided convolution sees."""
    B, Hh, Ww, Cin = inputs.shape
    ph, pw = self.patch_size
    gh, gw = Hh // ph, Ww // pw
    x = inputs[:, :gh * ph, :gw * pw]
    return x.reshape(B, gh, ph, gw, pw, Cin).permute(0, 1, 3, 2, 4, 5).reshape(
        B, gh, gw, ph * pw * Cin)

  def _encoder(self, grid_hw):
    encoder_kwargs = dict(self.encoder)
    if (encoder_kwargs.get("position_emb") or {}).get("name") == "sincos2d":
      encoder_kwargs["position_emb"] = dict(encoder_kwargs["position_emb"], h=grid_hw[0],
                                            w=grid_hw[1])
    key = tuple(grid_hw)
    cache = self.__dict__.setdefault("_encoders", {})
    if key not in cache:
      cls = self.encoder_cls or EncoderMoe
      cache[key] = cls(name="Encoder", deterministic=self.deterministic, **encoder_kwargs)
    return cache[key]

  def _map_head(self):
    if not hasattr(self, "_maphead"):
      self._maphead = MapHead(num_heads=self.encoder["num_heads"], mlp_dim=self.encoder["mlp_dim"],
                              qk_norm=self.encoder.get("attention_qk_norm", False), name="MapHead")
    return self._maphead

  def init(self, rng, inputs: Array):
    gen = module.generator(rng)
    fold = vmoe_amd.moe._fold_seed
    dev = inputs.device
    ph, pw = self.patch_size
    Cin, D = inputs.shape[-1], self.hidden_size
    params = {"embedding": {
        "kernel": module.lecun_normal(gen, (ph, pw, Cin, D), fan_in=ph * pw * Cin, device=dev),
        "bias": torch.zeros((D,), device=dev)}}
    x = self._embed(params, inputs)
    grid = x.shape[1:3]
    x = x.reshape(x.shape[0], -1, D)
    if self.classifier == "token":
      params["cls"] = torch.zeros((1, 1, D), device=dev)
      x = torch.cat([params["cls"].expand(x.shape[0], 1, D), x], dim=1)
    params["Encoder"] = self._encoder(grid).init(fold(rng, 1), x)["params"]
    if self.classifier == "map":
      params["MapHead"] = self._map_head().init(fold(rng, 2), x)["params"]
    feat = D
    if self.representation_size is not None:
      feat = self.representation_size
      params["pre_logits"] = {
          "kernel": module.lecun_normal(gen, (D, feat), fan_in=D, device=dev),
          "bias": torch.zeros((feat,), device=dev)}
    if self.num_classes:
      kernel = (torch.zeros((feat, self.num_classes), device=dev) if self.head_kernel_zero_init
                else module.lecun_normal(gen, (feat, self.num_classes), fan_in=feat, device=dev))
      params["head"] = {"kernel": kernel,
                        "bias": torch.full((self.num_classes,), float(self.head_bias_init),
                                           device=dev)}
    return {"params": params}

  def _embed(self, params, inputs: Array) -> Array:
    p = params["embedding"]
    k = p["kernel"]
    if tuple(k.shape[:2]) != tuple(self.patch_size) or k.shape[-1] != self.hidden_size:
      raise ValueError(f"embedding kernel has shape {tuple(k.shape)}, expected "
                       f"{(*self.patch_size, inputs.shape[-1], self.hidden_size)}")
    rows = self._patches(inputs.float())
    return torch.addmm(p["bias"].float(), rows.reshape(-1, rows.shape[-1]),
                       k.float().reshape(-1, k.shape[-1])).view(*rows.shape[:3], k.shape[-1])

  def apply(self, variables, inputs: Array, rngs=None):
    params = variables["params"]
    x = self._embed(params, inputs)
    grid = x.shape[1:3]
    x = x.reshape(x.shape[0], -1, x.shape[-1])
    if self.classifier == "token":
      x = torch.cat([params["cls"].to(x.dtype).expand(x.shape[0], 1, x.shape[-1]), x], dim=1)
    x, metrics = self._encoder(grid).apply({"params": params["Encoder"]}, x, rngs=rngs)
    if self.classifier in ("token", "0"):
      x = x[:, 0]
    elif self.classifier == "gap":
      x = x.mean(dim=tuple(range(1, x.ndim - 1)))
    elif self.classifier == "map":
      x = self._map_head().apply({"params": params["MapHead"]}, x)
    else:
      raise ValueError(f"Unknown classifier: {self.classifier!r}")
    if self.representation_size is not None:
      p = params["pre_logits"]
      x = torch.tanh(torch.addmm(p["bias"].float(), x, p["kernel"].float()))
    if self.num_classes:
      p = params["head"]
      return torch.addmm(p["bias"].float(), x, p["kernel"].float()), metrics
    return x, metrics
