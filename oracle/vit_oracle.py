"""TEST INFRASTRUCTURE ONLY: CPU restatement (NumPy, float32 internals) of the
V-MoE vision transformer that surrounds the MoE layer, vmoe/nn/vit_moe.py:127-383.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import this
module; the product never does.

What pins it:
  * the position-embedding known answers of vmoe/nn/vit_moe_test.py:78-127
    (learned and sincos2d, with and without a class token) and the parameter
    tree of :159-187 (tests/test_vit_oracle.py);
  * layer norm, attention and the patch convolution against torch's CPU library
    routines on random inputs (same file);
  * the MoE block is oracle.moe_oracle.mlp_moe_block, pinned by the goldens of
    vmoe/moe_test.py.

flax.linen.MultiHeadDotProductAttention / LayerNorm / Conv and
vit_jax.models_vit.{MlpBlock, AddPositionEmbs} are third-party code that is not
part of the reference checkout; they are restated from their published
definitions.  In bfloat16 the exact rounding points inside flax's attention
(logits and probabilities held in bfloat16) are modelled but PARITY UNPINNED:
no vector of the reference covers them.
"""
from __future__ import annotations

import math
from typing import Any, Dict, Mapping, Optional, Tuple

import numpy as np

from oracle import moe_oracle as O

F32, BF16 = O.F32, O.BF16


def layer_norm(x, scale, bias, dtype: Optional[str], eps: float = 1e-6) -> np.ndarray:
  """flax.linen.LayerNorm over the last axis: statistics and normalisation in
  float32 (variance as E[x^2] - E[x]^2), result cast to ``dtype`` (None keeps
  float32, the promotion of the float32 parameters)."""
  x = np.asarray(x, np.float32)
  mean = x.mean(axis=-1, keepdims=True, dtype=np.float32)
  mean2 = (x * x).mean(axis=-1, keepdims=True, dtype=np.float32)
  var = np.maximum(mean2 - mean * mean, 0.0)
  y = (x - mean) * (1.0 / np.sqrt(var + np.float32(eps)))
  if scale is not None:
    y = y * np.asarray(scale, np.float32)
  if bias is not None:
    y = y + np.asarray(bias, np.float32)
  return O.cast(y, dtype or F32)


def _module_dtype(dtype: Optional[str], *arrays_dtypes: str) -> str:
  """dtype of a flax module's computation: its ``dtype`` attribute, else the
  promotion of inputs and float32 parameters, which is float32."""
  return dtype or F32


def multi_head_attention(inputs_q, inputs_kv, params, num_heads: int, dtype: Optional[str],
                         normalize_qk: bool = False) -> np.ndarray:
  """flax.linen.MultiHeadDotProductAttention at inference (no mask, no dropout).

  params: query/key/value {'kernel': (D, H, hd), 'bias': (H, hd)},
  out {'kernel': (H, hd, D_out), 'bias': (D_out,)}; with normalize_qk also
  query_ln/key_ln {'scale': (hd,)}.  Call sites: vmoe/nn/vit_moe.py:139-144, :166-174.
  """
  dt = _module_dtype(dtype)
  H = num_heads

  def proj(x, p):
    D, h, hd = p["kernel"].shape
    assert h == H
    y = O.dense(x, np.reshape(p["kernel"], (D, h * hd)), np.reshape(p["bias"], (h * hd,)), dt)
    return y.reshape(*x.shape[:-1], h, hd)

  q, k, v = proj(inputs_q, params["query"]), proj(inputs_kv, params["key"]), proj(
      inputs_kv, params["value"])
  if normalize_qk:
    q = layer_norm(q, params["query_ln"]["scale"], None, dt)
    k = layer_norm(k, params["key_ln"]["scale"], None, dt)
  hd = q.shape[-1]
  q = O.cast(q / O.cast(np.sqrt(np.float32(hd)), dt), dt)
  logits = O.cast(np.einsum("bqhd,bkhd->bhqk", q, k, dtype=np.float32), dt)
  probs = O.cast(O.softmax(logits, axis=-1), dt)
  ctx = O.cast(np.einsum("bhqk,bkhd->bqhd", probs, v, dtype=np.float32), dt)
  out = params["out"]
  h, hd2, Dout = out["kernel"].shape
  return O.dense(ctx.reshape(*ctx.shape[:-2], h * hd2), np.reshape(out["kernel"], (h * hd2, Dout)),
                 out["bias"], dt)


def mlp(x, params, dtype: Optional[str]) -> np.ndarray:
  """The dense MlpBlock (vmoe/nn/vit_moe.py:38-45): one expert of moe_oracle.mlp_block."""
  dt = _module_dtype(dtype)
  lead = x.shape[:-1]
  p0, p1 = params["Dense_0"], params["Dense_1"]
  y = O.mlp_block(np.reshape(x, (1, -1, x.shape[-1])), p0["kernel"][None], p0["bias"][None],
                  p1["kernel"][None], p1["bias"][None], dt)
  return y.reshape(*lead, y.shape[-1])


def sincos2d(h: int, w: int, c: int, temperature: float = 10_000.) -> np.ndarray:
  """vmoe/nn/vit_moe.py:277-298: (1, h*w, c) float32."""
  if c % 4 != 0 or c < 8:
    raise ValueError(f"The hidden_size={c} must be multiple of 4 and >= 8.")
  y, x = np.mgrid[:h, :w].astype(np.float32)
  y, x = y.flatten(), x.flatten()
  omega = np.arange(c // 4, dtype=np.float32) / np.float32(c // 4 - 1)
  omega = (1.0 / (np.float32(temperature) ** omega)).astype(np.float32)
  x = np.einsum("n,d->nd", x, omega)
  y = np.einsum("n,d->nd", y, omega)
  return np.concatenate([np.sin(x), np.cos(x), np.sin(y), np.cos(y)], axis=-1)[None].astype(
      np.float32)


def add_position_emb(inputs, params, position_emb: Optional[Mapping[str, Any]]) -> np.ndarray:
  """vmoe/nn/vit_moe.py:262-309."""
  position_emb = position_emb or {}
  name = position_emb.get("name", "learned")
  if name == "none":
    return inputs
  if name == "learned":
    return inputs + np.asarray(params["posembed_input"]["pos_embedding"], np.float32)
  if name == "sincos2d":
    _, n, c = inputs.shape
    h, w = position_emb["h"], position_emb["w"]
    emb = sincos2d(h, w, c, position_emb.get("temperature", 10_000.))
    if n == h * w:
      return inputs + emb
    if n == h * w + 1:
      return np.concatenate([inputs[:, :1], inputs[:, 1:] + emb], axis=1)
    raise ValueError(f"Unsupported sequence length {n=} for the given {h=} and {w=}.")
  raise ValueError(f"Unsupported position embedding: {position_emb}")


def encoder_block(inputs, params, *, num_heads: int, dtype: Optional[str], moe: Optional[dict],
                  attention_qk_norm: bool = False):
  """vmoe/nn/vit_moe.py:151-184.  ``moe`` holds the MlpMoeBlock options for a
  block with experts (None for a dense block).  Returns x or (x, metrics)."""
  x = layer_norm(inputs, params["LayerNorm_0"]["scale"], params["LayerNorm_0"]["bias"], dtype)
  x = multi_head_attention(x, x, params["SelfAttention"], num_heads, dtype, attention_qk_norm)
  x = x + np.asarray(inputs, np.float32)     # bf16 + float32 promotes: the residual stays float32
  y = layer_norm(x, params["LayerNorm_1"]["scale"], params["LayerNorm_1"]["bias"], dtype)
  if moe is None:
    return x + mlp(y, params["Mlp"], dtype)
  router = dict(moe.get("router") or {})
  dispatcher_kwargs = dict(router.get("dispatcher") or {})
  y, metrics = O.mlp_moe_block(
      y, params["Moe"], group_size=moe["group_size"],
      num_selected_experts=router.get("num_selected_experts", 1),
      dispatcher_kwargs=dispatcher_kwargs, dtype=_module_dtype(dtype),
      gshard_loss_weight=router.get("gshard_loss_weight", 0.0),
      importance_loss_weight=router.get("importance_loss_weight", 1.0))
  return x + y, metrics


def encoder_moe(inputs, params, *, num_layers: int, mlp_dim: int, num_heads: int,
                moe: Optional[dict] = None, dtype: Optional[str] = None,
                position_emb: Optional[dict] = None, attention_qk_norm: bool = False,
                **unused):
  """vmoe/nn/vit_moe.py:187-260 at inference."""
  del mlp_dim, unused
  assert inputs.ndim == 3, f"Expected ndim = 3, but got shape {inputs.shape}"
  x = add_position_emb(np.asarray(inputs, np.float32), params, position_emb)
  moe_params = dict(moe or {})
  moe_layers = tuple(moe_params.pop("layers", ()))
  metrics: Dict[str, Any] = {}
  for block in range(num_layers):
    p = params[f"encoderblock_{block}"]
    if block in moe_layers:
      x, metrics[f"encoderblock_{block}"] = encoder_block(
          x, p, num_heads=num_heads, dtype=dtype, moe=moe_params,
          attention_qk_norm=attention_qk_norm)
    else:
      x = encoder_block(x, p, num_heads=num_heads, dtype=dtype, moe=None,
                        attention_qk_norm=attention_qk_norm)
  encoded = layer_norm(x, params["encoder_norm"]["scale"], params["encoder_norm"]["bias"], None)
  metrics["auxiliary_loss"] = sum(m["auxiliary_loss"] for m in metrics.values())
  return encoded, metrics


def patch_embedding(images, kernel, bias) -> np.ndarray:
  """flax.linen.Conv with kernel == stride == patch, 'VALID' (vmoe/nn/vit_moe.py:331-333):
  images (B, H, W, Cin), kernel (ph, pw, Cin, D) -> (B, H/ph, W/pw, D), float32."""
  B, Hh, Ww, Cin = images.shape
  ph, pw, cin, D = kernel.shape
  assert cin == Cin
  gh, gw = Hh // ph, Ww // pw
  x = np.asarray(images, np.float32)[:, :gh * ph, :gw * pw]
  x = x.reshape(B, gh, ph, gw, pw, Cin).transpose(0, 1, 3, 2, 4, 5).reshape(B, gh, gw, ph * pw * Cin)
  y = np.matmul(x, np.asarray(kernel, np.float32).reshape(ph * pw * Cin, D))
  return (y + np.asarray(bias, np.float32)).astype(np.float32)


def map_head(x, params, *, mlp_dim: int, num_heads: int, qk_norm: bool = False) -> np.ndarray:
  """Multihead attention pooling, vmoe/nn/vit_moe.py:127-148 (float32 module)."""
  del mlp_dim
  probe = np.tile(np.asarray(params["probe"], np.float32), (x.shape[0], 1, 1))
  x = multi_head_attention(probe, x, params["MultiHeadDotProductAttention"], num_heads, None,
                           qk_norm)
  y = layer_norm(x, params["LayerNorm"]["scale"], params["LayerNorm"]["bias"], None)
  y = mlp(y, params["Mlp"], None)
  return (x + y)[:, 0, :]


def vision_transformer_moe(images, params, *, num_classes: Optional[int], patch_size,
                           hidden_size: int, encoder: Mapping[str, Any],
                           classifier: str = "token", representation_size: Optional[int] = None,
                           **unused) -> Tuple[np.ndarray, Dict[str, Any]]:
  """vmoe/nn/vit_moe.py:312-383 at inference.  Returns (logits or features, metrics)."""
  del unused
  x = patch_embedding(images, params["embedding"]["kernel"], params["embedding"]["bias"])
  assert x.shape[-1] == hidden_size and tuple(params["embedding"]["kernel"].shape[:2]) == tuple(
      patch_size)
  encoder_kwargs = dict(encoder)
  if (encoder_kwargs.get("position_emb") or {}).get("name") == "sincos2d":
    encoder_kwargs["position_emb"] = dict(encoder_kwargs["position_emb"], h=x.shape[1],
                                          w=x.shape[2])
  x = x.reshape(x.shape[0], -1, x.shape[-1])
  if classifier == "token":
    cls = np.tile(np.asarray(params["cls"], np.float32), (x.shape[0], 1, 1))
    x = np.concatenate([cls, x], axis=1)
  for k in ("dropout_rate", "attention_dropout_rate", "deterministic"):
    encoder_kwargs.pop(k, None)
  x, metrics = encoder_moe(x, params["Encoder"], **encoder_kwargs)
  if classifier in ("token", "0"):
    x = x[:, 0]
  elif classifier == "gap":
    x = x.mean(axis=1, dtype=np.float32)
  elif classifier == "map":
    x = map_head(x, params["MapHead"], num_heads=encoder["num_heads"],
                 mlp_dim=encoder["mlp_dim"], qk_norm=encoder.get("attention_qk_norm", False))
  else:
    raise ValueError(f"Unknown classifier: {classifier!r}")
  if representation_size is not None:
    p = params["pre_logits"]
    x = np.tanh(O.dense(x, p["kernel"], p["bias"], F32))
  if num_classes:
    p = params["head"]
    return O.dense(x, p["kernel"], p["bias"], F32), metrics
  return x, metrics


def init_params(rng: np.random.Generator, image_shape, *, num_classes, patch_size, hidden_size,
                encoder, classifier="token", representation_size=None, **unused):
  """A random parameter tree with the names and shapes of vmoe/nn/vit_moe_test.py:159-187
  (values are seeded test data, not the reference's initialisers)."""
  del unused
  D = hidden_size
  ph, pw = patch_size
  _, Hh, Ww, Cin = image_shape
  n = (Hh // ph) * (Ww // pw) + (1 if classifier == "token" else 0)
  H = encoder["num_heads"]
  hd = D // H
  M = encoder["mlp_dim"]
  f = lambda *shape, s=1.0: (rng.standard_normal(shape) * s).astype(np.float32)

  def ln():
    return {"scale": 1.0 + f(D, s=0.1), "bias": f(D, s=0.1)}

  def attn(qk_norm=False):
    p = {k: {"kernel": f(D, H, hd, s=D ** -0.5), "bias": f(H, hd, s=0.02)}
         for k in ("query", "key", "value")}
    p["out"] = {"kernel": f(H, hd, D, s=D ** -0.5), "bias": f(D, s=0.02)}
    if qk_norm:
      p["query_ln"] = {"scale": 1.0 + f(hd, s=0.1)}
      p["key_ln"] = {"scale": 1.0 + f(hd, s=0.1)}
    return p

  def dense_mlp():
    return {"Dense_0": {"kernel": f(D, M, s=D ** -0.5), "bias": f(M, s=0.02)},
            "Dense_1": {"kernel": f(M, D, s=M ** -0.5), "bias": f(D, s=0.02)}}

  moe = dict(encoder.get("moe") or {})
  moe_layers = tuple(moe.get("layers", ()))
  qk_norm = encoder.get("attention_qk_norm", False)
  enc: Dict[str, Any] = {"encoder_norm": ln()}
  if (encoder.get("position_emb") or {}).get("name", "learned") == "learned":
    enc["posembed_input"] = {"pos_embedding": f(1, n, D, s=0.02)}
  for b in range(encoder["num_layers"]):
    blk = {"LayerNorm_0": ln(), "LayerNorm_1": ln(), "SelfAttention": attn(qk_norm)}
    if b in moe_layers:
      E = moe["num_experts"]
      blk["Moe"] = {
          "Router": {"dense": {"kernel": f(D, E, s=D ** -0.5)}},
          "Mlp": {"Dense_0": {"kernel": f(E, D, M, s=D ** -0.5), "bias": f(E, M, s=0.02)},
                  "Dense_1": {"kernel": f(E, M, D, s=M ** -0.5), "bias": f(E, D, s=0.02)}}}
    else:
      blk["Mlp"] = dense_mlp()
    enc[f"encoderblock_{b}"] = blk
  params: Dict[str, Any] = {
      "Encoder": enc,
      "embedding": {"kernel": f(ph, pw, Cin, D, s=(ph * pw * Cin) ** -0.5), "bias": f(D, s=0.02)}}
  if classifier == "token":
    params["cls"] = f(1, 1, D, s=0.02)
  if classifier == "map":
    params["MapHead"] = {"probe": f(1, 1, D, s=D ** -0.5),
                         "MultiHeadDotProductAttention": attn(qk_norm),
                         "LayerNorm": ln(), "Mlp": dense_mlp()}
  feat = D
  if representation_size is not None:
    params["pre_logits"] = {"kernel": f(D, representation_size, s=D ** -0.5),
                            "bias": f(representation_size, s=0.02)}
    feat = representation_size
  if num_classes:
    params["head"] = {"kernel": f(feat, num_classes, s=feat ** -0.5), "bias": f(num_classes, s=0.02)}
  return params
