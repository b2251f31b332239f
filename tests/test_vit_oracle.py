"""Pins the CPU restatement of the vision transformer around the MoE layer
(oracle/vit_oracle.py): the reference's own known answers for the position
embeddings (vmoe/nn/vit_moe_test.py:78-127), its parameter tree (:159-187) and
output shapes (:189-199), and torch's CPU library routines for layer norm,
attention and the patch convolution."""
import copy
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O
from oracle import vit_oracle as V

# vmoe/nn/vit_moe_test.py:28-55, minus the training-only router options.
DEFAULT_TEST_CONFIG = {
    "num_classes": 4,
    "patch_size": (2, 2),
    "hidden_size": 8,
    "encoder": {
        "num_layers": 2,
        "mlp_dim": 16,
        "num_heads": 2,
        "moe": {
            "layers": (1,),
            "num_experts": 4,
            "group_size": 4,
            "router": {
                "num_selected_experts": 1,
                "importance_loss_weight": 0.02,
                "dispatcher": {"name": "einsum", "capacity": 2, "batch_priority": False,
                               "bfloat16": False},
            },
        },
        "dropout_rate": 0.0,
        "attention_dropout_rate": 0.0,
    },
    "classifier": "gap",
    "representation_size": None,
}


def _standardize(x):
  x = np.asarray(x, np.float64)
  return (x - x.mean(-1, keepdims=True)) / np.sqrt(x.var(-1, keepdims=True) + 1e-5)


def test_position_embedding_learned():
  """vmoe/nn/vit_moe_test.py:78-91."""
  x = np.zeros((2, 4, 8), np.float32)
  pos = np.arange(32, dtype=np.float32).reshape(1, 4, 8)
  y, _ = V.encoder_moe(x, {"posembed_input": {"pos_embedding": pos},
                           "encoder_norm": {"bias": np.zeros(8), "scale": np.ones(8)}},
                       num_layers=0, mlp_dim=4, num_heads=1)
  want = _standardize(np.concatenate([pos, pos]))
  np.testing.assert_allclose(y, want, rtol=1e-5, atol=1e-5)


S1, C1 = math.sin(1), math.cos(1)
_SINCOS_ROWS = [
    [0, 0, 1, 1, 0, 0, 1, 1],
    [S1, S1, C1, C1, 0, 0, 1, 1],
    [0, 0, 1, 1, S1, S1, C1, C1],
    [S1, S1, C1, C1, S1, S1, C1, C1],
]


@pytest.mark.parametrize("seq_len,rows", [(4, _SINCOS_ROWS), (5, [[0] * 8] + _SINCOS_ROWS)])
def test_position_embedding_sincos2d(seq_len, rows):
  """vmoe/nn/vit_moe_test.py:93-127."""
  x = np.zeros((2, seq_len, 8), np.float32)
  y, _ = V.encoder_moe(x, {"encoder_norm": {"bias": np.zeros(8), "scale": np.ones(8)}},
                       num_layers=0, mlp_dim=4, num_heads=1,
                       position_emb={"name": "sincos2d", "h": 2, "w": 2, "temperature": 1.})
  pos = np.asarray([rows], np.float64)
  mean = pos.mean(-1, keepdims=True)
  var = pos.var(-1, keepdims=True)
  want = (pos - mean) / np.sqrt(var + 1e-6)
  want = np.concatenate([want, want])
  # the all-zero class-token row has zero variance: standardised to zero on both sides
  np.testing.assert_allclose(y, want, rtol=1e-3, atol=1e-3)


def test_position_embedding_sincos2d_raises():
  """vmoe/nn/vit_moe_test.py:129-135."""
  with pytest.raises(ValueError, match="Unsupported sequence length"):
    V.encoder_moe(np.zeros((2, 6, 8), np.float32),
                  {"encoder_norm": {"bias": np.zeros(8), "scale": np.ones(8)}},
                  num_layers=0, mlp_dim=4, num_heads=1,
                  position_emb={"name": "sincos2d", "h": 2, "w": 2, "temperature": 1.})


def test_layer_norm_vs_torch():
  rng = np.random.default_rng(0)
  x = (rng.standard_normal((5, 7, 48)) * 3 + 1).astype(np.float32)
  scale = rng.standard_normal(48).astype(np.float32)
  bias = rng.standard_normal(48).astype(np.float32)
  want = F.layer_norm(torch.from_numpy(x).double(), (48,), torch.from_numpy(scale).double(),
                      torch.from_numpy(bias).double(), eps=1e-6).numpy()
  np.testing.assert_allclose(V.layer_norm(x, scale, bias, None), want, rtol=2e-5, atol=2e-5)
  got_bf16 = V.layer_norm(x, scale, bias, O.BF16)
  np.testing.assert_array_equal(got_bf16, O.bf16_round(V.layer_norm(x, scale, bias, None)))


def _attention_params(rng, D, H, Dout=None, qk_norm=False):
  hd = D // H
  Dout = Dout or D
  f = lambda *s: (rng.standard_normal(s) / math.sqrt(s[0])).astype(np.float32)
  p = {k: {"kernel": f(D, H, hd), "bias": (rng.standard_normal((H, hd)) * 0.1).astype(np.float32)}
       for k in ("query", "key", "value")}
  p["out"] = {"kernel": f(H, hd, Dout).astype(np.float32),
              "bias": (rng.standard_normal(Dout) * 0.1).astype(np.float32)}
  if qk_norm:
    p["query_ln"] = {"scale": (1 + 0.1 * rng.standard_normal(hd)).astype(np.float32)}
    p["key_ln"] = {"scale": (1 + 0.1 * rng.standard_normal(hd)).astype(np.float32)}
  return p


def test_attention_vs_torch_multi_head_attention():
  """Self- and cross-attention against torch.nn.functional.multi_head_attention_forward
  (float64), whose packed weights are the same projections in (out, in) order."""
  rng = np.random.default_rng(1)
  B, Sq, Sk, D, H = 3, 5, 9, 24, 4
  p = _attention_params(rng, D, H)
  xq = rng.standard_normal((B, Sq, D)).astype(np.float32)
  xkv = rng.standard_normal((B, Sk, D)).astype(np.float32)
  got = V.multi_head_attention(xq, xkv, p, H, None)
  t = lambda a: torch.from_numpy(np.asarray(a)).double()
  w = lambda k: t(p[k]["kernel"]).reshape(D, D).T
  in_proj_w = torch.cat([w("query"), w("key"), w("value")])
  in_proj_b = torch.cat([t(p[k]["bias"]).reshape(D) for k in ("query", "key", "value")])
  want, _ = F.multi_head_attention_forward(
      t(xq).transpose(0, 1), t(xkv).transpose(0, 1), t(xkv).transpose(0, 1), D, H,
      in_proj_w, in_proj_b, None, None, False, 0.0, t(p["out"]["kernel"]).reshape(D, D).T,
      t(p["out"]["bias"]), training=False, need_weights=False)
  np.testing.assert_allclose(got, want.transpose(0, 1).numpy(), rtol=1e-4, atol=1e-5)


def test_attention_brute_force_and_qk_norm():
  """Tiny case by explicit loops, including the per-head layer norm of q and k."""
  rng = np.random.default_rng(2)
  B, S, D, H = 2, 3, 8, 2
  hd = D // H
  p = _attention_params(rng, D, H, qk_norm=True)
  x = rng.standard_normal((B, S, D)).astype(np.float64)
  got = V.multi_head_attention(x.astype(np.float32), x.astype(np.float32), p, H, None, True)
  want = np.zeros((B, S, D))
  for b in range(B):
    ctx = np.zeros((S, H, hd))
    for h in range(H):
      q = x[b] @ p["query"]["kernel"][:, h].astype(np.float64) + p["query"]["bias"][h]
      k = x[b] @ p["key"]["kernel"][:, h].astype(np.float64) + p["key"]["bias"][h]
      v = x[b] @ p["value"]["kernel"][:, h].astype(np.float64) + p["value"]["bias"][h]
      norm = lambda a, s: (a - a.mean(-1, keepdims=True)) / np.sqrt(
          a.var(-1, keepdims=True) + 1e-6) * s
      q, k = norm(q, p["query_ln"]["scale"]), norm(k, p["key_ln"]["scale"])
      for i in range(S):
        logits = np.asarray([q[i] @ k[j] / math.sqrt(hd) for j in range(S)])
        w = np.exp(logits - logits.max())
        w /= w.sum()
        ctx[i, h] = sum(w[j] * v[j] for j in range(S))
    want[b] = ctx.reshape(S, D) @ p["out"]["kernel"].reshape(D, D).astype(np.float64) + p["out"]["bias"]
  np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5)


def test_patch_embedding_vs_torch_conv():
  rng = np.random.default_rng(3)
  img = rng.standard_normal((2, 12, 8, 3)).astype(np.float32)
  kernel = rng.standard_normal((4, 2, 3, 5)).astype(np.float32)    # (ph, pw, Cin, D)
  bias = rng.standard_normal(5).astype(np.float32)
  want = F.conv2d(torch.from_numpy(img).permute(0, 3, 1, 2).double(),
                  torch.from_numpy(kernel).permute(3, 2, 0, 1).double(),
                  torch.from_numpy(bias).double(), stride=(4, 2)).permute(0, 2, 3, 1).numpy()
  np.testing.assert_allclose(V.patch_embedding(img, kernel, bias), want, rtol=1e-5, atol=1e-5)


def _shapes(tree):
  return {k: _shapes(v) if isinstance(v, dict) else tuple(v.shape) for k, v in tree.items()}


@pytest.mark.parametrize("position_emb", [{}, {"name": "sincos2d"}])
def test_initialize_shapes(position_emb):
  """vmoe/nn/vit_moe_test.py:142-187."""
  config = copy.deepcopy(DEFAULT_TEST_CONFIG)
  config["encoder"]["position_emb"] = position_emb
  params = V.init_params(np.random.default_rng(0), (16, 4, 4, 3), **config)
  ln = {"bias": (8,), "scale": (8,)}
  att = {"key": {"bias": (2, 4), "kernel": (8, 2, 4)}, "out": {"bias": (8,), "kernel": (2, 4, 8)},
         "query": {"bias": (2, 4), "kernel": (8, 2, 4)},
         "value": {"bias": (2, 4), "kernel": (8, 2, 4)}}
  want = {
      "Encoder": {
          "encoder_norm": ln,
          "encoderblock_0": {
              "LayerNorm_0": ln, "LayerNorm_1": ln, "SelfAttention": att,
              "Mlp": {"Dense_0": {"bias": (16,), "kernel": (8, 16)},
                      "Dense_1": {"bias": (8,), "kernel": (16, 8)}}},
          "encoderblock_1": {
              "LayerNorm_0": ln, "LayerNorm_1": ln, "SelfAttention": att,
              "Moe": {"Mlp": {"Dense_0": {"bias": (4, 16), "kernel": (4, 8, 16)},
                              "Dense_1": {"bias": (4, 8), "kernel": (4, 16, 8)}},
                      "Router": {"dense": {"kernel": (8, 4)}}}},
      },
      "embedding": {"bias": (8,), "kernel": (2, 2, 3, 8)},
      "head": {"bias": (4,), "kernel": (8, 4)},
  }
  if not position_emb:
    want["Encoder"]["posembed_input"] = {"pos_embedding": (1, 4, 8)}
  assert _shapes(params) == want


@pytest.mark.parametrize("classifier", ["gap", "token", "map"])
def test_forward(classifier):
  """vmoe/nn/vit_moe_test.py:189-199: output shape and the metrics it must carry."""
  config = copy.deepcopy(DEFAULT_TEST_CONFIG)
  config["classifier"] = classifier
  if classifier == "token":
    config["encoder"]["moe"]["group_size"] = 5   # 4 patches + class token per image
  rng = np.random.default_rng(0)
  params = V.init_params(rng, (16, 4, 4, 3), **config)
  x = rng.standard_normal((16, 4, 4, 3)).astype(np.float32)
  out, metrics = V.vision_transformer_moe(x, params, **config)
  assert out.shape == (16, 4) and np.isfinite(out).all()
  assert "auxiliary_loss" in metrics and "encoderblock_1" in metrics
  np.testing.assert_allclose(metrics["auxiliary_loss"],
                             metrics["encoderblock_1"]["auxiliary_loss"])


def test_dense_block_matches_moe_block_with_one_expert():
  """An MoE block with a single expert that takes every item is the dense block."""
  rng = np.random.default_rng(4)
  D, M, H = 8, 16, 2
  base = dict(num_classes=None, patch_size=(2, 2), hidden_size=D, classifier="gap")
  enc = dict(num_layers=1, mlp_dim=M, num_heads=H)
  dense_cfg = dict(base, encoder=enc)
  moe_cfg = dict(base, encoder=dict(enc, moe=dict(
      layers=(0,), num_experts=1, group_size=4,
      router=dict(num_selected_experts=1, dispatcher=dict(name="indices", capacity=4,
                                                          batch_priority=False)))))
  p = V.init_params(np.random.default_rng(5), (3, 4, 4, 3), **dense_cfg)
  pm = copy.deepcopy(p)
  blk = pm["Encoder"]["encoderblock_0"]
  mlp = blk.pop("Mlp")
  blk["Moe"] = {"Router": {"dense": {"kernel": rng.standard_normal((D, 1)).astype(np.float32)}},
                "Mlp": {k: {kk: vv[None] for kk, vv in v.items()} for k, v in mlp.items()}}
  x = rng.standard_normal((3, 4, 4, 3)).astype(np.float32)
  a, _ = V.vision_transformer_moe(x, p, **dense_cfg)
  b, _ = V.vision_transformer_moe(x, pm, **moe_cfg)
  np.testing.assert_allclose(a, b, rtol=1e-6, atol=1e-6)
