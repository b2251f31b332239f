"""The vision transformer around the MoE layer (vmoe_amd.nn.vit_moe) against its
CPU restatement (oracle/vit_oracle.py) and the reference's own tests for it
(vmoe/nn/vit_moe_test.py)."""
import copy
import math

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from oracle import vit_oracle as V
from tests.test_vit_oracle import DEFAULT_TEST_CONFIG, _SINCOS_ROWS, _shapes
from tests.util import assert_close, dev, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def vit_moe():
  from vmoe_amd.nn import vit_moe
  return vit_moe


def tree_to_dev(tree):
  if isinstance(tree, dict):
    return {k: tree_to_dev(v) for k, v in tree.items()}
  return torch.from_numpy(np.ascontiguousarray(tree, dtype=np.float32)).to(dev())


def product_config(config, dtype):
  """The oracle's config with torch dtypes and deterministic=True."""
  config = copy.deepcopy(config)
  config["deterministic"] = True
  config["encoder"]["dtype"] = None if dtype == O.F32 else torch.bfloat16
  return config


def oracle_config(config, dtype):
  config = copy.deepcopy(config)
  config["encoder"]["dtype"] = None if dtype == O.F32 else O.BF16
  return config


# ------------------------------------------------------------------ EncoderMoeTest
def test_position_embedding_learned(vit_moe):
  """vmoe/nn/vit_moe_test.py:78-91."""
  encoder = vit_moe.EncoderMoe(num_layers=0, mlp_dim=4, num_heads=1)
  x = torch.zeros((2, 4, 8), device=dev())
  pos = torch.arange(32, dtype=torch.float32, device=dev()).reshape(1, 4, 8)
  y, _ = encoder.apply({"params": {
      "posembed_input": {"pos_embedding": pos},
      "encoder_norm": {"bias": torch.zeros(8, device=dev()), "scale": torch.ones(8, device=dev())},
  }}, x)
  p = to_np(torch.cat([pos, pos])).astype(np.float64)
  want = (p - p.mean(-1, keepdims=True)) / np.sqrt(p.var(-1, keepdims=True) + 1e-6)
  np.testing.assert_allclose(to_np(y), want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("seq_len,rows", [(4, _SINCOS_ROWS), (5, [[0] * 8] + _SINCOS_ROWS)])
def test_position_embedding_sincos2d(vit_moe, seq_len, rows):
  """vmoe/nn/vit_moe_test.py:93-127."""
  encoder = vit_moe.EncoderMoe(num_layers=0, mlp_dim=4, num_heads=1,
                               position_emb={"name": "sincos2d", "h": 2, "w": 2, "temperature": 1.})
  x = torch.zeros((2, seq_len, 8), device=dev())
  y, _ = encoder.apply({"params": {"encoder_norm": {
      "bias": torch.zeros(8, device=dev()), "scale": torch.ones(8, device=dev())}}}, x)
  pos = np.asarray([rows], np.float64)
  want = (pos - pos.mean(-1, keepdims=True)) / np.sqrt(pos.var(-1, keepdims=True) + 1e-6)
  np.testing.assert_allclose(to_np(y), np.concatenate([want, want]), rtol=1e-3, atol=1e-3)


def test_position_embedding_sincos2d_raises(vit_moe):
  """vmoe/nn/vit_moe_test.py:129-135."""
  encoder = vit_moe.EncoderMoe(num_layers=0, mlp_dim=4, num_heads=1,
                               position_emb={"name": "sincos2d", "h": 2, "w": 2, "temperature": 1.})
  with pytest.raises(ValueError, match="Unsupported sequence length"):
    encoder.init(0, torch.zeros((2, 6, 8), device=dev()))


# ------------------------------------------------------------------ VitMoeTest
@pytest.mark.parametrize("position_emb", [{}, {"name": "sincos2d"}])
def test_initialize_shapes(vit_moe, position_emb):
  """vmoe/nn/vit_moe_test.py:142-187: same tree as the oracle's (which that test pins)."""
  config = product_config(DEFAULT_TEST_CONFIG, O.F32)
  config["encoder"]["position_emb"] = position_emb
  model = vit_moe.VisionTransformerMoe(**config)
  variables = model.init(0, torch.randn((16, 4, 4, 3), device=dev()))
  ocfg = copy.deepcopy(DEFAULT_TEST_CONFIG)
  ocfg["encoder"]["position_emb"] = position_emb
  want = _shapes(V.init_params(np.random.default_rng(0), (16, 4, 4, 3), **ocfg))
  assert _shapes(variables["params"]) == want


def test_forward(vit_moe):
  """vmoe/nn/vit_moe_test.py:189-199."""
  model = vit_moe.VisionTransformerMoe(**product_config(DEFAULT_TEST_CONFIG, O.F32))
  x = torch.randn((16, 4, 4, 3), device=dev())
  variables = model.init(0, x)
  output = model.apply(variables, x)
  assert isinstance(output, tuple)
  output, metrics = output
  assert "auxiliary_loss" in metrics
  assert tuple(output.shape) == (16, 4)


def test_forward_noisy_router(vit_moe):
  """The reference's default test config (vmoe/nn/vit_moe_test.py:28-55) has a noisy
  router: the forward pass needs a 'gating' rng and reports the load loss."""
  config = product_config(DEFAULT_TEST_CONFIG, O.F32)
  config["deterministic"] = False
  config["encoder"]["moe"]["router"].update(noise_std=1e-3, load_loss_weight=0.02)
  model = vit_moe.VisionTransformerMoe(**config)
  x = torch.randn((16, 4, 4, 3), device=dev())
  variables = model.init(0, x)
  with pytest.raises(ValueError, match="rngs"):
    model.apply(variables, x)
  out, metrics = model.apply(variables, x, rngs={"gating": 1})
  assert tuple(out.shape) == (16, 4)
  assert "load_loss" in metrics["encoderblock_1"]
  config["encoder"]["dropout_rate"] = 0.1
  with pytest.raises(NotImplementedError):
    vit_moe.VisionTransformerMoe(**config).apply(variables, x, rngs={"gating": 1})


# ------------------------------------------------------------------ parity with the CPU restatement
@pytest.mark.parametrize("rows,D", [(5, 8), (33, 64), (1000, 768), (7, 1000), (9, 2048), (6, 2052),
                                    (11, 770), (4099, 256)])
@pytest.mark.parametrize("branch_dtype", [None, O.F32, O.BF16])
@pytest.mark.parametrize("out_dtype", [O.F32, O.BF16])
def test_add_layer_norm_kernel(rows, D, branch_dtype, out_dtype):
  from vmoe_amd import kernels as K
  rng = np.random.default_rng(rows * D)
  resid = (rng.standard_normal((rows, D)) * 2 + 0.5).astype(np.float32)
  scale = (1 + 0.2 * rng.standard_normal(D)).astype(np.float32)
  bias = (0.2 * rng.standard_normal(D)).astype(np.float32)
  branch = None
  x = resid
  if branch_dtype is not None:
    branch = O.cast(rng.standard_normal((rows, D)).astype(np.float32), branch_dtype)
    x = resid + branch
  tb = None if branch is None else tree_to_dev(branch).to(
      torch.bfloat16 if branch_dtype == O.BF16 else torch.float32)
  got_x, got_y = K.add_layer_norm(tree_to_dev(resid), tb, tree_to_dev(scale), tree_to_dev(bias),
                                  1e-6, torch.bfloat16 if out_dtype == O.BF16 else torch.float32)
  np.testing.assert_array_equal(to_np(got_x), x)           # one float32 add: exact
  exact = V.layer_norm(x, scale, bias, None)
  if out_dtype == O.F32:
    np.testing.assert_allclose(to_np(got_y), exact, rtol=2e-5, atol=2e-5)
  else:   # within one bfloat16 step of the rounded float32 result
    assert got_y.dtype == torch.bfloat16
    np.testing.assert_allclose(to_np(got_y), exact, rtol=2 ** -7, atol=1e-5)
  # add only, and norm only without parameters
  if branch is not None:
    only_x, none_y = K.add_layer_norm(tree_to_dev(resid), tb, None, None, 1e-6, None)
    assert none_y is None
    np.testing.assert_array_equal(to_np(only_x), x)
  _, plain = K.add_layer_norm(tree_to_dev(resid), None, None, None, 1e-6, torch.float32)
  np.testing.assert_allclose(to_np(plain), V.layer_norm(resid, None, None, None), rtol=2e-5,
                             atol=2e-5)


@pytest.mark.parametrize("B,H,Sq,Sk,packed", [
    (2, 3, 196, 196, True), (2, 2, 197, 197, True), (3, 2, 1, 50, False), (1, 4, 33, 33, True),
    (2, 2, 300, 300, True), (1, 2, 64, 512, False), (1, 1, 40, 7, False)])
def test_attention_kernel(B, H, Sq, Sk, packed):
  """softmax(q k^T / 8) v against float64 on the same bfloat16 operands; operands are
  slices of a packed (B, S, 3, H, 64) projection output or separate tensors."""
  from vmoe_amd import kernels as K
  rng = np.random.default_rng(B * 1000 + Sq + Sk)
  hd = 64
  if packed:
    qkv = torch.from_numpy(rng.standard_normal((B, Sq, 3, H, hd)).astype(np.float32) * 1.5).to(
        dev()).to(torch.bfloat16)
    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
  else:
    mk = lambda S: torch.from_numpy(rng.standard_normal((B, S, H, hd)).astype(np.float32) * 1.5).to(
        dev()).to(torch.bfloat16)
    q, k, v = mk(Sq), mk(Sk), mk(Sk)
  assert K.attention_supported(q, k)
  got = K.attention(q, k, v, hd ** -0.5)
  assert tuple(got.shape) == (B, Sq, H * hd) and got.dtype == torch.bfloat16
  qn, kn, vn = (to_np(t).astype(np.float64) for t in (q, k, v))
  logits = np.einsum("bqhd,bkhd->bhqk", qn, kn) / 8.0
  w = np.exp(logits - logits.max(-1, keepdims=True))
  w /= w.sum(-1, keepdims=True)
  want = np.einsum("bhqk,bkhd->bqhd", w, vn).reshape(B, Sq, H * hd)
  assert_close(to_np(got), want, 1e-2, "attention kernel")


@pytest.mark.parametrize("dtype", [O.F32, O.BF16])
@pytest.mark.parametrize("cross,qk_norm,D", [(False, False, 128), (True, False, 128),
                                             (False, True, 128), (False, False, 256),
                                             (False, True, 256)])
def test_attention_vs_oracle(vit_moe, dtype, cross, qk_norm, D):
  from tests.test_vit_oracle import _attention_params
  rng = np.random.default_rng(3)
  B, Sq, Sk, H = 4, 1 if cross else 50, 50, 4
  p = _attention_params(rng, D, H, qk_norm=qk_norm)
  xq = O.cast(rng.standard_normal((B, Sq, D)).astype(np.float32), dtype)
  xkv = O.cast(rng.standard_normal((B, Sk, D)).astype(np.float32), dtype) if cross else xq
  odt = None if dtype == O.F32 else O.BF16
  tdt = None if dtype == O.F32 else torch.bfloat16
  want = V.multi_head_attention(xq, xkv, p, H, odt, qk_norm)
  layer = vit_moe.MultiHeadDotProductAttention(num_heads=H, dtype=tdt, normalize_qk=qk_norm)
  tq = tree_to_dev(xq)
  got = layer.apply({"params": tree_to_dev(p)}, tq, tree_to_dev(xkv) if cross else None)
  assert got.dtype == (torch.float32 if dtype == O.F32 else torch.bfloat16)
  if dtype == O.F32:
    assert_close(to_np(got), want, 1e-4, "attention")
    return
  # bfloat16: flax holds logits and probabilities in bfloat16, the fused library
  # attention keeps them in float32 until the second product, so single elements
  # differ by a few bfloat16 steps of the output sum.  Bound that, and require the
  # GPU result to be at least as close to the float32 answer as the restatement is.
  assert_close(to_np(got), want, 5e-2, "attention")
  exact = V.multi_head_attention(xq, xkv, p, H, None, qk_norm)
  rms = lambda a: float(np.sqrt(np.mean(np.square(a, dtype=np.float64))))
  assert rms(to_np(got) - exact) <= 1.1 * rms(want - exact)


SMALL = {
    "num_classes": 10,
    "patch_size": (4, 4),
    "hidden_size": 64,
    "encoder": {
        "num_layers": 3,
        "mlp_dim": 128,
        "num_heads": 4,
        "moe": {
            "layers": (1,),
            "num_experts": 4,
            "group_size": 32,
            "router": {"num_selected_experts": 2,
                       "dispatcher": {"name": "indices", "capacity_factor": 1.5,
                                      "batch_priority": True}},
        },
    },
    "classifier": "gap",
    "representation_size": None,
}


def _variant(**changes):
  cfg = copy.deepcopy(SMALL)
  for k, v in changes.items():
    if k in cfg:
      cfg[k] = v
    else:
      cfg["encoder"][k] = v
  return cfg


VARIANTS = {
    "gap": _variant(),
    "token": _variant(classifier="token", moe=dict(SMALL["encoder"]["moe"], group_size=34)),
    "map_qknorm": _variant(classifier="map", attention_qk_norm=True, representation_size=48),
    "sincos2d_einsum": _variant(
        position_emb={"name": "sincos2d"},
        moe=dict(SMALL["encoder"]["moe"], router={
            "num_selected_experts": 1,
            "dispatcher": {"name": "einsum", "capacity": 12, "batch_priority": False}})),
    "all_moe": _variant(moe=dict(SMALL["encoder"]["moe"], layers=(0, 1, 2))),
}


@pytest.mark.parametrize("name", sorted(VARIANTS))
def test_model_fp32_vs_oracle(vit_moe, name):
  cfg = VARIANTS[name]
  rng = np.random.default_rng(11)
  images = rng.uniform(-1, 1, (8, 16, 16, 3)).astype(np.float32)     # 16 patches per image
  params = V.init_params(rng, images.shape, **cfg)
  want, want_metrics = V.vision_transformer_moe(images, params, **oracle_config(cfg, O.F32))
  model = vit_moe.VisionTransformerMoe(**product_config(cfg, O.F32))
  got, metrics = model.apply({"params": tree_to_dev(params)}, tree_to_dev(images))
  assert got.dtype == torch.float32 and tuple(got.shape) == want.shape
  assert_close(to_np(got), want, 2e-4, f"{name} logits")
  assert set(metrics) == set(want_metrics)
  np.testing.assert_allclose(to_np(metrics["auxiliary_loss"]),
                             np.asarray(want_metrics["auxiliary_loss"]), rtol=1e-3, atol=1e-6)


def test_model_bf16_vs_oracle(vit_moe):
  """bfloat16 encoder (the residual stream stays float32, as under jnp promotion).
  Rounding differs inside attention, and an item whose two best gates are nearly
  equal can be routed differently: compared at the 2e-2 of bfloat16 parity on the
  scale of the logits, for all but a few images."""
  cfg = VARIANTS["gap"]
  rng = np.random.default_rng(12)
  images = rng.uniform(-1, 1, (16, 16, 16, 3)).astype(np.float32)
  params = V.init_params(rng, images.shape, **cfg)
  want, _ = V.vision_transformer_moe(images, params, **oracle_config(cfg, O.BF16))
  model = vit_moe.VisionTransformerMoe(**product_config(cfg, O.BF16))
  got, metrics = model.apply({"params": tree_to_dev(params)}, tree_to_dev(images))
  assert got.dtype == torch.float32
  err = np.abs(to_np(got) - want)
  scale = float(np.sqrt(np.mean(want ** 2)))
  bad_images = (err.max(axis=1) > 2e-2 * (scale + np.abs(want).max(axis=1))).sum()
  assert bad_images <= 1, f"{bad_images} of {len(want)} images outside 2e-2 (scale {scale:.3f})"
  assert np.isfinite(to_np(metrics["auxiliary_loss"])).all()


def test_model_b16_width_bf16_vs_oracle(vit_moe):
  """The full model's real width (hidden 768, 12 heads of 64, mlp 3072, 224 px images in
  16 x 16 patches, 1000 classes, global average pooling, bfloat16 encoder) on three
  blocks, the middle one sparse as in the B/16 model (E = 8, top-2 with batch priority
  routing, capacity factor 1.05, groups of 8 images): 16 images, two routing groups."""
  from vmoe_amd import configs
  cfg = configs.vit_b16_moe_model(dtype=None)
  cfg["encoder"]["num_layers"] = 3
  cfg["encoder"]["moe"]["layers"] = (1,)
  cfg.pop("deterministic")
  cfg.pop("head_kernel_zero_init")
  rng = np.random.default_rng(21)
  images = rng.uniform(-1, 1, (16, 224, 224, 3)).astype(np.float32)
  params = V.init_params(rng, images.shape, **cfg)
  want, want_metrics = V.vision_transformer_moe(images, params, **oracle_config(cfg, O.BF16))
  model = vit_moe.VisionTransformerMoe(**product_config(cfg, O.BF16))
  got, metrics = model.apply({"params": tree_to_dev(params)}, tree_to_dev(images))
  assert got.dtype == torch.float32 and tuple(got.shape) == want.shape == (16, 1000)
  err = np.abs(to_np(got) - want)
  scale = float(np.sqrt(np.mean(want ** 2)))
  bad_images = (err.max(axis=1) > 2e-2 * (scale + np.abs(want).max(axis=1))).sum()
  print(f"b16 width: images outside 2e-2: {bad_images} / {len(want)}; max err {err.max():.3e}, scale {scale:.3f}")
  assert bad_images <= 1, f"{bad_images} of {len(want)} images outside 2e-2 (scale {scale:.3f})"
  np.testing.assert_allclose(to_np(metrics["auxiliary_loss"]),
                             np.asarray(want_metrics["auxiliary_loss"]), rtol=2e-2, atol=1e-4)


def test_full_model_follows_a_permutation_of_its_routing_groups(vit_moe):
  """The full B/16 model at the benchmark's size (12 blocks, six of them sparse, batch 512 at
  224 px, bfloat16 encoder), random parameters: attention, layer norms and dense blocks work
  image by image and the sparse blocks group by group (8 consecutive images), so permuting
  whole groups of the batch permutes the logits.  The vendor library's projections may add
  in another order for rows at other positions, and a gate that moves by one rounding step
  can flip a routing decision, so images are compared at the tolerance of the oracle tests and
  a small fraction may lie outside; every logit must be finite."""
  from vmoe_amd import configs
  B, group = configs.VIT_B16_MOE_BATCH, 8
  model = vit_moe.VisionTransformerMoe(**configs.vit_b16_moe_model(dtype=torch.bfloat16))
  gen = torch.Generator(device=dev())
  gen.manual_seed(7)
  images = torch.rand((B, 224, 224, 3), generator=gen, device=dev()) * 2 - 1
  variables = model.init(0, images)
  logits, metrics = model.apply(variables, images)
  assert tuple(logits.shape) == (B, 1000) and torch.isfinite(logits).all()
  perm = torch.randperm(B // group, generator=torch.Generator().manual_seed(1)).to(dev())
  index = (perm[:, None] * group + torch.arange(group, device=dev())[None, :]).reshape(-1)
  logits_p, _ = model.apply(variables, images[index].contiguous())
  want = logits[index]
  scale = want.square().mean().sqrt()
  bad = ((logits_p - want).abs() > 2e-2 * (scale + want.abs())).any(-1)
  print(f"full model: {int(bad.sum())} of {B} images outside 2e-2 under a permutation of the groups; "
        f"identical logits on {int((logits_p == want).all(-1).sum())}")
  assert bad.sum().item() <= B // 50
  assert not torch.equal(logits_p, logits)


def test_model_from_checkpoint_files(vit_moe, tmp_path):
  """A dense model's parameters written in the reference's sharded checkpoint format,
  read back, upcycled (every expert a copy of the dense MLP) and run on the GPU."""
  from vmoe_amd import checkpoints as C
  dense_cfg = copy.deepcopy(SMALL)
  dense_cfg["encoder"].pop("moe")
  rng = np.random.default_rng(31)
  images = rng.uniform(-1, 1, (8, 16, 16, 3)).astype(np.float32)
  dense = V.init_params(rng, images.shape, **dense_cfg)
  prefix = str(tmp_path / "ckpt_1")
  C.save_checkpoint(prefix, {"params": dense}, num_shards=3, max_chunk_bytes=4096)
  restored = C.restore_checkpoint(prefix)["params"]
  sparse = C.dense_to_moe_params(restored, moe_layers=(1,), num_experts=4)
  want, _ = V.vision_transformer_moe(images, sparse, **oracle_config(SMALL, O.F32))
  model = vit_moe.VisionTransformerMoe(**product_config(SMALL, O.F32))
  got, _ = model.apply({"params": C.to_device(sparse, dev())}, tree_to_dev(images))
  assert_close(to_np(got), want, 2e-4, "logits from restored parameters")
