"""Rules and tree mapping (vmoe_amd/initialization.py).  CPU only.

The cases and expected values are those of the reference's own tests,
vmoe/initialization/mapping_test.py:44-189 and vmoe/initialization/rules_test.py:24-146,
with NumPy / torch leaves in place of jax arrays (``ShapeDtype`` for
jax.ShapeDtypeStruct)."""
import numpy as np
import pytest
import torch

from vmoe_amd import checkpoints as C
from vmoe_amd import initialization as I

f32 = np.float32


def ones(*shape):
  return np.ones(shape, f32)


def zeros(*shape):
  return np.zeros(shape, f32)


def test_rename_with_groups():
  # mapping_test.py:46-63 (two Dense layers renamed layer_N)
  rng = np.random.default_rng(0)
  source = {"params": {f"Dense_{i}": {"kernel": rng.standard_normal((3 + 5 * i, 8 * (i + 1))).astype(f32),
                                      "bias": rng.standard_normal(8 * (i + 1)).astype(f32)} for i in range(2)}}
  target = {"params": {f"layer_{i}": {"kernel": I.ShapeDtype((3 + 5 * i, 8 * (i + 1))),
                                      "bias": I.ShapeDtype((8 * (i + 1),))} for i in range(2)}}
  out = I.map_state_dict(source, target, [(r"params/Dense_(\d+)/(kernel|bias)", r"params/layer_\1/\2")])
  for i in range(2):
    for leaf in ("kernel", "bias"):
      np.testing.assert_array_equal(out["params"][f"layer_{i}"][leaf], source["params"][f"Dense_{i}"][leaf])


def test_skip_name():
  out = I.map_state_dict({"a": zeros(1), "b": ones(2)}, {"c": ones(1)}, [("a", "c"), ("b", None)])
  assert set(out) == {"c"}
  np.testing.assert_array_equal(out["c"], zeros(1))


def test_transform_expand_tile():
  out = I.map_state_dict({"a": ones(1), "b": ones(2)}, {"c": zeros(5, 1), "d": zeros(4, 2, 3)},
                         [("a", "c", "expand_tile", 0, 5), ("b", "d", "expand_tile", (0, 2), (4, 3))])
  np.testing.assert_array_equal(out["c"], ones(5, 1))
  np.testing.assert_array_equal(out["d"], ones(4, 2, 3))


def test_transform_reshape():
  out = I.map_state_dict({"a": zeros(4, 3, 2), "b": zeros(3, 2)}, {"c": ones(4, 6), "d": ones(6)},
                         [("a", "c", "reshape", (4, 6)), ("b", "d", "reshape")])
  np.testing.assert_array_equal(out["c"], zeros(4, 6))
  np.testing.assert_array_equal(out["d"], zeros(6))


def test_transform_squeeze():
  out = I.map_state_dict({"a": zeros(4, 1, 2)}, {"b": ones(4, 2)}, [("a", "b", "squeeze", 1)])
  np.testing.assert_array_equal(out["b"], zeros(4, 2))


def test_transform_stack_natural_order():
  source = {"a_0": 1 * ones(1), "a_1": 2 * ones(1), "a_11": 3 * ones(1), "a_2": 4 * ones(1)}
  out = I.map_state_dict(source, {"b": zeros(1, 4)}, [(r"a_\d+", "b", "stack", 1)])
  np.testing.assert_array_equal(out["b"], [[1, 2, 4, 3]])


def test_shape_mismatch():
  with pytest.raises(ValueError, match="Target key .* has mismatched shapes."):
    I.map_state_dict({"a": zeros(1)}, {"b": ones(2)}, [("a", "b")])
  out = I.map_state_dict({"a": zeros(1)}, {"b": ones(1, 1, 1)}, [("a", "b")],
                         raise_if_shape_mismatched=False)
  np.testing.assert_array_equal(out["b"], zeros(1, 1, 1))


def test_dtype_mismatch():
  out = I.map_state_dict({"a": np.zeros(2, np.float64)}, {"b": ones(2)}, [("a", "b")])
  assert out["b"].dtype == f32
  with pytest.raises(ValueError, match="Target key .* has mismatched dtypes."):
    I.map_state_dict({"a": np.zeros(2, np.float64)}, {"b": ones(2)}, [("a", "b")],
                     raise_if_dtype_mismatched=True)


def test_source_unmatched():
  with pytest.raises(KeyError, match="Source key .* does not match"):
    I.map_state_dict({"a": zeros(1)}, {"a": ones(1)}, [])
  out = I.map_state_dict({"a": zeros(1)}, {"a": ones(1)}, [], raise_if_source_unmatched=False)
  np.testing.assert_array_equal(out["a"], zeros(1))


def test_target_unmatched():
  with pytest.raises(ValueError, match="Target key .* is unmatched"):
    I.map_state_dict({"a": zeros(1)}, {"b": ones(1), "c": zeros(2)}, [("a", "b")])
  out = I.map_state_dict({"a": zeros(1)}, {"b": ones(1), "c": zeros(2)}, [("a", "b")],
                         raise_if_target_unmatched=False)
  assert set(out) == {"b", "c"}
  np.testing.assert_array_equal(out["b"], zeros(1))
  np.testing.assert_array_equal(out["c"], zeros(2))


def test_target_not_exists_and_matched_twice():
  with pytest.raises(KeyError, match=r"Source key .* was matched with target key .*, but it does not exist\."):
    I.map_state_dict({"a": zeros(1)}, {"b": ones(2)}, [("a", "c")])
  with pytest.raises(ValueError, match="was matched more than once"):
    I.map_state_dict({"a1": zeros(1), "a2": zeros(1)}, {"b": ones(1)}, [(r"a\d", "b")])


def test_unknown_transform():
  with pytest.raises(ValueError, match=r"Rule .* cannot be parsed\."):
    I.map_state_dict({"a": zeros(1)}, {"b": ones(1)}, [("a", "b", "unknown")])


def test_empty_nodes():
  out = I.map_state_dict({"a": {}, "b": ones(1)}, {"a": {}, "b": zeros(1)}, [("(.*)", r"\1")])
  assert out == {"a": {}, "b": ones(1)}
  with pytest.raises(ValueError, match="empty node"):
    I.map_state_dict({"a": {}}, {"a": zeros(1)}, [("(.*)", r"\1")])


@pytest.mark.parametrize("x,expected", [
    (["c/3", "a/1", "b/2"], ["a/1", "b/2", "c/3"]),
    (["a0", "a11", "a3"], ["a0", "a3", "a11"]),
])
def test_natural_sort(x, expected):
  assert I._natural_sort(x) == expected


def test_zoom_rule():
  rules = I.Rules.parse([("a", "b", "zoom")])
  assert len(rules.rules) == 1 and isinstance(rules.rules[0], I.ZoomRule)
  out = I.map_state_dict({"a": ones(6, 4, 8)}, {"b": I.ShapeDtype((6, 8, 12))}, rules)
  np.testing.assert_allclose(out["b"], ones(6, 8, 12))


def test_vit_zoom_rule():
  rules = I.Rules.parse([("a", "b", "vit_zoom")])
  assert len(rules.rules) == 1 and isinstance(rules.rules[0], I.VitZoomRule)
  # no token on either side
  out = I.map_state_dict({"a": ones(1, 64, 14)}, {"b": I.ShapeDtype((1, 16, 14))}, rules)
  np.testing.assert_allclose(out["b"], ones(1, 16, 14))
  # token on both sides: kept from the source
  out = I.map_state_dict({"a": ones(1, 65, 14)}, {"b": zeros(1, 17, 14)}, rules)
  np.testing.assert_allclose(out["b"], ones(1, 17, 14))
  # token only in the target array: its own row survives
  out = I.map_state_dict({"a": ones(1, 64, 14)}, {"b": zeros(1, 17, 14)}, rules)
  np.testing.assert_allclose(out["b"], np.concatenate([zeros(1, 1, 14), ones(1, 16, 14)], axis=1))
  # token only in a target known by shape: row 0 is noise, the grid is interpolated
  out = I.map_state_dict({"a": ones(1, 64, 14)}, {"b": I.ShapeDtype((1, 17, 14))}, rules)
  np.testing.assert_allclose(out["b"][:, 1:], ones(1, 16, 14))
  assert np.abs(out["b"][:, 0]).max() < 0.2
  with pytest.raises(ValueError, match="perfect square"):
    I.map_state_dict({"a": ones(1, 63, 14)}, {"b": zeros(1, 17, 14)}, rules)


def test_torch_leaves_keep_dtype_and_device():
  source = {"w": np.arange(6, dtype=f32).reshape(2, 3)}
  target = {"experts": {"w": torch.zeros(4, 2, 3, dtype=torch.bfloat16)}, "keep": torch.ones(2)}
  out = I.map_state_dict(source, target, [("w", "experts/w", "expand_tile", 0, 4)],
                         raise_if_target_unmatched=False)
  assert out["experts"]["w"].dtype == torch.bfloat16 and tuple(out["experts"]["w"].shape) == (4, 2, 3)
  np.testing.assert_array_equal(out["experts"]["w"].float().numpy(), np.tile(source["w"], (4, 1, 1)))
  assert out["keep"] is target["keep"]
  # torch sources work too
  out = I.map_state_dict({"w": torch.full((2,), 3.0)}, {"v": zeros(2)}, [("w", "v")])
  np.testing.assert_array_equal(out["v"], 3 * ones(2))


def test_upcycling_rules_on_a_block(tmp_path):
  """Dense ViT block -> sparse block with the rules of the reference's upcycling configs
  (expand_tile of the MLP over a new expert axis), read from a checkpoint on disk."""
  rng = np.random.default_rng(1)
  E, D, M = 4, 8, 16
  dense = {"target": {"Encoder": {
      "encoderblock_1": {"Mlp": {"Dense_0": {"kernel": rng.standard_normal((D, M)).astype(f32),
                                             "bias": rng.standard_normal(M).astype(f32)},
                                 "Dense_1": {"kernel": rng.standard_normal((M, D)).astype(f32),
                                             "bias": rng.standard_normal(D).astype(f32)}}},
      "posembed_input": {"pos_embedding": rng.standard_normal((1, 16, D)).astype(f32)}}},
           "opt_state": {"mu": zeros(3)}}
  C.save_checkpoint(str(tmp_path / "ckpt"), dense, num_shards=2)
  router = rng.standard_normal((D, E)).astype(f32)
  target = {"params": {"Encoder": {
      "encoderblock_1": {"Moe": {"Mlp": {"Dense_0": {"kernel": I.ShapeDtype((E, D, M)), "bias": I.ShapeDtype((E, M))},
                                         "Dense_1": {"kernel": I.ShapeDtype((E, M, D)), "bias": I.ShapeDtype((E, D))}},
                                 "Router": {"dense": {"kernel": router}}}},
      "posembed_input": {"pos_embedding": I.ShapeDtype((1, 64, D))}}}}
  rules = [
      (r"opt_state/.*", None),
      (r"target/(Encoder/encoderblock_\d+)/Mlp/(.*)", r"params/\1/Moe/Mlp/\2", "expand_tile", 0, E),
      (r"target/(.*pos_embedding)", r"params/\1", "vit_zoom"),
      (r"target/(.*)", r"params/\1"),
  ]
  out = I.initialize_from_vmoe(target=target, prefix=str(tmp_path / "ckpt"), rules=rules, mesh=None,
                               raise_if_target_unmatched=False)
  blk = out["params"]["Encoder"]["encoderblock_1"]["Moe"]
  src = dense["target"]["Encoder"]["encoderblock_1"]["Mlp"]
  for d in ("Dense_0", "Dense_1"):
    for leaf in ("kernel", "bias"):
      got = blk["Mlp"][d][leaf]
      assert got.shape[0] == E
      for e in range(E):
        np.testing.assert_array_equal(got[e], src[d][leaf])
  assert blk["Router"]["dense"]["kernel"] is router
  pe = out["params"]["Encoder"]["posembed_input"]["pos_embedding"]
  np.testing.assert_allclose(pe, C.vit_zoom(dense["target"]["Encoder"]["posembed_input"]["pos_embedding"], (1, 64, D)))


def test_initialize_from_vit_npz(tmp_path):
  rng = np.random.default_rng(2)
  kernel = rng.standard_normal((3, 5)).astype(f32)
  as_bf16 = (kernel.view(np.uint32) >> 16).astype(np.uint16)          # truncated bit patterns
  path = str(tmp_path / "vit.npz")
  np.savez(path, **{"Transformer/encoderblock_0/MlpBlock_3/Dense_0/kernel": kernel,
                    "head/kernel": as_bf16.view(np.dtype("V2"))})
  target = {"Encoder": {"encoderblock_0": {"Mlp": {"Dense_0": {"kernel": I.ShapeDtype((3, 5))}}}},
            "head": {"kernel": I.ShapeDtype((3, 5))}}
  out = I.initialize_from_vit(target=target, filepath=path, mesh=None, rules=[
      (r"Transformer/(encoderblock_\d+)/MlpBlock_\d+/(.*)", r"Encoder/\1/Mlp/\2"),
      (r"(head/.*)", r"\1")])
  np.testing.assert_array_equal(out["Encoder"]["encoderblock_0"]["Mlp"]["Dense_0"]["kernel"], kernel)
  np.testing.assert_array_equal(out["head"]["kernel"], (as_bf16.astype(np.uint32) << 16).view(f32))
