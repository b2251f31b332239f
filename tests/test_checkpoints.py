"""Reader / writer of the reference's sharded checkpoint format and the upcycling
transformations (vmoe_amd/checkpoints.py).  CPU only.

No file produced by the reference exists here, so the format is checked by round
trips and by a byte string assembled by hand from the layout stated in
vmoe/checkpoints/serialization.py:148-330 — parity with real checkpoint files is
unpinned."""
import os

import msgpack
import numpy as np
import pytest
import scipy.ndimage

from vmoe_amd import checkpoints as C


def _tree(rng):
  return {
      "params": {
          "Encoder": {
              "encoderblock_0": {"Mlp": {"Dense_0": {"kernel": rng.standard_normal((8, 16)).astype(np.float32),
                                                     "bias": rng.standard_normal(16).astype(np.float32)}}},
              "posembed_input": {"pos_embedding": rng.standard_normal((1, 17, 8)).astype(np.float32)},
          },
          "head": {"kernel": C.bfloat16_bits(rng.standard_normal((8, 4)).astype(np.float32)),
                   "bias": np.zeros(4, np.float32)},
      },
      "step": np.asarray(1234, np.int32),
      "big": rng.integers(0, 255, size=(64, 33), dtype=np.uint8),
  }


def _assert_tree_equal(a, b):
  assert sorted(a) == sorted(b)
  for k in a:
    if isinstance(a[k], dict):
      _assert_tree_equal(a[k], b[k])
    else:
      want = a[k].to_float32() if hasattr(a[k], "to_float32") else a[k]
      np.testing.assert_array_equal(b[k], want)
      assert b[k].dtype == want.dtype and b[k].shape == want.shape


@pytest.mark.parametrize("num_shards,max_chunk_bytes", [(1, None), (3, None), (4, 200)])
def test_round_trip(tmp_path, num_shards, max_chunk_bytes):
  tree = _tree(np.random.default_rng(0))
  prefix = str(tmp_path / "ckpt" / "checkpoint_7")
  files = C.save_checkpoint(prefix, tree, num_shards=num_shards, max_chunk_bytes=max_chunk_bytes)
  assert sorted(os.path.basename(f) for f in files) == sorted(
      [f"checkpoint_7.data-{i:05d}-of-{num_shards:05d}" for i in range(num_shards)]
      + ["checkpoint_7.index"])
  _assert_tree_equal(tree, C.restore_checkpoint(prefix))
  if max_chunk_bytes:   # the big leaves really were cut and spread over the shards
    with open(prefix + ".index", "rb") as fp:
      index = C.msgpack_restore(fp.read())
    info = index["index"]["big"]
    assert len(info.global_slices) > 1 and len(set(info.shards)) > 1
    assert info.global_shape.shape == (64, 33) and info.global_shape.dtype == "uint8"


def test_hand_assembled_files(tmp_path):
  """Index and data shard written byte by byte with msgpack from the layout the reference's
  encoders state: ext 8 = (ext-4 payload, (slice-nd payloads), shards), ext 6 = (slice
  payloads), slice payload = (start, stop, step), ext 1 = (shape, dtype name, bytes)."""
  pk = lambda o: msgpack.packb(o, use_bin_type=True)
  sl = lambda a, b: pk((a, b, None))
  snd = lambda *pairs: pk(tuple(sl(a, b) for a, b in pairs))
  arr = np.arange(12, dtype=np.float32).reshape(4, 3)
  info_a = pk((pk(((4, 3), "float32", False, {})), (snd((0, 2), (0, 3)), snd((2, 4), (0, 3))), (0, 1)))
  info_b = pk((pk(((2,), "bfloat16", False, {})), (snd((0, 2)),), (1,)))
  info_s = pk((pk(((), "int32", False, {})), (snd(),), (0,)))          # a scalar leaf: no slices
  index = msgpack.packb({"shard_count": 2, "version": "20220622",
                         "index": {"w": msgpack.ExtType(8, info_a), "b": msgpack.ExtType(8, info_b),
                                   "step": msgpack.ExtType(8, info_s)}})
  nd = lambda a, name=None: msgpack.ExtType(1, pk((a.shape, name or a.dtype.name, a.tobytes())))
  magic = "__msgpack_array_chunk_a87ca2__"
  bf = np.asarray([0x3F80, 0xC000], np.uint16)          # 1.0, -2.0
  # leaf ids follow sorted keys: b = 0, step = 1, w = 2
  shard0 = msgpack.packb({magic: True, "2": [[[nd(arr[:2].reshape(-1))], msgpack.ExtType(6, snd((0, 2), (0, 3)))]],
                          "1": [[[nd(np.asarray([7], np.int32))], msgpack.ExtType(6, snd())]]})
  shard1 = msgpack.packb({magic: True,
                          "2": [[[nd(arr[2:].reshape(-1)[:4]), nd(arr[2:].reshape(-1)[4:])],
                                 msgpack.ExtType(6, snd((2, 4), (0, 3)))]],
                          "0": [[[nd(bf, "bfloat16")], msgpack.ExtType(6, snd((0, 2)))]]})
  prefix = str(tmp_path / "c")
  for name, data in [(".index", index), (".data-00000-of-00002", shard0), (".data-00001-of-00002", shard1)]:
    with open(prefix + name, "wb") as fp:
      fp.write(data)
  out = C.restore_checkpoint(prefix)
  np.testing.assert_array_equal(out["w"], arr)
  np.testing.assert_array_equal(out["b"], np.asarray([1.0, -2.0], np.float32))
  assert np.asarray(out["step"]).shape == () and int(out["step"]) == 7


def test_errors(tmp_path):
  prefix = str(tmp_path / "c")
  with open(prefix + ".index", "wb") as fp:
    fp.write(msgpack.packb({"shard_count": 1, "index": {}}))
  with pytest.raises(NotImplementedError, match="version"):
    C.restore_checkpoint(prefix)
  tree = {"a": np.arange(6, dtype=np.float32)}
  C.save_checkpoint(prefix, tree, num_shards=2, max_chunk_bytes=8)
  os.remove(prefix + ".data-00001-of-00002")
  with pytest.raises(FileNotFoundError):
    C.restore_checkpoint(prefix)


def test_flax_chunked_array():
  """flax splits arrays above 2**30 bytes into {'__msgpack_chunked_array__', 'shape', 'chunks'}."""
  a = np.arange(10, dtype=np.int64)
  nd = lambda x: msgpack.ExtType(1, msgpack.packb((x.shape, x.dtype.name, x.tobytes()), use_bin_type=True))
  enc = msgpack.packb({"x": {"__msgpack_chunked_array__": True, "shape": {"0": 2, "1": 5},
                             "chunks": {"0": nd(a[:6]), "1": nd(a[6:])}}})
  np.testing.assert_array_equal(C.msgpack_restore(enc)["x"], a.reshape(2, 5))


def test_bfloat16_bits_round_to_nearest_even():
  import torch
  x = np.random.default_rng(1).standard_normal(4096).astype(np.float32)
  want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
  np.testing.assert_array_equal(C.bfloat16_bits(x).bits, want)


def test_expand_tile():
  """vmoe/initialization/rules.py:242-258 == expand_dims + tile."""
  a = np.arange(6).reshape(2, 3)
  out = C.expand_tile(a, 0, 4)
  assert out.shape == (4, 2, 3) and all((out[e] == a).all() for e in range(4))
  out = C.expand_tile(a, (0, 2), (2, 3))
  assert out.shape == (2, 2, 3, 3)
  np.testing.assert_array_equal(out, np.tile(a[None, :, None, :], (2, 1, 3, 1)))
  with pytest.raises(ValueError):
    C.expand_tile(a, (0, 1), 2)


def test_vit_zoom():
  """vmoe/initialization/rules.py:328-381: grid part through scipy.ndimage.zoom(order=1),
  class-token row carried over."""
  rng = np.random.default_rng(2)
  src = rng.standard_normal((1, 1 + 4 * 4, 8)).astype(np.float32)
  out = C.vit_zoom(src, (1, 1 + 6 * 6, 8))
  assert out.shape == (1, 37, 8)
  np.testing.assert_array_equal(out[:, :1], src[:, :1])
  want = scipy.ndimage.zoom(src[:, 1:].reshape(1, 4, 4, 8), (1, 1.5, 1.5, 1), order=1)
  np.testing.assert_array_equal(out[:, 1:].reshape(1, 6, 6, 8), want)
  # no token on either side; identity when the grids agree
  grid = rng.standard_normal((1, 9, 8)).astype(np.float32)
  np.testing.assert_allclose(C.vit_zoom(grid, (1, 9, 8)), grid, rtol=1e-6)
  assert C.vit_zoom(grid, (1, 16, 8)).shape == (1, 16, 8)
  # token wanted but the source has none: taken from the target array
  tgt = rng.standard_normal((1, 17, 8)).astype(np.float32)
  out = C.vit_zoom(grid, (1, 17, 8), target=tgt)
  np.testing.assert_array_equal(out[:, :1], tgt[:, :1])
  with pytest.raises(ValueError, match="perfect square"):
    C.vit_zoom(rng.standard_normal((1, 7, 8)), (1, 9, 8))
  with pytest.raises(ValueError):
    C.vit_zoom(grid, (1, 9, 4))


def test_dense_to_moe_params():
  from oracle import vit_oracle as V
  cfg = dict(num_classes=5, patch_size=(4, 4), hidden_size=16, classifier="gap",
             encoder=dict(num_layers=2, mlp_dim=32, num_heads=2))
  dense = V.init_params(np.random.default_rng(3), (2, 8, 8, 3), **cfg)
  sparse = C.dense_to_moe_params(dense, moe_layers=(1,), num_experts=4)
  blk = sparse["Encoder"]["encoderblock_1"]
  assert "Mlp" not in blk and blk["Moe"]["Router"]["dense"]["kernel"].shape == (16, 4)
  assert blk["Moe"]["Mlp"]["Dense_0"]["kernel"].shape == (4, 16, 32)
  assert blk["Moe"]["Mlp"]["Dense_1"]["bias"].shape == (4, 16)
  assert "Mlp" in dense["Encoder"]["encoderblock_1"]          # the input tree is untouched
  # every expert starts as the dense MLP: with all experts equal and capacity for every
  # item, the sparse model computes gate-weighted copies of the dense MLP's output
  x = np.random.default_rng(4).standard_normal((2, 8, 8, 3)).astype(np.float32)
  moe_cfg = dict(cfg, encoder=dict(cfg["encoder"], moe=dict(
      layers=(1,), num_experts=4, group_size=4,
      router=dict(num_selected_experts=4, dispatcher=dict(name="indices", capacity=4,
                                                          batch_priority=False)))))
  a, _ = V.vision_transformer_moe(x, dense, **cfg)
  b, _ = V.vision_transformer_moe(x, sparse, **moe_cfg)   # gates of the 4 picks sum to 1
  np.testing.assert_allclose(a, b, rtol=2e-5, atol=2e-5)
