"""Reader (and writer) of the reference's sharded checkpoint files, and the array
transformations it uses to initialise a sparse model from a dense one.

File format (vmoe/checkpoints/partitioned.py:89-125, 131-260, 417-540 and
vmoe/checkpoints/serialization.py:58-330): a checkpoint ``prefix`` is

  ``prefix.index``                      msgpack of ``{'shard_count': n, 'index': tree,
                                        'version': '20220622'}``; the leaves of ``tree``
                                        are IndexInfo records (global shape and dtype,
                                        the slices the array was cut into, the shard
                                        holding each slice);
  ``prefix.data-00000-of-0000n`` ...    msgpack of ``{magic: True, '<leaf id>': [[[sub-chunks],
                                        slice], ...]}``: flattened pieces of the leaves,
                                        leaf ids counting the index tree's leaves in
                                        sorted-key depth-first order.

Arrays and the record types travel as msgpack extension types 1-8
(serialization.py:148-157); arrays use flax's encoding ``(shape, dtype name, bytes)``.
Everything is host-side NumPy: nothing here touches the GPU.  bfloat16 leaves come
back as float32 (exactly), since NumPy has no bfloat16.

No file written by the reference itself is available to test against: the format
is restated from the source lines above and checked by round trips and by
hand-assembled byte strings only.
"""
from __future__ import annotations

import math
import os
from typing import Any, Dict, List, Mapping, Optional, Sequence, Tuple

import msgpack
import numpy as np

VERSION_V1 = "20220622"
_ARRAY_CHUNKS_MAGIC_KEY = "__msgpack_array_chunk_a87ca2__"
_FLAX_CHUNKED_KEY = "__msgpack_chunked_array__"
_MAX_CHUNK_SIZE = 2 ** 30       # flax.serialization.MAX_CHUNK_SIZE

# serialization.py:148-157
_EXT_NDARRAY, _EXT_COMPLEX, _EXT_NPSCALAR, _EXT_SHAPED_ARRAY = 1, 2, 3, 4
_EXT_SLICE, _EXT_SLICE_ND, _EXT_SLICE_ND_ARRAY, _EXT_INDEX_INFO = 5, 6, 7, 8

SliceNd = Tuple[slice, ...]


class ShapeDtype:
  """Shape and dtype name of a checkpointed array (jax.core.ShapedArray in the reference)."""

  def __init__(self, shape, dtype: str, weak_type: bool = False):
    self.shape = tuple(int(d) for d in shape)
    self.dtype = str(dtype)
    self.weak_type = bool(weak_type)

  def __repr__(self):
    return f"ShapeDtype({self.shape}, {self.dtype})"


class IndexInfo:
  """vmoe/checkpoints/types.py:181-195."""

  def __init__(self, global_shape: ShapeDtype, global_slices: Sequence[SliceNd],
               shards: Sequence[int]):
    self.global_shape = global_shape
    self.global_slices = tuple(global_slices)
    self.shards = tuple(int(s) for s in shards)


# --------------------------------------------------------------------------- arrays
def _np_dtype(name: str):
  """NumPy dtype used in memory for a stored dtype name (bfloat16 is held as uint16)."""
  return np.dtype(np.uint16) if name == "bfloat16" else np.dtype(name)


def _ndarray_from_bytes(data: bytes):
  shape, dtype_name, buffer = msgpack.unpackb(data, raw=True)
  name = dtype_name.decode() if isinstance(dtype_name, bytes) else dtype_name
  arr = np.frombuffer(buffer, dtype=_np_dtype(name)).reshape(tuple(shape))
  return _Bf16Bits(arr) if name == "bfloat16" else arr


def _ndarray_to_bytes(arr) -> bytes:
  if isinstance(arr, _Bf16Bits):
    return msgpack.packb((arr.bits.shape, "bfloat16", arr.bits.tobytes("C")), use_bin_type=True)
  arr = np.asarray(arr)
  return msgpack.packb((arr.shape, arr.dtype.name, arr.tobytes("C")), use_bin_type=True)


class _Bf16Bits:
  """bfloat16 data as its uint16 bit patterns."""

  def __init__(self, bits: np.ndarray):
    self.bits = np.asarray(bits, np.uint16)

  @property
  def shape(self):
    return self.bits.shape

  def to_float32(self) -> np.ndarray:
    return (self.bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def bfloat16_bits(x: np.ndarray) -> _Bf16Bits:
  """float32 -> bfloat16 bit patterns (round to nearest even), for writing bfloat16 leaves."""
  u = np.ascontiguousarray(x, np.float32).view(np.uint32)
  bias = ((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)
  return _Bf16Bits(((u + bias) >> np.uint32(16)).astype(np.uint16))


# --------------------------------------------------------------------------- record types
def _slice_to_bytes(s: slice) -> bytes:
  return msgpack.packb((s.start, s.stop, s.step), use_bin_type=True)


def _slice_from_bytes(data: bytes) -> slice:
  start, stop, step = msgpack.unpackb(data, raw=True)
  return slice(start, stop, step)


def _slice_nd_to_bytes(x: SliceNd) -> bytes:
  return msgpack.packb(tuple(_slice_to_bytes(s) for s in x), use_bin_type=True)


def _slice_nd_from_bytes(data: bytes) -> SliceNd:
  return tuple(_slice_from_bytes(b) for b in msgpack.unpackb(data, raw=True))


def _shape_dtype_to_bytes(x: ShapeDtype) -> bytes:
  return msgpack.packb((x.shape, x.dtype, x.weak_type, {}), use_bin_type=True)


def _shape_dtype_from_bytes(data: bytes) -> ShapeDtype:
  shape, dtype_name, weak_type, _ = msgpack.unpackb(data, raw=True)
  name = dtype_name.decode() if isinstance(dtype_name, bytes) else dtype_name
  return ShapeDtype(shape, name, weak_type)


def _index_info_to_bytes(x: IndexInfo) -> bytes:
  return msgpack.packb((_shape_dtype_to_bytes(x.global_shape),
                        tuple(_slice_nd_to_bytes(s) for s in x.global_slices),
                        tuple(x.shards)), use_bin_type=True)


def _index_info_from_bytes(data: bytes) -> IndexInfo:
  global_shape, global_slices, shards = msgpack.unpackb(data, raw=True)
  return IndexInfo(_shape_dtype_from_bytes(global_shape),
                   tuple(_slice_nd_from_bytes(b) for b in global_slices), tuple(shards))


def _ext_unpack(code: int, data: bytes):
  """serialization.py:306-330."""
  if code == _EXT_NDARRAY:
    return _ndarray_from_bytes(data)
  if code == _EXT_NPSCALAR:
    arr = _ndarray_from_bytes(data)
    return arr.to_float32()[()] if isinstance(arr, _Bf16Bits) else arr[()]
  if code == _EXT_COMPLEX:
    re, im = msgpack.unpackb(data)
    return complex(re, im)
  if code == _EXT_SHAPED_ARRAY:
    return _shape_dtype_from_bytes(data)
  if code == _EXT_SLICE:
    return _slice_from_bytes(data)
  if code == _EXT_SLICE_ND:
    return _slice_nd_from_bytes(data)
  if code == _EXT_INDEX_INFO:
    return _index_info_from_bytes(data)
  if code == _EXT_SLICE_ND_ARRAY:
    shape, slice_nd_bytes = msgpack.unpackb(data, raw=True)
    out = np.empty(len(slice_nd_bytes), dtype=object)
    for i, b in enumerate(slice_nd_bytes):
      out[i] = _slice_nd_from_bytes(b)
    return out.reshape(tuple(shape))
  return msgpack.ExtType(code, data)


def _ext_pack(x):
  """serialization.py:279-303, for the types a checkpoint holds."""
  if isinstance(x, complex):
    return msgpack.ExtType(_EXT_COMPLEX, msgpack.packb((x.real, x.imag)))
  if isinstance(x, ShapeDtype):
    return msgpack.ExtType(_EXT_SHAPED_ARRAY, _shape_dtype_to_bytes(x))
  if isinstance(x, slice):
    return msgpack.ExtType(_EXT_SLICE, _slice_to_bytes(x))
  if isinstance(x, IndexInfo):
    return msgpack.ExtType(_EXT_INDEX_INFO, _index_info_to_bytes(x))
  if isinstance(x, _SliceNdBox):
    return msgpack.ExtType(_EXT_SLICE_ND, _slice_nd_to_bytes(x.value))
  if isinstance(x, (np.ndarray, _Bf16Bits)):
    return msgpack.ExtType(_EXT_NDARRAY, _ndarray_to_bytes(x))
  if isinstance(x, np.generic):
    return msgpack.ExtType(_EXT_NPSCALAR, _ndarray_to_bytes(np.asarray(x)))
  raise TypeError(f"cannot serialise {type(x)}")


class _SliceNdBox:
  """Marks a tuple of slices as one SliceNd record (a bare tuple would be packed as a list)."""

  def __init__(self, value: SliceNd):
    self.value = tuple(value)


class ArrayChunks:
  """vmoe/checkpoints/types.py:133-162: pieces of arrays by leaf id, with their slices."""

  def __init__(self):
    self.chunks: Dict[int, List[np.ndarray]] = {}
    self.global_slices: Dict[int, List[SliceNd]] = {}

  def add(self, index: int, chunk, global_slice: SliceNd):
    self.chunks.setdefault(index, []).append(chunk)
    self.global_slices.setdefault(index, []).append(tuple(global_slice))


def _object_hook(mapping: Mapping[str, Any]):
  """Data-shard dictionaries become ArrayChunks (serialization.py:244-263); arrays that flax
  split because they exceed 2**30 bytes are put together again."""
  if _ARRAY_CHUNKS_MAGIC_KEY in mapping:
    out = ArrayChunks()
    for key, chunks in mapping.items():
      if key == _ARRAY_CHUNKS_MAGIC_KEY:
        continue
      for subchunks, global_slice in chunks:
        shape = tuple(s.stop - s.start for s in global_slice)
        if isinstance(subchunks[0], _Bf16Bits):
          flat = _Bf16Bits(np.concatenate([c.bits for c in subchunks]).reshape(shape))
        else:
          flat = np.concatenate(subchunks).reshape(shape)
        out.add(int(key), flat, global_slice)
    return out
  if _FLAX_CHUNKED_KEY in mapping:
    shape = tuple(mapping["shape"][str(i)] for i in range(len(mapping["shape"])))
    parts = [mapping["chunks"][str(i)] for i in range(len(mapping["chunks"]))]
    if isinstance(parts[0], _Bf16Bits):
      return _Bf16Bits(np.concatenate([c.bits for c in parts]).reshape(shape))
    return np.concatenate(parts).reshape(shape)
  return mapping


def msgpack_restore(encoded: bytes):
  """serialization.py:74-93."""
  return msgpack.unpackb(encoded, ext_hook=_ext_unpack, object_hook=_object_hook, raw=False,
                         strict_map_key=False)


def msgpack_serialize(tree) -> bytes:
  return msgpack.packb(tree, default=_ext_pack, strict_types=True)


# --------------------------------------------------------------------------- trees
def _flatten(tree, path=()) -> List[Tuple[Tuple[str, ...], Any]]:
  """Leaves in sorted-key depth-first order, the order jax.tree_util gives for dicts."""
  if isinstance(tree, Mapping):
    out = []
    for k in sorted(tree):
      out.extend(_flatten(tree[k], path + (k,)))
    return out
  return [(path, tree)]


def _unflatten(items: Sequence[Tuple[Tuple[str, ...], Any]]):
  root: Dict[str, Any] = {}
  for path, value in items:
    node = root
    for k in path[:-1]:
      node = node.setdefault(k, {})
    node[path[-1]] = value
  return root


def add_shard_suffix(filepath: str, shard: int, shard_count: int) -> str:
  """vmoe/checkpoints/base.py:48-49."""
  return f"{filepath}-{shard:05d}-of-{shard_count:05d}"


def restore_checkpoint(prefix: str, bfloat16_as_float32: bool = True) -> Dict[str, Any]:
  """Reads ``prefix.index`` and the data shards it names; returns the nested dict
  (the flax state dict) with NumPy leaves.  vmoe/checkpoints/partitioned.py:89-125."""
  with open(prefix + ".index", "rb") as fp:
    index = msgpack_restore(fp.read())
  version = index.get("version")
  if version != VERSION_V1:
    raise NotImplementedError(
        f"Unsupported checkpoint version {version!r}: only {VERSION_V1!r} files carry a "
        "self-describing index (older ones need the reference's model definition).")
  shard_count = int(index["shard_count"])
  leaves = _flatten(index["index"])
  for path, info in leaves:
    if not isinstance(info, IndexInfo):
      raise ValueError(f"index leaf {'/'.join(path)} is {type(info).__name__}, not an IndexInfo")
  buffers = [np.zeros(info.global_shape.shape, dtype=_np_dtype(info.global_shape.dtype))
             for _, info in leaves]
  filled = [0] * len(leaves)
  shards = sorted({s for _, info in leaves for s in info.shards})
  for shard in shards:
    path = add_shard_suffix(prefix + ".data", shard, shard_count)
    with open(path, "rb") as fp:
      chunks = msgpack_restore(fp.read())
    if not isinstance(chunks, ArrayChunks):
      raise ValueError(f"{path} does not hold array chunks")
    for i, pieces in chunks.chunks.items():
      if i >= len(buffers):
        raise ValueError(f"{path} holds leaf id {i}, the index has {len(buffers)} leaves")
      for piece, sl in zip(pieces, chunks.global_slices[i]):
        data = piece.bits if isinstance(piece, _Bf16Bits) else piece
        buffers[i][tuple(sl)] = data
        filled[i] += int(np.prod(data.shape, dtype=np.int64))
  out = []
  for (path, info), buf, n in zip(leaves, buffers, filled):
    if n != int(np.prod(info.global_shape.shape, dtype=np.int64)):
      raise ValueError(f"leaf {'/'.join(path)}: {n} of {buf.size} elements found in the shards")
    if info.global_shape.dtype == "bfloat16":
      buf = _Bf16Bits(buf).to_float32() if bfloat16_as_float32 else buf
    out.append((path, buf))
  return _unflatten(out)


def save_checkpoint(prefix: str, tree: Mapping[str, Any], num_shards: int = 1,
                    max_chunk_bytes: Optional[int] = None) -> List[str]:
  """Writes ``tree`` (nested dict, NumPy leaves or bfloat16_bits(...)) in the format above.
  Leaves larger than ``max_chunk_bytes`` are cut along their first axis; every piece goes
  to the shard that holds the fewest bytes so far (partitioned.py:131-216).  Returns the
  file names."""
  leaves = _flatten(tree)
  bytes_per_shard = [0] * num_shards
  per_shard: List[Dict[str, list]] = [{_ARRAY_CHUNKS_MAGIC_KEY: True} for _ in range(num_shards)]
  index_leaves = []
  for i, (path, leaf) in enumerate(leaves):
    is_bf16 = isinstance(leaf, _Bf16Bits)
    arr = leaf.bits if is_bf16 else np.asarray(leaf)
    dtype_name = "bfloat16" if is_bf16 else arr.dtype.name
    rows = arr.shape[0] if arr.ndim else 1
    step = rows
    if max_chunk_bytes and arr.ndim and arr.nbytes > max_chunk_bytes:
      row_bytes = max(1, arr.nbytes // max(rows, 1))
      step = max(1, max_chunk_bytes // row_bytes)
    slices, shards = [], []
    for r0 in range(0, max(rows, 1), max(step, 1)):
      if arr.ndim:
        sl = (slice(r0, min(r0 + step, rows), None),) + tuple(
            slice(0, d, None) for d in arr.shape[1:])
        piece = arr[r0:r0 + step]
      else:
        sl, piece = (), arr
      shard = int(np.argmin(bytes_per_shard))
      bytes_per_shard[shard] += piece.nbytes
      flat = np.ascontiguousarray(piece).reshape(-1)
      sub = max(1, _MAX_CHUNK_SIZE // max(flat.dtype.itemsize, 1))
      subchunks = [(_Bf16Bits(flat[j:j + sub]) if is_bf16 else flat[j:j + sub])
                   for j in range(0, max(flat.size, 1), sub)]
      per_shard[shard].setdefault(str(i), []).append([subchunks, _SliceNdBox(sl)])
      slices.append(sl)
      shards.append(shard)
    index_leaves.append((path, IndexInfo(ShapeDtype(arr.shape, dtype_name), slices, shards)))
  os.makedirs(os.path.dirname(os.path.abspath(prefix)), exist_ok=True)
  files = []
  for shard in range(num_shards):
    name = add_shard_suffix(prefix + ".data", shard, num_shards)
    with open(name, "wb") as fp:
      fp.write(msgpack_serialize(per_shard[shard]))
    files.append(name)
  index = {"shard_count": num_shards, "index": _unflatten(index_leaves), "version": VERSION_V1}
  with open(prefix + ".index", "wb") as fp:
    fp.write(msgpack_serialize(index))
  return files + [prefix + ".index"]


# --------------------------------------------------------------------------- transformations
def expand_tile(array: np.ndarray, axis, reps) -> np.ndarray:
  """vmoe/initialization/rules.py:242-258: new axes at ``axis``, tiled ``reps`` times
  (a dense MLP kernel (D, M) becomes the experts' (E, D, M) with axis=0, reps=E)."""
  axes = (axis,) if isinstance(axis, int) else tuple(axis)
  rep = (reps,) if isinstance(reps, int) else tuple(reps)
  if len(axes) != len(rep):
    raise ValueError(f"axis {axes} and reps {rep} differ in length")
  out = np.expand_dims(np.asarray(array), axis=axes)
  tiles = [1] * out.ndim
  for a, r in zip(axes, rep):
    tiles[a] = r
  return np.tile(out, tiles)


def zoom(source: np.ndarray, target_shape: Sequence[int]) -> np.ndarray:
  """vmoe/initialization/rules.py:290-325: linear interpolation to ``target_shape``."""
  import scipy.ndimage
  factors = tuple(n / o for n, o in zip(target_shape, source.shape))
  return scipy.ndimage.zoom(source, factors, order=1)


def _tok_and_grid_shape(shape):
  _, num_tokens, hidden_size = shape
  sqrt_tokens = int(math.sqrt(num_tokens))
  if num_tokens not in (sqrt_tokens ** 2, sqrt_tokens ** 2 + 1):
    raise ValueError(f"{num_tokens=} is neither a perfect square nor a perfect square + 1. "
                     "This means that the grid used is not squared. This isn't supported.")
  return sqrt_tokens ** 2 != num_tokens, (1, sqrt_tokens, sqrt_tokens, hidden_size)


def vit_zoom(source: np.ndarray, target_shape: Sequence[int],
             target: Optional[np.ndarray] = None) -> np.ndarray:
  """vmoe/initialization/rules.py:328-381: resizes a (1, n, D) position embedding to the
  target's token grid; a class-token row is kept from the source, else taken from
  ``target``, else drawn N(0, 0.02) from a fixed seed."""
  source = np.asarray(source)
  target_shape = tuple(target_shape)
  if source.ndim != 3 or source.shape[0] != 1:
    raise ValueError(f"{source.shape=} is not (1, ?, ?)")
  if len(target_shape) != 3 or target_shape[0] != 1:
    raise ValueError(f"{target_shape=} is not (1, ?, ?)")
  if source.shape[2] != target_shape[2]:
    raise ValueError(f"{source.shape[2]=} != {target_shape[2]}")
  source_has_tok, source_grid_shape = _tok_and_grid_shape(source.shape)
  grid = source[:, 1:, :] if source_has_tok else source
  target_has_tok, target_grid_shape = _tok_and_grid_shape(target_shape)
  out = zoom(grid.reshape(source_grid_shape), target_grid_shape)
  out = out.reshape(1, -1, out.shape[-1])
  if not target_has_tok:
    return out
  if source_has_tok:
    tok = source[:, :1, :]
  elif target is not None:
    tok = np.asarray(target)[:, :1, :]
  else:
    tok = (0.02 * np.random.default_rng(0).standard_normal((1, 1, out.shape[-1]))).astype(
        source.dtype)
  return np.concatenate([tok, out], axis=1)


def dense_to_moe_params(params: Mapping[str, Any], moe_layers: Sequence[int], num_experts: int,
                        router_std: float = 0.02, seed: int = 0) -> Dict[str, Any]:
  """Turns the parameter tree of a dense ViT into the tree of the sparse model that has
  experts in ``moe_layers``: each chosen block's ``Mlp`` becomes ``Moe/Mlp`` with every
  leaf tiled over a leading expert axis (the expand_tile rule, as in
  vmoe/configs/vmoe_paper/*upcycling*), and ``Moe/Router/dense/kernel`` (D, E) is drawn
  N(0, router_std)."""
  rng = np.random.default_rng(seed)
  out = {k: v for k, v in params.items()}
  enc = dict(out["Encoder"])
  for layer in moe_layers:
    name = f"encoderblock_{layer}"
    blk = dict(enc[name])
    mlp = blk.pop("Mlp")
    D = np.asarray(mlp["Dense_0"]["kernel"]).shape[0]
    blk["Moe"] = {
        "Mlp": {dn: {ln: expand_tile(np.asarray(leaf), 0, num_experts) for ln, leaf in d.items()}
                for dn, d in mlp.items()},
        "Router": {"dense": {"kernel": (router_std * rng.standard_normal((D, num_experts))).astype(
            np.float32)}}}
    enc[name] = blk
  out["Encoder"] = enc
  return out


def to_device(tree, device, dtype=None):
  """NumPy leaves -> torch tensors on ``device`` (optionally cast), same nesting."""
  import torch
  if isinstance(tree, Mapping):
    return {k: to_device(v, device, dtype) for k, v in tree.items()}
  t = torch.from_numpy(np.ascontiguousarray(tree))
  if dtype is not None and t.is_floating_point():
    t = t.to(dtype)
  return t.to(device)
