"""Mapping of checkpoint trees onto a model's parameter tree with regex rules.

Host-side counterpart of vmoe/initialization/rules.py (rule parsing and the
transformations), vmoe/initialization/mapping.py (``map_state_dict``) and the
V-MoE / ViT entry points of vmoe/initialization/initialization.py.  Trees are nested
dicts whose leaves are NumPy arrays or torch tensors; every transformation runs in
NumPy on the host (parameters are imported once, before anything is timed) and a
leaf comes back in the container type of the target leaf it replaces.
"""
import dataclasses
import logging
import re
from typing import Any, Dict, Iterable, List, Mapping, Optional, Sequence, Tuple, Union

import numpy as np

from vmoe_amd import checkpoints

UnparsedRules = Sequence[Union["Rule", Tuple[Any, ...]]]

__all__ = ["Rules", "Rule", "DropRule", "RegexRule", "ExpandTileRule", "ReshapeRule",
           "SqueezeRule", "StackRule", "VitZoomRule", "ZoomRule", "ShapeDtype",
           "map_state_dict", "initialize_from_vmoe", "initialize_from_vit"]


@dataclasses.dataclass(frozen=True)
class ShapeDtype:
  """Stand-in for a target leaf whose values do not exist yet (jax.ShapeDtypeStruct in
  the reference's tests): only shape and dtype are known."""
  shape: Tuple[int, ...]
  dtype: Any = np.float32

  @property
  def ndim(self) -> int:
    return len(self.shape)


class EmptyNode:
  """Marks an empty dict in a flattened tree (flax.traverse_util's keep_empty_nodes)."""

  def __repr__(self):
    return "EmptyNode()"


_EMPTY = EmptyNode()


# ----------------------------------------------------------------------------- rules
@dataclasses.dataclass
class Rule:
  pattern: Any

  def __post_init__(self):
    if isinstance(self.pattern, str):
      self.pattern = re.compile(self.pattern)

  def rename(self, key: str) -> str:
    return key


@dataclasses.dataclass
class DropRule(Rule):
  """rules.py:136-138: matched source arrays are not used."""


@dataclasses.dataclass
class RegexRule(Rule):
  """rules.py:141-158: renames the matched arrays, values copied."""
  replacement: str = ""

  def rename(self, key: str) -> str:
    return self.pattern.sub(self.replacement, key)

  def transform(self, sources: List[np.ndarray], target) -> np.ndarray:
    return sources[0]


@dataclasses.dataclass
class ExpandTileRule(RegexRule):
  """rules.py:161-171, 242-258."""
  axis: Union[int, Tuple[int, ...]] = 0
  reps: Union[int, Tuple[int, ...]] = 1

  def transform(self, sources, target):
    return checkpoints.expand_tile(sources[0], self.axis, self.reps)


@dataclasses.dataclass
class ReshapeRule(RegexRule):
  """rules.py:174-188: to ``shape``, or to the target's shape when none is given."""
  shape: Optional[Tuple[int, ...]] = None

  def transform(self, sources, target):
    return np.reshape(sources[0], self.shape or tuple(target.shape))


@dataclasses.dataclass
class SqueezeRule(RegexRule):
  """rules.py:191-198."""
  axis: int = 0

  def transform(self, sources, target):
    return np.squeeze(sources[0], axis=self.axis)


@dataclasses.dataclass
class StackRule(RegexRule):
  """rules.py:201-209: all matched sources, in natural order of their names."""
  axis: int = 0

  def transform(self, sources, target):
    return np.stack(sources, axis=self.axis)


@dataclasses.dataclass
class ZoomRule(RegexRule):
  """rules.py:222-228, 290-325: linear interpolation to the target's shape."""

  def transform(self, sources, target):
    return checkpoints.zoom(sources[0], tuple(target.shape))


@dataclasses.dataclass
class VitZoomRule(RegexRule):
  """rules.py:212-219, 328-381: position embeddings, token row handled apart."""

  def transform(self, sources, target):
    values = None if isinstance(target, ShapeDtype) else _to_numpy(target)
    return checkpoints.vit_zoom(sources[0], tuple(target.shape), values)


@dataclasses.dataclass
class Rules:
  """rules.py:40-120."""
  rules: List[Rule] = dataclasses.field(default_factory=list)

  def find(self, key: str) -> Optional[Rule]:
    for rule in self.rules:
      if rule.pattern.search(key):
        return rule
    return None

  @classmethod
  def parse(cls, rules: UnparsedRules) -> "Rules":
    """Tuples ``(regex, replacement[, transform, *args])`` -> Rules; a replacement of
    None or '' drops the matched arrays."""
    parsed = []
    for rule in rules:
      if isinstance(rule, Rule):
        parsed.append(rule)
        continue
      pattern, replacement, *transform = rule
      pattern = re.compile(pattern)
      if not transform:
        parsed.append(RegexRule(pattern, replacement) if replacement else DropRule(pattern))
      elif transform[0] == "reshape":
        assert len(transform) in (1, 2)
        parsed.append(ReshapeRule(pattern, replacement,
                                  shape=transform[1] if len(transform) == 2 else None))
      elif transform[0] == "squeeze":
        assert len(transform) == 2 and isinstance(transform[1], int)
        parsed.append(SqueezeRule(pattern, replacement, axis=transform[1]))
      elif transform[0] == "stack":
        assert len(transform) == 2 and isinstance(transform[1], int)
        parsed.append(StackRule(pattern, replacement, axis=transform[1]))
      elif transform[0] == "expand_tile":
        assert len(transform) == 3
        parsed.append(ExpandTileRule(pattern, replacement, axis=transform[1], reps=transform[2]))
      elif transform[0] == "vit_zoom":
        parsed.append(VitZoomRule(pattern, replacement))
      elif transform[0] == "zoom":
        parsed.append(ZoomRule(pattern, replacement))
      else:
        raise ValueError(f"Rule {rule!r} cannot be parsed.")
    return cls(rules=parsed)


_IDENTITY_RULE = RegexRule(pattern=re.compile("^(.*)$"), replacement=r"\1")
_SIGNED_FLOAT_RE = re.compile(r"([-+]?(?:\d+(?:\.\d*)?|\.\d+)(?:[eE][-+]?\d+)?)")


# --------------------------------------------------------------------------- mapping
def _natural_sort(names: Iterable[str]) -> List[str]:
  """mapping.py:218-227: numerical substrings compare as numbers ('a3' < 'a11')."""
  def split_keys(s):
    # Numbers and text alternate; tagging them keeps mixed positions comparable.
    return [(0, float(c), "") if _SIGNED_FLOAT_RE.fullmatch(c) else (1, 0.0, c)
            for c in _SIGNED_FLOAT_RE.split(s)]
  return sorted(names, key=split_keys)


def _raise_or_warn(cls, exception_msg, raise_exception, warn_msg=None):
  if raise_exception:
    raise cls(exception_msg)
  logging.warning(warn_msg or exception_msg)


def _flatten(tree, prefix=()) -> Dict[str, Any]:
  if not isinstance(tree, Mapping):
    return {"/".join(prefix): tree}
  if not tree and prefix:
    return {"/".join(prefix): _EMPTY}
  out = {}
  for k, v in tree.items():
    out.update(_flatten(v, prefix + (str(k),)))
  return out


def _unflatten(flat: Mapping[str, Any]):
  out: Dict[str, Any] = {}
  for key, value in flat.items():
    node = out
    parts = key.split("/")
    for part in parts[:-1]:
      node = node.setdefault(part, {})
    node[parts[-1]] = {} if isinstance(value, EmptyNode) else value
  return out


def _to_numpy(x) -> np.ndarray:
  if isinstance(x, np.ndarray):
    return x
  if hasattr(x, "detach"):   # torch tensor
    t = x.detach().cpu()
    if str(t.dtype) == "torch.bfloat16":
      t = t.float()
    return t.numpy()
  return np.asarray(x)


def _like(value: np.ndarray, target):
  """``value`` in the container, dtype and device of the target leaf."""
  if hasattr(target, "detach"):   # torch tensor
    import torch
    return torch.as_tensor(np.ascontiguousarray(value)).to(device=target.device, dtype=target.dtype)
  return value


def _dtype_name(x) -> str:
  d = x.dtype
  return str(d).replace("torch.", "") if not isinstance(d, type) else np.dtype(d).name


def map_state_dict(source, target, rules: Union[Rules, UnparsedRules],
                   raise_if_dtype_mismatched: bool = False,
                   raise_if_shape_mismatched: bool = True,
                   raise_if_source_unmatched: bool = True,
                   raise_if_target_unmatched: bool = True):
  """mapping.py:79-99: every source array goes through the first rule whose regex is
  found in its '/'-joined name, is renamed, transformed, checked against the target leaf
  of that name (dtype: converted unless asked to raise; shape: broadcast only when asked
  not to raise) and replaces it.  Target leaves no source maps to are kept."""
  if not isinstance(rules, Rules):
    rules = Rules.parse(rules)
  source_flat, target_flat = _flatten(source), _flatten(target)
  used = {k: False for k in target_flat}
  pending: Dict[str, Tuple[RegexRule, List[np.ndarray]]] = {}
  for src_key in _natural_sort(source_flat.keys()):
    rule = rules.find(src_key)
    if rule is None:
      msg = f"Source key {src_key!r} does not match any rule."
      _raise_or_warn(KeyError, msg, raise_if_source_unmatched, msg + " Assuming the identity rule.")
      rule = _IDENTITY_RULE
    if isinstance(rule, DropRule):
      continue
    dst_key = rule.rename(src_key)
    if dst_key not in target_flat:
      raise KeyError(f"Source key {src_key!r} was matched with target key {dst_key!r}, "
                     "but it does not exist.")
    if used[dst_key] and not isinstance(rule, StackRule):
      raise ValueError(f"Target key {dst_key!r} was matched more than once.")
    used[dst_key] = True
    src_value, dst_value = source_flat[src_key], target_flat[dst_key]
    if isinstance(src_value, EmptyNode) != isinstance(dst_value, EmptyNode):
      raise ValueError("One of the values represents an empty node, but not the other. "
                       f"{src_key=} has type={type(src_value)!r} and {dst_key=} has "
                       f"type={type(dst_value)!r}.")
    if isinstance(src_value, EmptyNode):
      continue
    if not isinstance(rule, RegexRule):
      raise TypeError(f"Unexpected type for rule: {rule!r}")
    if isinstance(rule, StackRule) and dst_key in pending:
      pending[dst_key][1].append(_to_numpy(src_value))
    else:
      pending[dst_key] = (rule, [_to_numpy(src_value)])
  for dst_key, was_used in used.items():
    leaf = target_flat[dst_key]
    if not was_used and not isinstance(leaf, EmptyNode):
      msg = f"Target key {dst_key!r} is unmatched."
      _raise_or_warn(ValueError, msg, raise_if_target_unmatched,
                     msg + f" The original value with shape {tuple(leaf.shape)} and type "
                     f"{_dtype_name(leaf)} will be preserved.")
  output = dict(target_flat)
  for key, (rule, sources) in pending.items():
    leaf = target_flat[key]
    value = np.asarray(rule.transform(sources, leaf))
    expected_dtype = _dtype_name(leaf)
    if value.dtype.name != expected_dtype:
      msg = (f"Target key {key!r} has mismatched dtypes. Actual = {value.dtype.name}, "
             f"expected = {expected_dtype}.")
      _raise_or_warn(ValueError, msg, raise_if_dtype_mismatched,
                     msg + " Converting to the expected dtype.")
      if expected_dtype != "bfloat16":   # NumPy has no bfloat16; _like() converts torch leaves
        value = value.astype(expected_dtype)
    expected_shape = tuple(leaf.shape)
    if tuple(value.shape) != expected_shape:
      msg = (f"Target key {key!r} has mismatched shapes. Actual = {tuple(value.shape)!r}, "
             f"expected = {expected_shape!r}.")
      _raise_or_warn(ValueError, msg, raise_if_shape_mismatched,
                     msg + " Broadcasting to the expected shape.")
      value = np.broadcast_to(value, expected_shape)
    output[key] = _like(value, leaf)
  return _unflatten(output)


# ----------------------------------------------------------------------- entry points
def initialize_from_vmoe(*, target, prefix: str, rules: Union[Rules, UnparsedRules], mesh=None,
                         axis_resources_regexes=None, thread_pool=None, **map_state_dict_kwargs):
  """initialization.py:205-267: reads the sharded checkpoint ``prefix.index`` /
  ``prefix.data-*`` and maps it onto ``target``.  ``mesh``, ``axis_resources_regexes``
  and ``thread_pool`` describe how the reference spreads the arrays over devices while
  reading; one GPU holds everything here and they are accepted and ignored."""
  del mesh, axis_resources_regexes, thread_pool
  ckpt = checkpoints.restore_checkpoint(prefix)
  return map_state_dict(ckpt, target, rules, **map_state_dict_kwargs)


def initialize_from_vit(*, target, filepath: str, rules: Union[Rules, UnparsedRules], mesh=None,
                        axis_resources_regexes=None, **map_state_dict_kwargs):
  """initialization.py:149-202: a VisionTransformer ``.npz`` checkpoint (flat
  '/'-joined names, the format of vit_jax.checkpoint.load) mapped onto ``target``.
  Two-byte void arrays are bfloat16 bit patterns (initialization.py:179-185) and are
  widened to float32, which holds every bfloat16 value exactly."""
  del mesh, axis_resources_regexes
  flat = {}
  with np.load(filepath, allow_pickle=False) as data:
    for name in data.files:
      value = data[name]
      if value.dtype.type is np.void:
        if value.itemsize != 2:
          raise ValueError(f"{name!r}: unknown dtype {value.dtype}")
        value = (value.view(np.uint16).astype(np.uint32) << 16).view(np.float32)
      flat[name] = value
  return map_state_dict(_unflatten(flat), target, rules, **map_state_dict_kwargs)
