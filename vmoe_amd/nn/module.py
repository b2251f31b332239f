"""A minimal stand-in for flax.linen.Module: hyper-parameters are constructor
keyword arguments with class-level defaults, parameters live in a nested dict
``{'params': {...}}`` with the reference's names, ``init(seed, *inputs)``
creates them and ``apply(variables, *inputs)`` runs the module."""
from __future__ import annotations

from typing import Any, Dict

import weakref

import torch


class Module:
  _fields: Dict[str, Any] = {}

  def __init__(self, **kwargs):
    fields = {}
    for cls in reversed(type(self).__mro__):
      fields.update(getattr(cls, "_fields", {}))
    self.name = kwargs.pop("name", None)
    unknown = set(kwargs) - set(fields)
    if unknown:
      raise TypeError(f"{type(self).__name__} got unexpected arguments {sorted(unknown)}")
    missing = [k for k, v in fields.items() if v is _REQUIRED and k not in kwargs]
    if missing:
      raise TypeError(f"{type(self).__name__} missing required arguments {missing}")
    for k, v in fields.items():
      setattr(self, k, kwargs.get(k, v))

  def init(self, rng, *inputs):
    raise NotImplementedError

  def apply(self, variables, *inputs, **kwargs):
    raise NotImplementedError

  def __call__(self, variables, *inputs, **kwargs):
    return self.apply(variables, *inputs, **kwargs)


class _Required:
  def __repr__(self):
    return "<required>"


_REQUIRED = _Required()


def generator(rng, device="cpu") -> torch.Generator:
  if isinstance(rng, torch.Generator):
    return rng
  g = torch.Generator(device=device)
  g.manual_seed(int(rng))
  return g


def lecun_normal(gen: torch.Generator, shape, fan_in: int, dtype=torch.float32, device=None):
  """jax.nn.initializers.lecun_normal: truncated normal with variance 1/fan_in."""
  t = torch.empty(shape, dtype=torch.float32)
  torch.nn.init.trunc_normal_(t, mean=0.0, std=1.0, a=-2.0, b=2.0, generator=gen)
  t = t * (1.0 / 0.87962566103423978) / (fan_in ** 0.5)
  return t.to(dtype).to(device) if device is not None else t.to(dtype)


def require_no_grad(what: str, *tensors) -> None:
  """The gating, routing and expert kernels are forward-only (inference).  Called with
  the parameters and inputs of such a module: raises instead of silently cutting the
  graph when autograd is recording and one of them requires a gradient."""
  if torch.is_grad_enabled() and any(
      isinstance(t, torch.Tensor) and t.requires_grad for t in tensors):
    raise NotImplementedError(
        f"{what} has no backward pass (inference path): call it under torch.no_grad() or "
        "detach its parameters and inputs.")


def make_rngs(rngs, device):
  """``rngs={'gating': seed or torch.Generator}`` (flax's ``rngs=`` argument of apply)
  with every seed turned into a generator on ``device``, so that modules that draw
  one after the other get different numbers.  None stays None."""
  if rngs is None:
    return None
  out = {}
  for name, rng in rngs.items():
    out[name] = rng if isinstance(rng, torch.Generator) else generator(rng, device=device)
  return out


class ParamCache:
  """Derived copies of parameter tensors (casts, packed layouts).

  An entry is valid while the very tensors it was built from are alive and
  unmodified: they are identified by object (views by their base tensor, offset,
  shape and strides), held weakly, and their version counters are compared.  An
  address alone does not identify a tensor: the allocator hands a freed block
  to the next tensor of that size."""

  def __init__(self, limit: int = 16):
    self._entries = {}
    self._limit = limit

  @staticmethod
  def _ident(t: torch.Tensor):
    base = t._base if t._base is not None else t
    return base, (id(base), t.storage_offset(), tuple(t.shape), tuple(t.stride()), t.dtype)

  def get(self, tensors, tag, build):
    tensors = tuple(tensors)
    idents = [self._ident(t) for t in tensors]
    key = (tuple(i[1] for i in idents), tag)
    versions = tuple(t._version for t in tensors)
    hit = self._entries.get(key)
    if hit is not None:
      refs, vers, value = hit
      if vers == versions and all(r() is i[0] for r, i in zip(refs, idents)):
        return value
    value = build()
    if len(self._entries) >= self._limit:
      self._entries.clear()
    self._entries[key] = (tuple(weakref.ref(i[0]) for i in idents), versions, value)
    return value
