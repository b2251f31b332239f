"""Shared helpers for the parity tests."""
import numpy as np
import torch

from oracle import moe_oracle as O


def dev():
  return torch.device("cuda:0")


def to_dev(a: np.ndarray, dtype: str = O.F32) -> torch.Tensor:
  """NumPy float32 (already holding dtype-representable values) -> device tensor of dtype."""
  t = torch.from_numpy(np.ascontiguousarray(a))
  if t.dtype == torch.float32 and dtype == O.BF16:
    t = t.to(torch.bfloat16)
  return t.to(dev())


def to_np(t: torch.Tensor) -> np.ndarray:
  t = t.detach().cpu()
  if t.dtype == torch.bfloat16:
    t = t.to(torch.float32)
  return t.numpy()


def tdtype(dtype: str):
  return torch.bfloat16 if dtype == O.BF16 else torch.float32


def assert_close(actual, desired, rtol, what=""):
  """|a - b| <= rtol * (rms(b) + |b|): relative tolerance with an absolute floor
  tied to the scale of the data (outputs are sums of signed terms)."""
  actual = np.asarray(actual, np.float64)
  desired = np.asarray(desired, np.float64)
  rms = float(np.sqrt(np.mean(desired ** 2))) if desired.size else 0.0
  err = np.abs(actual - desired)
  tol = rtol * (rms + np.abs(desired))
  bad = err > tol
  assert not bad.any(), (
      f"{what}: {bad.sum()} / {bad.size} outside rtol={rtol}; max abs err {err.max():.3e}, "
      f"rms {rms:.3e}, worst at {np.unravel_index(np.argmax(err - tol), err.shape)}")
