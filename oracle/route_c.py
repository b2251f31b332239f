"""ctypes loader for the C part of the oracle (TEST INFRASTRUCTURE ONLY)."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "liboracle_route.so")
_lib = None


def build() -> str:
  """Compiles oracle/route_greedy.c with gcc (always recompiles)."""
  subprocess.run(["make", "-B", "-C", _HERE], check=True, stdout=subprocess.DEVNULL)
  return _SO


def lib() -> ctypes.CDLL:
  global _lib
  if _lib is None:
    if not os.path.exists(_SO):
      build()
    _lib = ctypes.CDLL(_SO)
  return _lib


def _p(a, t):
  return a.ctypes.data_as(ctypes.POINTER(t))


def route_batch(gates: np.ndarray, num_selected_experts: int, batch_priority: bool):
  """gates (G,S,E) float32 -> indices (G,S,K,2) int32, weights (G,S,K) float32."""
  gates = np.ascontiguousarray(gates, np.float32)
  G, S, E = gates.shape
  K = num_selected_experts
  indices = np.empty((G, S, K, 2), np.int32)
  weights = np.empty((G, S, K), np.float32)
  lib().oracle_route_batch(_p(gates, ctypes.c_float), G, S, E, K, int(batch_priority),
                           _p(indices, ctypes.c_int32), _p(weights, ctypes.c_float))
  return indices, weights


def route_greedy(expert_idx: np.ndarray, top1, num_experts: int, batch_priority: bool):
  """expert_idx (S,K) int32, top1 (S,) float32 -> pos (S,K), count (E,)."""
  expert_idx = np.ascontiguousarray(expert_idx, np.int32)
  S, K = expert_idx.shape
  pos = np.empty((S, K), np.int32)
  count = np.empty((num_experts,), np.int32)
  t1 = None if top1 is None else np.ascontiguousarray(top1, np.float32)
  lib().oracle_route_greedy(_p(expert_idx, ctypes.c_int32),
                            None if t1 is None else _p(t1, ctypes.c_float),
                            S, K, num_experts, int(batch_priority and t1 is not None),
                            _p(pos, ctypes.c_int32), _p(count, ctypes.c_int32))
  return pos, count
