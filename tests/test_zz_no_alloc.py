"""vmoe_compact_rows_static: the row compaction for callers that cannot allocate (its
(G, E) scratch is a static device array inside the library) against vmoe_compact_rows,
through the C ABI, on calls in a row that share the array."""
import ctypes

import numpy as np
import pytest
import torch

from tests.util import dev, to_dev, to_np

pytestmark = pytest.mark.gpu


def _routed(seed, G, S, E, K, C):
  """Fill counts and slot rows of a seeded routing problem (the slot-assignment kernel)."""
  from vmoe_amd import kernels as Kn
  rng = np.random.default_rng(seed)
  gates = rng.random((G, S, E)).astype(np.float32)
  val, idx = Kn.topk(to_dev(gates), K)
  _, token_slot, _, fill = Kn.route_assign(val, idx, E, C, True)
  return fill, token_slot


def _compact(entry, fill, token_slot, C, with_prefix):
  from vmoe_amd import _hip as H
  G, E = fill.shape
  _, S, K = token_slot.shape
  token_row = torch.full((G, S, K), -7, dtype=torch.int32, device=dev())
  rows = torch.full((E,), -7, dtype=torch.int32, device=dev())
  row_token = torch.full((E, G * C), -1, dtype=torch.int32, device=dev())
  prefix = torch.zeros((G, E), dtype=torch.int32, device=dev()) if with_prefix else None
  p = H.CompactRowsParams(H.ptr(fill), H.ptr(token_slot), H.ptr(token_row), H.ptr(rows),
                          H.ptr(prefix), H.ptr(row_token), G, S, E, K, C)
  code = getattr(H.lib(), entry)(ctypes.byref(p), H.stream())
  assert code == 0, (entry, code)
  return token_row, rows, row_token


# (G, S, E, K, C): the first two take the two-launch form that uses the scratch (fewer than
# 256 assignments per group), the second smaller than the first; the third takes the
# single-launch form; the last has more than 256 experts.
CASES = [(40, 64, 8, 2, 20), (12, 32, 4, 2, 12), (4, 256, 8, 2, 72), (3, 40, 300, 1, 2)]


def test_compact_rows_static_matches_compact_rows():
  from vmoe_amd import _hip as H
  assert H.lib().vmoe_compact_rows_static is not None
  problems = [(_routed(i, *c), c) for i, c in enumerate(CASES)]
  want = [_compact("vmoe_compact_rows", f, t, c[4], True) for (f, t), c in problems]
  # back to back on one stream, sharing the static array; then once more in reverse order
  got = [_compact("vmoe_compact_rows_static", f, t, c[4], False) for (f, t), c in problems]
  again = [_compact("vmoe_compact_rows_static", f, t, c[4], False) for (f, t), c in reversed(problems)]
  torch.cuda.synchronize()
  for w, g, a, c in zip(want, got, reversed(again), CASES):
    for name, x, y, z in zip(("token_row", "rows_per_expert", "row_token"), w, g, a):
      np.testing.assert_array_equal(to_np(y), to_np(x), err_msg=f"{name} {c}")
      np.testing.assert_array_equal(to_np(z), to_np(x), err_msg=f"{name} {c} (second round)")
    assert int(to_np(w[1]).sum()) == int((to_np(w[0]) >= 0).sum()) > 0


def test_compact_rows_static_allocates_nothing_and_can_be_captured():
  """After the one call per device that looks up the array's address, a call changes neither
  the device's free memory nor torch's allocator statistics (outputs are allocated before the
  measurement), and a call captured into a HIP graph (kernels only) gives the eager result on
  every replay, with eager work and synchronisations between the replays."""
  from vmoe_amd import _hip as H
  G, S, E, K, C = CASES[0]
  fill, token_slot = _routed(11, G, S, E, K, C)
  want = _compact("vmoe_compact_rows", fill, token_slot, C, True)
  _compact("vmoe_compact_rows_static", fill, token_slot, C, False)      # the address look-up, outside any capture
  token_row = torch.full((G, S, K), -7, dtype=torch.int32, device=dev())
  rows = torch.full((E,), -7, dtype=torch.int32, device=dev())
  row_token = torch.full((E, G * C), -1, dtype=torch.int32, device=dev())
  p = H.CompactRowsParams(H.ptr(fill), H.ptr(token_slot), H.ptr(token_row), H.ptr(rows),
                          None, H.ptr(row_token), G, S, E, K, C)
  torch.cuda.synchronize()
  free_before, _ = torch.cuda.mem_get_info()
  reserved_before = torch.cuda.memory_reserved()
  for _ in range(3):
    assert H.lib().vmoe_compact_rows_static(ctypes.byref(p), H.stream()) == 0
  torch.cuda.synchronize()
  free_after, _ = torch.cuda.mem_get_info()
  assert free_after == free_before and torch.cuda.memory_reserved() == reserved_before
  for name, x, y in zip(("token_row", "rows_per_expert", "row_token"), want, (token_row, rows, row_token)):
    np.testing.assert_array_equal(to_np(y), to_np(x), err_msg=name)
  # captured: the graph holds the call's kernels and nothing else
  graph = torch.cuda.CUDAGraph()
  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):
    with torch.cuda.graph(graph, stream=side):
      assert H.lib().vmoe_compact_rows_static(ctypes.byref(p), H.stream()) == 0
  torch.cuda.current_stream().wait_stream(side)
  for replay in range(3):
    token_row.fill_(-7)
    rows.fill_(-7)
    row_token.fill_(-1)
    _compact("vmoe_compact_rows_static", *_routed(20 + replay, *CASES[1]), CASES[1][4], False)   # eager work on the shared array in between
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    for name, x, y in zip(("token_row", "rows_per_expert", "row_token"), want, (token_row, rows, row_token)):
      np.testing.assert_array_equal(to_np(y), to_np(x), err_msg=f"{name}, replay {replay}")


def test_compact_rows_static_rejects_oversize_and_null():
  from vmoe_amd import _hip as H
  lib = H.lib()
  G, E = 65537, 1                      # G * E beyond the static array
  t = torch.zeros((8,), dtype=torch.int32, device=dev())
  p = H.CompactRowsParams(H.ptr(t), H.ptr(t), H.ptr(t), H.ptr(t), None, None, G, 1, E, 1, 1)
  assert lib.vmoe_compact_rows_static(ctypes.byref(p), H.stream()) == -7      # VMOE_E_WORKSPACE
  p = H.CompactRowsParams(None, H.ptr(t), H.ptr(t), H.ptr(t), None, None, 2, 2, 2, 1, 1)
  assert lib.vmoe_compact_rows_static(ctypes.byref(p), H.stream()) == -1      # VMOE_E_NULL
  assert lib.vmoe_compact_rows_static(None, H.stream()) == -1
