"""Parity of each HIP kernel (called through the C ABI) against the CPU oracle."""
import os
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from oracle import route_c
from tests.util import assert_close, dev, tdtype, to_dev, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
  from vmoe_amd import kernels
  return kernels


# ------------------------------------------------------------------ cast
def test_cast_matches_round_to_nearest_even(K):
  rng = np.random.default_rng(0)
  x = (rng.standard_normal(100003) * 10.0 ** rng.integers(-10, 10, 100003)).astype(np.float32)
  x[:4] = [0.0, -0.0, 1.00390625, 1.01171875]   # exact ties
  got = to_np(K.cast(to_dev(x), torch.bfloat16))
  np.testing.assert_array_equal(got, O.bf16_round(x))
  back = to_np(K.cast(K.cast(to_dev(x), torch.bfloat16), torch.float32))
  np.testing.assert_array_equal(back, O.bf16_round(x))


# ------------------------------------------------------------------ top-k
@pytest.mark.parametrize("E,k", [(3, 2), (8, 2), (32, 2), (32, 5), (100, 7), (1000, 3)])
def test_topk_exact_with_ties(K, E, k):
  rng = np.random.default_rng(E)
  g = rng.integers(0, 4, (257, E)).astype(np.float32) / 4     # heavy ties
  g[0] = 0.0
  val, idx = K.topk(to_dev(g), k)
  want_v, want_i = O.top_k(g, k)
  np.testing.assert_array_equal(to_np(idx), want_i)
  np.testing.assert_array_equal(to_np(val), want_v)


# ------------------------------------------------------------------ gating
GATE_CASES = [
    # G, S, D, E, K, dtype
    (2, 49, 512, 8, 2, O.F32),
    (3, 50, 64, 5, 3, O.F32),
    (2, 100, 768, 32, 2, O.BF16),
    (1, 33, 1024, 32, 2, O.BF16),
    (2, 64, 264, 40, 4, O.BF16),
    (2, 37, 128, 100, 2, O.F32),
    (1, 1568, 768, 32, 2, O.BF16),
    (1, 33000, 1024, 32, 2, O.BF16),   # streaming kernel, rings of two slots (the router kernel takes 66 KB)
    (1, 8200, 768, 32, 2, O.BF16),     # streaming kernel, rings of three slots, a last tile of 8 items
    (3, 2741, 768, 8, 2, O.BF16),      # streaming kernel, experts padded to the 32-wide tile
    (2, 4100, 256, 24, 3, O.BF16),     # streaming kernel, four chunks of k
    (1, 8192, 64, 16, 1, O.BF16),      # streaming kernel, a single chunk of k
    (2, 77, 2048, 32, 2, O.BF16),      # router kernel staged in two chunks along D
    (2, 45, 768, 16, 2, O.BF16),       # experts padded to the 32-wide tile
    (2, 45, 320, 12, 3, O.BF16),       # expert count not a multiple of 8: element-wise staging
    (3, 31, 72, 8, 1, O.BF16),         # D not a multiple of 64
    (2, 50, 256, 64, 2, O.BF16),       # two expert tiles
    (1, 70, 192, 128, 4, O.BF16),      # four expert tiles
    (1, 70, 96, 128, 4, O.F32),
]


@pytest.mark.parametrize("G,S,D,E,k,dtype", GATE_CASES)
def test_gate_topk(K, G, S, D, E, k, dtype):
  rng = np.random.default_rng(G * 1000 + S)
  x = O.cast(rng.standard_normal((G, S, D)), dtype)
  w = O.cast(rng.standard_normal((D, E)) / np.sqrt(D), dtype)
  gates, val, idx = K.gate_topk(to_dev(x, dtype), to_dev(w, dtype), k)
  gates, val, idx = to_np(gates), to_np(val), to_np(idx)
  want = O.router_gates(x, w, dtype)
  # Float part: tolerance stated by the north star (1e-5 fp32, 2e-2 bf16).
  assert_close(gates, want, 1e-5 if dtype == O.F32 else 2e-2, "gates")
  np.testing.assert_allclose(gates.sum(-1), 1.0, atol=1e-5 if dtype == O.F32 else 2e-2)
  # Integer part: the selection is exact given the kernel's own gates.
  want_v, want_i = O.top_k(gates, k)
  np.testing.assert_array_equal(idx, want_i)
  np.testing.assert_array_equal(val, want_v)
  flips = int((O.top_k(want, k)[1] != idx).any(-1).sum())
  print(f"gate_topk {dtype} items={G*S} top-k rows differing from oracle gates: {flips}")
  assert flips <= max(2, G * S // 100)


def test_gate_topk_logit_bias(K):
  rng = np.random.default_rng(5)
  G, S, D, E = 2, 40, 256, 32
  x = O.cast(rng.standard_normal((G, S, D)), O.BF16)
  w = O.cast(rng.standard_normal((D, E)) / np.sqrt(D), O.BF16)
  b = (rng.standard_normal(E) * 2).astype(np.float32)
  gates, _, _ = K.gate_topk(to_dev(x, O.BF16), to_dev(w, O.BF16), 2, logit_bias=to_dev(b))
  assert_close(to_np(gates), O.router_gates(x, w, O.BF16, b), 2e-2, "gates with bias")


@pytest.mark.parametrize("n,D,E", [(1568, 512, 8), (45, 64, 5), (4100, 384, 32), (33, 1024, 24)])
def test_gate_topk_float32_split_k_form(K, monkeypatch, n, D, E):
  """float32 gating over few items deals the k range of a tile to the four waves of a workgroup
  (partial logits added in wave order): against the one-wave-per-tile form
  (VMOE_GATE_NO_SPLIT_K=1) bit for bit on operands whose partial sums are exact, within float32
  rounding otherwise; logits output and logit bias included."""
  rng = np.random.default_rng(n + D)
  xi = rng.integers(-2, 3, (1, n, D)).astype(np.float32)
  wi = rng.integers(-2, 3, (D, E)).astype(np.float32) / 64
  b = (rng.integers(-8, 9, E) / 4).astype(np.float32)
  xr = rng.standard_normal((1, n, D)).astype(np.float32)
  wr = (rng.standard_normal((D, E)) / np.sqrt(D)).astype(np.float32)
  for x, w, exact in ((xi, wi, True), (xr, wr, False)):
    monkeypatch.delenv("VMOE_GATE_NO_SPLIT_K", raising=False)
    g_s, v_s, i_s, l_s = K.gate_topk(to_dev(x), to_dev(w), 2, logit_bias=to_dev(b), return_logits=True)
    g_p, v_p, i_p = K.gate_topk(to_dev(x), to_dev(w), 2)
    monkeypatch.setenv("VMOE_GATE_NO_SPLIT_K", "1")
    g_d, v_d, i_d, l_d = K.gate_topk(to_dev(x), to_dev(w), 2, logit_bias=to_dev(b), return_logits=True)
    monkeypatch.delenv("VMOE_GATE_NO_SPLIT_K")
    want = x[0].astype(np.float64) @ w.astype(np.float64) + b
    np.testing.assert_allclose(to_np(l_s)[0], want, rtol=1e-5, atol=1e-5)
    assert_close(to_np(g_p), O.router_gates(x, w, O.F32), 1e-5, "gates without bias")
    if exact:
      np.testing.assert_array_equal(to_np(l_s), to_np(l_d))
      np.testing.assert_array_equal(to_np(g_s), to_np(g_d))
      np.testing.assert_array_equal(to_np(i_s), to_np(i_d))
      np.testing.assert_array_equal(to_np(v_s), to_np(v_d))
    else:
      np.testing.assert_allclose(to_np(l_s), to_np(l_d), rtol=1e-5, atol=1e-5)
      np.testing.assert_allclose(to_np(g_s), to_np(g_d), rtol=1e-5, atol=1e-6)


def test_gate_topk_streaming_and_direct_loads_agree(K, monkeypatch):
  """The two forms of the bfloat16 gating kernel (item rows through LDS by DMA, or by direct
  loads: VMOE_GATE_DIRECT_LOADS=1) add the same products in a different order of k: equal
  bit for bit where every partial sum is exact, within a few bfloat16 steps otherwise; the
  logit bias and a call without the gates output take the streaming form too."""
  rng = np.random.default_rng(11)
  n, D, E = 8192 + 40, 768, 32
  xi = rng.integers(-2, 3, (1, n, D)).astype(np.float32)          # exact in bfloat16, sums below 2^24
  wi = rng.integers(-2, 3, (D, E)).astype(np.float32) / 64
  b = (rng.integers(-8, 9, E) / 4).astype(np.float32)
  xr = O.cast(rng.standard_normal((1, n, D)), O.BF16)
  wr = O.cast(rng.standard_normal((D, E)) / np.sqrt(D), O.BF16)
  for x, w, exact in ((xi, wi, True), (xr, wr, False)):
    monkeypatch.delenv("VMOE_GATE_DIRECT_LOADS", raising=False)
    g_s, v_s, i_s = K.gate_topk(to_dev(x, O.BF16), to_dev(w, O.BF16), 2, logit_bias=to_dev(b))
    _, v_n, i_n = K.gate_topk(to_dev(x, O.BF16), to_dev(w, O.BF16), 2, logit_bias=to_dev(b), return_gates=False)
    monkeypatch.setenv("VMOE_GATE_DIRECT_LOADS", "1")
    g_d, v_d, i_d = K.gate_topk(to_dev(x, O.BF16), to_dev(w, O.BF16), 2, logit_bias=to_dev(b))
    monkeypatch.delenv("VMOE_GATE_DIRECT_LOADS")
    np.testing.assert_array_equal(to_np(i_s), to_np(i_n))
    np.testing.assert_array_equal(to_np(v_s), to_np(v_n))
    if exact:
      np.testing.assert_array_equal(to_np(g_s), to_np(g_d))
      np.testing.assert_array_equal(to_np(i_s), to_np(i_d))
      np.testing.assert_array_equal(to_np(v_s), to_np(v_d))
      assert_close(to_np(g_s), O.router_gates(x, w, O.BF16, b), 2e-2, "gates")
    else:
      gs, gd = to_np(g_s).astype(np.float64), to_np(g_d).astype(np.float64)
      # (a logit of magnitude 2 .. 4 that rounds the other way moves by 2^-6, its gate by
      # 1.6 %, and the other gates of the item through the sum)
      assert np.all(np.abs(gs - gd) <= 2.0 ** -5 * np.maximum(np.abs(gs), np.abs(gd)) + 1e-30)
      assert float((gs != gd).mean()) < 0.05
      assert int((to_np(i_s) != to_np(i_d)).any(-1).sum()) <= n // 100


def test_router_metrics(K, goldens):
  g = goldens["router_aux_losses"]
  gates = np.asarray(g["gates"], np.float32)[None]
  _, idx = K.topk(to_dev(gates), 1)
  imp, gsh, aux = K.router_metrics(to_dev(gates), idx, 0.0, 1.0)
  assert float(gsh[0]) == pytest.approx(g["gshard"], abs=1e-6)
  assert float(imp[0]) == pytest.approx(g["importance"], abs=1e-6)
  assert float(aux[0]) == pytest.approx(g["importance"], abs=1e-6)
  rng = np.random.default_rng(1)
  for (G, S, E) in [(4, 1568, 32), (3, 49, 8), (2, 100, 300)]:
    gt = O.softmax(rng.standard_normal((G, S, E)).astype(np.float32) * 2)
    _, idx = K.topk(to_dev(gt), 2)
    imp, gsh, aux = K.router_metrics(to_dev(gt), idx, 0.5, 2.0)
    want = O.router_metrics(gt, 0.5, 2.0)
    np.testing.assert_allclose(to_np(imp), want["importance_loss"], rtol=1e-4)
    np.testing.assert_allclose(to_np(gsh), want["gshard_loss"], rtol=1e-4)
    np.testing.assert_allclose(to_np(aux), want["auxiliary_loss"], rtol=1e-4)


# ------------------------------------------------------------------ slot assignment
ROUTE_CASES = [
    # G, S, E, K, C, ties
    (1, 3, 3, 2, 2, False),
    (2, 49, 8, 2, 16, False),
    (4, 64, 8, 2, 4, True),
    (3, 100, 5, 3, 7, True),
    (32, 1568, 32, 2, 100, False),   # B/16 layer
    (16, 2304, 32, 2, 72, False),    # L/16@384, heavy dropping
    (8, 1568, 8, 2, 412, False),     # full-model layer
    (2, 1568, 32, 2, 100, True),
    (2, 513, 7, 1, 30, True),
    (1, 1, 2, 2, 1, False),
    (2, 1024, 8, 2, 100, True),      # one key per thread, lane and LDS exchanges
    (3, 1025, 4, 1, 300, False),     # two keys per thread
    (2, 2304, 32, 2, 72, True),      # four
    (1, 5000, 4, 2, 700, True),      # eight
]


@pytest.mark.parametrize("bpr", [False, True])
@pytest.mark.parametrize("G,S,E,k,C,ties", ROUTE_CASES)
def test_route_assign_bit_exact(K, G, S, E, k, C, ties, bpr):
  rng = np.random.default_rng(S * 7 + E)
  if ties:   # bf16-like coarse gates: many equal first-choice gates
    gates = O.bf16_round(O.softmax(rng.integers(-3, 4, (G, S, E)).astype(np.float32)))
  else:
    gates = O.softmax(rng.standard_normal((G, S, E)).astype(np.float32) * 2)
  val, idx = K.topk(to_dev(gates), k)
  indices, token_slot, slot_token, fill = K.route_assign(val, idx, E, C, bpr)
  indices, token_slot, slot_token, fill = map(to_np, (indices, token_slot, slot_token, fill))
  want_idx, want_w = route_c.route_batch(gates, k, bpr)
  np.testing.assert_array_equal(indices, want_idx)
  np.testing.assert_array_equal(to_np(val), want_w)
  if G * S <= 20000:   # the literal one-hot/cumsum restatement on the smaller cases
    d = O.get_top_experts_per_item_dispatcher(gates, "indices", k, bpr, capacity=C)
    np.testing.assert_array_equal(indices, d.indices)
  # Derived maps.
  e, p = want_idx[..., 0], want_idx[..., 1]
  kept = p < C
  gi = np.arange(G)[:, None, None]
  if G % E == 0:
    q = G // E
    row = ((gi % q) * E + gi // q) * C + p
  else:
    row = gi * C + p
  want_slot = np.where(kept, e * (G * C) + row, -1)
  np.testing.assert_array_equal(token_slot, want_slot)
  want_st = np.full(E * G * C, -1, np.int32)
  item = (np.arange(G * S).reshape(G, S, 1) + np.zeros((1, 1, k), np.int64))
  want_st[want_slot[kept]] = item[kept]
  np.testing.assert_array_equal(slot_token, want_st)
  demand = np.stack([np.bincount(e[g].ravel(), minlength=E) for g in range(G)])
  np.testing.assert_array_equal(fill, np.minimum(demand, C))


@pytest.mark.parametrize("bpr", [False, True])
@pytest.mark.parametrize("G,S,E,k,C,dtype", [(4, 64, 8, 2, 4, O.F32), (32, 1568, 32, 2, 100, O.BF16),
                                             (3, 100, 5, 3, 7, O.F32), (2, 2304, 32, 2, 72, O.BF16),
                                             (2, 50, 100, 2, 3, O.F32)])
def test_route_assign_with_metrics_equals_separate_calls(K, G, S, E, k, C, dtype, bpr):
  """One launch for slot assignment and the router's losses: every output has the bits
  of the two separate entry points."""
  rng = np.random.default_rng(S + E)
  gates = to_dev(O.cast(O.softmax(rng.standard_normal((G, S, E)).astype(np.float32) * 2), dtype), dtype)
  val, idx = K.topk(gates.float(), k)
  want = K.route_assign(val, idx, E, C, bpr)
  want_losses = K.router_metrics(gates, idx, 0.25, 1.0)
  got = K.route_assign(val, idx, E, C, bpr, metrics=(gates, 0.25, 1.0))
  for a, b in zip(got[:4], want):
    assert torch.equal(a, b)
  for a, b in zip(got[4], want_losses):
    assert torch.equal(a, b)


def test_route_assign_random_shapes(K):
  """Seeded sweep over group sizes around the sort's switch points (keys per thread,
  partial waves), expert counts, gate flavours (float32, bfloat16-valued -> 32-bit sort
  keys, coarse values with many ties, negative and zero gates) against the sequential
  C statement of the assignment."""
  rng = np.random.default_rng(2024)
  sizes = [1, 2, 3, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, 513, 1000,
           1023, 1024, 1025, 1500, 2047, 2048, 2049, 3000, 4095, 4096, 4097]
  for case, S in enumerate(sizes * 2):
    E = int(rng.integers(1, 41))
    k = int(rng.integers(1, min(E, 4) + 1))
    G = int(rng.integers(1, 4))
    C = int(rng.integers(1, max(2, (S * k) // E + 3)))
    flavour = case % 4
    pow2 = 1 << max(0, (S - 1).bit_length())
    keys = 8 * max(pow2, (2 * 1024 + S + 1) // 2)   # sort keys, or the counting rank's two 1 024-word arrays and S items
    lds = keys + 8 * E * ((S * k + 31) // 32) + 4 * S + 4 * E
    if lds > 160 * 1024:      # the entry point's documented limit: such shapes are refused
      E = max(k, (160 * 1024 - keys - 4 * S) // (8 * ((S * k + 31) // 32) + 4) - 1)
    logits = rng.standard_normal((G, S, E)).astype(np.float32) * 2
    if flavour == 0:
      gates = O.softmax(logits)
    elif flavour == 1:
      gates = O.bf16_round(O.softmax(logits))
    elif flavour == 2:
      gates = O.bf16_round(O.softmax(np.round(logits)))      # many equal gates
    else:
      gates = np.round(logits * 2).astype(np.float32) / 4       # negative, zero and tied "gates"
    val, idx = K.topk(to_dev(gates), k)
    got, _, _, fill = K.route_assign(val, idx, E, C, True)
    want, want_w = route_c.route_batch(gates, k, True)
    np.testing.assert_array_equal(to_np(got), want, err_msg=f"S={S} E={E} k={k} G={G} C={C} flavour={flavour}")
    np.testing.assert_array_equal(to_np(val), want_w)
    e = want[..., 0]
    demand = np.stack([np.bincount(e[g].ravel(), minlength=E) for g in range(G)])
    np.testing.assert_array_equal(to_np(fill), np.minimum(demand, C))


def test_route_assign_golden(K, goldens):
  g = goldens["top_experts_per_item"]
  gates = np.asarray(g["gates"], np.float32)[None]
  val, idx = K.topk(to_dev(gates), 2)
  for bpr, key in ((False, "vanilla"), (True, "bpr")):
    indices, *_ = K.route_assign(val, idx, 3, g["capacity"], bpr)
    np.testing.assert_array_equal(to_np(indices)[0], np.asarray(g["indices"][key]))
    cw, dw = K.densify(indices, val, 3, g["capacity"])
    np.testing.assert_array_almost_equal(to_np(cw)[0], np.asarray(g["einsum_combine_weights"][key]))
    np.testing.assert_array_equal(to_np(dw)[0], np.asarray(g["einsum_combine_weights"][key]) > 0)
  np.testing.assert_array_almost_equal(to_np(val)[0], np.asarray(g["indices_combine_weights"]))


# ------------------------------------------------------------------ dispatch / combine
@pytest.mark.parametrize("case", ["dispatcher_experts_divide_groups",
                                  "dispatcher_groups_divide_experts"])
def test_dispatch_combine_golden(K, goldens, case):
  g = goldens[case]
  E, C = g["num_experts"], g["capacity"]
  data = np.asarray(goldens["dispatcher_data"]["data"], np.float32)
  idx = to_dev(np.asarray(g["indices"], np.int32))
  w = np.tile(np.asarray(g["indices_combine_weights_tile"], np.float32)[None, None], (2, 3, 1))
  token_slot, slot_token, counters = K.indices_to_slots(idx, E, C)
  assert to_np(counters).tolist() == [0, 0]
  buf = K.dispatch(to_dev(data.reshape(6, 4)), token_slot.view(6, 2), slot_token)
  np.testing.assert_array_equal(to_np(buf).reshape(E, 2 * C, 4), np.asarray(g["expected_dispatch"]))
  out = K.combine(buf, token_slot.view(6, 2), to_dev(w.reshape(6, 2)))
  np.testing.assert_array_almost_equal(to_np(out).reshape(2, 3, 4), np.asarray(g["expected_combine"]))


def test_indices_to_slots_flags_duplicates_and_negatives(K):
  idx = np.asarray([[[[0, 0]], [[0, 0]], [[-1, 0]]]], np.int32)   # G=1,S=3,K=1
  _, _, counters = K.indices_to_slots(to_dev(idx), 2, 2)
  assert to_np(counters).tolist() == [1, 1]


MOVE_CASES = [
    # G, S, E, K, C, D, dtype
    (2, 49, 8, 2, 16, 512, O.F32),
    (4, 33, 8, 2, 4, 64, O.F32),      # G/E not integral -> swapaxes branch
    (8, 64, 4, 2, 20, 256, O.BF16),   # G/E = 2 -> permuted branch
    (3, 50, 6, 3, 9, 72, O.BF16),
    (4, 1568, 32, 2, 100, 768, O.BF16),
    (2, 2304, 32, 2, 72, 1024, O.BF16),
]


@pytest.mark.parametrize("G,S,E,k,C,D,dtype", MOVE_CASES)
def test_dispatch_combine_bit_exact(K, G, S, E, k, C, D, dtype):
  rng = np.random.default_rng(D + S)
  gates = O.cast(O.softmax(rng.standard_normal((G, S, E)).astype(np.float32) * 2), dtype)
  x = O.cast(rng.standard_normal((G, S, D)), dtype)
  d = O.get_top_experts_per_item_dispatcher(gates, "indices", k, True, capacity=C)
  val, idx = K.topk(to_dev(gates), k)
  indices, token_slot, slot_token, _ = K.route_assign(val, idx, E, C, True)
  np.testing.assert_array_equal(to_np(indices), d.indices)
  buf = K.dispatch(to_dev(x, dtype).view(G * S, D), token_slot.view(G * S, k), slot_token)
  want_buf = d.dispatch(x)
  np.testing.assert_array_equal(to_np(buf).reshape(E, G * C, D), want_buf)
  y = O.cast(rng.standard_normal((E, G * C, D)), dtype)
  out = K.combine(to_dev(y, dtype).view(E * G * C, D), token_slot.view(G * S, k), val.view(G * S, k))
  want = O.cast(d.combine(y), dtype)
  np.testing.assert_array_equal(to_np(out).reshape(G, S, D), want)
  # Idempotence / determinism: a second run gives the same bits.
  buf2 = K.dispatch(to_dev(x, dtype).view(G * S, D), token_slot.view(G * S, k), slot_token)
  assert torch.equal(buf, buf2)


def test_dispatch_combine_round_trip_full_size(K):
  """B/16 layer size: combine(dispatch(x)) with unit weights returns x times the
  number of kept assignments of each item (size-independent property)."""
  G, S, E, k, C, D = 32, 1568, 32, 2, 100, 768
  gen = torch.Generator(device="cpu").manual_seed(0)
  gates = torch.softmax(torch.randn((G, S, E), generator=gen) * 2, -1).to(dev())
  x = torch.randn((G * S, D), generator=gen).to(torch.bfloat16).to(dev())
  val, idx = K.topk(gates, k)
  indices, token_slot, slot_token, fill = K.route_assign(val, idx, E, C, True)
  buf = K.dispatch(x, token_slot.view(G * S, k), slot_token)
  ones = torch.ones((G * S, k), dtype=torch.float32, device=dev())
  out = K.combine(buf, token_slot.view(G * S, k), ones)
  kept = (token_slot.view(G * S, k) >= 0).sum(-1, keepdim=True).to(torch.float32)
  want = (x.to(torch.float32) * kept).to(torch.bfloat16)
  assert torch.equal(out, want)
  # Every slot is either an exact copy of its item or zero; fill matches occupancy.
  st = slot_token.view(E, -1)
  assert int((st >= 0).sum()) == int(fill.sum())
  empty = (slot_token < 0)
  assert float(buf[empty].abs().max() if empty.any() else 0.0) == 0.0


# ------------------------------------------------------------------ expert MLP
MLP_CASES = [
    # E, R, D, M, dtype
    (2, 40, 64, 128, O.F32),
    (8, 512, 512, 2048, O.F32),       # S/32-style layer, full size
    (3, 100, 96, 200, O.F32),         # column tile that ends inside the matrix; second product's k not whole tiles
    (3, 100, 96, 160, O.F32),         # both products through the LDS-DMA kernel, ragged rows and columns
    (3, 100, 72, 136, O.BF16),        # ragged everything
    (2, 300, 256, 512, O.BF16),
    (3, 300, 64, 192, O.BF16),        # shortest second product the tile-walking kernel takes (6 k tiles)
    (4, 3200, 768, 3072, O.BF16),     # B/16 experts (4 of 32)
]


@pytest.mark.parametrize("prepacked", [False, True])
@pytest.mark.parametrize("E,R,D,M,dtype", MLP_CASES)
def test_expert_mlp(K, E, R, D, M, dtype, prepacked):
  if prepacked and dtype == O.F32:
    pytest.skip("float32 path reads the reference layout directly")
  rng = np.random.default_rng(R)
  x = O.cast(rng.standard_normal((E, R, D)), dtype)
  w0 = O.cast(rng.standard_normal((E, D, M)) / np.sqrt(D), dtype)
  b0 = O.cast(rng.standard_normal((E, M)) * 0.1, dtype)
  w1 = O.cast(rng.standard_normal((E, M, D)) / np.sqrt(M), dtype)
  b1 = O.cast(rng.standard_normal((E, D)) * 0.1, dtype)
  dx, dw0, db0, dw1, db1 = (to_dev(a, dtype) for a in (x, w0, b0, w1, b1))
  kw = {}
  if prepacked:
    kw = dict(w0t=K.pack_expert_weights(dw0), w1t=K.pack_expert_weights(dw1))
    np.testing.assert_array_equal(to_np(kw["w0t"]), w0.transpose(0, 2, 1))
  out = to_np(K.expert_mlp(dx, dw0, db0, dw1, db1, **kw))
  want = O.mlp_block(x, w0, b0, w1, b1, dtype)
  assert_close(out, want, 1e-5 if dtype == O.F32 else 2e-2, "expert mlp")


def test_expert_mlp_erf_gelu_and_no_bias(K):
  rng = np.random.default_rng(9)
  E, R, D, M = 2, 64, 64, 128
  x = rng.standard_normal((E, R, D)).astype(np.float32)
  w0 = (rng.standard_normal((E, D, M)) / 8).astype(np.float32)
  w1 = (rng.standard_normal((E, M, D)) / 11).astype(np.float32)
  out = to_np(K.expert_mlp(to_dev(x), to_dev(w0), None, to_dev(w1), None, approximate_gelu=False))
  assert_close(out, O.mlp_block(x, w0, None, w1, None, O.F32, approximate_gelu=False), 1e-5, "erf")


# ------------------------------------------------------------------ error handling
def test_bad_arguments_return_error_codes(K):
  from vmoe_amd import _hip as H
  x = torch.randn((1, 4, 12), device=dev()).to(torch.bfloat16)       # D % 8 != 0
  w = torch.randn((12, 4), device=dev()).to(torch.bfloat16)
  val = torch.empty((4, 2), dtype=torch.float32, device=dev())
  idx = torch.empty((4, 2), dtype=torch.int32, device=dev())
  with pytest.raises(H.VmoeError, match="aligned"):                  # the C ABI refuses the width
    H.call("vmoe_gate_topk", H.GateTopkParams(H.ptr(x), H.ptr(w), None, None, H.ptr(val),
                                              H.ptr(idx), 4, 12, 4, 2, H.BF16, None))
  gates, _, _ = K.gate_topk(x, w, 2)                                 # the wrapper pads with zeros
  want = torch.softmax((x.float() @ w.float()).to(torch.bfloat16).float(), -1)
  np.testing.assert_allclose(to_np(gates), to_np(want), rtol=1e-2, atol=1e-3)
  x = torch.zeros((1, 4, 16), dtype=torch.float32, device=dev())
  w = torch.zeros((16, 4), dtype=torch.float32, device=dev())
  with pytest.raises(H.VmoeError, match="invalid sizes"):
    K.gate_topk(x, w, 5)                                             # K > E
  with pytest.raises(H.VmoeError, match="no CPU fallback"):
    K.gate_topk(x.cpu(), w.cpu(), 2)
  with pytest.raises(TypeError):
    K.gate_topk(x.double(), w.double(), 2)
  idx = torch.zeros((1, 4, 2), dtype=torch.int32, device=dev())
  with pytest.raises(H.VmoeError, match="invalid sizes"):
    K.route_assign(None, idx, 1, 4, False)                           # K > E
  with pytest.raises(H.VmoeError, match="null"):
    K.route_assign(None, idx, 4, 4, True)                            # BPR needs the gates


# ------------------------------------------------------------------ Soft MoE
SOFT_CASES = [
    # G, S, D, n, p, dtype
    (1, 8, 16, 5, 2, O.F32),
    (3, 50, 64, 7, 3, O.F32),
    (2, 196, 768, 128, 1, O.BF16),
    (4, 100, 256, 16, 2, O.BF16),
    (1, 2, 16, 4, 2, O.F32),          # inputs smaller than mu: the scale multiplies the inputs
    # every model width of the register-resident bf16 path, ragged S and N
    (3, 77, 384, 24, 1, O.BF16),
    (2, 130, 512, 8, 5, O.BF16),
    (2, 33, 1024, 128, 1, O.BF16),
    (1, 300, 256, 104, 1, O.BF16),
    (1, 20, 768, 64, 2, O.BF16),      # inputs smaller than mu on the bf16 path
    (2, 64, 768, 20, 1, O.BF16),      # N % 8 != 0: generic path
    (2, 64, 320, 16, 1, O.BF16),      # width outside the fast path
    # two-role kernel with 16-row item tiles (two 32-row tiles do not fit LDS beside the
    # logits): dispatch softmax from registers (S <= 256) and in three passes
    (1, 250, 768, 128, 1, O.BF16),
    (2, 260, 768, 128, 1, O.BF16),
]


@pytest.mark.parametrize("G,S,D,n,p,dtype", SOFT_CASES)
def test_soft_route(K, G, S, D, n, p, dtype):
  rng = np.random.default_rng(S + n)
  x = O.cast(rng.standard_normal((G, S, D)), dtype)
  mu = O.cast(rng.standard_normal((D, n, p)) / np.sqrt(D), dtype)
  scale = 1.75
  dw, cw, lg = K.soft_route(to_dev(x, dtype), to_dev(mu.reshape(D, n * p), dtype), scale,
                            return_logits=True)
  wl, wd, wc, _ = O.soft_router_weights(x, mu, scale, dtype)
  tol = 1e-5 if dtype == O.F32 else 2e-2
  assert_close(to_np(lg), wl.reshape(G, S, n * p), tol * (1 if dtype == O.BF16 else 4), "logits")
  assert_close(to_np(dw), wd.reshape(G, S, n * p), tol * 4, "dispatch weights")
  assert_close(to_np(cw), wc.reshape(G, S, n * p), tol * 4, "combine weights")
  _check_soft_weights_against_own_logits(to_np(lg), to_np(dw), to_np(cw), dtype, "")
  atol = 1e-4 if dtype == O.F32 else 3e-2
  np.testing.assert_allclose(to_np(dw).sum(1), 1.0, atol=atol)
  np.testing.assert_allclose(to_np(cw).sum(2), 1.0, atol=atol)


def _check_soft_weights_against_own_logits(lg, dw, cw, dtype, tag):
  """The two softmaxes themselves.  Against the oracle the weights carry the difference of the
  logits (a bfloat16 logit that rounds the other way moves a weight by exp(step) - 1, which is
  why those comparisons are loose); against the float64 softmaxes of the logits that the kernel
  itself returned -- the values its softmaxes start from -- nothing is left but the softmax
  arithmetic and one rounding: two units in the last place of the weights' type (bfloat16: 8
  significant bits; float32: rtol 1e-5 for the float32 exponentials and sums).  A wrong
  denominator, a missing maximum or a softmax over the wrong axis does not pass."""
  lg64 = np.asarray(lg, np.float64)
  for name, got, axis in (("dispatch weights", dw, 1), ("combine weights", cw, 2)):
    e = np.exp(lg64 - lg64.max(axis=axis, keepdims=True))
    want = e / e.sum(axis=axis, keepdims=True)
    got = np.asarray(got, np.float64)
    if dtype == O.BF16:
      allowed = 2.0 ** (np.floor(np.log2(np.maximum(want, 1e-300))) - 7 + 1) + 1e-38
    else:
      allowed = 1e-5 * want + 1e-30
    bad = np.abs(got - want) > allowed
    assert not bad.any(), (f"{name} {tag}: {bad.sum()} of {bad.size} further than two units in the last "
                           f"place from the softmax of the kernel's own logits; worst ratio "
                           f"{float((np.abs(got - want) / allowed).max()):.2f}")


def test_soft_route_seeded_shapes(K):
  """Seeded sweep over the shapes of the bfloat16 fast paths (model widths, N a multiple of 8 up
  to 128, group sizes around the tile heights and around the 256 items that the
  register-resident dispatch softmax holds) against the oracle."""
  rng = np.random.default_rng(2024)
  special_s = [1, 15, 16, 17, 31, 32, 33, 63, 64, 65, 223, 224, 225, 255, 256, 257, 300]
  for trial in range(16):
    D = int(rng.choice([256, 384, 512, 768, 1024]))
    n = int(rng.integers(1, 17)) * 8
    S = int(rng.choice(special_s)) if trial % 2 == 0 else int(rng.integers(1, 320))
    G = int(rng.integers(1, 4))
    x = O.cast(rng.standard_normal((G, S, D)), O.BF16)
    mu = O.cast(rng.standard_normal((D, n, 1)) / np.sqrt(D), O.BF16)
    scale = float(rng.uniform(0.5, 2.0))
    dw, cw, lg = K.soft_route(to_dev(x, O.BF16), to_dev(mu.reshape(D, n), O.BF16), scale,
                              return_logits=True)
    wl, wd, wc, _ = O.soft_router_weights(x, mu, scale, O.BF16)
    tag = f"G={G} S={S} D={D} N={n}"
    assert_close(to_np(lg), wl.reshape(G, S, n), 2e-2, "logits " + tag)
    assert_close(to_np(dw), wd.reshape(G, S, n), 8e-2, "dispatch weights " + tag)
    assert_close(to_np(cw), wc.reshape(G, S, n), 8e-2, "combine weights " + tag)
    _check_soft_weights_against_own_logits(to_np(lg), to_np(dw), to_np(cw), O.BF16, tag)
    np.testing.assert_allclose(to_np(dw).sum(1), 1.0, atol=3e-2, err_msg=tag)
    np.testing.assert_allclose(to_np(cw).sum(2), 1.0, atol=3e-2, err_msg=tag)


@pytest.mark.parametrize("G,S,D,N", [(5, 196, 768, 128), (2, 250, 768, 128), (3, 100, 512, 64),
                                     (2, 300, 256, 104), (2, 37, 384, 40)])
def test_soft_route_two_roles_and_single_role_agree(K, G, S, D, N):
  """The kernel whose waves split into producers and consumers against the single-role kernel
  (VMOE_SOFT_ROUTE_SINGLE_ROLE=1): same arithmetic per element, different summation order in
  the norms and softmax sums: a norm that rounds the other way moves a normalised item by one
  bfloat16 step, a logit by about as much, and a weight by up to exp(step) - 1, in few places."""
  rng = np.random.default_rng(G * S + N)
  x = to_dev(O.cast(rng.standard_normal((G, S, D)), O.BF16), O.BF16)
  mu = to_dev(O.cast(rng.standard_normal((D, N)) / np.sqrt(D), O.BF16), O.BF16)
  got = [to_np(a) for a in K.soft_route(x, mu, 1.3, return_logits=True)]
  os.environ["VMOE_SOFT_ROUTE_SINGLE_ROLE"] = "1"
  try:
    want = [to_np(a) for a in K.soft_route(x, mu, 1.3, return_logits=True)]
  finally:
    del os.environ["VMOE_SOFT_ROUTE_SINGLE_ROLE"]
  for name, a, b in zip(("dispatch weights", "combine weights", "logits"), got, want):
    diff = np.abs(a - b)
    floor = 2.0 ** -7 * np.abs(b).max() if name == "logits" else 0.0
    assert (diff <= 2.0 ** -5 * np.abs(b) + floor).all(), (name, float((diff / (np.abs(b) + 1e-30)).max()))
    assert (diff > 0).mean() <= 1e-3, (name, float((diff > 0).mean()))


EINSUM_CASES = [
    # G, S, E, C, D, wdtype, ddtype
    (2, 3, 2, 2, 4, O.F32, O.F32),
    (2, 3, 4, 1, 4, O.F32, O.F32),
    (4, 50, 2, 3, 40, O.F32, O.BF16),     # Bfloat16Dispatcher over float32 weights
    (8, 196, 4, 2, 96, O.BF16, O.BF16),
    (3, 33, 5, 1, 20, O.F32, O.F32),
    # all-bfloat16 cases take the bf16 matrix-core path where its limits allow
    (5, 17, 3, 8, 72, O.BF16, O.BF16),      # G % 8 != 0, ragged S and D
    (8, 256, 4, 34, 200, O.BF16, O.BF16),   # E*C = 136: two row blocks in dispatch, generic combine
    (16, 196, 128, 1, 128, O.BF16, O.BF16), # Soft MoE B/16 rows, E does not divide G
    (8, 100, 4, 8, 64, O.BF16, O.BF16),     # E divides G: interleaved buffer order
    (3, 257, 2, 4, 64, O.BF16, O.BF16),     # S above the bf16 path's limit
]


@pytest.mark.parametrize("G,S,E,C,D,wdtype,ddtype", EINSUM_CASES)
def test_einsum_dispatch_combine(K, G, S, E, C, D, wdtype, ddtype):
  rng = np.random.default_rng(G + S)
  w = O.cast(O.softmax(rng.standard_normal((G, S, E * C)).astype(np.float32)), wdtype)
  w = w.reshape(G, S, E, C)
  x = O.cast(rng.standard_normal((G, S, D)), ddtype)
  d = O.EinsumDispatcher(w, w)
  out_dtype = wdtype if wdtype == ddtype else O.F32
  buf = K.einsum_dispatch(to_dev(w, wdtype), to_dev(x, ddtype), tdtype(out_dtype))
  want = O.cast(d.dispatch(x), out_dtype)
  # bf16 x bf16 products are exact in float32: only the summation order differs.
  tol = 1e-5 if out_dtype == O.F32 else 8e-3
  assert_close(to_np(buf).reshape(E, G * C, D), want, tol, "einsum dispatch")
  y = O.cast(rng.standard_normal((E, G * C, D)), ddtype)
  out = K.einsum_combine(to_dev(w, wdtype), to_dev(y, ddtype).view(E * G * C, D), tdtype(out_dtype))
  assert_close(to_np(out), O.cast(d.combine(y), out_dtype), tol, "einsum combine")


def test_einsum_golden_and_bool_weights(K, goldens):
  data = np.asarray(goldens["dispatcher_data"]["data"], np.float32)
  for case in ("dispatcher_experts_divide_groups", "dispatcher_groups_divide_experts"):
    g = goldens[case]
    cw = np.asarray(g["einsum_combine_weights"], np.float32)
    E, C = g["num_experts"], g["capacity"]
    buf = K.einsum_dispatch(to_dev(cw > 0), to_dev(data), torch.float32)
    np.testing.assert_array_almost_equal(to_np(buf).reshape(E, 2 * C, 4), np.asarray(g["expected_dispatch"]))
    out = K.einsum_combine(to_dev(cw), buf, torch.float32)
    np.testing.assert_array_almost_equal(to_np(out), np.asarray(g["expected_combine"]))


# ------------------------------------------------------------------ packed expert rows
@pytest.mark.parametrize("G,S,E,Kk,C,bpr", [(4, 64, 4, 2, 20, True), (8, 50, 8, 2, 16, False), (8, 128, 8, 2, 30, False), (32, 1568, 32, 2, 100, True),
                                            (3, 33, 5, 1, 8, True), (300, 16, 4, 2, 6, False),
                                            (64, 128, 4, 2, 6, True), (9, 300, 7, 2, 40, True), (2, 200, 300, 2, 3, False),
                                            (32, 49, 8, 2, 16, False),      # S/32 layer: a block of 256 assignments touches four groups
                                            (40, 19, 8, 2, 6, True)])        # 38 per group: eight groups per block, the most the one-launch form takes
def test_compact_rows(K, G, S, E, Kk, C, bpr):
  """token_row = e*G*C + (kept items of expert e in the groups before g) + position."""
  rng = np.random.default_rng(G * S + E)
  gates = O.softmax(rng.standard_normal((G, S, E)).astype(np.float32) * 2)
  val, idx = K.topk(to_dev(gates), Kk)
  indices, token_slot, slot_token, fill = K.route_assign(val, idx, E, C, bpr)
  token_row, rows, row_token = K.compact_rows(fill, token_slot, C)
  f = to_np(fill)
  np.testing.assert_array_equal(to_np(rows), f.sum(0))
  ind = to_np(indices)
  prefix = np.cumsum(f, axis=0) - f                         # (G, E)
  e, pos = ind[..., 0], ind[..., 1]
  kept = pos < C
  want = np.where(kept, e * (G * C) + np.take_along_axis(
      prefix[:, None, :].repeat(S, 1), e, axis=2) + pos, -1)
  np.testing.assert_array_equal(to_np(token_row), want)
  # row_token is the inverse map on the packed rows
  tr, rt = to_np(token_row).reshape(G * S, Kk), to_np(row_token).reshape(-1)
  items = np.repeat(np.arange(G * S), Kk).reshape(G * S, Kk)
  np.testing.assert_array_equal(rt[tr[tr >= 0]], items[tr >= 0])
  # a bijection onto the first rows of every expert
  r = to_np(token_row)[kept]
  assert len(np.unique(r)) == r.size
  for ee in range(E):
    mine = r[(r // (G * C)) == ee] - ee * G * C
    assert sorted(mine) == list(range(f.sum(0)[ee]))


@pytest.mark.parametrize("E,R,D,M", [
    (8, 416, 512, 2048),      # the S/32 layer: one expert per die
    (5, 700, 512, 1024),      # runs that begin and end inside an expert
    (3, 1000, 512, 1536),
])
def test_expert_mlp_float32_products_on_the_dma_kernel(K, monkeypatch, E, R, D, M):
  """The float32 products on the LDS-DMA kernel (64 x 128 or 64 x 64 tiles, one run of the tile
  list per die, rows past a count skipped in blocks of 32) against the register-staged kernel
  and against the oracle; dense and over ragged rows."""
  rng = np.random.default_rng(E + R)
  x = rng.standard_normal((E, R, D)).astype(np.float32)
  w0 = (rng.standard_normal((E, D, M)) / np.sqrt(D)).astype(np.float32)
  b0 = (rng.standard_normal((E, M)) * 0.1).astype(np.float32)
  w1 = (rng.standard_normal((E, M, D)) / np.sqrt(M)).astype(np.float32)
  b1 = (rng.standard_normal((E, D)) * 0.1).astype(np.float32)
  args = [to_dev(a) for a in (x, w0, b0, w1, b1)]
  rows = rng.integers(0, R + 1, E).astype(np.int32)
  rows[:3] = [R, 0, 33]
  want = O.mlp_block(x, w0, b0, w1, b1, O.F32)
  outs = {}
  for form in ("dma", "64", "plain"):
    if form != "dma":
      monkeypatch.setenv("VMOE_F32_GEMM", form)
    dense = to_np(K.expert_mlp(*args))
    ragged = torch.full((E, R, D), 7.0, dtype=torch.float32, device=dev())
    K.expert_mlp(*args, out=ragged, rows_per_expert=to_dev(rows))
    outs[form] = (dense, to_np(ragged))
    assert_close(dense, want, 1e-5, f"{form}: dense")
    for e, n in enumerate(rows):
      np.testing.assert_array_equal(outs[form][1][e, :n], dense[e, :n], err_msg=f"{form}: expert {e}")
      assert (outs[form][1][e, n:] == 7.0).all(), f"{form}: expert {e} wrote past its rows"
  monkeypatch.delenv("VMOE_F32_GEMM")
  assert_close(outs["dma"][0], outs["plain"][0], 1e-5, "dma against plain")   # other order of k
  np.testing.assert_array_equal(outs["dma"][0], outs["64"][0])              # same order of k


def test_expert_mlp_float32_seeded_shapes(K):
  """A seeded sweep of float32 expert MLPs over odd shapes (rows short of a block, widths that
  end inside a tile, k that is or is not whole 32-wide tiles, many or few experts), dense and
  over ragged rows, against the oracle at 1e-5: whichever kernel the shape takes."""
  rng = np.random.default_rng(2024)
  for case in range(14):
    E = int(rng.choice([1, 2, 3, 8, 11, 40]))
    R = int(rng.choice([1, 7, 31, 33, 64, 65, 130, 257]))
    D = int(rng.choice([32, 36, 64, 96, 100, 160, 224]))
    M = int(rng.choice([32, 40, 64, 128, 132, 192, 288]))
    x = rng.standard_normal((E, R, D)).astype(np.float32)
    w0 = (rng.standard_normal((E, D, M)) / np.sqrt(D)).astype(np.float32)
    b0 = (rng.standard_normal((E, M)) * 0.1).astype(np.float32)
    w1 = (rng.standard_normal((E, M, D)) / np.sqrt(M)).astype(np.float32)
    b1 = (rng.standard_normal((E, D)) * 0.1).astype(np.float32)
    rows = rng.integers(0, R + 1, E).astype(np.int32)
    rows[0] = R
    want = O.mlp_block(x, w0, b0, w1, b1, O.F32)
    args = [to_dev(a) for a in (x, w0, b0, w1, b1)]
    dense = to_np(K.expert_mlp(*args))
    assert_close(dense, want, 1e-5, f"case {case}: E={E} R={R} D={D} M={M} dense")
    ragged = torch.full((E, R, D), 7.0, dtype=torch.float32, device=dev())
    K.expert_mlp(*args, out=ragged, rows_per_expert=to_dev(rows))
    ragged = to_np(ragged)
    for e, n in enumerate(rows):
      np.testing.assert_array_equal(ragged[e, :n], dense[e, :n], err_msg=f"case {case}: E={E} R={R} D={D} M={M} expert {e}")
      assert (ragged[e, n:] == 7.0).all(), f"case {case}: expert {e} wrote past its rows"


def test_expert_mlp_bfloat16_seeded_shapes(K):
  """The same sweep in bfloat16 (widths in multiples of 8): dense against the oracle, ragged
  rows bit for bit against the dense call and nothing written past them, and, where the shape
  allows it, rows gathered from the items bit for bit against rows indexed beforehand."""
  rng = np.random.default_rng(2025)
  gathered = 0
  for case in range(14):
    E = int(rng.choice([1, 2, 3, 8, 11, 40]))
    R = int(rng.choice([1, 7, 31, 33, 64, 65, 130, 257, 300]))
    D = int(rng.choice([32, 40, 64, 96, 104, 160, 256]))
    M = int(rng.choice([32, 48, 64, 128, 136, 192, 512]))
    T = int(rng.choice([R, 3 * R + 5]))
    name = f"case {case}: E={E} R={R} D={D} M={M} T={T}"
    items = O.cast(rng.standard_normal((T, D)).astype(np.float32), O.BF16)
    w0 = O.cast((rng.standard_normal((E, D, M)) / np.sqrt(D)).astype(np.float32), O.BF16)
    b0 = O.cast((rng.standard_normal((E, M)) * 0.1).astype(np.float32), O.BF16)
    w1 = O.cast((rng.standard_normal((E, M, D)) / np.sqrt(M)).astype(np.float32), O.BF16)
    b1 = O.cast((rng.standard_normal((E, D)) * 0.1).astype(np.float32), O.BF16)
    rows = rng.integers(0, R + 1, E).astype(np.int32)
    rows[0] = R
    x_rows = rng.integers(0, T, (E, R)).astype(np.int32)
    x = items[x_rows]                                                      # (E, R, D)
    want = O.mlp_block(x, w0, b0, w1, b1, O.BF16)
    wd = [to_dev(a, O.BF16) for a in (w0, b0, w1, b1)]
    dense = K.expert_mlp(to_dev(x, O.BF16), *wd)
    assert_close(to_np(dense), want, 2e-2, name + " dense")
    ragged = torch.full((E, R, D), 7.0, dtype=torch.bfloat16, device=dev())
    K.expert_mlp(to_dev(x, O.BF16), *wd, out=ragged, rows_per_expert=to_dev(rows))
    for e, n in enumerate(rows):
      assert torch.equal(ragged[e, :n], dense[e, :n]), name + f" expert {e}"
      assert (to_np(ragged[e, n:]) == 7.0).all(), name + f": expert {e} wrote past its rows"
    if K.expert_mlp_can_gather(torch.bfloat16, D, T):
      gathered += 1
      for e, n in enumerate(rows):
        x_rows[e, n:] = 2 ** 30                                            # never followed
      got = torch.full((E, R, D), 7.0, dtype=torch.bfloat16, device=dev())
      K.expert_mlp(to_dev(items, O.BF16), *wd, out=got, rows_per_expert=to_dev(rows),
                   x_rows=to_dev(x_rows))
      assert torch.equal(got, ragged), name + " gathered"
  assert gathered >= 4


@pytest.mark.parametrize("dtype", [O.F32, O.BF16])
def test_expert_mlp_gathers_its_rows_from_the_items(K, dtype):
  """x_rows: the first product reads row r of expert e from item x_rows[e][r] of the (T, D)
  matrix of items.  Bit for bit what the same call computes on a buffer built by indexing;
  entries past an expert's count (here out of range on purpose) are never followed."""
  rng = np.random.default_rng(17)
  E, R, D, M, T = 6, 200, 96, 160, 500
  items = to_dev(O.cast(rng.standard_normal((T, D)).astype(np.float32), dtype), dtype)
  w0 = to_dev(O.cast(rng.standard_normal((E, D, M)).astype(np.float32) / np.sqrt(D), dtype), dtype)
  w1 = to_dev(O.cast(rng.standard_normal((E, M, D)).astype(np.float32) / np.sqrt(M), dtype), dtype)
  b0 = to_dev(O.cast(rng.standard_normal((E, M)).astype(np.float32) * 0.1, dtype), dtype)
  b1 = to_dev(O.cast(rng.standard_normal((E, D)).astype(np.float32) * 0.1, dtype), dtype)
  rows = np.asarray([200, 0, 1, 65, 128, 199], np.int32)
  x_rows = np.full((E, R), 2 ** 30, np.int32)
  for e, n in enumerate(rows):
    x_rows[e, :n] = rng.integers(0, T, n)
  assert K.expert_mlp_can_gather(tdtype(dtype), D, T)
  got = torch.full((E, R, D), 7.0, dtype=tdtype(dtype), device=dev())
  K.expert_mlp(items, w0, b0, w1, b1, out=got, rows_per_expert=to_dev(rows), x_rows=to_dev(x_rows))
  buf = items[torch.from_numpy(np.where(x_rows < T, x_rows, 0)).to(dev()).long()]      # (E, R, D)
  want = torch.full((E, R, D), 7.0, dtype=tdtype(dtype), device=dev())
  K.expert_mlp(buf, w0, b0, w1, b1, out=want, rows_per_expert=to_dev(rows))
  assert torch.equal(got, want)
  for e, n in enumerate(rows):
    assert (to_np(got[e, n:]) == 7.0).all()
  full = O.mlp_block(to_np(buf).astype(np.float32), to_np(w0), to_np(b0), to_np(w1), to_np(b1), dtype)
  for e, n in enumerate(rows):
    assert_close(to_np(got[e, :n]), full[e, :n], 1e-5 if dtype == O.F32 else 2e-2, f"expert {e}")


@pytest.mark.parametrize("dtype", [O.F32, O.BF16])
@pytest.mark.parametrize("E", [5, 20])      # fewer / more experts than dies in the launch plan
def test_expert_mlp_rows_per_expert(K, dtype, E):
  """Leading rows equal the full computation bit for bit; the other rows are not written."""
  rng = np.random.default_rng(3)
  R, D, M = 300, 64, 128
  x = to_dev(O.cast(rng.standard_normal((E, R, D)).astype(np.float32), dtype), dtype)
  w0 = to_dev(O.cast(rng.standard_normal((E, D, M)).astype(np.float32) / 8, dtype), dtype)
  w1 = to_dev(O.cast(rng.standard_normal((E, M, D)).astype(np.float32) / 11, dtype), dtype)
  b0 = to_dev(O.cast(rng.standard_normal((E, M)).astype(np.float32) * 0.1, dtype), dtype)
  b1 = to_dev(O.cast(rng.standard_normal((E, D)).astype(np.float32) * 0.1, dtype), dtype)
  full = K.expert_mlp(x, w0, b0, w1, b1)
  rows = np.asarray(([300, 0, 1, 129, 256] * 4)[:E], np.int32)
  out = torch.full_like(full, 7.0)
  x_bad = x.clone()
  for e, n in enumerate(rows):
    x_bad[e, n:] = float("nan")                      # rows past the count must not matter
  K.expert_mlp(x_bad, w0, b0, w1, b1, out=out, rows_per_expert=to_dev(rows))
  for e, n in enumerate(rows):
    np.testing.assert_array_equal(to_np(out[e, :n]), to_np(full[e, :n]))
    assert (to_np(out[e, n:]) == 7.0).all()


def test_expert_mlp_planned_launch_random_fill(K):
  """bf16 expert products over packed rows with a die-balanced launch plan: random row
  counts (empty, one row, tile boundaries, full), expert counts below and above the
  number of dies, row capacities below and above a tile."""
  rng = np.random.default_rng(11)
  dtype = O.BF16
  for E, R, D, M in [(1, 700, 64, 96), (3, 130, 96, 64), (8, 520, 64, 128), (9, 257, 128, 64),
                     (17, 300, 64, 64), (40, 100, 64, 96), (64, 33, 96, 64),
                     (5, 520, 64, 224), (12, 700, 520, 192)]:   # tile-walking second product
    x = to_dev(O.cast(rng.standard_normal((E, R, D)).astype(np.float32), dtype), dtype)
    w0 = to_dev(O.cast(rng.standard_normal((E, D, M)).astype(np.float32) / 8, dtype), dtype)
    w1 = to_dev(O.cast(rng.standard_normal((E, M, D)).astype(np.float32) / 11, dtype), dtype)
    b0 = to_dev(O.cast(rng.standard_normal((E, M)).astype(np.float32) * 0.1, dtype), dtype)
    b1 = to_dev(O.cast(rng.standard_normal((E, D)).astype(np.float32) * 0.1, dtype), dtype)
    full = K.expert_mlp(x, w0, b0, w1, b1)
    for trial in range(3):
      special = np.asarray([0, 1, 127, 128, 129, 255, 256, 257, R], np.int64)
      rows = np.where(rng.random(E) < 0.5, rng.integers(0, R + 1, E), rng.choice(special, E))
      rows = np.minimum(rows, R).astype(np.int32)
      out = torch.full_like(full, 7.0)
      K.expert_mlp(x, w0, b0, w1, b1, out=out, rows_per_expert=to_dev(rows))
      for e, n in enumerate(rows):
        np.testing.assert_array_equal(to_np(out[e, :n]), to_np(full[e, :n]),
                                      err_msg=f"E={E} R={R} rows={rows.tolist()} expert {e}")
        assert (to_np(out[e, n:]) == 7.0).all(), f"E={E} R={R} rows={rows.tolist()} expert {e}"


@pytest.mark.parametrize("E,R,D,M", [(64, 384, 1024, 128), (32, 1152, 1024, 256), (90, 384, 520, 160)])
def test_expert_mlp_wide_second_product(K, E, R, D, M):
  """Shapes whose second product takes the wide kernel (384 x 256 tiles, eight waves; it runs
  where the tile-walking 256 x 256 kernel does not apply, and VMOE_SECOND_PRODUCT=wide asks
  for it wherever it applies itself): all rows against the oracle, then packed rows with a
  launch plan (row counts around the tile height, empty experts) bit for bit against the
  dense launch."""
  os.environ["VMOE_SECOND_PRODUCT"] = "wide"
  try:
    _wide_second_product(K, E, R, D, M)
  finally:
    del os.environ["VMOE_SECOND_PRODUCT"]


def _wide_second_product(K, E, R, D, M):
  rng = np.random.default_rng(E + R)
  dtype = O.BF16
  x = O.cast(rng.standard_normal((E, R, D)).astype(np.float32), dtype)
  w0 = O.cast(rng.standard_normal((E, D, M)).astype(np.float32) / np.sqrt(D), dtype)
  w1 = O.cast(rng.standard_normal((E, M, D)).astype(np.float32) / np.sqrt(M), dtype)
  b0 = O.cast(rng.standard_normal((E, M)).astype(np.float32) * 0.1, dtype)
  b1 = O.cast(rng.standard_normal((E, D)).astype(np.float32) * 0.1, dtype)
  dx, dw0, db0, dw1, db1 = (to_dev(a, dtype) for a in (x, w0, b0, w1, b1))
  full = K.expert_mlp(dx, dw0, db0, dw1, db1)
  pick = np.unique(np.concatenate([[0, E - 1], rng.integers(0, E, 4)]))
  want = O.mlp_block(x[pick], w0[pick], b0[pick], w1[pick], b1[pick], dtype)
  assert_close(to_np(full)[pick], want, 2e-2, "wide second product")
  nobias = K.expert_mlp(dx, dw0, db0, dw1, None)
  want = O.mlp_block(x[pick[:2]], w0[pick[:2]], b0[pick[:2]], w1[pick[:2]], None, dtype)
  assert_close(to_np(nobias)[pick[:2]], want, 2e-2, "wide second product, no bias")
  special = np.asarray([0, 1, 95, 96, 97, 383, 384, 385, R - 1, R], np.int64)
  for trial in range(3):
    rows = np.where(rng.random(E) < 0.5, rng.integers(0, R + 1, E), rng.choice(special, E))
    rows = np.minimum(rows, R).astype(np.int32)
    out = torch.full_like(full, 7.0)
    K.expert_mlp(dx, dw0, db0, dw1, db1, out=out, rows_per_expert=to_dev(rows))
    got, ref = to_np(out), to_np(full)
    for e, n in enumerate(rows):
      np.testing.assert_array_equal(got[e, :n], ref[e, :n], err_msg=f"rows={rows.tolist()} expert {e}")
      assert (got[e, n:] == 7.0).all(), f"rows={rows.tolist()} expert {e}"


def _sparse_signs(rng, shape, nonzeros, axis):
  """Entries in {-1, 0, 1} with exactly `nonzeros` non-zero entries along `axis`."""
  shape = list(shape)
  n = shape.pop(axis)
  flat = np.zeros((int(np.prod(shape)), n), np.float32)
  for row in flat:
    pos = rng.choice(n, size=min(nonzeros, n), replace=False)
    row[pos] = rng.choice(np.asarray([-1.0, 1.0], np.float32), size=pos.size)
  return np.ascontiguousarray(np.moveaxis(flat.reshape(*shape, n), -1, axis))


@pytest.mark.parametrize("E,R,D,M", [
    (2, 96, 64, 256),         # one-tile-per-workgroup first product (2 k tiles), tile-walking second product
    (3, 200, 72, 136),        # widths outside the fast path: register-staged kernel, k edge
    (64, 384, 1024, 128),     # wide second product
    (2, 300, 256, 2048),      # long k loops on both kernels' steady state
])
def test_matrix_core_results_are_read_whole(K, E, R, D, M):
  """Every accumulator register of the matrix-core loops must be complete when the
  epilogue reads it: a v_mfma_f32_32x32x16_bf16 result read too early comes back with
  its last register stale, which showed as wrong rows 27 and 31 of every 32-row tile (the
  kernels put a fixed gap of wait states between the loop and the first read).  Operands
  are small integers chosen so that every product, sum and rounding step of the MLP is
  exact in bfloat16 and the GELU is the identity (pre-activations of 8 and more): the
  result must equal the float64 answer bit for bit, in particular rows 27 and 31."""
  rng = np.random.default_rng(D + M)
  x = rng.integers(-1, 2, (E, R, D)).astype(np.float32)
  w0 = _sparse_signs(rng, (E, D, M), 8, axis=1)             # |x @ w0| <= 8
  b0 = np.full((E, M), 16.0, np.float32)                    # hidden = 16 + (x @ w0) in [8, 24]
  w1 = _sparse_signs(rng, (E, M, D), 4, axis=1)             # |hidden @ w1| <= 96
  b1 = rng.integers(-3, 4, (E, D)).astype(np.float32)
  hidden = np.einsum("erd,edm->erm", x.astype(np.float64), w0.astype(np.float64)) + 16.0
  assert hidden.min() >= 8 and hidden.max() <= 24
  want = np.einsum("erm,emd->erd", hidden, w1.astype(np.float64)) + b1[:, None, :]
  assert np.abs(want).max() <= 128
  dtype = O.BF16
  got = to_np(K.expert_mlp(*(to_dev(a, dtype) for a in (x, w0, b0, w1, b1)))).astype(np.float64)
  rows = np.arange(R)
  late = (rows % 32 == 27) | (rows % 32 == 31)
  np.testing.assert_array_equal(got[:, late], want[:, late], err_msg="rows 27 / 31 of a 32-row tile")
  np.testing.assert_array_equal(got, want)


def test_gating_logits_are_read_whole(K):
  """The gating kernel's matrix-core loop under the same check: integer operands, exact
  float32 logits, all rows (27 and 31 of each 32-item tile first)."""
  rng = np.random.default_rng(3)
  G, S, D, E = 3, 100, 256, 32
  x = rng.integers(-2, 3, (G, S, D)).astype(np.float32)
  w = rng.integers(-1, 2, (D, E)).astype(np.float32)
  want = (x.astype(np.float64) @ w.astype(np.float64))          # |sum| <= 512: exact in float32
  want_bf = np.asarray(O.cast(want.astype(np.float32), O.BF16), np.float64)   # the logits are rounded to the dtype
  for dtype, ref in ((O.F32, want), (O.BF16, want_bf)):
    _, _, _, logits = K.gate_topk(to_dev(x, dtype), to_dev(w, dtype), 2, return_logits=True)
    got = to_np(logits).astype(np.float64).reshape(G * S, E)
    rows = np.arange(G * S)
    late = (rows % 32 == 27) | (rows % 32 == 31)
    np.testing.assert_array_equal(got[late], ref.reshape(G * S, E)[late], err_msg=f"{dtype}: rows 27 / 31")
    np.testing.assert_array_equal(got, ref.reshape(G * S, E), err_msg=dtype)


def test_resident_delivery_probe(K):
  """The load-only kernel over shared, L2-resident tiles runs to its end for both request shapes
  and reports the bytes it moved; bad arguments come back as error codes."""
  from vmoe_amd import _hip as H
  buf = torch.zeros(3 * 512 * 1024 + 100, dtype=torch.uint8, device=dev())      # three tiles and a bit
  for seg in (128, 64):
    assert K.resident_delivery_probe(buf, 1024, 8, 2, seg) == 256 * 2 * 8 * 65536
  torch.cuda.synchronize()
  with pytest.raises(H.VmoeError, match="invalid sizes"):
    K.resident_delivery_probe(buf, 1024, 9, 2, 128)          # 9 k tiles of 128 bytes > row
  with pytest.raises(H.VmoeError, match="invalid sizes"):
    K.resident_delivery_probe(buf, 1024, 8, 2, 32)
  with pytest.raises(H.VmoeError, match="invalid sizes"):
    K.resident_delivery_probe(buf[:1000], 1024, 8, 2, 128)   # not one whole tile


def test_operand_delivery_probe(K):
  """The load-only measurement kernel reports the operand bytes of the 256 x 256 tiling
  and refuses what the tiling refuses."""
  from vmoe_amd import _hip as H
  a = torch.randn((3, 700, 256), device=dev()).to(torch.bfloat16)
  bt = torch.randn((3, 520, 256), device=dev()).to(torch.bfloat16)
  moved = K.operand_delivery_probe(a, bt)
  torch.cuda.synchronize()
  assert moved == 3 * 3 * 3 * 512 * 256 * 2          # 3 batches x (3 x 3) tiles x 512 rows x K x 2 bytes
  assert K.operand_delivery_probe(a[0], bt[0]) == 3 * 3 * 512 * 256 * 2
  assert K.operand_delivery_probe(a, bt, k_tile=64) == moved     # same tiles, 128-byte row segments
  torch.cuda.synchronize()
  with pytest.raises(H.VmoeError):                     # K not a multiple of 64
    K.operand_delivery_probe(a[:, :, :96].contiguous(), bt[:, :, :96].contiguous(), k_tile=64)
  with pytest.raises(H.VmoeError):                     # K not a multiple of 32
    K.operand_delivery_probe(a[:, :, :40].contiguous(), bt[:, :, :40].contiguous())
  with pytest.raises(ValueError):
    K.operand_delivery_probe(a.float(), bt.float())


@pytest.mark.parametrize("G,S,E,k,C,D,M", [
    (4, 1568, 32, 2, 100, 256, 512),     # headline routing shapes, a narrow MLP
    (2, 1568, 8, 2, 412, 128, 256),      # few experts, many rows each
    (3, 300, 5, 3, 200, 128, 192),       # expert count that does not divide 256
])
def test_expert_mlp_with_compaction_in_the_planning_launch(K, monkeypatch, G, S, E, k, C, D, M):
  """expert_mlp(compact=...) (vmoe_compact_rows_planned + vmoe_expert_mlp_planned) against
  vmoe_compact_rows followed by vmoe_expert_mlp: the integer maps bit for bit, the output
  rows of kept assignments bit for bit as well (the same kernels run on the same plan)."""
  rng = np.random.default_rng(G * 100 + E)
  gates = O.softmax(rng.standard_normal((G, S, E)).astype(np.float32) * 2)
  val, idx = K.topk(to_dev(gates), k)
  _, token_slot, _, fill = K.route_assign(val, idx, E, C, True)
  items = to_dev(O.cast(rng.standard_normal((G * S, D)), O.BF16), O.BF16)
  w0 = to_dev(O.cast(rng.standard_normal((E, D, M)) / np.sqrt(D), O.BF16), O.BF16)
  w1 = to_dev(O.cast(rng.standard_normal((E, M, D)) / np.sqrt(M), O.BF16), O.BF16)
  b0 = to_dev(O.cast(rng.standard_normal((E, M)) * 0.1, O.BF16), O.BF16)
  b1 = to_dev(O.cast(rng.standard_normal((E, D)) * 0.1, O.BF16), O.BF16)
  w0t, w1t = K.pack_expert_weights(w0), K.pack_expert_weights(w1)
  token_row, rows, row_token = K.compact_rows(fill, token_slot, C)
  want = K.expert_mlp(items, None, b0, None, b1, w0t=w0t, w1t=w1t, rows_per_expert=rows, x_rows=row_token)
  for separate in (False, True):
    if separate:
      monkeypatch.setenv("VMOE_PLAN_SEPARATE_LAUNCH", "1")
    else:
      monkeypatch.delenv("VMOE_PLAN_SEPARATE_LAUNCH", raising=False)
    for _ in range(2):
      got, maps = K.expert_mlp(items, None, b0, None, b1, w0t=w0t, w1t=w1t,
                               compact=(fill, token_slot, C))
      np.testing.assert_array_equal(to_np(maps[0]), to_np(token_row))
      np.testing.assert_array_equal(to_np(maps[1]), to_np(rows))
      r = to_np(rows)
      g_np, w_np = to_np(got), to_np(want)
      rt_g, rt_w = to_np(maps[2]), to_np(row_token)
      for e in range(E):
        np.testing.assert_array_equal(rt_g[e, :r[e]], rt_w[e, :r[e]])
        np.testing.assert_array_equal(g_np[e, :r[e]], w_np[e, :r[e]])
  monkeypatch.delenv("VMOE_PLAN_SEPARATE_LAUNCH", raising=False)


def test_expert_mlp_hidden_layer_beyond_4_gib(K):
  """A hidden layer of 4.3 GiB: the second product cannot address it with 32-bit byte
  offsets from its start, which the tile-walking kernel needs, so the one-tile-per-
  workgroup kernel (offsets per expert) must take over.  Sampled rows of every expert
  against a float32 restatement on the device."""
  rng = np.random.default_rng(31)
  E, R, D, M = 8, 70000, 64, 4096
  assert E * R * M * 2 >= 1 << 32
  bf = torch.bfloat16
  gen = torch.Generator(device=dev())
  gen.manual_seed(5)
  x = torch.randn((E, R, D), generator=gen, device=dev()).to(bf)
  w0 = (torch.randn((E, D, M), generator=gen, device=dev()) / D ** 0.5).to(bf)
  w1 = (torch.randn((E, M, D), generator=gen, device=dev()) / M ** 0.5).to(bf)
  b0 = (torch.randn((E, M), generator=gen, device=dev()) * 0.1).to(bf)
  b1 = (torch.randn((E, D), generator=gen, device=dev()) * 0.1).to(bf)
  out = K.expert_mlp(x, w0, b0, w1, b1)
  pick = torch.from_numpy(np.unique(np.concatenate(
      [[0, 1, 255, 256, R - 257, R - 2, R - 1], rng.integers(0, R, 50)]))).to(dev())
  for e in range(E):
    h = ((x[e, pick].float() @ w0[e].float()).to(bf).float() + b0[e].float()).to(bf)
    h = torch.nn.functional.gelu(h.float(), approximate="tanh").to(bf)
    y = ((h.float() @ w1[e].float()).to(bf).float() + b1[e].float()).to(bf)
    np.testing.assert_allclose(to_np(out[e, pick]), to_np(y), rtol=2e-2, atol=2e-2, err_msg=f"expert {e}")
  del out, x
  torch.cuda.empty_cache()


@pytest.mark.parametrize("with_bias", [True, False])
def test_expert_mlp_second_product_walks_several_tiles(K, with_bias):
  """The second product's workgroups walk a list of tiles and fetch a tile's first
  operands while they finish the tile before: enough tiles (480 of 256 x 256, 60 per die)
  that most workgroups compute two, dense and over packed rows with a launch plan, the
  last column tile 8 wide.  Checked against a float32 restatement with the bfloat16
  rounding points of flax's Dense (accumulator, + bias) on the device, tolerance one
  bfloat16 step; packed rows against the dense result bit for bit."""
  rng = np.random.default_rng(23)
  E, R, D, M = 16, 2321, 520, 256
  bf = torch.bfloat16
  x = to_dev(O.cast(rng.standard_normal((E, R, D)).astype(np.float32), O.BF16), O.BF16)
  w0 = to_dev(O.cast(rng.standard_normal((E, D, M)).astype(np.float32) / np.sqrt(D), O.BF16), O.BF16)
  w1 = to_dev(O.cast(rng.standard_normal((E, M, D)).astype(np.float32) / np.sqrt(M), O.BF16), O.BF16)
  b0 = to_dev(O.cast(rng.standard_normal((E, M)).astype(np.float32) * 0.1, O.BF16), O.BF16) if with_bias else None
  b1 = to_dev(O.cast(rng.standard_normal((E, D)).astype(np.float32) * 0.1, O.BF16), O.BF16) if with_bias else None
  full = K.expert_mlp(x, w0, b0, w1, b1)
  for e in range(E):                       # one expert at a time: plain 2-D products
    h = (x[e].float() @ w0[e].float()).to(bf)
    if with_bias:
      h = (h.float() + b0[e].float()).to(bf)
    h = torch.nn.functional.gelu(h.float(), approximate="tanh").to(bf)
    y = (h.float() @ w1[e].float()).to(bf)
    if with_bias:
      y = (y.float() + b1[e].float()).to(bf)
    np.testing.assert_allclose(to_np(full[e]), to_np(y), rtol=2e-2, atol=2e-2, err_msg=f"expert {e}")
  rows = rng.integers(0, R + 1, E).astype(np.int32)
  rows[:4] = [R, 0, 257, 1]
  out = torch.full_like(full, 7.0)
  K.expert_mlp(x, w0, b0, w1, b1, out=out, rows_per_expert=to_dev(rows))
  for e, n in enumerate(rows):
    np.testing.assert_array_equal(to_np(out[e, :n]), to_np(full[e, :n]), err_msg=f"expert {e}")
    assert (to_np(out[e, n:]) == 7.0).all(), f"expert {e}"


@pytest.mark.parametrize("which", ["eight", "narrow"])
@pytest.mark.parametrize("E,R,D,M", [
    (64, 1100, 768, 256),     # 960 / 1280 tiles: the kernels' own range; four k tiles (the shortest k they take)
    (40, 1300, 1024, 512),    # four column tiles of 256, five and a third of 192
    (3, 500, 520, 1024),      # forced: a column tile that ends inside the tile, few tiles per die
    (5, 257, 264, 320),       # forced: one row past a tile, k of five tiles
])
def test_expert_mlp_second_product_on_eight_waves(K, monkeypatch, E, R, D, M, which):
  """The eight-wave forms of the second product (two waves per SIMD, output leaving through lane
  exchanges instead of LDS; "eight": 256 x 256 tiles and 32 x 32 x 16 MFMAs, "narrow": 256 x 192
  tiles and 16 x 16 x 32 MFMAs) against the four-wave tile-walking kernel with whole tiles:
  all add the same products in the same order of k, so the outputs must agree bit for bit;
  dense and over packed rows with a launch plan (rows past a count are not written)."""
  rng = np.random.default_rng(E * 100 + M)
  args = [to_dev(O.cast(a, O.BF16), O.BF16) for a in (
      rng.standard_normal((E, R, D)).astype(np.float32),
      rng.standard_normal((E, D, M)).astype(np.float32) / np.sqrt(D),
      rng.standard_normal((E, M)).astype(np.float32) * 0.1,
      rng.standard_normal((E, M, D)).astype(np.float32) / np.sqrt(M),
      rng.standard_normal((E, D)).astype(np.float32) * 0.1)]
  rows = rng.integers(0, R + 1, E).astype(np.int32)
  rows[:3] = [R, 0, 257][:min(3, E)]
  outs = {}
  for kernel in (which, "shared"):
    monkeypatch.setenv("VMOE_SECOND_PRODUCT", kernel)
    monkeypatch.setenv("VMOE_WHOLE_TILES", "1")
    dense = K.expert_mlp(*args)
    ragged = torch.full_like(dense, 7.0)
    K.expert_mlp(*args, out=ragged, rows_per_expert=to_dev(rows))
    outs[kernel] = (to_np(dense), to_np(ragged))
    assert K.expert_mlp_status() == (0, 0)
  monkeypatch.delenv("VMOE_SECOND_PRODUCT")
  monkeypatch.delenv("VMOE_WHOLE_TILES")
  np.testing.assert_array_equal(outs[which][0], outs["shared"][0])
  for e, n in enumerate(rows):
    np.testing.assert_array_equal(outs[which][1][e, :n], outs["shared"][1][e, :n], err_msg=f"expert {e}")
    np.testing.assert_array_equal(outs[which][1][e, :n], outs[which][0][e, :n], err_msg=f"expert {e}")
    assert (outs[which][1][e, n:] == 7.0).all(), f"expert {e}"
  # and against a float32 restatement of one expert
  e = E - 1
  x, w0, b0, w1, b1 = (a[e].float() for a in args)
  bf = torch.bfloat16
  h = ((x @ w0).to(bf).float() + b0).to(bf)
  h = torch.nn.functional.gelu(h.float(), approximate="tanh").to(bf)
  want = ((h.float() @ w1).to(bf).float() + b1).to(bf)
  np.testing.assert_allclose(outs[which][0][e], to_np(want), rtol=2e-2, atol=2e-2)


SHARED_ROUND_CASES = [
    (16, 2321, 520, 1024),    # 60 tiles per die: one round, then 28 tiles shared by 32 workgroups (pieces of 12-16 k tiles)
    (32, 768, 768, 768),      # 36 per die: 4 tiles in pieces of 4 k tiles, chains of three
    (12, 2048, 1024, 512),    # 48 per die: 16 tiles, each halved
    (40, 1300, 768, 1280),    # 90 per die: two rounds, then 26 tiles
    (3, 500, 768, 1024),      # 2-3 tiles per die: no whole round, every tile in many pieces
]


@pytest.mark.parametrize("E,R,D,M", SHARED_ROUND_CASES)
def test_expert_mlp_second_product_shares_partial_round(K, monkeypatch, E, R, D, M):
  """The tile-walking second product cuts the tiles of a die's last, partial round along k
  among the die's workgroups; the float32 sums travel from piece to piece through memory.
  Against the same experts computed one at a time and against a float32 restatement: a cut
  changes the order of one float32 addition per output, so an output may differ from the
  uncut computation by one bfloat16 step (few do); dense and over packed rows with a launch
  plan (random row counts move the cuts); rows past a count are not written."""
  monkeypatch.setenv("VMOE_SECOND_PRODUCT", "shared")      # whatever the launch geometry would choose
  rng = np.random.default_rng(E * 1000 + R)
  bf = torch.bfloat16
  x = to_dev(O.cast(rng.standard_normal((E, R, D)).astype(np.float32), O.BF16), O.BF16)
  w0 = to_dev(O.cast(rng.standard_normal((E, D, M)).astype(np.float32) / np.sqrt(D), O.BF16), O.BF16)
  w1 = to_dev(O.cast(rng.standard_normal((E, M, D)).astype(np.float32) / np.sqrt(M), O.BF16), O.BF16)
  b0 = to_dev(O.cast(rng.standard_normal((E, M)).astype(np.float32) * 0.1, O.BF16), O.BF16)
  b1 = to_dev(O.cast(rng.standard_normal((E, D)).astype(np.float32) * 0.1, O.BF16), O.BF16)
  full = K.expert_mlp(x, w0, b0, w1, b1)
  again = K.expert_mlp(x, w0, b0, w1, b1)
  assert torch.equal(full, again), "two runs of the same launch differ"
  ref = []
  for e in range(E):                       # one expert at a time: plain 2-D products
    h = ((x[e].float() @ w0[e].float()).to(bf).float() + b0[e].float()).to(bf)
    h = torch.nn.functional.gelu(h.float(), approximate="tanh").to(bf)
    ref.append(((h.float() @ w1[e].float()).to(bf).float() + b1[e].float()).to(bf))
  ref = to_np(torch.stack(ref)).astype(np.float64)

  def check(got, n_rows, what):
    for e, n in enumerate(n_rows):
      np.testing.assert_allclose(got[e, :n], ref[e, :n], rtol=2e-2, atol=2e-2, err_msg=f"{what} expert {e}")

  got_full = to_np(full).astype(np.float64)
  bias1 = to_np(b1).astype(np.float64)
  check(got_full, [R] * E, "dense")
  for trial in range(4):
    rows = rng.integers(0, R + 1, E).astype(np.int32)
    rows[:3] = [R, 0, 257]
    out = torch.full_like(full, 7.0)
    K.expert_mlp(x, w0, b0, w1, b1, out=out, rows_per_expert=to_dev(rows))
    got = to_np(out).astype(np.float64)
    check(got, rows, f"rows={rows.tolist()}")
    differ = 0
    for e, n in enumerate(rows):
      assert (got[e, n:] == 7.0).all(), f"rows={rows.tolist()} expert {e}"
      d = np.abs(got[e, :n] - got_full[e, :n])
      # one step of the rounded accumulator (output minus bias), carried through the rounded sum with the bias
      step = 2.0 ** -6 * (np.abs(got_full[e, :n]) + np.abs(bias1[e])[None, :])
      assert (d <= step + 1e-30).all(), "more than one bfloat16 step from the dense launch"
      differ += int((d > 0).sum())
    assert differ <= 0.02 * max(1, int(rows.sum())) * D, f"{differ} outputs differ from the dense launch"
  assert K.expert_mlp_status() == (0, 0), "a piece gave up its wait, or a launch found no plan"


@pytest.mark.parametrize("E,R,D,M", [(12, 2048, 1024, 512), (3, 500, 768, 1024)])
def test_shared_partial_round_is_exact_on_exact_operands(K, monkeypatch, E, R, D, M):
  """The same cuts on operands whose every product, sum and rounding step is exact (small
  integers, GELU the identity): whatever the order of the additions, the result must
  equal the float64 answer bit for bit, dense and over packed rows."""
  monkeypatch.setenv("VMOE_SECOND_PRODUCT", "shared")      # whatever the launch geometry would choose
  rng = np.random.default_rng(D + M)
  x = rng.integers(-1, 2, (E, R, D)).astype(np.float32)
  w0 = _sparse_signs(rng, (E, D, M), 8, axis=1)
  b0 = np.full((E, M), 16.0, np.float32)
  w1 = _sparse_signs(rng, (E, M, D), 4, axis=1)
  b1 = rng.integers(-3, 4, (E, D)).astype(np.float32)
  hidden = np.einsum("erd,edm->erm", x.astype(np.float64), w0.astype(np.float64)) + 16.0
  want = np.einsum("erm,emd->erd", hidden, w1.astype(np.float64)) + b1[:, None, :]
  assert hidden.min() >= 8 and hidden.max() <= 24 and np.abs(want).max() <= 128
  dev_args = [to_dev(a, O.BF16) for a in (x, w0, b0, w1, b1)]
  got = to_np(K.expert_mlp(*dev_args)).astype(np.float64)
  np.testing.assert_array_equal(got, want)
  rows = rng.integers(0, R + 1, E).astype(np.int32)
  rows[0] = R
  out = torch.full((E, R, D), 7.0, dtype=torch.bfloat16, device=dev())
  K.expert_mlp(*dev_args, out=out, rows_per_expert=to_dev(rows))
  got = to_np(out).astype(np.float64)
  for e, n in enumerate(rows):
    np.testing.assert_array_equal(got[e, :n], want[e, :n], err_msg=f"expert {e}")
    assert (got[e, n:] == 7.0).all()
  assert K.expert_mlp_status() == (0, 0), "a piece gave up its wait, or a launch found no plan"


def test_shared_round_wait_that_gives_up_is_loud(K, monkeypatch):
  """The bounded wait of the shared round, forced from the host: with
  VMOE_STREAMK_TEST_GIVE_UP the pieces wait (for a handful of polls) for a deposit count that
  is never reached.  Every kernel still runs to its end; the pieces that gave up are counted
  in the status words and their outputs are NaN, not sums that were never delivered.  The
  count stays when later calls on the same workspace go well."""
  monkeypatch.setenv("VMOE_SECOND_PRODUCT", "shared")      # whatever the launch geometry would choose
  E, R, D, M = 3, 500, 768, 1024           # 2-3 tiles per die: every tile is shared
  rng = np.random.default_rng(5)
  args = [to_dev(O.cast(a, O.BF16), O.BF16) for a in (
      rng.standard_normal((E, R, D)).astype(np.float32),
      rng.standard_normal((E, D, M)).astype(np.float32) / np.sqrt(D),
      rng.standard_normal((E, M)).astype(np.float32) * 0.1,
      rng.standard_normal((E, M, D)).astype(np.float32) / np.sqrt(M),
      rng.standard_normal((E, D)).astype(np.float32) * 0.1)]
  ws = torch.zeros(K.expert_mlp_workspace_bytes(E, R, D, M, torch.bfloat16, prepacked=False),
                   dtype=torch.uint8, device=dev())
  good = K.expert_mlp(*args, workspace=ws)
  torch.cuda.synchronize()
  assert K.expert_mlp_status() == (0, 0)
  assert not torch.isnan(good).any()
  monkeypatch.setenv("VMOE_STREAMK_TEST_GIVE_UP", "4")
  bad = K.expert_mlp(*args, workspace=ws)
  torch.cuda.synchronize()
  monkeypatch.delenv("VMOE_STREAMK_TEST_GIVE_UP")
  abandoned, mismatches = K.expert_mlp_status()
  assert abandoned >= 1 and mismatches == 0
  nan_rows = torch.isnan(bad).any(-1)
  assert nan_rows.any(), "a piece gave up but no output row says so"
  ok = ~nan_rows
  assert torch.equal(bad[ok], good[ok]), "rows that are not NaN must be the product"
  again = K.expert_mlp(*args, workspace=ws)
  torch.cuda.synchronize()
  assert torch.equal(again, good)
  assert K.expert_mlp_status() == (abandoned, 0), "the status words only grow"


def test_expert_mlp_planned_is_repeatable_and_checks_its_plan(K):
  """vmoe_expert_mlp_planned twice after one vmoe_compact_rows_planned (unchanged routing: a
  serving loop, a graph of the experts alone) gives the same output both times -- each call
  resets the exchange counters of its shared round -- and a call on a workspace whose plans
  were never written runs nothing and says so in the status words."""
  from vmoe_amd import _hip as H
  G, S, E, k, C, D, M = 4, 1568, 32, 2, 100, 256, 512     # 64 tiles of the second product: shared pieces on every die
  rng = np.random.default_rng(23)
  gates = O.softmax(rng.standard_normal((G, S, E)).astype(np.float32) * 2)
  val, idx = K.topk(to_dev(gates), k)
  _, token_slot, _, fill = K.route_assign(val, idx, E, C, True)
  items = to_dev(O.cast(rng.standard_normal((G * S, D)), O.BF16), O.BF16)
  w0 = to_dev(O.cast(rng.standard_normal((E, D, M)) / np.sqrt(D), O.BF16), O.BF16)
  w1 = to_dev(O.cast(rng.standard_normal((E, M, D)) / np.sqrt(M), O.BF16), O.BF16)
  b0 = to_dev(O.cast(rng.standard_normal((E, M)) * 0.1, O.BF16), O.BF16)
  b1 = to_dev(O.cast(rng.standard_normal((E, D)) * 0.1, O.BF16), O.BF16)
  w0t, w1t = K.pack_expert_weights(w0), K.pack_expert_weights(w1)
  first, maps = K.expert_mlp(items, None, b0, None, b1, w0t=w0t, w1t=w1t, compact=(fill, token_slot, C))
  first = first.clone()
  rows = to_np(maps[1])
  for _ in range(2):
    out = K.expert_mlp_replay_planned()
    first_np, out_np = to_np(first), to_np(out)
    for e in range(E):
      np.testing.assert_array_equal(out_np[e, :rows[e]], first_np[e, :rows[e]], err_msg=f"expert {e}")
  assert K.expert_mlp_status() == (0, 0)
  # a workspace that was never planned: every product launch leaves at once
  R = G * C
  ws = torch.randint(0, 255, (K.expert_mlp_workspace_bytes(E, R, D, M, torch.bfloat16, prepacked=True) + (1 << 20),),
                     dtype=torch.uint8, device=dev())
  out = torch.full((E, R, D), 7.0, dtype=torch.bfloat16, device=dev())
  p = H.ExpertMlpParams(H.ptr(items), None, H.ptr(b0), None, H.ptr(b1), H.ptr(w0t), H.ptr(w1t), H.ptr(out),
                        H.ptr(ws), ws.numel(), E, R, D, M, H.BF16, H.GELU_TANH, H.ptr(maps[1]),
                        H.ptr(maps[2]), G * S)
  need = H.lib().vmoe_expert_mlp_workspace_bytes(H.ctypes.byref(p))
  assert need <= ws.numel()
  H.call("vmoe_expert_mlp_planned", p)
  torch.cuda.synchronize()
  addr = H.ctypes.c_void_p()
  H.check(H.lib().vmoe_expert_mlp_status(H.ctypes.byref(p), H.ctypes.byref(addr)), "vmoe_expert_mlp_status")
  words = ws[addr.value - ws.data_ptr():][:8].view(torch.int32).cpu()
  assert int(words[H.MLP_STATUS_PLAN_MISMATCHES]) == 2, "both products must report the missing plan"
  assert int(words[H.MLP_STATUS_ABANDONED_WAITS]) == 0
  assert (to_np(out) == 7.0).all(), "a launch without a valid plan must not write"


@pytest.mark.parametrize("G,S,D,N", [(6, 196, 768, 128), (3, 250, 768, 128), (2, 37, 384, 40),
                                     (4, 100, 512, 64), (2, 256, 256, 8), (1, 1, 768, 8),
                                     (2, 300, 256, 104), (2, 33, 1024, 128), (2, 64, 768, 20)])
def test_soft_route_with_stats(K, G, S, D, N):
  """vmoe_soft_route_stats: the weights are those of vmoe_soft_route bit for bit, and the
  scalars are the means of vmoe/projects/soft_moe/router.py:119-125 of exactly those stored
  weights, whether the routing launch takes the partial sums itself (bfloat16, up to 256 items,
  widths up to 768) or the separate launches run (the last three shapes)."""
  rng = np.random.default_rng(G * S + N)
  x = to_dev(O.cast(rng.standard_normal((G, S, D)), O.BF16), O.BF16)
  mu = to_dev(O.cast(rng.standard_normal((D, N)) / np.sqrt(D), O.BF16), O.BF16)
  dw0, cw0 = K.soft_route(x, mu, 1.2)
  dw, cw, scalars = K.soft_route(x, mu, 1.2, with_stats=True)
  np.testing.assert_array_equal(to_np(dw), to_np(dw0))
  np.testing.assert_array_equal(to_np(cw), to_np(cw0))
  d, c = to_np(dw).astype(np.float64), to_np(cw).astype(np.float64)
  want = [c.min(axis=2).mean(), c.max(axis=2).mean(), d.min(axis=1).mean(), d.max(axis=1).mean()]
  got = [float(v) for v in scalars]
  np.testing.assert_allclose(got[:4], want, rtol=3e-6)
  assert got[4] == 0.0
  np.testing.assert_allclose(got[:4], [float(v) for v in K.soft_router_stats(cw, dw)][:4], rtol=3e-6)


@pytest.mark.parametrize("G,S,N,dtype", [(3, 50, 16, O.F32), (4, 196, 128, O.BF16), (2, 7, 300, O.BF16), (3, 196, 128, O.F32),
                          (2, 9, 96, O.BF16), (5, 33, 8, O.BF16), (2, 300, 512, O.BF16)])
def test_soft_router_stats(K, G, S, N, dtype):
  """The four means of vmoe/projects/soft_moe/router.py:119-125 in one kernel."""
  rng = np.random.default_rng(G + S + N)
  cw = O.cast(O.softmax(rng.standard_normal((G, S, N)).astype(np.float32), axis=2), dtype)
  dw = O.cast(O.softmax(rng.standard_normal((G, S, N)).astype(np.float32), axis=1), dtype)
  got = [float(v) for v in K.soft_router_stats(to_dev(cw, dtype), to_dev(dw, dtype))]
  want = [cw.min(axis=2).mean(), cw.max(axis=2).mean(), dw.min(axis=1).mean(), dw.max(axis=1).mean()]
  np.testing.assert_allclose(got[:4], want, rtol=2e-6)
  assert got[4] == 0.0   # auxiliary_loss
