"""Pins the CPU oracle against the golden vectors held by the reference's own
tests (tests/golden/reference_goldens.json) and against independent statements
(brute force, closed forms, library routines)."""
import math

import einops
import numpy as np
import pytest
import scipy.spatial.distance

from oracle import moe_oracle as O
from oracle import route_c


def test_compute_capacity(goldens):
  g = goldens["compute_capacity"]
  with pytest.raises(ValueError, match="The values .* lead to capacity .*, but it must be greater "
                     "than or equal to 1"):
    O.compute_capacity(**g["raises"])
  for c in g["cases"]:
    c = dict(c)
    exp = c.pop("expected")
    assert O.compute_capacity(**c) == exp
  with pytest.raises(ValueError, match="Unsupported"):
    O.compute_capacity(8, 2, 1.0, "floor")
  # Banker's rounding of Python round(): 2.5 -> 2, 3.5 -> 4.
  assert O.compute_capacity(5, 2, 1.0, "round", 1) == 2
  assert O.compute_capacity(7, 2, 1.0, "round", 1) == 4
  # Shapes quoted for the benchmark configurations.
  assert O.compute_capacity(49 * 2, 8, 1.05) == 16
  assert O.compute_capacity(1568 * 2, 32, 1.0) == 100
  assert O.compute_capacity(2304 * 2, 32, 0.5) == 72
  assert O.compute_capacity(1568 * 2, 8, 1.05) == 412


@pytest.mark.parametrize("case", ["dispatcher_experts_divide_groups",
                                  "dispatcher_groups_divide_experts"])
def test_dispatchers(goldens, case):
  g = goldens[case]
  data = np.asarray(goldens["dispatcher_data"]["data"], np.float32)
  exp_d = np.asarray(g["expected_dispatch"], np.float32)
  exp_c = np.asarray(g["expected_combine"], np.float32)
  ein = O.EinsumDispatcher(np.asarray(g["einsum_combine_weights"], np.float32))
  cw = np.tile(np.asarray(g["indices_combine_weights_tile"], np.float32)[None, None], (2, 3, 1))
  ind = O.ExpertIndicesDispatcher(np.asarray(g["indices"], np.int32), cw,
                                  g["num_experts"], g["capacity"])
  for d in (ein, ind):
    out = d.dispatch(data)
    np.testing.assert_array_almost_equal(out, exp_d)
    np.testing.assert_array_almost_equal(d.combine(out), exp_c)


@pytest.mark.parametrize("bpr", [False, True])
def test_top_experts_per_item(goldens, bpr):
  g = goldens["top_experts_per_item"]
  key = "bpr" if bpr else "vanilla"
  gates = np.asarray(g["gates"], np.float32)
  cw, dw = O.top_experts_per_item_einsum(gates, 2, 2, bpr)
  np.testing.assert_array_almost_equal(cw, np.asarray(g["einsum_combine_weights"][key]))
  assert np.array_equal(dw, cw > 0)
  idx, w = O.top_experts_per_item_indices(gates, 2, bpr)
  np.testing.assert_array_equal(idx, np.asarray(g["indices"][key]))
  np.testing.assert_array_almost_equal(w, np.asarray(g["indices_combine_weights"]))
  # The C greedy simulator agrees with the goldens too.
  idx_c, w_c = route_c.route_batch(gates[None], 2, bpr)
  np.testing.assert_array_equal(idx_c[0], np.asarray(g["indices"][key]))
  np.testing.assert_array_almost_equal(w_c[0], np.asarray(g["indices_combine_weights"]))


def test_top_items_per_expert(goldens):
  g = goldens["top_items_per_expert"]
  gates = np.asarray(g["gates"], np.float32)
  cw, dw, metrics = O.top_items_per_expert_einsum(gates, g["capacity"])
  np.testing.assert_array_equal(dw, np.asarray(g["dispatch_weights"], bool))
  np.testing.assert_array_almost_equal(cw, np.asarray(g["combine_weights"], np.float32))
  for k, v in g["metrics"].items():
    assert float(metrics[k]) == pytest.approx(v, rel=1e-6)


def test_get_dispatcher_errors():
  gates = np.zeros((1, 4, 32), np.float32)
  with pytest.raises(ValueError, match="Unknown dispatcher type"):
    O.get_top_experts_per_item_dispatcher(gates, "foo", 2, False, capacity=2)
  with pytest.raises(ValueError, match="You must specify either 'capacity' or 'capacity_factor'"):
    O.get_top_experts_per_item_dispatcher(gates, "foo", 2, False)
  d = O.get_top_experts_per_item_dispatcher(np.zeros((1, 32, 32), np.float32), "indices", 2,
                                            False, capacity_factor=1.0)
  assert d.capacity == 4


def _apply_generators(batch_size, group_size, num_experts, capacity):
  """The two dispatcher generators of vmoe/moe_test.py:362-417, restated."""
  G = batch_size // group_size
  e = (np.arange(2 * batch_size) % num_experts).reshape(G, group_size, 2)
  pos = np.stack([O.route_greedy(e[g], None, num_experts) for g in range(G)])
  idx = np.stack([e, pos], -1).astype(np.int32)
  w = np.tile(np.asarray([0.7, 0.3], np.float32)[None, None], (G, group_size, 1))
  ind = O.ExpertIndicesDispatcher(idx, w, num_experts, capacity)
  cw = np.zeros((G, group_size, num_experts, capacity), np.float32)
  for g in range(G):
    for s in range(group_size):
      for k in range(2):
        if pos[g, s, k] < capacity:
          cw[g, s, e[g, s, k], pos[g, s, k]] = w[g, s, k]
  return ind, O.EinsumDispatcher(cw)


def test_sparse_moe_apply_closed_form(goldens):
  p = goldens["sparse_moe_apply"]
  B, S, C, E = p["batch_size"], p["group_size"], p["capacity"], p["num_experts"]
  x = (10.0 * np.arange(1, B + 1, dtype=np.float32)).reshape(B // S, S, 1)
  expert = lambda buf: buf + (1 + np.arange(E, dtype=np.float32))[:, None, None]
  b = ((1 + np.arange(2 * B) % E).reshape(B, 2) * np.asarray([[0.7, 0.3]])).sum(1)
  expected = (10 * (1 + np.arange(B)) + b).reshape(-1, S, 1)
  for d in _apply_generators(B, S, E, C):
    np.testing.assert_array_almost_equal(O.sparse_moe(d, expert, x), expected, decimal=4)


def test_sparse_moe_with_axes_closed_form(goldens):
  p = goldens["sparse_moe_with_axes"]
  S, E, C = p["S"], p["E"], p["C"]
  for G in (1, 2, 4, 8):
    x = np.tile(np.arange(S, dtype=np.float32).reshape(1, S, 1), (G, 1, 1))
    w = np.tile(np.arange(S).reshape(1, S, 1, 1) == np.arange(S).reshape(1, 1, E, C),
                (G, 1, 1, 1)).astype(np.float32)
    expert = lambda buf: buf + (1 + np.arange(E, dtype=np.float32))[:, None, None]
    out = O.sparse_moe(O.EinsumDispatcher(w), expert, x)
    expected = np.tile((np.arange(S) + (np.arange(S) // 4 + 1)).reshape(1, S, 1), (G, 1, 1))
    np.testing.assert_array_almost_equal(out, expected, decimal=5)


def test_router_aux_losses(goldens):
  g = goldens["router_aux_losses"]
  gates = np.asarray(g["gates"], np.float32)
  assert float(O.gshard_auxiliary_loss(gates)) == pytest.approx(g["gshard"], abs=5e-7)
  assert float(O.importance_auxiliary_loss(gates)) == pytest.approx(g["importance"], abs=5e-7)
  ld = g["load"]
  logits = np.asarray(ld["logits"], np.float32)
  noisy = logits + np.asarray(ld["noise"], np.float32)
  out = O.load_auxiliary_loss(logits, noisy, ld["noise_std"], ld["num_selected_experts"])
  assert float(out) == pytest.approx(ld["expected"], abs=5e-7)
  m = O.router_metrics(gates[None])
  assert float(m["auxiliary_loss"][0]) == pytest.approx(g["importance"], abs=5e-7)
  m = O.router_metrics(gates[None], gshard_loss_weight=2.0, importance_loss_weight=0.0)
  assert float(m["auxiliary_loss"][0]) == pytest.approx(2 * g["gshard"], abs=1e-6)


def test_soft_router_metrics(goldens):
  g = goldens["soft_router_metrics"]
  x = np.asarray(g["x"], np.float32)
  mu = np.asarray(g["mu"], np.float32)
  metrics = O.soft_router_metrics(x, x, mu)
  assert set(metrics) == set(g["expected"])
  for k, v in g["expected"].items():
    assert float(metrics[k]) == pytest.approx(v, abs=1e-5), k


def test_cosine_psim_vs_scipy():
  # vmoe/projects/soft_moe/router_test.py:33-49 with NumPy random data.
  x = np.random.default_rng(0).standard_normal((6, 5, 4, 3, 2)).astype(np.float32)
  y = O.cosine_psim(x, (0,), (3, 4))
  assert y.shape == (6, 5, 4, 5, 4)
  pdist, squareform = scipy.spatial.distance.pdist, scipy.spatial.distance.squareform
  expected = np.stack([
      (1 - squareform(pdist(xi.reshape(20, -1), metric="cosine"))).reshape(5, 4, 5, 4)
      for xi in x])
  np.testing.assert_allclose(y, expected, rtol=1e-3, atol=1e-6)


def test_soft_router_forward_shapes(goldens):
  g = goldens["soft_router_forward"]
  G, m, D = g["x_shape"]
  n = g["num_experts"]
  p = O.soft_num_slots(m, n, None, 1.0)
  assert [D, n, p] == g["mu_shape"]
  rng = np.random.default_rng(0)
  x = np.ones((G, m, D), np.float32)
  mu = rng.standard_normal((D, n, p)).astype(np.float32)
  disp, metrics = O.soft_router(x, mu, 1.0)
  assert isinstance(disp, O.Bfloat16Dispatcher)
  assert metrics["auxiliary_loss"] == 0


def test_soft_router_weights_invariants():
  rng = np.random.default_rng(1)
  x = rng.standard_normal((3, 10, 16)).astype(np.float32)
  mu = rng.standard_normal((16, 4, 2)).astype(np.float32)
  logits, dw, cw, mu_unit = O.soft_router_weights(x, mu, 1.7)
  # Closed form in float64.
  xn = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).sum(-1, keepdims=True) + 1e-6)
  mn = mu.astype(np.float64) / np.sqrt((mu.astype(np.float64) ** 2).sum(0, keepdims=True) + 1e-6)
  L = 1.7 * np.einsum("gmd,dnp->gmnp", xn, mn)
  np.testing.assert_allclose(logits, L, rtol=1e-5, atol=1e-6)
  np.testing.assert_allclose(dw.sum(axis=1), 1.0, rtol=1e-5)
  np.testing.assert_allclose(cw.sum(axis=(2, 3)), 1.0, rtol=1e-5)
  e = np.exp(L)
  np.testing.assert_allclose(dw, e / e.sum(1, keepdims=True), rtol=1e-4)
  np.testing.assert_allclose(cw, e / e.sum((2, 3), keepdims=True), rtol=1e-4)
  # The scale multiplies the inputs instead when they are the smaller operand.
  x2 = rng.standard_normal((1, 2, 16)).astype(np.float32)
  l2 = O.soft_router_weights(x2, mu, 1.7)[0]
  l1 = O.soft_router_weights(x2, mu, 1.0)[0]
  np.testing.assert_allclose(l2, 1.7 * l1, rtol=1e-5, atol=1e-6)


def test_bf16_round_vs_torch():
  import torch
  rng = np.random.default_rng(2)
  x = np.concatenate([rng.standard_normal(100000).astype(np.float32) * 10.0 ** rng.integers(-20, 20, 100000),
                      np.asarray([0.0, -0.0, 1.0, 1.00390625, 1.0078125, 3.3895314e38, np.inf, -np.inf], np.float32)])
  x = x.astype(np.float32)
  want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
  np.testing.assert_array_equal(O._bf16_round_numpy(x), want)
  big = np.tile(x, 12)
  np.testing.assert_array_equal(O.bf16_round(big), np.tile(want, 12))
  assert np.isnan(O.bf16_round(np.asarray([np.nan], np.float32))[0])


def test_bfloat16_dispatcher():
  # vmoe/moe_test.py:54-69: the inner dispatcher only ever sees bfloat16 values.
  class Inner:
    def dispatch(self, x):
      np.testing.assert_array_equal(x, O.bf16_round(x))
      return x
    combine = dispatch
  x = np.random.default_rng(0).standard_normal((5, 4, 3)).astype(np.float32)
  d = O.Bfloat16Dispatcher(Inner())
  assert d.dispatch(x).dtype == np.float32 and d.combine(x).dtype == np.float32


# ---------------------------------------------------------------- independent checks
def _layout_einops(data):
  G, E = data.shape[:2]
  if G % E == 0:
    # moe.py:493-495: reshape(E, G/E, E, C), swapaxes(0, 2): g = g_hi*(G/E) + g_lo.
    return einops.rearrange(data, "(ghi glo) e c ... -> e (glo ghi c) ...", ghi=E)
  return einops.rearrange(data, "g e c ... -> e (g c) ...")


@pytest.mark.parametrize("G,E,C", [(2, 2, 2), (2, 4, 1), (4, 2, 3), (32, 8, 16), (16, 32, 4),
                                   (6, 4, 2), (256, 128, 1), (3, 3, 5), (1, 7, 2)])
def test_layout_vs_einops_and_closed_form(G, E, C):
  data = np.arange(G * E * C * 2, dtype=np.float32).reshape(G, E, C, 2)
  out = O.dispatch_layout(data)
  if G % E == 0:
    # Independent statement: hand-built G=4,E=2 case has expert rows from groups 0,2,1,3.
    np.testing.assert_array_equal(out, _layout_einops(data))
  else:
    np.testing.assert_array_equal(out, _layout_einops(data))
  np.testing.assert_array_equal(O.receive_layout(out, G), data)
  for g in range(G):
    for c in range(C):
      r = O.buffer_row(g, c, G, E, C)
      np.testing.assert_array_equal(out[:, r], data[g, :, c])


def test_layout_group_order_g4_e2():
  data = np.zeros((4, 2, 1, 1), np.float32)
  data[:, :, 0, 0] = np.arange(4)[:, None]
  out = O.dispatch_layout(data)
  np.testing.assert_array_equal(out[0, :, 0], [0, 2, 1, 3])
  np.testing.assert_array_equal(out[1, :, 0], [0, 2, 1, 3])


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("bpr", [False, True])
def test_cumsum_formulation_vs_greedy(seed, bpr):
  rng = np.random.default_rng(seed)
  S, E, K = int(rng.integers(1, 40)), int(rng.integers(2, 9)), 0
  K = int(rng.integers(1, E + 1))
  if seed % 2:  # heavy ties: few distinct gate values
    gates = rng.integers(0, 3, (S, E)).astype(np.float32) / 4
  else:
    gates = O.softmax(rng.standard_normal((S, E)).astype(np.float32))
  idx, w = O.top_experts_per_item_indices(gates, K, bpr)
  pos = O.route_greedy(idx[..., 0], w[:, 0] if bpr else None, E)
  np.testing.assert_array_equal(idx[..., 1], pos)
  idx_c, w_c = route_c.route_batch(gates[None], K, bpr)
  np.testing.assert_array_equal(idx_c[0], idx)
  np.testing.assert_array_equal(w_c[0], w)


@pytest.mark.parametrize("bpr", [False, True])
def test_routing_invariants(bpr):
  rng = np.random.default_rng(7)
  G, S, E, K, C = 3, 64, 8, 2, 12
  gates = O.softmax(rng.standard_normal((G, S, E)).astype(np.float32) * 2)
  d = O.get_top_experts_per_item_dispatcher(gates, "indices", K, bpr, capacity=C)
  de = O.get_top_experts_per_item_dispatcher(gates, "einsum", K, bpr, capacity=C)
  for g in range(G):
    e, p = d.indices[g, ..., 0], d.indices[g, ..., 1]
    for x in range(E):
      # positions handed out for an expert are exactly 0..demand-1, first choices first.
      p0 = np.sort(p[:, 0][e[:, 0] == x])
      p1 = np.sort(p[:, 1][e[:, 1] == x])
      np.testing.assert_array_equal(np.concatenate([p0, p1]), np.arange(len(p0) + len(p1)))
    # einsum and indices dispatchers describe the same assignment.
    dense = np.zeros((S, E, C), np.float32)
    for s in range(S):
      for k in range(K):
        if p[s, k] < C:
          dense[s, e[s, k], p[s, k]] = d.combine_weights[g, s, k]
    np.testing.assert_array_equal(dense, de.combine_weights[g])
  x = rng.standard_normal((G, S, 5)).astype(np.float32)
  np.testing.assert_allclose(d.dispatch(x), de.dispatch(x), rtol=0, atol=0)
  y = rng.standard_normal((E, G * C, 3)).astype(np.float32)
  np.testing.assert_allclose(d.combine(y), de.combine(y), rtol=1e-6, atol=1e-6)


def test_bpr_is_permutation_equivariant():
  rng = np.random.default_rng(11)
  S, E, K = 50, 6, 2
  gates = O.softmax(rng.standard_normal((S, E)).astype(np.float32))
  perm = rng.permutation(S)
  a, _ = O.top_experts_per_item_indices(gates, K, True)
  b, _ = O.top_experts_per_item_indices(gates[perm], K, True)
  np.testing.assert_array_equal(a[perm], b)


def test_softmax_dense_gelu_closed_forms():
  rng = np.random.default_rng(3)
  x = rng.standard_normal((4, 7, 16)).astype(np.float32)
  w = rng.standard_normal((16, 5)).astype(np.float32)
  g = O.router_gates(x, w, O.F32)
  z = x.astype(np.float64) @ w.astype(np.float64)
  e = np.exp(z - z.max(-1, keepdims=True))
  np.testing.assert_allclose(g, e / e.sum(-1, keepdims=True), rtol=1e-5)
  t = np.linspace(-6, 6, 101)
  ref = [0.5 * v * (1 + math.tanh(math.sqrt(2 / math.pi) * (v + 0.044715 * v ** 3))) for v in t]
  np.testing.assert_allclose(O.gelu(t), ref, rtol=1e-5, atol=1e-6)
  ref_erf = [0.5 * v * (1 + math.erf(v / math.sqrt(2))) for v in t]
  np.testing.assert_allclose(O.gelu(t, approximate=False), ref_erf, rtol=1e-5, atol=1e-6)
  # bf16 mode only ever produces bf16-representable values.
  gb = O.router_gates(x, w, O.BF16)
  np.testing.assert_array_equal(gb, O.bf16_round(gb))
  np.testing.assert_allclose(gb, g, rtol=6e-2, atol=2e-3)


def test_gelu_vs_torch():
  """The oracle's two GELUs against torch's CPU implementations (an independent statement of
  flax.linen.gelu's approximate=True / False forms; several GPU tests use torch's as their
  reference, so the two must agree).  In the negative tail 1 + tanh (1 + erf) cancels in
  float32, hence the absolute floor of a few float32 steps of 1."""
  import torch
  t = np.concatenate([np.linspace(-9, 9, 2001), [0.0, -0.0, 1e-8, -1e-8, 20.0, -20.0]]).astype(np.float32)
  tt = torch.from_numpy(t)
  np.testing.assert_allclose(O.gelu(t), torch.nn.functional.gelu(tt, approximate="tanh").numpy(),
                             rtol=2e-6, atol=5e-7)
  np.testing.assert_allclose(O.gelu(t, approximate=False), torch.nn.functional.gelu(tt).numpy(),
                             rtol=2e-6, atol=1e-6)


def test_mlp_block_vs_float64():
  rng = np.random.default_rng(4)
  E, R, D, M = 3, 5, 8, 12
  x = rng.standard_normal((E, R, D)).astype(np.float32)
  w0 = rng.standard_normal((E, D, M)).astype(np.float32) / np.sqrt(D)
  b0 = rng.standard_normal((E, M)).astype(np.float32)
  w1 = rng.standard_normal((E, M, D)).astype(np.float32) / np.sqrt(M)
  b1 = rng.standard_normal((E, D)).astype(np.float32)
  y = O.mlp_block(x, w0, b0, w1, b1, O.F32)
  h = np.einsum("erd,edm->erm", x.astype(np.float64), w0.astype(np.float64)) + b0[:, None]
  h = 0.5 * h * (1 + np.tanh(np.sqrt(2 / np.pi) * (h + 0.044715 * h ** 3)))
  want = np.einsum("erm,emd->erd", h, w1.astype(np.float64)) + b1[:, None]
  np.testing.assert_allclose(y, want, rtol=1e-5, atol=1e-5)
  yb = O.mlp_block(x, w0, b0, w1, b1, O.BF16)
  np.testing.assert_allclose(yb, want, rtol=5e-2, atol=5e-2)


def test_mlp_moe_block_runs_and_matches_manual():
  rng = np.random.default_rng(5)
  N, L, D, M, E, K, S = 4, 6, 8, 16, 4, 2, 12
  x = rng.standard_normal((N, L, D)).astype(np.float32)
  params = {
      "Router": {"dense": {"kernel": rng.standard_normal((D, E)).astype(np.float32)}},
      "Mlp": {"Dense_0": {"kernel": rng.standard_normal((E, D, M)).astype(np.float32) / 3,
                          "bias": np.zeros((E, M), np.float32)},
              "Dense_1": {"kernel": rng.standard_normal((E, M, D)).astype(np.float32) / 4,
                          "bias": np.zeros((E, D), np.float32)}}}
  out, metrics = O.mlp_moe_block(x, params, group_size=S, num_selected_experts=K,
                                 dispatcher_kwargs=dict(name="indices", batch_priority=True,
                                                        capacity_factor=4.0))
  assert out.shape == x.shape and metrics["auxiliary_loss"].shape == (2,)
  # capacity_factor 4 => nothing dropped => y[t] = sum_k gate_k * mlp_{e_k}(x[t]).
  xt = x.reshape(-1, D)
  gates = O.router_gates(xt[None], params["Router"]["dense"]["kernel"], O.F32)[0]
  val, idx = O.top_k(gates, K)
  want = np.zeros_like(xt)
  for t in range(xt.shape[0]):
    for k in range(K):
      e = idx[t, k]
      y = O.mlp_block(xt[None, t:t + 1], params["Mlp"]["Dense_0"]["kernel"][e:e + 1], None,
                      params["Mlp"]["Dense_1"]["kernel"][e:e + 1], None, O.F32)[0, 0]
      want[t] += val[t, k] * y
  np.testing.assert_allclose(out.reshape(-1, D), want, rtol=1e-4, atol=1e-5)
