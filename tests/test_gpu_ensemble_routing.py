"""vmoe/nn/ensemble_routing_test.py restated on the drop-in surface, plus parity of the
ensemble router with its CPU restatement."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.util import dev, to_dev, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ens():
  from vmoe_amd.nn import ensemble_routing
  return ensemble_routing


def _layer_and_inputs(ens, num_groups, ens_size, deterministic):
  num_experts, batch_size = 4, 6
  rep = batch_size * ens_size
  dim_x = num_experts
  x = torch.arange(dim_x * rep * num_groups, dtype=torch.float32, device=dev()).reshape(
      num_groups, rep, dim_x)
  kernel = torch.eye(dim_x, device=dev()).reshape(dim_x, ens_size, num_experts // ens_size)
  layer = ens.NoisyTopExpertsPerItemEnsembleRouter(
      num_experts=num_experts, ensemble_size=ens_size, num_selected_experts=2, noise_std=1.0,
      deterministic=deterministic, dispatcher=dict(name="einsum", capacity=rep, batch_priority=False))
  return layer, {"params": {"dense": {"kernel": kernel}}}, x


@pytest.mark.parametrize("num_groups,ens_size", [(1, 1), (1, 2), (2, 1), (2, 2)])
def test_forward_deterministic(ens, num_groups, ens_size):
  """ensemble_routing_test.py:45-76."""
  layer, variables, x = _layer_and_inputs(ens, num_groups, ens_size, True)
  d1, m1 = layer.apply(variables, x, rngs={"gating": 0})
  d2, m2 = layer.apply(variables, x, rngs={"gating": 1})
  np.testing.assert_array_equal(to_np(d1.combine_weights), to_np(d2.combine_weights))
  for k in m1:
    np.testing.assert_array_equal(to_np(m1[k]), to_np(m2[k]))
    assert tuple(m1[k].shape) == (num_groups, ens_size)


@pytest.mark.parametrize("num_groups,ens_size", [(1, 1), (1, 2), (2, 1), (2, 2)])
def test_forward_not_deterministic(ens, num_groups, ens_size):
  """ensemble_routing_test.py:78-121."""
  layer, variables, x = _layer_and_inputs(ens, num_groups, ens_size, False)
  g1, m1 = layer._compute_ensemble_gates_softmax_and_metrics(
      x, variables["params"]["dense"]["kernel"], {"gating": 0})
  g2, m2 = layer._compute_ensemble_gates_softmax_and_metrics(
      x, variables["params"]["dense"]["kernel"], {"gating": 1})
  assert (g1 - g2).abs().sum() > 1e-3
  np.testing.assert_allclose(to_np(m1["importance_loss"]), to_np(m2["importance_loss"]))
  for k in ("auxiliary_loss", "gshard_loss", "load_loss"):
    assert (m1[k] - m2[k]).abs().sum() > 1e-3, k
    assert tuple(m1[k].shape) == (num_groups, ens_size)


def test_expert_partitioning(ens):
  """ensemble_routing_test.py:123-162: selection stays inside each member's experts."""
  x = torch.arange(2 * 3, dtype=torch.float32, device=dev()).reshape(1, 2, 3)
  kernel = torch.tensor([[[1.0, 1.0], [-1.0, -1.0]],
                         [[-1.0, 1.0], [-1.0, -1.0]],
                         [[-1.0, -1.0], [-1.0, 1.0]]], device=dev())
  layer = ens.NoisyTopExpertsPerItemEnsembleRouter(
      num_experts=4, ensemble_size=2, num_selected_experts=1, noise_std=1.0, deterministic=False)
  gates, _ = layer._compute_ensemble_gates_softmax_and_metrics(x, kernel, {"gating": 0})
  selected = to_np(gates.argmax(-1))
  assert selected[0, 0] in (0, 1) and selected[0, 1] in (2, 3)
  free = to_np((x @ kernel.reshape(3, 4)).argmax(-1))
  assert free[0, 0] != selected[0, 0] and free[0, 1] != selected[0, 1]


def test_diag_blocks(ens):
  """ensemble_routing_test.py:164-185 against scipy's block_diag."""
  import scipy.linalg
  blocks = np.stack([[k * np.ones((2, 3)) for k in range(1, 5)],
                     [-k * np.ones((2, 3)) for k in range(1, 5)]]).astype(np.float32)
  out = to_np(ens.reshape_from_diag_blocks(to_dev(blocks)))
  for g in range(2):
    np.testing.assert_array_equal(out[g], scipy.linalg.block_diag(*blocks[g]))


def test_reshape_to_and_from_group_representation(ens):
  """ensemble_routing_test.py:187-225: copies of an image stay in one group, round trip exact."""
  num_images, M, T, H, G = 4, 2, 3, 1, 2
  group_size = num_images * M * T // G
  x = np.zeros((num_images * M, T, H), np.float32)
  for i in range(num_images):
    for m in range(M):
      x[i * M + m, :, 0] = 100 * i + np.arange(T)       # the M copies of image i are equal
  y = ens.reshape_to_group_size_representation(to_dev(x), group_size, M)
  assert tuple(y.shape) == (G, group_size, H)
  yn = to_np(y).reshape(G, group_size // M, M)
  assert (yn[:, :, 0] == yn[:, :, 1]).all()               # items (i, m) adjacent, m minor
  back = ens.reshape_from_group_size_representation(y, T, M)
  np.testing.assert_array_equal(to_np(back), x)


@pytest.mark.parametrize("dtype", [O.F32, O.BF16])
@pytest.mark.parametrize("noisy", [False, True])
def test_ensemble_router_vs_oracle(ens, dtype, noisy):
  rng = np.random.default_rng(5)
  G, S, D, E, M, K = 2, 48, 32, 8, 2, 2
  x = O.cast(rng.standard_normal((G, S, D)).astype(np.float32), dtype)
  kernel = O.cast(rng.standard_normal((D, M, E // M)).astype(np.float32) / np.sqrt(D), dtype)
  dkw = dict(name="indices", capacity=16, batch_priority=True)
  layer = ens.NoisyTopExpertsPerItemEnsembleRouter(
      num_experts=E, ensemble_size=M, num_selected_experts=K, noise_std=1.5,
      deterministic=not noisy, gshard_loss_weight=0.3, importance_loss_weight=0.7,
      load_loss_weight=0.5, dispatcher=dkw)
  variables = {"params": {"dense": {"kernel": to_dev(kernel, dtype)}}}
  dispatcher, metrics = layer.apply(variables, to_dev(x, dtype), rngs={"gating": 3})
  noises = None
  if noisy:
    gen = torch.Generator(device=dev()).manual_seed(3)
    noises = [to_np(torch.randn((G, S // M, E // M), generator=gen, device=dev())) for _ in range(M)]
  want_d, want_m, _ = O.ensemble_router(
      x, kernel, M, K, dkw, dtype, gshard_loss_weight=0.3, importance_loss_weight=0.7,
      noises=noises, noise_std=1.5, load_loss_weight=0.5)
  assert set(metrics) == set(want_m)
  tol = 2e-2 if dtype == O.BF16 else 2e-4
  for k in metrics:
    assert tuple(metrics[k].shape) == (G, M)
    np.testing.assert_allclose(to_np(metrics[k]), want_m[k], rtol=tol, atol=1e-6, err_msg=k)
  got_idx = to_np(dispatcher.indices)
  agree = (got_idx == want_d.indices).all(axis=(2, 3)).mean()
  assert agree >= (0.97 if dtype == O.BF16 else 0.999), agree
  # block structure: item i*M+m only reaches experts of member m
  member = np.arange(S) % M
  assert ((got_idx[..., 0] // (E // M)) == member[None, :, None]).all()


def test_argument_errors(ens):
  x = torch.zeros((1, 6, 4), device=dev())
  k = torch.zeros((4, 2, 2), device=dev())
  mk = lambda **kw: ens.NoisyTopExpertsPerItemEnsembleRouter(
      **{**dict(num_experts=4, ensemble_size=2, deterministic=True), **kw})
  with pytest.raises(ValueError, match="inputs.ndim must be 3"):
    mk().apply({"params": {"dense": {"kernel": k}}}, x[0])
  with pytest.raises(ValueError, match="num_experts must be multiple of ensemble_size"):
    mk(ensemble_size=3).apply({"params": {"dense": {"kernel": k}}}, x)
  with pytest.raises(ValueError, match="group_size must be multiple of ensemble_size"):
    mk().apply({"params": {"dense": {"kernel": k}}}, x[:, :5])
  with pytest.raises(ValueError, match="Ensemble size must be >= 1"):
    mk(ensemble_size=0).apply({"params": {"dense": {"kernel": k}}}, x)
