"""Host-side logic of the drop-in surface that needs no GPU: name resolution of routers
(vmoe/utils.py:59-109, vmoe/nn/vit_moe.py:76-88), capacity arithmetic, the public
factories, and the refusal to run forward-only kernels under autograd."""
import numpy as np
import pytest
import torch

from vmoe_amd import moe, utils
from vmoe_amd.nn import routing, vit_moe
from vmoe_amd.projects.soft_moe import router as soft_router


def test_parse_call_forms():
  fn, args, kwargs = utils.parse_call("NoisyTopExpertsPerItemRouter", default_module=routing)
  assert fn is routing.NoisyTopExpertsPerItemRouter and args == () and kwargs == {}
  fn, args, kwargs = utils.parse_call("vmoe_amd.projects.soft_moe.router.SoftRouter", routing)
  assert fn is soft_router.SoftRouter
  fn, args, kwargs = utils.parse_call("NoisyTopItemsPerExpertRouter(noise_std=0.5)", routing)
  assert fn is routing.NoisyTopItemsPerExpertRouter and kwargs == {"noise_std": 0.5}
  fn, args, kwargs = utils.parse_call("compute_capacity(128, 32, 2.0)", moe)
  assert fn(*args, **kwargs) == 8
  with pytest.raises(AttributeError):
    utils.parse_call("NoSuchRouter", routing)
  with pytest.raises(ValueError):
    utils.parse_call("f()()", routing)


@pytest.mark.parametrize("spec,cls", [
    ({}, routing.NoisyTopExpertsPerItemRouter),
    ({"name": "NoisyTopExpertsPerItemRouter"}, routing.NoisyTopExpertsPerItemRouter),
    ({"name": "NoisyTopItemsPerExpertRouter"}, routing.NoisyTopItemsPerExpertRouter),
    ({"name": "vmoe_amd.projects.soft_moe.router.SoftRouter", "num_slots": 2}, soft_router.SoftRouter),
])
def test_create_router_by_name(spec, cls):
  """vmoe/nn/vit_moe.py:76-88: `name` picks the class, `deterministic` is inherited from the
  block unless the router's own arguments set it, dtype and the module name are passed on."""
  block = vit_moe.MlpMoeBlock(mlp_dim=8, num_experts=4, group_size=16, deterministic=True,
                              router=spec, dtype=torch.bfloat16)
  router = block.create_router()
  assert type(router) is cls
  assert router.num_experts == 4 and router.deterministic is True
  assert router.dtype == torch.bfloat16 and router.name == "Router"
  override = vit_moe.MlpMoeBlock(mlp_dim=8, num_experts=4, group_size=16, deterministic=True,
                                 router=dict(spec, deterministic=False))
  assert override.create_router().deterministic is False


def test_create_split_rngs():
  """vmoe/nn/vit_moe.py:90-99."""
  mk = lambda v: vit_moe.MlpMoeBlock(mlp_dim=8, num_experts=4, group_size=16, split_rngs=v)
  assert mk(False).create_split_rngs() == {"params": False, "dropout": False}
  assert mk(True).create_split_rngs() == {"params": True, "dropout": True}
  assert mk(("dropout",)).create_split_rngs() == {"params": False, "dropout": True}


def test_compute_capacity_values(goldens):
  for case in goldens["compute_capacity"]["cases"]:
    case = dict(case)
    expected = case.pop("expected")
    assert moe.compute_capacity(**case) == expected
  with pytest.raises(ValueError, match="must be greater than or equal to 1"):
    moe.compute_capacity(128, 32, -1.0)
  # Python's round() rounds halves to even (vmoe/moe.py:240)
  assert moe.compute_capacity(20, 8, 1.0, ceil_or_round="round", multiple_of=1) == 2
  assert moe.compute_capacity(28, 8, 1.0, ceil_or_round="round", multiple_of=1) == 4


def test_get_dense_einsum_dispatcher():
  """vmoe/moe.py:260-264: the gates are the combine weights, keyword arguments pass through."""
  gates = torch.rand((2, 6, 3))
  d = moe.get_dense_einsum_dispatcher(gates, partition_spec=("a",))
  assert isinstance(d, moe.DenseEinsumDispatcher)
  assert d.combine_weights is gates and d.partition_spec == ("a",)


def test_forward_only_modules_refuse_autograd():
  """The gating, routing and expert kernels have no backward pass: with a parameter or an
  input that requires a gradient they raise instead of returning a result cut out of the
  graph.  (The check comes before any device call, so CPU tensors do here.)"""
  x = torch.zeros((2, 8, 16))
  w = torch.zeros((16, 4), requires_grad=True)
  for layer in (routing.NoisyTopExpertsPerItemRouter(num_experts=4, deterministic=True),
                routing.NoisyTopItemsPerExpertRouter(num_experts=4, deterministic=True,
                                                     dispatcher=dict(name="einsum", capacity=2))):
    with pytest.raises(NotImplementedError, match="no backward pass"):
      layer.apply({"params": {"dense": {"kernel": w}}}, x)
  soft = soft_router.SoftRouter(num_experts=4, num_slots=1)
  mu = torch.zeros((16, 4, 1), requires_grad=True)
  with pytest.raises(NotImplementedError, match="no backward pass"):
    soft.apply({"params": {"mu": mu, "scale": torch.ones(())}}, x)
  mlp = vit_moe.MlpBlock(mlp_dim=8)
  params = {"Dense_0": {"kernel": torch.zeros((1, 16, 8), requires_grad=True), "bias": torch.zeros((1, 8))},
            "Dense_1": {"kernel": torch.zeros((1, 8, 16)), "bias": torch.zeros((1, 16))}}
  with pytest.raises(NotImplementedError, match="no backward pass"):
    mlp.apply_experts({"params": params}, torch.zeros((1, 4, 16)))
  with pytest.raises(NotImplementedError, match="no backward pass"):
    mlp.apply_experts_gathered({"params": params}, torch.zeros((4, 16)),
                               torch.zeros((1, 4), dtype=torch.int32),
                               torch.zeros((1,), dtype=torch.int32))
  # without autograd recording the same calls reach the device layer (and fail there on CPU tensors)
  with torch.no_grad():
    with pytest.raises(Exception) as info:
      mlp.apply_experts({"params": params}, torch.zeros((1, 4, 16)))
    assert not isinstance(info.value, NotImplementedError)
