"""Shapes and seeded synthetic inputs of the MoE-layer benchmark configurations.

Inputs are drawn on the host with NumPy's PCG64 so that the HIP path and any
checker see identical bytes.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, Optional

import numpy as np


@dataclasses.dataclass(frozen=True)
class LayerConfig:
  name: str
  d_model: int
  mlp_dim: int
  num_experts: int
  num_selected_experts: int
  num_images: int
  tokens_per_image: int
  group_images: int
  capacity_factor: float
  batch_priority: bool
  dtype: str                     # "float32" | "bfloat16"
  layer_norm_inputs: bool = False
  logit_bias_std: float = 0.0

  @property
  def group_size(self) -> int:
    return self.group_images * self.tokens_per_image

  @property
  def num_tokens(self) -> int:
    return self.num_images * self.tokens_per_image

  @property
  def num_groups(self) -> int:
    return self.num_tokens // self.group_size

  def dispatcher_kwargs(self, name: str = "indices") -> Dict:
    return dict(name=name, batch_priority=self.batch_priority,
                capacity_factor=self.capacity_factor)


# Single V-MoE S/32-style layer (fp32, vanilla routing, cf 1.05).
S32 = LayerConfig("vmoe_s32_layer", 512, 2048, 8, 2, 32, 49, 1, 1.05, False, "float32")
# V-MoE B/16 layer: the headline configuration (bf16, BPR, cf 1.0).
B16 = LayerConfig("vmoe_b16_layer_E32_k2_bpr", 768, 3072, 32, 2, 256, 196, 8, 1.0, True,
                  "bfloat16", layer_norm_inputs=True)
# V-MoE L/16 at 384px with reduced capacity and skewed logits.
L16 = LayerConfig("vmoe_l16_384_layer_cf0.5", 1024, 4096, 32, 2, 64, 576, 4, 0.5, True,
                  "bfloat16", layer_norm_inputs=True, logit_bias_std=2.0)
# One MoE layer of the full B/16 model (E=8, cf 1.05, batch 512).
B16_FULL = LayerConfig("vmoe_b16_model_layer_E8", 768, 3072, 8, 2, 512, 196, 8, 1.05, True,
                       "bfloat16", layer_norm_inputs=True)

CONFIGS = {c.name: c for c in (S32, B16, L16, B16_FULL)}


@dataclasses.dataclass(frozen=True)
class SoftConfig:
  name: str
  d_model: int
  mlp_dim: int
  num_experts: int
  num_slots: int
  num_images: int
  tokens_per_image: int
  dtype: str


SOFT_B16 = SoftConfig("soft_moe_b16_128x1", 768, 3072, 128, 1, 256, 196, "bfloat16")


def vit_b16_moe_model(dtype=None, num_classes: int = 1000) -> Dict:
  """Constructor arguments of the full V-MoE B/16 at 224 px: 12 blocks, 12 heads,
  d = 768, mlp 3072, experts (E = 8, top-2, batch priority routing, capacity factor
  1.05, groups of 8 images) on every odd block, global-average-pool head."""
  return dict(
      num_classes=num_classes, patch_size=(16, 16), hidden_size=768, classifier="gap",
      representation_size=None, deterministic=True, head_kernel_zero_init=False,
      encoder=dict(
          num_layers=12, mlp_dim=3072, num_heads=12, dtype=dtype,
          moe=dict(layers=(1, 3, 5, 7, 9, 11), num_experts=8, group_size=8 * 196,
                   router=dict(num_selected_experts=2,
                               dispatcher=dict(name="indices", batch_priority=True,
                                               capacity_factor=1.05)))))


VIT_B16_MOE_NAME = "vmoe_b16_model_E8_k2_224"
VIT_B16_MOE_BATCH = 512


def make_layer_inputs(cfg: LayerConfig, seed: int = 0, num_images: Optional[int] = None):
  """float32 NumPy arrays: x (N, L, D), router kernel (D, E), optional logit bias
  (E,), expert kernels (E, D, M) / (E, M, D) LeCun-normal, zero biases."""
  rng = np.random.Generator(np.random.PCG64(seed))
  N = num_images or cfg.num_images
  D, M, E = cfg.d_model, cfg.mlp_dim, cfg.num_experts
  x = rng.standard_normal((N, cfg.tokens_per_image, D), dtype=np.float32)
  if cfg.layer_norm_inputs:
    x = (x - x.mean(-1, keepdims=True)) / np.sqrt(x.var(-1, keepdims=True) + 1e-6)
    x = x.astype(np.float32)
  router = (rng.standard_normal((D, E), dtype=np.float32) / np.sqrt(D)).astype(np.float32)
  bias = None
  if cfg.logit_bias_std:
    bias = (rng.standard_normal(E, dtype=np.float32) * cfg.logit_bias_std).astype(np.float32)
  w0 = rng.standard_normal((E, D, M), dtype=np.float32) / np.float32(np.sqrt(D))
  w1 = rng.standard_normal((E, M, D), dtype=np.float32) / np.float32(np.sqrt(M))
  params = {
      "Router": {"dense": {"kernel": router}},
      "Mlp": {"Dense_0": {"kernel": w0, "bias": np.zeros((E, M), np.float32)},
              "Dense_1": {"kernel": w1, "bias": np.zeros((E, D), np.float32)}},
  }
  return x, params, bias


def make_soft_inputs(cfg: SoftConfig, seed: int = 0, num_images: Optional[int] = None):
  rng = np.random.Generator(np.random.PCG64(seed))
  N = num_images or cfg.num_images
  D, M, n, p = cfg.d_model, cfg.mlp_dim, cfg.num_experts, cfg.num_slots
  x = rng.standard_normal((N, cfg.tokens_per_image, D), dtype=np.float32)
  mu = (rng.standard_normal((D, n, p), dtype=np.float32) / np.sqrt(D)).astype(np.float32)
  w0 = rng.standard_normal((n, D, M), dtype=np.float32) / np.float32(np.sqrt(D))
  w1 = rng.standard_normal((n, M, D), dtype=np.float32) / np.float32(np.sqrt(M))
  params = {"Router": {"mu": mu, "scale": np.float32(1.0)},
            "Mlp": {"Dense_0": {"kernel": w0, "bias": np.zeros((n, M), np.float32)},
                    "Dense_1": {"kernel": w1, "bias": np.zeros((n, D), np.float32)}}}
  return x, params
