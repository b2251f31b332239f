"""Benchmark of the MoE layer on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config NAME] [--no-cpu-baseline]

A step is one pass of the whole layer (gating + top-k, losses, slot assignment
with batch priority routing, dispatch, expert MLPs, combine) over one batch of
synthetic tokens already resident in HBM.  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import gc
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)

# Steps run first so that no one-time initialisation (first launches, memory pools) falls
# into the warm-up or the timed steps; the timing events are created after them.
COLD_STEPS = 3
# The expert MLP's two products run under vmoe_expert_mlp or, when the packed rows were
# computed in the launch that plans them (vmoe_compact_rows_planned), under
# vmoe_expert_mlp_planned; the stage tables report the two as vmoe_expert_mlp.
MLP_CALLS = ("vmoe_expert_mlp", "vmoe_expert_mlp_planned")


def merge_mlp_calls(stage_ms):
  if "vmoe_expert_mlp_planned" in stage_ms:
    stage_ms["vmoe_expert_mlp"] = stage_ms.get("vmoe_expert_mlp", 0.0) + stage_ms.pop("vmoe_expert_mlp_planned")
  return stage_ms
# Steps run right in front of the W warm-up steps, after everything that leaves the GPU idle
# (creating events, a garbage collection): an idle GPU takes about 25 ms of work to get its
# clocks back, more than a few warm-up steps of a millisecond each.
INIT_STEPS = 30
# Entry-point calls of one layer step, rounded up: their timing events are created
# before the timed region, which then only records them.
CALLS_PER_STEP = 12

# Published MI355X peaks used as roofline denominators.
PEAK_BF16_TFLOPS = 2500.0
PEAK_FP32_MATRIX_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0

# Short passes of the other workloads that the default run attaches to its line.
OTHER_STEPS, OTHER_WARMUP = 10, 5

# Figures that cannot be measured from inside the run (hardware counters need rocprofv3
# around the process): copied from the summaries under profiles/, and reported under
# roofline.from_profile together with the file they come from.
# HBM bytes per launch of the dominant kernel (FETCH_SIZE + WRITE_SIZE, scaled by a copy
# kernel of known size).
MEASURED_TRAFFIC_BYTES = {
    # mean of the two GEMM launches of a layer: (630 + 565 + 1034 + 148) / 2 MiB;
    # FETCH_SIZE x 2.0, WRITE_SIZE x 1.0 (copy-kernel calibration);
    # profiles/hbm_traffic__vmoe_b16_layer.md.
    "vmoe_b16_layer_E32_k2_bpr": 1.246e9,
}
# Share of the launch during which the matrix cores are busy (SQ_VALU_MFMA_BUSY_CYCLES over
# GRBM_GUI_ACTIVE x 1 024 SIMDs), from the rocprofv3 --pmc runs of this command summarised in
# profiles/mfma_util__vmoe_b16_layer.md: counters cannot be read from inside the run.
MEASURED_MFMA_BUSY = {
    "vmoe_b16_layer_E32_k2_bpr": {
        "first_product": 0.444, "second_product": 0.611, "vendor_gemm_second_product_shape": 0.527,
        "register_resident_mfma_loop": 0.897,
        "source": "profiles/mfma_util__vmoe_b16_layer.md (rocprofv3 --pmc, same command, 5 steps)"},
}


def parse_args():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=20)
  ap.add_argument("--warmup", type=int, default=5)
  ap.add_argument("--config", default="vmoe_b16_layer_E32_k2_bpr")
  ap.add_argument("--no-cpu-baseline", action="store_true")
  ap.add_argument("--no-dispatch-pass", action="store_true",
                  help="skip the extra pass that times dispatcher.dispatch() (for counter runs "
                       "that should see the step's kernels only)")
  ap.add_argument("--no-other-workloads", action="store_true",
                  help="headline configuration only: skip the short passes of the other "
                       "BASELINE configurations")
  ap.add_argument("--cpu-groups", type=int, default=32,
                  help="groups of the workload the CPU baseline is timed on")
  return ap.parse_args()


def device_weights(cfg, torch, dev, seed):
  """Seeded LeCun-normal expert kernels drawn on the device (fast), biases 0."""
  gen = torch.Generator(device=dev)
  gen.manual_seed(seed)
  D, M, E = cfg.d_model, cfg.mlp_dim, cfg.num_experts
  tdt = torch.bfloat16 if cfg.dtype == "bfloat16" else torch.float32
  w0 = (torch.randn((E, D, M), generator=gen, device=dev) / D ** 0.5).to(tdt)
  w1 = (torch.randn((E, M, D), generator=gen, device=dev) / M ** 0.5).to(tdt)
  return w0, w1, torch.zeros((E, M), dtype=tdt, device=dev), torch.zeros((E, D), dtype=tdt, device=dev)


_marker_buffers = None


def trace_marker(kernels, torch, dev):
  """A 48-byte launch of the copy kernel, issued right before and right after the timed steps
  (outside the region the step events bracket): in a kernel trace of the run the dispatches
  between the two markers are the timed passes."""
  global _marker_buffers
  if _marker_buffers is None:
    _marker_buffers = (torch.zeros(48, dtype=torch.uint8, device=dev), torch.zeros(48, dtype=torch.uint8, device=dev))
  kernels.copy_bytes(*_marker_buffers)


def host_cpu_model():
  """Model name of the host CPU the baseline ran on (first entry of /proc/cpuinfo)."""
  try:
    with open("/proc/cpuinfo") as f:
      for line in f:
        if line.lower().startswith("model name"):
          return line.split(":", 1)[1].strip()
  except OSError:
    pass
  return "unknown"


def cpu_baseline(cfg, x_np, params_np, bias_np, groups, gpu_out=None):
  """Times the CPU oracle (NumPy/torch-CPU restatement of the reference path) on
  the first `groups` groups of the same workload.  With gpu_out (the layer's output
  for the same items, float32 NumPy) the oracle's output is also compared with it:
  an item is bad if any element differs by more than 2e-2 * (rms + |want|)
  (bfloat16; 2e-5 in float32)."""
  from oracle import moe_oracle as O
  S = cfg.group_size
  imgs = groups * cfg.group_images
  xs = x_np[:imgs]
  dtype = O.BF16 if cfg.dtype == "bfloat16" else O.F32
  def run():
    return O.mlp_moe_block(xs, params_np, group_size=S,
                           num_selected_experts=cfg.num_selected_experts,
                           dispatcher_kwargs=cfg.dispatcher_kwargs("indices"), dtype=dtype,
                           logit_bias=bias_np)
  want, _ = run()
  times = []
  for _ in range(3):
    t0 = time.perf_counter()
    run()
    times.append(time.perf_counter() - t0)
  t = float(np.median(times))
  import torch
  parity = None
  if gpu_out is not None:
    D = want.shape[-1]
    want = np.asarray(want, np.float32).reshape(-1, D)
    got = np.asarray(gpu_out, np.float32).reshape(-1, D)[: want.shape[0]]
    tol = 2e-2 if dtype == O.BF16 else 2e-5
    rms = float(np.sqrt((want.astype(np.float64) ** 2).mean()))
    bad = (np.abs(got - want) > tol * (rms + np.abs(want))).any(-1)
    parity = {"items": int(bad.size), "bad": int(bad.sum()), "rtol": tol,
              "allowed_bad_fraction": 0.01 if dtype == O.BF16 else 0.0,
              "note": "timed path's output for input buffer 0 vs oracle/moe_oracle.py mlp_moe_block"}
  # The same layer in the formulation the reference's released configs use (the einsum
  # dispatcher with its dense (G, S, E, C) weights, vmoe/moe.py:127-161), on two groups.
  eg = min(2, groups)
  xe = x_np[:eg * cfg.group_images]
  t0 = time.perf_counter()
  O.mlp_moe_block(xe, params_np, group_size=S, num_selected_experts=cfg.num_selected_experts,
                  dispatcher_kwargs=cfg.dispatcher_kwargs("einsum"), dtype=dtype, logit_bias=bias_np)
  te = time.perf_counter() - t0
  return parity, {
      "value": groups * S / t, "unit": "tokens/s", "cores": int(torch.get_num_threads()),
      "kind": "port",
      "sample": (f"oracle/moe_oracle.py mlp_moe_block (indices dispatcher) on {groups} of "
                 f"{cfg.num_groups} groups ({groups * S} tokens, all {cfg.num_experts} experts), "
                 f"median of 3 runs of {t:.2f} s; NumPy BLAS + torch CPU threads"),
      "host_cpus": os.cpu_count(), "cpu_model": host_cpu_model(),
      "einsum_dispatcher_formulation": {
          "value": eg * S / te, "unit": "tokens/s",
          "sample": f"same oracle with the einsum dispatcher on {eg} groups ({eg * S} tokens), one run of {te:.2f} s"},
  }


def soft_run(args, short=False):
  """Soft MoE layer (SoftRouter + expert MLPs), same protocol as the sparse layer.  `short`:
  no CPU leg."""
  import torch
  from vmoe_amd import _hip, configs, kernels, moe
  from vmoe_amd.nn import vit_moe
  from vmoe_amd.projects.soft_moe import router as soft_router

  cfg = configs.SOFT_B16
  dev = torch.device("cuda:0")
  torch.cuda.set_device(dev)
  tdt = torch.bfloat16
  D, M, n, p = cfg.d_model, cfg.mlp_dim, cfg.num_experts, cfg.num_slots
  G, m = cfg.num_images, cfg.tokens_per_image
  rng = np.random.Generator(np.random.PCG64(0))
  xs = [torch.from_numpy(rng.standard_normal((G, m, D), dtype=np.float32)).to(dev).to(tdt)
        for _ in range(4)]
  mu = torch.from_numpy((rng.standard_normal((D, n, p), dtype=np.float32) / np.sqrt(D)).astype(np.float32)).to(dev)
  gen = torch.Generator(device=dev)
  gen.manual_seed(1)
  w0 = (torch.randn((n, D, M), generator=gen, device=dev) / D ** 0.5).to(tdt)
  w1 = (torch.randn((n, M, D), generator=gen, device=dev) / M ** 0.5).to(tdt)
  rvars = {"params": {"mu": mu, "scale": torch.ones((), device=dev)}}
  mvars = {"params": {"Dense_0": {"kernel": w0, "bias": torch.zeros((n, M), dtype=tdt, device=dev)},
                      "Dense_1": {"kernel": w1, "bias": torch.zeros((n, D), dtype=tdt, device=dev)}}}
  layer = soft_router.SoftRouter(num_experts=n, num_slots=p, compute_similarity_metrics=False, dtype=tdt)
  mlp = moe.sparse_moe_spmd(vit_moe.MlpBlock, variable_axes={"params": 0})(mlp_dim=M, dtype=tdt)

  def step(i):
    dispatcher, metrics = layer.apply(rvars, xs[i % 4])
    return mlp.apply(mvars, dispatcher, xs[i % 4])

  _hip.set_timing_sink({})
  for i in range(COLD_STEPS):
    step(i)
  torch.cuda.synchronize()
  # As in main(): events only around the dominant entry point inside the timed region,
  # the other stages from a second, fully instrumented pass.
  sink = _hip.TimingSink(pairs=args.steps * 2, only=MLP_CALLS)
  warm_sink = _hip.TimingSink(pairs=(INIT_STEPS + args.warmup) * 2, only=MLP_CALLS)
  # One event per step boundary (the per-step times whose median is reported) and one
  # host time stamp per step (which step, if any, kept the host waiting).
  marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
  for ev in marks:
    ev.record()
  torch.cuda.synchronize()
  host_t = [0.0] * (args.steps + 1)
  # A full collection of Python's cyclic garbage collector walks every object that torch and
  # numpy have created (tens of milliseconds) and fires after a fixed number of allocations,
  # i.e. at a fixed step: it runs now, before the warm-up (an idle GPU takes several steps
  # to get its clocks back), and stays off until the timed loop is over.
  gc.collect()
  gc.disable()
  _hip.set_timing_sink(warm_sink)
  for i in range(INIT_STEPS + args.warmup):
    step(i)
  torch.cuda.synchronize()
  _hip.set_timing_sink(sink)
  trace_marker(kernels, torch, dev)
  t0 = time.perf_counter()
  marks[0].record()
  host_t[0] = t0
  for i in range(args.steps):
    step(i)
    marks[i + 1].record()
    host_t[i + 1] = time.perf_counter()
  t_enqueued = time.perf_counter()
  trace_marker(kernels, torch, dev)
  torch.cuda.synchronize()
  t1 = time.perf_counter()
  gc.enable()
  step_ms = [marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps)]
  host_step_ms = [(host_t[i + 1] - host_t[i]) * 1e3 for i in range(args.steps)]
  ms = float(np.median(step_ms))
  wall_ms = (t1 - t0) * 1e3 / args.steps
  host_ms = (t_enqueued - t0) * 1e3 / args.steps
  full = _hip.TimingSink(pairs=args.steps * CALLS_PER_STEP)
  _hip.set_timing_sink(full)
  for i in range(args.steps):
    step(i)
  torch.cuda.synchronize()
  _hip.set_timing_sink(None)
  per_step = lambda d: {name: float(np.mean([a.elapsed_time(b) for a, b in pairs])) *
                        (len(pairs) / args.steps) for name, pairs in d.items()}
  stage_ms = merge_mlp_calls(per_step(full))
  stage_ms.update(merge_mlp_calls(per_step(sink)))
  T = G * m
  # Dominant kernel: the expert GEMM, weight-bandwidth bound here (1.2 GB of weights
  # for 309 GFLOP): algorithmic bytes = weights + slot activations in and out + hidden.
  rows = G * p
  bytes_mlp = 2 * (2 * n * D * M + 2 * n * rows * D + 2 * n * rows * M)
  mlp_ms = stage_ms["vmoe_expert_mlp"]
  achieved = bytes_mlp / (mlp_ms * 1e-3) / 1e9
  result = {
      "metric": "Soft MoE layer tokens/sec at B/16, 128 experts x 1 slot, bf16",
      "value": T / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
      "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
      "vs_baseline": None, "dtype": "bf16", "data": "synthetic (seeded N(0,1) tokens and parameters)",
      "config": {"workload": cfg.name, "tokens": T, "d_model": D, "mlp_dim": M, "experts": n,
                 "slots_per_expert": p, "groups": G, "group_size": m},
      "roofline": {"bound": "hbm", "kernel": "gemm_bf16_mixed_kernel (first product) / gemm_bf16_persistent_kernel (second product)", "achieved": achieved,
                   "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": achieved / PEAK_HBM_GBS,
                   "traffic": None, "launch_ms": mlp_ms / 2, "bytes_per_layer": bytes_mlp},
      "stage_ms": stage_ms, "host_enqueue_ms_per_step": host_ms, "wall_ms_per_step": wall_ms,
      "ms_per_step_note": ("ms_per_step and value: median of the K per-step times between events "
                           "recorded at the step boundaries; wall_ms_per_step: host clock around the "
                           "same K steps, synchronised on both sides, divided by K"),
      "step_ms_min_max": [float(min(step_ms)), float(max(step_ms))],
      "step_ms_p10_p50_p90": [float(np.percentile(step_ms, q)) for q in (10, 50, 90)],
      "slowest_step": {"gpu": int(np.argmax(step_ms)), "gpu_ms": float(max(step_ms)),
                       "host": int(np.argmax(host_step_ms)), "host_ms": float(max(host_step_ms))},
      "cpu_baseline": None,
  }
  result["expert_mlp_status"] = mlp_status(kernels)
  if not args.no_cpu_baseline and not short:
    # The oracle's Soft MoE layer on the first groups of the same batch (the expert
    # MLPs see `groups` rows each instead of G, all 128 experts' weights are read).
    from oracle import moe_oracle as O
    groups = 32
    f = lambda t: t.detach().float().cpu().numpy()
    x_np, mu_np, w0_np, w1_np = f(xs[0][:groups]), f(mu), f(w0), f(w1)
    b0_np, b1_np = np.zeros((n, M), np.float32), np.zeros((n, D), np.float32)

    def run():
      odisp, _ = O.soft_router(x_np, mu_np, 1.0, O.BF16, compute_similarity_metrics=False)
      return O.sparse_moe(odisp, lambda b: O.mlp_block(b, w0_np, b0_np, w1_np, b1_np, O.BF16), x_np)
    run()
    times = []
    for _ in range(3):
      t0 = time.perf_counter()
      run()
      times.append(time.perf_counter() - t0)
    t = float(np.median(times))
    result["cpu_baseline"] = {
        "value": groups * m / t, "unit": "tokens/s", "cores": int(torch.get_num_threads()),
        "kind": "port",
        "sample": (f"oracle/moe_oracle.py soft_router + sparse_moe(mlp_block) on {groups} of {G} "
                   f"groups ({groups * m} tokens, all {n} experts), median of 3 runs of {t:.2f} s; "
                   "NumPy BLAS + torch CPU threads"),
        "host_cpus": os.cpu_count(), "cpu_model": host_cpu_model()}
  return result


def vit_run(args, short=False):
  """Full V-MoE B/16 forward at 224 px, batch 512: images/s, time per module kind
  broken out with events around the modules' apply methods.  `short`: no CPU leg."""
  import copy
  import torch
  from vmoe_amd import _hip, configs, kernels
  from vmoe_amd.nn import vit_moe

  dev = torch.device("cuda:0")
  torch.cuda.set_device(dev)
  B = configs.VIT_B16_MOE_BATCH
  model_cfg = configs.vit_b16_moe_model(dtype=torch.bfloat16)
  model = vit_moe.VisionTransformerMoe(**model_cfg)
  gen = torch.Generator(device=dev)
  gen.manual_seed(0)
  images = [torch.rand((B, 224, 224, 3), generator=gen, device=dev) * 2 - 1 for _ in range(2)]
  variables = model.init(0, images[0])

  spans = {}

  def timed(cls, method, label):
    fn = getattr(cls, method)

    def wrapper(self, *a, **kw):
      if not spans.get("on"):
        return fn(self, *a, **kw)
      e0, e1 = spans["pool"].take()
      e0.record()
      out = fn(self, *a, **kw)
      e1.record()
      spans.setdefault(label, []).append((e0, e1))
      return out
    setattr(cls, method, wrapper)

  timed(vit_moe.MlpMoeBlock, "apply", "moe_layers")
  timed(vit_moe.MlpBlock, "apply", "dense_mlps")
  timed(vit_moe.MultiHeadDotProductAttention, "apply", "attention")

  def step(i):
    return model.apply(variables, images[i % 2])

  _hip.set_timing_sink({})
  for i in range(3 + args.warmup):
    step(i)
  torch.cuda.synchronize()
  # Timed region: events only around the dominant entry point (the MLP GEMMs); module
  # spans and the other stages come from a second, fully instrumented pass of the same
  # steps (events between kernels serialise their hand-over and would slow the pass).
  sink = _hip.TimingSink(pairs=args.steps * 14, only=MLP_CALLS)
  _hip.set_timing_sink(sink)
  trace_marker(kernels, torch, dev)
  torch.cuda.synchronize()
  t0 = time.perf_counter()
  for i in range(args.steps):
    logits, metrics = step(i)
  torch.cuda.synchronize()
  t1 = time.perf_counter()
  trace_marker(kernels, torch, dev)
  ms = (t1 - t0) * 1e3 / args.steps
  full = _hip.TimingSink(pairs=args.steps * 120)     # about 110 entry-point calls per pass
  spans["pool"] = _hip.TimingSink(pairs=args.steps * 24)
  _hip.set_timing_sink(full)
  spans["on"] = True
  ti0 = time.perf_counter()
  for i in range(args.steps):
    step(i)
  torch.cuda.synchronize()
  ms_instrumented = (time.perf_counter() - ti0) * 1e3 / args.steps
  _hip.set_timing_sink(None)
  spans.pop("on")
  spans.pop("pool")
  module_ms = {k: float(sum(a.elapsed_time(b) for a, b in v)) / args.steps for k, v in spans.items()}
  per_step = lambda d: {name: float(np.mean([a.elapsed_time(b) for a, b in pairs])) *
                        (len(pairs) / args.steps) for name, pairs in d.items()}
  stage_ms = merge_mlp_calls(per_step(full))
  stage_ms.update(merge_mlp_calls(per_step(sink)))
  module_ms["other (patch embedding, layer norms, residuals, head)"] = ms_instrumented - sum(
      module_ms.values())
  module_ms["instrumented_pass_ms_per_step"] = ms_instrumented

  # Dominant kernel: the bf16 GEMM behind the dense and the expert MLPs
  # (two launches per MLP).  Flops: dense 2*T*D*M per launch; experts 2*A*D*M.
  enc = model_cfg["encoder"]
  D, M = model_cfg["hidden_size"], enc["mlp_dim"]
  T = B * 196
  moe_cfg = enc["moe"]
  n_moe = len(moe_cfg["layers"])
  n_dense = enc["num_layers"] - n_moe
  # Rows the expert MLPs really compute: the kept assignments of every MoE block
  # (dropped ones are skipped), read from one more, untimed, pass.
  from vmoe_amd import moe as moe_lib
  live_rows = {}
  packed = moe_lib.ExpertIndicesDispatcher._packed

  def recording(self):
    maps = packed(self)
    live_rows[id(self)] = maps[1]          # rows_per_expert of this block's dispatcher
    recording.keep.append(self)            # keeps ids distinct until they are read
    return maps
  recording.keep = []
  set_maps = moe_lib.ExpertIndicesDispatcher.set_packed_maps

  def recording_set(self, maps):           # (packed rows computed by the expert's planning launch)
    set_maps(self, maps)
    live_rows[id(self)] = maps[1]
    recording.keep.append(self)
  moe_lib.ExpertIndicesDispatcher._packed = recording
  moe_lib.ExpertIndicesDispatcher.set_packed_maps = recording_set
  step(0)
  torch.cuda.synchronize()
  moe_lib.ExpertIndicesDispatcher._packed = packed
  moe_lib.ExpertIndicesDispatcher.set_packed_maps = set_maps
  live_rows = list(live_rows.values())
  kept_per_block = [int(r.sum()) for r in live_rows]
  assert len(kept_per_block) == n_moe
  flops_mlp = 2 * 2.0 * D * M * (n_dense * T + sum(kept_per_block))
  mlp_ms = stage_ms["vmoe_expert_mlp"]
  achieved = flops_mlp / (mlp_ms * 1e-3) / 1e12
  # Whole-model matrix flops per image (projections, attention, MLPs), for scale.
  H, hd, S = enc["num_heads"], D // enc["num_heads"], 196
  flops_attn = enc["num_layers"] * T * (2.0 * D * 3 * D + 2.0 * D * D + 2 * 2.0 * S * D)
  flops_total = flops_mlp + flops_attn + 2.0 * T * (16 * 16 * 3) * D
  result = {
      "metric": "V-MoE B/16 (E=8, top-2 BPR, every odd block) forward images/sec at 224 px",
      "value": B / (ms * 1e-3), "unit": "images/s", "n_gpus": 1, "steps": args.steps,
      "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
      "vs_baseline": None, "dtype": "bf16",
      "data": "synthetic (seeded U(-1,1) images, random-init parameters)",
      "config": {"workload": configs.VIT_B16_MOE_NAME, "batch": B, "image": [224, 224, 3],
                 "tokens": T, "blocks": enc["num_layers"], "moe_blocks": list(moe_cfg["layers"]),
                 "experts": moe_cfg["num_experts"], "selected": 2, "group_size": moe_cfg["group_size"],
                 "capacity_factor": 1.05},
      "roofline": {"bound": "mfma", "kernel": "gemm_bf16_mixed_kernel (first product) / gemm_bf16_w8_kernel<0, true, 8> (second product)", "achieved": achieved,
                   "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": achieved / PEAK_BF16_TFLOPS,
                   "traffic": None, "launch_ms": mlp_ms / (2 * enc["num_layers"]),
                   "flops_all_mlps": flops_mlp, "kept_rows_per_moe_block": kept_per_block,
                   "assignments_per_moe_block": T * moe_cfg["router"]["num_selected_experts"]},
      "model_TFLOPs_per_step": flops_total / 1e12,
      "model_TFLOPs_per_s": flops_total / (ms * 1e-3) / 1e12,
      "moe_ms": module_ms.get("moe_layers"), "module_ms": module_ms, "stage_ms": stage_ms,
      "expert_mlp_status": mlp_status(kernels),
  }
  if not args.no_cpu_baseline and not short:
    from oracle import moe_oracle as O
    from oracle import vit_oracle as V
    n_img = 8                                  # one routing group
    ocfg = copy.deepcopy(configs.vit_b16_moe_model(dtype=O.BF16))
    to_np = lambda t: t.detach().float().cpu().numpy()

    def tree(t):
      return {k: tree(v) for k, v in t.items()} if isinstance(t, dict) else to_np(t)
    params_np = tree(variables["params"])
    imgs_np = to_np(images[0][:n_img])
    t0 = time.perf_counter()
    V.vision_transformer_moe(imgs_np, params_np, **ocfg)
    t = time.perf_counter() - t0
    result["cpu_baseline"] = {
        "value": n_img / t, "unit": "images/s", "cores": int(torch.get_num_threads()),
        "kind": "port",
        "sample": (f"oracle/vit_oracle.py vision_transformer_moe (bfloat16 rounding modelled) on "
                   f"{n_img} of {B} images (one routing group), one run of {t:.2f} s; NumPy BLAS + "
                   "torch CPU threads"),
        "host_cpus": os.cpu_count(), "cpu_model": host_cpu_model()}
  else:
    result["cpu_baseline"] = None
  return result


def mlp_status(kernels):
  """Status words of the expert MLP's workspace after the run (vmoe_expert_mlp_status):
  pieces of the second product's shared round that gave up a wait, launches that found no
  valid plan.  Anything but zeros means that an output of the run was not the product."""
  st = kernels.expert_mlp_status()
  return None if st is None else {"abandoned_waits": st[0], "plan_mismatches": st[1]}


def sparse_run(args, name, short=False):
  """One sparse MoE layer configuration.  `short`: the timed passes only (no CPU leg, no
  probes, no vendor GEMMs, no graph pass, no reference-layout dispatch pass)."""
  import torch
  from vmoe_amd import _hip, configs, kernels
  from vmoe_amd.nn import vit_moe

  cfg = configs.CONFIGS[name]
  dev = torch.device("cuda:0")
  torch.cuda.set_device(dev)
  tdt = torch.bfloat16 if cfg.dtype == "bfloat16" else torch.float32
  D, M, E, K = cfg.d_model, cfg.mlp_dim, cfg.num_experts, cfg.num_selected_experts
  T, S, G = cfg.num_tokens, cfg.group_size, cfg.num_groups

  # Inputs: tokens and router on the host generator, expert weights on the device one.
  rng = np.random.Generator(np.random.PCG64(0))
  n_rot = 4
  xs_np = []
  for _ in range(n_rot):
    x = rng.standard_normal((cfg.num_images, cfg.tokens_per_image, D), dtype=np.float32)
    if cfg.layer_norm_inputs:
      x = ((x - x.mean(-1, keepdims=True)) / np.sqrt(x.var(-1, keepdims=True) + 1e-6)).astype(np.float32)
    xs_np.append(x)
  router_np = (rng.standard_normal((D, E), dtype=np.float32) / np.sqrt(D)).astype(np.float32)
  bias_np = None
  if cfg.logit_bias_std:
    bias_np = (rng.standard_normal(E, dtype=np.float32) * cfg.logit_bias_std).astype(np.float32)
  w0, w1, b0, b1 = device_weights(cfg, torch, dev, seed=1)
  xs = [torch.from_numpy(x).to(dev).to(tdt) for x in xs_np]
  variables = {"params": {
      "Router": {"dense": {"kernel": torch.from_numpy(router_np).to(dev)}},
      "Mlp": {"Dense_0": {"kernel": w0, "bias": b0}, "Dense_1": {"kernel": w1, "bias": b1}}}}
  router_kwargs = dict(num_selected_experts=K, dispatcher=cfg.dispatcher_kwargs("indices"))
  if bias_np is not None:
    router_kwargs["logit_bias"] = torch.from_numpy(bias_np).to(dev)
  layer = vit_moe.MlpMoeBlock(mlp_dim=M, num_experts=E, group_size=S, deterministic=True,
                              router=router_kwargs, dtype=tdt)

  def step(i):
    return layer.apply(variables, xs[i % n_rot])

  # Untimed: one-time costs (code objects, allocator pools, timing events) and
  # then the W warm-up steps, run exactly as the timed steps are.
  _hip.set_timing_sink({})
  for i in range(COLD_STEPS):
    out, metrics = step(i)
  torch.cuda.synchronize()

  # Timed region: only the dominant entry point (the expert GEMMs) carries timing events.
  # An event between two kernels serialises their hand-over, and eight pairs per step
  # cost the layer about 6 % of its throughput; the other stages are timed in a second,
  # fully instrumented pass of the same K steps right after.
  sink = _hip.TimingSink(pairs=args.steps * 2, only=MLP_CALLS)
  warm_sink = _hip.TimingSink(pairs=(INIT_STEPS + args.warmup) * 2, only=MLP_CALLS)
  # One event per step boundary: the per-step times whose median is reported.
  marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
  for ev in marks:
    ev.record()
  torch.cuda.synchronize()
  # A full collection of Python's cyclic garbage collector fires after a fixed number of
  # allocations and takes tens of milliseconds: it runs here and stays off until the timed
  # loop is over.  Everything that leaves the GPU idle (creating events, this collection)
  # comes before the initialisation and warm-up steps, never between them and the timed
  # steps: after 40 ms of idling the clocks take some twenty steps (25 ms) to come back,
  # which is what the INIT_STEPS in front of the W warm-up steps are for.
  gc.collect()
  gc.disable()
  _hip.set_timing_sink(warm_sink)
  for i in range(INIT_STEPS + args.warmup):
    out, metrics = step(i)
  torch.cuda.synchronize()
  _hip.set_timing_sink(sink)
  trace_marker(kernels, torch, dev)
  t0 = time.perf_counter()
  marks[0].record()
  for i in range(args.steps):
    out, metrics = step(i)
    marks[i + 1].record()
  t_enqueued = time.perf_counter()      # the host has issued everything; the GPU is still running
  trace_marker(kernels, torch, dev)
  torch.cuda.synchronize()
  t1 = time.perf_counter()
  gc.enable()
  _hip.set_timing_sink(None)
  wall_ms_per_step = (t1 - t0) * 1e3 / args.steps
  step_ms = [marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps)]
  ms_per_step = float(np.median(step_ms))
  host_ms_per_step = (t_enqueued - t0) * 1e3 / args.steps
  tokens_per_s = T / (ms_per_step * 1e-3)
  out0 = step(0)[0].float().cpu().numpy() if not (args.no_cpu_baseline or short) else None

  def per_step(pairs_by_name):
    return {name: float(np.mean([a.elapsed_time(b) for a, b in pairs])) * (len(pairs) / args.steps)
            for name, pairs in pairs_by_name.items()}
  full = _hip.TimingSink(pairs=args.steps * CALLS_PER_STEP)
  _hip.set_timing_sink(full)
  for i in range(args.steps):
    step(i)
  torch.cuda.synchronize()
  _hip.set_timing_sink(None)
  stage_ms = merge_mlp_calls(per_step(full))
  stage_ms_instrumented_mlp = stage_ms["vmoe_expert_mlp"]
  stage_ms.update(merge_mlp_calls(per_step(sink)))    # the GEMMs' time is the one of the timed region

  # Kept assignments (rows that carry an item) for the algorithmic flop count.
  gates, val, idx = kernels.gate_topk(xs[0].view(G, S, D), variables["params"]["Router"]["dense"]["kernel"].to(tdt), K,
                                      logit_bias=router_kwargs.get("logit_bias"))
  C = cfg_capacity(cfg)
  _, token_slot, slot_token, fill = kernels.route_assign(val, idx, E, C, cfg.batch_priority)
  kept = int(fill.sum())
  b = 2 if tdt == torch.bfloat16 else 4
  # Dominant kernel: the expert GEMM (two launches per step, 2*A*D*M flops each).
  mlp_ms = stage_ms["vmoe_expert_mlp"]
  gemm_ms = mlp_ms / 2.0
  flops_per_launch = 2.0 * kept * D * M
  achieved_tflops = flops_per_launch / (gemm_ms * 1e-3) / 1e12
  peak = PEAK_BF16_TFLOPS if tdt == torch.bfloat16 else PEAK_FP32_MATRIX_TFLOPS
  roofline = {"bound": "mfma",
              "kernel": "gemm_bf16_mixed_kernel (first product) / gemm_bf16_w8_kernel<0, true, 8> (second product)" if b == 2 else "gemm_f32_dma_kernel<1, 128> (first product) / gemm_f32_dma_kernel<0, 64> (second product)",
              "achieved": achieved_tflops, "peak": peak, "unit": "TFLOP/s",
              "frac": achieved_tflops / peak, "traffic": MEASURED_TRAFFIC_BYTES.get(cfg.name),
              "from_profile": {"traffic_bytes_per_launch": MEASURED_TRAFFIC_BYTES.get(cfg.name),
                               "traffic_source": "profiles/hbm_traffic__vmoe_b16_layer.md",
                               "mfma_busy": MEASURED_MFMA_BUSY.get(cfg.name),
                               "note": "hardware counters from rocprofv3 --pmc runs of this command, "
                                       "not read by this run"} if cfg.name in MEASURED_TRAFFIC_BYTES else None,
              "launch_ms": gemm_ms, "flops_per_launch": flops_per_launch, "kept_rows": kept,
              "buffer_rows": E * G * C}

  # HBM-bound stages, algorithmic bytes (each item row read once, whole buffer written).
  # dispatch: in the bf16 layer the first expert product gathers its rows itself and no
  # dispatch kernel runs inside the step; the kernel (what ExpertIndicesDispatcher.dispatch
  # runs: reference layout, every slot row written, empty ones zeroed) is timed on its own.
  bytes_dispatch = T * D * b + E * G * C * D * b + 8 * T * K
  dispatch_ms = None
  if "vmoe_dispatch" not in stage_ms and (args.no_dispatch_pass or short):
    pass
  elif "vmoe_dispatch" not in stage_ms:
    # the layer through the dispatcher's own dispatch() / combine(), as a caller of the
    # reference API would run it: same kernels before and after it as in the step
    router, mlp = layer._modules()
    p_ = variables["params"]

    def reference_layout_step(i):
      xg = xs[i % n_rot].view(G, S, D)
      dispatcher, _ = router.apply({"params": p_["Router"]}, xg)
      buf = dispatcher.dispatch(xg)
      return dispatcher.combine(mlp.expert.apply_experts({"params": p_["Mlp"]}, buf))
    for i in range(3):
      reference_layout_step(i)
    ref_sink = _hip.TimingSink(pairs=args.steps * CALLS_PER_STEP)
    _hip.set_timing_sink(ref_sink)
    for i in range(args.steps):
      reference_layout_step(i)
    torch.cuda.synchronize()
    _hip.set_timing_sink(None)
    dispatch_ms = per_step(ref_sink)["vmoe_dispatch"]
    stage_ms["vmoe_dispatch (reference-layout pass, not in the step)"] = dispatch_ms
  else:
    dispatch_ms = stage_ms["vmoe_dispatch"]
    bytes_dispatch = T * D * b + kept * D * b + 8 * T * K      # packed: kept rows only
  bytes_combine = kept * D * b + 12 * T * K + T * D * b
  bytes_gate = T * D * b + D * E * b + 12 * T * K + T * E * b
  # Measured copy ceiling of the same device (read + write of 512 MiB).
  n = 512 << 20
  src = torch.empty(n, dtype=torch.uint8, device=dev)
  dst = torch.empty_like(src)
  for _ in range(2):
    kernels.copy_bytes(src, dst)
  e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
  e0.record()
  for _ in range(5):
    kernels.copy_bytes(src, dst)
  e1.record()
  torch.cuda.synchronize()
  copy_gbs = 2 * n * 5 / (e0.elapsed_time(e1) * 1e-3) / 1e9
  del src, dst
  # Measured arithmetic ceiling of the same device: a register-resident MFMA loop
  # on operand fragments taken from the layer's own hidden activations.
  if b == 2 and not short:
    seed = out.reshape(-1)[: 1 << 20].contiguous()
    kernels.mfma_probe(seed, 256, 500)
    e0.record()
    probe_flops = kernels.mfma_probe(seed, 256, 4000)
    e1.record()
    torch.cuda.synchronize()
    roofline["measured_mfma_loop_TFLOPs"] = probe_flops / (e0.elapsed_time(e1) * 1e-3) / 1e12
    roofline["frac_of_measured_loop"] = achieved_tflops / roofline["measured_mfma_loop_TFLOPs"]
  # The vendor library's GEMM on the same two products as dense matrices of the kept
  # rows (torch.nn.functional.linear -> hipBLASLt, no GELU), same run: a reference
  # point for what this part sustains on these shapes.
  if b == 2 and not short:
    a_up = xs[0].reshape(-1, D)[:1].expand(kept, D).contiguous()
    w_up = torch.randn((M, D), device=dev).to(tdt) * D ** -0.5
    a_dn = torch.randn((kept, M), device=dev).to(tdt)
    w_dn = torch.randn((D, M), device=dev).to(tdt) * M ** -0.5
    a_up.copy_(torch.randn((kept, D), device=dev).to(tdt))
    lib = {}
    for name, a_, w_ in (("up", a_up, w_up), ("down", a_dn, w_dn)):
      for _ in range(3):
        torch.nn.functional.linear(a_, w_)
      e0.record()
      for _ in range(10):
        torch.nn.functional.linear(a_, w_)
      e1.record()
      torch.cuda.synchronize()
      lib[name] = 2.0 * kept * D * M * 10 / (e0.elapsed_time(e1) * 1e-3) / 1e12
    roofline["library_gemm_same_shapes_TFLOPs"] = lib
    # The rate at which operand tiles can be moved from global memory into LDS at all,
    # measured by a kernel that issues exactly the DMA requests of a 256 x 256 product and
    # nothing else, on operands of the layer's shape (E experts with their own weights, the
    # kept rows spread evenly over them): with 32-wide k tiles (64-byte row segments per
    # request, as the first product issues them) and with 64-wide ones (128-byte segments,
    # the second product's).  Times the flop per operand byte of a tiling it is the
    # FLOP/s that no kernel of that tiling and request shape can exceed.
    a_e = a_dn[: E * (kept // E)].view(E, kept // E, M)
    w_e = (torch.randn((E, D, M), device=dev) * M ** -0.5).to(tdt)
    delivery = {}
    for name, k_tile, seg, fpb, what in (
        ("segments_64B", 32, 64, 2.0 * 128 * 256 / ((128 + 256) * 2), "32-wide k tiles; flop per byte of 128 x 256 tiles"),
        ("segments_128B", 64, 128, 2.0 * 256 * 256 / ((256 + 256) * 2), "64-wide k tiles; flop per byte of 256 x 256 tiles")):
      for _ in range(3):
        kernels.operand_delivery_probe(a_e, w_e, k_tile=k_tile)
      e0.record()
      for _ in range(10):
        moved = kernels.operand_delivery_probe(a_e, w_e, k_tile=k_tile)
      e1.record()
      torch.cuda.synchronize()
      tbps = moved * 10 / (e0.elapsed_time(e1) * 1e-3) / 1e12
      delivery[name] = {"row_segment_bytes": seg, "TBps": tbps, "tiling": what, "flop_per_byte": fpb,
                        "ceiling_TFLOPs": tbps * fpb}
    # ... and the same kind of requests over tiles that the workgroups share: 64 tiles (201 MB:
    # they stay in L2 and the Infinity Cache, 16 workgroups per tile and launch) and all 188
    # tiles of the buffer (592 MB: more than the caches hold).  What the request path delivers
    # when no request waits for HBM, and what is left when most do.
    flat = a_dn.view(torch.uint8).view(-1)
    for name, seg, tiles in (("cached_128B", 128, 64), ("cached_64B", 64, 64), ("beyond_caches_128B", 128, 188)):
      resident = flat[: tiles * 512 * M * 2]
      for _ in range(3):
        kernels.resident_delivery_probe(resident, M * 2, M * 2 // 128, 4, seg)
      e0.record()
      for _ in range(10):
        moved = kernels.resident_delivery_probe(resident, M * 2, M * 2 // 128, 4, seg)
      e1.record()
      torch.cuda.synchronize()
      delivery[name] = {"row_segment_bytes": seg, "TBps": moved * 10 / (e0.elapsed_time(e1) * 1e-3) / 1e12,
                        "operands": f"{tiles} tiles of 512 rows x {M * 2} bytes shared by 256 workgroups, "
                                    "two k tiles of 64 KB in flight per workgroup"}
    delivery["note"] = ("load-only kernel on 256 x 256 tiles of the second product's operands; the rate depends "
                        "on the shape of the requests, the ceiling on the flop per operand byte of the tiling named; "
                        "the second product requests 128-byte segments, the first product 128-byte segments for its "
                        "weights (two thirds of its requests) and 64-byte ones for its rows; cached_* / beyond_caches_*: "
                        "requests of the same shapes over shared tiles that stay in the caches, or do not: the products' "
                        "own rates lie between them, set by their misses at the depth of their rings")
    roofline["operand_delivery"] = delivery
    del a_up, a_dn, w_up, w_dn, a_e, w_e
  # The same K steps replayed from HIP graphs (one per rotating input buffer), as a
  # serving loop would run the layer; reported beside the eager figure, never as `value`.
  graph_ms = None
  graph_many_ms = None
  try:
    if short:
      raise StopIteration
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
      for i in range(n_rot):
        step(i)
    torch.cuda.current_stream().wait_stream(side)
    graphs, keep = [], []
    for i in range(n_rot):
      g_ = torch.cuda.CUDAGraph()
      with torch.cuda.graph(g_):
        keep.append(step(i))
      graphs.append(g_)
    for i in range(args.warmup):
      graphs[i % n_rot].replay()
    torch.cuda.synchronize()
    tg0 = time.perf_counter()
    for i in range(args.steps):
      graphs[i % n_rot].replay()
    torch.cuda.synchronize()
    graph_ms = (time.perf_counter() - tg0) * 1e3 / args.steps
    if not torch.equal(keep[(args.steps - 1) % n_rot][0], step(args.steps - 1)[0]):
      raise RuntimeError("graph replay and eager step disagree")
    del graphs, keep
    # One graph that holds n_rot steps: what a replay costs at its boundaries shows as the
    # difference between this figure and the one above.
    many = torch.cuda.CUDAGraph()
    with torch.cuda.graph(many):
      keep = [step(i) for i in range(n_rot)]
    for _ in range(max(1, args.warmup // n_rot)):
      many.replay()
    torch.cuda.synchronize()
    reps = max(1, args.steps // n_rot)
    tg0 = time.perf_counter()
    for _ in range(reps):
      many.replay()
    torch.cuda.synchronize()
    graph_many_ms = (time.perf_counter() - tg0) * 1e3 / (reps * n_rot)
    del many, keep
  except StopIteration:
    pass
  except Exception as e:   # pylint: disable=broad-except
    print(f"bench.py: HIP graph pass skipped: {e}", file=sys.stderr)
    graph_ms = None
  hbm = {
      "dispatch_GBps": bytes_dispatch / (dispatch_ms * 1e-3) / 1e9 if dispatch_ms else None,
      "combine_GBps": bytes_combine / (stage_ms["vmoe_combine"] * 1e-3) / 1e9,
      "gate_topk_GBps": bytes_gate / (stage_ms["vmoe_gate_topk"] * 1e-3) / 1e9,
      "copy_kernel_GBps": copy_gbs, "peak_GBps": PEAK_HBM_GBS,
  }
  hbm["dispatch_frac_of_peak"] = hbm["dispatch_GBps"] / PEAK_HBM_GBS if dispatch_ms else None
  hbm["combine_frac_of_peak"] = hbm["combine_GBps"] / PEAK_HBM_GBS

  result = {
      "metric": ("MoE-layer tokens/sec at B/16 E=32 k=2 bf16; dispatch/combine HBM GB/s" if cfg.name == HEADLINE
                 else f"MoE-layer tokens/sec, {cfg.name}"),
      "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
      "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
      "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if b == 2 else "f32",
      "data": "synthetic (seeded N(0,1) tokens, LayerNorm-ed; LeCun-normal experts; random-init router)",
      "config": {"workload": cfg.name, "tokens": T, "d_model": D, "mlp_dim": M, "experts": E,
                 "selected": K, "groups": G, "group_size": S, "capacity": C,
                 "batch_priority": cfg.batch_priority, "capacity_factor": cfg.capacity_factor},
      "roofline": roofline,
      "stage_ms": stage_ms,
      "stage_ms_note": ("vmoe_expert_mlp: events in the timed region; other stages: second pass of "
                        "the same steps with events around every call (its vmoe_expert_mlp read "
                        f"{stage_ms_instrumented_mlp:.4f} ms)"),
      "hbm": hbm,
      "hip_graph_ms_per_step": graph_ms,
      "hip_graph_ms_per_step_four_steps_per_graph": graph_many_ms,
      "host_enqueue_ms_per_step": host_ms_per_step,
      "wall_ms_per_step": wall_ms_per_step,
      "ms_per_step_note": ("ms_per_step and value: median of the K per-step times between events "
                           "recorded at the step boundaries; wall_ms_per_step: host clock around "
                           "the same K steps, synchronised on both sides, divided by K"),
      "step_ms_min_max": [float(min(step_ms)), float(max(step_ms))],
      "step_ms_p10_p50_p90": [float(np.percentile(step_ms, q)) for q in (10, 50, 90)],
      "step_ms_first_five": [float(v) for v in step_ms[:5]],
      "untimed_steps_before_warmup": COLD_STEPS + INIT_STEPS,
      "expert_mlp_status": mlp_status(kernels),
  }
  if not args.no_cpu_baseline and not short:
    params_np = {
        "Router": {"dense": {"kernel": router_np}},
        "Mlp": {"Dense_0": {"kernel": w0.float().cpu().numpy(), "bias": b0.float().cpu().numpy()},
                "Dense_1": {"kernel": w1.float().cpu().numpy(), "bias": b1.float().cpu().numpy()}}}
    parity, result["cpu_baseline"] = cpu_baseline(cfg, xs_np[0], params_np, bias_np,
                                                  min(args.cpu_groups, G), gpu_out=out0)
    result["parity_checked"] = parity
  else:
    result["cpu_baseline"] = None
    result["parity_checked"] = None
  return result


SOFT_NAME = "soft_moe_b16_128x1"
MODEL_NAME = "vmoe_b16_model_E8_k2_224"
HEADLINE = "vmoe_b16_layer_E32_k2_bpr"
# The other BASELINE configurations, run as short passes behind the headline one.
OTHER_WORKLOADS = ("vmoe_s32_layer", "vmoe_l16_384_layer_cf0.5", SOFT_NAME, MODEL_NAME)


def run_config(args, name, short=False):
  if name == SOFT_NAME:
    return soft_run(args, short)
  if name == MODEL_NAME:
    return vit_run(args, short)
  return sparse_run(args, name, short)


def other_workloads(args):
  """Short passes (OTHER_WARMUP warm-up steps behind the initialisation steps, OTHER_STEPS
  timed steps, no CPU leg) of the BASELINE configurations that are not the headline one."""
  import copy
  import torch
  short_args = copy.copy(args)
  short_args.steps, short_args.warmup = OTHER_STEPS, OTHER_WARMUP
  out = []
  for name in OTHER_WORKLOADS:
    gc.collect()
    torch.cuda.empty_cache()
    try:
      r = run_config(short_args, name, short=True)
    except Exception as e:   # pylint: disable=broad-except
      out.append({"workload": name, "error": f"{type(e).__name__}: {e}"})
      continue
    roof = r["roofline"]
    entry = {"workload": r["config"]["workload"], "metric": r["metric"], "ms_per_step": r["ms_per_step"],
             "value": r["value"], "unit": r["unit"], "dtype": r["dtype"], "steps": r["steps"],
             "warmup": r["warmup"],
             "roofline": {k: roof.get(k) for k in ("bound", "kernel", "achieved", "peak", "unit", "frac", "launch_ms")},
             "kept_rows": roof.get("kept_rows", roof.get("kept_rows_per_moe_block")),
             "stage_ms": r.get("stage_ms"), "expert_mlp_status": r.get("expert_mlp_status")}
    if "moe_ms" in r:
      entry["moe_ms"] = r["moe_ms"]
    if "hbm" in r:
      entry["hbm"] = {k: r["hbm"][k] for k in ("combine_GBps", "gate_topk_GBps", "copy_kernel_GBps")}
    out.append(entry)
  return out


def main():
  args = parse_args()
  if args.gpus != 1:
    print("bench.py: this build runs on ONE GPU (all experts resident, no collectives); "
          f"--gpus {args.gpus} is not supported.", file=sys.stderr)
    sys.exit(2)
  result = run_config(args, args.config)
  if args.config == HEADLINE and not args.no_other_workloads:
    result["other_workloads"] = other_workloads(args)
  print(json.dumps(result))
  st = result.get("expert_mlp_status")
  if st and (st["abandoned_waits"] or st["plan_mismatches"]):
    print(f"bench.py: the expert MLP's status words are not zero: {st}", file=sys.stderr)
    sys.exit(1)
  parity = result.get("parity_checked")
  if parity and parity["bad"] > parity["allowed_bad_fraction"] * parity["items"]:
    print(f"bench.py: the timed path's output differs from the oracle on {parity['bad']} of "
          f"{parity['items']} items", file=sys.stderr)
    sys.exit(1)


def cfg_capacity(cfg):
  from vmoe_amd import moe
  return moe.compute_capacity(cfg.group_size * cfg.num_selected_experts, cfg.num_experts,
                              cfg.capacity_factor)


if __name__ == "__main__":
  main()
