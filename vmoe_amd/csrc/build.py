"""Builds libvmoe_hip.so for gfx950 with hipcc (run: python -m vmoe_amd.csrc.build)."""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT_DIR = os.path.join(os.path.dirname(HERE), "_lib")
LIB = os.path.join(OUT_DIR, "libvmoe_hip.so")
SOURCES = ["capi.hip", "gate_topk.hip", "route_assign.hip", "dispatch_combine.hip",
           "expert_mlp.hip", "soft_moe.hip", "vit_ops.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument",
         "-I", os.path.join(ROOT, "include"), "-I", HERE]


def _hipcc() -> str:
  for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
    if cand and (os.path.sep not in cand or os.path.exists(cand)):
      return cand
  raise RuntimeError("hipcc not found")


def _compile(src: str) -> str:
  obj = os.path.join(OUT_DIR, "obj", src.replace(".hip", ".o"))
  cmd = [_hipcc(), *FLAGS, "-c", os.path.join(HERE, src), "-o", obj]
  r = subprocess.run(cmd, capture_output=True, text=True)
  if r.returncode != 0:
    raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr}")
  noise = "is not a recognized feature"
  err = "\n".join(l for l in r.stderr.splitlines() if noise not in l and l.strip())
  if err:
    sys.stderr.write(err + "\n")
  return obj


def build(verbose: bool = True) -> str:
  """Compiles every HIP source and links the shared library. Always recompiles."""
  os.makedirs(os.path.join(OUT_DIR, "obj"), exist_ok=True)
  with concurrent.futures.ThreadPoolExecutor(max_workers=min(6, os.cpu_count() or 1)) as ex:
    objs = list(ex.map(_compile, SOURCES))
  cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
  r = subprocess.run(cmd, capture_output=True, text=True)
  if r.returncode != 0:
    raise RuntimeError(f"link failed:\n{r.stderr}")
  if verbose:
    print(f"built {LIB}")
  return LIB


if __name__ == "__main__":
  build()
