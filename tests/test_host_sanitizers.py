"""The routing kernels' index arithmetic (vmoe_amd/csrc/route_index.h: sort keys, bitmap
positions, slot rows, packed rows, launch-plan entries -- the scalar functions the device
threads call) built as plain C++ for the host and run under AddressSanitizer and
UndefinedBehaviorSanitizer on a seeded sweep of shapes, against the sequential C statement
of the assignment (oracle/route_greedy.c).  An index that leaves a buffer aborts the run."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "host_build")


@pytest.fixture(scope="module")
def checker():
  if shutil.which("g++") is None or shutil.which("make") is None:
    pytest.skip("no host C++ toolchain")
  r = subprocess.run(["make", "-B", "-C", HERE], capture_output=True, text=True)
  assert r.returncode == 0, r.stdout + r.stderr
  return os.path.join(HERE, "_build", "route_host_check")


@pytest.mark.parametrize("seed", [2024, 7])
def test_routing_index_arithmetic_under_sanitizers(checker, seed):
  env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:verify_asan_link_order=0",
             UBSAN_OPTIONS="print_stacktrace=1")
  r = subprocess.run([checker, str(seed)], capture_output=True, text=True, env=env, timeout=600)
  assert r.returncode == 0, (r.stdout + r.stderr)[-4000:]
  assert "0 failures" in r.stdout
