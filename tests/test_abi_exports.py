"""CPU-side checks of the drop-in boundary: the shared library loads, exports
every symbol declared in include/vmoe_hip.h, and the ctypes structs match the
header's layout.  No compute call is made (there may be no GPU)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "vmoe_hip.h")


def _declared_functions():
  text = open(HEADER).read()
  text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
  return sorted(set(re.findall(r"\b(vmoe_[a-z0-9_]+)\s*\(", text)))


def _lib():
  from vmoe_amd import _hip
  if not os.path.exists(_hip.lib_path()):
    from vmoe_amd.csrc import build
    build.build(verbose=False)
  return ctypes.CDLL(_hip.lib_path())


def test_header_functions_are_exported():
  lib = _lib()
  names = _declared_functions()
  assert len(names) >= 18
  for n in names:
    assert hasattr(lib, n), f"{n} declared in vmoe_hip.h but not exported"


def test_python_export_list_matches_header():
  from vmoe_amd import _hip
  assert sorted(_hip.EXPORTS) == _declared_functions()


def test_version_and_error_strings():
  lib = _lib()
  assert lib.vmoe_abi_version() == 1
  lib.vmoe_error_string.restype = ctypes.c_char_p
  assert lib.vmoe_error_string(0) == b"ok"
  for code in range(-7, 0):
    assert lib.vmoe_error_string(code) != b"unknown vmoe error"


def test_struct_layouts_match_header():
  """Field order/types of each ctypes struct follow the header's typedef."""
  from vmoe_amd import _hip
  text = open(HEADER).read()
  text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
  structs = {n: b for b, n in re.findall(r"typedef struct \{(.*?)\}\s*(\w+);", text, flags=re.S)}
  cmap = {"int32_t": ctypes.c_int32, "float": ctypes.c_float, "size_t": ctypes.c_size_t,
          "int64_t": ctypes.c_int64}
  py = {"VmoeGateTopkParams": _hip.GateTopkParams, "VmoeTopkParams": _hip.TopkParams,
        "VmoeRouterMetricsParams": _hip.RouterMetricsParams,
        "VmoeRouteAssignParams": _hip.RouteAssignParams,
        "VmoeIndicesToSlotsParams": _hip.IndicesToSlotsParams,
        "VmoeDispatchParams": _hip.DispatchParams, "VmoeCombineParams": _hip.CombineParams,
        "VmoeDensifyParams": _hip.DensifyParams, "VmoeExpertMlpParams": _hip.ExpertMlpParams,
        "VmoeTransposeParams": _hip.TransposeParams, "VmoeSoftRouteParams": _hip.SoftRouteParams,
        "VmoeEinsumParams": _hip.EinsumParams, "VmoeCastParams": _hip.CastParams,
        "VmoeTopItemsParams": _hip.TopItemsParams,
        "VmoeAddLayerNormParams": _hip.AddLayerNormParams,
        "VmoeAttentionParams": _hip.AttentionParams,
        "VmoeNoisyGatesParams": _hip.NoisyGatesParams,
        "VmoeCompactRowsParams": _hip.CompactRowsParams,
        "VmoeCombineBackwardParams": _hip.CombineBackwardParams,
        "VmoeSoftStatsParams": _hip.SoftStatsParams}
  assert set(py) == set(structs)
  for name, body in structs.items():
    want = []
    for decl in body.split(";"):
      decl = decl.strip()
      if not decl:
        continue
      m = re.match(r"(const\s+)?(\w+)\s*(\*?)\s*(.*)", decl)
      base, star, names = m.group(2), m.group(3), m.group(4)
      for nm in names.split(","):
        nm = nm.strip()
        is_ptr = bool(star) or nm.startswith("*")
        want.append(ctypes.c_void_p if is_ptr else cmap[base])
    got = [t for _, t in py[name]._fields_]
    assert got == want, name


def test_null_params_are_rejected_without_a_gpu():
  lib = _lib()
  for fn in ("vmoe_gate_topk", "vmoe_route_assign", "vmoe_dispatch", "vmoe_combine",
             "vmoe_expert_mlp", "vmoe_soft_route", "vmoe_einsum_dispatch", "vmoe_cast"):
    assert getattr(lib, fn)(None, None) == -1


def _params_entry_points():
  """(function name, struct name) of every `int vmoe_x(const VmoeXParams* p, vmoe_stream_t)`."""
  text = open(HEADER).read()
  text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
  return sorted(set(re.findall(r"\bint\s+(vmoe_[a-z0-9_]+)\s*\(\s*const\s+(Vmoe\w+Params)\s*\*\s*\w+\s*,\s*vmoe_stream_t", text)))


def test_entry_points_reject_null_and_empty_params():
  """Argument checks run before any device call: a null parameter block and an all-zero
  one (null buffers, zero sizes) come back as negative VMOE_E_* codes.  Nothing is
  launched, so this runs without a GPU."""
  from vmoe_amd import _hip
  lib = _lib()
  lib.vmoe_error_string.restype = ctypes.c_char_p
  by_name = {"Vmoe" + cls.__name__: cls for cls in vars(_hip).values()
             if isinstance(cls, type) and issubclass(cls, ctypes.Structure)}
  entries = _params_entry_points()
  assert len(entries) >= 20
  for fn_name, struct_name in entries:
    fn = getattr(lib, fn_name)
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    rc = fn(None, None)
    assert rc < 0, f"{fn_name}(NULL) returned {rc}"
    assert lib.vmoe_error_string(rc) != b"unknown vmoe error"
    zeroed = by_name[struct_name]()
    rc = fn(ctypes.byref(zeroed), None)
    assert rc < 0, f"{fn_name}(zeroed {struct_name}) returned {rc}"


def test_two_block_entry_point_rejects_null():
  from vmoe_amd import _hip
  lib = _lib()
  fn = lib.vmoe_route_assign_metrics
  fn.restype = ctypes.c_int
  fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
  assert fn(None, None, None) < 0
  assert fn(ctypes.byref(_hip.RouteAssignParams()), ctypes.byref(_hip.RouterMetricsParams()), None) < 0


# ------------------------------------------------------------------ the jax.ffi shim (source only)
FFI_SOURCE = os.path.join(ROOT, "vmoe_amd", "csrc", "ffi", "vmoe_xla_ffi.cc")


def _camel(name: str) -> str:
  return "".join(part.capitalize() for part in name.split("_"))


def test_xla_ffi_shim_covers_every_entry_point():
  """The XLA FFI shim cannot be compiled here (no jaxlib headers), so its coverage is
  checked on the text: every entry point of the header that takes a parameter block has
  a handler symbol (the entry point's name in CamelCase) whose implementation calls it,
  and every field of every parameter block is assigned somewhere in the shim."""
  header = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
  shim = open(FFI_SOURCE).read()
  code = re.sub(r"//[^\n]*", "", shim)
  entry_points = [(f, s_) for f, s_ in re.findall(
      r"\bint\s+(vmoe_[a-z0-9_]+)\s*\(\s*const\s+(Vmoe\w+Params)\s*\*", header)
                  if f != "vmoe_expert_mlp_status"]      # no launch: the MLP handlers call it themselves
  assert len(entry_points) >= 24
  assert len(re.findall(r"\bCopyStatus\(stream, p, status\)", code)) == 3, "every MLP handler returns the status words"
  assert re.search(r"\bvmoe_expert_mlp_status\s*\(\s*&", code)
  # the fused custom call falls back to the two-launch compaction where the one-launch form does not exist
  fused = code[code.index("CompactRowsPlannedImpl("):code.index("XLA_FFI_DEFINE_HANDLER_SYMBOL(VmoeCompactRowsPlanned")]
  assert "VMOE_E_UNSUPPORTED" in fused and "vmoe_compact_rows(&c" in fused and "vmoe_expert_mlp(&p" in fused
  handlers = set(re.findall(r"XLA_FFI_DEFINE_HANDLER_SYMBOL\(\s*(\w+)\s*,", code))
  for fn, _ in entry_points:
    assert _camel(fn) in handlers, f"no XLA FFI handler symbol {_camel(fn)} for {fn}"
    assert re.search(rf"\b{fn}\s*\(\s*&", code), f"the shim never calls {fn}"
  assert len(handlers) == len(entry_points), sorted(handlers - {_camel(f) for f, _ in entry_points})
  structs = {n: b for b, n in re.findall(r"typedef struct \{(.*?)\}\s*(\w+);", header, flags=re.S)}
  for _, struct in set(entry_points):
    for field in re.findall(r"(\w+)\s*(?:,|;)", re.sub(r"\[[^\]]*\]", "", structs[struct])):
      if field in ("int32_t", "float", "size_t", "int64_t"):
        continue
      assert re.search(rf"(?:\.|->){field}\s*=", code), f"{struct}.{field} is never set in the shim"
  # the registration loop of the integration guide names the same handlers
  doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
  for fn, _ in entry_points:
    assert fn in doc, f"{fn} is not mentioned in INTEGRATION.md"
