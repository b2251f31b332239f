"""Small host utilities mirroring the parts of vmoe/utils.py the MoE layer uses."""
from __future__ import annotations

import ast
import importlib
from typing import Any, Dict, Tuple


def parse_call(expr: str, default_module) -> Tuple[Any, Tuple, Dict[str, Any]]:
  """Resolves ``"Name"``, ``"pkg.mod.Name"`` or ``"Name(arg, k=v)"`` to
  (callable, args, kwargs), looking bare names up in ``default_module``
  (vmoe/utils.py:59-109).  Arguments must be Python literals."""
  node = ast.parse(expr.strip(), mode="eval").body
  args, kwargs = (), {}
  if isinstance(node, ast.Call):
    args = tuple(ast.literal_eval(a) for a in node.args)
    kwargs = {k.arg: ast.literal_eval(k.value) for k in node.keywords}
    node = node.func
  parts = []
  while isinstance(node, ast.Attribute):
    parts.append(node.attr)
    node = node.value
  if not isinstance(node, ast.Name):
    raise ValueError(f"Cannot parse {expr!r}")
  parts.append(node.id)
  parts.reverse()
  if len(parts) == 1:
    return getattr(default_module, parts[0]), args, kwargs
  module = importlib.import_module(".".join(parts[:-1]))
  return getattr(module, parts[-1]), args, kwargs
