"""Operator discovery: every directory under tritonbench_amd/operators/ that holds an
__init__.py is an operator, its module exports `Operator`
(the contract of tritonbench/operators/op.py:27-78)."""
import importlib
import os
from typing import List

_OPS_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "operators")
_OPS_PKG = "tritonbench_amd.operators"


def list_operators() -> List[str]:
    return sorted(
        d for d in os.listdir(_OPS_DIR)
        if os.path.isfile(os.path.join(_OPS_DIR, d, "__init__.py")) and not d.startswith("_")
    )


def load_opbench_by_name(op_name: str):
    matches = [o for o in list_operators() if o.lower() == op_name.lower()]
    if not matches:
        raise RuntimeError(f"{op_name} is not found in the operator list: {list_operators()}")
    if len(matches) > 1:
        raise RuntimeError(f"found more than one operator named {op_name}: {matches}")
    module = importlib.import_module(f"{_OPS_PKG}.{matches[0]}")
    cls = getattr(module, "Operator", None)
    if cls is None:
        raise RuntimeError(f"{_OPS_PKG}.{matches[0]} does not export Operator")
    cls.name = matches[0]
    return cls
