"""`--export input|output|both --export-dir DIR`: dumps a run's tensors for comparing backends
or machines offline. File names follow tritonbench/components/export/export.py:19-50
(`x_<x_val>-input`, `x_<x_val>-<backend>-fwd-output`); the payload is written with torch.save
(tensors moved to the CPU, fp8 tensors kept as such) under the extension `.pt`."""
import os
from typing import Any, Callable

import torch


def _to_cpu(obj: Any) -> Any:
    if isinstance(obj, torch.Tensor):
        return obj.detach().cpu()
    if isinstance(obj, (list, tuple)):
        return type(obj)(_to_cpu(o) for o in obj)
    if isinstance(obj, dict):
        return {k: _to_cpu(v) for k, v in obj.items()}
    return obj


def _x_name(x_val: Any) -> str:
    return str(x_val).replace(" ", "")


def export_input(x_val: Any, inputs: Any, export_dir: str) -> str:
    if not export_dir or not os.path.isdir(export_dir):
        raise RuntimeError(f"export dir {export_dir!r} must exist")
    path = os.path.join(export_dir, f"x_{_x_name(x_val)}-input.pt")
    torch.save(_to_cpu(inputs), path)
    return path


def export_output(x_val: Any, fn_name: str, fn_mode: str, fn: Callable, export_dir: str) -> str:
    if not export_dir or not os.path.isdir(export_dir):
        raise RuntimeError(f"export dir {export_dir!r} must exist")
    if fn_mode != "fwd":
        raise NotImplementedError("only forward outputs are exported")
    out = fn()
    if getattr(out, "is_cuda", False):
        torch.cuda.synchronize()
    path = os.path.join(export_dir, f"x_{_x_name(x_val)}-{fn_name}-fwd-output.pt")
    torch.save(_to_cpu(out), path)
    return path
