"""PyTorch-facing wrappers around the C ABI. PyTorch supplies device memory and the
current stream; all arithmetic happens in the HIP library."""
from typing import Callable, Optional, Tuple

import torch

from . import _lib

FP8_DTYPE = torch.float8_e4m3fn
E4M3_MAX_POS = 448.0


def _require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            f"{name} is on {t.device}: the MI355X backend only runs on a ROCm device "
            "(there is no CPU fallback)"
        )
    _lib.init_device(t.device.index if t.device.index is not None else torch.cuda.current_device())


def _stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


def select_variant(m: int, n: int, k: int) -> int:
    v = _lib.load().mi355x_fp8_rowwise_select_variant(m, n, k)
    if v < 0:
        _lib.check(v, "select_variant")
    return v


def gemm_workspace(m: int, n: int, k: int, device, variant: int = _lib.VARIANT_AUTO) -> Optional[torch.Tensor]:
    """Device workspace the plan for this shape wants (fp32 split-K partial sums), or None.
    Allocate it once and pass it as `workspace=` to keep allocation out of repeated calls."""
    nbytes = _lib.load().mi355x_fp8_rowwise_workspace_bytes(m, n, k, variant)
    return torch.empty(nbytes, dtype=torch.uint8, device=device) if nbytes else None


def fp8_gemm_rowwise(
    xq: torch.Tensor,
    wq: torch.Tensor,
    x_scale: torch.Tensor,
    w_scale: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
    variant: int = _lib.VARIANT_AUTO,
    workspace: Optional[torch.Tensor] = None,
    out_dtype: torch.dtype = torch.bfloat16,
) -> torch.Tensor:
    """[M,N] = ((xq @ wq.T) * x_scale[:,None] * w_scale[None,:] + bias) in bfloat16 (default)
    or float16 (`out_dtype`).

    Same operands as the callables of tritonbench/operators/fp8_gemm_rowwise/operator.py:187-217:
    xq [M,K] and wq [N,K] float8_e4m3fn, x_scale [M] and w_scale [N] float32, bias [N]
    bfloat16 or None. Only enqueues work on the current stream (graph-capturable). Shapes
    whose plan splits K need a workspace: pass one from gemm_workspace(), or leave it to this
    call (a torch.empty per call; too small a workspace makes the library run a plan that
    needs none).
    """
    lib = _lib.load()
    for t, name in ((xq, "xq"), (wq, "wq"), (x_scale, "x_scale"), (w_scale, "w_scale")):
        _require_gpu(t, name)
    if xq.dtype != FP8_DTYPE or wq.dtype != FP8_DTYPE:
        raise TypeError(f"xq and wq must be {FP8_DTYPE}, got {xq.dtype} and {wq.dtype}")
    if xq.dim() != 2 or wq.dim() != 2 or xq.shape[1] != wq.shape[1]:
        raise ValueError(f"expected xq [M,K] and wq [N,K], got {tuple(xq.shape)} and {tuple(wq.shape)}")
    m, k = xq.shape
    n = wq.shape[0]
    if x_scale.dtype != torch.float32 or w_scale.dtype != torch.float32:
        raise TypeError("x_scale and w_scale must be float32")
    if x_scale.numel() != m or w_scale.numel() != n:
        raise ValueError("x_scale must have M entries and w_scale N entries")
    if xq.stride(1) != 1 or wq.stride(1) != 1:
        raise ValueError("xq and wq must be K-contiguous")
    if not x_scale.is_contiguous() or not w_scale.is_contiguous():
        raise ValueError("scales must be contiguous")
    bias_ptr = None
    if bias is not None:
        _require_gpu(bias, "bias")
        if bias.dtype != torch.bfloat16 or bias.numel() != n or not bias.is_contiguous():
            raise ValueError("bias must be a contiguous bfloat16 vector of N entries")
        bias_ptr = bias.data_ptr()
    if out_dtype not in (torch.bfloat16, torch.float16):
        raise TypeError(f"out_dtype must be bfloat16 or float16, got {out_dtype}")
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=xq.device)
    else:
        _require_gpu(out, "out")
        if out.dtype != out_dtype or tuple(out.shape) != (m, n) or out.stride(1) != 1:
            raise ValueError(f"out must be {out_dtype} [M,N] with unit column stride")
    if workspace is not None:
        _require_gpu(workspace, "workspace")
        if not workspace.is_contiguous():
            raise ValueError("workspace must be contiguous")
        ws, ws_bytes = workspace, workspace.numel() * workspace.element_size()
    else:
        ws_bytes = lib.mi355x_fp8_rowwise_workspace_bytes(m, n, k, variant)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=xq.device) if ws_bytes else None
    st = lib.mi355x_fp8_rowwise_gemm_ex(
        xq.data_ptr(), wq.data_ptr(), x_scale.data_ptr(), w_scale.data_ptr(), bias_ptr,
        out.data_ptr(), _lib.OUT_F16 if out_dtype == torch.float16 else _lib.OUT_BF16,
        m, n, k, xq.stride(0), wq.stride(0), out.stride(0),
        ws.data_ptr() if ws is not None else None, ws_bytes, variant, _stream_ptr(),
    )
    _lib.check(st, "mi355x_fp8_rowwise_gemm")
    return out


def fp8_gemm_rowwise_clocks(xq, wq, x_scale, w_scale, out, workspace=None, variant: int = _lib.VARIANT_AUTO) -> Optional[dict]:
    """One launch of fp8_gemm_rowwise through mi355x_fp8_rowwise_gemm_stamped, read back: what the
    launch took in shader cycles and at which clock every XCD ran it (workgroup g runs on XCD g % 8;
    each XCD has a clock of its own). Returns None when the plan is not of the tiled family (only
    that one records readings). Synchronises; for benchmarks, outside their timed regions."""
    lib = _lib.load()
    for t, name in ((xq, "xq"), (wq, "wq"), (x_scale, "x_scale"), (w_scale, "w_scale"), (out, "out")):
        _require_gpu(t, name)
    m, k = xq.shape
    n = wq.shape[0]
    stamps = torch.zeros(_lib.STAMP_ENTRIES, dtype=torch.int64, device=xq.device)
    ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
    st = lib.mi355x_fp8_rowwise_gemm_stamped(
        xq.data_ptr(), wq.data_ptr(), x_scale.data_ptr(), w_scale.data_ptr(), None, out.data_ptr(),
        m, n, k, xq.stride(0), wq.stride(0), out.stride(0),
        workspace.data_ptr() if workspace is not None else None, ws_bytes, variant,
        stamps.data_ptr(), _lib.STAMP_ENTRIES, _stream_ptr(),
    )
    _lib.check(st, "mi355x_fp8_rowwise_gemm_stamped")
    torch.cuda.synchronize()
    t = stamps.cpu().view(-1, 4)
    t = t[t[:, 0] != 0]
    if t.numel() == 0:
        return None
    groups = torch.nonzero(stamps.cpu().view(-1, 4)[:, 0] != 0).flatten()
    cycles = (t[:, 1] - t[:, 0]).double()
    ticks = (t[:, 3] - t[:, 2]).double()          # 100 MHz
    ghz = cycles / (ticks * 10.0)
    per_xcd = [float(ghz[(groups % 8) == x].mean()) for x in range(8) if bool(((groups % 8) == x).any())]
    return {
        "workgroups": int(t.shape[0]),
        "cycles_per_workgroup_mean": float(cycles.mean()),
        "cycles_per_workgroup_max": float(cycles.max()),
        "span_us": float((t[:, 3].max() - t[:, 2].min()).item()) / 100.0,
        "xcd_clock_ghz": [round(v, 4) for v in per_xcd],
        "clock_ghz_mean": float(ghz.mean()),
        "clock_ghz_min_xcd": min(per_xcd),
        "clock_ghz_max_xcd": max(per_xcd),
    }


def fp8_gemm_tensorwise(
    a: torch.Tensor,
    b: torch.Tensor,
    scale_a: torch.Tensor,
    scale_b: torch.Tensor,
    out_dtype: torch.dtype = torch.float16,
    out: Optional[torch.Tensor] = None,
) -> Callable[[], torch.Tensor]:
    """Tensor-wise scaled product with the operands of torch._scaled_mm as the reference's
    fp8_gemm operator passes them (tritonbench/operators/fp8_gemm/fp8_gemm.py:57-101):
    a [M,K] row-major, b [K,N] column-major (b.T is [N,K] K-contiguous), scale_a and scale_b
    one-element float32 DEVICE tensors (or [M,1] / [1,N] for its row-wise flag). Returns a
    zero-argument callable; the scalars are spread into vectors on the device here, once,
    outside the callable, and never read by the host."""
    if b.dim() != 2 or b.stride(0) != 1:
        raise ValueError("b must be [K,N] column-major (b.T contiguous), as torch._scaled_mm wants it")
    m, n = a.shape[0], b.shape[1]
    xs = scale_a.to(torch.float32).reshape(-1).expand(m).contiguous() if scale_a.numel() == 1 else scale_a.reshape(-1).contiguous()
    ws = scale_b.to(torch.float32).reshape(-1).expand(n).contiguous() if scale_b.numel() == 1 else scale_b.reshape(-1).contiguous()
    wq = b.t()
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=a.device)
    space = gemm_workspace(m, n, a.shape[1], a.device)
    return lambda: fp8_gemm_rowwise(a, wq, xs, ws, out=out, workspace=space, out_dtype=out_dtype)


def fp8_gemm_rowwise_grouped(
    group_a: torch.Tensor,
    group_b: torch.Tensor,
    m_sizes: torch.Tensor,
    a_scale: torch.Tensor,
    b_scale: torch.Tensor,
    out: Optional[torch.Tensor] = None,
    tile_config: int = -1,
) -> torch.Tensor:
    """Grouped row-wise FP8 GEMM: bf16 [M,N], rows of group g = group_a rows of that group times
    group_b[g*N:(g+1)*N].T, scaled row- and column-wise.

    Same operands as the callables of
    tritonbench/operators/fp8_gemm_rowwise_grouped/operator.py:400-455: group_a [M,K] and
    group_b [G*N,K] float8_e4m3fn, m_sizes int32 [G] ON THE DEVICE (never read by the host),
    a_scale [M] and b_scale [G*N] float32. Rows past sum(m_sizes) keep what `out` held
    (zeros when this call allocates it). Only enqueues work on the current stream.
    """
    lib = _lib.load()
    for t, name in ((group_a, "group_a"), (group_b, "group_b"), (m_sizes, "m_sizes"), (a_scale, "a_scale"),
                    (b_scale, "b_scale")):
        _require_gpu(t, name)
    if group_a.dtype != FP8_DTYPE or group_b.dtype != FP8_DTYPE:
        raise TypeError(f"group_a and group_b must be {FP8_DTYPE}")
    if group_a.dim() != 2 or group_b.dim() != 2 or group_a.shape[1] != group_b.shape[1]:
        raise ValueError("expected group_a [M,K] and group_b [G*N,K]")
    if m_sizes.dtype != torch.int32 or m_sizes.dim() != 1 or not m_sizes.is_contiguous() or m_sizes.numel() < 1:
        raise ValueError("m_sizes must be a contiguous int32 vector with one entry per group")
    g = m_sizes.numel()
    m, k = group_a.shape
    if group_b.shape[0] % g:
        raise ValueError(f"group_b has {group_b.shape[0]} rows, not a multiple of the {g} groups")
    n = group_b.shape[0] // g
    if a_scale.dtype != torch.float32 or b_scale.dtype != torch.float32:
        raise TypeError("a_scale and b_scale must be float32")
    if a_scale.numel() != m or b_scale.numel() != g * n or not a_scale.is_contiguous() or not b_scale.is_contiguous():
        raise ValueError("a_scale must have M entries and b_scale G*N entries, both contiguous")
    if group_a.stride(1) != 1 or group_b.stride(1) != 1:
        raise ValueError("group_a and group_b must be K-contiguous")
    if out is None:
        out = torch.zeros((m, n), dtype=torch.bfloat16, device=group_a.device)
    else:
        _require_gpu(out, "out")
        if out.dtype != torch.bfloat16 or tuple(out.shape) != (m, n) or out.stride(1) != 1:
            raise ValueError("out must be bfloat16 [M,N] with unit column stride")
    st = lib.mi355x_fp8_rowwise_grouped_gemm(
        group_a.data_ptr(), group_b.data_ptr(), a_scale.data_ptr(), b_scale.data_ptr(), m_sizes.data_ptr(),
        out.data_ptr(), g, m, n, k, group_a.stride(0), group_b.stride(0), out.stride(0), tile_config,
        _stream_ptr(),
    )
    _lib.check(st, "mi355x_fp8_rowwise_grouped_gemm")
    return out


BLOCK = 128  # rows and columns one block scale covers


def fp8_gemm_blockwise(
    xq: torch.Tensor,
    wq: torch.Tensor,
    x_scale: torch.Tensor,
    w_scale: torch.Tensor,
    out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Block-scaled FP8 GEMM: bf16 [M,N] = sum over 128-wide K blocks of (xq_blk @ wq_blk.T) *
    x_scale[m // 128, kb] * w_scale[n // 128, kb].

    Same operands as the callables of tritonbench/operators/fp8_gemm_blockwise/operator.py:139-145:
    xq [M,K], wq [N,K] float8_e4m3fn; x_scale [ceil(M/128), ceil(K/128)] and w_scale
    [ceil(N/128), ceil(K/128)] float32 as fp8_block_quantize returns them (:86-118).
    Only enqueues work on the current stream.
    """
    lib = _lib.load()
    for t, name in ((xq, "xq"), (wq, "wq"), (x_scale, "x_scale"), (w_scale, "w_scale")):
        _require_gpu(t, name)
    if xq.dtype != FP8_DTYPE or wq.dtype != FP8_DTYPE:
        raise TypeError(f"xq and wq must be {FP8_DTYPE}")
    if xq.dim() != 2 or wq.dim() != 2 or xq.shape[1] != wq.shape[1]:
        raise ValueError("expected xq [M,K] and wq [N,K]")
    m, k = xq.shape
    n = wq.shape[0]
    gm, gn, gk = -(-m // BLOCK), -(-n // BLOCK), -(-k // BLOCK)
    if x_scale.dtype != torch.float32 or w_scale.dtype != torch.float32:
        raise TypeError("x_scale and w_scale must be float32")
    if tuple(x_scale.shape) != (gm, gk) or tuple(w_scale.shape) != (gn, gk):
        raise ValueError(f"expected x_scale [{gm},{gk}] and w_scale [{gn},{gk}], got {tuple(x_scale.shape)} and {tuple(w_scale.shape)}")
    if not x_scale.is_contiguous() or not w_scale.is_contiguous():
        raise ValueError("scales must be contiguous")
    if xq.stride(1) != 1 or wq.stride(1) != 1:
        raise ValueError("xq and wq must be K-contiguous")
    if out is None:
        out = torch.empty((m, n), dtype=torch.bfloat16, device=xq.device)
    else:
        _require_gpu(out, "out")
        if out.dtype != torch.bfloat16 or tuple(out.shape) != (m, n) or out.stride(1) != 1:
            raise ValueError("out must be bfloat16 [M,N] with unit column stride")
    st = lib.mi355x_fp8_blockwise_gemm(
        xq.data_ptr(), wq.data_ptr(), x_scale.data_ptr(), w_scale.data_ptr(), out.data_ptr(),
        m, n, k, xq.stride(0), wq.stride(0), out.stride(0), _stream_ptr(),
    )
    _lib.check(st, "mi355x_fp8_blockwise_gemm")
    return out


def fp8_row_quantize(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Row-wise e4m3fn quantisation on the GPU; returns (xq, inverse scale) like
    fp8_row_quantize in tritonbench/operators/fp8_gemm_rowwise/operator.py:136-145."""
    lib = _lib.load()
    _require_gpu(x, "x")
    if x.dim() != 2 or x.stride(1) != 1:
        raise ValueError("x must be 2-D with unit column stride")
    if x.dtype == torch.float32:
        src = _lib.SRC_F32
    elif x.dtype == torch.bfloat16:
        src = _lib.SRC_BF16
    else:
        raise TypeError(f"unsupported source dtype {x.dtype}")
    r, k = x.shape
    xq = torch.empty((r, k), dtype=FP8_DTYPE, device=x.device)
    inv_scale = torch.empty((r,), dtype=torch.float32, device=x.device)
    st = lib.mi355x_fp8_rowwise_quantize(
        x.data_ptr(), src, xq.data_ptr(), inv_scale.data_ptr(), r, k, x.stride(0), xq.stride(0),
        _stream_ptr(),
    )
    _lib.check(st, "mi355x_fp8_rowwise_quantize")
    return xq, inv_scale


def fp8_block_quantize(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """128 x 128 block-wise e4m3fn quantisation on the GPU; returns (xq, inverse scales
    [ceil(M/128), ceil(K/128)]) like fp8_block_quantize in
    tritonbench/operators/fp8_gemm_blockwise/operator.py:86-118."""
    lib = _lib.load()
    _require_gpu(x, "x")
    if x.dim() != 2 or x.stride(1) != 1:
        raise ValueError("x must be 2-D with unit column stride")
    if x.dtype == torch.float32:
        src = _lib.SRC_F32
    elif x.dtype == torch.bfloat16:
        src = _lib.SRC_BF16
    else:
        raise TypeError(f"unsupported source dtype {x.dtype}")
    m, k = x.shape
    xq = torch.empty((m, k), dtype=FP8_DTYPE, device=x.device)
    inv_scale = torch.empty((-(-m // BLOCK), -(-k // BLOCK)), dtype=torch.float32, device=x.device)
    st = lib.mi355x_fp8_blockwise_quantize(
        x.data_ptr(), src, xq.data_ptr(), inv_scale.data_ptr(), m, k, x.stride(0), xq.stride(0),
        _stream_ptr(),
    )
    _lib.check(st, "mi355x_fp8_blockwise_quantize")
    return xq, inv_scale


def _fused_quant_outputs(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    r, k = x.shape
    return (torch.empty((r, k), dtype=FP8_DTYPE, device=x.device),
            torch.empty((r,), dtype=torch.float32, device=x.device))


def rms_norm_fp8_rowwise_quant(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5) -> Tuple[torch.Tensor, torch.Tensor]:
    """RMSNorm with a weight vector and row-wise e4m3fn quantisation in one kernel; returns
    (xq, inverse scale). Stands in for rms_norm_fp8_rowwise_quant(x1, wd) of
    tritonbench/operators/fp8_fused_quant_gemm_rowwise/operator.py:86-94."""
    lib = _lib.load()
    _require_gpu(x, "x")
    _require_gpu(weight, "weight")
    if x.dim() != 2 or x.stride(1) != 1 or x.dtype != torch.bfloat16:
        raise ValueError("x must be a 2-D bfloat16 tensor with unit column stride")
    if weight.dtype != torch.bfloat16 or tuple(weight.shape) != (x.shape[1],) or weight.stride(0) != 1:
        raise ValueError("weight must be a contiguous bfloat16 vector of length K")
    xq, inv_scale = _fused_quant_outputs(x)
    st = lib.mi355x_fp8_rmsnorm_rowwise_quantize(
        x.data_ptr(), weight.data_ptr(), float(eps), xq.data_ptr(), inv_scale.data_ptr(),
        x.shape[0], x.shape[1], x.stride(0), xq.stride(0), _stream_ptr(),
    )
    _lib.check(st, "mi355x_fp8_rmsnorm_rowwise_quantize")
    return xq, inv_scale


def silu_mul_fp8_rowwise_quant(x1: torch.Tensor, x2: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """SiLU(x1) * x2 and row-wise e4m3fn quantisation in one kernel; returns (xq, inverse scale).
    Stands in for silu_mul_fp8_rowwise_quant(x1, x2) of
    tritonbench/operators/fp8_fused_quant_gemm_rowwise/operator.py:111-119."""
    lib = _lib.load()
    _require_gpu(x1, "x1")
    _require_gpu(x2, "x2")
    for name, t in (("x1", x1), ("x2", x2)):
        if t.dim() != 2 or t.stride(1) != 1 or t.dtype != torch.bfloat16:
            raise ValueError(f"{name} must be a 2-D bfloat16 tensor with unit column stride")
    if x1.shape != x2.shape:
        raise ValueError("x1 and x2 must have the same shape")
    xq, inv_scale = _fused_quant_outputs(x1)
    st = lib.mi355x_fp8_silu_mul_rowwise_quantize(
        x1.data_ptr(), x2.data_ptr(), xq.data_ptr(), inv_scale.data_ptr(),
        x1.shape[0], x1.shape[1], x1.stride(0), x2.stride(0), xq.stride(0), _stream_ptr(),
    )
    _lib.check(st, "mi355x_fp8_silu_mul_rowwise_quantize")
    return xq, inv_scale
