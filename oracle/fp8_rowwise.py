"""CPU restatement of the tritonbench `fp8_gemm_rowwise` path. TEST INFRASTRUCTURE ONLY
(see oracle/__init__.py): the checker for tests/, smoke() and bench.py's cpu_baseline leg.

What is restated, and from where (paths relative to the tritonbench checkout):
  fp8_row_quantize      tritonbench/operators/fp8_gemm_rowwise/operator.py:130-145
  dequant_matmul        the result the timed callables produce, operator.py:187-217, written as
                        fp32 dequantise + matmul (the arithmetic itself lives in FBGEMM
                        `fbgemm_gpu.experimental.gemm.triton_gemm.fp8_gemm.matmul_fp8_row` and
                        `torch.ops.fbgemm.f8f8bf16_rowwise`; FBGEMM is an un-vendored, unpinned
                        submodule of the checkout, so the published contract
                        C = (A . B^T) * a_scale[:,None] * b_scale[None,:] + bias is restated)
  flops / moved_bytes   operator.py:248-271
  make_inputs           operator.py:280-297 (shapes, per-row A and per-row-of-[N,K] B
                        quantisation, optional bf16 bias), seeded as utils/env_utils.py:20

  rms_norm / silu_mul / *_fp8_rowwise_quant
                        the front ends of tritonbench/operators/fp8_fused_quant_gemm_rowwise/
                        operator.py:86-131. The kernels that operator times (rms_norm,
                        rms_norm_fp8_rowwise_quant, silu_mul, silu_mul_fp8_rowwise_quant) are
                        imported from `gen_ai.llm_inference.fb.llm.kernel`, which is not part of the
                        checkout, so the published definitions are restated: RMSNorm
                        y = x * rsqrt(mean(x^2) + eps) * w and SwiGLU's SiLU(x1) * x2, evaluated in
                        fp32 on the bf16 inputs, followed by fp8_row_quantize on the fp32 result.
                        Parity unpinned for what those definitions leave open: the default eps, the
                        order of the two multiplications and any bf16 rounding inside the absent kernels.

How each function is pinned (tests/test_oracle_*.py):
  fp8_row_quantize      against an independent numpy restatement built on the bit-level
                        codec of oracle/e4m3.py, against oracle/fp8_rowwise_ref.c, and through
                        invariants (|xq| <= 448, max |xq| == 448 on non-zero rows, half-ulp
                        reconstruction error, inverse scale is 1/(448/amax) bitwise)
  dequant_matmul        against float64 brute force (gemm_f64, numpy) on small and ragged
                        shapes, bit-exact integer cases, identity / one-hot operands, and
                        oracle/fp8_rowwise_ref.c
  rms_norm              against torch.nn.functional.rms_norm, a float64 loop over small rows, scale
                        invariance at eps = 0 and the constant-row closed form
  silu_mul              against torch.nn.functional.silu and the float64 definition
  matmul_fp8_row's own rounding / accumulation order and f8f8bf16_rowwise's CK instance
  are NOT reproducible without FBGEMM: parity unpinned for those (the tolerance
  rtol 1e-2 / atol 1e-2 is what absorbs them).
"""
import hashlib
from typing import Optional, Tuple

import numpy as np
import torch

from . import e4m3

MAIN_RANDOM_SEED = 1337  # tritonbench/utils/env_utils.py:20
FP8_DTYPE = torch.float8_e4m3fn
E4M3_MAX_POS = torch.finfo(FP8_DTYPE).max  # 448.0, operator.py:131
EPS = 1e-12  # operator.py:132
FP16_MAX_POS = torch.finfo(torch.float16).max  # operator.py:133


def fp8_row_quantize(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """operator.py:136-145. Arithmetic runs in x.dtype; returns (xq, 1/scale as f32).
    Note `float / tensor` is evaluated by torch as `tensor.reciprocal() * float`, so
    scale = fl(fl(1/amax) * 448), not the correctly rounded quotient."""
    row_max = x.abs().max(dim=1).values
    scale = E4M3_MAX_POS / row_max.clamp(min=EPS)
    if x.dtype is torch.float16:
        scale = scale.clamp(max=FP16_MAX_POS)
    xq = (x * scale[:, None]).clamp(min=-E4M3_MAX_POS, max=E4M3_MAX_POS).to(FP8_DTYPE)
    return xq, scale.reciprocal().to(torch.float32)


def fp8_row_quantize_numpy(x: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """Same computation for float32 input, in numpy with the bit-level codec; returns
    (uint8 codes, f32 inverse scale). Exists to cross-check fp8_row_quantize."""
    x = np.asarray(x, dtype=np.float32)
    amax = np.max(np.abs(x), axis=1)
    # torch evaluates `448.0 / tensor` as `tensor.reciprocal() * 448.0` (Tensor.__rtruediv__):
    # two fp32 roundings, which is what the reference's `E4M3_MAX_POS / torch.clamp(...)` does
    recip = (np.float32(1.0) / np.maximum(amax, np.float32(1e-12))).astype(np.float32)
    scale = (recip * np.float32(448.0)).astype(np.float32)
    y = (x * scale[:, None]).astype(np.float32)
    y = np.minimum(np.maximum(y, np.float32(-448.0)), np.float32(448.0))
    inv = (np.float32(1.0) / scale).astype(np.float32)
    return e4m3.encode_rne(y), inv


def dequant_matmul(
    xq: torch.Tensor,
    wq: torch.Tensor,
    x_scale: torch.Tensor,
    w_scale: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    out_dtype: torch.dtype = torch.bfloat16,
) -> torch.Tensor:
    """The parity reference: fp32 dequantise-then-matmul on host cores, one rounding to the
    output type (bf16; float16 for the tensor-wise form of
    tritonbench/operators/fp8_gemm/fp8_gemm.py:87-101)."""
    a = xq.to(torch.float32) * x_scale[:, None]
    b = wq.to(torch.float32) * w_scale[:, None]
    out = a @ b.t()
    if bias is not None:
        out = out + bias.to(torch.float32)
    return out.to(out_dtype)


def dequantize(q: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """fp32 value of a row-wise quantised operand (one half of dequant_matmul)."""
    return q.to(torch.float32) * scale[:, None]


def dequant_matmul_rows(a_deq: torch.Tensor, b_deq: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """dequant_matmul on operands already passed through dequantize(): lets a caller check
    many row subsets against one dequantised weight without redoing the widening."""
    out = a_deq @ b_deq.t()
    if bias is not None:
        out = out + bias.to(torch.float32)
    return out.to(torch.bfloat16)


def to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit pattern (uint16), round to nearest even."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = np.isnan(x)
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    r = np.where(nan, (u >> 16) | 0x40, r)
    return r.astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def gemm_f64(
    a_codes: np.ndarray,
    b_codes: np.ndarray,
    a_scale: np.ndarray,
    b_scale: np.ndarray,
    bias_bf16_bits: Optional[np.ndarray] = None,
) -> np.ndarray:
    """Brute force in float64 from raw codes; returns float64 [M,N] BEFORE the bf16 rounding."""
    a = e4m3.decode(a_codes).astype(np.float64)
    b = e4m3.decode(b_codes).astype(np.float64)
    out = (a @ b.T) * a_scale.astype(np.float64)[:, None] * b_scale.astype(np.float64)[None, :]
    if bias_bf16_bits is not None:
        out = out + bf16_bits_to_f32(bias_bf16_bits).astype(np.float64)[None, :]
    return out


def flops(m: int, n: int, k: int, bias: bool) -> int:
    """operator.py:248-259."""
    return 2 * m * n * k + (2 * m * n if bias else 0)


def moved_bytes(m: int, n: int, k: int) -> int:
    """operator.py:261-271: fp8 A + fp8 B + bf16 C (scales and bias not counted)."""
    return m * k + n * k + 2 * m * n


def _sub_seed(m: int, n: int, k: int, role: str) -> int:
    h = hashlib.sha256(f"{MAIN_RANDOM_SEED}:{m}:{n}:{k}:{role}".encode()).digest()
    return int.from_bytes(h[:7], "little")


def randn_f32(rows: int, cols: int, sigma: float, seed: int) -> torch.Tensor:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    x = torch.randn((rows, cols), generator=g, dtype=torch.float32)
    if sigma != 1.0:
        x.mul_(sigma)
    return x


def make_weight(n: int, k: int, sigma: float = 1.0):
    """(wq, w_scale) for B [N,K]; depends only on (n, k) so an M sweep can reuse it."""
    w = randn_f32(n, k, sigma, _sub_seed(0, n, k, "w"))
    return fp8_row_quantize(w)


def make_activation(m: int, n: int, k: int, sigma: float = 1.0):
    x = randn_f32(m, k, sigma, _sub_seed(m, n, k, "x"))
    return fp8_row_quantize(x)


def make_bias(m: int, n: int, k: int, sigma: float = 0.1) -> torch.Tensor:
    g = torch.Generator(device="cpu")
    g.manual_seed(_sub_seed(m, n, k, "bias"))
    return (sigma * torch.randn((n,), generator=g, dtype=torch.float32)).to(torch.bfloat16)


def make_inputs(m: int, n: int, k: int, sigma: float = 1.0, bias: bool = False):
    """Seeded host-side inputs (xq, wq, x_scale, w_scale, bias) as get_input_iter yields them."""
    xq, x_scale = make_activation(m, n, k, sigma)
    wq, w_scale = make_weight(n, k, sigma)
    b = make_bias(m, n, k) if bias else None
    return xq, wq, x_scale, w_scale, b


# The five workload families the parity and bench code iterate over.
def fp8_block_quantize(x: torch.Tensor, block_m: int = 128, block_k: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """One scale per block_m x block_k block. Follows fp8_block_quantize,
    tritonbench/operators/fp8_gemm_blockwise/operator.py:86-118: zero-pad to whole blocks,
    block_max = amax |x| per block clamped at 1e-12, scale = 448 / block_max (in fp32), a scale
    of inf becomes 1, xq = (x * scale).to(e4m3fn) (no clamp: |x * scale| <= 448 up to rounding),
    returns (xq, 1 / scale) with the scale grid [ceil(M/block_m), ceil(K/block_k)]."""
    m, k = x.shape
    gm, gk = -(-m // block_m), -(-k // block_k)
    padded = torch.zeros(gm * block_m, gk * block_k, dtype=x.dtype)
    padded[:m, :k] = x
    block_max = padded.abs().reshape(gm, block_m, gk, block_k).amax(dim=(1, 3))
    block_max = torch.clamp(block_max, min=EPS)
    scale = E4M3_MAX_POS / block_max.to(torch.float32)
    scale[scale == float("inf")] = 1.0
    xq = (padded * scale.repeat_interleave(block_m, dim=0).repeat_interleave(block_k, dim=1))[:m, :k]
    return xq.to(FP8_DTYPE), 1 / scale


def blockwise_dequant_matmul(xq, wq, x_scale, w_scale, block: int = 128) -> torch.Tensor:
    """Block-scaled product on the CPU: every element is widened to fp32 and multiplied by its
    block's scale, then one fp32 matmul and one bf16 rounding. Mathematically the sum over K
    blocks of (xq_blk @ wq_blk.T) * x_scale[m // 128, kb] * w_scale[n // 128, kb] that the
    callables at tritonbench/operators/fp8_gemm_blockwise/operator.py:139-145 compute."""
    m, k = xq.shape
    n = wq.shape[0]
    xs = x_scale.repeat_interleave(block, dim=0).repeat_interleave(block, dim=1)[:m, :k]
    ws = w_scale.repeat_interleave(block, dim=0).repeat_interleave(block, dim=1)[:n, :k]
    return ((xq.to(torch.float32) * xs) @ (wq.to(torch.float32) * ws).t()).to(torch.bfloat16)


def make_blockwise_inputs(m, n, k, sigma=1.0, seed_tag=0):
    """Seeded operands of the block-scaled form, quantised per 128x128 block."""
    xq, xs = fp8_block_quantize(randn_f32(m, k, sigma, seed=MAIN_RANDOM_SEED + 13 * m + k + seed_tag))
    wq, ws = fp8_block_quantize(randn_f32(n, k, sigma, seed=MAIN_RANDOM_SEED + 29 * n + k + seed_tag))
    return xq, wq, xs, ws


def grouped_dequant_matmul(xq, wq, m_sizes, x_scale, w_scale):
    """Grouped form on the CPU: rows of group g (m_sizes[g] consecutive rows, in order) times
    wq[g*N:(g+1)*N].T with both scales, fp32 dequantise + matmul, one bf16 rounding; rows past
    sum(m_sizes) are zero. Follows the per-group expression of the reference's torch baseline,
    tritonbench/operators/fp8_gemm_rowwise_grouped/operator.py:689-699, with the group
    boundaries taken from m_sizes as its Triton and CK backends do (:400-455); the random
    boundaries the reference baseline draws at :676-686 are a quirk of that baseline and are
    not restated."""
    sizes = [int(v) for v in m_sizes]
    g = len(sizes)
    m, k = xq.shape
    n = wq.shape[0] // g
    out = torch.zeros((m, n), dtype=torch.bfloat16)
    start = 0
    for i, mg in enumerate(sizes):
        end = min(start + max(mg, 0), m)
        if end > start:
            out[start:end] = dequant_matmul(xq[start:end], wq[i * n:(i + 1) * n], x_scale[start:end],
                                            w_scale[i * n:(i + 1) * n])
        start = end
    return out


def make_grouped_inputs(g, m, n, k, sigma=1.0, sizes=None, seed_tag=0):
    """Seeded operands of the grouped form: A [M,K], B [G*N,K] quantised row-wise, m_sizes int32
    [G] (equal split M // G as at operator.py:563-565 unless `sizes` is given)."""
    xq, xs = fp8_row_quantize(randn_f32(m, k, sigma, seed=MAIN_RANDOM_SEED + 17 * m + k + seed_tag))
    wq, ws = fp8_row_quantize(randn_f32(g * n, k, sigma, seed=MAIN_RANDOM_SEED + 31 * n + k + g + seed_tag))
    if sizes is None:
        sizes = [m // g] * g
    return xq, wq, torch.tensor(sizes, dtype=torch.int32), xs, ws


LLAMA3_70B_NK = {"qkv": (10240, 8192), "o_proj": (8192, 8192), "gate_up": (57344, 8192), "down": (8192, 28672)}
LLAMA3_70B_M = (1, 32, 128, 1024, 4096)
CONFIGS = {
    "c1_plumbing": dict(shapes=[(128, 256, 512)], sigma=1.0, bias=False),
    "c2_square": dict(shapes=[(8192, 8192, 8192)], sigma=1.0, bias=False),
    "c3_skinny": dict(shapes=[(16, 8192, 8192)], sigma=1.0, bias=False),
    "c4_llama70b": dict(
        shapes=[(m, n, k) for (n, k) in LLAMA3_70B_NK.values() for m in LLAMA3_70B_M], sigma=0.02, bias=False
    ),
    "c5_ragged_bias": dict(shapes=[(1000, 3000, 4112), (4097, 7168, 2048)], sigma=1.0, bias=True),
}


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """RMSNorm with a weight vector in fp32: (x * rstd) * w, rstd = 1/sqrt(mean(x^2) + eps) with the
    mean taken in float64 and rounded once (the front end of operator.py:86-109 of
    fp8_fused_quant_gemm_rowwise; the kernel there is not in the checkout)."""
    xf = x.to(torch.float32)
    ms = xf.to(torch.float64).pow(2).mean(dim=1)
    rstd = (1.0 / torch.sqrt(ms + eps)).to(torch.float32)
    return (xf * rstd[:, None]) * weight.to(torch.float32)[None, :]


def silu_mul(x1: torch.Tensor, x2: torch.Tensor) -> torch.Tensor:
    """SiLU(x1) * x2 in fp32 (operator.py:111-131 of fp8_fused_quant_gemm_rowwise)."""
    a = x1.to(torch.float32)
    return (a / (1.0 + torch.exp(-a))) * x2.to(torch.float32)


def rms_norm_fp8_rowwise_quant(x, weight, eps: float = 1e-5):
    """(xq, inverse scale) of the normalised activation, quantised as an fp32 tensor."""
    return fp8_row_quantize(rms_norm(x, weight, eps))


def silu_mul_fp8_rowwise_quant(x1, x2):
    return fp8_row_quantize(silu_mul(x1, x2))


def make_fused_inputs(m: int, n: int, k: int, seed_tag: int = 0):
    """x1, x2 [m,k], w [n,k], wd [k] as bf16 standard normals (get_input_iter of
    fp8_fused_quant_gemm_rowwise/operator.py:154-165), plus the quantised weight."""
    g = torch.Generator().manual_seed(_sub_seed(m, n, k, f"fused{seed_tag}"))
    x1 = torch.randn((m, k), generator=g).to(torch.bfloat16)
    x2 = torch.randn((m, k), generator=g).to(torch.bfloat16)
    w = torch.randn((n, k), generator=g).to(torch.bfloat16)
    wd = torch.randn((k,), generator=g).to(torch.bfloat16)
    wq, w_scale = fp8_row_quantize(w)
    return x1, x2, wq, w_scale, wd
