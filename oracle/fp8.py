"""CPU oracle for the FP8 W8A8 path: activation quantisation and the scaled GEMM.

TEST INFRASTRUCTURE ONLY -- never imported by the product package.

FP8 format is OCP e4m3fn (max 448, no inf, NaN = S.1111.111): gfx950 is not an FNUZ part
(vllm/platforms/rocm.py:447-452; csrc/quantization/w8a8/fp8/common.cuh:17-26).
"""
from __future__ import annotations

import numpy as np
import torch

FP8_MAX = 448.0                                   # torch.finfo(float8_e4m3fn).max; csrc/quantization/utils.cuh:27-29
MIN_SCALE = np.float32(1.0) / (np.float32(448.0) * np.float32(512.0))   # csrc/quantization/utils.cuh:47-52


# --------------------------------------------------------------------------- independent bit-level e4m3fn encoder

def e4m3fn_encode_rne_sat(x: np.ndarray) -> np.ndarray:
    """fp32 -> e4m3fn code (uint8), round-to-nearest-even, saturating at +-448; NaN -> 0x7F|sign.

    Written from the format definition (bias 7, 3 mantissa bits, subnormal step 2**-9), *not* from any
    library cast: used to pin torch's CPU ``.to(float8_e4m3fn)`` and the device ``v_cvt_pk_fp8_f32``.
    """
    x = np.asarray(x, dtype=np.float32)
    sign = (x.view(np.uint32) >> 31).astype(np.uint8) << 7
    ax = np.abs(x).astype(np.float64)
    out = np.zeros(x.shape, dtype=np.uint8)
    nan = np.isnan(ax)
    ax = np.where(nan, 0.0, ax)
    ax = np.minimum(ax, 448.0)                                   # saturate (inputs are pre-clamped anyway)
    # exponent of the quantisation step: normal numbers use 2**(e-3), subnormals 2**-9
    with np.errstate(divide="ignore"):
        e = np.floor(np.log2(np.where(ax > 0, ax, 1.0)))
    e = np.maximum(e, -6.0)
    step = np.exp2(e - 3.0)
    qf = ax / step                                               # exact in fp64 (power-of-two scaling)
    qi = np.rint(qf)                                             # numpy rint = ties-to-even
    val = qi * step
    # re-derive exponent/mantissa from the rounded value (rounding may carry into the next binade)
    with np.errstate(divide="ignore"):
        e2 = np.floor(np.log2(np.where(val > 0, val, 1.0)))
    normal = val >= 2.0 ** -6
    mant_n = np.rint(val / np.exp2(e2 - 3.0)) - 8.0
    code_n = ((e2 + 7.0) * 8.0 + mant_n)
    code_s = np.rint(val / 2.0 ** -9)
    code = np.where(normal, code_n, code_s).astype(np.uint8)
    out = np.where(nan, np.uint8(0x7F), code) | sign
    return out.astype(np.uint8)


def e4m3fn_decode(code: np.ndarray) -> np.ndarray:
    """e4m3fn code (uint8) -> fp32 value (exact)."""
    c = np.asarray(code, dtype=np.uint8).astype(np.int32)
    s = np.where(c & 0x80, -1.0, 1.0)
    e = (c >> 3) & 0xF
    m = c & 7
    val = np.where(e == 0, m * 2.0 ** -9, (8 + m) * np.exp2(e.astype(np.float64) - 10.0))
    val = np.where((c & 0x7F) == 0x7F, np.nan, val)
    return (s * val).astype(np.float32)


# --------------------------------------------------------------------------- activation quantisation

def ref_dynamic_per_token_quant(x: torch.Tensor, scale_ub: torch.Tensor | None = None):
    """Per-row dynamic quantisation, same operation order as the device kernel
    (csrc/quantization/w8a8/fp8/common.cu:91-131, common.cuh:41-60) and as the reference's own
    test oracle (tests/kernels/quant_utils.py:21-72):

        amax = max|float(x)|;  s = max(min(amax, ub) / 448, 1/(448*512));  q = cast(clamp(float(x) / s, +-448))

    True fp32 division -- ``x * (1/s)`` gives different codes for ~0.03 % of elements.
    Returns (codes as torch.float8_e4m3fn [M,K], scales fp32 [M,1]).
    """
    xf = x.to(torch.float32)
    amax = xf.abs().amax(dim=-1, keepdim=True)
    if scale_ub is not None:
        amax = torch.minimum(amax, scale_ub.to(torch.float32).reshape(()))
    s = torch.maximum(amax / torch.tensor(FP8_MAX, dtype=torch.float32),
                      torch.tensor(float(MIN_SCALE), dtype=torch.float32))
    q = (xf / s).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q, s


def ref_dynamic_per_tensor_quant(x: torch.Tensor):
    """tests/kernels/quant_utils.py:78-106 / common.cu:32-89: scale = amax/448 (no floor), codes use the
    *reciprocal* multiply ``x * (1/scale)`` (scaled_fp8_conversion<true>)."""
    xf = x.to(torch.float32)
    scale = xf.abs().max() / torch.tensor(FP8_MAX, dtype=torch.float32)
    inv = torch.tensor(1.0, dtype=torch.float32) / scale
    q = (xf * inv).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q, scale.reshape(1, 1)


def ref_static_quant(x: torch.Tensor, scale: torch.Tensor):
    """common.cu:11-30: ``cast(clamp(x * (1/scale)))`` with a given per-tensor scale."""
    xf = x.to(torch.float32)
    inv = torch.tensor(1.0, dtype=torch.float32) / scale.to(torch.float32).reshape(())
    return (xf * inv).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)


# --------------------------------------------------------------------------- scaled GEMM

def scaled_mm_ref(a_q: torch.Tensor, b_q: torch.Tensor, scale_a: torch.Tensor, scale_b: torch.Tensor,
                  out_dtype: torch.dtype, bias: torch.Tensor | None = None, *, order: str = "cutlass") -> torch.Tensor:
    """``D = round_out(sa[m] * (sb[n] * sum_k A[m,k] B[k,n]) + bias[n])``.

    ``a_q`` [M,K] e4m3fn, ``b_q`` [K,N] e4m3fn (any strides), ``scale_a`` [M,1] or scalar, ``scale_b`` [N,1] or scalar.
    The accumulation is done in fp64 (fp8 products are exact, so this is the exact sum); the epilogue order
    follows ``order``:

    * ``"cutlass"``  -- fp32 ``sa*(sb*acc)+bias`` then one rounding
      (csrc/cutlass_extensions/epilogue/scaled_mm_epilogues_c3x.hpp:136-216); the order the build implements.
    * ``"triton"``   -- ``acc*sa*sb`` cast to out dtype, then ``+bias`` in out dtype
      (compressed_tensors/triton_scaled_mm.py:103-126).
    * ``"baseline"`` -- ``mm(sa*A, sb*B)`` in fp32 then ``+bias`` (tests/kernels/utils.py:1333-1376).
    """
    acc = (a_q.to(torch.float64) @ b_q.to(torch.float64))
    sa = scale_a.to(torch.float32).reshape(-1, 1) if scale_a.numel() > 1 else scale_a.to(torch.float32).reshape(1, 1)
    sb = scale_b.to(torch.float32).reshape(1, -1) if scale_b.numel() > 1 else scale_b.to(torch.float32).reshape(1, 1)
    acc32 = acc.to(torch.float32)
    if order == "cutlass":
        out = sa * (sb * acc32)
        if bias is not None:
            out = out + bias.to(torch.float32)
        return out.to(out_dtype)
    if order == "triton":
        out = (acc32 * sa * sb).to(out_dtype)
        return out + bias if bias is not None else out
    if order == "baseline":
        out = ((sa.double() * a_q.double()) @ (sb.double() * b_q.double())).to(torch.float32)
        if bias is not None:
            out = out + bias.to(torch.float32)
        return out.to(out_dtype)
    raise ValueError(order)


def ref_rms_norm_dynamic_per_token_quant(x: torch.Tensor, weight: torch.Tensor, eps: float,
                                         scale_ub: torch.Tensor | None = None, residual: torch.Tensor | None = None):
    """Fused RMSNorm + per-token FP8 quant, operation order of
    csrc/quantization/fused_kernels/layernorm_utils.cuh:17-130 (the reference's own test oracle is the unfused
    composition, tests/kernels/core/test_fused_quant_layernorm.py:40-75):

        xf = float(x) (+ float(residual));  new_residual = T(xf)
        rms = rsqrt(sum(xf*xf)/hidden + eps)             # the sum here is accumulated in fp64, then rounded
        y = float(T(T(xf * rms) * weight));  s = max(min(max|y|, ub)/448, 1/(448*512));  q = cast(clamp(y / s))

    Returns (q e4m3fn, scales [tokens,1] fp32, new_residual or None).  The order of the fp32 additions inside the sum
    is the one degree of freedom a device kernel has; everything else is bit-determined."""
    dt = x.dtype
    xf = x.to(torch.float32)
    new_res = None
    if residual is not None:
        xf = xf + residual.to(torch.float32)
        new_res = xf.to(dt)
    hidden = x.shape[-1]
    ss = (xf.double() * xf.double()).sum(dim=-1, keepdim=True).to(torch.float32)
    rms = torch.rsqrt(ss / torch.tensor(float(hidden), dtype=torch.float32) + torch.tensor(eps, dtype=torch.float32))
    y = ((xf * rms).to(dt) * weight.to(dt)).to(torch.float32)
    amax = y.abs().amax(dim=-1, keepdim=True)
    if scale_ub is not None:
        amax = torch.minimum(amax, scale_ub.to(torch.float32).reshape(()))
    s = torch.maximum(amax / FP8_MAX, torch.tensor(1.0 / (FP8_MAX * 512.0), dtype=torch.float32))
    q = (y / s).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q, s, new_res


def ref_rms_norm_static_fp8_quant(x: torch.Tensor, weight: torch.Tensor, scale: torch.Tensor, eps: float,
                                  residual: torch.Tensor | None = None):
    """Fused RMSNorm (+ residual) + static per-tensor FP8 quant, operation order of
    csrc/layernorm_quant_kernels.cu:21-66 (no residual) and :138-178 (residual):

        z = x  or  T(float(x) + float(residual))  (written back to residual);  xf = float(z)
        rms = rsqrt(sum(xf*xf)/hidden + eps)            # sum accumulated in fp64 here, then rounded
        y = float(T(T(xf * rms) * weight));  q = cast(clamp(y * (1/scale), +-448))

    Returns (q e4m3fn, new_residual or None)."""
    dt = x.dtype
    new_res = None
    z = x
    if residual is not None:
        z = (x.to(torch.float32) + residual.to(torch.float32)).to(dt)
        new_res = z
    xf = z.to(torch.float32)
    hidden = x.shape[-1]
    ss = (xf.double() * xf.double()).sum(dim=-1, keepdim=True).to(torch.float32)
    rms = torch.rsqrt(ss / torch.tensor(float(hidden), dtype=torch.float32) + torch.tensor(eps, dtype=torch.float32))
    y = ((xf * rms).to(dt) * weight.to(dt)).to(torch.float32)
    inv = torch.tensor(1.0, dtype=torch.float32) / scale.to(torch.float32).reshape(())
    q = (y * inv).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q, new_res


def ref_silu_and_mul_quant(x: torch.Tensor, scale: torch.Tensor):
    """silu(x[..., :d]) * x[..., d:] quantised with a static scale, operation order of
    csrc/quantization/activation_kernels.cu:35-119: silu in fp32 (x / (1 + exp(-x))) rounded to the activation type,
    the product rounded to the activation type, then q = cast(clamp(float(product) * (1/scale), +-448)).  exp here
    is torch's fp32 exp, which may differ from a device's expf in the last bit."""
    dt = x.dtype
    d = x.shape[-1] // 2
    a = x[..., :d].to(torch.float32)
    b = x[..., d:]
    s = (a / (1.0 + torch.exp(-a))).to(dt)
    v = (s * b).to(torch.float32)
    inv = torch.tensor(1.0, dtype=torch.float32) / scale.to(torch.float32).reshape(())
    return (v * inv).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)


def make_fp8_weight(n: int, k: int, seed: int = 0, dtype: torch.dtype = torch.bfloat16):
    """BASELINE.json config 4 weight: ``randn([N,K])*0.02`` quantised per output channel (amax/448 fp32 scales).
    Returns (w_q [N,K] e4m3fn row-major, w_scale [N,1] fp32).  Per-channel quantisation of a weight is the same
    per-row op as the activation quant (ptpc_fp8.py:107-123)."""
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(n, k, generator=g) * 0.02).to(dtype)
    return ref_dynamic_per_token_quant(w)
