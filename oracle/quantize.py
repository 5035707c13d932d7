"""CPU restatement of the reference's *weight quantisers* -- the functions its GEMM tests use to turn random float weights
into codes, scales and zero points, and the dequantised weight the tolerance is measured against.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  Follows
``vllm/model_executor/layers/quantization/utils/quant_utils.py`` (group_broadcast :142-153, scaled_quantize :162-205,
scaled_dequantize :208-238, quantize_weights :376-468, gptq_quantize_weights :475-506, sort_weights :509-521) and
``.../utils/marlin_utils_test.py`` (marlin_quantize :96-132, awq_marlin_quantize :135-161).

All arithmetic runs in the dtype of the weight that is passed in, operation by operation, as the reference's torch code
does (every elementwise torch op is correctly rounded in that dtype on any device, so CPU and GPU agree).

Pinned by mathematics in ``tests/test_oracle_quantize.py``: the dequantised weight is within half a quantisation step
of the input wherever no clamp applies, a group's extreme value maps to the extreme code, zero points stay in range,
the act_order bookkeeping is a permutation that ``sort_weights`` undoes group-wise, ``scaled_quantize`` /
``scaled_dequantize`` round-trip to within one step of the target format, and brute force over tiny inputs.
"""
from __future__ import annotations

import numpy as np
import torch

from . import w4a16 as ow

# (min, max) of the integer value a code stands for and the bias added to store it: vllm/scalar_type.py:327-351
# (uint4b8 / uint8b128 are unsigned fields with a bias; uint4 / uint8 are plain unsigned and take run-time zero points)
QUANT_TYPES = {
    "uint4b8": dict(bits=4, lo=-8, hi=7, bias=8),
    "uint8b128": dict(bits=8, lo=-128, hi=127, bias=128),
    "uint4": dict(bits=4, lo=0, hi=15, bias=0),
    "uint8": dict(bits=8, lo=0, hi=255, bias=0),
}


def _to_groups(w: torch.Tensor, group_size: int) -> torch.Tensor:
    """[K, N] -> [group_size, (K / group_size) * N]: column (g, n) holds the group_size values of group g, column n
    (quant_utils.py:400-404)."""
    k, n = w.shape
    return w.reshape(k // group_size, group_size, n).permute(1, 0, 2).reshape(group_size, -1)


def _from_groups(x: torch.Tensor, group_size: int, k: int, n: int) -> torch.Tensor:
    """Inverse of :func:`_to_groups` (quant_utils.py:449-456)."""
    return x.reshape(group_size, k // group_size, n).permute(1, 0, 2).reshape(k, n).contiguous()


def quantize_weights(w: torch.Tensor, quant_type: str, group_size: int | None, zero_points: bool = False,
                     ref_zero_points_after_scales: bool = False):
    """quant_utils.py:376-468.  Returns ``(w_ref [K,N] in w.dtype, w_q int32 [K,N] stored codes, w_s [G,N] in w.dtype or
    None, w_zp int32 [G,N] or None)``.

    Symmetric: ``s = max(|max / hi|, |min / lo|)`` per group and column, ``q = clamp(round(w / s), lo, hi)``,
    ``w_ref = q * s``, stored code ``q + bias``.  With zero points: ``s = max(max - min, 1e-5) / hi``,
    ``zp = clamp(round(|min / s|), lo, hi)``, ``q = clamp(round(w / s) + zp, lo, hi)``, ``w_ref = (q - zp) * s``.
    ``torch.round`` rounds halves to even.
    """
    t = QUANT_TYPES[quant_type]
    assert w.is_floating_point() and w.dim() == 2
    assert not zero_points or group_size is not None
    k, n = w.shape
    dtype = w.dtype
    if group_size == -1:
        group_size = k
    grouped = group_size is not None and group_size < k
    x = _to_groups(w, group_size) if grouped else w
    hi_val = x.max(dim=0, keepdim=True).values
    lo_val = x.min(dim=0, keepdim=True).values
    lo, hi = t["lo"], t["hi"]
    s = torch.ones(1, dtype=dtype)
    zp = None
    if group_size is not None:
        if zero_points:
            assert lo == 0 and hi > 0
            s = (hi_val - lo_val).clamp(min=1e-5) / hi
            zp = torch.round(torch.abs(lo_val / s)).clamp(lo, hi).int()
        else:
            s = torch.max((hi_val / (hi if hi != 0 else float("inf"))).abs(),
                          (lo_val / (lo if lo != 0 else float("inf"))).abs())
    q = torch.round(x / s).int() + (zp if zero_points else 0)
    q = torch.clamp(q, lo, hi)
    if ref_zero_points_after_scales and zp is not None:
        w_ref = q.to(dtype) * s - zp.to(dtype) * s
    else:
        w_ref = (q - (zp if zero_points else 0)).to(dtype) * s
    q = q + t["bias"]
    if grouped:
        q = _from_groups(q, group_size, k, n)
        w_ref = _from_groups(w_ref, group_size, k, n)
        s = s.reshape(-1, n).contiguous()
    if zp is not None:
        zp = zp.reshape(-1, n).contiguous()
    return w_ref, q.to(torch.int32), (s if group_size is not None else None), zp


def permute_rows(q_w: torch.Tensor, w_ref: torch.Tensor, group_size: int, rand_perm: torch.Tensor):
    """quant_utils.py:346-373: act_order as a random permutation of the K rows.  Returns
    ``(w_ref[perm], q_w[perm], g_idx[perm], perm)`` with ``g_idx[i] = i // group_size`` before the permutation."""
    assert q_w.shape == w_ref.shape
    k = q_w.shape[0]
    g_idx = (torch.arange(k, dtype=torch.int32) // group_size).to(torch.int32)
    return w_ref[rand_perm].contiguous(), q_w[rand_perm].contiguous(), g_idx[rand_perm].contiguous(), rand_perm


def gptq_quantize_weights(w: torch.Tensor, quant_type: str, group_size: int, act_order: bool,
                          test_perm: torch.Tensor | None = None, seed: int = 0):
    """quant_utils.py:475-506: symmetric quantisation, then (act_order) the row permutation.  Returns
    ``(w_ref, w_q, w_s, g_idx, rand_perm)``; ``g_idx`` / ``rand_perm`` are empty without act_order.  The reference draws
    the permutation from the global RNG; here it is ``test_perm`` or a seeded one."""
    k = w.shape[0]
    assert quant_type in ("uint4b8", "uint8b128") and group_size in (-1, 32, 64, 128, k)
    w_ref, w_q, w_s, _ = quantize_weights(w, quant_type, group_size)
    g_idx = torch.empty(0, dtype=torch.int32)
    rand_perm = torch.empty(0, dtype=torch.int64)
    if act_order:
        assert 0 < group_size < k, "act_order needs more than one group"
        perm = test_perm if test_perm is not None else torch.randperm(k, generator=torch.Generator().manual_seed(seed))
        w_ref, w_q, g_idx, rand_perm = permute_rows(w_q, w_ref, group_size, perm)
    return w_ref, w_q, w_s, g_idx, rand_perm


def sort_weights(q_w: torch.Tensor, g_idx: torch.Tensor):
    """quant_utils.py:509-521: rows ordered by group id.  Returns ``(q_w[order], g_idx[order], order int32)``.  (The
    reference's argsort is not stable; any order of the rows inside a group is valid, this one is the stable one.)"""
    order = torch.argsort(g_idx, stable=True).to(torch.int32)
    return q_w[order.long()].contiguous(), g_idx[order.long()].contiguous(), order


def marlin_quantize(w: torch.Tensor, quant_type: str, group_size: int, act_order: bool,
                    test_perm: torch.Tensor | None = None, seed: int = 0):
    """marlin_utils_test.py:96-132.  Returns ``[w_ref, marlin_q_w, marlin_s, g_idx, sort_indices, rand_perm]`` with the
    weights in the reference's Marlin order (int32 numpy) and the scales Marlin-permuted."""
    k, n = w.shape
    bits = QUANT_TYPES[quant_type]["bits"]
    if group_size == -1:
        group_size = k
    assert group_size <= k
    w_ref, q_w, s, g_idx, rand_perm = gptq_quantize_weights(w, quant_type, group_size, act_order, test_perm, seed)
    sort_indices = torch.empty(0, dtype=torch.int32)
    if act_order:
        q_w, g_idx, sort_indices = sort_weights(q_w, g_idx)
    marlin_q_w = ow.marlin_weights(q_w.numpy(), bits)
    marlin_s = torch.from_numpy(ow.marlin_permute_scales(s.view(torch.int16).numpy(), k, n, group_size)).view(s.dtype)
    return [w_ref, marlin_q_w, marlin_s, g_idx, sort_indices, rand_perm]


def awq_marlin_quantize(w: torch.Tensor, quant_type: str, group_size: int):
    """marlin_utils_test.py:135-161.  Returns ``[w_ref, marlin_q_w, marlin_s, marlin_zp]``."""
    k, n = w.shape
    bits = QUANT_TYPES[quant_type]["bits"]
    if group_size == -1:
        group_size = k
    assert group_size <= k and k % group_size == 0
    groups = k // group_size
    w_ref, q_w, s, zp = quantize_weights(w, quant_type, group_size, zero_points=True)
    marlin_q_w = ow.marlin_weights(q_w.numpy(), bits)
    marlin_s = torch.from_numpy(ow.marlin_permute_scales(s.view(torch.int16).numpy(), k, n, group_size)).view(s.dtype)
    marlin_zp = ow.marlin_zero_points(zp.numpy(), groups, n, bits)
    return [w_ref, marlin_q_w, marlin_s, marlin_zp]


def quantized_case(w: torch.Tensor, quant_type: str, group_size: int, act_order: bool = False, seed: int = 0) -> dict:
    """A float weight [K, N] through the reference's quantisers, as a checkpoint-format case like
    ``w4a16.make_w4a16_case`` builds from random codes, plus ``w_ref`` (the reference's own dequantised weight, rows in
    checkpoint order, so that ``C = A @ w_ref``)."""
    k, n = w.shape
    bits = QUANT_TYPES[quant_type]["bits"]
    if quant_type in ("uint4", "uint8"):
        assert not act_order
        w_ref, q, s, zp = quantize_weights(w, quant_type, group_size, zero_points=True)
        g_idx = None
    else:
        w_ref, q, s, g_idx_t, _ = gptq_quantize_weights(w, quant_type, group_size, act_order, seed=seed)
        zp = None
        g_idx = g_idx_t.numpy().astype(np.int32) if act_order else None
    qn = np.ascontiguousarray(q.numpy().astype(np.int32))
    zpn = None if zp is None else np.ascontiguousarray(zp.numpy().astype(np.int32))
    return dict(q=qn, qweight=ow.gptq_pack(qn, bits), scales=s, zp_vals=zpn,
                qzeros=None if zpn is None else ow.pack_cols(zpn, bits), g_idx=g_idx, group_size=group_size,
                num_bits=bits, w_ref=w_ref)


# --------------------------------------------------------------------------- floating-point group quantisation

def group_broadcast(t: torch.Tensor, shape) -> torch.Tensor:
    """quant_utils.py:142-153: repeat every entry of ``t`` over its group so that the result has ``shape`` (dimensions
    of extent 1 are left to broadcasting)."""
    for i, s in enumerate(shape):
        if t.shape[i] != s and t.shape[i] != 1:
            assert s % t.shape[i] == 0
            t = t.repeat_interleave(s // t.shape[i], dim=i)
    return t


def _normalize_group_shape(x: torch.Tensor, group_shape) -> tuple[int, int]:
    """-1 stands for the full extent of that dimension (quant_utils.py:131-138)."""
    return (group_shape[0] if group_shape[0] > 0 else x.shape[-2], group_shape[1] if group_shape[1] > 0 else x.shape[-1])


def scaled_quantize(x: torch.Tensor, group_shape, quant_dtype: torch.dtype):
    """quant_utils.py:162-205: one scale per ``group_shape`` block, ``scale = finfo.max / max(amax, 1e-12)``,
    ``x_q = clamp(x * scale, finfo.min, finfo.max).to(quant_dtype)``; returns ``(x_q, 1 / scale as fp32
    [M / gm, N / gn])``."""
    gm, gn = _normalize_group_shape(x, group_shape)
    assert quant_dtype.is_floating_point and x.dim() == 2 and x.shape[0] % gm == 0 and x.shape[1] % gn == 0
    finfo = torch.finfo(quant_dtype)
    bm, bn = x.shape[0] // gm, x.shape[1] // gn
    blocks = x.reshape(bm, gm, bn, gn).permute(0, 2, 1, 3).flatten(start_dim=2)
    lo, hi = blocks.aminmax(dim=-1)
    amax = torch.maximum(lo.abs(), hi.abs()).clamp(min=1e-12)
    scale = finfo.max / amax
    scaled = (blocks * scale.unsqueeze(-1)).clamp(min=finfo.min, max=finfo.max)
    scaled = scaled.reshape(bm, bn, gm, gn).permute(0, 2, 1, 3).reshape(x.shape)
    return scaled.to(quant_dtype).contiguous(), scale.float().reciprocal()


def scaled_dequantize(x_q: torch.Tensor, x_s: torch.Tensor, group_shape=None, out_dtype: torch.dtype = torch.float32):
    """quant_utils.py:208-238: ``x_q.float() * x_s`` with ``x_s`` repeated over its groups."""
    if group_shape is not None:
        group_shape = _normalize_group_shape(x_q, group_shape)
    if x_s.dim() == 0:
        x_s = x_s.reshape(1, 1)
    if x_s.dim() == 1:
        assert group_shape is not None, "a vector of scales needs the group shape to say which dimension it spans"
        if group_shape[0] == x_q.shape[-2]:
            x_s = x_s.unsqueeze(-2)
        elif group_shape[1] == x_q.shape[-1]:
            x_s = x_s.unsqueeze(-1)
        else:
            raise AssertionError("a vector of scales must span the full extent of one dimension")
    if group_shape is not None:
        assert x_s.shape[-1] == x_q.shape[-1] // group_shape[1] and x_s.shape[-2] == x_q.shape[-2] // group_shape[0]
    return (x_q.to(torch.float32) * group_broadcast(x_s.to(torch.float32), x_q.shape)).to(out_dtype)


# --------------------------------------------------------------------------- weight-only FP8 (e4m3 weights, 16-bit activations)

def marlin_quant_fp8_torch(weight: torch.Tensor, group_size: int):
    """marlin_utils_fp8.py:316-351 without the Marlin re-ordering: ``weight`` [N, K] float ->
    ``(w_ref [K, N] in weight.dtype, fp8 codes uint8 [K, N], scales [G, N] in weight.dtype)`` with
    ``scale = amax(group) / 448``, ``fp8 = (weight / scale).to(float8_e4m3fn)``, ``w_ref = fp8.to(dtype) * scale``
    (one group spanning K for ``group_size == -1``)."""
    n, k = weight.shape
    g = k if group_size == -1 else group_size
    scales = weight.view(n, k // g, g).abs().max(-1)[0] / 448
    rep = scales.repeat_interleave(g, 1)
    fp8 = (weight / rep).to(torch.float8_e4m3fn)
    w_ref = fp8.to(weight.dtype) * rep
    return w_ref.T.contiguous(), fp8.view(torch.uint8).T.contiguous(), scales.T.contiguous()


def fp8_weight_case(weight: torch.Tensor, group_size: int) -> dict:
    """A weight-only FP8 layer in the GPTQ-style container the repack takes (int32 [K/4, N], four consecutive k per
    word, low byte first: marlin_utils_fp8.py:299-313 ``pack_fp8_to_int32``), plus the codes, scales and ``w_ref``."""
    w_ref, codes, scales = marlin_quant_fp8_torch(weight, group_size)
    k, n = codes.shape
    qn = codes.numpy().astype(np.int32)
    return dict(q=qn, qweight=ow.gptq_pack(qn, 8), scales=scales, group_size=group_size, w_ref=w_ref)
