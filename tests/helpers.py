"""Shared helpers of the GPU parity tests: build a layer on the device from an oracle case and run it through the
public op surface (which calls the C ABI)."""
from __future__ import annotations

import numpy as np
import torch

from oracle import w4a16 as o


def to_dev(x, device, dtype=None):
    if x is None:
        return None
    t = torch.from_numpy(np.ascontiguousarray(x)) if isinstance(x, np.ndarray) else x
    if dtype is not None:
        t = t.to(dtype)
    return t.to(device)


class W4A16Layer:
    """GPTQ layer prepared the way ``process_weights_after_loading`` does it, from an oracle case dict."""

    def __init__(self, case: dict, device, dtype=torch.bfloat16):
        import vllm_amd._custom_ops as ops
        from vllm_amd.layers.quantization.utils import marlin_utils as mu
        from vllm_amd.scalar_type import scalar_types
        self.ops = ops
        k, n = case["q"].shape
        self.k, self.n, self.g = k, n, case["group_size"]
        self.dtype = dtype
        qweight = to_dev(case["qweight"], device)
        empty = torch.empty(0, dtype=torch.int32, device=device)
        if case["g_idx"] is not None:
            g_idx = to_dev(case["g_idx"], device)
            self.g_idx, self.sort_idx = mu.marlin_sort_g_idx(g_idx)
        else:
            self.g_idx, self.sort_idx = empty, empty
        bits = case.get("num_bits", 4)
        self.w = ops.gptq_marlin_repack(qweight, self.sort_idx, k, n, bits)
        self.scales = mu.marlin_permute_scales(to_dev(case["scales"], device, dtype), k, n, self.g)
        if case["zp_vals"] is not None:
            self.zp = mu.marlin_zero_points(to_dev(case["zp_vals"], device), case["zp_vals"].shape[0], n, 4)
            self.wtype = scalar_types.uint4
        else:
            self.zp = empty
            self.wtype = scalar_types.uint4b8 if bits == 4 else scalar_types.uint8b128
        self.workspace = mu.marlin_make_workspace_new(device)

    def __call__(self, a: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
        return self.ops.gptq_marlin_gemm(a, None, self.w, bias, self.scales, None, self.zp, self.g_idx, self.sort_idx,
                                         self.workspace, self.wtype, a.shape[0], self.n, self.k, is_k_full=True,
                                         use_fp32_reduce=True)


def check_gemm_close(out: torch.Tensor, ref64: torch.Tensor, what: str, max_rel: float = 2e-2, mean_rel: float = 0.04):
    """Tolerances: max|d|/max|ref| <= 2e-2 (the stated bar for 16-bit outputs with fp32 accumulation) and the
    reference's own metric mean|d|/mean|ref| < 0.04 (test_marlin_gemm.py:78-82).  In practice both are ~2e-3
    (one output rounding)."""
    out64 = out.detach().cpu().double()
    assert torch.isfinite(out64).all(), f"{what}: non-finite output"
    e_max = o.rel_err_max(out64, ref64)
    e_mean = o.rel_err_mean(out64, ref64)
    assert e_max <= max_rel, f"{what}: max-abs-rel {e_max:.3e} > {max_rel}"
    assert e_mean < mean_rel, f"{what}: mean-rel {e_mean:.3e} >= {mean_rel}"
    return e_max, e_mean
