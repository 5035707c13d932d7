"""The W4A16 GEMM on library-owned scratch (``vaq_w4a16_gemm_static``), called through the C ABI: same bits as
``vaq_w4a16_gemm`` with caller scratch, on calls in a row that shrink (the array keeps the previous call's contents)."""
from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

from oracle import w4a16 as o
from tests.helpers import W4A16Layer, check_gemm_close

pytestmark = pytest.mark.gpu


def _ptr(t):
    return None if t is None or t.numel() == 0 else ctypes.c_void_p(t.data_ptr())


def _run_both(lib, _lib, layer, a, m, n, k, has_perm):
    dev = a.device
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    wtype = _lib.VAQ_WTYPE_U4 if layer.zp.numel() else _lib.VAQ_WTYPE_U4B8
    perm = layer.sort_idx if has_perm else None
    # the existing entry point, scratch from the caller
    t, at, cn = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    _lib.check(lib.vaq_w4a16_gemm_workspace(m, n, k, int(has_perm), 0, ctypes.byref(t), ctypes.byref(at), ctypes.byref(cn)))
    c_tmp = torch.empty(max(t.value // 4, 1), dtype=torch.float32, device=dev)
    a_tmp = torch.empty(max(at.value // 2, 1), dtype=torch.bfloat16, device=dev)
    counters = torch.zeros(max(cn.value, 1), dtype=torch.int32, device=dev)
    ref = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    _lib.check(lib.vaq_w4a16_gemm(_ptr(a), a.stride(0), _ptr(layer.w), _ptr(layer.scales), _ptr(layer.zp), _ptr(perm), None,
                                  _ptr(ref), _ptr(c_tmp), t.value, _ptr(a_tmp), _ptr(counters), counters.numel(), m, n, k,
                                  128, _lib.VAQ_BF16, wtype, 0, stream))
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    _lib.check(lib.vaq_w4a16_gemm_static(_ptr(a), a.stride(0), _ptr(layer.w), _ptr(layer.scales), _ptr(layer.zp), _ptr(perm),
                                         None, _ptr(out), m, n, k, 128, _lib.VAQ_BF16, wtype, stream))
    torch.cuda.synchronize()
    return out, ref, (t.value, at.value, cn.value)


def test_w4a16_gemm_static_matches_caller_scratch_on_shrinking_calls(device):
    from vllm_amd import _lib
    lib = _lib.load()
    # (M, K, N, asymmetric, act_order): decode split over workgroups (partial tiles + counters), the tile kernel with K
    # split and permuted activations, then smaller problems of both kinds on the scratch the earlier calls left behind
    cases = [(16, 14336, 256, False, False), (130, 4096, 512, True, True), (8, 7168, 128, True, False),
             (70, 2048, 256, False, True), (3, 1024, 64, False, False)]
    used = []
    for i, (m, k, n, asym, act_order) in enumerate(cases):
        case = o.make_w4a16_case(k, n, 128, asym=asym, act_order=act_order, seed=40 + i)
        layer = W4A16Layer(case, device)
        a = torch.randn(m, k, generator=torch.Generator().manual_seed(i)).to(torch.bfloat16).to(device)
        for rep in range(2):      # twice in a row on the same scratch
            out, ref, sizes = _run_both(lib, _lib, layer, a, m, n, k, act_order)
            assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), f"case {i} rep {rep}: static scratch differs"
        used.append(sizes)
        check_gemm_close(out, o.gemm_ref(a.cpu(), o.case_w_ref(case)), f"static scratch case {i}")
    assert used[0][0] > 0 and used[0][2] > 0 and used[1][1] > 0, f"the cases no longer exercise the scratch: {used}"
    assert used[2][0] > 0 and used[2][0] < used[0][0], f"the third case should use less scratch than the first: {used}"


def test_w4a16_gemm_static_rejects_oversized_scratch(device):
    from vllm_amd import _lib
    lib = _lib.load()
    # vocabulary-sized layer, three m-blocks: 96 MB of partial tiles, above the library-owned 16 MiB
    rc = lib.vaq_w4a16_gemm_static(None, 4096, None, None, None, None, None, None, 40, 128256, 4096, 128, _lib.VAQ_BF16,
                                   _lib.VAQ_WTYPE_U4B8, None)
    assert rc == _lib.VAQ_ERR_INVALID_ARG and b"library-owned scratch" in lib.vaq_last_error()
