"""Weight-only FP8 (e4m3 weights, 16-bit activations) on the W4A16 GEMM -- the reference's Marlin FP8 path
(marlin_utils_fp8.py; exercised by test_marlin_gemm.py:262-270 with b_q_type float8_e4m3fn): byte-layout repack
bit-exact against the layout's CPU statement, GEMM against `a @ w_ref`, exact rows from one-hot activations, and the
linear method forced onto this path."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import native_layout as nl
from oracle import quantize as oq
from oracle import w4a16 as o
from tests.helpers import check_gemm_close, to_dev

pytestmark = pytest.mark.gpu


class Fp8WeightLayer:
    def __init__(self, case: dict, device, dtype):
        import vllm_amd._custom_ops as ops
        from vllm_amd.layers.quantization.utils import marlin_utils as mu
        from vllm_amd.scalar_type import scalar_types
        self.ops = ops
        self.k, self.n = case["q"].shape
        self.empty = torch.empty(0, dtype=torch.int32, device=device)
        self.w = ops.gptq_marlin_repack(to_dev(case["qweight"], device), self.empty, self.k, self.n, 8, layout="native_bytes")
        self.scales = case["scales"].to(dtype).to(device).contiguous()
        self.workspace = mu.marlin_make_workspace_new(device)
        self.wtype = scalar_types.float8_e4m3fn

    def __call__(self, a, bias=None):
        return self.ops.gptq_marlin_gemm(a, None, self.w, bias, self.scales, None, self.empty, self.empty, self.empty,
                                         self.workspace, self.wtype, a.shape[0], self.n, self.k)


def _weight(n, k, dtype, seed):
    return torch.randn(n, k, generator=torch.Generator().manual_seed(seed)).to(dtype)


@pytest.mark.parametrize("k,n", [(128, 64), (256, 320), (128 * 13, 64 * 5), (4096, 256)])
def test_repack_byte_layout_bit_exact(device, k, n):
    import vllm_amd._custom_ops as ops
    q = np.random.default_rng(k + n).integers(0, 256, size=(k, n), dtype=np.int32)
    qweight = to_dev(o.gptq_pack(q, 8), device)
    empty = torch.empty(0, dtype=torch.int32, device=device)
    out = ops.gptq_marlin_repack(qweight, empty, k, n, 8, layout="native_bytes")
    assert out.shape == (k // 16, 4 * n)
    assert np.array_equal(out.cpu().numpy(), nl.native_pack8_bytes(q))
    assert np.array_equal(nl.native_unpack8_bytes(out.cpu().numpy(), k, n), q)
    with pytest.raises(RuntimeError):
        ops.gptq_marlin_repack(to_dev(o.gptq_pack(q & 15, 4), device), empty, k, n, 4, layout="native_bytes")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("group_size", [-1, 128])
@pytest.mark.parametrize("k,n", [(128, 64), (1024, 192), (2048, 576), (14336 // 4, 128)])
def test_gemm_fp8_weights(device, k, n, group_size, dtype):
    case = oq.fp8_weight_case(_weight(n, k, dtype, k + n), group_size)
    layer = Fp8WeightLayer(case, device, dtype)
    for m in (1, 3, 16, 29, 33, 64, 100, 300):
        a = torch.randn(m, k, generator=torch.Generator().manual_seed(m)).to(dtype)
        out = layer(a.to(device))
        check_gemm_close(out, o.gemm_ref(a, case["w_ref"]), f"fp8 weights k={k} n={n} g={group_size} m={m} {dtype}")
    assert bool((layer.workspace == 0).all())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m", [1, 16, 200])
def test_one_hot_activation_returns_fp8_rows_exactly(device, dtype, m):
    """A one-hot activation row picks one dequantised weight row: `fp8.to(dtype) * scale`, one rounding, bit for bit --
    on the decode kernel (scale applied to the fp32 accumulator) and on the tile kernel (weights scaled before the MFMA)."""
    k, n = 512, 128
    case = oq.fp8_weight_case(_weight(n, k, dtype, 7) * 3, 128)
    layer = Fp8WeightLayer(case, device, dtype)
    rows = np.random.default_rng(m).integers(0, k, size=m)
    a = torch.zeros(m, k, dtype=dtype)
    a[torch.arange(m), torch.from_numpy(rows)] = 1.0
    out = layer(a.to(device)).cpu()
    assert torch.equal(out.view(torch.int16), case["w_ref"][rows].view(torch.int16))


def test_every_byte_value_converts_exactly(device):
    """All 256 e4m3 codes as weights of one column each (two are NaN and left out), scale 1: a one-hot activation returns
    the code's value, which pins the in-kernel FP8 -> 16-bit conversion against the bit-level decoder of the oracle."""
    from oracle import fp8 as of
    k, n = 128, 256
    codes = np.arange(256, dtype=np.int32)
    codes[codes == 0x7F] = 0
    codes[codes == 0xFF] = 0x80
    q = np.tile(codes[None, :], (k, 1))
    case = dict(q=q, qweight=o.gptq_pack(q, 8), scales=torch.ones(1, n), group_size=-1)
    for dtype in (torch.bfloat16, torch.float16):
        layer = Fp8WeightLayer(case, device, dtype)
        for m in (1, 100):
            a = torch.zeros(m, k, dtype=dtype)
            a[:, 5] = 1.0
            out = layer(a.to(device)).cpu().float().numpy()
            want = of.e4m3fn_decode(codes.astype(np.uint8))[None, :].repeat(m, 0)
            assert np.array_equal(out, want.astype(np.float32)), (dtype, m)


@pytest.mark.parametrize("k,n", [(4096, 6144), (14336, 4096)])
def test_gemm_fp8_weights_llama_shapes(device, k, n):
    case = oq.fp8_weight_case(_weight(n, k, torch.bfloat16, 3) * 0.02, -1)
    layer = Fp8WeightLayer(case, device, torch.bfloat16)
    for m in (1, 16, 32, 512):
        a = torch.randn(m, k, generator=torch.Generator().manual_seed(m)).to(torch.bfloat16)
        out = layer(a.to(device))
        rows = np.arange(m) if m <= 32 else np.random.default_rng(m).choice(m, 24, replace=False)
        check_gemm_close(out[rows], o.gemm_ref(a[rows], case["w_ref"]), f"fp8 weights llama k={k} n={n} m={m}")
        assert torch.isfinite(out.float()).all()


def test_fp8_linear_method_forced_weight_only(device, monkeypatch):
    """`Fp8LinearMethod` with VLLM_TEST_FORCE_FP8_MARLIN (fp8.py:353-363, :531-533, :655-664): a serialized FP8 checkpoint
    of a fused module with one scale per shard runs un-requantised on the weight-only path, activations stay 16-bit."""
    from oracle import fp8 as of
    from vllm_amd.layers.linear import QKVParallelLinear
    from vllm_amd.layers.quantization import get_quantization_config
    monkeypatch.setenv("VLLM_TEST_FORCE_FP8_MARLIN", "1")
    k = 512
    cfg = get_quantization_config("fp8").from_config(dict(quant_method="fp8", activation_scheme="dynamic"))
    layer = QKVParallelLinear(k, 64, 4, 2, bias=True, quant_config=cfg, params_dtype=torch.bfloat16, return_bias=False).to(device)
    assert layer.quant_method.use_marlin
    g = torch.Generator().manual_seed(4)
    scales = [torch.tensor(0.011), torch.tensor(0.023), torch.tensor(0.017)]
    parts = [of.ref_static_quant(torch.randn(nn, k, generator=g) * (0.5 + 0.4 * i), scales[i]) for i, nn in enumerate(layer.output_sizes)]
    for sid, part, sc in zip("qkv", parts, scales):
        layer.weight.weight_loader(layer.weight, part.to(device), sid)
        layer.weight_scale.weight_loader(layer.weight_scale, sc, sid)
    bias = (torch.randn(sum(layer.output_sizes), generator=g) * 0.1).to(torch.bfloat16)
    layer.bias.data.copy_(bias)
    layer.process_weights_after_loading()
    assert layer.input_scale is None and layer.weight.dtype == torch.int32
    w_ref = torch.cat([p.to(torch.bfloat16) * s.to(torch.bfloat16) for p, s in zip(parts, scales)], dim=0).T      # [K, N]
    for m in (2, 90):
        a = torch.randn(m, k, generator=g).to(torch.bfloat16)
        check_gemm_close(layer(a.to(device)), o.gemm_ref(a, w_ref, bias), f"forced weight-only fp8 m={m}")
