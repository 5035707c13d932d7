"""Pins the FP8 CPU oracle: an independent bit-level e4m3fn encoder versus torch's CPU cast over every bf16 input,
edge cases of the per-token quantiser, and the epilogue orders of the scaled GEMM."""
import os

import numpy as np
import pytest
import torch

from oracle import fp8 as f

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _all_bf16():
    bits = (np.arange(65536, dtype=np.uint32) << 16)
    x = bits.view(np.float32)
    return x[np.isfinite(x)]


def test_encoder_matches_torch_cast_on_every_bf16_value():
    x = np.clip(_all_bf16(), -448, 448)
    mine = f.e4m3fn_encode_rne_sat(x)
    tor = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(mine, tor)


@pytest.mark.parametrize("scale", [1.0, 0.37, 3.0e-3, 117.0])
def test_encoder_matches_torch_cast_on_scaled_values(scale):
    x = np.clip(_all_bf16() / np.float32(scale), -448, 448).astype(np.float32)
    assert np.array_equal(f.e4m3fn_encode_rne_sat(x), torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy())


def test_encoder_known_answers():
    enc = lambda v: int(f.e4m3fn_encode_rne_sat(np.array([v], dtype=np.float32))[0])  # noqa: E731
    assert enc(448.0) == 0x7E and enc(-448.0) == 0xFE and enc(0.0) == 0x00
    assert enc(1.0) == 0x38 and enc(1.0625) == 0x38 and enc(1.1875) == 0x3A and enc(1.3125) == 0x3A   # ties to even
    assert enc(2.0 ** -9) == 0x01 and enc(2.0 ** -10) == 0x00 and enc(1.5 * 2.0 ** -9) == 0x02       # subnormals
    assert enc(2.0 ** -6) == 0x08 and enc(7.5 * 2.0 ** -9) == 0x08
    dec = f.e4m3fn_decode(np.arange(256, dtype=np.uint8))
    tdec = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.nan_to_num(dec, nan=-1.0), np.nan_to_num(tdec, nan=-1.0))


def test_unclamped_overflow_is_nan_in_torch_so_the_clamp_is_required():
    y = torch.tensor([448.0, 464.0, 465.0, 1000.0]).to(torch.float8_e4m3fn).float()
    assert y[0] == 448 and y[1] == 448 and torch.isnan(y[2]) and torch.isnan(y[3])


def test_per_token_quant_edge_cases():
    x = torch.zeros(3, 64, dtype=torch.bfloat16)
    x[1, 5] = 3.0
    x[1, 6] = -1.5
    x[2] = torch.linspace(-2, 2, 64).to(torch.bfloat16)
    q, s = f.ref_dynamic_per_token_quant(x)
    assert s.shape == (3, 1) and s.dtype == torch.float32
    assert s[0, 0].item() == float(np.float32(1.0) / (np.float32(448.0) * np.float32(512.0)))      # all-zero row
    assert abs(s[0, 0].item() - 4.359654212748865e-06) < 1e-20
    assert s[1, 0].item() == float(np.float32(3.0) / np.float32(448.0))
    codes = q.view(torch.uint8)
    assert codes[1, 5].item() == 0x7E and (codes[0] == 0).all()                                    # amax element -> 448
    assert codes[1, 6].item() == int(f.e4m3fn_encode_rne_sat(np.float32(-1.5) / np.float32(s[1, 0].item()))[()])
    # scale_ub clamps the row maximum before the division
    q2, s2 = f.ref_dynamic_per_token_quant(x, torch.tensor([1.0]))
    assert s2[1, 0].item() == float(np.float32(1.0) / np.float32(448.0))
    assert q2.view(torch.uint8)[1, 5].item() == 0x7E                                               # saturates


def test_division_and_reciprocal_multiply_are_not_interchangeable():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(256, 4096, generator=g).to(torch.bfloat16)
    q, s = f.ref_dynamic_per_token_quant(x)
    q_rcp = (x.float() * (1.0 / s)).clamp(-448, 448).to(torch.float8_e4m3fn)
    diff = (q.view(torch.uint8) != q_rcp.view(torch.uint8)).sum().item()
    assert 0 < diff < 0.01 * x.numel()


def test_per_token_codes_match_independent_encoder():
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(16, 1025, generator=g) * 5).to(torch.bfloat16)
    q, s = f.ref_dynamic_per_token_quant(x)
    ratio = (x.float().numpy() / s.numpy()).astype(np.float32)
    assert np.array_equal(q.view(torch.uint8).numpy(), f.e4m3fn_encode_rne_sat(np.clip(ratio, -448, 448)))


def test_per_tensor_quant():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(7, 300, generator=g).to(torch.bfloat16)
    q, s = f.ref_dynamic_per_tensor_quant(x)
    assert s.shape == (1, 1) and s.item() == float(np.float32(x.float().abs().max().item()) / np.float32(448.0))
    assert torch.equal(f.ref_static_quant(x, s).view(torch.uint8), q.view(torch.uint8))


def test_scaled_mm_epilogue_orders_agree_within_one_ulp():
    g = torch.Generator().manual_seed(3)
    m, k, n = 33, 256, 48
    a_q, sa = f.ref_dynamic_per_token_quant(torch.randn(m, k, generator=g).to(torch.bfloat16))
    w_q, sb = f.make_fp8_weight(n, k, seed=4)
    bias = (torch.randn(n, generator=g) * 0.01).to(torch.bfloat16)
    b = w_q.t()
    ref = f.scaled_mm_ref(a_q, b, sa, sb, torch.bfloat16, bias, order="cutlass")
    prod = sa.double() * (a_q.double() @ b.double()) * sb.double().reshape(1, -1)
    exact = prod + bias.double()
    ulp = exact.abs().clamp_min(2.0 ** -126) * 2.0 ** -7
    assert bool(((ref.double() - exact).abs() <= 0.51 * ulp + 1e-30).all())
    # the other two orders round intermediate terms, so their distance is one bf16 ulp of the larger TERM
    # (product or bias), not of the possibly cancelled sum
    term_ulp = torch.maximum(prod.abs(), bias.double().abs().expand_as(prod)).clamp_min(2.0 ** -126) * 2.0 ** -7
    for order in ("triton", "baseline"):
        other = f.scaled_mm_ref(a_q, b, sa, sb, torch.bfloat16, bias, order=order)
        assert bool(((other.double() - ref.double()).abs() <= 2.0 * term_ulp).all()), order
    # per-tensor scales broadcast
    ref_t = f.scaled_mm_ref(a_q, b, sa[:1].reshape(1), sb[:1].reshape(1), torch.bfloat16)
    assert ref_t.shape == (m, n)


def test_golden_vectors():
    gd = np.load(os.path.join(GOLDEN, "fp8_quant_small.npz"))
    x = torch.from_numpy(gd["x_bits"]).view(torch.bfloat16)
    q, s = f.ref_dynamic_per_token_quant(x)
    assert np.array_equal(q.view(torch.uint8).numpy(), gd["codes"]) and np.array_equal(s.numpy(), gd["scales"])
    q, s = f.ref_dynamic_per_token_quant(x, torch.from_numpy(gd["ub"]))
    assert np.array_equal(q.view(torch.uint8).numpy(), gd["codes_ub"]) and np.array_equal(s.numpy(), gd["scales_ub"])
    q, s = f.ref_dynamic_per_tensor_quant(x)
    assert np.array_equal(q.view(torch.uint8).numpy(), gd["codes_tensor"]) and np.array_equal(s.numpy(), gd["scale_tensor"])
    # the codes of the fixture also satisfy the independent encoder
    ratio = (x.float().numpy() / gd["scales"]).astype(np.float32)
    assert np.array_equal(gd["codes"], f.e4m3fn_encode_rne_sat(np.clip(ratio, -448, 448)))


def test_fused_rms_norm_quant_oracle_equals_unfused_composition():
    """The fused oracle must equal RMSNorm (the reference layer's forward_native: fp32 statistics, cast to the
    activation type, multiply by the weight; layernorm.py) followed by the unfused per-token quantiser, bit for bit
    whenever the fp64 and fp32 row sums round alike (they do for these sizes), with and without residual / scale_ub."""
    g = torch.Generator().manual_seed(0)
    for dtype in (torch.bfloat16, torch.float16):
        for hidden in (64, 1000, 4096):
            x = (torch.randn(7, hidden, generator=g) / hidden ** 0.5).to(dtype)
            res = (torch.randn(7, hidden, generator=g) / hidden ** 0.5).to(dtype)
            w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(dtype)
            for residual in (None, res):
                for ub in (None, torch.tensor(0.5)):
                    q, s, new_res = f.ref_rms_norm_dynamic_per_token_quant(x, w, 1e-5, ub, residual)
                    xf = x.float() + (residual.float() if residual is not None else 0.0)
                    normed = (xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + 1e-5)).to(dtype) * w
                    q2, s2 = f.ref_dynamic_per_token_quant(normed, ub)
                    assert torch.allclose(s, s2, rtol=2e-7, atol=0)
                    same = (q.view(torch.uint8) == q2.view(torch.uint8)).float().mean().item()
                    assert same > 0.999, same
                    if residual is not None:
                        assert torch.equal(new_res, xf.to(dtype))


def test_static_fused_norm_and_silu_oracles_equal_unfused_compositions():
    """The static-scale fused oracles against independent compositions, as the reference's own tests check the kernels
    (tests/kernels/core/test_layernorm.py:81-153, tests/kernels/test_fused_quant_activation.py:19-68): RMSNorm written
    with mean() and rsqrt, then the static quantiser oracle; torch.nn.functional.silu (the SiluAndMul layer's
    forward_native) times the gate, then the static quantiser oracle.  Bit-equal except where a last-bit difference of
    rsqrt/exp moves a value over a rounding boundary (< 0.2 % of the codes, one code step)."""
    g = torch.Generator().manual_seed(3)
    for dtype in (torch.bfloat16, torch.float16):
        for hidden in (64, 1000, 4096):
            x = (torch.randn(7, hidden, generator=g) / (2 * hidden)).to(dtype)
            res = (torch.randn(7, hidden, generator=g) / (2 * hidden)).to(dtype)
            w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(dtype)
            for qs in (1.0, 0.01):
                scale = torch.tensor([qs])
                for residual in (None, res):
                    q, new_res = f.ref_rms_norm_static_fp8_quant(x, w, scale, 1e-6, residual)
                    z = x if residual is None else (x + residual)
                    zf = z.float()
                    normed = (zf * torch.rsqrt(zf.pow(2).mean(-1, keepdim=True) + 1e-6)).to(dtype) * w
                    q2 = f.ref_static_quant(normed, scale)
                    a, b = q.view(torch.uint8).int(), q2.view(torch.uint8).int()
                    assert (a != b).float().mean().item() < 2e-3
                    assert ((a & 0x7f) - (b & 0x7f)).abs().max().item() <= 1
                    if residual is not None:
                        assert torch.equal(new_res, z)
            y = torch.randn(5, 2 * hidden, generator=g).to(dtype)
            scale = torch.tensor([0.05])
            q = f.ref_silu_and_mul_quant(y, scale)
            q2 = f.ref_static_quant(torch.nn.functional.silu(y[..., :hidden]) * y[..., hidden:], scale)
            a, b = q.view(torch.uint8).int(), q2.view(torch.uint8).int()
            assert (a != b).float().mean().item() < 2e-3
            assert ((a & 0x7f) - (b & 0x7f)).abs().max().item() <= 1

