"""GPU parity tests of the FP8 path: activation quantisation (bit-exact codes and scales) and the scaled GEMM,
through the op surface that sits on the C ABI."""
import os

import numpy as np
import pytest
import torch

from oracle import fp8 as f

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")

LLAMA_SHAPES = [(4096, 6144), (4096, 4096), (4096, 28672), (14336, 4096)]


def _codes(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().view(torch.uint8).numpy()


# ------------------------------------------------------------------------------------------------ quantisation

def test_quant_every_bf16_value_bit_exact(device):
    """All 65 280 finite bf16 inputs in one row block, at several row scales: codes and scales equal the oracle."""
    import vllm_amd._custom_ops as ops
    bits = torch.arange(65536, dtype=torch.int32)
    vals = (bits << 16).view(torch.float32)
    vals = vals[torch.isfinite(vals)]
    finite = vals.to(torch.bfloat16)
    rows = []
    for cap in (3.0e38, 1.0e4, 448.0, 1.0, 1.0e-3, 1.0e-30):
        rows.append(torch.where(finite.float().abs() <= cap, finite, torch.zeros_like(finite)))
    x = torch.stack(rows)                      # [6, 65280]; every row has a different amax, hence a different scale
    q_ref, s_ref = f.ref_dynamic_per_token_quant(x)
    q, s = ops.scaled_fp8_quant(x.to(device), use_per_token_if_dynamic=True)
    assert np.array_equal(s.cpu().numpy(), s_ref.numpy())
    assert np.array_equal(_codes(q), _codes(q_ref))


# hidden sizes / token counts / dtypes of the reference's own test grid (tests/kernels/quantization/test_fp8_quant.py:15-21)
@pytest.mark.parametrize("hidden", [17, 1024, 1025, 1026, 5137, 8193, 4096, 14336, 16384, 16392])
@pytest.mark.parametrize("tokens", [1, 7, 257])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("use_ub", [False, True])
def test_per_token_quant_bit_exact(device, hidden, tokens, dtype, use_ub):
    import vllm_amd._custom_ops as ops
    torch.manual_seed(0)
    x = (torch.rand(tokens, hidden) + 1e-6).to(dtype)            # reference test input: rand + 1e-6, seed 0
    x[::2] *= -1.7
    ub = torch.tensor([x.float().abs().mean().item()], dtype=torch.float32) if use_ub else None
    q_ref, s_ref = f.ref_dynamic_per_token_quant(x, ub)
    q, s = ops.scaled_fp8_quant(x.to(device), scale_ub=None if ub is None else ub.to(device), use_per_token_if_dynamic=True)
    assert q.dtype == torch.float8_e4m3fn and s.shape == (tokens, 1) and s.dtype == torch.float32
    assert np.array_equal(s.cpu().numpy(), s_ref.numpy())
    assert np.array_equal(_codes(q), _codes(q_ref))


def test_per_token_quant_edge_rows_and_golden(device):
    import vllm_amd._custom_ops as ops
    gd = np.load(os.path.join(GOLDEN, "fp8_quant_small.npz"))
    x = torch.from_numpy(gd["x_bits"]).view(torch.bfloat16)
    q, s = ops.scaled_fp8_quant(x.to(device), use_per_token_if_dynamic=True)
    assert np.array_equal(_codes(q), gd["codes"]) and np.array_equal(s.cpu().numpy(), gd["scales"])
    assert s[4, 0].item() == float(np.float32(1.0) / (np.float32(448.0) * np.float32(512.0)))     # all-zero row
    q, s = ops.scaled_fp8_quant(x.to(device), scale_ub=torch.from_numpy(gd["ub"]).to(device), use_per_token_if_dynamic=True)
    assert np.array_equal(_codes(q), gd["codes_ub"]) and np.array_equal(s.cpu().numpy(), gd["scales_ub"])
    q, s = ops.scaled_fp8_quant(x.to(device))
    assert np.array_equal(_codes(q), gd["codes_tensor"]) and np.array_equal(s.cpu().numpy(), gd["scale_tensor"])


def test_per_token_quant_strided_rows_and_padding(device):
    import vllm_amd._custom_ops as ops
    torch.manual_seed(1)
    big = torch.randn(9, 3000).to(torch.bfloat16)
    big_dev = big.to(device)
    x = big[:, 8:8 + 2048]                                       # row stride 3000 elements, 16-byte aligned rows
    for lo, hi in ((8, 8 + 2048), (3, 3 + 1000)):                # second slice: unaligned rows -> scalar path
        q_ref, s_ref = f.ref_dynamic_per_token_quant(big[:, lo:hi])
        view = big_dev[:, lo:hi]
        assert view.stride() == (3000, 1)
        q, s = ops.scaled_fp8_quant(view, use_per_token_if_dynamic=True)
        assert np.array_equal(_codes(q), _codes(q_ref)) and np.array_equal(s.cpu().numpy(), s_ref.numpy())
    # padded output: rows beyond the input are allocated but not written
    q, s = ops.scaled_fp8_quant(x.contiguous().to(device), num_token_padding=17, use_per_token_if_dynamic=True)
    assert q.shape == (17, 2048) and s.shape == (17, 1)
    q_ref, s_ref = f.ref_dynamic_per_token_quant(x)
    assert np.array_equal(_codes(q[:9]), _codes(q_ref)) and np.array_equal(s[:9].cpu().numpy(), s_ref.numpy())


@pytest.mark.parametrize("hidden,tokens", [(8, 515), (1000, 601), (1024, 4096), (1032, 2051), (2048, 2050),
                                           (4096, 2049), (5128, 2050), (8192, 2048), (2056, 4097)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_per_token_quant_many_short_rows_bit_exact(device, hidden, tokens, dtype):
    """Large batches of short rows take the kernel that keeps one row per wavefront (no barrier), longer rows in large
    batches the one with a workgroup per row; ragged row lengths, a row count that does not fill the last workgroup,
    strided rows, scale_ub.  Scales and codes bit-exact."""
    import vllm_amd._custom_ops as ops
    g = torch.Generator().manual_seed(hidden + tokens)
    big = (torch.randn(tokens, hidden + 16, generator=g) * 3).to(dtype)
    big[5] = 0
    ub = torch.tensor([1.5], dtype=torch.float32)
    big_dev = big.to(device)
    for lo in (0, 8):
        x = big[:, lo:lo + hidden]
        for u in (None, ub):
            q_ref, s_ref = f.ref_dynamic_per_token_quant(x, u)
            q, s = ops.scaled_fp8_quant(big_dev[:, lo:lo + hidden], scale_ub=None if u is None else u.to(device),
                                        use_per_token_if_dynamic=True)
            assert np.array_equal(s.cpu().numpy(), s_ref.numpy())
            assert np.array_equal(_codes(q), _codes(q_ref))


@pytest.mark.parametrize("hidden", [17, 1024, 5137, 14336])
@pytest.mark.parametrize("tokens", [1, 7, 300])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_per_tensor_quant_bit_exact(device, hidden, tokens, dtype):
    import vllm_amd._custom_ops as ops
    torch.manual_seed(0)
    x = (torch.rand(tokens, hidden) + 1e-6).to(dtype) * 3 - 1
    q_ref, s_ref = f.ref_dynamic_per_tensor_quant(x)
    q, s = ops.scaled_fp8_quant(x.to(device))
    assert s.shape == (1, 1) and np.array_equal(s.cpu().numpy(), s_ref.numpy())
    assert np.array_equal(_codes(q), _codes(q_ref))
    # static quantisation with the scale just computed reproduces the same codes
    q2, s2 = ops.scaled_fp8_quant(x.to(device), scale=s.reshape(1))
    assert np.array_equal(_codes(q2), _codes(q_ref))


def test_quant_large_row_count(device):
    """Many rows (the reference's int64-indexing case, test_fp8_quant.py:99-120, scaled to stay quick)."""
    import vllm_amd._custom_ops as ops
    torch.manual_seed(2)
    x = torch.randn(70000, 1152).to(torch.bfloat16)
    q_ref, s_ref = f.ref_dynamic_per_token_quant(x)
    q, s = ops.scaled_fp8_quant(x.to(device), use_per_token_if_dynamic=True)
    assert np.array_equal(s.cpu().numpy(), s_ref.numpy()) and np.array_equal(_codes(q), _codes(q_ref))


# ------------------------------------------------------------------------------------------------ scaled GEMM

def _mm_case(m, k, n, seed, per_token=True, per_channel=True, bias=True, out_dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16)
    a_q, sa = f.ref_dynamic_per_token_quant(a)
    if not per_token:
        a_q, sa = f.ref_dynamic_per_tensor_quant(a)
        sa = sa.reshape(1)
    w_q, sb = f.make_fp8_weight(n, k, seed=seed + 1)
    if not per_channel:
        w = (torch.randn(n, k, generator=g) * 0.02).to(torch.bfloat16)
        w_q, sb = f.ref_dynamic_per_tensor_quant(w)
        sb = sb.reshape(1)
    b = (torch.randn(n, generator=g) * 0.01).to(out_dtype) if bias else None
    return a_q, sa, w_q, sb, b


def _check_mm(out, ref, what):
    """Tolerance: the reference's own test uses rtol 0.5 / atol 0.15 (test_cutlass_scaled_mm.py:96); the products of
    fp8 numbers are exact and accumulation is fp32, so this build holds one output rounding:
    |out - ref| <= 2 ulp(out dtype) of max(|ref|, tiny) plus 1e-3 of the row-independent magnitude."""
    o64, r64 = out.detach().cpu().double(), ref.double()
    assert torch.isfinite(o64).all(), what
    eps = 2.0 ** -7 if out.dtype == torch.bfloat16 else 2.0 ** -10
    tol = 2 * eps * r64.abs() + 2e-3 * r64.abs().mean()
    bad = (o64 - r64).abs() > tol
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} of {bad.numel()} outside tolerance, max err {(o64 - r64).abs().max():.4e}"


MNK = [(1, 256, 128), (1, 16384, 1024), (1, 24576, 496), (16, 256, 496), (16, 16384, 128), (16, 24576, 4096),
       (32, 8192, 4096), (32, 16384, 4096), (33, 1024, 1024), (33, 8192, 128), (64, 2048, 496), (64, 16384, 1024),
       (100, 8192, 496), (128, 32768, 4096), (256, 4096, 4096), (512, 256, 1024), (512, 8192, 4096),
       (512, 16384, 128), (512, 24576, 128)]   # (M, N, K) grid of the reference's test (test_cutlass_scaled_mm.py:18-38)


@pytest.mark.parametrize("m,n,k", MNK)
@pytest.mark.parametrize("per_token,per_channel", [(True, True), (False, False)])
@pytest.mark.parametrize("bias", [False, True])
def test_scaled_mm_reference_grid(device, m, n, k, per_token, per_channel, bias):
    import vllm_amd._custom_ops as ops
    a_q, sa, w_q, sb, b = _mm_case(m, k, n, seed=m + n + k, per_token=per_token, per_channel=per_channel, bias=bias)
    ref = f.scaled_mm_ref(a_q, w_q.t(), sa, sb, torch.bfloat16, b)
    out = ops.cutlass_scaled_mm(a_q.to(device), w_q.to(device).t(), sa.to(device), sb.to(device), torch.bfloat16,
                                None if b is None else b.to(device))
    assert out.shape == (m, n) and out.dtype == torch.bfloat16
    _check_mm(out, ref, f"scaled_mm m={m} n={n} k={k}")


@pytest.mark.parametrize("m", [1, 16, 256])
def test_scaled_mm_mixed_scales_fp16_and_padded_weight(device, m):
    """per-token x per-tensor, per-tensor x per-channel, fp16 output, and a weight whose rows are padded by 256 bytes
    (b.stride(1) = K + 256, as the reference pads FP8 weights on ROCm, fp8_utils.py:952-966)."""
    import vllm_amd._custom_ops as ops
    n, k = 512, 1024
    a_q, sa, w_q, sb, b = _mm_case(m, k, n, seed=5, out_dtype=torch.float16)
    for sa_, sb_ in ((sa, sb[:1].reshape(1)), (sa[:1].reshape(1), sb)):
        ref = f.scaled_mm_ref(a_q, w_q.t(), sa_, sb_, torch.float16, b)
        out = ops.cutlass_scaled_mm(a_q.to(device), w_q.to(device).t(), sa_.to(device), sb_.to(device), torch.float16, b.to(device))
        _check_mm(out, ref, f"mixed scales m={m}")
    padded = torch.zeros(n, k + 256, dtype=torch.uint8, device=device)
    padded[:, :k] = w_q.view(torch.uint8).to(device)
    w_view = padded.view(torch.float8_e4m3fn)[:, :k].t()
    assert w_view.stride() == (1, k + 256)
    ref = f.scaled_mm_ref(a_q, w_q.t(), sa, sb, torch.float16, b)
    out = ops.cutlass_scaled_mm(a_q.to(device), w_view, sa.to(device), sb.to(device), torch.float16, b.to(device))
    _check_mm(out, ref, f"padded weight m={m}")


@pytest.mark.parametrize("seed", range(10))
def test_scaled_mm_random_shapes(device, seed):
    """Seeded sweep over irregular problems: M from 1 to 700, N and K any multiple of 16 (K not a multiple of 64 or 128
    takes the kernels' tail paths), every scale combination, bias or not, both output types."""
    import vllm_amd._custom_ops as ops
    rng = np.random.default_rng(2000 + seed)
    for _ in range(6):
        m = int(rng.choice([1, 2, 7, 16, 17, 32, 33, 63, 64, 65, 128, 200, 256, 257, 511, 700]))
        n = 16 * int(rng.integers(1, 80))
        k = 16 * int(rng.integers(1, 300))
        per_token, per_channel, bias = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        out_dtype = torch.bfloat16 if rng.integers(0, 2) else torch.float16
        a_q, sa, w_q, sb, b = _mm_case(m, k, n, seed=int(rng.integers(0, 1 << 30)), per_token=per_token,
                                       per_channel=per_channel, bias=bias, out_dtype=out_dtype)
        ref = f.scaled_mm_ref(a_q, w_q.t(), sa, sb, out_dtype, b)
        out = ops.cutlass_scaled_mm(a_q.to(device), w_q.to(device).t(), sa.to(device), sb.to(device), out_dtype,
                                    None if b is None else b.to(device))
        _check_mm(out, ref, f"m={m} n={n} k={k} per_token={per_token} per_channel={per_channel} bias={bias} {out_dtype}")
    assert all(bool((t == 0).all()) for t in ops._FP8_COUNTERS.values())


def test_scaled_mm_exact_small_integers(device):
    """With scales 1 and small-integer operands every partial sum is an exactly representable integer, so any
    dropped / duplicated k or transposed operand changes the result: the output must equal the integer GEMM."""
    import vllm_amd._custom_ops as ops
    g = torch.Generator().manual_seed(0)
    for m, n, k in ((5, 64, 272), (40, 48, 1040), (300, 320, 144)):
        a = torch.randint(-3, 4, (m, k), generator=g).float()
        w = torch.randint(-2, 3, (n, k), generator=g).float()
        one_m, one_n = torch.ones(m, 1), torch.ones(n, 1)
        out = ops.cutlass_scaled_mm(a.to(torch.float8_e4m3fn).to(device), w.to(torch.float8_e4m3fn).to(device).t(),
                                    one_m.to(device), one_n.to(device), torch.float16)
        assert torch.equal(out.cpu().float(), a @ w.t()), (m, n, k)


@pytest.mark.parametrize("m", [1, 16, 17, 32, 33, 40, 48, 49, 64, 65])
def test_scaled_mm_small_m_every_route_exact(device, m):
    """M around the switch points of the small-M routes: the weight-streaming kernel with one to four blocks of 16
    rows (three for K = 1664 .. 4096, four only up to two rounds of workgroups), with one and with several n-tiles per
    workgroup, the same kernel over two halves of K with a hand-over (16 < M <= 32 up to K = 16384),
    the tile kernel with K split over workgroups for a K beyond it (also at M <= 32) and without a split.
    Up to 32 rows the streaming kernel exists in two forms -- weights fetched in the MFMA operand layout, or as whole
    cache lines through wavefront-private LDS rings with 4, 8 or 16 K steps per wavefront -- and each case runs with the
    automatic choice, with the LDS form switched off and with each of its step counts forced (per-call tuning override).
    Small-integer operands, power-of-two scales and an integer bias: the result must equal the integer GEMM, scaled and
    shifted, rounded once to bf16; the arrival counters of the splits must be back at zero."""
    import vllm_amd._custom_ops as ops
    from vllm_amd import _tuning
    g = torch.Generator().manual_seed(m)
    for n, k in ((128, 1664), (256, 4096), (4096, 2048), (4112, 2048), (8208, 1664), (64, 1536), (128, 14336),
                 (4096, 8192 + 128), (48, 4224), (272, 8192), (4112, 5120), (128, 28672), (4112, 14336 + 256),
                 (64, 16384 + 128)):
        a = torch.randint(-2, 3, (m, k), generator=g).float()
        w = torch.randint(-1, 2, (n, k), generator=g).float()
        sa = torch.pow(2.0, -(torch.arange(m) % 2).float()).reshape(m, 1)
        sb = torch.pow(2.0, (torch.arange(n) % 3).float()).reshape(n, 1)
        bias = (torch.arange(n) % 5).float()
        want = (sa * (sb.t() * (a @ w.t())) + bias).to(torch.bfloat16)
        a_dev, w_dev = a.to(torch.float8_e4m3fn).to(device), w.to(torch.float8_e4m3fn).to(device).t()
        for lds_form in ((0, 9, 1, 2, 3) if m <= 32 else (0,)):
            switches = [0] * 15
            switches[4] = lds_form
            with _tuning.override(exp=switches):
                out = ops.cutlass_scaled_mm(a_dev, w_dev, sa.to(device), sb.to(device), torch.bfloat16,
                                            bias.to(torch.bfloat16).to(device))
            assert torch.equal(out.cpu().float(), want.float()), (m, n, k, lds_form)
    assert all(bool((t == 0).all()) for t in ops._FP8_COUNTERS.values()), "arrival counters not restored to zero"


@pytest.mark.parametrize("tokens,hidden", [(1, 17), (11, 1024), (1, 2), (4096, 64), (7, 5120), (83, 4096), (3, 17000)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("add_residual", [False, True])
@pytest.mark.parametrize("use_ub", [False, True])
def test_fused_rms_norm_per_token_quant(device, tokens, hidden, dtype, add_residual, use_ub):
    """Twin of the reference's test_rms_norm (tests/kernels/core/test_fused_quant_layernorm.py:109-200, same size grid
    and input scaling) for FP8 output.  Scales must agree to one fp32 ulp of the row statistics, the residual sum
    exactly; codes may differ from the oracle only where the last bit of `rms` (the one order-dependent quantity) moves a
    value across a rounding boundary: at most one code step, in at most 0.1 % of the elements."""
    import vllm_amd._custom_ops as ops
    g = torch.Generator().manual_seed(tokens * 31 + hidden)
    scale = 1.0 / hidden
    x = (torch.randn(tokens, hidden, generator=g) * scale).to(dtype)
    res = (torch.randn(tokens, hidden, generator=g) * scale).to(dtype) if add_residual else None
    w = (1.0 + 0.1 * torch.randn(hidden, generator=g)).to(dtype)
    ub = None
    if use_ub:
        xf = x.float() + (res.float() if res is not None else 0.0)
        normed = (xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + 1e-5)).to(dtype) * w
        ub = normed.float().mean().abs().reshape(1) + 0.05
    q_ref, s_ref, res_ref = f.ref_rms_norm_dynamic_per_token_quant(x, w, 1e-5, ub, res)
    res_dev = res.to(device).clone() if res is not None else None
    q, s = ops.rms_norm_dynamic_per_token_quant(x.to(device), w.to(device), 1e-5, torch.float8_e4m3fn,
                                                ub.to(device) if ub is not None else None, res_dev)
    assert q.shape == x.shape and q.dtype == torch.float8_e4m3fn and s.shape == (tokens, 1)
    assert torch.allclose(s.cpu(), s_ref, rtol=3e-7, atol=0)
    if add_residual:
        assert torch.equal(res_dev.cpu(), res_ref)
    a, b = _codes(q).astype(np.int32), _codes(q_ref).astype(np.int32)
    diff = a != b
    assert diff.mean() <= 1e-3, f"{diff.mean():.2e} of the codes differ"
    if diff.any():
        # neighbouring codes of the same sign differ by 1; across zero the pair is (0x00, 0x80) or a +-1 subnormal
        step = np.abs((a & 0x7f) - (b & 0x7f))[diff]
        assert step.max() <= 1, step.max()


def _assert_codes_close(q, q_ref, frac):
    a, b = _codes(q).astype(np.int32), _codes(q_ref).astype(np.int32)
    diff = a != b
    assert diff.mean() <= frac, f"{diff.mean():.2e} of the codes differ"
    if diff.any():
        assert np.abs((a & 0x7f) - (b & 0x7f))[diff].max() <= 1


@pytest.mark.parametrize("tokens,hidden", [(7, 8), (83, 768), (83, 769), (83, 5120), (4096, 64), (3, 8199), (2, 17000)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("add_residual", [False, True])
@pytest.mark.parametrize("quant_scale", [1.0, 0.01, 10.0])
@pytest.mark.parametrize("strided_input", [False, True])
def test_fused_rms_norm_static_quant(device, tokens, hidden, dtype, add_residual, quant_scale, strided_input):
    """Twin of the reference's test_fused_rms_norm_quant (tests/kernels/core/test_layernorm.py:63-153: same size grid
    corners, input scaling 1/(2*hidden), quant scales and the strided-input case).  Residual sum exact; codes equal to the
    oracle's except where the last bit of `rms` moves a value over a rounding boundary (<= 0.1 %, one code step).
    The input must be left untouched by the residual variant."""
    import vllm_amd._custom_ops as ops
    g = torch.Generator().manual_seed(tokens * 31 + hidden)
    last = 2 * hidden if strided_input else hidden
    x_base = (torch.randn(tokens, last, generator=g) / (2 * hidden)).to(dtype)
    x = x_base[..., :hidden]
    res = (torch.randn(tokens, hidden, generator=g) / (2 * hidden)).to(dtype) if add_residual else None
    w = (1.0 + 0.1 * torch.randn(hidden, generator=g)).to(dtype)
    scale = torch.tensor([quant_scale], dtype=torch.float32)
    q_ref, res_ref = f.ref_rms_norm_static_fp8_quant(x, w, scale, 1e-6, res)
    xb_dev = x_base.to(device)
    x_dev = xb_dev[..., :hidden]
    assert x_dev.is_contiguous() != strided_input or tokens == 1
    out = torch.empty(tokens, hidden, dtype=torch.float8_e4m3fn, device=device)
    if add_residual:
        res_dev = res.to(device)
        ops.fused_add_rms_norm_static_fp8_quant(out, x_dev, res_dev, w.to(device), scale.to(device), 1e-6)
        assert torch.equal(res_dev.cpu(), res_ref)
    else:
        ops.rms_norm_static_fp8_quant(out, x_dev, w.to(device), scale.to(device), 1e-6)
    assert torch.equal(xb_dev.cpu(), x_base)
    _assert_codes_close(out, q_ref, 1e-3)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("hidden", [64, 1024, 4096, 17])
def test_fused_rms_norm_quant_keeps_the_sign_of_zero(device, dtype, hidden):
    """Zeros in a row: (-0) * rms * w is -0 and its FP8 code is 0x80, (+0) gives 0x00 -- on the dynamic and the static
    kernel, rows per wavefront and per workgroup, vector and element-by-element paths.  (A 16-bit product that the
    compiler forms as a fused multiply-add with a +0 addend would turn -0 into +0.)"""
    import vllm_amd._custom_ops as ops
    tokens = 2050 if hidden <= 1024 else 3
    g = torch.Generator().manual_seed(hidden)
    x = torch.randn(tokens, hidden, generator=g).to(dtype)
    x[:, 1::4] = -0.0
    x[:, 2::4] = 0.0
    w = (torch.rand(hidden, generator=g) + 0.5).to(dtype)
    want = torch.zeros(hidden, dtype=torch.uint8)
    want[1::4] = 0x80
    zeros = torch.zeros(hidden, dtype=torch.bool)
    zeros[1::4] = True
    zeros[2::4] = True
    q, _ = ops.rms_norm_dynamic_per_token_quant(x.to(device), w.to(device), 1e-5, torch.float8_e4m3fn)
    assert torch.equal(q.cpu().view(torch.uint8)[:, zeros], want[zeros].expand(tokens, -1)), "dynamic per token"
    out = torch.empty(tokens, hidden, dtype=torch.float8_e4m3fn, device=device)
    ops.rms_norm_static_fp8_quant(out, x.to(device), w.to(device), torch.tensor([0.05], device=device), 1e-6)
    assert torch.equal(out.cpu().view(torch.uint8)[:, zeros], want[zeros].expand(tokens, -1)), "static scale"


@pytest.mark.parametrize("tokens", [1, 17, 86, 1234, 3045])
@pytest.mark.parametrize("hidden", [16, 48, 128, 1562, 4096, 28672])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_silu_and_mul_quant(device, tokens, hidden, dtype):
    """Twin of the reference's test_silu_and_mul (tests/kernels/test_fused_quant_activation.py:33-68, same size grid
    plus Llama-3-8B's 2*14336).  Codes equal to the oracle's except where the device's exponential and reciprocal and
    the CPU's exp and division differ in the last bits and that moves a value over a rounding boundary (<= 0.2 %, one
    code step)."""
    import vllm_amd._custom_ops as ops
    g = torch.Generator().manual_seed(tokens + hidden)
    scale = torch.randn(1, generator=g).abs() + 0.05
    x = torch.randn(tokens, hidden, generator=g).to(dtype)
    out = torch.empty(tokens, hidden // 2, dtype=torch.float8_e4m3fn, device=device)
    ops.silu_and_mul_quant(out, x.to(device), scale.to(device))
    _assert_codes_close(out, f.ref_silu_and_mul_quant(x, scale), 2e-3)
    # 3-d input, as the layer passes it
    if tokens == 86:
        x3 = x.reshape(2, 43, hidden)
        out3 = torch.empty(2, 43, hidden // 2, dtype=torch.float8_e4m3fn, device=device)
        ops.silu_and_mul_quant(out3, x3.to(device), scale.to(device))
        assert torch.equal(out3.reshape(tokens, -1).view(torch.uint8), out.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_silu_and_mul_quant_saturation(device, dtype):
    """Gate values where the exponential overflows or underflows, signed zeros and +inf: the codes of the oracle, on both
    the 8-element and the element-by-element path of the kernel."""
    import vllm_amd._custom_ops as ops
    gate = torch.tensor([-1e4, -200.0, -100.0, -89.0, -88.0, -87.0, -30.0, -20.0, -0.0, 0.0, 20.0, 30.0, 88.0, 100.0,
                         1e4, float("inf"), 2.0, -2.0, 1.0, -1.0, 0.5, -0.5, 3.0, -3.0])
    for d in (24, 21):      # d % 8 == 0: vector path; otherwise scalar path
        x = torch.cat([gate[:d], torch.full((d,), 1.5)]).to(dtype).reshape(1, 2 * d).repeat(3, 1)
        out = torch.empty(3, d, dtype=torch.float8_e4m3fn, device=device)
        scale = torch.tensor([0.25])
        ops.silu_and_mul_quant(out, x.to(device), scale.to(device))
        ref = f.ref_silu_and_mul_quant(x, scale)
        assert torch.equal(out.cpu().view(torch.uint8), ref.view(torch.uint8)), (dtype, d)


@pytest.mark.parametrize("offset", [0, 4, 8])
def test_scaled_mm_into_a_view_of_a_wider_buffer(device, offset):
    """The registered op writes into the tensor it is given: a column range of a wider buffer (row stride a multiple of
    16 elements).  An offset of 4 elements starts the rows 8 bytes off a 16-byte boundary, which takes the tile kernel's
    8-byte store path instead of the LDS-staged 16-byte one; every element outside the view must stay untouched."""
    import vllm_amd._custom_ops as ops
    g = torch.Generator().manual_seed(offset)
    for m, n, k in ((300, 384, 512), (70, 256, 1024), (4, 128, 256)):
        a = torch.randint(-2, 3, (m, k), generator=g).float()
        w = torch.randint(-1, 2, (n, k), generator=g).float()
        big = torch.full((m, n + 32), 7.0, dtype=torch.bfloat16, device=device)
        view = big[:, offset:offset + n]
        torch.ops.vllm_amd.cutlass_scaled_mm(view, a.to(torch.float8_e4m3fn).to(device),
                                             w.to(torch.float8_e4m3fn).to(device).t(), torch.ones(m, 1, device=device),
                                             torch.ones(n, 1, device=device), None)
        got = big.cpu().float()
        assert torch.equal(got[:, offset:offset + n], a @ w.t()), (offset, m, n, k)
        assert bool((got[:, :offset] == 7).all()) and bool((got[:, offset + n:] == 7).all()), "wrote outside the view"


@pytest.mark.parametrize("cfg", [1, 8, 2, 10, 11, 3, 4, 5, 7, 9, 13, 23, 14, 24, 15, 16, 17])
def test_scaled_mm_every_tile_shape_exact(device, cfg):
    """Every shape of the multi-stage tile kernel, forced through a per-call tuning override (the automatic choice only reaches
    some of them at any one problem size), including the ones that take two k-slices per step: small-integer operands
    make the fp32 accumulation exact, so the result must equal the integer GEMM, also with K split over workgroups."""
    import vllm_amd._custom_ops as ops
    from vllm_amd import _tuning
    g = torch.Generator().manual_seed(cfg)
    for m, n, k, split in ((300, 384, 1024, 0), (64, 256, 8192 + 128, 2), (513, 512, 640, 0), (257, 272, 384, 0),
                           (100, 128, 448, 0), (520, 256, 64 * 13, 3), (70, 320, 128, 0), (258, 256, 256, 0),
                           (256, 512, 128 * 11, 3), (33, 64, 128 * 7, 5)):
        a = torch.randint(-2, 3, (m, k), generator=g).float()
        w = torch.randint(-1, 2, (n, k), generator=g).float()
        with _tuning.override(fp8_tile_cfg=cfg, fp8_split=split):
            out = ops.cutlass_scaled_mm(a.to(torch.float8_e4m3fn).to(device), w.to(torch.float8_e4m3fn).to(device).t(),
                                        torch.ones(m, 1, device=device), torch.ones(n, 1, device=device), torch.float16)
        assert torch.equal(out.cpu().float(), a @ w.t()), (cfg, m, n, k)
    for t in ops._FP8_COUNTERS.values():
        assert bool((t == 0).all()), "arrival counters not restored to zero"


@pytest.mark.parametrize("m,n,k", [(17 * 256, 4096, 2048), (21 * 256 - 5, 3328, 2048)])
def test_scaled_mm_tiles_of_last_round_split_exact(device, m, n, k):
    """More 256 x 256 tiles than compute units with a last round of workgroups at most half full (17 x 16 tiles on 256
    units; 21 x 13 with a ragged last tile row, whose 17 left-over tiles are no multiple of the 8 XCDs): the tiles of
    that round run in K parts, the others whole -- the library says so through the scratch it asks
    for.  Small-integer operands make every partial sum exact: the result must equal the integer GEMM on every tile,
    twice in a row, and the arrival counters return to zero."""
    import ctypes
    import vllm_amd._custom_ops as ops
    from vllm_amd import _lib
    lib = _lib.load()
    cus = lib.vaq_num_cus(torch.device(device).index or 0)
    tiles = ((m + 255) // 256) * (n // 256)
    if not (tiles > cus and 0 < tiles % cus <= cus // 2):
        pytest.skip(f"{tiles} tiles on {cus} compute units leave no half-empty last round")
    sizes = [ctypes.c_size_t() for _ in range(2)]
    _lib.check(lib.vaq_fp8_scaled_mm_workspace(m, n, k, *map(ctypes.byref, sizes)))
    rest, parts = tiles % cus, min(cus // (tiles % cus), 4, k // 64 // 16)
    assert sizes[0].value == rest * parts * 256 * 256 * 4, "the plan does not split exactly the tiles of the last round"
    g = torch.Generator().manual_seed(2)
    a = torch.randint(-2, 3, (m, k), generator=g).float()
    w = torch.randint(-1, 2, (n, k), generator=g).float()
    args = (a.to(torch.float8_e4m3fn).to(device), w.to(torch.float8_e4m3fn).to(device).t(),
            torch.ones(m, 1, device=device), torch.ones(n, 1, device=device), torch.float16)
    ref = (a.to(device) @ w.to(device).t()).cpu()
    for rep in range(2):
        assert torch.equal(ops.cutlass_scaled_mm(*args).cpu().float(), ref), f"run {rep}"
    assert all(bool((t == 0).all()) for t in ops._FP8_COUNTERS.values()), "arrival counters not restored to zero"


@pytest.mark.parametrize("m,n,k", [(320, 4096, 2048), (512, 4096, 4096), (1000, 2048, 2048 + 64), (200, 4096, 4096 + 192),
                                   (1024, 6144, 4096), (72, 6656, 1024), (200, 28672, 1024 + 64), (100, 32768, 512 + 64)])
def test_scaled_mm_rotated_k_loop_exact(device, m, n, k):
    """Unsplit tiles that fit one round of workgroups over small weights: every tile row starts its K loop at a
    different step and wraps around (2 to 16 tile rows here, step counts that the number of tile rows does not divide);
    a single tile row on a wide layer: every tile column does (the last two cases).
    Small-integer operands that differ from step to step make the sum exact: a step read twice or not at all changes it."""
    import vllm_amd._custom_ops as ops
    g = torch.Generator().manual_seed(m + k)
    a = torch.randint(-2, 3, (m, k), generator=g).float()
    w = torch.randint(-1, 2, (n, k), generator=g).float()
    out = ops.cutlass_scaled_mm(a.to(torch.float8_e4m3fn).to(device), w.to(torch.float8_e4m3fn).to(device).t(),
                                torch.ones(m, 1, device=device), torch.ones(n, 1, device=device), torch.float16)
    assert torch.equal(out.cpu().float(), a @ w.t())


@pytest.mark.parametrize("m,n,k", [(64, 4096, 4096), (50, 6144, 4096), (33, 8192, 4096), (100, 4096, 2048), (192, 4096, 1024),
                                   (384, 6144, 512), (130, 2048, 2048), (70, 5120, 5120), (190, 2048, 6656),
                                   (320, 4096, 4096), (136, 6144, 4096), (264, 4608, 3584),
                                   (64, 2048, 7168), (190, 1024, 8192), (100, 2048, 8192 + 64)])
def test_scaled_mm_tile_row_past_m_exact(device, m, n, k):
    """Up to three tile rows with compute units to spare: one more row of workgroups runs past M beside them (it reads the
    same weights, its activation rows do not exist, it stores nothing).  Small-integer operands: the result must equal
    the integer GEMM and two runs must agree (the activations come as the first M rows of a taller buffer whose other
    rows are not zero).  Three cases run 128 x 64 tiles, which the planner takes where such a row fits beside them and beside
    64 x 64 tiles it would not (the second of them without the extra row: too many tile columns).  The last three cases
    split K over workgroups as well: the extra row's workgroups take no part
    in the hand-over, and the arrival counters return to zero."""
    import vllm_amd._custom_ops as ops
    g = torch.Generator().manual_seed(m * 7 + k)
    a = torch.randint(-2, 3, (m, k), generator=g).float()
    w = torch.randint(-1, 2, (n, k), generator=g).float()
    a_dev = torch.zeros(m + 200, k, dtype=torch.float8_e4m3fn, device=device)      # rows past M exist in memory and are not zero
    a_dev[m:] = torch.ones(200, k).to(torch.float8_e4m3fn).to(device)
    a_dev[:m] = a.to(torch.float8_e4m3fn).to(device)
    args = (a_dev[:m], w.to(torch.float8_e4m3fn).to(device).t(), torch.ones(m, 1, device=device), torch.ones(n, 1, device=device),
            torch.float16)
    out = ops.cutlass_scaled_mm(*args)
    assert out.shape == (m, n)
    assert torch.equal(out.cpu().float(), a @ w.t())
    assert torch.equal(out, ops.cutlass_scaled_mm(*args))
    assert all(bool((t == 0).all()) for t in ops._FP8_COUNTERS.values()), "arrival counters not restored to zero"


@pytest.mark.parametrize("seed", range(8))
def test_scaled_mm_random_mid_m_exact(device, seed):
    """Seeded sweep through the tile planner's middle: 33 .. 420 rows on layers of 1024 .. 8320 columns and K = 512 .. 8320
    (some not a multiple of 64 or 128), where the automatic choice moves between tile shapes, K parts, rotated K loops and
    the tile row past M.  Small-integer operands, power-of-two scales and an integer bias keep every step exact: the
    result must equal the scaled integer GEMM, whichever plan ran, and the arrival counters must be back at zero."""
    import vllm_amd._custom_ops as ops
    rng = np.random.default_rng(7000 + seed)
    g = torch.Generator().manual_seed(7000 + seed)
    for _ in range(5):
        m = int(rng.integers(33, 421))
        n = 16 * int(rng.integers(64, 521))
        k = 64 * int(rng.integers(8, 131)) + int(rng.choice([0, 0, 0, 16, 32]))
        a = torch.randint(-2, 3, (m, k), generator=g).float()
        w = torch.randint(-1, 2, (n, k), generator=g).float()
        sa = torch.tensor(rng.choice([0.5, 1.0], size=(m, 1)), dtype=torch.float32)
        sb = torch.tensor(rng.choice([0.5, 1.0], size=(n, 1)), dtype=torch.float32)
        bias = torch.randint(-3, 4, (n,), generator=g).to(torch.float16) if rng.integers(0, 2) else None
        ref = (a @ w.t()) * sa * sb.t() + (0 if bias is None else bias.float())
        out = ops.cutlass_scaled_mm(a.to(torch.float8_e4m3fn).to(device), w.to(torch.float8_e4m3fn).to(device).t(),
                                    sa.to(device), sb.to(device), torch.float16, None if bias is None else bias.to(device))
        assert torch.equal(out.cpu().float(), ref), (m, n, k, bias is not None)
    assert all(bool((t == 0).all()) for t in ops._FP8_COUNTERS.values()), "arrival counters not restored to zero"


def test_scaled_mm_split_k_exact_and_deterministic(device):
    """Few output tiles and a long K: the tile kernel splits K over workgroups (fp32 partial tiles through the op's
    scratch, arrival counters left zero).  Small-integer operands make every partial sum exact, so the split result
    must equal the integer GEMM; two runs must agree bit for bit."""
    import vllm_amd._custom_ops as ops
    g = torch.Generator().manual_seed(1)
    for m, n, k in ((200, 256, 14336), (96, 128, 8192 + 64), (257, 384, 16384)):
        a = torch.randint(-2, 3, (m, k), generator=g).float()
        w = torch.randint(-1, 2, (n, k), generator=g).float()
        args = (a.to(torch.float8_e4m3fn).to(device), w.to(torch.float8_e4m3fn).to(device).t(),
                torch.ones(m, 1, device=device), torch.ones(n, 1, device=device), torch.float16)
        out = ops.cutlass_scaled_mm(*args)
        assert torch.equal(out.cpu().float(), a @ w.t()), (m, n, k)
        assert torch.equal(out, ops.cutlass_scaled_mm(*args))
        assert all(bool((t == 0).all()) for t in ops._FP8_COUNTERS.values()), "arrival counters not restored to zero"


@pytest.mark.parametrize("k,n", [(13824, 5120), (6656, 6656), (18944, 3584), (9216, 4608), (5120, 5120), (1024, 18944)])
def test_tile_plan_branches_other_model_shapes(device, k, n):
    """Layer shapes of other models on which the tile planner takes branches that the Llama-3-8B shapes do not reach
    (K parts rebalanced to one workgroup per compute unit, an unsplit K from 60 % fill on, 256 x 256 tiles in parts of
    a long K, 128 x 128 instead of 64 x 128 tiles for long parts, two m-blocks of K up to 8192 through LDS rings,
    256 x 128 tiles for one tile row of a wide layer):
    per-token x per-channel with bias, sampled rows against the fp64 oracle, bit-identical run to run, arrival
    counters back at zero."""
    import vllm_amd._custom_ops as ops
    w_q, sb = f.make_fp8_weight(n, k, seed=3)
    w_dev = w_q.to(device).t()
    g = torch.Generator().manual_seed(4)
    bias = (torch.randn(n, generator=g) * 0.01).to(torch.bfloat16)
    for m in (24, 32, 65, 96, 136, 192, 256, 384, 640, 896):
        a = torch.randn(m, k, generator=g).to(torch.bfloat16)
        a_q, sa = ops.scaled_fp8_quant(a.to(device), use_per_token_if_dynamic=True)
        rows = np.concatenate([np.random.default_rng(m).choice(m, 14, replace=False), [0, m - 1]])
        out = ops.cutlass_scaled_mm(a_q, w_dev, sa, sb.to(device), torch.bfloat16, bias.to(device))
        ref = f.scaled_mm_ref(a_q[rows].cpu(), w_q.t(), sa[rows].cpu(), sb, torch.bfloat16, bias)
        _check_mm(out[rows], ref, f"k={k} n={n} m={m}")
        assert torch.isfinite(out.float()).all()
        again = ops.cutlass_scaled_mm(a_q, w_dev, sa, sb.to(device), torch.bfloat16, bias.to(device))
        assert torch.equal(out, again), f"k={k} n={n} m={m}: not deterministic run to run"
    assert all(bool((t == 0).all()) for t in ops._FP8_COUNTERS.values())


@pytest.mark.parametrize("k,n", LLAMA_SHAPES)
def test_config4_llama_shapes(device, k, n):
    """BASELINE.json config 4: M in {1, 16, 256, 4096}, per-token x per-channel (+bias); activations quantised on the GPU
    (bit-exact with the oracle), M = 4096 checked on sampled rows."""
    import vllm_amd._custom_ops as ops
    w_q, sb = f.make_fp8_weight(n, k, seed=1)
    w_dev = w_q.to(device).t()
    g = torch.Generator().manual_seed(2)
    bias = (torch.randn(n, generator=g) * 0.01).to(torch.bfloat16)
    for m in (1, 16, 256, 4096):
        a = torch.randn(m, k, generator=g).to(torch.bfloat16)
        a_q, sa = ops.scaled_fp8_quant(a.to(device), use_per_token_if_dynamic=True)
        rows = np.arange(m) if m <= 256 else np.concatenate([np.random.default_rng(m).choice(m, 30, replace=False), [0, m - 1]])
        a_ref, sa_ref = f.ref_dynamic_per_token_quant(a[rows])
        assert np.array_equal(_codes(a_q[rows]), _codes(a_ref)) and np.array_equal(sa[rows].cpu().numpy(), sa_ref.numpy())
        out = ops.cutlass_scaled_mm(a_q, w_dev, sa, sb.to(device), torch.bfloat16, bias.to(device))
        ref = f.scaled_mm_ref(a_ref, w_q.t(), sa_ref, sb, torch.bfloat16, bias)
        _check_mm(out[rows], ref, f"config 4 k={k} n={n} m={m}")
        assert torch.isfinite(out.float()).all()


def test_scaled_mm_split_k_on_two_streams_at_once(device):
    """Two split-K GEMMs in flight on two streams: each stream has its own arrival counters, so the results must equal the
    ones computed one after the other (small-integer operands: every partial sum is exact, any lost or doubled partial
    tile changes the result)."""
    import vllm_amd._custom_ops as ops
    g = torch.Generator().manual_seed(21)
    probs = []
    for m, n, k in ((200, 256, 14336), (96, 384, 16384)):
        a = torch.randint(-2, 3, (m, k), generator=g).float()
        w = torch.randint(-1, 2, (n, k), generator=g).float()
        probs.append(((a.to(torch.float8_e4m3fn).to(device), w.to(torch.float8_e4m3fn).to(device).t(),
                       torch.ones(m, 1, device=device), torch.ones(n, 1, device=device), torch.float16), a @ w.t()))
    serial = [ops.cutlass_scaled_mm(*args) for args, _ in probs]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[], []]
    for _ in range(20):
        for i, st in enumerate(streams):
            with torch.cuda.stream(st):
                outs[i].append(ops.cutlass_scaled_mm(*probs[i][0]))
    torch.cuda.synchronize()
    keys = {key for key in ops._FP8_COUNTERS if key[1] in (streams[0].cuda_stream, streams[1].cuda_stream)}
    assert len(keys) == 2, "each stream must own its arrival counters"
    for i in range(2):
        assert torch.equal(serial[i].cpu().float(), probs[i][1])
        for o_ in outs[i]:
            assert torch.equal(o_, serial[i]), f"stream {i}: concurrent result differs from the serial one"
    assert all(bool((t == 0).all()) for t in ops._FP8_COUNTERS.values()), "arrival counters not restored to zero"


def test_scaled_mm_split_k_first_call_under_graph_capture(device):
    """A stream whose first split-K GEMM happens inside a HIP graph capture: the op takes zeroed counters from the
    capture's own pool (a fill kernel, no memset node), and every replay gives the eager result."""
    import vllm_amd._custom_ops as ops
    g = torch.Generator().manual_seed(22)
    m, n, k = 200, 256, 14336
    a = torch.randint(-2, 3, (m, k), generator=g).float()
    w = torch.randint(-1, 2, (n, k), generator=g).float()
    args = (a.to(torch.float8_e4m3fn).to(device), w.to(torch.float8_e4m3fn).to(device).t(),
            torch.ones(m, 1, device=device), torch.ones(n, 1, device=device), torch.float16)
    eager = ops.cutlass_scaled_mm(*args)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):          # runs on a fresh side stream that has no cached counters
        out = ops.cutlass_scaled_mm(*args)
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager) and torch.equal(out.cpu().float(), a @ w.t())
        assert torch.equal(ops.cutlass_scaled_mm(*args), eager)      # eager work between the replays
