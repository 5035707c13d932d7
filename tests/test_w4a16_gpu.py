"""GPU parity tests of the W4A16 path (repack, decode GEMM, prefill GEMM) against the CPU oracle, through the op
surface that sits on the C ABI."""
import numpy as np
import pytest
import torch

from oracle import native_layout as nl
from oracle import w4a16 as o
from tests.helpers import W4A16Layer, check_gemm_close, to_dev

pytestmark = pytest.mark.gpu

LLAMA_SHAPES = [(4096, 6144), (4096, 4096), (4096, 28672), (14336, 4096)]


def _acts(m, k, device, dtype=torch.bfloat16, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(m, k, generator=g).to(dtype).to(device)


@pytest.fixture(params=["auto", "lds_staged", "register_resident"])
def decode_kernel(request):
    """Runs a test once with the library's own choice of decode kernel and once with each of the two kernels forced, so
    that both are checked on every shape whichever one the selection rule would pick."""
    from vllm_amd import _tuning
    with _tuning.override(decode_impl={"auto": 0, "lds_staged": 1, "register_resident": 2}[request.param]):
        yield request.param


# ------------------------------------------------------------------------------------------------ repack

@pytest.mark.parametrize("k,n", [(128, 64), (128, 256), (1024, 256), (128 * 13, 64 * 37), (128 * 11, 64 * 13), (4096, 4096)])
@pytest.mark.parametrize("act_order", [False, True])
def test_repack_bit_exact_both_layouts(device, k, n, act_order):
    import vllm_amd._custom_ops as ops
    rng = np.random.default_rng(k + n)
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    qw = to_dev(o.gptq_pack(q, 4), device)
    if act_order:
        perm_np = rng.permutation(k).astype(np.int32)
        perm = to_dev(perm_np, device)
        q_sorted = q[perm_np]
    else:
        perm = torch.empty(0, dtype=torch.int32, device=device)
        q_sorted = q
    marlin = ops.gptq_marlin_repack(qw, perm, k, n, 4, layout="marlin")
    native = ops.gptq_marlin_repack(qw, perm, k, n, 4)
    assert marlin.shape == native.shape == (k // 16, 2 * n) and marlin.dtype == torch.int32
    assert np.array_equal(marlin.cpu().numpy(), o.marlin_weights(q_sorted)), "marlin order differs from the oracle"
    assert np.array_equal(native.cpu().numpy(), nl.native_pack(q_sorted)), "native order differs from its spec"
    assert np.array_equal(nl.native_unpack(native.cpu().numpy(), k, n), q_sorted)


@pytest.mark.parametrize("k,n", [(128, 64), (128, 256), (1024, 256), (128 * 13, 64 * 37), (4096, 4096)])
def test_awq_repack_bit_exact_both_layouts(device, k, n):
    """Twin of the reference's test_awq_marlin_repack (test_marlin_gemm.py:168-209): AWQ-packed codes -> Marlin order
    must equal the host construction `marlin_weights`; the native order must equal its specification."""
    import vllm_amd._custom_ops as ops
    rng = np.random.default_rng(k * 7 + n)
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    qw = to_dev(o.awq_pack(q, 4), device)
    assert qw.shape == (k, n // 8)
    marlin = ops.awq_marlin_repack(qw, k, n, 4, layout="marlin")
    native = ops.awq_marlin_repack(qw, k, n, 4)
    assert marlin.shape == native.shape == (k // 16, 2 * n) and marlin.dtype == torch.int32
    assert np.array_equal(marlin.cpu().numpy(), o.marlin_weights(q)), "marlin order differs from the oracle"
    assert np.array_equal(native.cpu().numpy(), nl.native_pack(q)), "native order differs from its spec"
    # the same codes through the GPTQ packing give the same bytes
    assert torch.equal(native, ops.gptq_marlin_repack(to_dev(o.gptq_pack(q, 4), device),
                                                      torch.empty(0, dtype=torch.int32, device=device), k, n, 4))


@pytest.mark.parametrize("k,n", [(128, 64), (1024, 256), (128 * 13, 64 * 37), (4096, 4096)])
@pytest.mark.parametrize("act_order", [False, True])
def test_repack_8bit_bit_exact_both_layouts(device, k, n, act_order):
    """num_bits = 8 of the reference's test_gptq_marlin_repack (test_marlin_gemm.py:98-156): the Marlin order must equal
    the host construction, the native order (two nibble planes per tile) its specification."""
    import vllm_amd._custom_ops as ops
    rng = np.random.default_rng(k + n + 8)
    q = rng.integers(0, 256, size=(k, n), dtype=np.int32)
    qw = to_dev(o.gptq_pack(q, 8), device)
    if act_order:
        perm_np = rng.permutation(k).astype(np.int32)
        perm = to_dev(perm_np, device)
        q_sorted = q[perm_np]
    else:
        perm = torch.empty(0, dtype=torch.int32, device=device)
        q_sorted = q
    marlin = ops.gptq_marlin_repack(qw, perm, k, n, 8, layout="marlin")
    native = ops.gptq_marlin_repack(qw, perm, k, n, 8)
    assert marlin.shape == native.shape == (k // 16, 4 * n) and marlin.dtype == torch.int32
    assert np.array_equal(marlin.cpu().numpy(), o.marlin_weights(q_sorted, 8)), "marlin order differs from the oracle"
    assert np.array_equal(native.cpu().numpy(), nl.native_pack8(q_sorted)), "native order differs from its spec"


# ------------------------------------------------------------------------------------------------ permute_cols

@pytest.mark.parametrize("m,k", [(1, 128), (3, 1024), (7, 4096), (130, 14336), (5, 70000)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_permute_cols_bit_exact(device, m, k, dtype):
    """out[:, j] = a[:, perm[j]] (reference: permute_cols.cu, used by the act_order path); rows may be a strided view.
    K = 70000 exceeds what the LDS-staged kernel holds and takes the direct-gather kernel."""
    import vllm_amd._custom_ops as ops
    g = torch.Generator().manual_seed(m * 131 + k)
    big = torch.randn(m, k + 24, generator=g).to(dtype)
    perm = torch.randperm(k, generator=g).to(torch.int32)
    big_dev = big.to(device)
    for lo, contiguous in ((0, True), (8, False), (3, False)):
        a_cpu = big[:, lo:lo + k]
        a_dev = big_dev[:, lo:lo + k].contiguous() if contiguous else big_dev[:, lo:lo + k]
        out = ops.permute_cols(a_dev, perm.to(device))
        assert out.shape == (m, k) and out.dtype == dtype and out.is_contiguous()
        assert torch.equal(out.cpu().view(torch.int16), a_cpu[:, perm.long()].contiguous().view(torch.int16))


# ------------------------------------------------------------------------------------------------ GEMM, small shapes

SMALL = [(128, 64), (512, 256), (1024, 192), (2048, 576), (14336 // 4, 128)]


@pytest.mark.parametrize("k,n", SMALL)
@pytest.mark.parametrize("m", [1, 3, 4, 5, 8, 16, 17, 32])
@pytest.mark.parametrize("asym,act_order", [(False, False), (True, False), (False, True), (True, True)])
def test_decode_gemm_small(device, decode_kernel, k, n, m, asym, act_order):
    if act_order and k == 128:
        pytest.skip("act_order needs more than one group (gptq_marlin.cu:805)")
    case = o.make_w4a16_case(k, n, 128, asym=asym, act_order=act_order, seed=k + n + m)
    layer = W4A16Layer(case, device)
    a = _acts(m, k, device, seed=m)
    out = layer(a)
    assert out.shape == (m, n) and out.dtype == torch.bfloat16
    check_gemm_close(out, o.gemm_ref(a.cpu(), o.case_w_ref(case)), f"decode k={k} n={n} m={m}")
    assert bool((layer.workspace == 0).all()), "workspace counters not restored to zero"


@pytest.mark.parametrize("kernel", ["lds_staged", "register_resident"])
@pytest.mark.parametrize("m", [1, 5, 16, 29])
def test_decode_gemm_forced_split_k(device, kernel, m):
    """K split over several workgroups on both decode kernels (forced through a per-call tuning override: the automatic
    choice only splits a long K): partial tiles through `c_tmp`, arrival counters in `workspace`.  Against the oracle,
    twice for determinism, counters left zero."""
    from vllm_amd import _tuning
    k, n = 2048, 320
    case = o.make_w4a16_case(k, n, 128, asym=True, seed=90 + m)
    layer = W4A16Layer(case, device)
    a = _acts(m, k, device, seed=m)
    if kernel == "lds_staged":
        forced = dict(decode_impl=1, decode2_gs=2, decode2_wks=2, decode2_wn=1)      # slabs of 4 groups: 4 splits
    else:
        forced = dict(decode_impl=2, decode_tg=1, decode_wk=4)      # 4 wavefronts of 1 group: 4 (M <= 16) splits
    with _tuning.override(**forced):
        out = layer(a)
        check_gemm_close(out, o.gemm_ref(a.cpu(), o.case_w_ref(case)), f"forced split-K {kernel} m={m}")
        assert torch.equal(out, layer(a)), "split-K result is not deterministic run to run"
    assert bool((layer.workspace == 0).all()), "workspace counters not restored to zero"


@pytest.mark.parametrize("k,n", SMALL)
@pytest.mark.parametrize("m", [33, 64, 200, 257])
@pytest.mark.parametrize("asym,act_order", [(False, False), (True, True)])
def test_prefill_gemm_small(device, k, n, m, asym, act_order):
    if act_order and k == 128:
        pytest.skip("act_order needs more than one group (gptq_marlin.cu:805)")
    case = o.make_w4a16_case(k, n, 128, asym=asym, act_order=act_order, seed=k + n + m)
    layer = W4A16Layer(case, device)
    a = _acts(m, k, device, seed=m)
    out = layer(a)
    check_gemm_close(out, o.gemm_ref(a.cpu(), o.case_w_ref(case)), f"prefill k={k} n={n} m={m}")


@pytest.mark.parametrize("k,n,m", [(4096, 256, 64), (4096, 512, 130), (3584, 1024, 257), (14336, 128, 48)])
@pytest.mark.parametrize("asym", [False, True])
def test_prefill_gemm_split_k(device, k, n, m, asym):
    """Few output tiles and a long K: the tile kernel splits K over workgroups (fp32 partial tiles, arrival counters in
    `workspace`, summed in split order by the last arriver).  Checked against the oracle, run twice for determinism,
    counters left zero."""
    case = o.make_w4a16_case(k, n, 128, asym=asym, seed=k + n + m)
    layer = W4A16Layer(case, device)
    a = _acts(m, k, device, seed=m)
    out = layer(a)
    check_gemm_close(out, o.gemm_ref(a.cpu(), o.case_w_ref(case)), f"split-K prefill k={k} n={n} m={m}")
    assert torch.equal(out, layer(a)), "split-K result is not deterministic run to run"
    assert bool((layer.workspace == 0).all()), "workspace counters not restored to zero"


@pytest.mark.parametrize("asym", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_prefill_every_tile_shape(device, asym, dtype):
    """Every tile shape of the prefill kernels, forced through a per-call tuning override (the automatic choice only reaches some of
    them at any one problem size), with and without K split over workgroups, against the oracle.  The direct-to-LDS
    shapes (ids 10-15 and 20, the one with alternating phases) dequantise exactly and add the same MFMA products in the
    same order, so without a K split they must agree with each other bit for bit."""
    from vllm_amd import _tuning
    for k, n, m in ((1024, 512, 300), (640, 320, 513), (384, 256, 257), (2048, 576, 70)):
        case = o.make_w4a16_case(k, n, 128, asym=asym, seed=k + n + m)
        layer = W4A16Layer(case, device, dtype)
        a = _acts(m, k, device, dtype, seed=m)
        ref = o.gemm_ref(a.cpu(), o.case_w_ref(case))
        first = None
        for tile in (10, 20, 11, 12, 13, 14, 15, 30, 0, 1, 2):
            for split in ((1, 0, 2, 3) if tile >= 10 else (0,)):      # 0: the automatic split, 1: none
                with _tuning.override(prefill_tile=tile + 1, prefill_split=split):
                    out = layer(a)
                check_gemm_close(out, ref, f"tile {tile} split {split} k={k} n={n} m={m}")
                # (tile 30 dequantises in registers and pairs other k-octets in an MFMA: same products, another order)
                if 10 <= tile < 30 and split == 1:
                    if first is None:
                        first = out
                    assert torch.equal(out, first), f"tile {tile} differs from tile 10 (k={k} n={n} m={m})"
        assert bool((layer.workspace == 0).all()), "workspace counters not restored to zero"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("asym", [False, True])
def test_prefill_register_dequant_tile(device, dtype, asym):
    """The 256 x 256 tile whose weights are dequantised in registers (tile id 30), forced: one-hot activations return
    rn16((q - z) * s) bit for bit (every k-octet lands in the MFMA slot its activation chunk is read for, every column in
    its lane after the lane swap), ragged M and N (columns past N, rows past M, a last tile of one 64-column strip),
    one to many K steps, channelwise scales, and K split over workgroups."""
    from vllm_amd import _tuning
    for k, n, g in ((128, 64, 128), (256, 320, 128), (1024, 576, 128), (512, 256, -1), (2560, 832, 128)):
        case = o.make_w4a16_case(k, n, g, asym=asym, dtype=dtype, seed=k + n)
        layer = W4A16Layer(case, device, dtype)
        w = o.case_w_ref(case)
        for m in (65, 256, 300):
            rows = [(37 * i + 32 * (i % 4) + m) % k for i in range(m)]
            a = torch.zeros(m, k, dtype=dtype)
            for i, r in enumerate(rows):
                a[i, r] = 1
            with _tuning.override(prefill_tile=31, prefill_split=1):
                assert torch.equal(layer(a.to(device)).cpu(), w[rows]), f"one-hot k={k} n={n} m={m}"
            a = _acts(m, k, device, dtype, seed=m)
            ref = o.gemm_ref(a.cpu(), w)
            for split in (1, 0, 2, 5):
                with _tuning.override(prefill_tile=31, prefill_split=split):
                    out = layer(a)
                    check_gemm_close(out, ref, f"tile 30 split {split} k={k} n={n} m={m}")
                    assert torch.equal(out, layer(a)), "not deterministic run to run"
        assert bool((layer.workspace == 0).all()), "workspace counters not restored to zero"


@pytest.mark.parametrize("k,n,m", [(2048, 4096, 17 * 256), (2048, 3328, 21 * 256 - 5)])
@pytest.mark.parametrize("asym,group_size", [(False, 128), (True, 128), (True, 32)])
def test_prefill_tiles_of_last_round_split(device, asym, group_size, k, n, m):
    """More 256 x 256 tiles than compute units with a last round of workgroups at most half full (17 x 16 tiles on 256
    units; 21 x 13 with a ragged last tile row, whose 17 left-over tiles are no multiple of the 8 XCDs): the tiles of
    that round run in K parts, the others whole.  The library says so through the scratch it asks
    for; one-hot activations come back exact from every tile, split or whole; against the same kernel with every tile
    whole the result is equal on the whole tiles' rows and one rounding apart elsewhere; counters return to zero.
    Groups of 32 rows take the same plan on the instances for groups below 128 rows."""
    from vllm_amd import _lib, _tuning
    import ctypes
    lib = _lib.load()
    cus = lib.vaq_num_cus(torch.device(device).index or 0)
    tiles = ((m + 255) // 256) * (n // 256)
    if not (tiles > cus and 0 < tiles % cus <= cus // 2):
        pytest.skip(f"{tiles} tiles on {cus} compute units leave no half-empty last round")
    sizes = [ctypes.c_size_t() for _ in range(3)]
    _lib.check(lib.vaq_w4a16_gemm_workspace(m, n, k, 0, 0, *map(ctypes.byref, sizes)))
    rest, parts = tiles % cus, min(cus // (tiles % cus), 4, k // 128 // 8)
    assert sizes[0].value == rest * parts * 256 * 256 * 4, "the plan does not split exactly the tiles of the last round"
    case = o.make_w4a16_case(k, n, group_size, asym=asym, seed=5)
    layer = W4A16Layer(case, device)
    w = o.case_w_ref(case)
    rows = [(37 * i + 32 * (i % 4)) % k for i in range(m)]
    a = torch.zeros(m, k, dtype=torch.bfloat16)
    a[torch.arange(m), torch.tensor(rows)] = 1
    assert torch.equal(layer(a.to(device)).cpu(), w[rows]), "one-hot rows through split and whole tiles"
    a = _acts(m, k, device, seed=3)
    out = layer(a)
    assert torch.equal(out, layer(a)), "not deterministic run to run"
    check_gemm_close(out[-512:], o.gemm_ref(a[-512:].cpu(), w), "rows of split and of whole tiles against the oracle")
    for tile in ((20, 30) if group_size == 128 else (10,)):      # the same tile kernel with and without the split
        with _tuning.override(prefill_tile=tile + 1):
            out = layer(a)
        with _tuning.override(prefill_tile=tile + 1, exp=[0] * 10 + [1]):
            whole = layer(a)
        check_gemm_close(out, whole.double().cpu(), f"tile {tile}: tiles of the last round split against whole tiles")
        same = (out == whole).all(dim=1)
        assert int(same.sum()) >= m - 256 * ((rest + n // 256 - 1) // (n // 256) + 4), "whole tiles changed as well"
        assert bool(same[:256].all()), "the first tile row is whole in both runs"
        assert not bool(same.all()), "no tile was split"
    assert bool((layer.workspace == 0).all()), "workspace counters not restored to zero"


@pytest.mark.parametrize("group_size", [-1, 32, 64])
@pytest.mark.parametrize("k,n", [(128, 64), (1024, 192), (2048, 576), (14336 // 4, 128)])
@pytest.mark.parametrize("m", [1, 4, 16, 17, 32, 33, 200, 257])
@pytest.mark.parametrize("asym,act_order", [(False, False), (True, False), (True, True)])
def test_gemm_other_group_sizes(device, group_size, k, n, m, asym, act_order):
    """Channelwise scales (group_size -1) and groups of 32 / 64 rows -- the other entries of the reference's
    MARLIN_SUPPORTED_GROUP_SIZES (marlin_utils.py:24; its GEMM test sweeps them, test_marlin_gemm.py:228-361) -- on both
    the decode and the prefill kernels, with zero points and with act_order."""
    if act_order and (group_size == -1 or k == 128):
        pytest.skip("act_order needs more than one group (gptq_marlin.cu:805)")
    case = o.make_w4a16_case(k, n, group_size, asym=asym, act_order=act_order, seed=k + n + m + group_size)
    layer = W4A16Layer(case, device)
    a = _acts(m, k, device, seed=m)
    out = layer(a)
    check_gemm_close(out, o.gemm_ref(a.cpu(), o.case_w_ref(case)), f"g={group_size} k={k} n={n} m={m}")
    assert bool((layer.workspace == 0).all()), "workspace counters not restored to zero"


@pytest.mark.parametrize("group_size", [-1, 32, 64])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m", [1, 48])
def test_one_hot_activation_other_group_sizes_exact(device, decode_kernel, group_size, dtype, m):
    """One-hot rows of A select single dequantised weight rows: every row must come back as rn16((q - z) * s) of ITS
    group, bit for bit -- a wrong scale or zero-point row for any sub-block of a 128-row tile shows here."""
    k, n = 512, 128
    case = o.make_w4a16_case(k, n, group_size, asym=True, dtype=dtype, seed=13 + group_size)
    layer = W4A16Layer(case, device, dtype)
    w = o.case_w_ref(case)
    for base in (0, 7):
        rows = [(37 * i + 32 * (i % 4) + base) % k for i in range(m)]
        a = torch.zeros(m, k, dtype=dtype)
        for i, r in enumerate(rows):
            a[i, r] = 1
        assert torch.equal(layer(a.to(device)).cpu(), w[rows])


def test_gemm_other_group_sizes_llama_shape(device):
    """Llama-3-8B's down_proj (K = 14336: K split over workgroups on the decode path) at group sizes 32 / 64 / -1."""
    k, n = 14336, 4096
    for group_size in (32, 64, -1):
        case = o.make_w4a16_case(k, n, group_size, asym=group_size == 32, seed=group_size + 40)
        layer = W4A16Layer(case, device)
        w_ref = o.case_w_ref(case)
        for m in (1, 16, 32, 160):
            a = _acts(m, k, device, seed=m)
            check_gemm_close(layer(a), o.gemm_ref(a.cpu(), w_ref), f"g={group_size} m={m}")
        assert bool((layer.workspace == 0).all())


@pytest.mark.parametrize("group_size", [128, -1, 64, 32])
@pytest.mark.parametrize("k,n", [(128, 64), (1024, 192), (2048, 576), (14336 // 4, 128), (14336, 256)])
@pytest.mark.parametrize("m", [1, 4, 16, 17, 32, 33, 200, 257])
@pytest.mark.parametrize("act_order", [False, True])
def test_gemm_8bit_weights(device, group_size, k, n, m, act_order):
    """uint8b128 weights (GPTQ 8-bit symmetric; the reference's GEMM test includes the type, test_marlin_gemm.py:228-361)
    on the decode and the prefill kernels."""
    if act_order and (group_size == -1 or k == 128):
        pytest.skip("act_order needs more than one group (gptq_marlin.cu:805)")
    case = o.make_w4a16_case(k, n, group_size, act_order=act_order, seed=k + n + m, num_bits=8)
    layer = W4A16Layer(case, device)
    a = _acts(m, k, device, seed=m)
    out = layer(a)
    check_gemm_close(out, o.gemm_ref(a.cpu(), o.case_w_ref(case)), f"8-bit g={group_size} k={k} n={n} m={m}")
    assert bool((layer.workspace == 0).all()), "workspace counters not restored to zero"


@pytest.mark.parametrize("group_size", [128, 64, 32])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m", [1, 4, 16, 32, 48])
def test_one_hot_activation_8bit_exact(device, group_size, dtype, m):
    """One-hot rows of A with 8-bit weights: rn16((q - 128) * s) bit for bit, on every kernel variant by M."""
    k, n = 512, 128
    case = o.make_w4a16_case(k, n, group_size, dtype=dtype, seed=21 + group_size, num_bits=8)
    layer = W4A16Layer(case, device, dtype)
    w = o.case_w_ref(case)
    rows = [(37 * i + 5) % k for i in range(m)]
    a = torch.zeros(m, k, dtype=dtype)
    for i, r in enumerate(rows):
        a[i, r] = 1
    assert torch.equal(layer(a.to(device)).cpu(), w[rows])


def test_gemm_8bit_llama_shapes(device):
    for k, n in LLAMA_SHAPES:
        case = o.make_w4a16_case(k, n, 128, seed=k + n, num_bits=8)
        layer = W4A16Layer(case, device)
        w_ref = o.case_w_ref(case)
        for m in (1, 16, 32, 300):
            a = _acts(m, k, device, seed=m)
            check_gemm_close(layer(a), o.gemm_ref(a.cpu(), w_ref), f"8-bit k={k} n={n} m={m}")
        assert bool((layer.workspace == 0).all())


@pytest.mark.parametrize("seed", range(12))
def test_gemm_random_shapes_and_formats(device, seed):
    """Seeded sweep over irregular problems: K any multiple of 128 (odd group counts, counts that no wavefront split
    divides), N any multiple of 64, M from 1 to 300, every weight format and group size, act_order, bias, fp16 / bf16.
    Each case against the oracle; the launch-shape choices of the kernels have many branches that only such sizes reach."""
    rng = np.random.default_rng(1000 + seed)
    for _ in range(6):
        k = 128 * int(rng.integers(1, 40))
        n = 64 * int(rng.integers(1, 20))
        m = int(rng.choice([1, 2, 3, 5, 8, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 100, 129, 300]))
        fmt = rng.choice(["u4b8", "u4", "u8b128"])
        group_size = int(rng.choice([128, 64, 32, -1]))
        act_order = bool(rng.integers(0, 2)) and group_size != -1 and k // group_size > 1
        dtype = torch.bfloat16 if rng.integers(0, 2) else torch.float16
        case = o.make_w4a16_case(k, n, group_size, asym=fmt == "u4", act_order=act_order, dtype=dtype,
                                 seed=int(rng.integers(0, 1 << 30)), num_bits=8 if fmt == "u8b128" else 4)
        layer = W4A16Layer(case, device, dtype)
        a = _acts(m, k, device, dtype, seed=m + k)
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.5).to(dtype) if rng.integers(0, 2) else None
        what = f"k={k} n={n} m={m} {fmt} g={group_size} act_order={act_order} {dtype} bias={bias is not None}"
        out = layer(a, None if bias is None else bias.to(device))
        check_gemm_close(out, o.gemm_ref(a.cpu(), o.case_w_ref(case), bias), what)
        assert bool((layer.workspace == 0).all()), what


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m", [1, 3, 16, 96])
def test_gemm_fp16_and_bias(device, decode_kernel, dtype, m):
    k, n = 1024, 256
    case = o.make_w4a16_case(k, n, 128, asym=True, dtype=dtype, seed=5)
    layer = W4A16Layer(case, device, dtype)
    a = _acts(m, k, device, dtype, seed=2)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(3)) * 0.5).to(dtype)
    out = layer(a, bias.to(device))
    assert out.dtype == dtype
    check_gemm_close(out, o.gemm_ref(a.cpu(), o.case_w_ref(case), bias), f"{dtype} m={m} bias")


@pytest.mark.parametrize("m", [1, 48])
def test_one_hot_activation_returns_dequantised_rows_exactly(device, m):
    """A one-hot row of A selects one dequantised weight row: the GEMM must return rn16((q - z) * s) bit-for-bit."""
    k, n = 512, 128
    case = o.make_w4a16_case(k, n, 128, asym=True, seed=11)
    layer = W4A16Layer(case, device)
    rows = [(37 * i + 5) % k for i in range(m)]
    a = torch.zeros(m, k, dtype=torch.bfloat16)
    for i, r in enumerate(rows):
        a[i, r] = 1
    out = layer(a.to(device)).cpu()
    w = o.case_w_ref(case)
    assert torch.equal(out, w[rows])


@pytest.mark.parametrize("m", [8, 40])
def test_unit_weights_give_row_sums(device, m):
    k, n = 1024, 128
    q = np.full((k, n), 9, dtype=np.int32)
    case = dict(q=q, qweight=o.gptq_pack(q, 4), scales=torch.ones(k // 128, n, dtype=torch.bfloat16), zp_vals=None,
                qzeros=None, g_idx=None, group_size=128)
    layer = W4A16Layer(case, device)
    a = _acts(m, k, device, seed=9)
    out = layer(a).cpu().double()
    expect = a.cpu().double().sum(dim=1, keepdim=True)
    assert (out - expect).abs().max() <= expect.abs().max() * 2.0 ** -7


def test_zero_point_eight_equals_symmetric(device):
    k, n, m = 512, 128, 5
    case = o.make_w4a16_case(k, n, 128, seed=4)
    sym = W4A16Layer(case, device)
    case_asym = dict(case, zp_vals=np.full((k // 128, n), 8, dtype=np.int32))
    asym = W4A16Layer(case_asym, device)
    a = _acts(m, k, device)
    # the two kernels order their fp32 operations differently (the symmetric one folds the zero point into the MFMA
    # chain), so the results agree to an output ulp, not necessarily bit for bit
    o_sym, o_asym = sym(a).float(), asym(a).float()
    assert (o_sym - o_asym).abs().max() <= 2.0 ** -7 * o_sym.abs().max()
    check_gemm_close(asym(a), o.gemm_ref(a.cpu(), o.case_w_ref(case)), "uint4 with zero point 8")


def test_strided_activations(device):
    """Rows of A may be a strided view (reference: test_marlin_gemm_subset_input, test_marlin_gemm.py:537-581)."""
    k, n = 512, 128
    case = o.make_w4a16_case(k, n, 128, seed=6)
    layer = W4A16Layer(case, device)
    for m in (7, 70):
        big = _acts(m, k + 128, device, seed=m)
        a = big[:, 64:64 + k]
        check_gemm_close(layer(a), o.gemm_ref(a.cpu(), o.case_w_ref(case)), f"strided m={m}")


def test_m_zero_returns_empty(device):
    case = o.make_w4a16_case(128, 64, 128)
    layer = W4A16Layer(case, device)
    out = layer(torch.empty(0, 128, dtype=torch.bfloat16, device=device))
    assert out.shape == (0, 64)


# ------------------------------------------------------------------------------------------------ BASELINE.json sizes

def test_config1_reference_cpu_case(device):
    """BASELINE.json config 1: M=16, K=N=4096, g=128, symmetric: bit-exact repack + output tolerance."""
    k = n = 4096
    case = o.make_w4a16_case(k, n, 128, seed=0)
    layer = W4A16Layer(case, device)
    assert np.array_equal(nl.native_unpack(layer.w.cpu().numpy(), k, n), case["q"])
    a = _acts(16, k, device)
    check_gemm_close(layer(a), o.gemm_ref(a.cpu(), o.case_w_ref(case)), "config 1")


@pytest.mark.parametrize("k,n", LLAMA_SHAPES)
def test_config2_decode_llama_shapes(device, decode_kernel, k, n):
    case = o.make_w4a16_case(k, n, 128, seed=1)
    layer = W4A16Layer(case, device)
    w_ref = o.case_w_ref(case)
    for m in (1, 4, 16):
        a = _acts(m, k, device, seed=m)
        out = layer(a)
        check_gemm_close(out, o.gemm_ref(a.cpu(), w_ref), f"config 2 k={k} n={n} m={m}")
        assert torch.equal(out, layer(a)), "decode GEMM is not deterministic run to run"


@pytest.mark.parametrize("k,n", LLAMA_SHAPES + [(1280, 192)])
@pytest.mark.parametrize("m", [33, 40, 48, 64])
def test_decode_three_and_four_m_blocks(device, k, n, m):
    """32 < M <= 64 runs on the LDS-staged decode kernel with three / four m-blocks (K split over workgroups, the
    reduction buffer on top of the activations); symmetric, and asymmetric with act_order."""
    for asym, act_order in ((False, False), (True, True)):
        case = o.make_w4a16_case(k, n, 128, asym=asym, act_order=act_order, seed=k + n + m)
        layer = W4A16Layer(case, device)
        a = _acts(m, k, device, seed=m)
        out = layer(a)
        check_gemm_close(out, o.gemm_ref(a.cpu(), o.case_w_ref(case)), f"k={k} n={n} m={m} asym={asym}")
        assert torch.equal(out, layer(a)), "not deterministic run to run"
        assert bool((layer.workspace == 0).all()), "workspace counters not restored to zero"


@pytest.mark.parametrize("k,n,m", [(4096, 4096, 128), (4096, 4096, 121), (4096, 6144, 80), (4096, 6144, 70), (2048, 2048, 256),
                                   (2048, 2048, 250), (4096, 2048, 128), (4096, 2048, 200), (1024, 1024, 96), (4096, 4096, 96)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rows_over_workgroups_beyond_four_m_blocks(device, k, n, m, dtype):
    """65 .. 256 rows on a narrow layer: where workgroups of 16 rows each make one round, the decode kernel takes the rows
    as five to sixteen m-blocks with workgroups of their own (a ragged last block among them; the last case with eight
    n-tiles per workgroup, because six would need a second round and seven lose to eight); with act_order the tile kernel
    does.  Same answer either way: symmetric and with zero
    points against the fp64 oracle, one-hot rows bit for bit, no scratch used, deterministic."""
    for asym, act_order in ((False, False), (True, False), (True, True)):
        case = o.make_w4a16_case(k, n, 128, asym=asym, act_order=act_order, dtype=dtype, seed=k + n + m)
        layer = W4A16Layer(case, device, dtype)
        w_ref = o.case_w_ref(case)
        a = _acts(m, k, device, dtype=dtype, seed=m)
        out = layer(a)
        assert out.shape == (m, n) and out.dtype == dtype
        check_gemm_close(out, o.gemm_ref(a.cpu(), w_ref), f"k={k} n={n} m={m} asym={asym} act_order={act_order}")
        assert torch.equal(out, layer(a)), "not deterministic run to run"
        assert bool((layer.workspace == 0).all()), "workspace counters not restored to zero"
        rows = [(37 * i + 5) % k for i in range(m)]
        hot = torch.zeros(m, k, dtype=dtype)
        for i, r in enumerate(rows):
            hot[i, r] = 1
        assert torch.equal(layer(hot.to(device)).cpu(), w_ref[rows]), "one-hot rows must return the dequantised weights exactly"


@pytest.mark.parametrize("k,n", [(4096, 4096), (4096, 6144), (1024, 1472), (2048, 1984), (4096, 3008), (2048, 2048), (14336, 4096)])
def test_decode_n_tiles_grouped_by_xcd_same_bits(device, k, n):
    """On narrow layers the decode kernel hands the workgroups of one XCD neighbouring n-tiles (a permutation of which
    workgroup computes which columns, nothing else): with the grouping switched off for one call the output must be the
    same bits, for 1 .. 48 rows (one m-block, two, and rows over workgroups), with zero points, also on column counts
    that are no power of two."""
    from vllm_amd import _tuning
    case = o.make_w4a16_case(k, n, 128, asym=True, dtype=torch.bfloat16, seed=k + n)
    layer = W4A16Layer(case, device, torch.bfloat16)
    w_ref = o.case_w_ref(case)
    for m in (1, 4, 16, 32, 48):
        a = _acts(m, k, device, seed=m)
        out = layer(a)
        with _tuning.override(exp=[0] * 7 + [1]):
            plain = layer(a)
        assert torch.equal(out, plain), (k, n, m)
        check_gemm_close(out, o.gemm_ref(a.cpu(), w_ref), f"k={k} n={n} m={m}")


# layer shapes of other models on which the planners take branches that the Llama-3-8B shapes do not reach: K slabs that
# would come out uneven (9216 x 4608, 10240 x 2560), a ragged single slab on a narrow layer (5120 x 5120), a short K on
# few tiles (1536 x 1536), an odd number of 64-row blocks on a wide short-K layer (2560 x 10240), long K parts on few
# 128 x 64 tiles (12288 x 3072)
OTHER_MODEL_SHAPES = [(9216, 4608), (10240, 2560), (5120, 5120), (1536, 1536), (2560, 10240), (12288, 3072)]


@pytest.mark.parametrize("k,n", OTHER_MODEL_SHAPES)
def test_planner_branches_other_model_shapes(device, k, n):
    """Symmetric 4-bit, groups of 128, M across the decode and tile kernels; M <= 64 against the full fp64 oracle, larger M
    on sampled rows.  Run to run the result must be bit-identical (the K splits sum in a fixed order) and the arrival
    counters must be back at zero."""
    case = o.make_w4a16_case(k, n, 128, seed=k + n)
    layer = W4A16Layer(case, device)
    w_ref = o.case_w_ref(case)
    for m in (1, 2, 4, 8, 16, 32, 48, 96, 160, 256, 384, 640):
        a = _acts(m, k, device, seed=m)
        out = layer(a)
        rows = np.arange(m) if m <= 64 else np.concatenate([np.random.default_rng(m).choice(m, 16, replace=False), [0, m - 1]])
        check_gemm_close(out[rows], o.gemm_ref(a.cpu()[rows], w_ref), f"k={k} n={n} m={m}")
        assert torch.isfinite(out).all() and bool((out.float().norm(dim=1) > 0).all())
        assert torch.equal(out, layer(a)), f"k={k} n={n} m={m}: not deterministic run to run"
    assert bool((layer.workspace == 0).all()), "workspace counters not restored to zero"


@pytest.mark.parametrize("k,n", LLAMA_SHAPES)
@pytest.mark.parametrize("group_level", [False, True])
def test_config3_prefill_llama_shapes_sampled(device, k, n, group_level):
    """Asymmetric + act_order at M in {512, 2048, 4096}: the oracle is evaluated on 24 sampled rows (the full fp64 GEMM
    would take minutes on the CPU); rows are independent in a GEMM, so a wrong tile shows up in its rows."""
    case = o.make_w4a16_case(k, n, 128, asym=True, act_order=True, group_level_perm=group_level, seed=2)
    layer = W4A16Layer(case, device)
    w_ref = o.case_w_ref(case)
    for m in (512, 2048, 4096):
        a = _acts(m, k, device, seed=m)
        out = layer(a)
        rows = np.random.default_rng(m).choice(m, size=24, replace=False)
        rows = np.concatenate([rows, [0, m - 1]])
        ref = o.gemm_ref(a.cpu()[rows], w_ref)
        check_gemm_close(out[rows], ref, f"config 3 k={k} n={n} m={m}")
        # every row must be finite and of plausible magnitude (catches tiles that were never written)
        assert torch.isfinite(out).all()
        col_norm = out.float().norm(dim=1)
        assert bool((col_norm > 0).all())


@pytest.mark.parametrize("k,n", LLAMA_SHAPES)
def test_config5_decode_step_gemm_llama_shapes(device, decode_kernel, k, n):
    """The GEMM of BASELINE.json config 5: symmetric 4-bit, groups of 128, batch 32 (two 16-row blocks) at the four
    Llama-3-8B projection shapes, full fp64 oracle."""
    case = o.make_w4a16_case(k, n, 128, seed=5)
    layer = W4A16Layer(case, device)
    a = _acts(32, k, device, seed=32)
    out = layer(a)
    check_gemm_close(out, o.gemm_ref(a.cpu(), o.case_w_ref(case)), f"config 5 GEMM k={k} n={n} m=32")
    assert bool((layer.workspace == 0).all()), "workspace counters not restored to zero"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("mnk", [(1, 1, 1), (1, 4, 8), (26, 37, 13), (257, 13, 11)])
@pytest.mark.parametrize("n_chunk", [64, 256])
@pytest.mark.parametrize("quant_type,act_order", [("uint4b8", False), ("uint4b8", True), ("uint4", False), ("uint8b128", False)])
def test_gemm_reference_grid_weights_quantized_from_float(device, quant_type, act_order, n_chunk, mnk, dtype):
    """The reference's own GEMM test (tests/kernels/quantization/test_marlin_gemm.py:228-361): random normal activations
    and weights, the weights pushed through the reference's quantisers (oracle/quantize.py) -- realistic scale spread,
    extreme codes at every group's maximum, zero points at both ends of their range -- on its size grid (k_chunk 128,
    n_chunk 64 / 256, its (M, N, K) factors) for every group size, against `a @ w_ref` of the quantiser's own
    dequantised weight."""
    from oracle import quantize as oq
    m, nf, kf = mnk
    k, n = 128 * kf, n_chunk * nf
    g = torch.Generator().manual_seed(1000 * kf + nf + m)
    for group_size in (-1, 32, 64, 128):
        if act_order and (group_size == -1 or group_size == k):
            continue                                  # needs more than one group (test_marlin_gemm.py:247-252)
        if k % max(group_size, 1) != 0:
            continue
        w = torch.randn(k, n, generator=g).to(dtype)
        a = torch.randn(m, k, generator=g).to(dtype)
        case = oq.quantized_case(w, quant_type, group_size, act_order=act_order, seed=kf)
        layer = W4A16Layer(case, device, dtype)
        out = layer(a.to(device))
        check_gemm_close(out, o.gemm_ref(a, case["w_ref"]), f"{quant_type} g={group_size} act_order={act_order} m={m} n={n} k={k}")
        # the reference's own pass criterion, against its own 16-bit matmul
        ref16 = o.gemm_ref_like_reference(a.float(), case["w_ref"].float())
        assert o.rel_err_mean(out.cpu().float(), ref16) < 0.04
