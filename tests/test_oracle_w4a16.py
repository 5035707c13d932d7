"""Pins the W4A16 CPU oracle without importing the reference: two independent descriptions of the Marlin order must
agree, closed forms / brute force for the packers, known-answer constants, invariants, committed golden vectors."""
import os

import numpy as np
import pytest
import torch

from oracle import native_layout as nl
from oracle import w4a16 as o

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")

# size grid of the reference's own repack test (tests/kernels/quantization/test_marlin_gemm.py:45-60, :98-156):
# K = 128 * k_chunk * k_factor, N = 64|256 * n_factor, capped so that the CPU suite stays fast
REF_GRID = [(128 * kf, nc * nf) for kf in (1, 8, 13, 11) for nc, nf in ((64, 1), (256, 1), (64, 4), (64, 37), (64, 13))]


def test_pack_rows_brute_force():
    rng = np.random.default_rng(0)
    q = rng.integers(0, 16, size=(16, 8), dtype=np.int32)
    packed = o.gptq_pack(q, 4).view(np.uint32)
    for r in range(2):
        for n in range(8):
            expect = 0
            for i in range(8):
                expect |= int(q[8 * r + i, n]) << (4 * i)
            assert int(packed[r, n]) == expect
    assert (o.unpack_rows(packed.view(np.int32), 4) == q).all()


def test_pack_cols_brute_force_and_roundtrip():
    rng = np.random.default_rng(1)
    q = rng.integers(0, 16, size=(5, 32), dtype=np.int32)
    packed = o.pack_cols(q, 4).view(np.uint32)
    for k in range(5):
        for c in range(4):
            expect = 0
            for i in range(8):
                expect |= int(q[k, 8 * c + i]) << (4 * i)
            assert int(packed[k, c]) == expect
    assert (o.unpack_cols(packed.view(np.int32), 4) == q).all()


def test_top_nibble_sign_handling():
    q = np.full((8, 1), 15, dtype=np.int32)
    assert o.gptq_pack(q, 4)[0, 0] == -1            # 0xFFFFFFFF as int32
    assert (o.unpack_rows(o.gptq_pack(q, 4), 4) == 15).all()


def test_weight_perm_known_answers():
    perm = o.get_weight_perm(4)
    assert perm.shape == (1024,) and sorted(perm.tolist()) == list(range(1024))
    # first output word of a tile: thread 0 / warp 0 -> rows {0,1,8,9} of column 0 then column 8, interleaved 0,2,4,6,1,3,5,7
    # element index within the flattened 16x16 sub-tile is 16*row + col
    assert perm[:8].tolist() == [0, 128, 8, 136, 16, 144, 24, 152]
    assert o.INTERLEAVE4 == (0, 2, 4, 6, 1, 3, 5, 7)


@pytest.mark.parametrize("k,n", REF_GRID)
def test_two_descriptions_of_marlin_order_agree(k, n):
    rng = np.random.default_rng(k * 7 + n)
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    qw = o.gptq_pack(q, 4)
    by_index_list = o.marlin_weights(q)
    by_thread_map = o.marlin_repack_thread_map(qw, None, k, n)
    assert by_index_list.shape == (k // 16, 2 * n)
    assert np.array_equal(by_index_list, by_thread_map)


@pytest.mark.parametrize("k,n", REF_GRID[:6] + [(128 * 13, 64 * 37)])
def test_two_descriptions_of_marlin_order_agree_8bit(k, n):
    """8-bit codes (uint8b128 weights): the host index list with interleave (0, 2, 1, 3) (marlin_utils_test.py:66-93) and
    the device kernel's thread map (two words per thread, gptq_marlin_repack.cu:189-203) must describe the same order;
    with act_order the thread map equals the order of the permuted rows; the order is a permutation of the codes."""
    rng = np.random.default_rng(k * 5 + n)
    q = rng.integers(0, 256, size=(k, n), dtype=np.int32)
    qw = o.gptq_pack(q, 8)
    assert qw.shape == (k // 4, n)
    by_index_list = o.marlin_weights(q, 8)
    assert by_index_list.shape == (k // 16, 4 * n)
    assert np.array_equal(by_index_list, o.marlin_repack_thread_map(qw, None, k, n, 8))
    perm = rng.permutation(k).astype(np.int32)
    assert np.array_equal(o.marlin_repack_thread_map(qw, perm, k, n, 8), o.marlin_weights(q[perm], 8))
    assert np.array_equal(o.marlin_unpack_to_logical(by_index_list, k, n, 8), q)
    # first word of a tile: thread 0 / warp 0 -> rows {0, 8, 1, 9} of column 0
    w0 = int(np.asarray(by_index_list).view(np.uint32)[0, 0])
    assert [(w0 >> (8 * i)) & 0xff for i in range(4)] == [q[0, 0], q[8, 0], q[1, 0], q[9, 0]]


@pytest.mark.parametrize("k,n", [(128, 64), (1024, 256), (128 * 13, 64 * 4)])
def test_marlin_order_with_perm_equals_order_of_permuted_rows(k, n):
    rng = np.random.default_rng(3)
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    perm = rng.permutation(k).astype(np.int32)
    assert np.array_equal(o.marlin_repack_thread_map(o.gptq_pack(q, 4), perm, k, n), o.marlin_weights(q[perm]))


@pytest.mark.parametrize("k,n", [(128, 64), (256, 192)])
def test_marlin_order_is_a_permutation_of_nibbles(k, n):
    rng = np.random.default_rng(4)
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    m = o.marlin_weights(q)
    assert np.array_equal(np.bincount(o.unpack_cols(m, 4).ravel(), minlength=16), np.bincount(q.ravel(), minlength=16))
    assert np.array_equal(o.marlin_unpack_to_logical(m, k, n), q)
    # position test: a single non-zero code moves to exactly one place
    z = np.zeros((k, n), dtype=np.int32)
    z[37, 21] = 9
    mz = o.unpack_cols(o.marlin_weights(z), 4)
    assert mz.sum() == 9 and (mz != 0).sum() == 1


@pytest.mark.parametrize("k,n", [(128, 64), (384, 128), (128 * 11, 64 * 13)])
def test_native_layout_roundtrip_and_word_content(k, n):
    rng = np.random.default_rng(5)
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    packed = nl.native_pack(q)
    assert packed.shape == (k // 16, 2 * n)
    assert np.array_equal(nl.native_unpack(packed, k, n), q)
    # spot-check the definition by hand for a few words
    words = packed.reshape(-1).view(np.uint32)
    k_tiles = k // 128
    for idx in (0, 1, 5, 255, 256, 4 * 64 * (k_tiles + 1) + 4 * 37 + 2, words.size - 1):
        if idx >= words.size:
            continue
        j, lane, tile = idx & 3, (idx >> 2) & 63, idx >> 8
        nt, kt = divmod(tile, k_tiles)
        o_, r = lane >> 4, lane & 15
        k0 = 128 * kt + 32 * j + 8 * o_
        col = 16 * nt + r
        expect = 0
        for p, e in enumerate((0, 2, 4, 6, 1, 3, 5, 7)):
            expect |= int(q[k0 + e, col]) << (4 * p)
        assert int(words[idx]) == expect


def test_scale_perm_known_answers():
    sp, sp1 = o.get_scale_perms()
    assert sp[:10] == [0, 8, 16, 24, 32, 40, 48, 56, 1, 9] and sorted(sp) == list(range(64))
    assert sp1 == [0, 1, 8, 9, 16, 17, 24, 25, 2, 3, 10, 11, 18, 19, 26, 27,
                   4, 5, 12, 13, 20, 21, 28, 29, 6, 7, 14, 15, 22, 23, 30, 31]
    s = np.arange(2 * 128, dtype=np.float32).reshape(2, 128)
    grouped = o.marlin_permute_scales(s, 256, 128, 128)
    assert grouped[0, :4].tolist() == [0, 8, 16, 24] and grouped[1, 64:66].tolist() == [128 + 64, 128 + 72]
    chan = o.marlin_permute_scales(s[:1], 128, 128, -1)
    assert chan[0, :6].tolist() == [0, 1, 8, 9, 16, 17]
    assert np.array_equal(np.sort(grouped.ravel()), s.ravel())


def test_zero_points_layout():
    rng = np.random.default_rng(6)
    zp = rng.integers(0, 16, size=(3, 128), dtype=np.int32)
    packed = o.marlin_zero_points(zp, 3, 128, 4)
    assert packed.shape == (3, 16)
    sp, _ = o.get_scale_perms()
    un = o.unpack_cols(packed, 4)                                   # interleaved, scale-permuted
    undo = np.argsort(np.asarray(o.INTERLEAVE4))
    un = un.reshape(-1, 8)[:, undo].reshape(-1, 64)
    inv = np.argsort(np.asarray(sp))
    assert np.array_equal(un[:, inv].reshape(3, 128), zp)
    # AWQ zero points: undo the AWQ interleave first (marlin_utils.py:349-370)
    awq = o.pack_cols(zp.reshape(-1, 8)[:, np.asarray(o.INTERLEAVE4)].reshape(3, 128), 4)
    assert np.array_equal(o.awq_to_marlin_zero_points(awq, 3, 128, 4), packed)


def test_dequant_closed_forms():
    k, n, g = 256, 64, 128
    # s = 1, code 9, zero 8  ->  every weight is exactly 1  ->  C = row sums of A
    q = np.full((k, n), 9, dtype=np.int32)
    s = torch.ones(k // g, n, dtype=torch.bfloat16)
    w = o.dequantize(q, s, 8, g)
    assert w.dtype == torch.bfloat16 and bool((w == 1).all())
    a = torch.randn(3, k, generator=torch.Generator().manual_seed(0)).to(torch.bfloat16)
    c = o.gemm_ref(a, w)
    assert torch.allclose(c, a.double().sum(dim=1, keepdim=True).expand(-1, n))
    # one-hot A picks a dequantised row, exactly
    case = o.make_w4a16_case(k, n, g, asym=True, seed=3)
    w = o.case_w_ref(case)
    onehot = torch.zeros(1, k, dtype=torch.bfloat16)
    onehot[0, 77] = 1
    assert torch.equal(o.gemm_ref(onehot, w)[0], w[77].double())
    # value check against the formula evaluated by hand in fp32 then rounded once
    z = case["zp_vals"][77 // g]
    manual = ((case["q"][77] - z).astype(np.float32) * case["scales"][77 // g].float().numpy())
    assert torch.equal(w[77], torch.from_numpy(manual).to(torch.bfloat16))


def test_uint4_with_zero_eight_equals_uint4b8():
    case = o.make_w4a16_case(256, 64, 128, seed=1)
    w_sym = o.case_w_ref(case)
    w_asym = o.dequantize(case["q"], case["scales"], np.full((2, 64), 8, dtype=np.int32), 128)
    assert torch.equal(w_sym, w_asym)


def test_act_order_equals_plain_gemm_on_permuted_activations():
    case = o.make_w4a16_case(512, 64, 128, asym=True, act_order=True, seed=2)
    w = o.case_w_ref(case)                                   # rows in checkpoint order, groups through g_idx
    a = torch.randn(4, 512, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    c_direct = o.gemm_ref(a, w)
    g_sorted, sort_idx = o.marlin_sort_g_idx(case["g_idx"])
    assert (np.diff(g_sorted) >= 0).all() and np.array_equal(g_sorted, np.arange(512) // 128)
    w_sorted = o.dequantize(case["q"][sort_idx], case["scales"], case["zp_vals"], 128)   # plain grouping r // 128
    c_sorted = o.gemm_ref(a[:, torch.from_numpy(sort_idx.astype(np.int64))], w_sorted)
    assert torch.allclose(c_direct, c_sorted, rtol=0, atol=1e-9)


def test_golden_vectors():
    g = np.load(os.path.join(GOLDEN, "w4a16_small.npz"))
    q = g["q"]
    assert np.array_equal(o.gptq_pack(q, 4), g["qweight"])
    assert np.array_equal(o.marlin_weights(q), g["marlin"])
    assert np.array_equal(o.marlin_repack_thread_map(g["qweight"], g["perm"], *q.shape), g["marlin_perm"])
    assert np.array_equal(nl.native_pack(q), g["native"])
    assert np.array_equal(o.marlin_zero_points(g["zp"], g["zp"].shape[0], q.shape[1], 4), g["marlin_zp"])


def test_native_layout_8bit_is_two_nibble_planes():
    k, n = 256, 64
    rng = np.random.default_rng(8)
    q = rng.integers(0, 256, size=(k, n), dtype=np.int32)
    p8 = nl.native_pack8(q)
    assert p8.shape == (k // 16, 4 * n)
    assert np.array_equal(nl.native_unpack8(p8, k, n), q)
    blocks = p8.reshape(-1, 256)
    assert np.array_equal(blocks[0::2].reshape(k // 16, 2 * n), nl.native_pack(q >> 4))
    assert np.array_equal(blocks[1::2].reshape(k // 16, 2 * n), nl.native_pack(q & 15))

