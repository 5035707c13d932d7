"""Pins for ``oracle/quantize.py`` (the reference's weight quantisers restated on the CPU).  None of these tests repeats
the oracle's formula: they check what the mathematics of uniform quantisation fixes -- error bounds, extreme codes, ranges,
permutation bookkeeping, round trips -- plus brute force over tiny inputs, chosen so that a dropped bias, a wrong sign,
a swapped min / max or a transposed group reshape fails one of them."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import quantize as oq
from oracle import w4a16 as ow

GROUPS = [-1, 32, 64, 128]


def _w(k, n, dtype, seed):
    return torch.randn(k, n, generator=torch.Generator().manual_seed(seed)).to(dtype)


def _expand(t: torch.Tensor, k: int) -> torch.Tensor:
    return t.repeat_interleave(k // t.shape[0], dim=0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("group_size", GROUPS)
@pytest.mark.parametrize("quant_type", ["uint4b8", "uint8b128"])
def test_symmetric_quantiser_error_bound_and_extremes(quant_type, group_size, dtype):
    k, n = 256, 48
    w = _w(k, n, dtype, 1)
    t = oq.QUANT_TYPES[quant_type]
    w_ref, q, s, zp = oq.quantize_weights(w, quant_type, group_size)
    assert zp is None and q.dtype == torch.int32 and w_ref.dtype == dtype
    groups = 1 if group_size == -1 else k // group_size
    assert s.shape == (groups, n) and bool((s > 0).all())
    assert int(q.min()) >= 0 and int(q.max()) <= (1 << t["bits"]) - 1            # stored codes are unsigned
    centred = q - t["bias"]
    assert int(centred.min()) >= t["lo"] and int(centred.max()) <= t["hi"]
    s_full = _expand(s, k).double()
    # dequantised weight is code * scale up to ONE rounding in the weight dtype ...
    eps = torch.finfo(dtype).eps
    assert bool(((w_ref.double() - centred.double() * s_full).abs() <= eps * (centred.double() * s_full).abs() + 1e-30).all())
    # ... and within half a step of the input (a few roundings of 16-bit arithmetic on top), except where the positive
    # side clamps: the scale is set by the larger of max / hi and |min| / |lo|, so values above hi * s saturate
    err = (w.double() - w_ref.double()).abs()
    slack = 4 * eps * w.double().abs() + 1e-12
    unclamped = w.double() <= (t["hi"] + 0.5) * s_full
    assert bool((err[unclamped] <= (0.5 * s_full + slack)[unclamped]).all())
    # a group's most negative value reaches lo or its largest reaches hi (whichever set the scale), to within a step
    wg = w.double().reshape(groups, k // groups, n)
    cg = centred.reshape(groups, k // groups, n)
    hits_lo = cg.min(dim=1).values <= t["lo"] + 1
    hits_hi = cg.max(dim=1).values >= t["hi"] - 1
    assert bool((hits_lo | hits_hi).all())
    # scale equals the textbook value max(max / hi, |min| / |lo|) up to the dtype's rounding
    s_true = torch.maximum(wg.max(dim=1).values / t["hi"], wg.min(dim=1).values.abs() / abs(t["lo"]))
    assert torch.allclose(s.double(), s_true, rtol=4 * eps, atol=0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("group_size", GROUPS)
def test_asymmetric_quantiser_ranges_and_error_bound(group_size, dtype):
    k, n = 256, 40
    w = _w(k, n, dtype, 2) + 0.3           # off-centre on purpose: zero points away from the middle
    w_ref, q, s, zp = oq.quantize_weights(w, "uint4", group_size, zero_points=True)
    groups = 1 if group_size == -1 else k // group_size
    assert zp.shape == (groups, n) and zp.dtype == torch.int32
    assert int(zp.min()) >= 0 and int(zp.max()) <= 15 and int(q.min()) >= 0 and int(q.max()) <= 15
    wg = w.double().reshape(groups, k // groups, n)
    eps = torch.finfo(dtype).eps
    span = wg.max(dim=1).values - wg.min(dim=1).values
    assert torch.allclose(s.double(), span / 15, rtol=4 * eps)                  # (max - min) / 15
    # every group uses both ends of the code range (its min maps near 0, its max near 15)
    qg = q.reshape(groups, k // groups, n)
    assert bool((qg.min(dim=1).values <= 1).all()) and bool((qg.max(dim=1).values >= 14).all())
    s_full, zp_full = _expand(s, k).double(), _expand(zp, k).double()
    assert bool(((w_ref.double() - (q.double() - zp_full) * s_full).abs() <= eps * w_ref.double().abs() + 1e-30).all())
    # within one step of the input (half a step from each of the two roundings: the value and the zero point)
    err = (w.double() - w_ref.double()).abs()
    assert bool((err <= 1.0 * s_full + 8 * eps * w.double().abs() + 1e-12).all())
    # zero point = where 0.0 lands: round(-min / s) for groups that straddle zero
    straddle = (wg.min(dim=1).values < 0) & (wg.max(dim=1).values > 0)
    zp_true = torch.round(-wg.min(dim=1).values / s.double())
    assert bool(((zp.double() - zp_true).abs()[straddle] <= 1).all())
    # the alternative reference form (zero point applied after the scale) differs by rounding only
    w_ref2 = oq.quantize_weights(w, "uint4", group_size, zero_points=True, ref_zero_points_after_scales=True)[0]
    assert bool(((w_ref2.double() - w_ref.double()).abs() <= 16 * eps * (15 * s_full)).all())


def test_quantiser_brute_force_tiny_group():
    """One group of four known values per column: codes and scales by hand."""
    w = torch.tensor([[-8.0, 0.0], [7.0, 3.5], [1.0, -3.5], [-0.5, 1.75]])
    w_ref, q, s, _ = oq.quantize_weights(w, "uint4b8", -1)
    assert s.tolist() == [[1.0, 0.5]]                       # max(7/7, 8/8) = 1;  max(3.5/7, 3.5/8) = 0.5
    assert q.tolist() == [[0, 8], [15, 15], [9, 1], [8, 12]]   # round(w / s) + 8, halves to even: -0.5 -> -0 ; 3.5 -> 4 ; 7 -> 7
    assert w_ref.tolist() == [[-8.0, 0.0], [7.0, 3.5], [1.0, -3.5], [0.0, 2.0]]
    w_ref, q, s, zp = oq.quantize_weights(torch.tensor([[0.0], [15.0], [7.4], [-0.0]]), "uint4", -1, zero_points=True)
    assert s.tolist() == [[1.0]] and zp.tolist() == [[0]] and q.tolist() == [[0], [15], [7], [0]]
    w_ref, q, s, zp = oq.quantize_weights(torch.tensor([[-3.0], [12.0], [0.0], [4.6]]), "uint4", -1, zero_points=True)
    assert s.tolist() == [[1.0]] and zp.tolist() == [[3]] and q.tolist() == [[0], [15], [3], [8]]
    assert w_ref.tolist() == [[-3.0], [12.0], [0.0], [5.0]]


def test_group_reshape_is_per_column_and_per_group():
    """A weight that is constant within each (group, column) block but different between blocks must come back exactly:
    a transposed or mis-strided group reshape mixes blocks and breaks it."""
    k, n, g = 128, 6, 32
    blocks = torch.arange(1, (k // g) * n + 1, dtype=torch.float32).reshape(k // g, n)
    w = blocks.repeat_interleave(g, dim=0)
    w_ref, q, s, _ = oq.quantize_weights(w, "uint4b8", g)
    assert torch.equal(w_ref, w) and torch.equal(s, blocks / 7) and bool((q == 15).all())


@pytest.mark.parametrize("group_size", [32, 64, 128])
def test_act_order_bookkeeping(group_size):
    k, n = 256, 24
    w = _w(k, n, torch.float16, 3)
    plain = oq.gptq_quantize_weights(w, "uint4b8", group_size, act_order=False)
    perm = torch.randperm(k, generator=torch.Generator().manual_seed(9))
    w_ref, q, s, g_idx, rand_perm = oq.gptq_quantize_weights(w, "uint4b8", group_size, act_order=True, test_perm=perm)
    assert torch.equal(rand_perm, perm)
    assert torch.equal(q, plain[1][perm]) and torch.equal(w_ref, plain[0][perm]) and torch.equal(s, plain[2])
    assert torch.equal(g_idx.long(), perm // group_size)                       # group of stored row i
    q_sorted, g_sorted, order = oq.sort_weights(q, g_idx)
    assert sorted(order.tolist()) == list(range(k))                            # a permutation
    assert torch.equal(g_sorted.long(), torch.arange(k) // group_size)         # grouped, every group complete
    assert torch.equal(q_sorted, q[order.long()])
    # inside every group the sorted rows are that group's original rows (as a set)
    for gi in range(k // group_size):
        rows_sorted = {tuple(r) for r in q_sorted[gi * group_size:(gi + 1) * group_size].tolist()}
        rows_orig = {tuple(r) for r in plain[1][gi * group_size:(gi + 1) * group_size].tolist()}
        assert rows_sorted == rows_orig
    # the GEMM identity act_order must keep: A @ w_ref_plain == A[:, perm] @ w_ref_permuted
    a = torch.randn(5, k, dtype=torch.float64)
    assert torch.allclose(a @ plain[0].double(), a[:, perm] @ w_ref.double(), rtol=1e-12, atol=1e-12)


def test_marlin_quantize_outputs_are_the_layout_functions_of_the_plain_quantiser():
    k, n, g = 256, 128, 64
    w = _w(k, n, torch.float16, 4)
    w_ref, marlin_q, marlin_s, g_idx, sort_idx, rand_perm = oq.marlin_quantize(w, "uint4b8", g, act_order=True, seed=5)
    # undoing the Marlin order gives the sorted codes; undoing the sort and the act_order permutation gives the plain codes
    logical = ow.marlin_unpack_to_logical(marlin_q, k, n, 4)
    plain = oq.quantize_weights(w, "uint4b8", g)
    q_perm = plain[1][rand_perm]
    assert np.array_equal(logical, q_perm[sort_idx.long()].numpy())
    assert torch.equal(g_idx.long(), torch.arange(k) // g)
    assert torch.equal(w_ref, plain[0][rand_perm])
    s_back = marlin_s.view(torch.int16).numpy()
    assert sorted(s_back.ravel().tolist()) == sorted(plain[2].view(torch.int16).numpy().ravel().tolist())
    w_ref2, marlin_q2, marlin_s2, marlin_zp = oq.awq_marlin_quantize(w, "uint4", g)
    plain2 = oq.quantize_weights(w, "uint4", g, zero_points=True)
    assert np.array_equal(ow.marlin_unpack_to_logical(marlin_q2, k, n, 4), plain2[1].numpy())
    assert torch.equal(w_ref2, plain2[0]) and marlin_zp.shape == (k // g, n // 8)


def test_quantized_case_is_consistent_with_the_dequantiser():
    """The case built from float weights must dequantise (oracle/w4a16.dequantize, pinned separately) to the reference's
    own w_ref bit for bit: two routes to the same weight."""
    k, n = 256, 64
    for qt, g, act in (("uint4b8", 128, False), ("uint4b8", 64, True), ("uint4", 32, False), ("uint8b128", -1, False),
                       ("uint4", -1, False)):
        w = _w(k, n, torch.bfloat16, 6)
        case = oq.quantized_case(w, qt, g, act_order=act, seed=1)
        assert torch.equal(ow.case_w_ref(case).view(torch.int16), case["w_ref"].view(torch.int16)), (qt, g, act)
        assert np.array_equal(ow.unpack_rows(case["qweight"], case["num_bits"]), case["q"])


@pytest.mark.parametrize("group_shape", [(-1, -1), (1, -1), (-1, 1), (4, 8), (1, 16)])
def test_scaled_quantize_round_trip(group_shape):
    x = torch.randn(8, 32, generator=torch.Generator().manual_seed(7)) * 3
    x_q, x_s = oq.scaled_quantize(x, group_shape, torch.float8_e4m3fn)
    gm = group_shape[0] if group_shape[0] > 0 else 8
    gn = group_shape[1] if group_shape[1] > 0 else 32
    assert x_q.dtype == torch.float8_e4m3fn and x_s.shape == (8 // gm, 32 // gn) and x_s.dtype == torch.float32
    back = oq.scaled_dequantize(x_q, x_s, group_shape)
    # e4m3 has 3 mantissa bits: relative error <= 2^-4 of the value, plus half the smallest subnormal (2^-10) of each block's scale
    scale_full = oq.group_broadcast(x_s, x.shape)
    assert bool(((back - x).abs() <= x.abs() * 2.0 ** -4 + scale_full * 2.0 ** -10 + 1e-6).all())
    # every block's largest magnitude maps to the format's maximum
    blocks = x_q.float().abs().reshape(8 // gm, gm, 32 // gn, gn).amax(dim=(1, 3))
    assert bool((blocks == 448).all())
    # a vector of scales is taken along the dimension it spans
    if group_shape == (1, -1):
        assert torch.equal(oq.scaled_dequantize(x_q, x_s.reshape(-1), group_shape), back)


def test_group_broadcast_known_answer():
    a = torch.tensor([[1, 2], [3, 4]])
    assert oq.group_broadcast(a, (2, 4)).tolist() == [[1, 1, 2, 2], [3, 3, 4, 4]]
    assert oq.group_broadcast(a, (4, 2)).tolist() == [[1, 2], [1, 2], [3, 4], [3, 4]]
    assert oq.group_broadcast(torch.tensor([[5]]), (3, 3)).tolist() == [[5]]       # extent 1 is left to broadcasting


def test_awq_pack_brute_force_one_word():
    """AutoAWQ's packing by hand (quant_utils.py:614-633): the eight 4-bit values of a word are the columns
    8c + {0,2,4,6,1,3,5,7}[p] in nibble position p."""
    row = np.array([[1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 0]], dtype=np.int32)
    packed = ow.awq_pack(row, 4)
    order = [0, 2, 4, 6, 1, 3, 5, 7]
    want = []
    for c in range(2):
        word = 0
        for p, e in enumerate(order):
            word |= int(row[0, 8 * c + e]) << (4 * p)
        want.append(np.uint32(word).astype(np.uint32).view(np.int32) if False else word)
    assert [int(np.uint32(v)) for v in packed.view(np.uint32)[0]] == want
    assert want[0] == 0x86427531                      # 1,3,5,7 in the low nibbles, then 2,4,6,8


@pytest.mark.parametrize("group_size", [-1, 128])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fp8_weight_quantiser_pins(dtype, group_size):
    """marlin_quant_fp8_torch restated: every group's largest magnitude maps to +-448 (code 0x7E / 0xFE), the
    dequantised weight is within the e4m3 step (2^-4 relative, plus the 16-bit roundings) of the input, and the codes
    decode (independent bit-level decoder of oracle/fp8.py) to w_ref / scale."""
    from oracle import fp8 as of
    n, k = 48, 256
    w = torch.randn(n, k, generator=torch.Generator().manual_seed(3)).to(dtype)
    w_ref, codes, scales = oq.marlin_quant_fp8_torch(w, group_size)
    g = k if group_size == -1 else group_size
    assert w_ref.shape == (k, n) and codes.shape == (k, n) and scales.shape == (k // g, n) and codes.dtype == torch.uint8
    mags = (codes & 0x7F).reshape(k // g, g, n).amax(dim=1)
    assert bool((mags == 0x7E).all()), "a group's maximum must land on 448"
    eps = torch.finfo(dtype).eps
    s_full = scales.repeat_interleave(g, 0).double()
    err = (w.T.double() - w_ref.double()).abs()
    assert bool((err <= w.T.double().abs() * (2.0 ** -4 + 8 * eps) + s_full * 2.0 ** -10).all())
    dec = torch.from_numpy(of.e4m3fn_decode(codes.numpy())).double()
    assert bool(((w_ref.double() - dec * s_full).abs() <= eps * w_ref.double().abs() + 1e-30).all())
    case = oq.fp8_weight_case(w, group_size)
    assert np.array_equal(ow.unpack_rows(case["qweight"], 8), case["q"])


def test_native_byte_layout_round_trip_and_first_words():
    from oracle import native_layout as nl
    k, n = 256, 32
    q = np.random.default_rng(0).integers(0, 256, size=(k, n), dtype=np.int32)
    packed = nl.native_pack8_bytes(q)
    assert packed.shape == (k // 16, 4 * n) and packed.dtype == np.int32
    assert np.array_equal(nl.native_unpack8_bytes(packed, k, n), q)
    words = packed.reshape(-1).view(np.uint32)
    # by hand: word 0 = rows 0..3 of column 0; word 2 = rows 32..35 (j = 1); word 4 = lane 1 -> column 1;
    # word 64 = lane 16 (o = 1) -> rows 8..11; word 256 = block 1 -> rows 64..67 (j = 2); word 512 = next K tile
    def word(rows, col):
        return sum(int(q[r, col]) << (8 * i) for i, r in enumerate(rows))
    assert int(words[0]) == word(range(0, 4), 0) and int(words[1]) == word(range(4, 8), 0)
    assert int(words[2]) == word(range(32, 36), 0) and int(words[4]) == word(range(0, 4), 1)
    assert int(words[64]) == word(range(8, 12), 0) and int(words[256]) == word(range(64, 68), 0)
    assert int(words[512]) == word(range(128, 132), 0) and int(words[1024]) == word(range(0, 4), 16)
