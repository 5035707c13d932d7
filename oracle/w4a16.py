"""CPU oracle for the GPTQ W4A16 path (numpy for integer work, CPU torch for bf16/fp16).

TEST INFRASTRUCTURE ONLY -- never imported by the product package.

All ``file:line`` citations are relative to the reference tree.
"""
from __future__ import annotations

import numpy as np
import torch

TILE = 16          # marlin tile edge, marlin_utils.py:19
TILE_N = 64        # repack kernel n-tile, gptq_marlin_repack.cu:12-13 (tile_k_size=16, tile_n_size=64)
INTERLEAVE4 = (0, 2, 4, 6, 1, 3, 5, 7)   # marlin_utils_test.py:82, gptq_marlin_repack.cu:180
INTERLEAVE8 = (0, 2, 1, 3)               # 8-bit codes: marlin_utils_test.py:84, gptq_marlin_repack.cu:191


def pack_factor(num_bits: int) -> int:
    """quant_utils.py:341-343"""
    assert 32 % num_bits == 0
    return 32 // num_bits


# --------------------------------------------------------------------------- packing

def pack_rows(q: np.ndarray, num_bits: int) -> np.ndarray:
    """``qweight[r, n] = OR_i q[pf*r + i, n] << (bits*i)`` -- quant_utils.py:524-545 (gptq_pack :605-611)."""
    q = np.asarray(q).astype(np.uint32)
    pf = pack_factor(num_bits)
    k, n = q.shape
    assert k % pf == 0
    grouped = q.reshape(k // pf, pf, n)
    shifts = (np.arange(pf, dtype=np.uint32) * num_bits).reshape(1, pf, 1)
    return np.bitwise_or.reduce(grouped << shifts, axis=1).astype(np.uint32).view(np.int32)


gptq_pack = pack_rows


def unpack_rows(packed: np.ndarray, num_bits: int) -> np.ndarray:
    """Inverse of :func:`pack_rows` (the reference has no such helper; round-trip pinned)."""
    p = np.asarray(packed).view(np.uint32)
    pf = pack_factor(num_bits)
    mask = np.uint32((1 << num_bits) - 1)
    shifts = (np.arange(pf, dtype=np.uint32) * num_bits).reshape(1, pf, 1)
    out = (p[:, None, :] >> shifts) & mask
    return out.reshape(p.shape[0] * pf, p.shape[1]).astype(np.int32)


def pack_cols(q: np.ndarray, num_bits: int) -> np.ndarray:
    """``out[k, c] = OR_i q[k, pf*c + i] << (bits*i)`` -- quant_utils.py:548-570."""
    q = np.asarray(q).astype(np.uint32)
    pf = pack_factor(num_bits)
    k, n = q.shape
    assert n % pf == 0
    grouped = q.reshape(k, n // pf, pf)
    shifts = (np.arange(pf, dtype=np.uint32) * num_bits).reshape(1, 1, pf)
    return np.bitwise_or.reduce(grouped << shifts, axis=2).astype(np.uint32).view(np.int32)


def unpack_cols(packed: np.ndarray, num_bits: int) -> np.ndarray:
    """quant_utils.py:573-602."""
    p = np.asarray(packed).view(np.uint32)
    pf = pack_factor(num_bits)
    mask = np.uint32((1 << num_bits) - 1)
    shifts = (np.arange(pf, dtype=np.uint32) * num_bits).reshape(1, 1, pf)
    out = (p[:, :, None] >> shifts) & mask
    return out.reshape(p.shape[0], p.shape[1] * pf).astype(np.int32)


def awq_pack(q: np.ndarray, num_bits: int) -> np.ndarray:
    """quant_utils.py:614-633: interleave each run of 8 columns, then pack along N."""
    assert num_bits == 4
    q = np.asarray(q)
    k, n = q.shape
    il = np.asarray(INTERLEAVE4)
    qi = q.reshape(-1, 8)[:, il].reshape(k, n)
    return pack_cols(qi, num_bits)


# --------------------------------------------------------------------------- marlin weight layout, description 1

def get_weight_perm(num_bits: int = 4) -> np.ndarray:
    """Index list of marlin_utils_test.py:66-93 (1024 entries over one 16x64 tile pair)."""
    assert num_bits in (4, 8)
    base = []
    for i in range(32):
        col = i // 4
        rows = (2 * (i % 4), 2 * (i % 4) + 1, 2 * (i % 4 + 4), 2 * (i % 4 + 4) + 1)
        one = [16 * r + col + 8 * blk for blk in (0, 1) for r in rows]
        for j in range(4):
            base.extend(p + 256 * j for p in one)
    perm = np.asarray(base, dtype=np.int64)
    il = np.asarray(INTERLEAVE4 if num_bits == 4 else INTERLEAVE8)
    return perm.reshape(-1, il.size)[:, il].ravel()


def marlin_permute_weights(q: np.ndarray, perm: np.ndarray) -> np.ndarray:
    """marlin_utils_test.py:32-45: 16x16 tiling, then the 1024-entry permutation."""
    k, n = q.shape
    assert k % TILE == 0 and n % TILE == 0
    t = q.reshape(k // TILE, TILE, n // TILE, TILE).transpose(0, 2, 1, 3).reshape(k // TILE, n * TILE)
    return t.reshape(-1, perm.size)[:, perm].reshape(t.shape)


def marlin_weights(q: np.ndarray, num_bits: int = 4) -> np.ndarray:
    """marlin_utils_test.py:48-63: permute + pack 8 nibbles (4 bytes) per int32 along the tiled axis -> int32
    [K/16, 2N] (4-bit) or [K/16, 4N] (8-bit)."""
    w = marlin_permute_weights(np.asarray(q), get_weight_perm(num_bits))
    return pack_cols(w, num_bits)


# --------------------------------------------------------------------------- marlin weight layout, description 2

def marlin_repack_thread_map(qweight: np.ndarray, perm: np.ndarray | None, size_k: int, size_n: int,
                             num_bits: int = 4) -> np.ndarray:
    """Thread->element restatement of the device repack kernel, gptq_marlin_repack.cu:112-203.

    ``qweight`` is the GPTQ tensor int32[K/pack_factor, N]; ``perm`` int32[K] (act_order sort indices) or None/empty.
    Output int32 [K/16, 2N] (4-bit: one word per thread, :177-188) or [K/16, 4N] (8-bit: two words per thread, one per
    column, :189-203).  Written as explicit loops over (warp, lane) vectorised over tiles.
    """
    pf = pack_factor(num_bits)
    qw = np.asarray(qweight).view(np.uint32)
    assert qw.shape == (size_k // pf, size_n)
    k_tiles, n_tiles = size_k // 16, size_n // TILE_N
    has_perm = perm is not None and len(perm) > 0
    tile_words = 16 * TILE_N // pf
    out = np.zeros((k_tiles * n_tiles * tile_words,), dtype=np.uint32)
    tc_offsets = (0, 1, 8, 9)
    mask = np.uint32((1 << num_bits) - 1)
    kt = np.arange(k_tiles).reshape(-1, 1)
    nt = np.arange(n_tiles).reshape(1, -1)
    for warp in range(4):
        for th in range(32):
            tc_col, tc_row = th // 4, (th % 4) * 2
            cur_n = warp * 16 + tc_col
            vals = []
            for half in (0, 8):            # b1 then b2  (cur_n, cur_n + 8)
                for off in tc_offsets:
                    k_in_tile = tc_row + off
                    dst_k = kt * 16 + k_in_tile                      # row of the (sorted) logical matrix
                    src_k = np.asarray(perm)[dst_k] if has_perm else dst_k
                    word = qw[src_k // pf, nt * TILE_N + cur_n + half]
                    vals.append((word >> ((src_k % pf) * num_bits).astype(np.uint32)) & mask)
            if num_bits == 4:
                res = np.zeros((k_tiles, n_tiles), dtype=np.uint32)
                for i, src in enumerate(INTERLEAVE4):
                    res |= vals[src] << np.uint32(4 * i)
                out_idx = (kt * n_tiles + nt) * tile_words + th * 4 + warp
                out[out_idx.ravel()] = res.ravel()
            else:
                for which in (0, 1):
                    res = np.zeros((k_tiles, n_tiles), dtype=np.uint32)
                    for i, src in enumerate(INTERLEAVE8):
                        res |= vals[4 * which + src] << np.uint32(8 * i)
                    out_idx = (kt * n_tiles + nt) * tile_words + th * 8 + warp * 2 + which
                    out[out_idx.ravel()] = res.ravel()
    return out.view(np.int32).reshape(k_tiles, size_n * 16 // pf)


def marlin_unpack_to_logical(marlin_w: np.ndarray, size_k: int, size_n: int, num_bits: int = 4) -> np.ndarray:
    """Inverse of :func:`marlin_weights` (int32 [K/16, 2N or 4N] -> code matrix [K, N]); used for invariants."""
    perm = get_weight_perm(num_bits)
    inv = np.argsort(perm)
    flat = unpack_cols(marlin_w, num_bits)               # [K/16, 16N]
    t = flat.reshape(-1, perm.size)[:, inv].reshape(size_k // TILE, size_n // TILE, TILE, TILE)
    return t.transpose(0, 2, 1, 3).reshape(size_k, size_n)


# --------------------------------------------------------------------------- scales / zero points / bias / g_idx

def get_scale_perms() -> tuple[list[int], list[int]]:
    """marlin_utils.py:278-285."""
    scale_perm = [i + 8 * j for i in range(8) for j in range(8)]
    single = [2 * i + j for i in range(4) for j in (0, 1, 8, 9, 16, 17, 24, 25)]
    return scale_perm, single


def marlin_permute_scales(s: np.ndarray, size_k: int, size_n: int, group_size: int) -> np.ndarray:
    """marlin_utils.py:288-298."""
    sp, sp1 = get_scale_perms()
    s = np.asarray(s)
    if group_size < size_k and group_size != -1:
        out = s.reshape(-1, 64)[:, sp]
    else:
        out = s.reshape(-1, 32)[:, sp1]
    return np.ascontiguousarray(out.reshape(-1, size_n))


def marlin_permute_bias(b: np.ndarray) -> np.ndarray:
    """marlin_utils.py:301-305."""
    _, sp1 = get_scale_perms()
    b = np.asarray(b)
    return np.ascontiguousarray(b.reshape(-1, 32)[:, sp1].reshape(b.shape))


def marlin_zero_points(zp: np.ndarray, size_k: int, size_n: int, num_bits: int = 4) -> np.ndarray:
    """marlin_utils.py:326-346: zp int[G, N] (values) -> int32 [G, N/8]."""
    assert num_bits == 4
    sp, _ = get_scale_perms()
    z = np.asarray(zp).reshape(-1, 64)[:, sp]
    z = z.reshape(-1, 8)[:, np.asarray(INTERLEAVE4)].reshape(-1, size_n)
    return pack_cols(z, num_bits)


def awq_to_marlin_zero_points(q_zp_packed: np.ndarray, size_k: int, size_n: int, num_bits: int = 4) -> np.ndarray:
    """marlin_utils.py:349-370."""
    z = unpack_cols(q_zp_packed, num_bits)
    undo = np.argsort(np.asarray(INTERLEAVE4))
    z = z.reshape(-1, 8)[:, undo].reshape(-1, size_n)
    return marlin_zero_points(z, size_k, size_n, num_bits)


def marlin_sort_g_idx(g_idx: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """marlin_utils.py:273-275 (stable argsort so the oracle is deterministic; any argsort of equal keys is valid)."""
    order = np.argsort(np.asarray(g_idx), kind="stable").astype(np.int32)
    return np.asarray(g_idx)[order], order


def permute_rows(q: np.ndarray, group_size: int, rand_perm: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """quant_utils.py:346-373 (act_order simulation): returns (q[rand_perm], g_idx[rand_perm])."""
    k = q.shape[0]
    g_idx = (np.arange(k) // group_size).astype(np.int32)
    return np.ascontiguousarray(q[rand_perm]), np.ascontiguousarray(g_idx[rand_perm])


# --------------------------------------------------------------------------- dequantise + GEMM (the tolerance oracle)

def dequantize(q: np.ndarray, scales: torch.Tensor, zp: np.ndarray | int, group_size: int,
               g_idx: np.ndarray | None = None) -> torch.Tensor:
    """``w_ref = (w_q - zp).to(dtype) * w_s`` -- quant_utils.py:441, evaluated in the 16-bit activation dtype.

    ``q`` int [K, N] codes (0..15, or 0..255 for 8-bit weights) in *storage row order*; ``scales`` [G, N] bf16/fp16 CPU tensor;
    ``zp`` either the bias of the symmetric type (8 for uint4b8, 128 for uint8b128) or an int [G, N] array; ``g_idx`` [K] group of each stored row
    (act_order) or None for ``row // group_size``.
    The product ``(q - z) * s`` is an exact fp32 value rounded once to the 16-bit dtype, which is what
    both the torch CPU multiply and the device ``__hmul2`` (marlin_template.h:162-171) produce.
    """
    k, n = q.shape
    if group_size == -1:
        group_size = k          # channelwise: one group spans K (marlin_utils.py:66, quant_utils.py:395-396)
    grp = (np.arange(k) // group_size) if g_idx is None else np.asarray(g_idx).astype(np.int64)
    grp_t = torch.from_numpy(np.asarray(grp, dtype=np.int64))
    if isinstance(zp, (int, np.integer)):
        centred = torch.from_numpy((np.asarray(q, dtype=np.int32) - int(zp)).astype(np.float32))
    else:
        centred = torch.from_numpy((np.asarray(q, dtype=np.int32) - np.asarray(zp, dtype=np.int32)[grp]).astype(np.float32))
    return centred.to(scales.dtype) * scales[grp_t]


def gemm_ref(a: torch.Tensor, w_ref: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """High-precision reference ``C = A @ W`` in fp64 (+bias), *not* rounded -- the tolerance is measured against this
    and against :func:`gemm_ref_like_reference` (the reference test's ``torch.matmul(a, w_ref)``,
    test_marlin_gemm.py:355)."""
    out = a.double() @ w_ref.double()
    if bias is not None:
        out = out + bias.double()
    return out


def gemm_ref_like_reference(a: torch.Tensor, w_ref: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    out = torch.matmul(a, w_ref)
    if bias is not None:
        out = out + bias
    return out


def rel_err_mean(out: torch.Tensor, ref: torch.Tensor) -> float:
    """Reference metric ``mean|out-ref| / mean|ref|`` -- test_marlin_gemm.py:78-82 (threshold 0.04 there)."""
    return float((out.double() - ref.double()).abs().mean() / ref.double().abs().mean())


def rel_err_max(out: torch.Tensor, ref: torch.Tensor) -> float:
    """max|out-ref| / max|ref| (the build's own stricter metric: <= 2e-2 required, see tests)."""
    return float((out.double() - ref.double()).abs().max() / ref.double().abs().max())


# --------------------------------------------------------------------------- synthetic layers (BASELINE.json configs)

def make_w4a16_case(k: int, n: int, group_size: int = 128, *, asym: bool = False, act_order: bool = False,
                    group_level_perm: bool = False, dtype: torch.dtype = torch.bfloat16, seed: int = 0,
                    num_bits: int = 4) -> dict:
    """Synthetic GPTQ layer in checkpoint format, as the BASELINE.json configs specify it.

    Keys: ``q`` int32[K,N] codes 0..15 (row r multiplies activation column r, as in a GPTQ checkpoint),
    ``qweight`` int32[K/8,N] = gptq_pack(q), ``scales`` [G,N] ``dtype`` (made in fp16 then cast, as a checkpoint
    loader would), ``zp_vals`` int32[G,N] / ``qzeros`` int32[G,N/8] (asym only, else None),
    ``g_idx`` int32[K] (act_order only: group of row r, = (arange(K)//g)[rand_perm], quant_utils.py:357-366),
    ``group_size`` (-1: channelwise, one group), ``num_bits`` (4, or 8: codes 0..255 with the fixed zero point 128,
    the ``uint8b128`` type).  ``group_level_perm`` permutes whole groups instead of single rows.
    """
    rng = np.random.default_rng(seed)
    orig_group_size = group_size
    if group_size == -1:
        group_size = k
    g = k // group_size
    assert num_bits == 4 or not asym, "8-bit codes are symmetric only (uint8b128)"
    q = rng.integers(0, 1 << num_bits, size=(k, n), dtype=np.int32)
    tg = torch.Generator().manual_seed(seed)
    scales = (torch.randn(g, n, generator=tg).abs() * 0.01 + 1e-3).to(torch.float16).to(dtype)
    zp_vals = rng.integers(0, 16, size=(g, n), dtype=np.int32) if asym else None
    g_idx = None
    if act_order:
        if group_level_perm:
            gp = rng.permutation(g)
            rand_perm = (gp[:, None] * group_size + np.arange(group_size)[None, :]).ravel()
        else:
            rand_perm = rng.permutation(k)
        g_idx = (np.arange(k) // group_size).astype(np.int32)[rand_perm]
    return dict(q=q, qweight=gptq_pack(q, num_bits), scales=scales, zp_vals=zp_vals,
                qzeros=pack_cols(zp_vals, 4) if asym else None, g_idx=g_idx, group_size=orig_group_size, num_bits=num_bits)


def case_w_ref(case: dict) -> torch.Tensor:
    """Dequantised weight [K, N] such that ``C = A @ w_ref`` (rows in checkpoint order)."""
    zp = (1 << (case.get("num_bits", 4) - 1)) if case["zp_vals"] is None else case["zp_vals"]     # uint4b8: 8, uint8b128: 128
    return dequantize(case["q"], case["scales"], zp, case["group_size"], case["g_idx"])
