"""CPU statement of this build's own NATIVE weight order (no reference counterpart: the reference treats the
repacked tensor as opaque, marlin.py:85-91 / :153-166).  TEST INFRASTRUCTURE ONLY.

Tile (kt, nt) = rows 128*kt.., columns 16*nt.. is the 256-word block number nt*(K/128)+kt (the tiles of a
16-column strip are contiguous along K).  Word 4*L + j of a tile,
L = 16*o + r, holds the codes of rows 128*kt + 32*j + 8*o + e (e = 0..7) of column 16*nt + r; code e sits in nibble
position p with {0,2,4,6,1,3,5,7}[p] == e.  The inverse (`native_unpack`) is the documented map back to the logical
[K, N] code matrix.

8-bit codes are stored as two 4-bit planes: the 1 KiB block 2*(nt*(K/128)+kt) is the tile of the high nibbles
(code >> 4) in the order above, the block after it the tile of the low nibbles (code & 15).
"""
from __future__ import annotations

import numpy as np

_POS_TO_E = np.array([0, 2, 4, 6, 1, 3, 5, 7])


def _index_maps(size_k: int, size_n: int):
    """For every output word (flat index) the row index of its 8 codes (in nibble-position order) and its column."""
    assert size_k % 128 == 0 and size_n % 16 == 0
    k_tiles = size_k // 128
    idx = np.arange(size_k * size_n // 8, dtype=np.int64)
    j = idx & 3
    lane = (idx >> 2) & 63
    tile = idx >> 8
    nt, kt = tile // k_tiles, tile % k_tiles
    o, r = lane >> 4, lane & 15
    k0 = kt * 128 + j * 32 + o * 8
    n = nt * 16 + r
    rows = k0[:, None] + _POS_TO_E[None, :]          # [words, 8] row of the code in nibble position p
    return rows, n


def native_pack(q: np.ndarray) -> np.ndarray:
    """Logical codes int[K, N] (rows already in sorted order for act_order) -> int32 [K/16, 2N]."""
    size_k, size_n = q.shape
    rows, n = _index_maps(size_k, size_n)
    codes = np.asarray(q).astype(np.uint32)[rows, n[:, None]]                 # [words, 8]
    shifts = (np.arange(8, dtype=np.uint32) * 4)[None, :]
    words = np.bitwise_or.reduce(codes << shifts, axis=1).astype(np.uint32)
    return words.view(np.int32).reshape(size_k // 16, 2 * size_n)


def native_unpack(packed: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    """Inverse of :func:`native_pack`."""
    words = np.asarray(packed).reshape(-1).view(np.uint32)
    rows, n = _index_maps(size_k, size_n)
    shifts = (np.arange(8, dtype=np.uint32) * 4)[None, :]
    codes = (words[:, None] >> shifts) & np.uint32(0xF)
    q = np.zeros((size_k, size_n), dtype=np.int32)
    q[rows, n[:, None]] = codes.astype(np.int32)
    return q


def native_pack8(q: np.ndarray) -> np.ndarray:
    """Logical 8-bit codes int[K, N] -> int32 [K/16, 4N]: per tile the high-nibble plane, then the low-nibble plane."""
    size_k, size_n = q.shape
    q = np.asarray(q).astype(np.int32)
    hi = native_pack(q >> 4).reshape(-1, 256)
    lo = native_pack(q & 15).reshape(-1, 256)
    return np.stack([hi, lo], axis=1).reshape(size_k // 16, 4 * size_n)


def native_unpack8(packed: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    """Inverse of :func:`native_pack8`."""
    planes = np.asarray(packed).reshape(-1, 2, 256)
    hi = native_unpack(planes[:, 0].reshape(size_k // 16, 2 * size_n), size_k, size_n)
    lo = native_unpack(planes[:, 1].reshape(size_k // 16, 2 * size_n), size_k, size_n)
    return (hi << 4) | lo


def _byte_index_maps(size_k: int, size_n: int):
    """For every output word of the byte layout the rows of its four bytes (low byte first) and its column."""
    assert size_k % 128 == 0 and size_n % 16 == 0
    k_tiles = size_k // 128
    idx = np.arange(size_k * size_n // 4, dtype=np.int64)
    q = idx & 3
    lane = (idx >> 2) & 63
    h = (idx >> 8) & 1
    tile = idx >> 9
    nt, kt = tile // k_tiles, tile % k_tiles
    o, r = lane >> 4, lane & 15
    j = 2 * h + (q >> 1)
    k0 = kt * 128 + j * 32 + o * 8 + (q & 1) * 4
    return k0[:, None] + np.arange(4)[None, :], nt * 16 + r


def native_pack8_bytes(q: np.ndarray) -> np.ndarray:
    """Logical 8-bit codes int[K, N] -> int32 [K/16, 4N], whole bytes (the layout of FP8 weights): per tile two 1 KiB
    blocks; block h gives lane L = 16*o + r the 16 bytes of rows 128*kt + 32*j + 8*o + e, j = 2h (bytes 0..7) and
    j = 2h + 1 (bytes 8..15), column 16*nt + r."""
    size_k, size_n = q.shape
    rows, n = _byte_index_maps(size_k, size_n)
    codes = np.asarray(q).astype(np.uint32)[rows, n[:, None]]
    shifts = (np.arange(4, dtype=np.uint32) * 8)[None, :]
    words = np.bitwise_or.reduce(codes << shifts, axis=1).astype(np.uint32)
    return words.view(np.int32).reshape(size_k // 16, 4 * size_n)


def native_unpack8_bytes(packed: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    """Inverse of :func:`native_pack8_bytes`."""
    words = np.asarray(packed).reshape(-1).view(np.uint32)
    rows, n = _byte_index_maps(size_k, size_n)
    shifts = (np.arange(4, dtype=np.uint32) * 8)[None, :]
    codes = (words[:, None] >> shifts) & np.uint32(0xFF)
    q = np.zeros((size_k, size_n), dtype=np.int32)
    q[rows, n[:, None]] = codes.astype(np.int32)
    return q
