"""Packing helpers of the checkpoint formats, device-resident (pure torch integer ops, no host round trip).

Same functions as the reference's ``quant_utils.py`` (get_pack_factor :341, pack_rows/gptq_pack :524-545/:605-611,
pack_cols :548-570, unpack_cols :573-602), which run in numpy on the host.
"""
from __future__ import annotations

import torch


def get_pack_factor(num_bits: int) -> int:
    assert 32 % num_bits == 0, f"Unsupported num_bits = {num_bits}"
    return 32 // num_bits


def _shifts(num_bits: int, device) -> torch.Tensor:
    return torch.arange(get_pack_factor(num_bits), dtype=torch.int64, device=device) * num_bits


def _to_i32(x64: torch.Tensor) -> torch.Tensor:
    """Low 32 bits of non-negative int64 values, reinterpreted as int32."""
    x64 = x64 & 0xFFFFFFFF
    return torch.where(x64 >= 2 ** 31, x64 - 2 ** 32, x64).to(torch.int32)


def pack_cols(q_w: torch.Tensor, num_bits: int, size_k: int, size_n: int) -> torch.Tensor:
    assert q_w.shape == (size_k, size_n)
    pf = get_pack_factor(num_bits)
    assert size_n % pf == 0
    g = q_w.to(torch.int64).reshape(size_k, size_n // pf, pf) & ((1 << num_bits) - 1)
    return _to_i32((g << _shifts(num_bits, q_w.device)).sum(dim=-1)).contiguous()


def unpack_cols(packed_q_w: torch.Tensor, num_bits: int, size_k: int, size_n: int) -> torch.Tensor:
    pf = get_pack_factor(num_bits)
    assert size_n % pf == 0
    assert packed_q_w.shape == (size_k, size_n // pf), (
        f"packed_q_w.shape = {tuple(packed_q_w.shape)} size_k = {size_k}, size_n = {size_n} pack_factor = {pf}")
    p = packed_q_w.to(torch.int64) & 0xFFFFFFFF
    vals = (p.unsqueeze(-1) >> _shifts(num_bits, packed_q_w.device)) & ((1 << num_bits) - 1)
    return vals.reshape(size_k, size_n).to(torch.int32).contiguous()


def pack_rows(q_w: torch.Tensor, num_bits: int, size_k: int, size_n: int) -> torch.Tensor:
    assert q_w.shape == (size_k, size_n)
    pf = get_pack_factor(num_bits)
    assert size_k % pf == 0
    g = q_w.to(torch.int64).reshape(size_k // pf, pf, size_n) & ((1 << num_bits) - 1)
    return _to_i32((g << _shifts(num_bits, q_w.device).reshape(1, pf, 1)).sum(dim=1)).contiguous()


def gptq_pack(q_w: torch.Tensor, num_bits: int, size_k: int, size_n: int) -> torch.Tensor:
    return pack_rows(q_w, num_bits, size_k, size_n)
