"""Writes the small committed fixtures under tests/golden/ from the CPU oracle (seeded).  They freeze the oracle's
answers -- themselves pinned by the cross-checks in tests/test_oracle_*.py -- so that a later edit of the oracle cannot
drift silently.  Run from the repo root:  python tests/golden/make_golden.py"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import fp8, native_layout, w4a16  # noqa: E402


def main():
    rng = np.random.default_rng(20240611)
    k, n = 128, 64
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    perm = rng.permutation(k).astype(np.int32)
    zp = rng.integers(0, 16, size=(1, n), dtype=np.int32)
    qweight = w4a16.gptq_pack(q, 4)
    np.savez_compressed(
        os.path.join(HERE, "w4a16_small.npz"), q=q, qweight=qweight, perm=perm, zp=zp,
        marlin=w4a16.marlin_weights(q), marlin_perm=w4a16.marlin_repack_thread_map(qweight, perm, k, n),
        native=native_layout.native_pack(q), marlin_zp=w4a16.marlin_zero_points(zp, 1, n, 4))

    g = torch.Generator().manual_seed(7)
    x = (torch.randn(5, 72, generator=g) * torch.tensor([1e-3, 1.0, 30.0, 500.0, 0.0]).reshape(5, 1)).to(torch.bfloat16)
    codes, scales = fp8.ref_dynamic_per_token_quant(x)
    ub = torch.tensor([20.0])
    codes_ub, scales_ub = fp8.ref_dynamic_per_token_quant(x, ub)
    codes_t, scale_t = fp8.ref_dynamic_per_tensor_quant(x)
    np.savez_compressed(
        os.path.join(HERE, "fp8_quant_small.npz"), x_bits=x.view(torch.int16).numpy(),
        codes=codes.view(torch.uint8).numpy(), scales=scales.numpy(), ub=ub.numpy(),
        codes_ub=codes_ub.view(torch.uint8).numpy(), scales_ub=scales_ub.numpy(),
        codes_tensor=codes_t.view(torch.uint8).numpy(), scale_tensor=scale_t.numpy())


if __name__ == "__main__":
    main()
