"""CPU oracle for the quantized-linear path (GPTQ W4A16 + FP8 W8A8).

TEST INFRASTRUCTURE ONLY.  Nothing in this package is part of the product: it
is imported by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / the timed CPU baseline,
never by ``vllm_amd``.  Every function restates, in numpy / CPU torch, what
one reference function computes and cites the reference file:line it follows.

Pinning status (what fixes each function besides its own formula):

* ``w4a16.gptq_pack / pack_cols / unpack_cols``   closed form + brute force on
  tiny inputs + pack/unpack round trip.
* ``w4a16.marlin_weights`` (index-list description) versus
  ``w4a16.marlin_repack_thread_map`` (thread->element description of the
  device kernel): two independent descriptions the reference's own test
  asserts equal; required bit-equal here on the reference's size grid, plus
  the permutation invariant (nibble multiset preserved, inverse exists) and
  "repack with perm == repack of q[perm]".
* ``w4a16.get_scale_perms / marlin_permute_scales / marlin_zero_points``
  known-answer constants + inverse round trips.
* ``w4a16.dequantize / gemm_ref``   special cases that reduce to closed forms
  (s=1,q-z=1 -> row sums; one-hot A picks a dequantised row; zp==8 with uint4
  equals uint4b8; act_order == plain GEMM on A[:, perm]).
* ``w4a16.awq_pack``   one word packed by hand + inverse round trip.
* ``quantize.quantize_weights / gptq_quantize_weights / sort_weights / marlin_quantize /
  awq_marlin_quantize / scaled_quantize / scaled_dequantize / group_broadcast`` (the reference's weight quantisers,
  which its GEMM tests feed with random normal weights)   error bound of uniform quantisation (half a step; one step
  with a rounded zero point), textbook scales, extreme codes reached in every group, ranges, block-constant weights
  returned exactly, act_order bookkeeping (a permutation that ``sort_weights`` undoes group-wise, GEMM identity),
  hand-computed tiny groups, fp8 round trip; the case built from float weights dequantises through
  ``w4a16.dequantize`` to the quantiser's own ``w_ref`` bit for bit.
* ``fp8.ref_dynamic_per_token_quant``   torch CPU float8_e4m3fn cast versus an
  independent bit-level e4m3fn encoder brute-forced over all 65 536 bf16
  inputs; edge cases (zero row -> 1/(448*512), amax -> 0x7E, ties-to-even,
  subnormals, scale_ub).
* ``fp8.scaled_mm_ref``   fp64 matmul + single rounding; the three epilogue
  orders that exist in the reference differ by <= 1 output ulp (tested).

Nothing here is "parity unpinned" except the per-token x per-channel FP8 GEMM
*bitwise* result, which no reference test pins beyond tolerance (rtol 0.5 /
atol 0.15 in tests/kernels/quantization/test_cutlass_scaled_mm.py:96); the
oracle pins it with its own fp64 accumulation and the build states a much
tighter tolerance in its tests.
"""
