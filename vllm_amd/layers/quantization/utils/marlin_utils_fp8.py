"""Weight-only FP8 (e4m3 weights, 16-bit activations) on the W4A16 GEMM -- the counterpart of the reference's
``vllm/model_executor/layers/quantization/utils/marlin_utils_fp8.py`` (pack_fp8_to_int32 :299-313,
prepare_fp8_layer_for_marlin :85-176, apply_fp8_marlin_linear :41-82, fp8_fused_exponent_bias_into_scales :25-38).  The
reference uses this path on GPUs without FP8 matrix hardware or when ``VLLM_TEST_FORCE_FP8_MARLIN`` is set; gfx950 has
FP8 MFMA, so here it only runs when forced."""
from __future__ import annotations

import torch

from vllm_amd import _custom_ops as ops
from vllm_amd.scalar_type import scalar_types
from .marlin_utils import (USE_FP32_REDUCE_DEFAULT, marlin_make_workspace_new, marlin_permute_bias,
                           marlin_permute_scales, should_use_atomic_add_reduce)


def is_fp8_marlin_supported() -> bool:
    return True


def fp8_fused_exponent_bias_into_scales(scales: torch.Tensor) -> torch.Tensor:
    """The reference's Marlin kernel turns an e4m3 byte into a 16-bit float by shifting its bits, which leaves the value
    short of a factor 2 ** (bias_16 - bias_8); that factor goes into the scales (marlin_utils_fp8.py:25-38).  Only the
    ``layout="marlin"`` parity path needs it: the gfx950 kernels convert exactly."""
    target_exponent = 5 if scales.dtype == torch.half else 8
    exponent_bias = 2 ** (target_exponent - 1) - 2 ** (4 - 1)
    return scales * (torch.ones_like(scales) * 2) ** exponent_bias


def pack_fp8_to_int32(fp8_tensor: torch.Tensor, size_k_first: bool = True) -> torch.Tensor:
    """FP8 weight -> GPTQ-style int32 [K/4, N]: four consecutive k of one column per word, low byte first."""
    assert fp8_tensor.dtype == torch.float8_e4m3fn and fp8_tensor.ndim == 2
    t = (fp8_tensor.T if size_k_first else fp8_tensor).contiguous()        # [N, K]
    packed = t.view(torch.int32)                                           # [N, K/4]
    return packed.T.contiguous() if size_k_first else packed


def prepare_fp8_layer_for_marlin(layer: torch.nn.Module, size_k_first: bool = True, layout: str = "native") -> None:
    """marlin_utils_fp8.py:85-176 for per-tensor / per-channel scales (block-wise FP8 is not built here): repack the
    weight, expand the scales to one row of one value per output channel in the activation dtype."""
    part_size_n = layer.output_size_per_partition
    part_size_k = layer.input_size_per_partition
    if getattr(layer, "weight_block_size", None) is not None:
        raise NotImplementedError("block-wise FP8 weights are not built for gfx950")
    assert layer.weight.shape == ((part_size_k, part_size_n) if size_k_first else (part_size_n, part_size_k))
    device = layer.weight.device
    layer.workspace = marlin_make_workspace_new(device, size_n=part_size_n)
    perm = torch.empty(0, dtype=torch.int, device=device)
    qweight = pack_fp8_to_int32(layer.weight, size_k_first)
    if not size_k_first:
        qweight = qweight.T.contiguous()
    repacked = ops.gptq_marlin_repack(b_q_weight=qweight, perm=perm, size_k=part_size_k, size_n=part_size_n, num_bits=8,
                                      layout="marlin" if layout == "marlin" else "native_bytes")
    layer.weight = torch.nn.Parameter(repacked, requires_grad=False)

    scales = layer.weight_scale.to(layer.orig_dtype)
    if scales.nelement() == 1:
        scales = scales.view(1, 1).repeat_interleave(part_size_n, 1)                 # per tensor -> per channel
    elif scales.nelement() != part_size_n:
        # one scale per logical shard of a fused module -> per channel.  (The reference repeats every scale
        # part_size_n / shards times, which is right for equal shards; with the layer's own widths it is right for
        # q / k / v of different widths too.)
        widths = getattr(layer, "logical_widths", None)
        if widths is not None and len(widths) == scales.nelement():
            scales = scales.view(-1).repeat_interleave(torch.tensor(list(widths), device=scales.device)).view(1, part_size_n)
        else:
            assert part_size_n % scales.nelement() == 0
            s_size = scales.nelement()
            scales = scales.view(1, s_size).repeat_interleave(part_size_n // s_size, 1)
    else:
        scales = scales.view(1, part_size_n)
    scales = marlin_permute_scales(s=scales.contiguous(), size_k=part_size_k, size_n=part_size_n, group_size=-1, layout=layout)
    if layout == "marlin":
        scales = fp8_fused_exponent_bias_into_scales(scales)
    layer.weight_scale = torch.nn.Parameter(scales, requires_grad=False)
    if hasattr(layer, "bias") and layer.bias is not None:
        assert layer.bias.shape == (part_size_n,)
        layer.bias.data = marlin_permute_bias(layer.bias.data, layout=layout)


def apply_fp8_marlin_linear(input: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
                            workspace: torch.Tensor, size_n: int, size_k: int, bias: torch.Tensor | None,
                            use_fp32_reduce: bool = USE_FP32_REDUCE_DEFAULT) -> torch.Tensor:
    """marlin_utils_fp8.py:41-82."""
    reshaped_x = input.reshape(-1, input.shape[-1])
    out_shape = input.shape[:-1] + (size_n,)
    use_atomic_add = should_use_atomic_add_reduce(m=reshaped_x.size(0), n=size_n, k=size_k, device=input.device,
                                                  dtype=input.dtype)
    output = ops.gptq_marlin_gemm(a=reshaped_x, c=None, b_q_weight=weight, b_bias=bias, b_scales=weight_scale,
                                  global_scale=None, b_zeros=None, g_idx=None, perm=None, workspace=workspace,
                                  b_q_type=scalar_types.float8_e4m3fn, size_m=reshaped_x.size(0), size_n=size_n,
                                  size_k=size_k, use_atomic_add=use_atomic_add, use_fp32_reduce=use_fp32_reduce)
    return output.reshape(out_shape)
