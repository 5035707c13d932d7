"""Host helpers of the GPTQ W4A16 linear, same names and argument meaning as the reference's
``vllm/model_executor/layers/quantization/utils/marlin_utils.py``.

The repacked weight, the permuted scales / zero points / bias are *opaque* between
``process_weights_after_loading`` and ``gptq_marlin_gemm`` (the reference only fixes their shapes), so each helper
takes ``layout``: ``"native"`` (default) is what the gfx950 kernels read -- scales and bias stay in their natural
order, zero points are packed 8 per int32 in natural column order -- and ``"marlin"`` reproduces the reference's
permutations bit-for-bit (kept for the parity contract; the gfx950 GEMM does not accept it).
"""
from __future__ import annotations

import torch

from vllm_amd import _custom_ops as ops
from vllm_amd.scalar_type import ScalarType, scalar_types
from .quant_utils import pack_cols, unpack_cols

GPTQ_MARLIN_TILE = 16
GPTQ_MARLIN_MIN_THREAD_N = 64
GPTQ_MARLIN_MIN_THREAD_K = 128
GPTQ_MARLIN_MAX_PARALLEL = 16

MARLIN_SUPPORTED_GROUP_SIZES = [-1, 32, 64, 128]
# what the gfx950 kernels implement out of the above (marlin_utils.py:24)
HIP_W4A16_SUPPORTED_GROUP_SIZES = [-1, 32, 64, 128]
HIP_W8A16_SUPPORTED_GROUP_SIZES = [-1, 32, 64, 128]      # uint8b128 weights

USE_FP32_REDUCE_DEFAULT = True

# int32 arrival counters handed to the GEMM: one per 16-column tile and m-block of the largest layer served.
_WORKSPACE_INTS = 65536

_INTERLEAVE4 = (0, 2, 4, 6, 1, 3, 5, 7)


def query_marlin_supported_quant_types(has_zp: bool | None = None, include_fp_type: bool = True,
                                       device_capability: int | None = None) -> list[ScalarType]:
    """marlin_utils.py:35-69, restricted to the integer types built for gfx950."""
    if has_zp is None:
        return (query_marlin_supported_quant_types(False, include_fp_type, device_capability) +
                query_marlin_supported_quant_types(True, include_fp_type, device_capability))
    return [scalar_types.uint4] if has_zp else [scalar_types.uint4b8, scalar_types.uint8b128]


def _check_marlin_supported(quant_type: ScalarType, group_size: int | None, has_zp: bool,
                            device_capability: int | None = None) -> tuple[bool, str | None]:
    supported_types = query_marlin_supported_quant_types(has_zp, True, device_capability)
    if quant_type not in supported_types:
        return (False, f"The gfx950 W4A16 kernels do not support weight_bits = {quant_type}. Only types = "
                       f"{supported_types} are supported (for group_size = {group_size}, zp = {has_zp}).")
    if group_size is None or group_size not in HIP_W4A16_SUPPORTED_GROUP_SIZES:
        return (False, f"The gfx950 W4A16 kernels do not support group_size = {group_size}. Only group_sizes = "
                       f"{HIP_W4A16_SUPPORTED_GROUP_SIZES} are supported.")
    if quant_type == scalar_types.uint8b128 and group_size not in HIP_W8A16_SUPPORTED_GROUP_SIZES:
        return (False, f"The gfx950 kernels do not support group_size = {group_size} for {quant_type}. Only group_sizes = "
                       f"{HIP_W8A16_SUPPORTED_GROUP_SIZES} are supported.")
    return True, None


def check_marlin_supported(quant_type: ScalarType, group_size: int, has_zp: bool = False,
                           device_capability: int | None = None) -> bool:
    return _check_marlin_supported(quant_type, group_size, has_zp, device_capability)[0]


def verify_marlin_supported(quant_type: ScalarType, group_size: int, has_zp: bool = False) -> None:
    cond, err_msg = _check_marlin_supported(quant_type, group_size, has_zp)
    if not cond:
        assert err_msg is not None
        raise ValueError(err_msg)


def verify_marlin_supports_shape(output_size_per_partition: int, input_size_per_partition: int, input_size: int,
                                 group_size: int) -> None:
    """marlin_utils.py:126-158."""
    if output_size_per_partition % GPTQ_MARLIN_MIN_THREAD_N != 0:
        raise ValueError(f"Weight output_size_per_partition = {output_size_per_partition} is not divisible by "
                         f" min_thread_n = {GPTQ_MARLIN_MIN_THREAD_N}. Consider reducing tensor_parallel_size or "
                         "running with --quantization gptq.")
    if input_size_per_partition % GPTQ_MARLIN_MIN_THREAD_K != 0:
        raise ValueError(f"Weight input_size_per_partition = {input_size_per_partition} is not divisible by "
                         f"min_thread_k = {GPTQ_MARLIN_MIN_THREAD_K}. Consider reducing tensor_parallel_size or "
                         "running with --quantization gptq.")
    if group_size < input_size and input_size_per_partition % group_size != 0:
        raise ValueError(f"Weight input_size_per_partition = {input_size_per_partition} is not divisible by "
                         f"group_size = {group_size}. Consider reducing tensor_parallel_size or running with "
                         "--quantization gptq.")


def check_marlin_supports_shape(output_size_per_partition: int, input_size_per_partition: int, input_size: int,
                                group_size: int) -> tuple[bool, str | None]:
    try:
        verify_marlin_supports_shape(output_size_per_partition, input_size_per_partition, input_size, group_size)
    except ValueError as e:
        return False, e.__str__()
    return True, None


def marlin_workspace_ints(size_n: int | None = None) -> int:
    """Arrival counters the GEMM can ask for on a layer with `size_n` output columns, whatever the batch size: the decode
    kernels use one per 16-column tile and 16-row block (up to four blocks: size_n / 4), the tile kernel at most 4096.
    Without a width: enough for 262144 columns."""
    if size_n is None:
        return _WORKSPACE_INTS
    return max(size_n // 4, 4096)


def marlin_make_workspace_new(device: torch.device, max_blocks_per_sm: int = 1, size_n: int | None = None) -> torch.Tensor:
    """Zeroed int32 counters for the GEMM's split-K hand-off (marlin_utils.py:237-245).  The GEMM requires them zero
    on entry and leaves them zero, and reports a workspace that is too small for the kernel it runs.  `size_n` (not in
    the reference, whose count depends on the device only) sizes the array for one layer."""
    return torch.zeros(marlin_workspace_ints(size_n) * max_blocks_per_sm, dtype=torch.int, device=device,
                       requires_grad=False)


def marlin_is_k_full(act_order: bool, is_row_parallel: bool) -> bool:
    return (not act_order) or (act_order and not is_row_parallel)


def marlin_repeat_scales_on_all_ranks(act_order: bool, group_size: int, is_row_parallel: bool) -> bool:
    is_channelwise = group_size == -1
    return act_order or (is_channelwise and is_row_parallel)


def marlin_make_empty_g_idx(device: torch.device) -> torch.Tensor:
    return torch.nn.Parameter(torch.empty(0, dtype=torch.int, device=device), requires_grad=False)


def marlin_make_empty_zp(device: torch.device) -> torch.Tensor:
    return torch.nn.Parameter(torch.empty(0, dtype=torch.int, device=device), requires_grad=False)


def marlin_sort_g_idx(g_idx: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    g_idx_sort_indices = torch.argsort(g_idx, stable=True).to(torch.int)
    return g_idx[g_idx_sort_indices], g_idx_sort_indices


def get_scale_perms() -> tuple[list[int], list[int]]:
    scale_perm = [i + 8 * j for i in range(8) for j in range(8)]
    scale_perm_single = [2 * i + j for i in range(4) for j in (0, 1, 8, 9, 16, 17, 24, 25)]
    return scale_perm, scale_perm_single


def marlin_permute_scales(s: torch.Tensor, size_k: int, size_n: int, group_size: int, *,
                          layout: str = "native") -> torch.Tensor:
    if layout == "native":
        return s.reshape((-1, size_n)).contiguous()
    scale_perm, scale_perm_single = get_scale_perms()
    if group_size < size_k and group_size != -1:
        s = s.reshape((-1, len(scale_perm)))[:, scale_perm]
    else:
        s = s.reshape((-1, len(scale_perm_single)))[:, scale_perm_single]
    return s.reshape((-1, size_n)).contiguous()


def marlin_permute_bias(s: torch.Tensor, *, layout: str = "native") -> torch.Tensor:
    if layout == "native":
        return s.contiguous()
    origin_shape = s.shape
    _, scale_perm_single = get_scale_perms()
    s = s.reshape((-1, len(scale_perm_single)))[:, scale_perm_single]
    return s.reshape(*origin_shape).contiguous()


def marlin_zero_points(zp: torch.Tensor, size_k: int, size_n: int, num_bits: int, *,
                       layout: str = "native") -> torch.Tensor:
    """``zp`` int [groups, N] (values) -> int32 [groups, N/8].  ``size_k`` is the number of groups, as in the
    reference (marlin_utils.py:326-346)."""
    if num_bits != 4:
        raise NotImplementedError(f"num_bits must be 4 for the gfx950 kernels, got {num_bits}")
    if layout == "native":
        return pack_cols(zp.reshape((-1, size_n)).contiguous(), num_bits, size_k, size_n)
    scale_perm, _ = get_scale_perms()
    zp = zp.reshape((-1, len(scale_perm)))[:, scale_perm]
    interleave = torch.tensor(_INTERLEAVE4, device=zp.device)
    zp = zp.reshape((-1, len(_INTERLEAVE4)))[:, interleave].reshape((-1, size_n)).contiguous()
    return pack_cols(zp, num_bits, size_k, size_n)


def awq_to_marlin_zero_points(q_zp_packed: torch.Tensor, size_k: int, size_n: int, num_bits: int, *,
                              layout: str = "native") -> torch.Tensor:
    """AWQ zero points (packed along N with the AWQ interleave) -> the GEMM's zero-point format
    (marlin_utils.py:349-370)."""
    q_zp = unpack_cols(q_zp_packed, num_bits, size_k, size_n)
    undo = torch.argsort(torch.tensor(_INTERLEAVE4, device=q_zp.device))
    q_zp = q_zp.reshape((-1, len(_INTERLEAVE4)))[:, undo].reshape((-1, size_n)).contiguous()
    return marlin_zero_points(q_zp, size_k, size_n, num_bits, layout=layout)


def should_use_atomic_add_reduce(m: int, n: int, k: int, device: torch.device, dtype: torch.dtype) -> bool:
    """The gfx950 GEMM has a single, deterministic fp32 reduction; the Marlin atomic-add variant does not exist."""
    return False


def apply_gptq_marlin_linear(input: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
                             weight_zp: torch.Tensor, g_idx: torch.Tensor, g_idx_sort_indices: torch.Tensor,
                             workspace: torch.Tensor, wtype: ScalarType, output_size_per_partition: int,
                             input_size_per_partition: int, is_k_full: bool, bias: torch.Tensor | None = None,
                             use_fp32_reduce: bool = USE_FP32_REDUCE_DEFAULT) -> torch.Tensor:
    """marlin_utils.py:435-482."""
    reshaped_x = input.reshape(-1, input.shape[-1])
    out_shape = input.shape[:-1] + (output_size_per_partition,)
    use_atomic_add = should_use_atomic_add_reduce(m=reshaped_x.size(0), n=output_size_per_partition,
                                                  k=reshaped_x.size(1), device=input.device, dtype=input.dtype)
    output = ops.gptq_marlin_gemm(reshaped_x, None, weight, bias, weight_scale, None, weight_zp, g_idx,
                                  g_idx_sort_indices, workspace, wtype, size_m=reshaped_x.shape[0],
                                  size_n=output_size_per_partition, size_k=input_size_per_partition,
                                  is_k_full=is_k_full, use_atomic_add=use_atomic_add, use_fp32_reduce=use_fp32_reduce,
                                  is_zp_float=False)
    return output.reshape(out_shape)


def apply_awq_marlin_linear(input: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
                            weight_zp: torch.Tensor, g_idx: torch.Tensor, g_idx_sort_indices: torch.Tensor,
                            workspace: torch.Tensor, quant_type: ScalarType, output_size_per_partition: int,
                            input_size_per_partition: int, bias: torch.Tensor | None = None,
                            use_fp32_reduce: bool = USE_FP32_REDUCE_DEFAULT) -> torch.Tensor:
    """marlin_utils.py:485-530."""
    reshaped_x = input.reshape(-1, input.shape[-1])
    out_shape = input.shape[:-1] + (output_size_per_partition,)
    use_atomic_add = should_use_atomic_add_reduce(m=reshaped_x.size(0), n=output_size_per_partition,
                                                  k=reshaped_x.size(1), device=input.device, dtype=input.dtype)
    output = ops.gptq_marlin_gemm(reshaped_x, None, weight, bias, weight_scale, None, weight_zp, g_idx,
                                  g_idx_sort_indices, workspace, quant_type, size_m=reshaped_x.shape[0],
                                  size_n=output_size_per_partition, size_k=input_size_per_partition,
                                  use_atomic_add=use_atomic_add, use_fp32_reduce=use_fp32_reduce, is_zp_float=False)
    return output.reshape(out_shape)


def check_marlin_supports_layer(layer: torch.nn.Module, group_size: int) -> bool:
    """marlin_utils.py:161-178: shape test of a linear layer before a method is attached to it."""
    output_size_per_partition = getattr(layer, "output_size_per_partition", None) or layer.output_size
    input_size_per_partition = getattr(layer, "input_size_per_partition", None) or layer.input_size
    return check_marlin_supports_shape(output_size_per_partition=output_size_per_partition,
                                       input_size_per_partition=input_size_per_partition,
                                       input_size=layer.input_size, group_size=group_size)[0]
