"""AWQ W4A16 quantization method, same plugin surface as the reference's
``vllm/model_executor/layers/quantization/awq_marlin.py`` (AWQMarlinConfig :66-259, AWQMarlinLinearMethod :264-413), with
the CUDA-only gate (``is_awq_marlin_compatible`` :217) lifted for gfx950.  AutoAWQ checkpoints store the weights as
int32 [K, N/8] and the zero points as int32 [K/g, N/8], both packed along N with the column interleave
{0,2,4,6,1,3,5,7}; after loading they are rewritten into what the W4A16 GEMM reads (native tile order, zero points in
natural column order).  Parameters are plain ``torch.nn.Parameter`` (one GPU: no sharded-loader metadata)."""
from __future__ import annotations

import logging
from typing import Any, Optional

import torch

from vllm_amd import _custom_ops as ops
from vllm_amd.parameter import GroupQuantScaleParameter, PackedvLLMParameter
from vllm_amd.scalar_type import scalar_types
from .base_config import LinearMethodBase, QuantizationConfig, QuantizeMethodBase
from .utils.marlin_utils import (apply_awq_marlin_linear, awq_to_marlin_zero_points, check_marlin_supported,
                                 check_marlin_supports_layer, marlin_make_empty_g_idx, marlin_make_workspace_new,
                                 marlin_permute_bias, marlin_permute_scales, verify_marlin_supported,
                                 verify_marlin_supports_shape)

logger = logging.getLogger(__name__)


def is_layer_skipped(prefix: str, ignored_layers: list[str], skip_with_substr: bool = False) -> bool:
    """quant_utils.py:283-343 without fused-module expansion (one GPU, no packed-module mapping here)."""
    if skip_with_substr:
        return any(ig in prefix for ig in ignored_layers)
    return prefix in ignored_layers


class AWQMarlinConfig(QuantizationConfig):
    """Config class for AWQ on the gfx950 W4A16 kernels."""

    # num_bits -> type   (8-bit is not built)
    TYPE_MAP = {4: scalar_types.uint4}

    def __init__(self, weight_bits: int, group_size: int, zero_point: bool, lm_head_quantized: bool = False,
                 modules_to_not_convert: list[str] | None = None, full_config: dict[str, Any] | None = None) -> None:
        super().__init__()
        if weight_bits not in self.TYPE_MAP:
            raise ValueError(f"Unsupported num_bits = {weight_bits}. Supported num_bits = {self.TYPE_MAP.keys()}")
        self.pack_factor = 32 // weight_bits
        self.group_size = group_size
        self.zero_point = zero_point
        self.lm_head_quantized = lm_head_quantized
        self.weight_bits = weight_bits
        self.modules_to_not_convert = modules_to_not_convert or []
        self.full_config = full_config or {}
        self.quant_type = self.TYPE_MAP[self.weight_bits]
        verify_marlin_supported(self.quant_type, group_size=self.group_size, has_zp=self.zero_point)

    def __repr__(self) -> str:
        return (f"AWQMarlinConfig(quant_type={self.quant_type}, group_size={self.group_size}, "
                f"zero_point={self.zero_point}, lm_head_quantized={self.lm_head_quantized}, "
                f"modules_to_not_convert={self.modules_to_not_convert})")

    @classmethod
    def get_name(cls) -> str:
        return "awq_marlin"

    @classmethod
    def get_supported_act_dtypes(cls) -> list[torch.dtype]:
        return [torch.half, torch.bfloat16]

    @classmethod
    def get_min_capability(cls) -> int:
        return 95

    @classmethod
    def get_config_filenames(cls) -> list[str]:
        return ["quantize_config.json"]

    @classmethod
    def from_config(cls, config: dict[str, Any]) -> "AWQMarlinConfig":
        weight_bits = cls.get_from_keys(config, ["bits"])
        group_size = cls.get_from_keys(config, ["group_size"])
        zero_point = cls.get_from_keys(config, ["zero_point"])
        lm_head_quantized = cls.get_from_keys_or(config, ["lm_head"], default=False)
        modules_to_not_convert = cls.get_from_keys_or(config, ["modules_to_not_convert"], None)
        return cls(weight_bits, group_size, zero_point, lm_head_quantized, modules_to_not_convert, config)

    @classmethod
    def override_quantization_method(cls, hf_quant_cfg, user_quant) -> str | None:
        """Upgrade a plain ``awq`` checkpoint to this method when it is compatible (awq_marlin.py:146-171)."""
        can_convert = cls.is_awq_marlin_compatible(hf_quant_cfg)
        is_valid_user_quant = user_quant is None or user_quant == "marlin" or user_quant == "awq_marlin"
        if can_convert and is_valid_user_quant:
            logger.info("The model is convertible to %s during runtime. Using %s kernel.", cls.get_name(), cls.get_name())
            return cls.get_name()
        if can_convert and user_quant == "awq":
            logger.info("Detected that the model can run with awq_marlin, however you specified quantization=awq "
                        "explicitly, so forcing awq. Use quantization=awq_marlin for faster inference")
        return None

    @classmethod
    def is_awq_marlin_compatible(cls, quant_config: dict[str, Any]) -> bool:
        quant_method = quant_config.get("quant_method", "").lower()
        num_bits = quant_config.get("bits")
        group_size = quant_config.get("group_size")
        zero_point = quant_config.get("zero_point")
        if quant_method != "awq":
            return False
        if num_bits is None or group_size is None or zero_point is None:
            return False
        if num_bits not in cls.TYPE_MAP:
            return False
        return check_marlin_supported(quant_type=cls.TYPE_MAP[num_bits], group_size=group_size, has_zp=zero_point)

    def get_quant_method(self, layer: torch.nn.Module, prefix: str) -> Optional[QuantizeMethodBase]:
        from ..linear import LinearBase, UnquantizedLinearMethod
        if isinstance(layer, LinearBase):
            if is_layer_skipped(prefix, self.modules_to_not_convert, skip_with_substr=True):
                return UnquantizedLinearMethod()
            if not check_marlin_supports_layer(layer, self.group_size):
                # the reference falls back to its unoptimised AWQ kernels here (awq_marlin.py:186-193); none are built
                raise NotImplementedError(f"Layer '{prefix}' has a shape the gfx950 W4A16 kernels do not support and "
                                          "there is no fallback AWQ kernel in this build")
            return AWQMarlinLinearMethod(self)
        return None


class AWQMarlinLinearMethod(LinearMethodBase):
    """Linear method for AWQ W4A16 on gfx950."""

    def __init__(self, quant_config: AWQMarlinConfig) -> None:
        self.quant_config = quant_config

    def create_weights(self, layer: torch.nn.Module, input_size_per_partition: int, output_partition_sizes: list[int],
                       input_size: int, output_size: int, params_dtype: torch.dtype, **extra_weight_attrs) -> None:
        del output_size
        output_size_per_partition = sum(output_partition_sizes)
        group_size = self.quant_config.group_size if self.quant_config.group_size != -1 else input_size
        verify_marlin_supports_shape(output_size_per_partition=output_size_per_partition,
                                     input_size_per_partition=input_size_per_partition, input_size=input_size,
                                     group_size=group_size)
        pf = self.quant_config.pack_factor
        num_groups = input_size_per_partition // group_size
        loader = extra_weight_attrs.get("weight_loader")
        # AutoAWQ checkpoint layout (awq_marlin.py:296-340): weights and zero points packed along the output dimension
        layer.register_parameter("qweight", PackedvLLMParameter(
            data=torch.empty(input_size_per_partition, output_size_per_partition // pf, dtype=torch.int32), input_dim=0,
            output_dim=1, packed_dim=1, packed_factor=pf, weight_loader=loader))
        layer.register_parameter("qzeros", PackedvLLMParameter(
            data=torch.empty(num_groups, output_size_per_partition // pf, dtype=torch.int32), input_dim=0, output_dim=1,
            packed_dim=1, packed_factor=pf, weight_loader=loader))
        layer.register_parameter("scales", GroupQuantScaleParameter(
            data=torch.empty(num_groups, output_size_per_partition, dtype=params_dtype), input_dim=0, output_dim=1,
            weight_loader=loader))
        layer.input_size_per_partition = input_size_per_partition
        layer.output_size_per_partition = output_size_per_partition
        layer.num_groups = num_groups

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        device = layer.qweight.device
        P = lambda t: torch.nn.Parameter(t, requires_grad=False)   # noqa: E731
        layer.workspace = marlin_make_workspace_new(device, size_n=layer.output_size_per_partition)
        num_bits = self.quant_config.quant_type.size_bits
        layer.qweight = P(ops.awq_marlin_repack(layer.qweight.data, size_k=layer.input_size_per_partition,
                                                size_n=layer.output_size_per_partition, num_bits=num_bits))
        layer.scales = P(marlin_permute_scales(layer.scales.data, size_k=layer.input_size_per_partition,
                                               size_n=layer.output_size_per_partition,
                                               group_size=self.quant_config.group_size))
        layer.qzeros = P(awq_to_marlin_zero_points(layer.qzeros.data, size_k=layer.num_groups,
                                                   size_n=layer.output_size_per_partition, num_bits=num_bits))
        layer.g_idx = marlin_make_empty_g_idx(device)
        layer.g_idx_sort_indices = marlin_make_empty_g_idx(device)
        if getattr(layer, "bias", None) is not None:
            layer.bias.data = marlin_permute_bias(layer.bias.data)

    def apply(self, layer: torch.nn.Module, x: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
        return apply_awq_marlin_linear(input=x, weight=layer.qweight, weight_scale=layer.scales, weight_zp=layer.qzeros,
                                       g_idx=layer.g_idx, g_idx_sort_indices=layer.g_idx_sort_indices,
                                       workspace=layer.workspace, quant_type=self.quant_config.quant_type,
                                       output_size_per_partition=layer.output_size_per_partition,
                                       input_size_per_partition=layer.input_size_per_partition, bias=bias)
