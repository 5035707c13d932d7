"""GPTQ W4A16 quantization method, same plugin surface as the reference's
``vllm/model_executor/layers/quantization/gptq_marlin.py`` (GPTQMarlinConfig :92-308, GPTQMarlinLinearMethod :311-466),
with the CUDA-only gate (``is_gptq_marlin_compatible`` :265) lifted for gfx950 and the kernel chosen among the HIP
mixed-precision kernels.  Parameters are plain ``torch.nn.Parameter`` (one GPU: no sharded-loader metadata)."""
from __future__ import annotations

import logging
from typing import Any, Optional

import torch

from vllm_amd.parameter import (ChannelQuantScaleParameter, GroupQuantScaleParameter, PackedColumnParameter,
                                PackedvLLMParameter, RowvLLMParameter)
from vllm_amd.scalar_type import scalar_types
from .base_config import LinearMethodBase, QuantizationConfig, QuantizeMethodBase
from .kernels.mixed_precision import MPLinearLayerConfig, choose_mp_linear_kernel
from .utils.marlin_utils import (check_marlin_supported, marlin_repeat_scales_on_all_ranks, verify_marlin_supported)

logger = logging.getLogger(__name__)


class GPTQMarlinConfig(QuantizationConfig):
    """Config class for GPTQ on the gfx950 W4A16 kernels."""

    # (num_bits, is_sym) -> quant_type   (gptq_marlin.py:96-99)
    TYPE_MAP = {(4, True): scalar_types.uint4b8, (8, True): scalar_types.uint8b128}

    def __init__(self, weight_bits: int, group_size: int, desc_act: bool, is_sym: bool, lm_head_quantized: bool = False,
                 dynamic: dict[str, dict[str, int | bool]] | None = None, full_config: dict[str, Any] | None = None,
                 modules_in_block_to_quantize: list[str] | None = None) -> None:
        super().__init__()
        if desc_act and group_size == -1:
            # one group per output channel: act_order changes nothing
            desc_act = False
        self.dynamic = dynamic or {}
        self.weight_bits = weight_bits
        self.is_sym = is_sym
        self.pack_factor = 32 // weight_bits
        self.group_size = group_size
        self.desc_act = desc_act
        self.lm_head_quantized = lm_head_quantized
        self.full_config = full_config or {}
        self.modules_in_block_to_quantize = modules_in_block_to_quantize or []
        if (weight_bits, is_sym) not in self.TYPE_MAP:
            raise ValueError(f"Unsupported quantization config: bits={weight_bits}, sym={is_sym}")
        self.quant_type = self.TYPE_MAP[(weight_bits, is_sym)]

    def __repr__(self) -> str:
        return (f"GPTQMarlinConfig(quant_type={self.quant_type}, group_size={self.group_size}, "
                f"desc_act={self.desc_act}, lm_head_quantized={self.lm_head_quantized})")

    @classmethod
    def get_name(cls) -> str:
        return "gptq_marlin"

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
    def from_config(cls, config: dict[str, Any]) -> "GPTQMarlinConfig":
        dynamic = cls.get_from_keys_or(config, ["dynamic"], default={}) or {}
        weight_bits = cls.get_from_keys(config, ["bits"])
        group_size = cls.get_from_keys(config, ["group_size"])
        desc_act = cls.get_from_keys(config, ["desc_act"])
        is_sym = cls.get_from_keys(config, ["sym"])
        lm_head_quantized = cls.get_from_keys_or(config, ["lm_head"], default=False)
        modules = cls.get_from_keys_or(config, ["modules_in_block_to_quantize"], default=None)
        return cls(weight_bits, group_size, desc_act, is_sym, lm_head_quantized, dynamic, config, modules)

    @classmethod
    def override_quantization_method(cls, hf_quant_cfg, user_quant) -> str | None:
        """Upgrade a plain ``gptq`` checkpoint to this method when it is compatible (gptq_marlin.py:213-238)."""
        can_convert = cls.is_gptq_marlin_compatible(hf_quant_cfg)
        is_valid_user_quant = user_quant is None or user_quant in ("marlin", "gptq_marlin")
        if can_convert and is_valid_user_quant:
            logger.info("The model is convertible to %s during runtime. Using %s kernel.", cls.get_name(), cls.get_name())
            return cls.get_name()
        if can_convert and user_quant == "gptq":
            logger.info("Detected that the model can run with gptq_marlin, however you specified quantization=gptq "
                        "explicitly, so forcing gptq. Use quantization=gptq_marlin for faster inference")
        return None

    @classmethod
    def is_gptq_marlin_compatible(cls, quant_config: dict[str, Any]) -> bool:
        quant_method = quant_config.get("quant_method", "").lower()
        num_bits = quant_config.get("bits")
        group_size = quant_config.get("group_size")
        sym = quant_config.get("sym")
        desc_act = quant_config.get("desc_act")
        if quant_method != "gptq":
            return False
        if num_bits is None or group_size is None or sym is None or desc_act is None:
            return False
        if (num_bits, sym) not in cls.TYPE_MAP:
            return False
        return check_marlin_supported(quant_type=cls.TYPE_MAP[(num_bits, sym)], group_size=group_size)

    def get_quant_method(self, layer: torch.nn.Module, prefix: str) -> Optional[QuantizeMethodBase]:
        from ..linear import LinearBase
        if isinstance(layer, LinearBase):
            return GPTQMarlinLinearMethod(self)
        return None


class GPTQMarlinLinearMethod(LinearMethodBase):
    """Linear method for GPTQ W4A16 on gfx950."""

    _kernel_backends_being_used: set[str] = set()

    def __init__(self, quant_config: GPTQMarlinConfig) -> None:
        self.quant_config = quant_config
        verify_marlin_supported(quant_type=self.quant_config.quant_type, group_size=self.quant_config.group_size)

    def create_weights(self, layer: torch.nn.Module, input_size_per_partition: int, output_partition_sizes: list[int],
                       input_size: int, output_size: int, params_dtype: torch.dtype, **extra_weight_attrs) -> None:
        output_size_per_partition = sum(output_partition_sizes)
        is_row_parallel = input_size != input_size_per_partition

        mp_linear_kernel_config = MPLinearLayerConfig(
            full_weight_shape=(input_size, output_size),
            partition_weight_shape=(input_size_per_partition, output_size_per_partition),
            weight_type=self.quant_config.quant_type, act_type=params_dtype, group_size=self.quant_config.group_size,
            zero_points=False, has_g_idx=self.quant_config.desc_act)
        kernel_type = choose_mp_linear_kernel(mp_linear_kernel_config)
        if kernel_type.__name__ not in self._kernel_backends_being_used:
            logger.info("Using %s for GPTQMarlinLinearMethod", kernel_type.__name__)
            self._kernel_backends_being_used.add(kernel_type.__name__)

        group_size = self.quant_config.group_size if self.quant_config.group_size != -1 else input_size
        if marlin_repeat_scales_on_all_ranks(self.quant_config.desc_act, self.quant_config.group_size, is_row_parallel):
            scales_and_zp_size = input_size // group_size
        else:
            scales_and_zp_size = input_size_per_partition // group_size

        pf = self.quant_config.pack_factor
        loader = extra_weight_attrs.get("weight_loader")
        # the checkpoint layout of gptq_marlin.py:380-440: qweight packed along the input dimension, qzeros along the
        # output dimension, scales / zero points one row per group (channelwise: one row)
        layer.register_parameter("qweight", PackedvLLMParameter(
            data=torch.empty(input_size_per_partition // pf, output_size_per_partition, dtype=torch.int32), input_dim=0,
            output_dim=1, packed_dim=0, packed_factor=pf, weight_loader=loader))
        layer.register_parameter("g_idx", RowvLLMParameter(
            data=torch.empty(input_size_per_partition, dtype=torch.int32), input_dim=0, weight_loader=loader))
        scale_cls = ChannelQuantScaleParameter if scales_and_zp_size == 1 and self.quant_config.group_size == -1 \
            else GroupQuantScaleParameter
        dims = dict(output_dim=1) if scale_cls is ChannelQuantScaleParameter else dict(output_dim=1, input_dim=0)
        layer.register_parameter("scales", scale_cls(
            data=torch.empty(scales_and_zp_size, output_size_per_partition, dtype=params_dtype), weight_loader=loader,
            **dims))
        if scale_cls is ChannelQuantScaleParameter:
            layer.register_parameter("qzeros", PackedColumnParameter(
                data=torch.empty(scales_and_zp_size, output_size_per_partition // pf, dtype=torch.int32), output_dim=1,
                packed_dim=1, packed_factor=pf, weight_loader=loader))
        else:
            layer.register_parameter("qzeros", PackedvLLMParameter(
                data=torch.empty(scales_and_zp_size, output_size_per_partition // pf, dtype=torch.int32), input_dim=0,
                output_dim=1, packed_dim=1, packed_factor=pf, weight_loader=loader))
        self.kernel = kernel_type(mp_linear_kernel_config, w_q_param_name="qweight", w_s_param_name="scales",
                                  w_zp_param_name="qzeros", w_gidx_param_name="g_idx")

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        self.kernel.process_weights_after_loading(layer)

    def apply(self, layer: torch.nn.Module, x: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
        return self.kernel.apply_weights(layer, x, bias)
