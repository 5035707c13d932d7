"""FP8 W8A8 quantization methods, same plugin surface as the reference's
``vllm/model_executor/layers/quantization/fp8.py`` (Fp8Config :150-327, Fp8LinearMethod :330-684, non-block,
non-Marlin branches) and ``ptpc_fp8.py`` (PTPCFp8LinearMethod :82-137: per-channel weights, per-token activations)."""
from __future__ import annotations

import os
from typing import Any, Optional

import torch
from torch.nn import Parameter

from vllm_amd import _custom_ops as ops
from vllm_amd.parameter import ModelWeightParameter, PerTensorScaleParameter
from .base_config import LinearMethodBase, QuantizationConfig, QuantizeMethodBase
from .input_quant_fp8 import GroupShape
from .utils.marlin_utils_fp8 import apply_fp8_marlin_linear, prepare_fp8_layer_for_marlin
from .utils.w8a8_utils import Fp8LinearOp

ACTIVATION_SCHEMES = ["static", "dynamic"]


class Fp8Config(QuantizationConfig):
    def __init__(self, is_checkpoint_fp8_serialized: bool = False, activation_scheme: str = "dynamic",
                 ignored_layers: list[str] | None = None, weight_block_size: list[int] | None = None) -> None:
        super().__init__()
        self.is_checkpoint_fp8_serialized = is_checkpoint_fp8_serialized
        if activation_scheme not in ACTIVATION_SCHEMES:
            raise ValueError(f"Unsupported activation scheme {activation_scheme}")
        self.activation_scheme = activation_scheme
        self.ignored_layers = ignored_layers or []
        if weight_block_size is not None:
            raise NotImplementedError("block-wise FP8 weights are not built for gfx950")
        self.weight_block_size = None

    @classmethod
    def get_name(cls) -> str:
        return "fp8"

    @classmethod
    def get_supported_act_dtypes(cls) -> list[torch.dtype]:
        return [torch.bfloat16, torch.half]

    @classmethod
    def get_min_capability(cls) -> int:
        return 95

    @classmethod
    def get_config_filenames(cls) -> list[str]:
        return []

    @classmethod
    def from_config(cls, config: dict[str, Any]) -> "Fp8Config":
        quant_method = cls.get_from_keys(config, ["quant_method"])
        is_checkpoint_fp8_serialized = "fp8" in quant_method
        activation_scheme = cls.get_from_keys(config, ["activation_scheme"])
        ignored_layers = cls.get_from_keys_or(config, ["ignored_layers"], None)
        weight_block_size = cls.get_from_keys_or(config, ["weight_block_size"], None)
        return cls(is_checkpoint_fp8_serialized, activation_scheme, ignored_layers, weight_block_size)

    def get_quant_method(self, layer: torch.nn.Module, prefix: str) -> Optional[QuantizeMethodBase]:
        from ..linear import LinearBase
        if isinstance(layer, LinearBase):
            if any(prefix == ig or prefix.startswith(ig + ".") for ig in self.ignored_layers):
                return None
            return Fp8LinearMethod(self)
        return None


class Fp8LinearMethod(LinearMethodBase):
    """FP8 linear: per-tensor weight scale, dynamic (per-token) or static (per-tensor) activation scale."""

    def __init__(self, quant_config: Fp8Config):
        self.quant_config = quant_config
        self.out_dtype = torch.get_default_dtype()
        self.block_quant = False
        # Weight-only FP8 on the W4A16 GEMM: the reference takes this route on GPUs without FP8 matrix hardware or when
        # VLLM_TEST_FORCE_FP8_MARLIN is set (fp8.py:353-363).  gfx950 has FP8 MFMA: only when forced.
        self.use_marlin = os.environ.get("VLLM_TEST_FORCE_FP8_MARLIN", "0").lower() in ("1", "true")
        self.act_q_static = self.quant_config.activation_scheme == "static"
        # per-token activation scales whenever they are dynamic: the fused GEMM takes them at no extra cost
        self.act_q_group_shape = GroupShape.PER_TENSOR if self.act_q_static else GroupShape.PER_TOKEN
        self.fp8_linear = Fp8LinearOp(act_quant_static=self.act_q_static, act_quant_group_shape=self.act_q_group_shape)

    def create_weights(self, layer: torch.nn.Module, input_size_per_partition: int, output_partition_sizes: list[int],
                       input_size: int, output_size: int, params_dtype: torch.dtype, **extra_weight_attrs):
        output_size_per_partition = sum(output_partition_sizes)
        layer.logical_widths = output_partition_sizes
        layer.input_size_per_partition = input_size_per_partition
        layer.output_size_per_partition = output_size_per_partition
        layer.orig_dtype = params_dtype
        layer.weight_block_size = None
        weight_dtype = ops.FP8_DTYPE if self.quant_config.is_checkpoint_fp8_serialized else params_dtype
        loader = extra_weight_attrs.get("weight_loader")
        layer.register_parameter("weight", ModelWeightParameter(
            data=torch.empty(output_size_per_partition, input_size_per_partition, dtype=weight_dtype), input_dim=1,
            output_dim=0, weight_loader=loader))
        if self.quant_config.is_checkpoint_fp8_serialized:
            # one scale per logical matrix of a fused layer, initialised to the most negative float so that the maximum
            # taken after loading ignores entries no checkpoint tensor filled (fp8.py:405-428)
            def per_part():
                return PerTensorScaleParameter(data=torch.full((len(output_partition_sizes),),
                                                               torch.finfo(torch.float32).min, dtype=torch.float32),
                                               weight_loader=loader)
            layer.register_parameter("weight_scale", per_part())
            if self.act_q_static:
                layer.register_parameter("input_scale", per_part())
            else:
                layer.register_parameter("input_scale", None)

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        input_scale = None
        if not self.quant_config.is_checkpoint_fp8_serialized:
            # 16-bit checkpoint: quantise the weight per tensor on the device (fp8.py:497-500)
            qweight, weight_scale = ops.scaled_fp8_quant(layer.weight, scale=None)
            weight = qweight.t()
        else:
            weight = layer.weight
            weight_scale = layer.weight_scale
            if weight_scale.numel() > 1:
                # fused module with one scale per logical shard (fp8_utils.py:1086-1111
                # process_fp8_weight_tensor_strategy; w8a8_utils.py:108-136 requantize_with_max_scale)
                max_w_scale = weight_scale.max()
                # A module that is already fused on disk brings ONE scale: it sits in entry 0 and the last entry still
                # holds its initial value.  Its weight is quantised with that single scale already and stays as it is.
                unfused_in_checkpoint = bool(weight_scale[-1] > torch.finfo(torch.float8_e4m3fn).min)
                if unfused_in_checkpoint and self.use_marlin:
                    max_w_scale = weight_scale      # the weight-only path keeps one scale per shard (expanded per channel below)
                elif unfused_in_checkpoint:
                    # one scale per shard: requantise every shard to the largest one
                    start = 0
                    deq = torch.zeros_like(weight, dtype=torch.float32)
                    for idx, width in enumerate(layer.logical_widths):
                        if width == 0:
                            continue
                        deq[start:start + width] = weight[start:start + width].to(torch.float32) * weight_scale[idx]
                        start += width
                    weight, _ = ops.scaled_fp8_quant(deq, max_w_scale.reshape(1))
                weight_scale = max_w_scale
            if self.act_q_static:
                input_scale = layer.input_scale.max()
            weight = weight.t()
        layer.weight = Parameter(weight.data, requires_grad=False)
        layer.weight_scale = Parameter(weight_scale.data.reshape(-1)[:1].reshape(()) if weight_scale.numel() == 1
                                       else weight_scale.data, requires_grad=False)
        layer.input_scale = Parameter(input_scale, requires_grad=False) if input_scale is not None else None
        if self.use_marlin:
            prepare_fp8_layer_for_marlin(layer, size_k_first=True)
            layer.input_scale = None          # activations are not quantised on this path

    def apply(self, layer: torch.nn.Module, x: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
        if self.use_marlin:
            return apply_fp8_marlin_linear(input=x, weight=layer.weight, weight_scale=layer.weight_scale,
                                           workspace=layer.workspace, size_n=layer.output_size_per_partition,
                                           size_k=layer.input_size_per_partition, bias=bias)
        return self.fp8_linear.apply(input=x, weight=layer.weight, weight_scale=layer.weight_scale,
                                     out_dtype=self.out_dtype if x.dtype not in (torch.float16, torch.bfloat16) else x.dtype,
                                     input_scale=layer.input_scale, bias=bias)


class PTPCFp8Config(Fp8Config):
    """Per-token activations x per-channel weights, quantised from a 16-bit checkpoint at load (ptpc_fp8.py:31-79)."""

    def __init__(self, activation_scheme: str = "dynamic", ignored_layers: list[str] | None = None) -> None:
        if activation_scheme == "static":
            raise ValueError("ptpc_fp8 as of now only support dynamic quantization.")
        super().__init__(is_checkpoint_fp8_serialized=False, activation_scheme=activation_scheme,
                         ignored_layers=ignored_layers)

    @classmethod
    def get_name(cls) -> str:
        return "ptpc_fp8"

    @classmethod
    def from_config(cls, config: dict[str, Any]) -> "PTPCFp8Config":
        activation_scheme = cls.get_from_keys_or(config, ["activation_scheme"], "dynamic")
        ignored_layers = cls.get_from_keys_or(config, ["ignored_layers"], None)
        return cls(activation_scheme=activation_scheme, ignored_layers=ignored_layers)

    def get_quant_method(self, layer: torch.nn.Module, prefix: str) -> Optional[QuantizeMethodBase]:
        from ..linear import LinearBase
        if isinstance(layer, LinearBase):
            if any(prefix == ig or prefix.startswith(ig + ".") for ig in self.ignored_layers):
                return None
            return PTPCFp8LinearMethod(self)
        return None


class PTPCFp8LinearMethod(Fp8LinearMethod):
    def __init__(self, quant_config: PTPCFp8Config):
        super().__init__(quant_config=quant_config)
        self.fp8_linear = Fp8LinearOp(act_quant_static=False, act_quant_group_shape=GroupShape.PER_TOKEN)

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        assert layer.weight.data.dtype in (torch.bfloat16, torch.float16), "PTPC quantises a 16-bit checkpoint"
        # one scale per output channel = the per-token quantiser applied to the [N, K] weight rows (ptpc_fp8.py:107-123)
        qweight, weight_scale = ops.scaled_fp8_quant(layer.weight, scale=None, use_per_token_if_dynamic=True)
        layer.weight = Parameter(qweight.t(), requires_grad=False)       # [K, N] column-major view
        layer.weight_scale = Parameter(weight_scale, requires_grad=False)  # [N, 1]
        layer.input_scale = None

    def apply(self, layer: torch.nn.Module, x: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
        return self.fp8_linear.apply(input=x, weight=layer.weight, weight_scale=layer.weight_scale, out_dtype=x.dtype,
                                     input_scale=None, input_scale_ub=None, bias=bias)
