"""Single-GPU linear layers that delegate to a quantization method -- the caller side of the plugin contract in the
reference's ``vllm/model_executor/layers/linear.py`` (LinearBase :243-300; forward -> ``quant_method.apply`` at
:399/:565/:1405).  Tensor-parallel sharding is out of scope: partition sizes equal full sizes."""
from __future__ import annotations

import torch

from .quantization.base_config import LinearMethodBase, QuantizationConfig


class UnquantizedLinearMethod(LinearMethodBase):
    def create_weights(self, layer, input_size_per_partition, output_partition_sizes, input_size, output_size,
                       params_dtype, **extra_weight_attrs):
        layer.register_parameter("weight", torch.nn.Parameter(
            torch.empty(sum(output_partition_sizes), input_size_per_partition, dtype=params_dtype), requires_grad=False))

    def apply(self, layer, x, bias=None):
        return torch.nn.functional.linear(x, layer.weight, bias)


class LinearBase(torch.nn.Module):
    """``y = quant_method.apply(self, x, bias)``; returns ``(output, output_bias)`` like the reference."""

    def __init__(self, input_size: int, output_size: int, bias: bool = False, skip_bias_add: bool = False,
                 params_dtype: torch.dtype | None = None, quant_config: QuantizationConfig | None = None,
                 prefix: str = "", *, output_sizes: list[int] | None = None, return_bias: bool = True):
        super().__init__()
        self.input_size = input_size
        self.output_size = output_size
        self.skip_bias_add = skip_bias_add
        self.params_dtype = params_dtype or torch.get_default_dtype()
        self.quant_config = quant_config
        self.prefix = prefix
        self.return_bias = return_bias
        self.output_sizes = output_sizes or [output_size]
        self.quant_method = None
        if quant_config is not None:
            self.quant_method = quant_config.get_quant_method(self, prefix=prefix)
        if self.quant_method is None:
            self.quant_method = UnquantizedLinearMethod()
        self.quant_method.create_weights(self, input_size, self.output_sizes, input_size, output_size,
                                         self.params_dtype)
        if bias:
            self.bias = torch.nn.Parameter(torch.zeros(output_size, dtype=self.params_dtype), requires_grad=False)
        else:
            self.register_parameter("bias", None)

    def process_weights_after_loading(self) -> None:
        self.quant_method.process_weights_after_loading(self)

    def forward(self, x: torch.Tensor):
        bias = self.bias if not self.skip_bias_add else None
        output = self.quant_method.apply(self, x, bias)
        if not self.return_bias:
            return output
        return output, (self.bias if self.skip_bias_add else None)


class ColumnParallelLinear(LinearBase):
    pass


class MergedColumnParallelLinear(LinearBase):
    def __init__(self, input_size: int, output_sizes: list[int], **kw):
        super().__init__(input_size, sum(output_sizes), output_sizes=list(output_sizes), **kw)


class QKVParallelLinear(LinearBase):
    def __init__(self, hidden_size: int, head_size: int, total_num_heads: int, total_num_kv_heads: int | None = None, **kw):
        kv = total_num_kv_heads if total_num_kv_heads is not None else total_num_heads
        sizes = [total_num_heads * head_size, kv * head_size, kv * head_size]
        super().__init__(hidden_size, sum(sizes), output_sizes=sizes, **kw)


class RowParallelLinear(LinearBase):
    pass
