"""Single-GPU linear layers that delegate to a quantization method -- the caller side of the plugin contract in the
reference's ``vllm/model_executor/layers/linear.py`` (LinearBase :243-300; forward -> ``quant_method.apply`` at
:399/:565/:1405) -- and the checkpoint side: every parameter carries ``weight_loader`` = the layer's
``weight_loader_v2``, which places a checkpoint tensor (the whole matrix, one logical part of a fused layer such as
``gate_proj`` / ``"q"``, or an already fused tensor) inside the layer's parameters (linear.py:549,:784-866,:948-1060,
:1379).  Tensor-parallel sharding is out of scope: partition sizes equal full sizes."""
from __future__ import annotations

import torch

from ..parameter import BasevLLMParameter, PerTensorScaleParameter, _ColumnvLLMParameter
from .quantization.base_config import LinearMethodBase, QuantizationConfig


class UnquantizedLinearMethod(LinearMethodBase):
    def create_weights(self, layer, input_size_per_partition, output_partition_sizes, input_size, output_size,
                       params_dtype, **extra_weight_attrs):
        from ..parameter import ModelWeightParameter
        layer.register_parameter("weight", ModelWeightParameter(
            data=torch.empty(sum(output_partition_sizes), input_size_per_partition, dtype=params_dtype), input_dim=1,
            output_dim=0, weight_loader=extra_weight_attrs.get("weight_loader")))

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
                                         self.params_dtype, weight_loader=self.weight_loader_v2)
        if bias:
            self.bias = _ColumnvLLMParameter(data=torch.zeros(output_size, dtype=self.params_dtype), output_dim=0,
                                             weight_loader=self.weight_loader_v2)
        else:
            self.register_parameter("bias", None)

    # ---- checkpoint loading ------------------------------------------------------------------------------------------
    def _part_offset_and_size(self, loaded_shard_id) -> tuple[int, int]:
        """Where logical part `loaded_shard_id` (an index, or "q" / "k" / "v") sits along the output dimension."""
        idx = {"q": 0, "k": 1, "v": 2}.get(loaded_shard_id, loaded_shard_id)
        if not isinstance(idx, int) or not 0 <= idx < len(self.output_sizes):
            raise ValueError(f"unknown shard id {loaded_shard_id!r} for a layer with {len(self.output_sizes)} parts")
        return sum(self.output_sizes[:idx]), self.output_sizes[idx]

    def weight_loader_v2(self, param: BasevLLMParameter, loaded_weight: torch.Tensor, loaded_shard_id=None) -> None:
        """Copy one checkpoint tensor into `param`.  Without a shard id the tensor covers the whole layer: a fused
        tensor is cut along the output dimension into the layer's logical parts (a per-tensor scale then belongs to all
        of them and goes to entry 0, the maximum over the entries is taken after loading); with a shard id it is
        one logical part."""
        if loaded_shard_id is None:
            if isinstance(param, PerTensorScaleParameter):
                param.load_merged_column_weight(loaded_weight=loaded_weight, shard_id=0)
            elif len(self.output_sizes) == 1 or param.output_dim is None:
                param.load_column_parallel_weight(loaded_weight)
            else:
                for idx in range(len(self.output_sizes)):
                    offset, size = self._part_offset_and_size(idx)
                    if param.packed_dim is not None and param.packed_dim == param.output_dim:
                        size, offset = param.adjust_shard_indexes_for_packing(size, offset)
                    self.weight_loader_v2(param, loaded_weight.narrow(param.output_dim, offset, size), idx)
            return
        offset, size = self._part_offset_and_size(loaded_shard_id)
        param.load_merged_column_weight(loaded_weight=loaded_weight, shard_id=loaded_shard_id, shard_offset=offset,
                                        shard_size=size)

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
