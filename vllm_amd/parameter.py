"""Parameter classes that know how a checkpoint tensor lands in a (possibly fused) linear layer -- the loader-side
contract of the reference's ``vllm/model_executor/parameter.py`` (BasevLLMParameter :31-126, column / row / per-tensor /
packed variants :129-408), for one GPU: a layer's partition is the whole matrix, so "this rank's slice" of a checkpoint
tensor is the tensor itself and only the placement of the logical sub-matrices (q/k/v, gate/up) inside a fused
parameter remains.

One implementation serves every class: a parameter records which of its dimensions is the output dimension, which the
input dimension and which (if any) is packed (several codes per int32); the classes only differ in which of these they
take.  Names, constructor keywords and the ``load_*`` methods are the reference's, so its layer-side loaders
(``weight_loader_v2``, linear.py:549,:820,:1009,:1379) and quantization methods work against them unchanged.
"""
from __future__ import annotations

from fractions import Fraction
from typing import Callable

import torch

__all__ = ["BasevLLMParameter", "ModelWeightParameter", "RowvLLMParameter", "GroupQuantScaleParameter",
           "ChannelQuantScaleParameter", "PerTensorScaleParameter", "PackedColumnParameter", "PackedvLLMParameter"]

_QKV_INDEX = {"q": 0, "k": 1, "v": 2}


class BasevLLMParameter(torch.nn.Parameter):
    """A frozen parameter plus the callable a model loader invokes for it (``param.weight_loader(param, tensor, ...)``).
    Without dimension metadata every ``load_*`` is a whole-tensor copy."""

    def __new__(cls, data: torch.Tensor | None = None, **kwargs):
        return super().__new__(cls, data=data, requires_grad=False)

    def __init__(self, data: torch.Tensor, weight_loader: Callable | None = None, *, output_dim: int | None = None,
                 input_dim: int | None = None, packed_dim: int | None = None,
                 packed_factor: int | Fraction | None = None, marlin_tile_size: int | None = None, **_ignored):
        self._weight_loader = weight_loader
        self._output_dim = output_dim
        self._input_dim = input_dim
        self._packed_dim = packed_dim
        self._packed_factor = packed_factor
        self._marlin_tile_size = marlin_tile_size
        self.tp_rank, self.tp_size = 0, 1

    # torch.nn.Parameter subclasses must pass through __torch_function__ untouched to keep their type on .to()/.data ops
    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        return super().__torch_function__(func, types, args, kwargs or {})

    @property
    def weight_loader(self) -> Callable:
        if self._weight_loader is None:
            raise AttributeError(f"{type(self).__name__} has no weight_loader")
        return self._weight_loader

    @weight_loader.setter
    def weight_loader(self, fn: Callable) -> None:
        self._weight_loader = fn

    # ---- placement helpers ------------------------------------------------------------------------------------------
    def _copy(self, dst: torch.Tensor, src: torch.Tensor) -> None:
        if src.ndim == 0 and dst.numel() == 1:
            src = src.reshape(dst.shape)           # a scalar scale from disk into a [1] parameter
        if dst.shape != src.shape:
            raise ValueError(f"{type(self).__name__}: checkpoint tensor of shape {tuple(src.shape)} does not fit the "
                             f"parameter region of shape {tuple(dst.shape)}")
        dst.copy_(src)

    def _region(self, shard_offset: int, shard_size: int) -> torch.Tensor:
        """The slice of this parameter that the logical sub-matrix [shard_offset, shard_offset + shard_size) of the output
        dimension occupies; offsets shrink by the pack factor when the output dimension is the packed one."""
        if self._output_dim is None:
            raise TypeError(f"{type(self).__name__} has no output dimension to shard")
        if self._packed_dim is not None and self._packed_dim == self._output_dim:
            shard_size, shard_offset = self.adjust_shard_indexes_for_packing(shard_size, shard_offset)
        return self.data.narrow(self._output_dim, shard_offset, shard_size)

    # ---- the loader contract ----------------------------------------------------------------------------------------
    def load_column_parallel_weight(self, loaded_weight: torch.Tensor) -> None:
        self._copy(self.data, loaded_weight)

    def load_row_parallel_weight(self, loaded_weight: torch.Tensor) -> None:
        self._copy(self.data, loaded_weight)

    def load_merged_column_weight(self, loaded_weight: torch.Tensor, **kwargs) -> None:
        if self._output_dim is None or kwargs.get("shard_offset") is None:
            self._copy(self.data, loaded_weight)
            return
        self._copy(self._region(kwargs["shard_offset"], kwargs["shard_size"]), loaded_weight)

    def load_qkv_weight(self, loaded_weight: torch.Tensor, **kwargs) -> None:
        # one GPU: every head lives here, so q, k and v are placed exactly like the parts of a merged column layer
        self.load_merged_column_weight(loaded_weight, **kwargs)

    # ---- metadata ---------------------------------------------------------------------------------------------------
    @property
    def output_dim(self):
        return self._output_dim

    @property
    def input_dim(self):
        return self._input_dim

    @property
    def packed_dim(self):
        return self._packed_dim

    @property
    def packed_factor(self):
        return self._packed_factor

    @property
    def marlin_tile_size(self):
        return self._marlin_tile_size

    def adjust_shard_indexes_for_packing(self, shard_size: int, shard_offset: int) -> tuple[int, int]:
        """Sizes in logical elements -> sizes in stored words (parameter.py:616-650)."""
        if self._packed_factor is None:
            return shard_size, shard_offset
        size, offset = shard_size // self._packed_factor, shard_offset // self._packed_factor
        if self._marlin_tile_size is not None:
            size, offset = size * self._marlin_tile_size, offset * self._marlin_tile_size
        return int(size), int(offset)

    def _shard_id_as_int(self, shard_id: str | int) -> int:
        return shard_id if isinstance(shard_id, int) else _QKV_INDEX[shard_id]


class _ColumnvLLMParameter(BasevLLMParameter):
    def __init__(self, output_dim: int, **kwargs):
        super().__init__(output_dim=output_dim, **kwargs)


class RowvLLMParameter(BasevLLMParameter):
    def __init__(self, input_dim: int, **kwargs):
        super().__init__(input_dim=input_dim, **kwargs)


class ModelWeightParameter(BasevLLMParameter):
    """A weight matrix: has both an input and an output dimension."""

    def __init__(self, input_dim: int, output_dim: int, **kwargs):
        super().__init__(input_dim=input_dim, output_dim=output_dim, **kwargs)


class GroupQuantScaleParameter(ModelWeightParameter):
    """Scales / zero points of group quantisation: [groups along the input dimension, output channels]."""


class ChannelQuantScaleParameter(_ColumnvLLMParameter):
    """One scale per output channel."""


class PackedColumnParameter(_ColumnvLLMParameter):
    def __init__(self, packed_factor: int | Fraction, packed_dim: int, marlin_tile_size: int | None = None, **kwargs):
        super().__init__(packed_factor=packed_factor, packed_dim=packed_dim, marlin_tile_size=marlin_tile_size, **kwargs)


class PackedvLLMParameter(ModelWeightParameter):
    """A weight matrix with several codes per stored word along ``packed_dim`` (GPTQ: the input dimension, AWQ: the
    output dimension)."""

    def __init__(self, packed_factor: int | Fraction, packed_dim: int, marlin_tile_size: int | None = None, **kwargs):
        super().__init__(packed_factor=packed_factor, packed_dim=packed_dim, marlin_tile_size=marlin_tile_size, **kwargs)


class PerTensorScaleParameter(BasevLLMParameter):
    """One scale per LOGICAL matrix of a fused layer (three for q/k/v): a checkpoint scalar goes to the entry of its
    shard; the quantization method merges the entries after loading (parameter.py:260-310)."""

    def _load_into_shard_id(self, loaded_weight: torch.Tensor, shard_id: str | int = 0, **_kwargs) -> None:
        if loaded_weight.ndim != 0:
            if loaded_weight.shape[0] != 1:
                raise ValueError(f"per-tensor scale of shape {tuple(loaded_weight.shape)}")
            loaded_weight = loaded_weight[0]
        self._copy(self.data[self._shard_id_as_int(shard_id)], loaded_weight)

    def load_merged_column_weight(self, loaded_weight: torch.Tensor, **kwargs) -> None:
        self._load_into_shard_id(loaded_weight, **kwargs)

    def load_qkv_weight(self, loaded_weight: torch.Tensor, **kwargs) -> None:
        self._load_into_shard_id(loaded_weight, **kwargs)
