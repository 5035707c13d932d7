"""FP8 activation quantisation op, same call contract as the reference's ``QuantFP8``
(vllm/model_executor/layers/quantization/input_quant_fp8.py:22-97, ``forward_cuda``).  Only the device path exists:
``forward_native`` in the reference multiplies by a reciprocal and is not bit-identical to the kernel."""
from __future__ import annotations

from typing import NamedTuple

import torch

from vllm_amd import _custom_ops as ops


class GroupShape(NamedTuple):
    """(rows, cols) covered by one scale; -1 means the full extent (quant_utils.py:33-60)."""
    row: int
    col: int

    def is_per_tensor(self) -> bool:
        return self.row == -1 and self.col == -1

    def is_per_token(self) -> bool:
        return self.row == 1 and self.col == -1


GroupShape.PER_TENSOR = GroupShape(-1, -1)
GroupShape.PER_TOKEN = GroupShape(1, -1)


class QuantFP8(torch.nn.Module):
    def __init__(self, static: bool, group_shape: GroupShape, num_token_padding: int | None = None):
        super().__init__()
        self.static = static
        self.group_shape = group_shape
        self.num_token_padding = num_token_padding
        assert group_shape in (GroupShape.PER_TOKEN, GroupShape.PER_TENSOR), "block-wise FP8 is not built"
        assert not static or group_shape == GroupShape.PER_TENSOR, "Only per-tensor scales supported for static quantization."
        self.use_per_token_if_dynamic = group_shape == GroupShape.PER_TOKEN

    def forward(self, x: torch.Tensor, scale: torch.Tensor | None = None,
                scale_ub: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
        assert (scale is not None) == self.static
        assert scale_ub is None or (not self.static and self.group_shape == GroupShape.PER_TOKEN
                                    and scale_ub.numel() == 1)
        return ops.scaled_fp8_quant(x, scale, num_token_padding=self.num_token_padding, scale_ub=scale_ub,
                                    use_per_token_if_dynamic=self.use_per_token_if_dynamic)

    forward_cuda = forward
    forward_hip = forward
