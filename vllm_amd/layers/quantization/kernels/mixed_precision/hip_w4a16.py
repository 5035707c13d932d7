"""The gfx950 W4A16 kernel as an ``MPLinearKernel`` -- the counterpart of the reference's ``MarlinLinearKernel``
(kernels/mixed_precision/marlin.py:28-166), with the CUDA-only gate removed: same parameter names, same
``process_weights_after_loading`` / ``apply_weights`` flow, the repack and GEMM done by the HIP library."""
from __future__ import annotations

import torch

from vllm_amd import _custom_ops as ops
from ...utils.marlin_utils import (HIP_W4A16_SUPPORTED_GROUP_SIZES, HIP_W8A16_SUPPORTED_GROUP_SIZES,
                                   apply_gptq_marlin_linear,
                                   check_marlin_supports_shape, marlin_is_k_full, marlin_make_empty_g_idx,
                                   marlin_make_workspace_new, marlin_permute_bias, marlin_permute_scales,
                                   marlin_sort_g_idx, marlin_zero_points, query_marlin_supported_quant_types)
from ...utils.quant_utils import unpack_cols
from .MPLinearKernel import MPLinearKernel, MPLinearLayerConfig


class HipW4A16LinearKernel(MPLinearKernel):
    @classmethod
    def get_min_capability(cls) -> int:
        return 95   # gfx950

    @classmethod
    def can_implement(cls, c: MPLinearLayerConfig) -> tuple[bool, str | None]:
        quant_types = query_marlin_supported_quant_types(c.zero_points)
        if c.weight_type not in quant_types:
            return False, (f"Quant type ({c.weight_type}) not supported by the gfx950 W4A16 kernel, supported types "
                           f"are: {quant_types}")
        if c.group_size not in (HIP_W8A16_SUPPORTED_GROUP_SIZES if c.weight_type.size_bits == 8
                                else HIP_W4A16_SUPPORTED_GROUP_SIZES):
            return False, (f"Group size ({c.group_size}) not supported by the gfx950 W4A16 kernel, supported group "
                           f"sizes are: {HIP_W4A16_SUPPORTED_GROUP_SIZES}")
        if c.act_type not in (torch.float16, torch.bfloat16):
            return False, f"Activation type {c.act_type} not supported (float16 / bfloat16)"
        if c.has_g_idx and c.partition_weight_shape[0] != c.full_weight_shape[0]:
            return False, "act_order with a row-parallel shard (is_k_full = False) is not built"
        return check_marlin_supports_shape(c.partition_weight_shape[1], c.partition_weight_shape[0],
                                           c.full_weight_shape[0], c.group_size)

    # `weight_packed` is {input_dim = 0, output_dim = 1, packed_dim = 0}; `weight_scale` is {input_dim = 0, output_dim = 1}
    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        device = getattr(layer, self.w_q_name).device
        c = self.config
        size_k, size_n = c.partition_weight_shape

        row_parallel = c.partition_weight_shape[0] != c.full_weight_shape[0]
        self.is_k_full = marlin_is_k_full(c.has_g_idx, row_parallel)
        self.workspace = marlin_make_workspace_new(device, size_n=size_n)

        if self.w_gidx_name is None:
            self.w_gidx_name = "g_idx"
        if self.w_zp_name is None:
            self.w_zp_name = "w_zp"

        # act_order whose g_idx moves whole groups (every run of `group_size` consecutive rows carries one group id, each
        # id once) needs no row permutation at all: the rows are already grouped, only group j's scales / zero points
        # sit in row g_idx[j * group_size].  Gather those rows once here and run the layer as if it had no act_order:
        # same weights, no activation reorder on any call.
        group_ids = None
        if c.has_g_idx and c.group_size > 0 and size_k % c.group_size == 0:
            g_idx_full = getattr(layer, self.w_gidx_name).data
            blocks = g_idx_full.reshape(size_k // c.group_size, c.group_size)
            first = blocks[:, 0]
            if bool((blocks == first[:, None]).all()) and first.numel() == getattr(layer, self.w_s_name).shape[0] and \
                    bool((torch.bincount(first.long(), minlength=first.numel()) == 1).all()):
                group_ids = first.long()
        self.act_order_folded = group_ids is not None

        if group_ids is not None:
            getattr(layer, self.w_s_name).data = getattr(layer, self.w_s_name).data[group_ids].contiguous()
            if c.zero_points:
                getattr(layer, self.w_zp_name).data = getattr(layer, self.w_zp_name).data[group_ids].contiguous()
            setattr(layer, self.w_gidx_name, marlin_make_empty_g_idx(device))
            layer.g_idx_sort_indices = marlin_make_empty_g_idx(device)
        elif c.has_g_idx:
            g_idx, g_idx_sort_indices = marlin_sort_g_idx(getattr(layer, self.w_gidx_name))
            # The kernels take the group of sorted row r to be r // group_size (the reference's kernel looks g_idx up
            # per row instead): every group id must label exactly group_size rows.
            group_len = c.group_size if c.group_size > 0 else size_k
            expect = torch.arange(size_k, device=g_idx.device, dtype=g_idx.dtype) // group_len
            if g_idx.numel() != size_k or not bool((g_idx == expect).all()):
                raise NotImplementedError("act_order: g_idx must assign exactly group_size rows to each group 0 .. K / "
                                          "group_size - 1; uneven groups are not built for gfx950")
            self._transform_param(layer, self.w_gidx_name, lambda _: g_idx)
            layer.g_idx_sort_indices = g_idx_sort_indices
        else:
            setattr(layer, self.w_gidx_name, marlin_make_empty_g_idx(device))
            layer.g_idx_sort_indices = marlin_make_empty_g_idx(device)

        if c.zero_points:
            grouped_k = size_k // c.group_size if c.group_size != -1 else 1
            # checkpoint layout of `qzeros` is [groups, N/8] packed along N (GPTQ) -- values are used as stored
            self._transform_param(
                layer, self.w_zp_name,
                lambda x: marlin_zero_points(unpack_cols(x.data.contiguous(), c.weight_type.size_bits, grouped_k, size_n),
                                             size_k=grouped_k, size_n=size_n, num_bits=c.weight_type.size_bits))
        else:
            setattr(layer, self.w_zp_name, marlin_make_empty_g_idx(device))

        def transform_w_q(x):
            x.data = ops.gptq_marlin_repack(x.data.contiguous(), perm=layer.g_idx_sort_indices, size_k=size_k,
                                            size_n=size_n, num_bits=c.weight_type.size_bits)
            return x

        def transform_w_s(x):
            x.data = marlin_permute_scales(x.data.contiguous(), size_k=size_k, size_n=size_n, group_size=c.group_size)
            return x

        self._transform_param(layer, self.w_q_name, transform_w_q)
        self._transform_param(layer, self.w_s_name, transform_w_s)

        if hasattr(layer, "bias") and layer.bias is not None:
            layer.bias.data = marlin_permute_bias(layer.bias)

    def apply_weights(self, layer: torch.nn.Module, x: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
        c = self.config
        w_q, w_s, w_zp, w_gidx = self._get_weight_params(layer)
        return apply_gptq_marlin_linear(input=x, weight=w_q, weight_scale=w_s, weight_zp=w_zp, g_idx=w_gidx,
                                        g_idx_sort_indices=layer.g_idx_sort_indices, workspace=self.workspace,
                                        wtype=c.weight_type, input_size_per_partition=c.partition_weight_shape[0],
                                        output_size_per_partition=c.partition_weight_shape[1],
                                        is_k_full=self.is_k_full, bias=bias)
