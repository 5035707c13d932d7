"""Kernel selection, same contract as the reference's ``kernels/mixed_precision/__init__.py``
(``_POSSIBLE_KERNELS`` :36-45, ``choose_mp_linear_kernel`` :48-100): first kernel in priority order whose
``can_implement`` accepts the layer and that is not named in ``VLLM_DISABLED_KERNELS``."""
from __future__ import annotations

import os

from .hip_w4a16 import HipW4A16LinearKernel
from .MPLinearKernel import MPLinearKernel, MPLinearLayerConfig

_POSSIBLE_KERNELS: list[type[MPLinearKernel]] = [HipW4A16LinearKernel]


def choose_mp_linear_kernel(config: MPLinearLayerConfig, compute_capability: int | None = None) -> type[MPLinearKernel]:
    disabled = [k for k in os.environ.get("VLLM_DISABLED_KERNELS", "").split(",") if k]
    failure_reasons = []
    for kernel in _POSSIBLE_KERNELS:
        if kernel.__name__ in disabled:
            failure_reasons.append(f" {kernel.__name__} disabled by environment variable")
            continue
        if compute_capability is not None and kernel.get_min_capability() > compute_capability:
            failure_reasons.append(f"{kernel.__name__} requires capability {kernel.get_min_capability()}, current "
                                   f"compute capability is {compute_capability}")
            continue
        can_implement, failure_reason = kernel.can_implement(config)
        if can_implement:
            return kernel
        failure_reasons.append(f" {kernel.__name__} cannot implement due to: {failure_reason}")
    raise ValueError("Failed to find a kernel that can implement the WNA16 linear layer. Reasons: \n" +
                     "\n".join(failure_reasons))


__all__ = ["MPLinearKernel", "MPLinearLayerConfig", "HipW4A16LinearKernel", "choose_mp_linear_kernel"]
