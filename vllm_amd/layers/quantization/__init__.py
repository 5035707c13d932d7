"""Quantization method registry, same hooks as the reference's
``vllm/model_executor/layers/quantization/__init__.py`` (register_quantization_config :45-84,
get_quantization_config :87-159) restricted to the methods this build implements."""
from __future__ import annotations

from .base_config import QuantizationConfig

QUANTIZATION_METHODS: list[str] = ["gptq_marlin", "awq_marlin", "fp8", "ptpc_fp8"]
_CUSTOMIZED_METHOD_TO_QUANT_CONFIG: dict[str, type[QuantizationConfig]] = {}


def register_quantization_config(quantization: str):
    """Decorator registering an out-of-tree QuantizationConfig under ``quantization``."""

    def _wrapper(quant_config_cls):
        if quantization in QUANTIZATION_METHODS and quantization not in _CUSTOMIZED_METHOD_TO_QUANT_CONFIG:
            raise ValueError(f"The quantization method `{quantization}` is already exists.")
        if not issubclass(quant_config_cls, QuantizationConfig):
            raise ValueError("The quantization config must be a subclass of `QuantizationConfig`.")
        _CUSTOMIZED_METHOD_TO_QUANT_CONFIG[quantization] = quant_config_cls
        if quantization not in QUANTIZATION_METHODS:
            QUANTIZATION_METHODS.append(quantization)
        return quant_config_cls

    return _wrapper


def get_quantization_config(quantization: str) -> type[QuantizationConfig]:
    if quantization not in QUANTIZATION_METHODS:
        raise ValueError(f"Invalid quantization method: {quantization}")
    from .awq_marlin import AWQMarlinConfig
    from .fp8 import Fp8Config, PTPCFp8Config
    from .gptq_marlin import GPTQMarlinConfig

    method_to_config: dict[str, type[QuantizationConfig]] = {
        "gptq_marlin": GPTQMarlinConfig,
        "awq_marlin": AWQMarlinConfig,
        "fp8": Fp8Config,
        "ptpc_fp8": PTPCFp8Config,
    }
    method_to_config.update(_CUSTOMIZED_METHOD_TO_QUANT_CONFIG)
    return method_to_config[quantization]


__all__ = ["QuantizationConfig", "QUANTIZATION_METHODS", "get_quantization_config", "register_quantization_config"]
