"""MI355X-native quantized-linear backend (GPTQ W4A16 + FP8 W8A8) behind vLLM's custom-op and plugin surface.

The compute path is a hand-written HIP library for gfx950 (``libvllm_amd_qlinear.so``, plain C ABI, see
``include/vllm_amd_qlinear.h``) reached through ``vllm_amd._custom_ops``.  There is no CPU or eager fallback: an
op called without the library, or on a non-GPU tensor, raises.
"""
__version__ = "0.1.0"
