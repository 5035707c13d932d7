"""ctypes binding of ``libvllm_amd_qlinear.so`` (the C ABI in ``include/vllm_amd_qlinear.h``).

Loading is lazy and loud: if the shared object is missing the first op call raises ``RuntimeError`` -- there is no
fallback implementation.  Build it with ``python -m vllm_amd.build``.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_int, c_int64, c_size_t, c_void_p, POINTER
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libvllm_amd_qlinear.so"

VAQ_OK = 0
VAQ_ERR_INVALID_ARG = -1
VAQ_ERR_UNSUPPORTED = -2
VAQ_ERR_LAUNCH = -3

VAQ_F16, VAQ_BF16, VAQ_F32 = 0, 1, 2
VAQ_LAYOUT_MARLIN, VAQ_LAYOUT_NATIVE, VAQ_LAYOUT_NATIVE_BYTES = 0, 1, 2
VAQ_WTYPE_U4B8, VAQ_WTYPE_U4, VAQ_WTYPE_U8B128, VAQ_WTYPE_FE4M3 = 0, 1, 2, 3

# name -> (restype, argtypes); must list every symbol the header declares (tests check this against the header)
_SIGNATURES = {
    "vaq_last_error": (c_char_p, []),
    "vaq_abi_version": (c_int, []),
    "vaq_num_cus": (c_int, [c_int]),
    "vaq_w4a16_repack": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_int, c_void_p]),
    "vaq_w4a16_repack_awq": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int, c_int, c_void_p]),
    "vaq_w4a16_gemm_workspace": (c_int, [c_int64, c_int64, c_int64, c_int, c_int, POINTER(c_size_t), POINTER(c_size_t),
                                         POINTER(c_size_t)]),
    "vaq_w4a16_gemm": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_int64, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_int,
                               c_int, c_void_p]),
    "vaq_w4a16_gemm_static": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_int64, c_int64, c_int64, c_int, c_int, c_int, c_void_p]),
    "vaq_permute_cols": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_void_p]),
    "vaq_fp8_quant_per_token": (c_int, [c_void_p, c_int, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_int64,
                                        c_int64, c_void_p]),
    "vaq_fp8_quant_static": (c_int, [c_void_p, c_int, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p]),
    "vaq_fp8_quant_dynamic": (c_int, [c_void_p, c_int, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64,
                                      c_void_p]),
    "vaq_fp8_scaled_mm": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p,
                                  c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_void_p]),
    "vaq_rms_norm_dynamic_per_token_fp8_quant": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p,
                                                         ctypes.c_float, c_void_p, c_int, c_int64, c_int64, c_void_p]),
    "vaq_rms_norm_static_fp8_quant": (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, ctypes.c_float, c_void_p,
                                              c_int, c_int64, c_int64, c_void_p]),
    "vaq_silu_and_mul_fp8_quant": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p]),
    "vaq_fp8_scaled_mm_workspace": (c_int, [c_int64, c_int64, c_int64, ctypes.POINTER(ctypes.c_size_t),
                                            ctypes.POINTER(ctypes.c_size_t)]),
    "vaq_fp8_scaled_mm_ws": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p,
                                     c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p,
                                     c_int64, c_void_p]),
}
class VaqTuning(ctypes.Structure):
    """``VaqTuning`` of the header: kernel-variant overrides for ONE call (tests, benchmarks); all zero = automatic."""
    _fields_ = [(n, c_int) for n in (
        "decode_impl", "decode2_gs", "decode2_wks", "decode2_wn", "decode_tg", "decode_wk", "decode_gx", "decode_depth",
        "prefill_tile", "prefill_split", "fp8_path", "fp8_tile_impl", "fp8_tile_cfg", "fp8_split", "fp8_gx",
        "fp8_stream_split", "quant_wg_per_row")] + [("exp", c_int * 15)]


_TUNING_P = POINTER(VaqTuning)
for _name in ("vaq_w4a16_gemm_workspace", "vaq_w4a16_gemm", "vaq_fp8_scaled_mm_workspace", "vaq_fp8_scaled_mm_ws",
              "vaq_fp8_quant_per_token"):
    _res, _args = _SIGNATURES[_name]
    _SIGNATURES[_name + "_tuned"] = (_res, [*_args, _TUNING_P])

_lib = None


def exported_symbols() -> list[str]:
    return sorted(_SIGNATURES)


def load() -> ctypes.CDLL:
    """Return the loaded library, loading it on first use.  Raises RuntimeError if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: the gfx950 kernels are not built (run `python -m vllm_amd.build`). "
            "vllm_amd has no fallback path.")
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (res, args) in _SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            raise RuntimeError(f"{LIB_PATH} does not export {name}; rebuild it") from None
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(status: int) -> None:
    """Translate a C-ABI status into the exception the reference would raise for the same condition."""
    if status == VAQ_OK:
        return
    msg = load().vaq_last_error().decode("utf-8", "replace")
    if status == VAQ_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)
