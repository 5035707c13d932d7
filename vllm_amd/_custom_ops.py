"""Python op surface of the quantized-linear path, same names and call signatures as the reference's
``vllm/_custom_ops.py`` (gptq_marlin_repack :1134-1141, gptq_marlin_gemm :1193-1232, scaled_fp8_quant :1456-1513,
cutlass_scaled_mm :754-802, permute_cols), registered as PyTorch custom ops in the ``vllm_amd`` namespace with the
schemas of ``csrc/torch_bindings.cpp`` (:304, :309-321, :412-414, :572-589) and fake (meta) implementations, and
implemented by the gfx950 library through its C ABI.

Argument validation repeats the reference's host checks (gptq_marlin.cu:689-902, gptq_marlin_repack.cu:255-280,
scaled_mm_entry.cu:179-193, common.cu:217-220) and raises ``RuntimeError`` / ``NotImplementedError`` where the
reference raises through ``TORCH_CHECK`` / ``TORCH_CHECK_NOT_IMPLEMENTED``.  There is no fallback: tensors that are
not on a GPU are rejected.
"""
from __future__ import annotations

import contextlib
import ctypes

import torch

from . import _lib, _tuning
from .scalar_type import ScalarType, scalar_types

FP8_DTYPE = torch.float8_e4m3fn        # gfx950 is an OCP part (reference: vllm/platforms/rocm.py:447-452)
GPTQ_MARLIN_TILE = 16
GPTQ_MARLIN_MIN_THREAD_N = 64
GPTQ_MARLIN_MIN_THREAD_K = 128

_LAYOUTS = {"marlin": _lib.VAQ_LAYOUT_MARLIN, "native": _lib.VAQ_LAYOUT_NATIVE, "native_bytes": _lib.VAQ_LAYOUT_NATIVE_BYTES}


def _check(cond: bool, msg) -> None:
    """``msg`` is a string, or a callable that builds one: formatted messages cost more than the test they belong to, so
    they are only built on failure."""
    if not cond:
        raise RuntimeError(msg() if callable(msg) else msg)


def _ptr(t: torch.Tensor | None):
    """Address of a tensor's first element for a ``void*`` parameter (a plain int: the declared argument types convert
    it, and building a ``c_void_p`` object per pointer cost more than the conversion)."""
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device: torch.device):
    """The hipStream_t that torch currently launches on for ``device``."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def _dtype_tag(dt: torch.dtype) -> int:
    if dt == torch.float16:
        return _lib.VAQ_F16
    if dt == torch.bfloat16:
        return _lib.VAQ_BF16
    if dt == torch.float32:
        return _lib.VAQ_F32
    raise RuntimeError(f"unsupported dtype {dt}")


def _is_gpu(t: torch.Tensor) -> bool:
    return t.device.type == "cuda"


_NO_GUARD = contextlib.nullcontext()


def _on(device: torch.device):
    """Context in which ``device`` is the current one for the library call.  Nothing is switched, and nothing is paid,
    when it already is (the usual case: ``torch.cuda.device`` costs 3-4 us of host time per call either way)."""
    idx = device.index
    if idx is None or idx == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(idx)


# ============================================================================ repack

def _check_repack_args(b_q_weight, perm, size_k, size_n, num_bits) -> None:
    """Host checks of gptq_marlin_repack.cu:255-280, same order."""
    _check(size_k % GPTQ_MARLIN_TILE == 0, lambda: f"size_k = {size_k} is not divisible by tile_k_size = {GPTQ_MARLIN_TILE}")
    _check(size_n % GPTQ_MARLIN_MIN_THREAD_N == 0,
           lambda: f"size_n = {size_n} is not divisible by tile_n_size = {GPTQ_MARLIN_MIN_THREAD_N}")
    _check(num_bits in (4, 8), lambda: f"num_bits must be 4 or 8. Got = {num_bits}")
    pack_factor = 32 // num_bits
    _check(b_q_weight.dim() == 2 and size_k // pack_factor == b_q_weight.size(0),
           lambda: f"Shape mismatch: b_q_weight.size(0) = {b_q_weight.size(0) if b_q_weight.dim() else None}, "
           f"size_k = {size_k}, pack_factor = {pack_factor}")
    _check(b_q_weight.size(1) == size_n, lambda: f"b_q_weight.size(1) = {b_q_weight.size(1)} is not size_n = {size_n}")
    _check(_is_gpu(b_q_weight), "b_q_weight is not on GPU")
    _check(b_q_weight.is_contiguous(), "b_q_weight is not contiguous")
    _check(b_q_weight.dtype == torch.int32, "b_q_weight type is not kInt")
    _check(_is_gpu(perm), "perm is not on GPU")
    _check(perm.is_contiguous(), "perm is not contiguous")
    _check(perm.dtype == torch.int32, "perm type is not at::kInt")
    _check(perm.numel() in (0, size_k), lambda: f"perm.numel() = {perm.numel()} must be 0 or size_k = {size_k}")


def _repack_impl(b_q_weight: torch.Tensor, perm: torch.Tensor, size_k: int, size_n: int, num_bits: int,
                 layout: int = _lib.VAQ_LAYOUT_NATIVE) -> torch.Tensor:
    _check_repack_args(b_q_weight, perm, size_k, size_n, num_bits)
    lib = _lib.load()
    pack_factor = 32 // num_bits
    with _on(b_q_weight.device):
        out = torch.empty((size_k // GPTQ_MARLIN_TILE, size_n * GPTQ_MARLIN_TILE // pack_factor),
                          dtype=torch.int32, device=b_q_weight.device)
        _lib.check(lib.vaq_w4a16_repack(_ptr(b_q_weight), _ptr(perm) if perm.numel() else None, _ptr(out), size_k,
                                        size_n, num_bits, layout, _stream(b_q_weight.device)))
    return out


def _repack_fake(b_q_weight, perm, size_k, size_n, num_bits, layout=1):
    pack_factor = 32 // num_bits
    return torch.empty((size_k // GPTQ_MARLIN_TILE, size_n * GPTQ_MARLIN_TILE // pack_factor),
                       dtype=b_q_weight.dtype, device=b_q_weight.device)


def _check_awq_repack_args(b_q_weight: torch.Tensor, size_k: int, size_n: int, num_bits: int) -> None:
    """Host checks of awq_marlin_repack.cu:208-232 in the same order."""
    _check(size_k % GPTQ_MARLIN_TILE == 0, lambda: f"size_k = {size_k} is not divisible by tile_k_size = {GPTQ_MARLIN_TILE}")
    _check(size_n % GPTQ_MARLIN_MIN_THREAD_N == 0,
           lambda: f"size_n = {size_n} is not divisible by tile_n_size = {GPTQ_MARLIN_MIN_THREAD_N}")
    _check(num_bits in (4, 8), lambda: f"num_bits must be 4 or 8. Got = {num_bits}")
    pack_factor = 32 // num_bits
    _check(b_q_weight.dim() == 2 and b_q_weight.size(0) == size_k,
           lambda: f"b_q_weight.size(0) = {b_q_weight.size(0) if b_q_weight.dim() else None} is not size_k = {size_k}")
    _check(size_n // pack_factor == b_q_weight.size(1),
           lambda: f"Shape mismatch: b_q_weight.size(1) = {b_q_weight.size(1)}, size_n = {size_n}, pack_factor = {pack_factor}")
    _check(_is_gpu(b_q_weight), "b_q_weight is not on GPU")
    _check(b_q_weight.is_contiguous(), "b_q_weight is not contiguous")
    _check(b_q_weight.dtype == torch.int32, "b_q_weight type is not kInt")
    if num_bits != 4:
        raise NotImplementedError("awq_marlin_repack: only num_bits = 4 is built for gfx950")


def _awq_repack_impl(b_q_weight: torch.Tensor, size_k: int, size_n: int, num_bits: int,
                     layout: int = _lib.VAQ_LAYOUT_NATIVE) -> torch.Tensor:
    _check_awq_repack_args(b_q_weight, size_k, size_n, num_bits)
    lib = _lib.load()
    pack_factor = 32 // num_bits
    with _on(b_q_weight.device):
        out = torch.empty((size_k // GPTQ_MARLIN_TILE, size_n * GPTQ_MARLIN_TILE // pack_factor),
                          dtype=torch.int32, device=b_q_weight.device)
        _lib.check(lib.vaq_w4a16_repack_awq(_ptr(b_q_weight), _ptr(out), size_k, size_n, num_bits, layout,
                                            _stream(b_q_weight.device)))
    return out


def _awq_repack_fake(b_q_weight, size_k, size_n, num_bits, layout=1):
    pack_factor = 32 // num_bits
    return torch.empty((size_k // GPTQ_MARLIN_TILE, size_n * GPTQ_MARLIN_TILE // pack_factor),
                       dtype=b_q_weight.dtype, device=b_q_weight.device)


# ============================================================================ W4A16 GEMM

def _opt(t: torch.Tensor | None) -> torch.Tensor | None:
    """The reference passes 'absent' tensors as empty tensors (marlin_utils.py:261-270); presence is size(-1) > 0."""
    if t is None or t.numel() == 0:
        return None
    return t


def _check_gemm_args(a, c, b_q_weight, b_bias, b_scales, global_scale, b_zeros, g_idx, perm, workspace, b_q_type_id,
                     size_m, size_n, size_k, is_k_full, is_zp_float):
    """Host checks of gptq_marlin.cu:689-902 in the same order.  Returns (group_size, has_act_order, has_zp, wtype).
    Written as plain tests (no helper call, no message built unless a test fails): the op is called once per layer and
    decode step, and these checks were a third of its host time."""
    b_q_type = _SCALAR_TYPE_BY_ID.get(b_q_type_id)      # the named types as the objects of `scalar_types`: compared by identity below
    if b_q_type is None:
        b_q_type = ScalarType.from_id(b_q_type_id)
    bits = b_q_type.size_bits
    if bits != 4 and bits != 8:
        raise RuntimeError(f"unsupported weight type {b_q_type}")
    pack_factor = 32 // bits
    a_shape, w_shape, s_shape = a.shape, b_q_weight.shape, b_scales.shape
    if len(a_shape) != 2 or a_shape[0] != size_m:
        raise RuntimeError(f"Shape mismatch: a.size(0) = {a.size(0)}, size_m = {size_m}")
    if a_shape[1] != size_k:
        raise RuntimeError(f"Shape mismatch: a.size(1) = {a.size(1)}, size_k = {size_k}")
    if size_k % GPTQ_MARLIN_TILE != 0:
        raise RuntimeError(f"size_k = {size_k} is not divisible by tile_size = {GPTQ_MARLIN_TILE}")
    if len(w_shape) != 2 or size_k // GPTQ_MARLIN_TILE != w_shape[0]:
        raise RuntimeError(f"Shape mismatch: b_q_weight.size(0) = {b_q_weight.size(0)}, size_k = {size_k}, "
                           f"tile_size = {GPTQ_MARLIN_TILE}")
    if w_shape[1] % GPTQ_MARLIN_TILE != 0:
        raise RuntimeError(f"b_q_weight.size(1) = {b_q_weight.size(1)} is not divisible by tile_size = {GPTQ_MARLIN_TILE}")
    actual_size_n = (w_shape[1] // GPTQ_MARLIN_TILE) * pack_factor
    if size_n != actual_size_n:
        raise RuntimeError(f"size_n = {size_n}, actual_size_n = {actual_size_n}")
    if not a.is_cuda:
        raise RuntimeError("A is not on GPU")
    a_stride = a.stride()
    if a_stride[1] != 1:
        raise RuntimeError("A.stride(1) is not 1")
    if a_stride[0] % 8 != 0:
        raise RuntimeError("A.stride(0) must divisible by 8")
    if a.data_ptr() % 16 != 0:
        raise RuntimeError("A must aligned to 16 bytes")
    if not b_q_weight.is_cuda:
        raise RuntimeError("b_q_weight is not on GPU")
    if not b_q_weight.is_contiguous():
        raise RuntimeError("b_q_weight is not contiguous")
    if not b_scales.is_cuda:
        raise RuntimeError("b_scales is not on GPU")
    if not b_scales.is_contiguous():
        raise RuntimeError("b_scales is not contiguous")
    if c is not None:
        if not c.is_cuda:
            raise RuntimeError("c is not on GPU")
        if not c.is_contiguous():
            raise RuntimeError("c is not contiguous")
        if c.size(0) != size_m:
            raise RuntimeError(f"Shape mismatch: c.size(0) = {c.size(0)}, size_m = {size_m}")
        if c.size(1) != size_n:
            raise RuntimeError(f"Shape mismatch: c.size(1) = {c.size(1)}, size_n = {size_n}")
    if len(s_shape) != 2:
        raise RuntimeError(f"b_scales rank = {b_scales.dim()} is not 2")
    if s_shape[1] != size_n:
        raise RuntimeError(f"b_scales dim 1 = {b_scales.size(1)} is not size_n = {size_n}")
    num_groups = s_shape[0]

    has_act_order = False
    if g_idx is not None and perm is not None:
        if not g_idx.is_cuda:
            raise RuntimeError("g_idx is not on GPU")
        if not g_idx.is_contiguous():
            raise RuntimeError("g_idx is not contiguous")
        if not perm.is_cuda:
            raise RuntimeError("perm is not on GPU")
        if not perm.is_contiguous():
            raise RuntimeError("perm is not contiguous")
        n_g, n_p = g_idx.size(-1), perm.size(-1)
        if not ((n_g == 0 and n_p == 0) or (n_g == size_k and n_p == size_k)):
            raise RuntimeError(f"Unexpected g_idx.size(-1) = {n_g} and perm.size(-1) = {n_p}, where size_k = {size_k}")
        has_act_order = n_g > 0 and n_p > 0
    if has_act_order:
        if is_k_full:
            if num_groups <= 1:
                raise RuntimeError("For act_order, num_groups must be > 1")
            if size_k % num_groups != 0:
                raise RuntimeError(f"size_k = {size_k}, is not divisible by num_groups = {num_groups}")
            group_size = size_k // num_groups
        else:
            group_size = 0
    elif num_groups > 1:
        if size_k % num_groups != 0:
            raise RuntimeError(f"size_k = {size_k}, is not divisible by b_scales.size(0) = {b_scales.size(0)}")
        group_size = size_k // num_groups
    else:
        group_size = -1

    if global_scale is not None:
        raise RuntimeError("global_scale can only be used for nvfp4 format.")
    if b_bias is not None:
        if not b_bias.is_cuda:
            raise RuntimeError("b_bias is not on GPU")
        if not b_bias.is_contiguous():
            raise RuntimeError("b_bias is not contiguous")
        if b_bias.size(0) != size_n:
            raise RuntimeError("b_bias.size(0) != size_n")
        if b_bias.stride(0) != 1:
            raise RuntimeError("b_bias.stride(0) != 1")
    has_zp = b_zeros is not None and b_zeros.size(-1) > 0
    if b_zeros is not None:
        if not b_zeros.is_cuda:
            raise RuntimeError("b_zeros is not on GPU")
        if not b_zeros.is_contiguous():
            raise RuntimeError("b_zeros is not contiguous")
    if has_zp:
        if b_q_type is not scalar_types.uint4 and b_q_type is not scalar_types.uint8:
            raise RuntimeError(f"b_q_type must be u4 or u8 when has_zp = True. Got = {b_q_type}")
    elif (b_q_type is not scalar_types.uint4b8 and b_q_type is not scalar_types.uint8b128
          and b_q_type is not scalar_types.float8_e4m3fn):
        raise RuntimeError("b_q_type must be uint4b8, uint8b128, float8_e4m3fn or float4_e2m1f when has_zp = False. "
                           f"Got = {b_q_type}")
    if has_zp and is_zp_float and a.dtype != torch.float16:
        raise RuntimeError("Computation type must be float16 (half) when using float zero points.")
    if has_zp:
        z_shape = b_zeros.shape
        if len(z_shape) != 2:
            raise RuntimeError(f"b_zeros rank = {b_zeros.dim()} is not 2")
        if is_zp_float:
            if z_shape[1] != size_n:
                raise RuntimeError(f"b_zeros dim 1 = {b_zeros.size(1)} is not size_n = {size_n}")
            if num_groups != z_shape[0]:
                raise RuntimeError(f"b_zeros dim 0 = {b_zeros.size(0)} is not num_groups = {num_groups}")
        else:
            if z_shape[0] != num_groups:
                raise RuntimeError(f"b_zeros dim 0 = {b_zeros.size(0)} is not num_groups = {num_groups}")
            if z_shape[1] != size_n // pack_factor:
                raise RuntimeError(f"b_zeros dim 1 = {b_zeros.size(1)} is not size_n / pack_factor = {size_n // pack_factor}")
    if size_n % GPTQ_MARLIN_MIN_THREAD_N != 0:
        raise RuntimeError(f"size_n = {size_n}, is not divisible by min_thread_n = {GPTQ_MARLIN_MIN_THREAD_N}")
    if not workspace.is_cuda or workspace.dtype != torch.int32:
        raise RuntimeError("workspace must be an int32 tensor on GPU")
    a_dtype = a.dtype
    if a_dtype != torch.float16 and a_dtype != torch.bfloat16:
        raise RuntimeError("gpt_marlin_gemm only supports bfloat16 and float16")
    if b_scales.dtype != a_dtype:
        raise RuntimeError(f"b_scales dtype {b_scales.dtype} must equal the activation dtype {a.dtype}")

    # what this build implements out of everything the reference accepts
    if (b_q_type is not scalar_types.uint4b8 and b_q_type is not scalar_types.uint4 and b_q_type is not scalar_types.uint8b128
            and b_q_type is not scalar_types.float8_e4m3fn):
        raise NotImplementedError(f"gptq_marlin_gemm: weight type {b_q_type} is not built for gfx950 "
                                  "(uint4b8 / uint4 / uint8b128 / float8_e4m3fn)")
    if is_zp_float:
        raise NotImplementedError("gptq_marlin_gemm: float zero points (is_zp_float) are not built for gfx950")
    if has_act_order and not is_k_full:
        raise NotImplementedError("gptq_marlin_gemm: is_k_full = False (act_order x row-parallel shard) is not built; "
                                  "one-GPU layers always have is_k_full = True")
    if group_size not in (-1, 32, 64, 128):
        if group_size == size_k:
            group_size = -1       # one group spanning all of K is channelwise
        else:
            raise NotImplementedError(f"gptq_marlin_gemm: group_size = {group_size} is not built for gfx950 "
                                      "(only -1, 32, 64, 128)")
    if size_k % GPTQ_MARLIN_MIN_THREAD_K != 0:
        raise RuntimeError(f"size_k = {size_k}, is not divisible by min_thread_k = {GPTQ_MARLIN_MIN_THREAD_K}")
    if b_q_type is scalar_types.float8_e4m3fn:
        # weight-only FP8 (marlin_utils_fp8.py): channelwise scales or groups of 128 rows, no act_order
        if group_size not in (-1, 128) or has_act_order:
            raise NotImplementedError("gptq_marlin_gemm: float8_e4m3fn weights take group_size -1 or 128 and no act_order")
        wtype = _lib.VAQ_WTYPE_FE4M3
    elif b_q_type is scalar_types.uint8b128:
        wtype = _lib.VAQ_WTYPE_U8B128
    else:
        wtype = _lib.VAQ_WTYPE_U4 if has_zp else _lib.VAQ_WTYPE_U4B8
    return group_size, has_act_order, has_zp, wtype


_SCALAR_TYPE_BY_ID: dict[int, ScalarType] = {
    t.id: t for t in (scalar_types.uint4, scalar_types.uint4b8, scalar_types.uint8, scalar_types.uint8b128,
                      scalar_types.float8_e4m3fn)}


def _gemm_impl(a: torch.Tensor, c_or_none: torch.Tensor | None, b_q_weight: torch.Tensor,
               b_bias_or_none: torch.Tensor | None, b_scales: torch.Tensor, global_scale: torch.Tensor | None,
               b_zeros_or_none: torch.Tensor | None, g_idx_or_none: torch.Tensor | None,
               perm_or_none: torch.Tensor | None, workspace: torch.Tensor, b_q_type: int, size_m: int, size_n: int,
               size_k: int, is_k_full: bool = True, use_atomic_add: bool = False, use_fp32_reduce: bool = False,
               is_zp_float: bool = False) -> torch.Tensor:
    # use_atomic_add / use_fp32_reduce select Marlin reduction variants; this build always reduces in fp32.
    group_size, has_act_order, has_zp, wtype = _check_gemm_args(
        a, c_or_none, b_q_weight, b_bias_or_none, b_scales, global_scale, b_zeros_or_none, g_idx_or_none, perm_or_none,
        workspace, b_q_type, size_m, size_n, size_k, is_k_full, is_zp_float)
    lib = _lib.load()
    dev = a.device
    with _on(dev):
        c = c_or_none if c_or_none is not None else torch.empty((size_m, size_n), dtype=a.dtype, device=dev)
        if size_m == 0:
            return c
        # Scratch for this problem: split-K partials and permuted activations from the caching allocator (safe under
        # graph capture), arrival counters from the caller's `workspace`.  The library checks what it is handed against
        # what the kernel it picks needs and reports a workspace that is too small (gptq_marlin.cu:899-902).
        tune = _tuning.current_ref()
        key = (size_m, size_n, size_k, has_act_order, dev.index or 0)
        sizes = _W4_WORKSPACE_SIZES.get(key) if tune is None else None
        if sizes is None:
            n_ctmp, n_atmp, n_cnt = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
            q_args = (size_m, size_n, size_k, int(has_act_order), dev.index or 0, ctypes.byref(n_ctmp),
                      ctypes.byref(n_atmp), ctypes.byref(n_cnt))
            _lib.check(lib.vaq_w4a16_gemm_workspace(*q_args) if tune is None
                       else lib.vaq_w4a16_gemm_workspace_tuned(*q_args, tune))
            sizes = (n_ctmp.value, n_atmp.value)
            if tune is None and len(_W4_WORKSPACE_SIZES) < 4096:
                _W4_WORKSPACE_SIZES[key] = sizes      # (the library's answer depends on the shape and the device only)
        ctmp_bytes, atmp_bytes = sizes
        c_tmp = torch.empty((ctmp_bytes // 4,), dtype=torch.float32, device=dev) if ctmp_bytes else None
        a_tmp = torch.empty((atmp_bytes // 2,), dtype=a.dtype, device=dev) if atmp_bytes else None
        g_args = (_ptr(a), a.stride(0), _ptr(b_q_weight), _ptr(b_scales), _ptr(b_zeros_or_none) if has_zp else None,
                  _ptr(perm_or_none) if has_act_order else None, _ptr(b_bias_or_none), _ptr(c), _ptr(c_tmp),
                  ctmp_bytes, _ptr(a_tmp), _ptr(workspace), workspace.numel(), size_m, size_n, size_k, group_size,
                  _dtype_tag(a.dtype), wtype, 0, _stream(dev))
        _lib.check(lib.vaq_w4a16_gemm(*g_args) if tune is None else lib.vaq_w4a16_gemm_tuned(*g_args, tune))
    return c


_W4_WORKSPACE_SIZES: dict[tuple, tuple[int, int]] = {}


def _gemm_fake(a, c_or_none, b_q_weight, b_bias_or_none, b_scales, global_scale, b_zeros_or_none, g_idx_or_none,
               perm_or_none, workspace, b_q_type, size_m, size_n, size_k, is_k_full=True, use_atomic_add=False,
               use_fp32_reduce=False, is_zp_float=False):
    return torch.empty((size_m, size_n), device=a.device, dtype=a.dtype)


# ============================================================================ permute_cols

def _permute_cols_impl(A: torch.Tensor, perm: torch.Tensor) -> torch.Tensor:
    _check(_is_gpu(A) and _is_gpu(perm), "A and perm must be on GPU")
    _check(A.dtype in (torch.float16, torch.bfloat16), "Currently only 16bit types are supported")
    _check(A.dim() == 2 and A.stride(1) == 1, "A must be a 2-D tensor with unit column stride")
    _check(perm.dtype == torch.int32 and perm.is_contiguous() and perm.numel() == A.size(1),
           "perm must be a contiguous int32 tensor of A.size(1) entries")
    _check(A.size(1) % 8 == 0, "A columns must be a multiple of 8")
    lib = _lib.load()
    with _on(A.device):
        out = torch.empty((A.size(0), A.size(1)), dtype=A.dtype, device=A.device)
        _lib.check(lib.vaq_permute_cols(_ptr(A), A.stride(0), _ptr(perm), _ptr(out), A.size(0), A.size(1),
                                        _stream(A.device)))
    return out


def _permute_cols_fake(A, perm):
    return torch.empty_like(A, memory_format=torch.contiguous_format)


# ============================================================================ FP8 activation quantisation

def _check_quant_io(result: torch.Tensor, input: torch.Tensor) -> tuple[int, int]:
    """common.cu:139-142 / :217-220 checks; returns (num_tokens, hidden)."""
    if not (input.is_cuda and result.is_cuda):
        raise RuntimeError("input and result must be on GPU")
    if input.dim() < 1 or input.stride(-1) != 1:
        raise RuntimeError("last dimension of input must be contiguous")
    if result.stride(-1) != 1:
        raise RuntimeError("last dimension of output must be contiguous")
    if result.dtype != FP8_DTYPE:
        raise RuntimeError(f"result must be {FP8_DTYPE}")
    dt = input.dtype
    if dt != torch.bfloat16 and dt != torch.float16 and dt != torch.float32:
        raise RuntimeError(f"unsupported input dtype {input.dtype}")
    in_shape, r_shape = input.shape, result.shape
    if len(in_shape) != 2 or len(r_shape) != 2:
        raise RuntimeError("input and result must be 2-D")
    hidden = in_shape[1]
    tokens = in_shape[0] if hidden else 0
    if r_shape[1] != hidden or r_shape[0] < tokens:
        raise RuntimeError("result shape does not cover input")
    return tokens, hidden


def _static_quant_impl(result: torch.Tensor, input: torch.Tensor, scale: torch.Tensor) -> None:
    tokens, hidden = _check_quant_io(result, input)
    _check(_is_gpu(scale) and scale.dtype == torch.float32 and scale.numel() == 1, "scale must be one fp32 on GPU")
    if tokens == 0:
        return
    lib = _lib.load()
    with _on(input.device):
        _lib.check(lib.vaq_fp8_quant_static(_ptr(input), _dtype_tag(input.dtype), input.stride(0), _ptr(result),
                                            result.stride(0), _ptr(scale), tokens, hidden, _stream(input.device)))


def _dynamic_quant_impl(result: torch.Tensor, input: torch.Tensor, scale: torch.Tensor) -> None:
    tokens, hidden = _check_quant_io(result, input)
    _check(_is_gpu(scale) and scale.dtype == torch.float32 and scale.numel() == 1, "scale must be one fp32 on GPU")
    if tokens == 0:
        return
    lib = _lib.load()
    with _on(input.device):
        _lib.check(lib.vaq_fp8_quant_dynamic(_ptr(input), _dtype_tag(input.dtype), input.stride(0), _ptr(result),
                                             result.stride(0), _ptr(scale), tokens, hidden, _stream(input.device)))


def _per_token_quant_impl(result: torch.Tensor, input: torch.Tensor, scale: torch.Tensor,
                          scale_ub: torch.Tensor | None) -> None:
    tokens, hidden = _check_quant_io(result, input)
    _check(_is_gpu(scale) and scale.dtype == torch.float32 and scale.is_contiguous() and scale.numel() >= tokens,
           "scale must be a contiguous fp32 tensor with one entry per token")
    if scale_ub is not None:
        _check(_is_gpu(scale_ub) and scale_ub.dtype == torch.float32 and scale_ub.numel() == 1,
               "scale_ub must be one fp32 on GPU")
    if tokens == 0:
        return
    lib = _lib.load()
    with _on(input.device):
        args = (_ptr(input), _dtype_tag(input.dtype), input.stride(0), _ptr(result), result.stride(0), _ptr(scale),
                _ptr(scale_ub), tokens, hidden, _stream(input.device))
        tune = _tuning.current_ref()
        _lib.check(lib.vaq_fp8_quant_per_token(*args) if tune is None else lib.vaq_fp8_quant_per_token_tuned(*args, tune))


# ============================================================================ FP8 scaled GEMM

def _check_scaled_mm_args(out, a, b, a_scales, b_scales, bias) -> None:
    """scaled_mm_entry.cu:179-193 plus the scale-shape rules of c3x/scaled_mm_helper.hpp:5-52 (plain tests, messages
    built on failure only: see ``_check_gemm_args``)."""
    a_shape, b_shape, o_shape = a.shape, b.shape, out.shape
    if len(a_shape) != 2 or len(b_shape) != 2 or len(o_shape) != 2:
        raise RuntimeError("a, b and out must be 2-D")
    m, k = a_shape
    n = b_shape[1]
    if o_shape[0] != m or k != b_shape[0] or n != o_shape[1]:
        raise RuntimeError(f"shape mismatch: a {tuple(a.shape)}, b {tuple(b.shape)}, out {tuple(out.shape)}")
    a_stride, b_stride, o_stride = a.stride(), b.stride(), out.stride()
    if a_stride[1] != 1 or o_stride[1] != 1:
        raise RuntimeError("a and out must be row-major")
    if b_stride[0] != 1:
        raise RuntimeError("b must be column-major")
    if o_stride[0] % 16 != 0 or b_stride[1] % 16 != 0:
        raise RuntimeError("out.stride(0) and b.stride(1) must be multiples of 16")
    o_dtype = out.dtype
    if bias is not None:
        if bias.numel() != n or not bias.is_contiguous() or bias.dim() != 1:
            raise RuntimeError("bias must be contiguous [N]")
        if bias.dtype != o_dtype:
            raise RuntimeError("bias dtype must equal the output dtype")
    if not (out.is_cuda and a.is_cuda and b.is_cuda and a_scales.is_cuda and b_scales.is_cuda):
        raise RuntimeError("all tensors must be on GPU")
    if a_scales.dtype != torch.float32 or b_scales.dtype != torch.float32:
        raise RuntimeError("scales must be fp32")
    if not (a_scales.is_contiguous() and b_scales.is_contiguous()):
        raise RuntimeError("scales must be contiguous")
    na, nb = a_scales.numel(), b_scales.numel()
    if na != 1 and na != m:
        raise RuntimeError(f"a_scales.numel() = {na} must be 1 or M = {m}")
    if nb != 1 and nb != n:
        raise RuntimeError(f"b_scales.numel() = {nb} must be 1 or N = {n}")
    if o_dtype != torch.float16 and o_dtype != torch.bfloat16:
        raise RuntimeError("out must be float16 or bfloat16")
    if a.dtype != FP8_DTYPE or b.dtype != FP8_DTYPE:
        raise NotImplementedError(f"cutlass_scaled_mm: only {FP8_DTYPE} x {FP8_DTYPE} is built for gfx950 "
                                  f"(got {a.dtype} x {b.dtype})")
    if a_stride[0] % 16 != 0:
        raise RuntimeError("a.stride(0) must be a multiple of 16")
    if k % 16 != 0 or n % 16 != 0:
        raise RuntimeError("K and N must be multiples of 16")


def _scaled_mm_impl(out: torch.Tensor, a: torch.Tensor, b: torch.Tensor, a_scales: torch.Tensor,
                    b_scales: torch.Tensor, bias: torch.Tensor | None) -> None:
    _check_scaled_mm_args(out, a, b, a_scales, b_scales, bias)
    if a.size(0) == 0:
        return
    lib = _lib.load()
    dev = a.device
    with _on(dev):
        # scratch for the K split of mid-sized M: partial tiles from the caching allocator (capture-safe), arrival
        # counters that are zero on entry and left zero, one array per (device, stream)
        tune = _tuning.current_ref()
        key = (a.size(0), b.size(1), a.size(1), dev.index or 0)
        sizes = _FP8_WORKSPACE_SIZES.get(key) if tune is None else None
        if sizes is None:
            n_ctmp, n_cnt = ctypes.c_size_t(), ctypes.c_size_t()
            q_args = (a.size(0), b.size(1), a.size(1), ctypes.byref(n_ctmp), ctypes.byref(n_cnt))
            _lib.check(lib.vaq_fp8_scaled_mm_workspace(*q_args) if tune is None
                       else lib.vaq_fp8_scaled_mm_workspace_tuned(*q_args, tune))
            sizes = (n_ctmp.value, n_cnt.value)
            if tune is None and len(_FP8_WORKSPACE_SIZES) < 4096:
                _FP8_WORKSPACE_SIZES[key] = sizes
        ctmp_bytes, cnt_ints = sizes
        c_tmp = counters = None
        if ctmp_bytes:
            counters = _fp8_counters(dev, cnt_ints)
            c_tmp = torch.empty((ctmp_bytes // 4,), dtype=torch.float32, device=dev)
        args = (_ptr(a), a.stride(0), _ptr(b), b.stride(1), _ptr(a_scales), a_scales.numel(), _ptr(b_scales),
                b_scales.numel(), _ptr(bias), _ptr(out), out.stride(0), _dtype_tag(out.dtype), a.size(0), b.size(1),
                a.size(1), _ptr(c_tmp), ctmp_bytes if c_tmp is not None else 0, _ptr(counters),
                counters.numel() if counters is not None else 0, _stream(dev))
        _lib.check(lib.vaq_fp8_scaled_mm_ws(*args) if tune is None else lib.vaq_fp8_scaled_mm_ws_tuned(*args, tune))


_FP8_WORKSPACE_SIZES: dict[tuple, tuple[int, int]] = {}
_FP8_COUNTERS: dict[tuple[int, int], torch.Tensor] = {}
_FP8_COUNTER_INTS = 16384


def _fp8_counters(dev: torch.device, need: int) -> torch.Tensor:
    """Zeroed int32 arrival counters for the FP8 GEMM's K split (the op has no workspace argument; the reference's
    CUTLASS path owns its workspace too).  One array per (device, stream): GEMMs on one stream run one after the other
    and each leaves the counters zero, GEMMs on different streams never share an array.  An array is created on a
    stream's first split-K call outside graph capture; a call that finds none while its stream is being captured, or
    that needs more counters than the array holds, takes a fresh zeroed one for that call alone (an allocation of the
    capture's own pool and a fill kernel, both legal inside a capture, replayed with the graph)."""
    idx = dev.index if dev.index is not None else torch.cuda.current_device()
    key = (idx, torch.cuda.current_stream(dev).cuda_stream)
    t = _FP8_COUNTERS.get(key)
    if t is not None and t.numel() >= need:
        return t
    if torch.cuda.is_current_stream_capturing() or need > _FP8_COUNTER_INTS:
        return torch.zeros(need, dtype=torch.int32, device=dev)
    t = torch.zeros(_FP8_COUNTER_INTS, dtype=torch.int32, device=dev)
    _FP8_COUNTERS[key] = t
    return t


# ============================================================================ fused RMSNorm + per-token FP8 quant

def _rms_norm_quant_impl(result: torch.Tensor, input: torch.Tensor, weight: torch.Tensor, scale: torch.Tensor,
                         epsilon: float, scale_ub: torch.Tensor | None, residual: torch.Tensor | None) -> None:
    """Host checks of fused_layernorm_dynamic_per_token_quant.cu:141-170."""
    _check(_is_gpu(input) and _is_gpu(result) and _is_gpu(weight) and _is_gpu(scale), "tensors must be on GPU")
    if result.dtype != FP8_DTYPE:
        raise NotImplementedError(f"rms_norm_dynamic_per_token_quant: only {FP8_DTYPE} output is built for gfx950 "
                                  f"(got {result.dtype})")
    _check(input.dtype in (torch.float16, torch.bfloat16), "input must be float16 or bfloat16")
    _check(weight.dtype == input.dtype, "weight.dtype must equal input.dtype")
    _check(scale.dtype == torch.float32, "scale must be float32")
    _check(result.is_contiguous() and input.stride(-1) == 1, "out must be contiguous and input row-contiguous")
    hidden = input.size(-1)
    tokens = input.numel() // hidden if hidden else 0
    _check(weight.numel() == hidden and weight.is_contiguous(), "weight must be a contiguous [hidden] tensor")
    _check(scale.numel() == tokens and scale.is_contiguous(), "scale must hold one value per token")
    if scale_ub is not None:
        _check(scale_ub.dtype == torch.float32 and scale_ub.numel() == 1 and _is_gpu(scale_ub),
               "scale_ub must be a float32 scalar on GPU")
    if residual is not None:
        _check(residual.dtype == input.dtype and residual.is_contiguous() and residual.shape == input.shape,
               "residual must match input and be contiguous")
    inp2 = input.reshape(-1, hidden) if input.dim() != 2 else input
    _check(inp2.data_ptr() == input.data_ptr(), "input must be viewable as [tokens, hidden]")
    if tokens == 0:
        return
    lib = _lib.load()
    with _on(input.device):
        _lib.check(lib.vaq_rms_norm_dynamic_per_token_fp8_quant(
            _ptr(result), _ptr(scale), _ptr(input), inp2.stride(0), _ptr(weight), _ptr(scale_ub), float(epsilon),
            _ptr(residual), _dtype_tag(input.dtype), tokens, hidden, _stream(input.device)))


def _rms_norm_static_common(who, result, input, residual, weight, scale, epsilon) -> None:
    """Host checks of layernorm_quant_kernels.cu:181-188 / 225-236."""
    _check(_is_gpu(input) and _is_gpu(result) and _is_gpu(weight) and _is_gpu(scale), "tensors must be on GPU")
    if result.dtype != FP8_DTYPE:
        raise NotImplementedError(f"{who}: only {FP8_DTYPE} output is built for gfx950 (got {result.dtype})")
    _check(input.dtype in (torch.float16, torch.bfloat16), lambda: f"{who}: input must be float16 or bfloat16")
    _check(weight.dtype == input.dtype, "weight.dtype must equal input.dtype")
    _check(scale.dtype == torch.float32 and scale.numel() == 1, "scale must be a float32 scalar")
    _check(result.is_contiguous(), "out must be contiguous")
    _check(input.stride(-1) == 1, "input rows must be contiguous")
    hidden = input.size(-1)
    tokens = input.numel() // hidden if hidden else 0
    _check(result.numel() == input.numel(), "out must have the shape of input")
    _check(weight.numel() == hidden and weight.is_contiguous(), "weight must be a contiguous [hidden] tensor")
    if residual is not None:
        _check(residual.is_contiguous(), "residual must be contiguous")
        _check(residual.dtype == input.dtype and residual.shape == input.shape, "residual must match input")
    inp2 = input.reshape(-1, hidden) if input.dim() != 2 else input
    _check(inp2.data_ptr() == input.data_ptr(), "input must be viewable as [tokens, hidden]")
    if tokens == 0:
        return
    lib = _lib.load()
    with _on(input.device):
        _lib.check(lib.vaq_rms_norm_static_fp8_quant(
            _ptr(result), _ptr(input), inp2.stride(0), _ptr(weight), _ptr(scale), float(epsilon), _ptr(residual),
            _dtype_tag(input.dtype), tokens, hidden, _stream(input.device)))


def _rms_norm_static_impl(result, input, weight, scale, epsilon) -> None:
    _rms_norm_static_common("rms_norm_static_fp8_quant", result, input, None, weight, scale, epsilon)


def _fused_add_rms_norm_static_impl(result, input, residual, weight, scale, epsilon) -> None:
    _rms_norm_static_common("fused_add_rms_norm_static_fp8_quant", result, input, residual, weight, scale, epsilon)


def _silu_and_mul_quant_impl(result: torch.Tensor, input: torch.Tensor, scale: torch.Tensor) -> None:
    """Host checks of activation_kernels.cu:560-568."""
    _check(_is_gpu(input) and _is_gpu(result) and _is_gpu(scale), "tensors must be on GPU")
    _check(result.dtype == FP8_DTYPE, lambda: f"silu_and_mul_quant: out must be {FP8_DTYPE}")
    _check(input.dtype in (torch.float16, torch.bfloat16), "silu_and_mul_quant: input must be float16 or bfloat16")
    _check(input.size(-1) % 2 == 0, "silu_and_mul_quant: the last dimension of input must be even")
    _check(scale.dtype == torch.float32 and scale.numel() == 1, "scale must be a float32 scalar")
    d = input.size(-1) // 2
    tokens = input.numel() // input.size(-1) if d else 0
    _check(input.is_contiguous() and result.is_contiguous(), "input and out must be contiguous")
    _check(result.numel() == tokens * d, "out must be [..., d] for input [..., 2*d]")
    if tokens == 0:
        return
    lib = _lib.load()
    with _on(input.device):
        _lib.check(lib.vaq_silu_and_mul_fp8_quant(_ptr(result), _ptr(input), _ptr(scale), _dtype_tag(input.dtype), tokens,
                                                  d, _stream(input.device)))


# ============================================================================ registration

_NS = "vllm_amd"
_library = torch.library.Library(_NS, "FRAGMENT")


def _register(name: str, schema: str, impl, fake=None) -> None:
    _library.define(f"{name}{schema}")
    _library.impl(name, impl, "CUDA")
    if fake is not None:
        torch.library.register_fake(f"{_NS}::{name}", fake, lib=_library)


_register("gptq_marlin_repack",
          "(Tensor b_q_weight, Tensor perm, SymInt size_k, SymInt size_n, int num_bits, int layout=1) -> Tensor",
          _repack_impl, _repack_fake)
_register("awq_marlin_repack",
          "(Tensor b_q_weight, SymInt size_k, SymInt size_n, int num_bits, int layout=1) -> Tensor",
          _awq_repack_impl, _awq_repack_fake)
_register("gptq_marlin_gemm",
          "(Tensor a, Tensor? c_or_none, Tensor b_q_weight, Tensor? b_bias_or_none, Tensor b_scales, "
          "Tensor? global_scale, Tensor? b_zeros_or_none, Tensor? g_idx_or_none, Tensor? perm_or_none, "
          "Tensor workspace, int b_q_type, SymInt size_m, SymInt size_n, SymInt size_k, bool is_k_full=True, "
          "bool use_atomic_add=False, bool use_fp32_reduce=False, bool is_zp_float=False) -> Tensor",
          _gemm_impl, _gemm_fake)
_register("permute_cols", "(Tensor A, Tensor perm) -> Tensor", _permute_cols_impl, _permute_cols_fake)
_register("static_scaled_fp8_quant", "(Tensor! result, Tensor input, Tensor scale) -> ()", _static_quant_impl,
          lambda result, input, scale: None)
_register("dynamic_scaled_fp8_quant", "(Tensor! result, Tensor input, Tensor! scale) -> ()", _dynamic_quant_impl,
          lambda result, input, scale: None)
_register("dynamic_per_token_scaled_fp8_quant", "(Tensor! result, Tensor input, Tensor! scale, Tensor? scale_ub) -> ()",
          _per_token_quant_impl, lambda result, input, scale, scale_ub: None)
_register("rms_norm_dynamic_per_token_quant",
          "(Tensor! result, Tensor input, Tensor weight, Tensor! scale, float epsilon, Tensor? scale_ub, "
          "Tensor!? residual) -> ()",
          _rms_norm_quant_impl, lambda result, input, weight, scale, epsilon, scale_ub, residual: None)
_register("rms_norm_static_fp8_quant", "(Tensor! result, Tensor input, Tensor weight, Tensor scale, float epsilon) -> ()",
          _rms_norm_static_impl, lambda result, input, weight, scale, epsilon: None)
_register("fused_add_rms_norm_static_fp8_quant",
          "(Tensor! result, Tensor input, Tensor! residual, Tensor weight, Tensor scale, float epsilon) -> ()",
          _fused_add_rms_norm_static_impl, lambda result, input, residual, weight, scale, epsilon: None)
_register("silu_and_mul_quant", "(Tensor! result, Tensor input, Tensor scale) -> ()",
          _silu_and_mul_quant_impl, lambda result, input, scale: None)
_register("cutlass_scaled_mm", "(Tensor! out, Tensor a, Tensor b, Tensor a_scales, Tensor b_scales, Tensor? bias) -> ()",
          _scaled_mm_impl, lambda out, a, b, a_scales, b_scales, bias: None)

_ops = getattr(torch.ops, _NS)


# ============================================================================ public wrappers (reference signatures)

def gptq_marlin_repack(b_q_weight: torch.Tensor, perm: torch.Tensor, size_k: int, size_n: int, num_bits: int, *,
                       layout: str = "native") -> torch.Tensor:
    """GPTQ int32[K/8, N] -> repacked int32[K/16, 2N].

    ``layout="native"`` (default) is the wavefront tile order ``gptq_marlin_gemm`` consumes; ``layout="marlin"``
    reproduces the reference's Marlin order bit-for-bit; ``layout="native_bytes"`` (``num_bits = 8`` only) keeps whole
    bytes in the native tiles, for FP8 weights (``b_q_type = float8_e4m3fn``).  Callers treat the result as opaque.
    """
    return _ops.gptq_marlin_repack(b_q_weight, perm, size_k, size_n, num_bits, _LAYOUTS[layout])


def awq_marlin_repack(b_q_weight: torch.Tensor, size_k: int, size_n: int, num_bits: int, *,
                      layout: str = "native") -> torch.Tensor:
    """AutoAWQ int32[K, N/8] -> repacked int32[K/16, 2N] (reference: _custom_ops.py:1145-1148).  Same two layouts as
    ``gptq_marlin_repack``: ``"marlin"`` is bit-exact with the reference, ``"native"`` is what the GEMM reads."""
    return _ops.awq_marlin_repack(b_q_weight, size_k, size_n, num_bits, _LAYOUTS[layout])


def gptq_marlin_gemm(a: torch.Tensor, c: torch.Tensor | None, b_q_weight: torch.Tensor, b_bias: torch.Tensor | None,
                     b_scales: torch.Tensor, global_scale: torch.Tensor | None, b_zeros: torch.Tensor | None,
                     g_idx: torch.Tensor | None, perm: torch.Tensor | None, workspace: torch.Tensor,
                     b_q_type: ScalarType, size_m: int, size_n: int, size_k: int, is_k_full: bool = True,
                     use_atomic_add: bool = False, use_fp32_reduce: bool = False,
                     is_zp_float: bool = False) -> torch.Tensor:
    return _ops.gptq_marlin_gemm(a, c, b_q_weight, b_bias, b_scales, global_scale, b_zeros, g_idx, perm, workspace,
                                 b_q_type.id, size_m, size_n, size_k, is_k_full, use_atomic_add, use_fp32_reduce,
                                 is_zp_float)


def permute_cols(a: torch.Tensor, perm: torch.Tensor) -> torch.Tensor:
    return _ops.permute_cols(a, perm)


def rms_norm_dynamic_per_token_quant(input: torch.Tensor, weight: torch.Tensor, epsilon: float, quant_dtype: torch.dtype,
                                     scale_ub: torch.Tensor | None = None,
                                     residual: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """RMSNorm (+ in-place residual add) and dynamic per-token quantisation in one pass (reference:
    _custom_ops.py:394-410).  Returns (quantised [.., hidden], scales [tokens, 1])."""
    output = torch.empty_like(input, dtype=quant_dtype)
    scales = torch.empty((input.numel() // input.shape[-1], 1), device=input.device, dtype=torch.float32)
    _ops.rms_norm_dynamic_per_token_quant(output, input, weight, scales, epsilon, scale_ub, residual)
    return output, scales


def rms_norm_static_fp8_quant(out: torch.Tensor, input: torch.Tensor, weight: torch.Tensor, scale: torch.Tensor,
                              epsilon: float) -> None:
    """``out = fp8(rms_norm(input) * weight / scale)``; the reference exposes it only as ``torch.ops._C`` op
    (csrc/torch_bindings.cpp:200-205)."""
    _ops.rms_norm_static_fp8_quant(out, input, weight, scale, epsilon)


def fused_add_rms_norm_static_fp8_quant(out: torch.Tensor, input: torch.Tensor, residual: torch.Tensor,
                                        weight: torch.Tensor, scale: torch.Tensor, epsilon: float) -> None:
    """``residual += input; out = fp8(rms_norm(residual) * weight / scale)`` (csrc/torch_bindings.cpp:208-213)."""
    _ops.fused_add_rms_norm_static_fp8_quant(out, input, residual, weight, scale, epsilon)


def silu_and_mul_quant(out: torch.Tensor, input: torch.Tensor, scale: torch.Tensor) -> None:
    """``out = fp8(silu(input[..., :d]) * input[..., d:] / scale)`` (csrc/torch_bindings.cpp:121-123)."""
    _ops.silu_and_mul_quant(out, input, scale)


def scaled_fp8_quant(input: torch.Tensor, scale: torch.Tensor | None = None, num_token_padding: int | None = None,
                     scale_ub: torch.Tensor | None = None, use_per_token_if_dynamic: bool = False,
                     output: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """Quantise ``input`` [tokens, hidden] to FP8 (e4m3fn); static if ``scale`` is given, else dynamic per tensor or,
    with ``use_per_token_if_dynamic``, per token.  Rows beyond ``input.shape[0]`` of a padded output are left
    uninitialised, as in the reference."""
    assert input.ndim == 2
    shape = tuple(input.shape)
    if num_token_padding:
        shape = (max(num_token_padding, input.shape[0]), shape[1])
    if output is None:
        output = torch.empty(shape, device=input.device, dtype=FP8_DTYPE)
    else:
        assert num_token_padding is None, "padding not supported if output passed in"
        assert output.dtype == FP8_DTYPE
    if scale is None:
        if use_per_token_if_dynamic:
            scale = torch.empty((shape[0], 1), device=input.device, dtype=torch.float32)
            _ops.dynamic_per_token_scaled_fp8_quant(output, input, scale, scale_ub)
        else:
            scale = torch.empty((1, 1), device=input.device, dtype=torch.float32)
            _ops.dynamic_scaled_fp8_quant(output, input, scale)
    else:
        assert scale.numel() == 1, f"{scale.shape}"
        _ops.static_scaled_fp8_quant(output, input, scale)
    return output, scale


def cutlass_scaled_mm(a: torch.Tensor, b: torch.Tensor, scale_a: torch.Tensor, scale_b: torch.Tensor,
                      out_dtype: torch.dtype, bias: torch.Tensor | None = None) -> torch.Tensor:
    """``(scale_a * a) @ (scale_b * b) + bias`` with fp8 ``a`` [M,K] row-major, ``b`` [K,N] column-major, fused."""
    assert out_dtype is torch.bfloat16 or out_dtype is torch.float16
    assert bias is None or bias.numel() == b.shape[1] and bias.dtype == out_dtype
    target_shape = (*a.shape[:-1], b.shape[1])
    a = a.view(-1, a.shape[-1])
    out = torch.empty((a.shape[0], b.shape[1]), dtype=out_dtype, device=a.device)
    _ops.cutlass_scaled_mm(out, a, b, scale_a, scale_b, bias)
    return out.view(*target_shape)
