"""CPU tests of the host side: the C-ABI library loads and exports what the header declares, the device-resident
packing helpers and the layout="marlin" helper modes equal the oracle, ScalarType known answers, argument validation
raises the reference's errors, and the plugin classes follow the reference's contract."""
import os
import re

import numpy as np
import pytest
import torch

from oracle import w4a16 as o

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ------------------------------------------------------------------------------------------------ C ABI

def _header_symbols():
    """Declared by the drop-in header plus the library's own tuning header (tests and benchmarks only)."""
    names = set()
    for path in (("include", "vllm_amd_qlinear.h"), ("vllm_amd", "csrc", "vaq_tuning.h")):
        text = open(os.path.join(ROOT, *path)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(vaq_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_library_exports_nothing_but_the_c_abi():
    """Built with hidden visibility: the dynamic symbol table holds the declared entry points and no C++ internals."""
    import subprocess
    from vllm_amd import _lib
    out = subprocess.run(["nm", "-D", "--defined-only", str(_lib.LIB_PATH)], capture_output=True, text=True, check=True).stdout
    # only code: the data symbols that remain are the device-code registration objects the HIP toolchain emits itself
    defined = sorted(l.split()[-1] for l in out.splitlines() if l.split() and l.split()[-2] in "Tt")
    extra = [n for n in defined if n not in _header_symbols() and not n.startswith(("_init", "_fini"))]
    assert not extra, f"symbols exported beyond the headers: {extra[:10]}"
    drop_in = open(os.path.join(ROOT, "include", "vllm_amd_qlinear.h")).read()
    assert "VaqTuning" not in drop_in and "_tuned" not in drop_in and "probe" not in drop_in


def test_library_loads_and_exports_every_declared_symbol():
    from vllm_amd import _lib
    lib = _lib.load()                     # raises if the shared object has not been built
    declared = _header_symbols()
    assert declared, "no declarations found in the header"
    assert declared == _lib.exported_symbols(), "ctypes signature table and header disagree"
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/vllm_amd_qlinear.h but not exported"
    assert lib.vaq_abi_version() == 1
    assert lib.vaq_last_error() is not None


def test_c_abi_rejects_bad_arguments_without_a_gpu():
    """Host-side validation happens before any HIP call, so it can be exercised here with null pointers."""
    from vllm_amd import _lib
    lib = _lib.load()
    rc = lib.vaq_w4a16_repack(None, None, None, 100, 64, 4, _lib.VAQ_LAYOUT_NATIVE, None)
    assert rc == _lib.VAQ_ERR_INVALID_ARG and b"size_k = 100" in lib.vaq_last_error()
    rc = lib.vaq_w4a16_repack(None, None, None, 128, 64, 2, _lib.VAQ_LAYOUT_NATIVE, None)
    assert rc == _lib.VAQ_ERR_INVALID_ARG and b"num_bits" in lib.vaq_last_error()
    rc = lib.vaq_w4a16_repack_awq(None, None, 128, 64, 8, _lib.VAQ_LAYOUT_NATIVE, None)
    assert rc == _lib.VAQ_ERR_UNSUPPORTED
    with pytest.raises(NotImplementedError):
        _lib.check(rc)
    rc = lib.vaq_w4a16_repack(None, None, None, 144, 64, 4, _lib.VAQ_LAYOUT_NATIVE, None)
    assert rc == _lib.VAQ_ERR_INVALID_ARG and b"128" in lib.vaq_last_error()
    rc = lib.vaq_w4a16_gemm(None, 4096, None, None, None, None, None, None, None, 0, None, None, 0, 16, 4096 + 32, 4096,
                            128, _lib.VAQ_BF16, _lib.VAQ_WTYPE_U4B8, 0, None)
    assert rc == _lib.VAQ_ERR_INVALID_ARG and b"min_thread_n" in lib.vaq_last_error()
    rc = lib.vaq_w4a16_gemm(None, 4096, None, None, None, None, None, None, None, 0, None, None, 0, 16, 4096, 4096, 256,
                            _lib.VAQ_BF16, _lib.VAQ_WTYPE_U4B8, 0, None)
    assert rc == _lib.VAQ_ERR_UNSUPPORTED and b"group_size" in lib.vaq_last_error()
    rc = lib.vaq_fp8_scaled_mm(None, 100, None, 128, None, 1, None, 1, None, None, 128, _lib.VAQ_BF16, 4, 128, 128, None)
    assert rc == _lib.VAQ_ERR_INVALID_ARG
    with pytest.raises(RuntimeError):
        _lib.check(rc)
    rc = lib.vaq_fp8_quant_per_token(None, _lib.VAQ_BF16, 8, None, 16, None, None, 4, 16, None)
    assert rc == _lib.VAQ_ERR_INVALID_ARG and b"row strides" in lib.vaq_last_error()
    rc = lib.vaq_rms_norm_static_fp8_quant(None, None, 8, None, None, 1e-6, None, _lib.VAQ_BF16, 4, 16, None)
    assert rc == _lib.VAQ_ERR_INVALID_ARG and b"row stride" in lib.vaq_last_error()
    rc = lib.vaq_silu_and_mul_fp8_quant(None, None, None, _lib.VAQ_F32, 4, 16, None)
    assert rc == _lib.VAQ_ERR_INVALID_ARG and b"dtype" in lib.vaq_last_error()
    assert lib.vaq_silu_and_mul_fp8_quant(None, None, None, _lib.VAQ_BF16, 0, 16, None) == _lib.VAQ_OK
    # M == 0 is a no-op that touches nothing
    assert lib.vaq_w4a16_gemm(None, 4096, None, None, None, None, None, None, None, 0, None, None, 0, 0, 4096, 4096, 128,
                              _lib.VAQ_BF16, _lib.VAQ_WTYPE_U4B8, 0, None) == _lib.VAQ_OK


# ------------------------------------------------------------------------------------------------ ScalarType

def test_scalar_type_known_answers():
    """tests/test_scalartype.py:9-43 of the reference, plus the id layout of vllm/scalar_type.py:136-164."""
    from vllm_amd.scalar_type import ScalarType, scalar_types as st
    assert (st.uint4b8.min(), st.uint4b8.max()) == (-8, 7)
    assert (st.uint4.min(), st.uint4.max()) == (0, 15)
    assert (st.uint8b128.min(), st.uint8b128.max()) == (-128, 127)
    assert (st.int4.min(), st.int4.max()) == (-8, 7)
    for tt, t in ((torch.int8, st.int8), (torch.uint8, st.uint8)):
        assert (torch.iinfo(tt).min, torch.iinfo(tt).max) == (t.min(), t.max())
    for tt, t in ((torch.float8_e5m2, st.float8_e5m2), (torch.float8_e4m3fn, st.float8_e4m3fn),
                  (torch.bfloat16, st.float16_e8m7), (torch.float16, st.float16_e5m10)):
        assert (torch.finfo(tt).min, torch.finfo(tt).max) == (t.min(), t.max())
    # exponent(8) | mantissa(8) | signed(1) | bias(32) | finite(1) | nan_repr(8); integer types carry nan_repr = IEEE (1)
    assert st.uint4b8.id == (4 << 8) | (8 << 17) | (1 << 50) and (st.uint4b8.id & ((1 << 50) - 1)) == 1049600
    assert st.uint4.id == (4 << 8) | (1 << 50)
    assert st.uint4b8.size_bits == 4 and str(st.uint4b8) == "uint4b8" and str(st.float8_e4m3fn) == "float8_e4m3fn"
    for t in (st.uint4b8, st.uint4, st.float8_e4m3fn, st.uint8b128, st.int4):
        assert ScalarType.from_id(t.id) == t


# ------------------------------------------------------------------------------------------------ host helpers

def test_device_packing_helpers_equal_oracle():
    from vllm_amd.layers.quantization.utils import quant_utils as qu
    rng = np.random.default_rng(0)
    q = rng.integers(0, 16, size=(64, 48), dtype=np.int32)
    q[:, -1] = 15                                   # top nibble set -> negative int32 words
    q[-1, :] = 15
    qt = torch.from_numpy(q)
    assert np.array_equal(qu.gptq_pack(qt, 4, 64, 48).numpy(), o.gptq_pack(q, 4))
    assert np.array_equal(qu.pack_cols(qt, 4, 64, 48).numpy(), o.pack_cols(q, 4))
    assert np.array_equal(qu.unpack_cols(torch.from_numpy(o.pack_cols(q, 4)), 4, 64, 48).numpy(), q)
    assert qu.get_pack_factor(4) == 8


def test_marlin_layout_helpers_equal_oracle_and_native_helpers_are_plain():
    from vllm_amd.layers.quantization.utils import marlin_utils as mu
    rng = np.random.default_rng(1)
    k, n, g = 512, 192, 128
    s = torch.from_numpy(rng.standard_normal((k // g, n)).astype(np.float32)).to(torch.bfloat16)
    assert torch.equal(mu.marlin_permute_scales(s, k, n, g, layout="marlin").float(),
                       torch.from_numpy(o.marlin_permute_scales(s.float().numpy(), k, n, g)))
    assert torch.equal(mu.marlin_permute_scales(s[:1], k, n, -1, layout="marlin").float(),
                       torch.from_numpy(o.marlin_permute_scales(s[:1].float().numpy(), k, n, -1)))
    assert torch.equal(mu.marlin_permute_scales(s, k, n, g), s)
    zp = rng.integers(0, 16, size=(k // g, n), dtype=np.int32)
    assert np.array_equal(mu.marlin_zero_points(torch.from_numpy(zp), k // g, n, 4, layout="marlin").numpy(),
                          o.marlin_zero_points(zp, k // g, n, 4))
    assert np.array_equal(mu.marlin_zero_points(torch.from_numpy(zp), k // g, n, 4).numpy(), o.pack_cols(zp, 4))
    awq = o.pack_cols(zp.reshape(-1, 8)[:, np.asarray(o.INTERLEAVE4)].reshape(zp.shape), 4)
    assert np.array_equal(mu.awq_to_marlin_zero_points(torch.from_numpy(awq), k // g, n, 4, layout="marlin").numpy(),
                          o.awq_to_marlin_zero_points(awq, k // g, n, 4))
    b = torch.arange(n, dtype=torch.float32)
    assert torch.equal(mu.marlin_permute_bias(b, layout="marlin"), torch.from_numpy(o.marlin_permute_bias(b.numpy())))
    g_idx = torch.from_numpy((np.arange(k) // g).astype(np.int32)[rng.permutation(k)])
    sorted_g, order = mu.marlin_sort_g_idx(g_idx)
    ref_sorted, ref_order = o.marlin_sort_g_idx(g_idx.numpy())
    assert np.array_equal(sorted_g.numpy(), ref_sorted) and np.array_equal(order.numpy(), ref_order)
    assert mu.marlin_is_k_full(True, False) and not mu.marlin_is_k_full(True, True) and mu.marlin_is_k_full(False, True)
    assert mu.get_scale_perms() == o.get_scale_perms()


def test_shape_and_type_support_checks():
    from vllm_amd.layers.quantization.utils import marlin_utils as mu
    from vllm_amd.scalar_type import scalar_types as st
    mu.verify_marlin_supports_shape(4096, 4096, 4096, 128)
    for bad in ((4096 + 32, 4096, 4096, 128), (4096, 4096 + 64, 4096 + 64, 128)):
        with pytest.raises(ValueError):
            mu.verify_marlin_supports_shape(*bad)
    assert mu.check_marlin_supported(st.uint4b8, 128) and not mu.check_marlin_supported(st.uint4b8, 256)
    assert all(mu.check_marlin_supported(st.uint4b8, g) for g in (-1, 32, 64))
    assert mu.check_marlin_supported(st.uint4, 128, has_zp=True) and not mu.check_marlin_supported(st.uint4, 128)
    for g in (-1, 32, 64, 128):
        mu.verify_marlin_supported(st.uint8b128, g)
    with pytest.raises(ValueError):
        mu.verify_marlin_supported(st.uint8b128, 256)
    with pytest.raises(ValueError):
        mu.verify_marlin_supported(st.uint8, 128, has_zp=True)


# ------------------------------------------------------------------------------------------------ op argument validation

def _gemm_args(**over):
    from vllm_amd.scalar_type import scalar_types as st
    k, n, m = 256, 128, 4
    args = dict(a=torch.zeros(m, k, dtype=torch.bfloat16), c=None, b_q_weight=torch.zeros(k // 16, 2 * n, dtype=torch.int32),
                b_bias=None, b_scales=torch.zeros(k // 128, n, dtype=torch.bfloat16), global_scale=None,
                b_zeros=torch.empty(0, dtype=torch.int32), g_idx=torch.empty(0, dtype=torch.int32),
                perm=torch.empty(0, dtype=torch.int32), workspace=torch.zeros(64, dtype=torch.int32),
                b_q_type_id=st.uint4b8.id, size_m=m, size_n=n, size_k=k, is_k_full=True, is_zp_float=False)
    args.update(over)
    return args


@pytest.mark.parametrize("over,exc,msg", [
    (dict(size_m=5), RuntimeError, "a.size(0)"),
    (dict(size_k=512), RuntimeError, "a.size(1)"),
    (dict(size_n=192), RuntimeError, "actual_size_n"),
    (dict(b_q_weight=torch.zeros(8, 256, dtype=torch.int32)), RuntimeError, "b_q_weight.size(0)"),
    (dict(a=torch.zeros(4, 256, dtype=torch.bfloat16)), RuntimeError, "A is not on GPU"),   # CPU tensors fail loudly
])
def test_gemm_argument_checks(over, exc, msg):
    from vllm_amd import _custom_ops as ops
    a = _gemm_args(**over)
    with pytest.raises(exc, match=re.escape(msg)):
        ops._check_gemm_args(a["a"], a["c"], a["b_q_weight"], a["b_bias"], a["b_scales"], a["global_scale"], a["b_zeros"],
                             a["g_idx"], a["perm"], a["workspace"], a["b_q_type_id"], a["size_m"], a["size_n"],
                             a["size_k"], a["is_k_full"], a["is_zp_float"])


def test_repack_and_scaled_mm_argument_checks():
    from vllm_amd import _custom_ops as ops
    qw = torch.zeros(16, 64, dtype=torch.int32)
    empty = torch.empty(0, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="tile_k_size"):
        ops._check_repack_args(qw, empty, 120, 64, 4)
    with pytest.raises(RuntimeError, match="tile_n_size"):
        ops._check_repack_args(qw, empty, 128, 96, 4)
    with pytest.raises(RuntimeError, match="num_bits must be 4 or 8"):
        ops._check_repack_args(qw, empty, 128, 64, 3)
    with pytest.raises(RuntimeError, match="Shape mismatch"):
        ops._check_repack_args(qw, empty, 256, 64, 4)
    with pytest.raises(RuntimeError, match="not on GPU"):
        ops._check_repack_args(qw, empty, 128, 64, 4)
    a = torch.zeros(4, 64, dtype=torch.float8_e4m3fn)
    b = torch.zeros(32, 64, dtype=torch.float8_e4m3fn).t()
    out = torch.zeros(4, 32, dtype=torch.bfloat16)
    one = torch.ones(1)
    with pytest.raises(RuntimeError, match="column-major"):
        ops._check_scaled_mm_args(out, a, b.t().contiguous().t().contiguous(), one, one, None)
    with pytest.raises(RuntimeError, match="shape mismatch"):
        ops._check_scaled_mm_args(out, a[:, :32], b, one, one, None)
    with pytest.raises(RuntimeError, match="GPU"):
        ops._check_scaled_mm_args(out, a, b, one, one, None)
    # calling an op with CPU tensors must fail loudly: there is no CPU implementation
    with pytest.raises((NotImplementedError, RuntimeError)):
        ops.scaled_fp8_quant(torch.zeros(2, 16, dtype=torch.bfloat16), use_per_token_if_dynamic=True)


def test_awq_repack_argument_checks_and_helpers():
    """Host checks of awq_marlin_repack (awq_marlin_repack.cu:208-232) and the AWQ zero-point conversion against the
    oracle, both layouts (marlin_utils.py:349-370)."""
    import vllm_amd._custom_ops as ops
    from oracle import w4a16 as o
    from vllm_amd.layers.quantization.utils import marlin_utils as mu
    qw = torch.zeros(128, 8, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="not divisible by tile_k_size"):
        ops._check_awq_repack_args(qw, 100, 64, 4)
    with pytest.raises(RuntimeError, match="not divisible by tile_n_size"):
        ops._check_awq_repack_args(qw, 128, 72, 4)
    with pytest.raises(RuntimeError, match="num_bits must be 4 or 8"):
        ops._check_awq_repack_args(qw, 128, 64, 3)
    with pytest.raises(RuntimeError, match="Shape mismatch"):
        ops._check_awq_repack_args(qw, 128, 128, 4)
    with pytest.raises(RuntimeError, match="not on GPU"):
        ops._check_awq_repack_args(qw, 128, 64, 4)
    rng = np.random.default_rng(3)
    groups, n = 6, 192
    zp = rng.integers(0, 16, size=(groups, n), dtype=np.int32)
    packed = torch.from_numpy(o.awq_pack(zp, 4))
    got_marlin = mu.awq_to_marlin_zero_points(packed, groups, n, 4, layout="marlin")
    assert np.array_equal(got_marlin.numpy(), o.awq_to_marlin_zero_points(o.awq_pack(zp, 4), groups, n, 4))
    got_native = mu.awq_to_marlin_zero_points(packed, groups, n, 4)
    assert np.array_equal(got_native.numpy(), o.pack_cols(zp, 4))


def test_fake_tensor_shapes():
    """The fake (meta) implementations give the reference's output shapes (_custom_ops.py:524-545,
    gptq_marlin_repack.cu:324-334)."""
    from vllm_amd import _custom_ops as ops  # noqa: F401
    from vllm_amd.scalar_type import scalar_types as st
    with torch._subclasses.fake_tensor.FakeTensorMode():
        qw = torch.empty(512 // 8, 256, dtype=torch.int32, device="cuda")
        perm = torch.empty(0, dtype=torch.int32, device="cuda")
        out = torch.ops.vllm_amd.gptq_marlin_repack(qw, perm, 512, 256, 4)
        assert out.shape == (512 // 16, 256 * 16 // 8) and out.dtype == torch.int32
        a = torch.empty(7, 512, dtype=torch.bfloat16, device="cuda")
        s = torch.empty(4, 256, dtype=torch.bfloat16, device="cuda")
        ws = torch.empty(64, dtype=torch.int32, device="cuda")
        c = torch.ops.vllm_amd.gptq_marlin_gemm(a, None, out, None, s, None, perm, perm, perm, ws, st.uint4b8.id, 7, 256, 512)
        assert c.shape == (7, 256) and c.dtype == torch.bfloat16


# ------------------------------------------------------------------------------------------------ plugin surface

def test_plugin_surface_contract():
    from vllm_amd.layers.linear import LinearBase, QKVParallelLinear
    from vllm_amd.layers.quantization import (QUANTIZATION_METHODS, QuantizationConfig, get_quantization_config,
                                              register_quantization_config)
    from vllm_amd.layers.quantization.gptq_marlin import GPTQMarlinConfig, GPTQMarlinLinearMethod
    from vllm_amd.layers.quantization.kernels.mixed_precision import (HipW4A16LinearKernel, MPLinearLayerConfig,
                                                                      choose_mp_linear_kernel)
    from vllm_amd.scalar_type import scalar_types as st
    cfg = get_quantization_config("gptq_marlin").from_config(dict(bits=4, group_size=128, desc_act=True, sym=True))
    assert isinstance(cfg, GPTQMarlinConfig) and cfg.quant_type == st.uint4b8 and cfg.pack_factor == 8
    layer = QKVParallelLinear(4096, 128, 32, 8, quant_config=cfg, params_dtype=torch.bfloat16)
    assert isinstance(layer.quant_method, GPTQMarlinLinearMethod)
    shapes = {n: tuple(p.shape) for n, p in layer.named_parameters()}
    assert shapes == {"qweight": (512, 6144), "g_idx": (4096,), "scales": (32, 6144), "qzeros": (32, 768)}
    assert GPTQMarlinConfig.is_gptq_marlin_compatible(dict(quant_method="gptq", bits=4, group_size=128, sym=True, desc_act=False))
    assert GPTQMarlinConfig.is_gptq_marlin_compatible(dict(quant_method="gptq", bits=8, group_size=128, sym=True, desc_act=False))
    assert GPTQMarlinConfig.is_gptq_marlin_compatible(dict(quant_method="gptq", bits=8, group_size=32, sym=True, desc_act=False))
    assert not GPTQMarlinConfig.is_gptq_marlin_compatible(dict(quant_method="gptq", bits=8, group_size=256, sym=True, desc_act=False))
    assert not GPTQMarlinConfig.is_gptq_marlin_compatible(dict(quant_method="gptq", bits=4, group_size=128, sym=False, desc_act=False))
    assert GPTQMarlinConfig.override_quantization_method(dict(quant_method="gptq", bits=4, group_size=128, sym=True, desc_act=False), None) == "gptq_marlin"
    mp = MPLinearLayerConfig((4096, 4096), (4096, 4096), st.uint4, torch.bfloat16, 128, True, False)
    assert choose_mp_linear_kernel(mp) is HipW4A16LinearKernel
    assert choose_mp_linear_kernel(MPLinearLayerConfig((4096, 4096), (4096, 4096), st.uint4b8, torch.bfloat16, 32, False,
                                                       False)) is HipW4A16LinearKernel
    bad = MPLinearLayerConfig((4096, 4096), (4096, 4096), st.uint4b8, torch.bfloat16, 256, False, False)
    with pytest.raises(ValueError, match="Group size"):
        choose_mp_linear_kernel(bad)
    os.environ["VLLM_DISABLED_KERNELS"] = "HipW4A16LinearKernel"
    try:
        with pytest.raises(ValueError, match="disabled"):
            choose_mp_linear_kernel(mp)
    finally:
        del os.environ["VLLM_DISABLED_KERNELS"]
    # FP8 methods
    f8 = get_quantization_config("fp8").from_config(dict(quant_method="fp8", activation_scheme="dynamic"))
    lin = LinearBase(256, 128, quant_config=f8, params_dtype=torch.bfloat16)
    assert lin.weight.dtype == torch.float8_e4m3fn and lin.weight.shape == (128, 256) and lin.input_scale is None
    ptpc = get_quantization_config("ptpc_fp8").from_config({})
    lin = LinearBase(256, 128, quant_config=ptpc, params_dtype=torch.bfloat16)
    assert lin.weight.dtype == torch.bfloat16
    # out-of-tree registration hook
    @register_quantization_config("my_method")
    class MyConfig(QuantizationConfig):
        def get_name(self): return "my_method"
        def get_supported_act_dtypes(self): return [torch.bfloat16]
        @classmethod
        def get_min_capability(cls): return 0
        @staticmethod
        def get_config_filenames(): return []
        @classmethod
        def from_config(cls, config): return cls()
        def get_quant_method(self, layer, prefix): return None
    assert "my_method" in QUANTIZATION_METHODS and get_quantization_config("my_method") is MyConfig
    with pytest.raises(ValueError):
        get_quantization_config("no_such_method")


# ------------------------------------------------------------------------------------------------ checkpoint loading

def test_weight_loaders_place_checkpoint_tensors_in_fused_layers():
    """The loader side of the plugin contract (parameter.py:129-408, linear.py:784-866,:948-1060): logical parts of
    a fused layer arrive one checkpoint tensor at a time, each parameter knows its output / packed dimension, and a
    tensor that is already fused on disk is cut into the parts.  Checked against plain concatenation."""
    from vllm_amd.layers.linear import MergedColumnParallelLinear, QKVParallelLinear, RowParallelLinear
    from vllm_amd.layers.quantization import get_quantization_config
    from vllm_amd.parameter import (GroupQuantScaleParameter, PackedvLLMParameter, PerTensorScaleParameter,
                                    RowvLLMParameter)
    g = torch.Generator().manual_seed(0)
    ri = lambda *shape: torch.randint(-2 ** 31, 2 ** 31 - 1, shape, dtype=torch.int32, generator=g)   # noqa: E731
    k = 256

    # GPTQ: qweight packed along K (output offsets unchanged), qzeros packed along N (output offsets / 8)
    cfg = get_quantization_config("gptq_marlin").from_config(dict(bits=4, group_size=128, desc_act=False, sym=True))
    sizes = [128, 192]
    layer = MergedColumnParallelLinear(k, sizes, quant_config=cfg, params_dtype=torch.float16, bias=True)
    assert isinstance(layer.qweight, PackedvLLMParameter) and layer.qweight.packed_dim == 0
    assert isinstance(layer.qzeros, PackedvLLMParameter) and layer.qzeros.packed_dim == layer.qzeros.output_dim == 1
    assert isinstance(layer.scales, GroupQuantScaleParameter) and isinstance(layer.g_idx, RowvLLMParameter)
    parts = [dict(qweight=ri(k // 8, n), qzeros=ri(k // 128, n // 8), scales=torch.randn(k // 128, n, generator=g).half(),
                  bias=torch.randn(n, generator=g).half()) for n in sizes]
    g_idx = torch.arange(k, dtype=torch.int32) // 128
    for name in ("qweight", "qzeros", "scales", "bias"):
        for shard_id in (1, 0):                                         # any order
            param = getattr(layer, name)
            param.weight_loader(param, parts[shard_id][name], shard_id)
        assert torch.equal(getattr(layer, name).data, torch.cat([p_[name] for p_ in parts], dim=-1)), name
    layer.g_idx.weight_loader(layer.g_idx, g_idx)
    assert torch.equal(layer.g_idx.data, g_idx)
    # the same layer from tensors that are already fused on disk
    layer2 = MergedColumnParallelLinear(k, sizes, quant_config=cfg, params_dtype=torch.float16)
    for name in ("qweight", "qzeros", "scales"):
        param = getattr(layer2, name)
        param.weight_loader(param, getattr(layer, name).data.clone())
        assert torch.equal(param.data, getattr(layer, name).data), name
    with pytest.raises(ValueError):
        layer.qweight.weight_loader(layer.qweight, ri(k // 8, 64), 0)   # wrong part size

    # AWQ: weights AND zero points packed along N; q / k / v shard ids
    cfg = get_quantization_config("awq_marlin").from_config(dict(quant_method="awq", bits=4, group_size=128, zero_point=True))
    qkv = QKVParallelLinear(k, 64, 4, 2, quant_config=cfg, params_dtype=torch.float16)          # q 256, k 128, v 128
    assert qkv.output_sizes == [256, 128, 128] and qkv.qweight.packed_dim == qkv.qweight.output_dim == 1
    shards = {sid: dict(qweight=ri(k, n // 8), qzeros=ri(k // 128, n // 8),
                        scales=torch.randn(k // 128, n, generator=g).half())
              for sid, n in zip("qkv", qkv.output_sizes)}
    for sid in "vqk":
        for name in ("qweight", "qzeros", "scales"):
            param = getattr(qkv, name)
            param.weight_loader(param, shards[sid][name], sid)
    for name in ("qweight", "qzeros", "scales"):
        assert torch.equal(getattr(qkv, name).data, torch.cat([shards[sid][name] for sid in "qkv"], dim=-1)), name

    # FP8 serialized: weight rows per part, one scale per part (a scalar on disk), static input scales
    from vllm_amd.layers.quantization.fp8 import Fp8Config
    fcfg = Fp8Config(is_checkpoint_fp8_serialized=True, activation_scheme="static")
    f8 = QKVParallelLinear(k, 64, 4, 2, quant_config=fcfg, params_dtype=torch.bfloat16)
    assert isinstance(f8.weight_scale, PerTensorScaleParameter) and f8.weight_scale.shape == (3,)
    ws = {sid: torch.randint(0, 255, (n, k), dtype=torch.uint8, generator=g).view(torch.float8_e4m3fn)
          for sid, n in zip("qkv", f8.output_sizes)}
    for i, sid in enumerate("kvq"):
        f8.weight.weight_loader(f8.weight, ws[sid], sid)
        f8.weight_scale.weight_loader(f8.weight_scale, torch.tensor(0.5 + i), sid)
        f8.input_scale.weight_loader(f8.input_scale, torch.tensor([0.25 * (i + 1)]), sid)
    assert torch.equal(f8.weight.data.view(torch.uint8), torch.cat([ws[sid] for sid in "qkv"]).view(torch.uint8))
    assert f8.weight_scale.data.tolist() == [2.5, 0.5, 1.5] and f8.input_scale.data.tolist() == [0.75, 0.25, 0.5]

    # a plain (row-parallel) layer takes the whole tensor; a scalar checkpoint scale lands in a one-element parameter
    row = RowParallelLinear(k, 64, quant_config=fcfg, params_dtype=torch.bfloat16)
    w = torch.randint(0, 255, (64, k), dtype=torch.uint8, generator=g).view(torch.float8_e4m3fn)
    row.weight.weight_loader(row.weight, w)
    row.weight_scale.weight_loader(row.weight_scale, torch.tensor(0.125))
    assert torch.equal(row.weight.data.view(torch.uint8), w.view(torch.uint8)) and row.weight_scale.data.tolist() == [0.125]



def test_fp8_module_fused_on_disk_keeps_its_weight():
    """A qkv / gate_up module that is already fused in an FP8 checkpoint brings ONE weight scale: `weight_loader_v2`
    puts it in entry 0 and the other entries keep their initial value (the most negative float).  The method must then
    keep the weight as loaded and use that one scale -- requantising the shards with the untouched entries would turn
    them into +-448 (the reference skips it the same way: w8a8_utils.py:108-136)."""
    from vllm_amd.layers.linear import MergedColumnParallelLinear
    from vllm_amd.layers.quantization.fp8 import Fp8Config
    k, sizes = 64, [32, 48]
    cfg = Fp8Config(is_checkpoint_fp8_serialized=True, activation_scheme="dynamic")
    layer = MergedColumnParallelLinear(k, sizes, quant_config=cfg, params_dtype=torch.bfloat16, return_bias=False)
    g = torch.Generator().manual_seed(11)
    w = torch.randint(0, 0x7E, (sum(sizes), k), dtype=torch.uint8, generator=g).view(torch.float8_e4m3fn)
    layer.weight.weight_loader(layer.weight, w)                              # no shard id: fused on disk
    layer.weight_scale.weight_loader(layer.weight_scale, torch.tensor(0.0375))
    assert layer.weight_scale.data[0] == torch.tensor(0.0375) and layer.weight_scale.data[1] == torch.finfo(torch.float32).min
    layer.process_weights_after_loading()                                    # no device work on this branch
    assert torch.equal(layer.weight.t().contiguous().view(torch.uint8), w.view(torch.uint8)), "weight was requantised"
    assert layer.weight_scale.dim() == 0 and float(layer.weight_scale) == float(torch.tensor(0.0375))
    assert layer.input_scale is None


def test_tuning_override_applies_to_one_call_only():
    """A VaqTuning travels with the call it is passed to: the `_tuned` workspace query sees the forced K split, the plain
    query right after it sees the automatic choice again (the library keeps no tuning state)."""
    import ctypes
    from vllm_amd import _lib
    lib = _lib.load()

    def query(tuning=None):
        t, a, n = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
        args = (8, 320, 2048, 0, 0, ctypes.byref(t), ctypes.byref(a), ctypes.byref(n))
        rc = lib.vaq_w4a16_gemm_workspace(*args) if tuning is None else lib.vaq_w4a16_gemm_workspace_tuned(*args, tuning)
        assert rc == _lib.VAQ_OK
        return t.value, n.value

    auto = query()
    assert auto == (0, 0)                      # K = 2048 fits one workgroup's LDS: no split, no scratch
    forced = _lib.VaqTuning(decode_impl=1, decode2_gs=2, decode2_wks=2, decode2_wn=1)     # slabs of 4 groups: 4 splits
    t, n = query(ctypes.byref(forced))
    assert n == 320 // 16 and t >= 4 * (320 // 16) * 1024      # (the query covers whichever decode kernel may run)
    assert query() == auto and query(None) == auto


def test_workspace_from_the_helper_covers_every_batch_size():
    """`marlin_make_workspace_new` must satisfy the GEMM's counter request for every M on the layer it was sized for, and
    its default size must do so on a vocabulary-sized layer (N = 128256: three m-blocks at M = 40 need 24048 counters)."""
    import ctypes
    from vllm_amd import _lib
    from vllm_amd.layers.quantization.utils.marlin_utils import marlin_workspace_ints
    lib = _lib.load()
    for n, k in ((128256, 4096), (4096, 14336), (28672, 4096), (64, 128)):
        for m in (1, 16, 17, 32, 33, 40, 48, 49, 64, 65, 100, 256, 1024, 4096):
            t, a, c = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
            assert lib.vaq_w4a16_gemm_workspace(m, n, k, 0, 0, ctypes.byref(t), ctypes.byref(a), ctypes.byref(c)) == _lib.VAQ_OK
            assert c.value <= marlin_workspace_ints(n), (n, k, m, c.value)
            assert c.value <= marlin_workspace_ints(None), (n, k, m, c.value)
