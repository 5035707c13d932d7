"""GPU tests of the plugin surface: quantization configs -> linear methods -> ``create_weights`` /
``process_weights_after_loading`` / ``apply`` on a device layer, checked against the CPU oracle; HIP-graph replays of the
same layers; dispatcher checks of the custom ops (schema + fake tensors) with device arguments.

The flow mirrors how the reference drives a quantized layer (linear.py:243-300, gptq_marlin.py:329-466, fp8.py:330-684):
a checkpoint's tensors are copied into the parameters that ``create_weights`` registered, then
``process_weights_after_loading`` rewrites them in place, then ``forward`` calls ``quant_method.apply``."""
import numpy as np
import pytest
import torch

from oracle import fp8 as of
from oracle import w4a16 as o
from tests.helpers import check_gemm_close, to_dev

pytestmark = pytest.mark.gpu


def _acts(m, k, dtype=torch.bfloat16, seed=0):
    return torch.randn(m, k, generator=torch.Generator().manual_seed(seed)).to(dtype)


def _gptq_layer(device, k, n_sizes, desc_act, dtype, seed, bias=False):
    """A MergedColumnParallelLinear with a synthetic GPTQ checkpoint loaded; returns (layer, oracle case, bias)."""
    from vllm_amd.layers.linear import MergedColumnParallelLinear
    from vllm_amd.layers.quantization import get_quantization_config
    n = sum(n_sizes)
    cfg = get_quantization_config("gptq_marlin").from_config(dict(bits=4, group_size=128, desc_act=desc_act, sym=True))
    layer = MergedColumnParallelLinear(k, n_sizes, quant_config=cfg, params_dtype=dtype, bias=bias, return_bias=False)
    case = o.make_w4a16_case(k, n, 128, asym=False, act_order=desc_act, dtype=dtype, seed=seed)
    layer = layer.to(device)
    layer.qweight.data.copy_(to_dev(case["qweight"], device))
    layer.scales.data.copy_(to_dev(case["scales"], device, dtype))
    g_idx = case["g_idx"] if case["g_idx"] is not None else np.arange(k, dtype=np.int32) // 128
    layer.g_idx.data.copy_(to_dev(g_idx, device))
    # a symmetric GPTQ checkpoint stores zero point 8 (as 7 in the v1 format); the method ignores qzeros
    layer.qzeros.data.fill_(0x77777777)
    b = None
    if bias:
        b = (torch.randn(n, generator=torch.Generator().manual_seed(seed + 1)) * 0.5).to(dtype)
        layer.bias.data.copy_(b.to(device))
    layer.process_weights_after_loading()
    return layer, case, b


@pytest.mark.parametrize("desc_act", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gptq_linear_method_end_to_end(device, desc_act, dtype):
    k, n_sizes = 1024, [256, 128, 128]
    layer, case, bias = _gptq_layer(device, k, n_sizes, desc_act, dtype, seed=3, bias=True)
    from vllm_amd.layers.quantization.gptq_marlin import GPTQMarlinLinearMethod
    assert isinstance(layer.quant_method, GPTQMarlinLinearMethod)
    # the loader's parameters were rewritten in place (marlin.py:85-140): same names, repacked contents
    assert layer.qweight.shape == (k // 16, 2 * sum(n_sizes)) and layer.qweight.dtype == torch.int32
    w_ref = o.case_w_ref(case)
    for m in (1, 16, 33, 200):
        a = _acts(m, k, dtype, seed=m)
        out = layer(a.to(device))
        assert out.shape == (m, sum(n_sizes)) and out.dtype == dtype
        check_gemm_close(out, o.gemm_ref(a, w_ref, bias), f"gptq method desc_act={desc_act} {dtype} m={m}")
    # leading batch dimensions are flattened and restored (marlin_utils.py:449-450,:481)
    a3 = _acts(6, k, dtype, seed=9).reshape(2, 3, k)
    out3 = layer(a3.to(device))
    assert out3.shape == (2, 3, sum(n_sizes))
    check_gemm_close(out3.reshape(6, -1), o.gemm_ref(a3.reshape(6, k), w_ref, bias), "gptq method 3-d input")


def test_gptq_group_level_act_order_is_folded_at_load(device):
    """g_idx that permutes whole groups (BASELINE.json config 3's wording): the method gathers the scale rows at load time and
    runs without any activation reorder; results equal the oracle's act_order semantics."""
    from vllm_amd.layers.linear import LinearBase
    from vllm_amd.layers.quantization import get_quantization_config
    k, n = 2048, 256
    cfg = get_quantization_config("gptq_marlin").from_config(dict(bits=4, group_size=128, desc_act=True, sym=True))
    case = o.make_w4a16_case(k, n, 128, act_order=True, group_level_perm=True, seed=31)
    layer = LinearBase(k, n, quant_config=cfg, params_dtype=torch.bfloat16, return_bias=False).to(device)
    layer.qweight.data.copy_(to_dev(case["qweight"], device))
    layer.scales.data.copy_(to_dev(case["scales"], device, torch.bfloat16))
    layer.g_idx.data.copy_(to_dev(case["g_idx"], device))
    layer.process_weights_after_loading()
    assert layer.quant_method.kernel.act_order_folded
    assert layer.g_idx.numel() == 0 and layer.g_idx_sort_indices.numel() == 0
    w_ref = o.case_w_ref(case)
    for m in (2, 16, 100):
        a = _acts(m, k, seed=m)
        check_gemm_close(layer(a.to(device)), o.gemm_ref(a, w_ref), f"folded act_order m={m}")
    # a row-level permutation is not folded
    case2 = o.make_w4a16_case(k, n, 128, act_order=True, seed=32)
    layer2 = LinearBase(k, n, quant_config=cfg, params_dtype=torch.bfloat16, return_bias=False).to(device)
    layer2.qweight.data.copy_(to_dev(case2["qweight"], device))
    layer2.scales.data.copy_(to_dev(case2["scales"], device, torch.bfloat16))
    layer2.g_idx.data.copy_(to_dev(case2["g_idx"], device))
    layer2.process_weights_after_loading()
    assert not layer2.quant_method.kernel.act_order_folded and layer2.g_idx_sort_indices.numel() == k
    a = _acts(9, k, seed=1)
    check_gemm_close(layer2(a.to(device)), o.gemm_ref(a, o.case_w_ref(case2)), "row-level act_order")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_awq_linear_method_end_to_end(device, dtype):
    """AutoAWQ checkpoint (weights and zero points packed along N with the AWQ interleave) through AWQMarlinConfig ->
    AWQMarlinLinearMethod (awq_marlin.py:264-413) against the oracle's dequantise + fp64 GEMM."""
    from vllm_amd.layers.linear import MergedColumnParallelLinear, UnquantizedLinearMethod
    from vllm_amd.layers.quantization import get_quantization_config
    from vllm_amd.layers.quantization.awq_marlin import AWQMarlinConfig, AWQMarlinLinearMethod
    hf = dict(quant_method="awq", bits=4, group_size=128, zero_point=True, modules_to_not_convert=["lm_head"])
    assert AWQMarlinConfig.override_quantization_method(hf, None) == "awq_marlin"
    assert AWQMarlinConfig.override_quantization_method(hf, "awq") is None
    assert not AWQMarlinConfig.is_awq_marlin_compatible(dict(hf, bits=8))
    cfg = get_quantization_config("awq_marlin").from_config(hf)
    k, sizes = 1024, [256, 192]
    n = sum(sizes)
    layer = MergedColumnParallelLinear(k, sizes, quant_config=cfg, params_dtype=dtype, bias=True, return_bias=False,
                                       prefix="model.layers.0.mlp.gate_up_proj").to(device)
    assert isinstance(layer.quant_method, AWQMarlinLinearMethod)
    skipped = MergedColumnParallelLinear(k, sizes, quant_config=cfg, params_dtype=dtype, prefix="lm_head")
    assert isinstance(skipped.quant_method, UnquantizedLinearMethod)
    case = o.make_w4a16_case(k, n, 128, asym=True, act_order=False, dtype=dtype, seed=21)
    layer.qweight.data.copy_(to_dev(o.awq_pack(case["q"], 4), device))
    layer.qzeros.data.copy_(to_dev(o.awq_pack(case["zp_vals"], 4), device))
    layer.scales.data.copy_(to_dev(case["scales"], device, dtype))
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(4)) * 0.5).to(dtype)
    layer.bias.data.copy_(bias.to(device))
    layer.process_weights_after_loading()
    assert layer.qweight.shape == (k // 16, 2 * n) and layer.qzeros.shape == (k // 128, n // 8)
    w_ref = o.case_w_ref(case)
    for m in (1, 8, 17, 150):
        a = _acts(m, k, dtype, seed=m)
        out = layer(a.to(device))
        assert out.shape == (m, n) and out.dtype == dtype
        check_gemm_close(out, o.gemm_ref(a, w_ref, bias), f"awq method {dtype} m={m}")


@pytest.mark.parametrize("group_size", [-1, 32, 64])
def test_gptq_and_awq_methods_other_group_sizes(device, group_size):
    """The linear methods at the reference's other supported group sizes (marlin_utils.py:24): a GPTQ layer (channelwise
    when group_size = -1; otherwise with act_order, once row-level and once moving whole groups, which is folded at load
    also for 32- and 64-row groups) and an AWQ layer."""
    from vllm_amd.layers.linear import LinearBase
    from vllm_amd.layers.quantization import get_quantization_config
    k, n = 1024, 256
    desc_act = group_size != -1
    cfg = get_quantization_config("gptq_marlin").from_config(dict(bits=4, group_size=group_size, desc_act=desc_act, sym=True))
    for group_level in ((False, True) if desc_act else (False,)):
        case = o.make_w4a16_case(k, n, group_size, act_order=desc_act, group_level_perm=group_level, seed=50 + group_size)
        layer = LinearBase(k, n, quant_config=cfg, params_dtype=torch.bfloat16, return_bias=False).to(device)
        assert layer.scales.shape == case["scales"].shape
        layer.qweight.data.copy_(to_dev(case["qweight"], device))
        layer.scales.data.copy_(to_dev(case["scales"], device, torch.bfloat16))
        gs = k if group_size == -1 else group_size
        g_idx = case["g_idx"] if case["g_idx"] is not None else np.arange(k, dtype=np.int32) // gs
        layer.g_idx.data.copy_(to_dev(g_idx, device))
        layer.process_weights_after_loading()
        assert layer.quant_method.kernel.act_order_folded == group_level
        w_ref = o.case_w_ref(case)
        for m in (1, 16, 32, 150):
            a = _acts(m, k, seed=m)
            check_gemm_close(layer(a.to(device)), o.gemm_ref(a, w_ref), f"gptq g={group_size} folded={group_level} m={m}")
    if group_size == -1:
        return      # AutoAWQ has no channelwise checkpoints
    hf = dict(quant_method="awq", bits=4, group_size=group_size, zero_point=True)
    cfg = get_quantization_config("awq_marlin").from_config(hf)
    case = o.make_w4a16_case(k, n, group_size, asym=True, seed=60 + group_size)
    layer = LinearBase(k, n, quant_config=cfg, params_dtype=torch.bfloat16, return_bias=False).to(device)
    layer.qweight.data.copy_(to_dev(o.awq_pack(case["q"], 4), device))
    layer.qzeros.data.copy_(to_dev(o.awq_pack(case["zp_vals"], 4), device))
    layer.scales.data.copy_(to_dev(case["scales"], device, torch.bfloat16))
    layer.process_weights_after_loading()
    w_ref = o.case_w_ref(case)
    for m in (1, 16, 32, 150):
        a = _acts(m, k, seed=m)
        check_gemm_close(layer(a.to(device)), o.gemm_ref(a, w_ref), f"awq g={group_size} m={m}")


@pytest.mark.parametrize("group_size,desc_act", [(128, False), (128, True), (-1, False), (64, True), (32, False)])
def test_gptq_8bit_method_end_to_end(device, group_size, desc_act):
    """A GPTQ 8-bit checkpoint (bits = 8, sym: the uint8b128 type, gptq_marlin.py:96-99) through GPTQMarlinConfig and
    the linear method: qweight packs 4 codes per int32 along K."""
    from vllm_amd.layers.linear import LinearBase
    from vllm_amd.layers.quantization import get_quantization_config
    from vllm_amd.scalar_type import scalar_types
    k, n = 1024, 256
    cfg = get_quantization_config("gptq_marlin").from_config(dict(bits=8, group_size=group_size, desc_act=desc_act, sym=True))
    assert cfg.quant_type == scalar_types.uint8b128 and cfg.pack_factor == 4
    case = o.make_w4a16_case(k, n, group_size, act_order=desc_act, seed=70 + group_size, num_bits=8)
    layer = LinearBase(k, n, quant_config=cfg, params_dtype=torch.bfloat16, return_bias=False).to(device)
    assert layer.qweight.shape == (k // 4, n)
    layer.qweight.data.copy_(to_dev(case["qweight"], device))
    layer.scales.data.copy_(to_dev(case["scales"], device, torch.bfloat16))
    gs = k if group_size == -1 else group_size
    g_idx = case["g_idx"] if case["g_idx"] is not None else np.arange(k, dtype=np.int32) // gs
    layer.g_idx.data.copy_(to_dev(g_idx, device))
    layer.process_weights_after_loading()
    assert layer.qweight.shape == (k // 16, 4 * n)
    w_ref = o.case_w_ref(case)
    for m in (1, 16, 32, 150):
        a = _acts(m, k, seed=m)
        check_gemm_close(layer(a.to(device)), o.gemm_ref(a, w_ref), f"gptq 8-bit g={group_size} act_order={desc_act} m={m}")


def _fp8_close(out, ref64, what):
    """Holds the result to 2 ulp of the output type + 2e-3 of the mean magnitude against an fp64 accumulation of the
    same quantised operands (bitwise parity of this GEMM is not pinned by any reference test)."""
    out64 = out.detach().cpu().double()
    assert torch.isfinite(out64).all(), what
    ulp = 2.0 ** -7 if out.dtype == torch.bfloat16 else 2.0 ** -10
    tol = 2 * ulp * ref64.abs() + 2e-3 * ref64.abs().mean()
    bad = (out64 - ref64).abs() > tol
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} elements out of tolerance, worst {(out64 - ref64).abs().max():.3e}"


def test_fp8_linear_method_from_16bit_checkpoint(device):
    """Fp8Config on a bf16 checkpoint: weight quantised per tensor at load (fp8.py:497-500), activations per token."""
    from vllm_amd.layers.linear import LinearBase
    from vllm_amd.layers.quantization import get_quantization_config
    k, n = 512, 384
    # a config dict with quant_method "fp8" announces an FP8 checkpoint (fp8.py:191-205); on-the-fly quantisation of a
    # 16-bit checkpoint is the config built without it
    cfg = get_quantization_config("fp8")(is_checkpoint_fp8_serialized=False, activation_scheme="dynamic")
    layer = LinearBase(k, n, quant_config=cfg, params_dtype=torch.bfloat16, bias=True, return_bias=False).to(device)
    w = (torch.randn(n, k, generator=torch.Generator().manual_seed(1)) * 0.02).to(torch.bfloat16)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(2)) * 0.01).to(torch.bfloat16)
    layer.weight.data.copy_(w.to(device))
    layer.bias.data.copy_(bias.to(device))
    layer.process_weights_after_loading()
    wq_ref, ws_ref = of.ref_dynamic_per_tensor_quant(w)
    assert layer.weight.dtype == torch.float8_e4m3fn and layer.weight.shape == (k, n)
    assert torch.equal(layer.weight.t().contiguous().cpu().view(torch.uint8), wq_ref.view(torch.uint8)), "weight codes"
    assert torch.equal(layer.weight_scale.cpu().reshape(()), ws_ref.reshape(())), "weight scale"
    for m in (1, 16, 100):
        a = _acts(m, k, seed=m)
        out = layer(a.to(device))
        aq, sa = of.ref_dynamic_per_token_quant(a)
        ref = of.scaled_mm_ref(aq, wq_ref.t(), sa, ws_ref, torch.float64, bias)
        _fp8_close(out, ref, f"fp8 method m={m}")


def test_fp8_linear_method_serialized_static_fused_shards(device):
    """FP8 checkpoint of a fused module: one weight scale and one input scale per logical shard; the method requantises
    to the largest weight scale and takes the largest input scale (fp8.py:517-570, w8a8_utils.py:105-156)."""
    from vllm_amd.layers.linear import MergedColumnParallelLinear
    from vllm_amd.layers.quantization import get_quantization_config
    k, sizes = 256, [128, 192]
    n = sum(sizes)
    cfg = get_quantization_config("fp8").from_config(dict(quant_method="fp8", activation_scheme="static"))
    assert cfg.is_checkpoint_fp8_serialized
    layer = MergedColumnParallelLinear(k, sizes, quant_config=cfg, params_dtype=torch.bfloat16, return_bias=False).to(device)
    g = torch.Generator().manual_seed(5)
    shards, scales = [], torch.tensor([0.011, 0.017], dtype=torch.float32)
    for i, width in enumerate(sizes):
        wf = torch.randn(width, k, generator=g) * (0.6 + 0.5 * i)
        shards.append(of.ref_static_quant(wf, scales[i]))
    wq = torch.cat(shards, dim=0)
    in_scales = torch.tensor([0.02, 0.015], dtype=torch.float32)
    layer.weight.data.copy_(wq.to(device))
    layer.weight_scale.data.copy_(scales.to(device))
    layer.input_scale.data.copy_(in_scales.to(device))
    layer.process_weights_after_loading()
    # oracle of the load-time transformation
    max_s = scales.max()
    deq = torch.cat([shards[i].to(torch.float32) * scales[i] for i in range(2)], dim=0)
    wq_ref = of.ref_static_quant(deq, max_s)
    assert torch.equal(layer.weight.t().contiguous().cpu().view(torch.uint8), wq_ref.view(torch.uint8))
    assert float(layer.weight_scale) == float(max_s) and float(layer.input_scale) == float(in_scales.max())
    for m in (3, 64):
        a = _acts(m, k, seed=m)
        out = layer(a.to(device))
        aq = of.ref_static_quant(a, in_scales.max())
        ref = of.scaled_mm_ref(aq, wq_ref.t(), in_scales.max(), max_s, torch.float64, None)
        _fp8_close(out, ref, f"fp8 static fused m={m}")


def test_fp8_linear_method_module_fused_on_disk(device):
    """An FP8 checkpoint whose qkv module is already fused: one weight tensor and ONE scalar scale arrive without a
    shard id.  The weight must be used as loaded with that scale (w8a8_utils.py:108-136 skips the requantisation)."""
    from vllm_amd.layers.linear import QKVParallelLinear
    from vllm_amd.layers.quantization import get_quantization_config
    k = 512
    cfg = get_quantization_config("fp8").from_config(dict(quant_method="fp8", activation_scheme="dynamic"))
    layer = QKVParallelLinear(k, 64, 4, 2, quant_config=cfg, params_dtype=torch.bfloat16, return_bias=False).to(device)
    n = sum(layer.output_sizes)
    g = torch.Generator().manual_seed(9)
    scale = torch.tensor(0.019)
    wq = of.ref_static_quant(torch.randn(n, k, generator=g) * 0.8, scale)
    layer.weight.weight_loader(layer.weight, wq.to(device))
    layer.weight_scale.weight_loader(layer.weight_scale, scale)
    layer.process_weights_after_loading()
    assert torch.equal(layer.weight.t().contiguous().cpu().view(torch.uint8), wq.view(torch.uint8)), "weight was requantised"
    assert float(layer.weight_scale) == float(scale)
    for m in (2, 50):
        a = _acts(m, k, seed=m)
        aq, sa = of.ref_dynamic_per_token_quant(a)
        ref = of.scaled_mm_ref(aq, wq.t(), sa, scale.reshape(1), torch.float64, None)
        _fp8_close(layer(a.to(device)), ref, f"fp8 fused on disk m={m}")


def test_layers_loaded_shard_by_shard_through_weight_loaders(device):
    """Checkpoint tensors enter the layers the way a model loader delivers them -- `param.weight_loader(param, tensor,
    shard_id)` per logical part, on a layer that already lives on the device (linear.py:820-866,:1009-1060) -- then
    `process_weights_after_loading` and a forward pass against the oracle of the concatenated layer."""
    from vllm_amd.layers.linear import MergedColumnParallelLinear, QKVParallelLinear
    from vllm_amd.layers.quantization import get_quantization_config
    k = 1024
    # GPTQ gate_up_proj from separate gate / up tensors
    sizes = [256, 192]
    cfg = get_quantization_config("gptq_marlin").from_config(dict(bits=4, group_size=128, desc_act=False, sym=True))
    layer = MergedColumnParallelLinear(k, sizes, quant_config=cfg, params_dtype=torch.bfloat16, return_bias=False).to(device)
    cases = [o.make_w4a16_case(k, n, 128, seed=80 + i) for i, n in enumerate(sizes)]
    for i, case in enumerate(cases):
        layer.qweight.weight_loader(layer.qweight, to_dev(case["qweight"], device), i)
        layer.scales.weight_loader(layer.scales, to_dev(case["scales"], device, torch.bfloat16), i)
        layer.qzeros.weight_loader(layer.qzeros, torch.full((k // 128, sizes[i] // 8), 0x77777777, dtype=torch.int32), i)
    layer.g_idx.weight_loader(layer.g_idx, torch.arange(k, dtype=torch.int32) // 128)
    layer.process_weights_after_loading()
    w_ref = torch.cat([o.case_w_ref(c) for c in cases], dim=1)
    for m in (1, 40, 150):
        a = _acts(m, k, seed=m)
        check_gemm_close(layer(a.to(device)), o.gemm_ref(a, w_ref), f"gptq merged from shards m={m}")
    # AWQ qkv_proj from q / k / v tensors
    hf = dict(quant_method="awq", bits=4, group_size=128, zero_point=True)
    qkv = QKVParallelLinear(k, 64, 4, 2, quant_config=get_quantization_config("awq_marlin").from_config(hf),
                            params_dtype=torch.float16, return_bias=False).to(device)
    cases = {sid: o.make_w4a16_case(k, n, 128, asym=True, dtype=torch.float16, seed=90 + i)
             for i, (sid, n) in enumerate(zip("qkv", qkv.output_sizes))}
    for sid, case in cases.items():
        qkv.qweight.weight_loader(qkv.qweight, to_dev(o.awq_pack(case["q"], 4), device), sid)
        qkv.qzeros.weight_loader(qkv.qzeros, to_dev(o.awq_pack(case["zp_vals"], 4), device), sid)
        qkv.scales.weight_loader(qkv.scales, to_dev(case["scales"], device, torch.float16), sid)
    qkv.process_weights_after_loading()
    w_ref = torch.cat([o.case_w_ref(cases[sid]) for sid in "qkv"], dim=1)
    for m in (2, 33):
        a = _acts(m, k, torch.float16, seed=m)
        check_gemm_close(qkv(a.to(device)), o.gemm_ref(a, w_ref), f"awq qkv from shards m={m}")
    # FP8 serialized gate_up_proj: per-part weights and scalar scales; requantised to the largest scale after loading
    fcfg = get_quantization_config("fp8").from_config(dict(quant_method="fp8", activation_scheme="dynamic"))
    f8 = MergedColumnParallelLinear(k, sizes, quant_config=fcfg, params_dtype=torch.bfloat16, return_bias=False).to(device)
    g = torch.Generator().manual_seed(6)
    scales = [torch.tensor(0.013), torch.tensor(0.021)]
    parts = [of.ref_static_quant(torch.randn(n, k, generator=g) * (0.5 + 0.6 * i), scales[i]) for i, n in enumerate(sizes)]
    for i in (1, 0):
        f8.weight.weight_loader(f8.weight, parts[i].to(device), i)
        f8.weight_scale.weight_loader(f8.weight_scale, scales[i], i)
    f8.process_weights_after_loading()
    max_s = torch.stack(scales).max()
    wq_ref = of.ref_static_quant(torch.cat([parts[i].float() * scales[i] for i in range(2)]), max_s)
    assert torch.equal(f8.weight.t().contiguous().cpu().view(torch.uint8), wq_ref.view(torch.uint8))
    a = _acts(20, k, seed=3)
    aq, sa = of.ref_dynamic_per_token_quant(a)          # the dynamic scheme quantises activations per token
    _fp8_close(f8(a.to(device)), of.scaled_mm_ref(aq, wq_ref.t(), sa, max_s.reshape(1), torch.float64, None),
               "fp8 merged from shards")


def test_ptpc_fp8_linear_method(device):
    """Per-token x per-channel (ptpc_fp8.py:82-137): bit-exact load-time weight quantisation, GEMM within tolerance."""
    from vllm_amd.layers.linear import LinearBase
    from vllm_amd.layers.quantization import get_quantization_config
    k, n = 1024, 320
    cfg = get_quantization_config("ptpc_fp8").from_config({})
    layer = LinearBase(k, n, quant_config=cfg, params_dtype=torch.bfloat16, return_bias=False).to(device)
    w = (torch.randn(n, k, generator=torch.Generator().manual_seed(7)) * 0.02).to(torch.bfloat16)
    layer.weight.data.copy_(w.to(device))
    layer.process_weights_after_loading()
    wq_ref, ws_ref = of.ref_dynamic_per_token_quant(w)
    assert torch.equal(layer.weight.t().contiguous().cpu().view(torch.uint8), wq_ref.view(torch.uint8))
    assert torch.equal(layer.weight_scale.cpu(), ws_ref)
    for m in (1, 40, 300):
        a = _acts(m, k, seed=m)
        out = layer(a.to(device))
        aq, sa = of.ref_dynamic_per_token_quant(a)
        _fp8_close(out, of.scaled_mm_ref(aq, wq_ref.t(), sa, ws_ref, torch.float64, None), f"ptpc m={m}")


# ------------------------------------------------------------------------------------------------ HIP graphs

@pytest.mark.parametrize("m", [4, 16, 96])
def test_layers_replay_in_a_hip_graph(device, m):
    """Capture a GPTQ layer (act_order: exercises the permute and split paths) and a PTPC FP8 layer in one HIP graph,
    replay it several times with eager work and synchronisations in between, and compare every replay with the eager
    result: the entry points must neither allocate behind the allocator's back nor record memset nodes."""
    from vllm_amd.layers.linear import LinearBase
    from vllm_amd.layers.quantization import get_quantization_config
    k = 3584            # 28 groups: the decode kernels split K for M > 4
    gptq, case, _ = _gptq_layer(device, k, [256], True, torch.bfloat16, seed=11)
    cfg = get_quantization_config("ptpc_fp8").from_config({})
    fp8 = LinearBase(256, 128, quant_config=cfg, params_dtype=torch.bfloat16, return_bias=False).to(device)
    fp8.weight.data.copy_((torch.randn(128, 256, generator=torch.Generator().manual_seed(1)) * 0.05).to(torch.bfloat16).to(device))
    fp8.process_weights_after_loading()

    static_in = torch.zeros(m, k, dtype=torch.bfloat16, device=device)

    def run():
        return fp8(gptq(static_in))

    inputs = [_acts(m, k, seed=s).to(device) for s in range(4)]
    eager = []
    for x in inputs:
        static_in.copy_(x)
        eager.append(run().clone())
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        static_in.copy_(inputs[0])
        run()                      # warm-up on the capture stream
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            static_out = run()
    torch.cuda.synchronize()
    for rep in range(2):
        for x, ref in zip(inputs, eager):
            static_in.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_out, ref), f"replay differs from eager (m={m}, repetition {rep})"
            # eager work between replays, as a serving loop would do
            assert torch.equal(run(), ref)
    assert bool((gptq.quant_method.kernel.workspace == 0).all()), "workspace counters not restored to zero"


# ------------------------------------------------------------------------------------------------ dispatcher checks

def test_custom_ops_pass_opcheck_on_device(device):
    """Schema and fake-tensor checks of the registered ops with real device arguments (the reference runs the same
    checks on its ops: tests/kernels/quantization/test_marlin_gemm.py:180-184,:334-352; test_fp8_quant.py:20-45)."""
    import vllm_amd._custom_ops as ops  # noqa: F401  (registers the ops)
    from vllm_amd.layers.quantization.utils import marlin_utils as mu
    from vllm_amd.scalar_type import scalar_types
    utils = ("test_schema", "test_faketensor")
    k, n, m = 256, 128, 8
    case = o.make_w4a16_case(k, n, 128, seed=0)
    qweight = to_dev(case["qweight"], device)
    empty = torch.empty(0, dtype=torch.int32, device=device)
    torch.library.opcheck(torch.ops.vllm_amd.gptq_marlin_repack, (qweight, empty, k, n, 4, 1), test_utils=utils)
    torch.library.opcheck(torch.ops.vllm_amd.awq_marlin_repack, (to_dev(o.awq_pack(case["q"], 4), device), k, n, 4, 0),
                          test_utils=utils)
    w = ops.gptq_marlin_repack(qweight, empty, k, n, 4)
    scales = to_dev(case["scales"], device, torch.bfloat16)
    a = _acts(m, k).to(device)
    ws = mu.marlin_make_workspace_new(device)
    torch.library.opcheck(torch.ops.vllm_amd.gptq_marlin_gemm,
                          (a, None, w, None, scales, None, empty, empty, empty, ws, scalar_types.uint4b8.id, m, n, k,
                           True, False, True, False), test_utils=utils)
    perm = torch.randperm(k, generator=torch.Generator().manual_seed(0)).to(torch.int32).to(device)
    torch.library.opcheck(torch.ops.vllm_amd.permute_cols, (a, perm), test_utils=utils)
    # ops with FP8 tensors: the schema checker compares mutated arguments with arithmetic torch lacks for float8, so
    # only the fake-tensor check applies
    utils = ("test_faketensor",)
    out = torch.empty(m, k, dtype=torch.float8_e4m3fn, device=device)
    sc = torch.empty(m, 1, dtype=torch.float32, device=device)
    torch.library.opcheck(torch.ops.vllm_amd.dynamic_per_token_scaled_fp8_quant, (out, a, sc, None), test_utils=utils)
    one = torch.ones(1, dtype=torch.float32, device=device)
    torch.library.opcheck(torch.ops.vllm_amd.static_scaled_fp8_quant, (out, a, one), test_utils=utils)
    torch.library.opcheck(torch.ops.vllm_amd.dynamic_scaled_fp8_quant, (out, a, torch.zeros(1, dtype=torch.float32, device=device)),
                          test_utils=utils)
    bq = torch.randn(n, k, device=device).to(torch.float8_e4m3fn).t()
    c = torch.empty(m, n, dtype=torch.bfloat16, device=device)
    sb = torch.ones(n, 1, dtype=torch.float32, device=device)
    torch.library.opcheck(torch.ops.vllm_amd.cutlass_scaled_mm, (c, out, bq, sc.fill_(1.0), sb, None), test_utils=utils)
    w = torch.ones(k, dtype=torch.bfloat16, device=device)
    torch.library.opcheck(torch.ops.vllm_amd.rms_norm_static_fp8_quant, (out, a, w, one, 1e-6), test_utils=utils)
    torch.library.opcheck(torch.ops.vllm_amd.fused_add_rms_norm_static_fp8_quant, (out, a, a.clone(), w, one, 1e-6),
                          test_utils=utils)
    torch.library.opcheck(torch.ops.vllm_amd.rms_norm_dynamic_per_token_quant, (out, a, w, sc, 1e-6, None, a.clone()),
                          test_utils=utils)
    half = torch.empty(m, k // 2, dtype=torch.float8_e4m3fn, device=device)
    torch.library.opcheck(torch.ops.vllm_amd.silu_and_mul_quant, (half, a, one), test_utils=utils)
