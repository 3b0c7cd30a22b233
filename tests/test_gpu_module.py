"""Front-door tests on the GPU, modelled on the reference's own WOQ tests
(tests/cpu/test_quantization_default_recipe.py:261-2227, tests/cpu/test_ipex_llm_quantization.py):
build the module the way a user does, compare with matmul on the dequantized weight."""
import copy
import os
import pickle

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _ipex():
    import ipex_amd

    return ipex_amd


@pytest.mark.parametrize("weight_dtype,group_size,lowp", [
    ("INT8", -1, "NONE"), ("INT8", -1, "BF16"), ("INT4", -1, "BF16"), ("INT4", 128, "BF16"), ("INT4", 32, "BF16"),
    ("INT4", 64, "FP16"), ("INT4", 128, "INT8"), ("INT8", -1, "INT8"),
    ("NF4", 64, "BF16"), ("NF4", -1, "NONE"), ("NF4", 32, "FP16"), ("NF4", 128, "INT8"),
])
@pytest.mark.parametrize("M", [1, 4, 33, 196])
def test_prepare_convert_matches_dequantized_matmul(cuda, weight_dtype, group_size, lowp, M):
    ipex = _ipex()
    q = ipex.quantization
    torch.manual_seed(0)
    K, N = 512, 272
    lin = torch.nn.Linear(K, N, bias=True).to(torch.bfloat16)
    model = torch.nn.Sequential(lin).eval()
    qmap = q.get_weight_only_quant_qconfig_mapping(
        weight_dtype=getattr(q.WoqWeightDtype, weight_dtype),
        lowp_mode=getattr(q.WoqLowpMode, lowp),
        act_quant_mode=q.WoqActQuantMode.PER_BATCH_IC_BLOCK_SYM,
        group_size=group_size,
    )
    w_float = lin.weight.detach().float().clone()
    qmodel = q.convert(q.prepare(copy.deepcopy(model).to(cuda), qmap, inplace=True), inplace=True)
    woq = qmodel[0]
    assert type(woq).__name__ == "WeightOnlyQuantizedLinear"
    assert woq.weight.is_cuda and woq.weight.dtype == torch.uint8
    x = torch.randn(M, K).to(torch.bfloat16)
    y = qmodel(x.to(cuda)).float().cpu()
    # expected: quantize with the same helpers, dequantize, matmul in fp32
    dt = getattr(q.WoqWeightDtype, weight_dtype)
    sym = qmap.global_qconfig.weight_qscheme == q.WoqWeightQScheme.SYMMETRIC
    if group_size == -1:
        qw, s, z = q.quantize_per_channel(w_float, dt, None, None, sym)
        dq = q.dequantize_per_channel(qw, s, z, dt, [N, K])
    else:
        qw, s, z = q.quantize_per_block(w_float, dt, group_size, None, None, sym)
        dq = q.dequantize_per_block(qw, s, z, dt, group_size, [N, K])
    ref = x.float() @ dq.t() + lin.bias.float()
    tol = 5e-2 if lowp == "INT8" else 2e-2
    assert torch.allclose(y, ref, atol=tol, rtol=2e-2), float((y - ref).abs().max())
    # context accessors return the un-permuted, un-padded parameters and the plain weight
    ctx = woq._op_context
    assert torch.equal(ctx.to_public(ctx.get_weight()).cpu(), qw)
    assert torch.equal(ctx.get_scales().cpu(), s.float())
    assert ctx.get_weight_shape() == [N, K]
    if z is not None:
        assert torch.equal(ctx.get_zero_points().cpu(), z.float())


@pytest.mark.parametrize("weight_dtype,group_size", [(None, -1), ("INT4", 128), ("NF4", 64)])
@pytest.mark.parametrize("M", [1, 70])
def test_default_qconfig_on_an_fp32_model_computes_in_fp32(cuda, weight_dtype, group_size, M):
    """get_weight_only_quant_qconfig_mapping() defaults to INT8 weights and lowp_mode NONE
    (quantization/_qconfig.py:188-196); on an fp32 model that is fp32 compute."""
    ipex = _ipex()
    q = ipex.quantization
    torch.manual_seed(1)
    K, N = 384, 100
    lin = torch.nn.Linear(K, N, bias=True)
    model = torch.nn.Sequential(lin).eval()
    if weight_dtype is None:
        qmap = q.get_weight_only_quant_qconfig_mapping()
        dt = q.WoqWeightDtype.INT8
    else:
        dt = getattr(q.WoqWeightDtype, weight_dtype)
        qmap = q.get_weight_only_quant_qconfig_mapping(weight_dtype=dt, group_size=group_size)
    assert qmap.global_qconfig.lowp_mode == q.WoqLowpMode.NONE
    w_float = lin.weight.detach().clone()
    qmodel = q.convert(q.prepare(copy.deepcopy(model).to(cuda), qmap, inplace=True), inplace=True)
    x = torch.randn(2, M, K)
    y = qmodel(x.to(cuda))
    assert y.dtype == torch.float32 and tuple(y.shape) == (2, M, N)
    sym = qmap.global_qconfig.weight_qscheme == q.WoqWeightQScheme.SYMMETRIC
    if group_size == -1:
        qw, s, z = q.quantize_per_channel(w_float, dt, None, None, sym)
        dq = q.dequantize_per_channel(qw, s, z, dt, [N, K])
    else:
        qw, s, z = q.quantize_per_block(w_float, dt, group_size, None, None, sym)
        dq = q.dequantize_per_block(qw, s, z, dt, group_size, [N, K])
    ref = (x.double() @ dq.double().t() + lin.bias.double()).float()
    assert torch.allclose(y.cpu(), ref, atol=1e-5, rtol=1e-5), float((y.cpu() - ref).abs().max())


@pytest.mark.parametrize("M", [4, 1024])
@pytest.mark.parametrize("has_bias", [True, False])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fp8_weight_through_from_float_and_qweight(cuda, M, has_bias, dtype):
    """The reference's own FP8 test (tests/cpu/test_quantization_default_recipe.py:2155-2226), same shapes,
    recipe, expected value and tolerance: group-wise absmax / 448 scales, weight / scale as float8 e4m3fn,
    compared with matmul on the dequantized weight in the compute dtype (fp16 for bf16 rows up to 4)."""
    ipex = _ipex()
    q = ipex.quantization
    from ipex_amd.nn.modules import WeightOnlyQuantizedLinear

    torch.manual_seed(2)
    K = N = 1024
    group_size = 128
    lin = torch.nn.Linear(K, N, has_bias).eval()
    data = torch.rand(M, K).to(dtype) * 0.1
    weight = lin.weight.detach()
    grouped = weight.view(N, K // group_size, group_size)
    w_scales = grouped.abs().max(-1)[0] / 448.0
    w_fp8 = (grouped / w_scales.unsqueeze(-1)).view(N, K).to(torch.float8_e4m3fn)
    w_dq = (w_fp8.view(N, K // group_size, group_size).float() * w_scales.unsqueeze(-1)).view(N, K)
    compute_dtype = torch.half if (dtype == torch.bfloat16 and M <= 4) else dtype
    w_dq = w_dq.to(compute_dtype)
    out1 = torch.matmul(data.to(compute_dtype).float(), w_dq.float().T).to(compute_dtype)
    out1 = (out1 + lin.bias.detach()) if has_bias else out1.float()
    lowp = q.WoqLowpMode.BF16 if dtype == torch.bfloat16 else q.WoqLowpMode.NONE
    qmap = q.get_weight_only_quant_qconfig_mapping(weight_dtype=q.WoqWeightDtype.FP8, lowp_mode=lowp)
    with torch.no_grad():
        lin.qconfig = qmap.global_qconfig
        woq = WeightOnlyQuantizedLinear.from_float_and_qweight(
            lin, w_fp8.to(cuda), q.WoqWeightDtype.FP8, w_scales, None, lin.bias, group_size
        )
        assert woq.weight is not None and woq.weight.dtype == torch.float8_e4m3fn
        out2 = woq(data.to(cuda)).float().cpu()
    torch.testing.assert_close(out1.float(), out2, atol=1e-3, rtol=1e-3)
    ctx = woq._op_context
    assert torch.equal(ctx.to_public(ctx.get_weight()).view(torch.uint8).cpu(), w_fp8.view(torch.uint8))
    # the registered context pickles with its float8 weight and gives the same output afterwards
    ctx2 = pickle.loads(pickle.dumps(ctx))
    assert ctx2.get_weight().dtype == torch.float8_e4m3fn
    y2 = torch.ops.torch_ipex.ipex_woq_linear(data.to(cuda), ctx2.get_data_handle())
    assert torch.equal(y2.float().cpu(), out2)


def test_all_zero_bias_is_dropped_and_weight_emptied(cuda):
    ipex = _ipex()
    q = ipex.quantization
    lin = torch.nn.Linear(256, 64, bias=True).to(cuda)
    with torch.no_grad():
        lin.bias.zero_()
    lin.qconfig = q.get_weight_only_quant_qconfig_mapping(weight_dtype=q.WoqWeightDtype.INT4).global_qconfig
    woq = ipex.nn.modules.WeightOnlyQuantizedLinear.from_float(lin)
    assert woq.bias is False and woq._op_context.get_bias() is None
    assert lin.weight.numel() == 0


def test_awq_fixture_through_llm_front_door(cuda):
    """The reference's own AutoAWQ tensors (tests/cpu/test_ipex_llm_quantization.py:112-151),
    checked against an independent decode at the reference's precision (0.1) and tighter."""
    ipex = _ipex()
    d = torch.load(os.path.join(GOLDEN, "awq_fixture.pt"), weights_only=True)
    K, N, G = 768, 2304, 128
    order = [0, 2, 4, 6, 1, 3, 5, 7]
    qw = d["qweight"].numpy().astype(np.int64) & 0xFFFFFFFF
    qz = d["qzeros"].numpy().astype(np.int64) & 0xFFFFFFFF
    w = np.zeros((K, N), dtype=np.int64)
    z = np.zeros((K // G, N), dtype=np.int64)
    for i in range(8):
        w[:, order[i]::8] = (qw >> (4 * i)) & 0xF
        z[:, order[i]::8] = (qz >> (4 * i)) & 0xF
    sc = d["scales"].float().numpy()
    g = np.arange(K) // G
    dq = ((w - z[g]) * sc[g]).astype(np.float32)  # [K, N]
    act = d["act"]
    ref = act.float().numpy() @ dq + d["bias"].float().numpy()
    lm = ipex.llm.quantization
    lin = lm.IPEXWeightOnlyQuantizedLinear.from_weight(
        d["qweight"], d["scales"], d["qzeros"], K, N, None, d["bias"], G, None, lm.QuantMethod.AWQ_GEMM,
        lm.QuantDtype.INT4,
    )
    y = lin(act.to(cuda)).float().cpu().numpy()
    assert np.max(np.abs(y - ref)) < 0.1
    assert np.linalg.norm(y - ref) / np.linalg.norm(ref) < 4e-3  # bf16 weights + bf16 output rounding


def test_gptq_checkpoint_through_llm_front_door(cuda):
    ipex = _ipex()
    gen = torch.Generator().manual_seed(3)
    K, N, G = 512, 256, 128
    q = torch.randint(0, 16, (K, N), generator=gen)  # [K, N]
    zp = torch.randint(0, 16, (K // G, N), generator=gen)
    scales = (0.005 + 0.015 * torch.rand(K // G, N, generator=gen)).half()
    qv = q.view(K // 8, 8, N)
    qweight = torch.zeros(K // 8, N, dtype=torch.int64)
    for i in range(8):
        qweight |= qv[:, i, :] << (4 * i)
    qweight = (qweight - (qweight >= 2**31) * 2**32).to(torch.int32)
    zv = ((zp - 1) % 16).view(K // G, N // 8, 8)
    qzeros = torch.zeros(K // G, N // 8, dtype=torch.int64)
    for i in range(8):
        qzeros |= zv[:, :, i] << (4 * i)
    qzeros = (qzeros - (qzeros >= 2**31) * 2**32).to(torch.int32)
    lm = ipex.llm.quantization
    lin = lm.IPEXWeightOnlyQuantizedLinear.from_weight(qweight, scales, qzeros, K, N, None, None, G)
    x = torch.randn(7, K, generator=gen).to(torch.bfloat16)
    y = lin(x.to(cuda)).float().cpu()
    gidx = torch.arange(K) // G
    dq = (q - zp[gidx]).float() * scales.float()[gidx]
    ref = x.float() @ dq
    assert torch.allclose(y, ref, atol=3e-2, rtol=2e-2)


class _TinyLM(torch.nn.Module):
    def __init__(self, K, H, N, V):
        super().__init__()
        self.norm = torch.nn.LayerNorm(K)
        self.block = torch.nn.ModuleDict({"up": torch.nn.Linear(K, H, bias=False), "down": torch.nn.Linear(H, N, bias=True)})
        self.lm_head = torch.nn.Linear(N, V, bias=False)

    def forward(self, x):
        return self.lm_head(self.block["down"](torch.nn.functional.silu(self.block["up"](self.norm(x)))))


@pytest.mark.parametrize("method", ["gptq", "gptq_act_order", "awq", "fp8", "int8"])
def test_model_from_low_precision_checkpoint(cuda, method):
    """A whole model from a checkpoint's state dict, as ipex.llm.optimize(low_precision_checkpoint=...) builds it
    (utils/weight_only_quantization.py:224-376): quantized linears from the checkpoint's tensors, the floating-point
    lm_head and the LayerNorm parameters loaded as they are; against the same model on the dequantized weights."""
    import checkpoints as C
    ipex = _ipex()
    q = ipex.quantization
    from ipex_amd.utils.weight_only_quantization import _convert_woq_with_low_precision_checkpoint

    gen = torch.Generator().manual_seed(11)
    K, H, N, V, G = 256, 512, 128, 64, 64
    sd = {"norm.weight": 1 + 0.1 * torch.randn(K, generator=gen), "norm.bias": 0.1 * torch.randn(K, generator=gen),
          "lm_head.weight": 0.05 * torch.randn(V, N, generator=gen)}
    dense = {}
    quant_config = {"quant_method": method.split("_")[0]}
    for name, (n_out, n_in) in {"block.up": (H, K), "block.down": (N, H)}.items():
        if method in ("gptq", "gptq_act_order", "awq"):
            codes = torch.randint(0, 16, (n_out, n_in), generator=gen)
            zp = torch.randint(0, 16, (n_out, n_in // G), generator=gen)
            sc = (0.002 + 0.006 * torch.rand(n_out, n_in // G, generator=gen)).half()
            if method == "gptq_act_order":
                g_idx = (torch.randperm(n_in, generator=gen) // G).to(torch.int32)
                dense[name] = (codes - zp[:, g_idx.long()]).float() * sc.float()[:, g_idx.long()]
                sd[name + ".g_idx"] = g_idx
            else:
                dense[name] = C.int4_dequant(codes, zp, sc, G)
            qw, s2, qz = (C.awq_layer if method == "awq" else C.gptq_layer)(codes, zp, sc)
            sd.update({name + ".qweight": qw, name + ".scales": s2, name + ".qzeros": qz})
        elif method == "fp8":
            w8, sinv, dq = C.fp8_layer(0.05 * torch.randn(n_out, n_in, generator=gen), 128, 128)
            sd.update({name + ".weight": w8, name + ".weight_scale_inv": sinv})
            dense[name] = dq
            quant_config["weight_block_size"] = [128, 128]
        else:
            w8 = torch.randint(-127, 128, (n_out, n_in), generator=gen, dtype=torch.int8)
            sc = 0.0005 + 0.001 * torch.rand(n_out, 1, generator=gen)
            sd.update({name + ".weight": w8, name + ".weight_scale": sc})
            dense[name] = w8.float() * sc
    sd["block.down.bias"] = 0.1 * torch.randn(N, generator=gen)
    for k in ("norm.weight", "norm.bias", "lm_head.weight", "block.down.bias"):  # a bf16 checkpoint
        sd[k] = sd[k].to(torch.bfloat16)
    model = _TinyLM(K, H, N, V).eval()
    qmap = q.get_weight_only_quant_qconfig_mapping(weight_dtype=q.WoqWeightDtype.INT4, lowp_mode=q.WoqLowpMode.BF16)
    sd_gpu = {k: v.to(cuda) for k, v in sd.items()}
    woq = _convert_woq_with_low_precision_checkpoint(copy.deepcopy(model).to(cuda).to(torch.bfloat16), qmap, sd_gpu,
                                                     quant_config, inplace=True)
    assert type(woq.block["up"]).__name__ == "WeightOnlyQuantizedLinear" and type(woq.block["down"]).__name__ == "WeightOnlyQuantizedLinear"
    assert isinstance(woq.lm_head, torch.nn.Linear) and torch.equal(woq.lm_head.weight.cpu(), sd["lm_head.weight"])
    assert torch.equal(woq.norm.weight.cpu(), sd["norm.weight"])
    # the same model on the dequantized weights, in fp32
    ref = copy.deepcopy(model)
    ref.load_state_dict({"norm.weight": sd["norm.weight"].float(), "norm.bias": sd["norm.bias"].float(),
                         "lm_head.weight": sd["lm_head.weight"].float(), "block.up.weight": dense["block.up"],
                         "block.down.weight": dense["block.down"], "block.down.bias": sd["block.down.bias"].float()})
    for M in (3, 70):
        x = torch.randn(M, K, generator=gen)
        with torch.no_grad():
            want = ref(x)
            got = woq(x.to(cuda).to(torch.bfloat16)).float().cpu()
        err = float((got - want).norm() / want.norm())
        assert err < 2e-2, (method, M, err)


def test_context_pickle_roundtrip(cuda):
    from ipex_amd.utils import synthetic
    from helpers import make_context

    case = synthetic.make_int4_case(30, 3, 512, 80, 128, bias=True)
    ctx = make_context(case, 2)
    x = case["x"].to(cuda)
    y0 = ctx.run(x)
    ctx2 = pickle.loads(pickle.dumps(ctx))
    assert torch.equal(ctx2.run(x), y0)
    assert torch.equal(ctx2.to_public(ctx2.get_weight()).cpu(), case["qweight"])
    assert ctx2.get_data_handle().item() != ctx.get_data_handle().item()


def test_stale_handle_raises(cuda):
    from ipex_amd.utils import synthetic
    from helpers import make_torch_context

    case = synthetic.make_int4_case(31, 1, 256, 32, 128)
    ctx = make_torch_context(case, 2)
    handle = ctx.get_data_handle()
    x = case["x"].to(cuda)
    torch.ops.torch_ipex.ipex_woq_linear(x, handle)
    del ctx
    with pytest.raises(RuntimeError, match="no longer exists"):
        torch.ops.torch_ipex.ipex_woq_linear(x, handle)
    with pytest.raises(RuntimeError, match="GPU"):
        torch.ops.torch_ipex.ipex_woq_linear(x.cpu(), handle)


def test_context_free_op_matches_module(cuda):
    """ipex_prepack::woq_linear_pack_weight -> unpack round trip and torch_ipex::woq_linear
    (tests/cpu/test_quantization_default_recipe.py:1805-1901)."""
    from ipex_amd.utils import synthetic
    from helpers import make_context

    for lowp, M in ((2, 3), (2, 20), (3, 9)):
        case = synthetic.make_int4_case(32, M, 512, 96, 128, bias=True)
        ctx = make_context(case, lowp, 6 if lowp == 3 else -1)
        x = case["x"].to(cuda)
        packed, scales, zeros, bias, comp = torch.ops.ipex_prepack.woq_linear_pack_weight(
            case["qweight"].to(cuda), "int4", [96, 512], case["scales"].to(cuda), case["zeros"].to(cuda),
            case["bias"].to(cuda), None, 128, lowp,
        )
        back = torch.ops.ipex_prepack.woq_linear_unpack_weight(packed, "int4", [96, 512], lowp)
        assert torch.equal(back.cpu(), case["qweight"])
        y = torch.ops.torch_ipex.woq_linear(
            x, packed, "int4", [96, 512], scales, zeros, bias, None, 128, lowp, 6 if lowp == 3 else -1, comp
        )
        want = ctx.run(x)
        # the context-free op has no decode-kernel parameters, so M < 5 takes the general kernel
        assert torch.allclose(y.float(), want.float(), atol=2e-2, rtol=1e-2)
    with pytest.raises(RuntimeError, match="Unsupported weight dtype"):
        torch.ops.torch_ipex.woq_linear(x, packed, "int3", [96, 512], scales, zeros, bias, None, 128, 2, -1, None)


def test_context_free_op_rejects_tensors_it_could_not_read(cuda):
    """torch_ipex::woq_linear hands its tensor arguments to the kernels as raw device pointers: a tensor on the CPU, of
    another dtype or of a size that does not fit [N, K] and the group size must raise, not reach a kernel."""
    from ipex_amd.utils import synthetic

    case = synthetic.make_int4_case(34, 6, 512, 96, 128, bias=True)
    x = case["x"].to(cuda)
    packed, scales, zeros, bias, comp = torch.ops.ipex_prepack.woq_linear_pack_weight(
        case["qweight"].to(cuda), "int4", [96, 512], case["scales"].to(cuda), case["zeros"].to(cuda),
        case["bias"].to(cuda), None, 128, 2,
    )
    call = lambda **kw: torch.ops.torch_ipex.woq_linear(
        kw.get("x", x), kw.get("packed", packed), "int4", kw.get("shape", [96, 512]), kw.get("scales", scales),
        kw.get("zeros", zeros), kw.get("bias", bias), None, kw.get("G", 128), 2, -1, None)
    call()
    cpu_list = lambda ts, i: [t.cpu() if j == i else t for j, t in enumerate(ts)]
    with pytest.raises(RuntimeError, match="same device"):
        call(packed=packed.cpu())
    for i in range(3):
        with pytest.raises(RuntimeError, match="same device"):
            call(scales=cpu_list(scales, i))
    with pytest.raises(RuntimeError, match="same device"):
        call(zeros=cpu_list(zeros, 3))
    with pytest.raises(RuntimeError, match="same device"):
        call(bias=cpu_list(bias, 0))
    with pytest.raises(RuntimeError, match="packed weight has"):
        call(shape=[192, 512])  # twice the rows the packed tensor holds
    with pytest.raises(RuntimeError, match="packed weight has"):
        call(packed=packed.reshape(-1)[:-1024])
    with pytest.raises(RuntimeError, match=r"scales\[1\] must be"):
        call(scales=[scales[0], scales[1].float(), scales[2]])
    with pytest.raises(RuntimeError, match=r"scales\[0\] must be"):
        call(G=64)  # twice the groups the tables hold
    with pytest.raises(RuntimeError, match=r"zeros\[3\] must be uint8"):
        call(zeros=[zeros[0], zeros[1], zeros[2], zeros[3].to(torch.int32)])
    with pytest.raises(RuntimeError, match="bias has"):
        call(bias=[b[:50] for b in bias])
    with pytest.raises(RuntimeError, match="weight_shape must be positive"):
        call(shape=[0, 512], x=x)
    # a post-op operand on the CPU is rejected by the context's operators as well
    from helpers import make_torch_context

    tctx = make_torch_context(case, 2)
    other = torch.zeros(6, 96, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="same device"):
        torch.ops.torch_ipex.woq_linear_add(x, tctx.get_data_handle(), [other])
    torch.ops.torch_ipex.woq_linear_add(x, tctx.get_data_handle(), [other.to(cuda)])


def test_handles_of_the_two_bindings_do_not_cross(cuda):
    """The ctypes twin (ipex_amd.ops) and the registered custom class number their contexts apart: a handle of one kind
    given to an operator of the other raises instead of resolving to some live context of that kind."""
    from ipex_amd import ops
    from ipex_amd.utils import synthetic
    from helpers import make_context, make_torch_context

    case = synthetic.make_int4_case(35, 3, 256, 32, 128)
    twin, registered = make_context(case, 2), make_torch_context(case, 2)
    x = case["x"].to(cuda)
    assert twin.get_data_handle().item() < 0 < registered.get_data_handle().item()
    with pytest.raises(RuntimeError, match="does not come from"):
        torch.ops.torch_ipex.ipex_woq_linear(x, twin.get_data_handle())
    with pytest.raises(RuntimeError, match="belongs to a torch.classes"):
        ops.ipex_woq_linear(x, registered.get_data_handle())
    assert torch.equal(ops.ipex_woq_linear(x, twin.get_data_handle()),
                       torch.ops.torch_ipex.ipex_woq_linear(x, registered.get_data_handle()))


def test_k_mismatch_and_bad_arguments(cuda):
    from ipex_amd import ops
    from ipex_amd.utils import synthetic
    from helpers import make_context

    case = synthetic.make_int4_case(33, 2, 256, 32, 128)
    ctx = make_context(case, 2)
    with pytest.raises(RuntimeError, match="input and weight shapes do not match"):
        ctx.run(torch.zeros(2, 128, dtype=torch.bfloat16, device=cuda))
    with pytest.raises(RuntimeError, match="zero points must be integers"):
        ops.WoqLinearOpContext(case["qweight"].to(cuda), 2, [32, 256], case["scales"].to(cuda),
                               case["zeros"].to(cuda) + 0.5, None, None, None, 128, 2, -1)
    with pytest.raises(RuntimeError, match="g_idx"):
        ops.WoqLinearOpContext(case["qweight"].to(cuda), 2, [32, 256], case["scales"].to(cuda),
                               case["zeros"].to(cuda), None, torch.zeros(256, dtype=torch.int32), None, 128, 2, -1)
    with pytest.raises(RuntimeError, match="symmetric quantization is required"):
        ops.WoqLinearOpContext(torch.zeros(32, 256, dtype=torch.int8, device=cuda), 1, [32, 256],
                               torch.ones(32, device=cuda), torch.zeros(32, device=cuda), None, None, None, -1, 3, 6)


def test_weight_cache_flag_keeps_a_dense_copy_and_changes_no_result(cuda):
    """cache_weight_for_large_batch (tests/cpu/test_quantization_default_recipe.py:1522-1579): under lowp_mode BF16
    the context keeps a dequantized bf16 copy of the weight (get_cached_weight), made again when a pickled context
    is loaded; results with and without it are bit-identical, through both bindings, below and above the batch size
    from which the copy is used."""
    from ipex_amd import _lib
    from ipex_amd.utils import synthetic
    from helpers import make_context, make_torch_context

    case = synthetic.make_int4_case(34, 640, 512, 8192, 128, bias=True)
    x = case["x"].to(cuda)
    plain = make_context(case, 2)
    y_plain = plain.run(x)
    assert plain.get_cached_weight() is None and _lib.last_kernel() == "woq_gemm_w4_kernel"
    cached = make_context(case, 2, cache=True)
    assert tuple(cached.get_cached_weight().shape) == (4, 512, 4, 64, 8)
    assert torch.equal(cached.run(x), y_plain) and _lib.last_kernel() == "woq_gemm_dense_kernel"
    assert torch.equal(cached.run(x[:80]), plain.run(x[:80]))
    again = pickle.loads(pickle.dumps(cached))
    assert again.cache_weight_for_large_batch_ is True
    assert torch.equal(again.get_cached_weight(), cached.get_cached_weight())
    tc = make_torch_context(case, 2, cache=True)
    assert torch.equal(tc.get_cached_weight(), cached.get_cached_weight())
    assert torch.equal(torch.ops.torch_ipex.ipex_woq_linear(x, tc.get_data_handle()), y_plain)
    assert _lib.last_kernel() == "woq_gemm_dense_kernel"
    assert torch.equal(torch.ops.torch_ipex.ipex_woq_linear(x[:80], tc.get_data_handle()), plain.run(x[:80]))
    tc2 = pickle.loads(pickle.dumps(tc))
    assert torch.equal(tc2.get_cached_weight(), cached.get_cached_weight())
    assert torch.equal(torch.ops.torch_ipex.ipex_woq_linear(x, tc2.get_data_handle()), y_plain)
    assert make_torch_context(case, 2).get_cached_weight() is None
    assert make_torch_context(case, 3, act_quant_mode=6, cache=True).get_cached_weight() is None


def test_fused_ops_through_torch_ops(cuda):
    from ipex_amd.utils import synthetic
    from helpers import make_torch_context

    case = synthetic.make_int4_case(35, 6, 256, 48, 128, bias=True)
    ctx = make_torch_context(case, 2)
    h = ctx.get_data_handle()
    x = case["x"].to(cuda)
    base = torch.ops.torch_ipex.ipex_woq_linear(x, h)
    o = torch.randn(6, 48, device=cuda).bfloat16()
    assert torch.equal(torch.ops.torch_ipex.woq_linear_add(x, h, [o]), (base.float() + o.float()).bfloat16())
    assert torch.equal(torch.ops.torch_ipex.woq_linear_mul(x, h, [o]), (base.float() * o.float()).bfloat16())
    assert torch.equal(torch.ops.torch_ipex.woq_linear_relu(x, h), torch.relu(base))
    got = torch.ops.torch_ipex.woq_linear_silu(x, h)
    assert torch.allclose(got.float(), torch.nn.functional.silu(base.float()), atol=2e-2, rtol=2e-2)


# ---------------------------------------------------------------------------------------------
# ipex.llm.modules linear fusions over WOQ linears
# ---------------------------------------------------------------------------------------------
def _woq_module(ipex, K, N, weight_dtype="INT4", group_size=128, lowp="BF16", bias=True, seed=0, device="cuda"):
    q = ipex.quantization
    torch.manual_seed(seed)
    lin = torch.nn.Linear(K, N, bias=bias).to(torch.bfloat16)
    qmap = q.get_weight_only_quant_qconfig_mapping(
        weight_dtype=getattr(q.WoqWeightDtype, weight_dtype), lowp_mode=getattr(q.WoqLowpMode, lowp),
        group_size=group_size,
    )
    model = torch.nn.Sequential(lin).eval().to(device)
    return q.convert(q.prepare(model, qmap, inplace=True), inplace=True)[0]


@pytest.mark.parametrize("M", [3, 40, 150])
def test_llm_linear_fusion_modules_match_unfused_composition(cuda, M):
    """Each fusion module against the same WOQ linear followed by the torch elementwise op
    (the reference's fallback branch, fusions/linear_fusion.py:63-64 and siblings)."""
    ipex = _ipex()
    F = torch.nn.functional
    mods = ipex.llm.modules
    K, N = 512, 272
    woq = _woq_module(ipex, K, N)
    torch.manual_seed(M)
    x = torch.randn(M, K).to(torch.bfloat16).to(cuda)
    y = torch.randn(M, N).to(torch.bfloat16).to(cuda)
    z = torch.randn(M, N).to(torch.bfloat16).to(cuda)
    base = woq(x)

    def close(a, b):
        assert a.dtype == b.dtype and a.shape == b.shape
        assert torch.allclose(a.float(), b.float(), atol=2e-2, rtol=2e-2), float((a.float() - b.float()).abs().max())

    close(mods.LinearSilu(woq)(x), F.silu(base))
    close(mods.LinearRelu(woq)(x), F.relu(base))
    close(mods.LinearGelu(woq)(x), F.gelu(base))
    close(mods.LinearNewGelu(woq)(x), F.gelu(base, approximate="tanh"))
    close(mods.LinearMul(woq)(x, y), base * y)
    close(mods.LinearAdd(woq)(x, y), base + y)
    close(mods.LinearAddAdd(woq)(x, y, z), base + y + z)
    close(mods.LinearSiluMul(woq)(x, y), F.silu(base) * y)
    up = _woq_module(ipex, K, N, seed=1)
    close(mods.Linear2SiluMul(woq, up)(x), F.silu(base) * up(x))
    # a module that is not a WOQ linear takes the unfused path
    plain = torch.nn.Linear(K, N).to(torch.bfloat16).to(cuda)
    close(mods.LinearSilu(plain)(x), F.silu(plain(x)))
    close(mods.Linear2SiluMul(plain, up)(x), F.silu(plain(x)) * up(x))


@pytest.mark.parametrize("weight_dtype,group_size,lowp", [("INT4", 128, "BF16"), ("INT4", 32, "INT8"), ("INT8", -1, "BF16"), ("NF4", 64, "BF16")])
@pytest.mark.parametrize("M", [1, 7, 70])
def test_concat_linear_equals_the_separate_linears(cuda, weight_dtype, group_size, lowp, M):
    ipex = _ipex()
    K = 512
    outs = (256, 64, 80)
    lins = [_woq_module(ipex, K, n, weight_dtype, group_size, lowp, bias=(i != 1), seed=10 + i) for i, n in enumerate(outs)]
    torch.manual_seed(M)
    x = torch.randn(2, M, K).to(torch.bfloat16).to(cuda)
    want = [lin(x) for lin in lins]
    cat = ipex.llm.modules.ConcatLinear(lins)
    assert cat.concat_linear is not None and cat.concat_linear.out_features == sum(outs)
    assert not hasattr(cat, "linear_0")
    got = cat(x)
    assert len(got) == 3
    for g, w in zip(got, want):
        assert g.shape == w.shape
        if lowp == "INT8":
            # per-tensor activation statistics do not depend on N: same quantized activations, same sums
            assert torch.allclose(g.float(), w.float(), atol=1e-2, rtol=1e-2)
        else:
            assert torch.equal(g, w)
    # the merged context holds the concatenation of the stored codes and parameters
    ctx = cat.concat_linear._op_context
    assert torch.equal(ctx.to_public(ctx.get_weight()), torch.cat([l._op_context.to_public(l._op_context.get_weight()) for l in lins], 0))
    assert torch.equal(ctx.get_scales(), torch.cat([l._op_context.get_scales() for l in lins], 0))


def test_concat_linear_falls_back_when_the_linears_differ(cuda):
    ipex = _ipex()
    a = _woq_module(ipex, 256, 64, "INT4", 128)
    b = _woq_module(ipex, 256, 32, "INT4", 64, seed=3)
    cat = ipex.llm.modules.ConcatLinear([a, b])
    assert cat.concat_linear is None
    x = torch.randn(5, 256).to(torch.bfloat16).to(cuda)
    ya, yb = cat(x)
    assert torch.equal(ya, a(x)) and torch.equal(yb, b(x))
    plain = torch.nn.Linear(256, 16).to(torch.bfloat16).to(cuda)
    cat2 = ipex.llm.modules.ConcatLinear([a, plain])
    assert cat2.concat_linear is None and len(cat2(x)) == 2


# ---------------------------------------------------------------------------------------------
# mixture of experts over WOQ linears (torch_ipex::mixtral_moe_woq / deepseek_moe_woq)
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("H", [128, 100])  # 16-byte chunks / element by element
def test_moe_gather_and_weighted_scatter_bit_exact(cuda, dtype, H):
    from ipex_amd import _kernels
    from oracle import woq_oracle as O

    name = {torch.bfloat16: "bf16", torch.float16: "fp16", torch.float32: "fp32"}[dtype]
    g = torch.Generator().manual_seed(H)
    T, topk = 37, 4
    hidden = torch.randn(T, H, generator=g).to(dtype)
    rw = torch.rand(T, topk, generator=g).to(dtype)
    top_x = torch.randperm(T, generator=g)[:21].sort()[0]
    idx = torch.randint(0, topk, (21,), generator=g)
    cur = _kernels.moe_gather_rows(hidden.to(cuda), top_x.to(cuda))
    assert torch.equal(cur.cpu(), hidden[top_x])
    out0 = torch.randn(T, H, generator=g).to(dtype)
    expert_out = torch.randn(21, H, generator=g).to(dtype)
    got = _kernels.moe_scale_add_rows(out0.to(cuda).clone(), expert_out.to(cuda), rw.to(cuda), top_x.to(cuda), idx.to(cuda))
    want = O.moe_index_mul_index_add(out0.float().numpy(), expert_out.float().numpy(), rw.float().numpy(),
                                     top_x.numpy(), idx.numpy(), name)
    assert np.array_equal(got.float().cpu().numpy(), want)


def _moe_layer(ipex, E, H, I, seed):
    gate = [_woq_module(ipex, H, I, "INT4", 64, "BF16", bias=False, seed=seed + 3 * e) for e in range(E)]
    up = [_woq_module(ipex, H, I, "INT4", 64, "BF16", bias=False, seed=seed + 3 * e + 1) for e in range(E)]
    down = [_woq_module(ipex, I, H, "INT4", 64, "BF16", bias=False, seed=seed + 3 * e + 2) for e in range(E)]
    return gate, up, down


@pytest.mark.parametrize("T,topk", [(12, 2), (1, 2), (70, 3)])
def test_deepseek_moe_woq_matches_per_expert_composition(cuda, T, topk):
    from oracle import woq_oracle as O

    ipex = _ipex()
    # (K not a multiple of 256 in any linear: experts with few rows then run the dequantizing kernel on both paths)
    E, H, I = 5, 384, 640
    gate, up, down = _moe_layer(ipex, E, H, I, 100)
    g = torch.Generator().manual_seed(T)
    hidden = torch.randn(T, H, generator=g).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(T)])
    rw = torch.softmax(torch.randn(T, topk, generator=g), -1).to(torch.bfloat16)
    ctxs = [[m._op_context for m in ms] for ms in (gate, up, down)]
    got = torch.ops.torch_ipex.deepseek_moe_woq(hidden.to(cuda), ids.to(cuda), ctxs[0], ctxs[1], ctxs[2], rw.to(cuda), False)
    assert got.shape == hidden.shape and got.dtype == torch.bfloat16

    # the same experts one by one through the fusion modules, scatter by the oracle on the host
    top_x, idx = O.expert_token_lists(ids.numpy(), E)
    want = np.zeros((T, H), dtype=np.float32)
    dense = torch.zeros(T, H)
    mods = ipex.llm.modules
    for e in range(E):
        if len(top_x[e]) == 0:
            continue
        cur = hidden[torch.from_numpy(top_x[e])].to(cuda)
        y = down[e](mods.Linear2SiluMul(gate[e], up[e])(cur))
        want = O.moe_index_mul_index_add(want, y.float().cpu().numpy(), rw.float().numpy(), top_x[e], idx[e], "bf16")
        # float reference on the dequantized weights
        w = [c.get_scales() for c in (ctxs[0][e], ctxs[1][e], ctxs[2][e])]  # noqa: F841 (kept alive)
        deq = lambda m: ipex.quantization.dequantize_per_block(
            m._op_context.to_public(m._op_context.get_weight()).cpu(), m._op_context.get_scales().cpu(),
            m._op_context.get_zero_points().cpu(), ipex.quantization.WoqWeightDtype.INT4, 64,
            [m.out_features, m.in_features])
        xc = cur.float().cpu()
        ye = (torch.nn.functional.silu(xc @ deq(gate[e]).t()) * (xc @ deq(up[e]).t())) @ deq(down[e]).t()
        sel = torch.from_numpy(top_x[e])
        dense[sel] += ye * rw.float()[sel, torch.from_numpy(idx[e])].unsqueeze(-1)
    assert np.array_equal(got.float().cpu().numpy(), want)
    err = (got.float().cpu() - dense).abs().max() / dense.abs().max()
    assert float(err) < 3e-2, float(err)


_BINDING_ALONE = r"""
import sys
import torch

torch.ops.load_library(sys.argv[1])  # the operator / custom-class binding; the Python package is never imported
d = torch.load(sys.argv[2])
E, G = d["E"], d["G"]
mk = lambda w, s, z, n, k: torch.ops.ipex_prepack.weight_only_qlinear_prepack(
    w.cuda(), 2, [n, k], s.cuda(), z.cuda(), None, None, None, G, 2, -1, False)
H, I = d["H"], d["I"]
gate = [mk(*d["gate"][e], I, H) for e in range(E)]
up = [mk(*d["up"][e], I, H) for e in range(E)]
down = [mk(*d["down"][e], H, I) for e in range(E)]
hidden, ids, rw = d["hidden"].cuda(), d["ids"].cuda(), d["rw"].cuda()
layer = torch.ops.torch_ipex.deepseek_moe_woq(hidden, ids, gate, up, down, rw, False)
one_by_one = torch.zeros_like(hidden)
for e in range(E):
    tok, slot = (d["ids"] == e).nonzero(as_tuple=True)
    r = torch.ops.torch_ipex.mixtral_moe_woq(hidden, tok, slot, gate[e].get_data_handle(), up[e].get_data_handle(),
                                             down[e].get_data_handle(), rw, one_by_one, False)
    assert r.data_ptr() == one_by_one.data_ptr()
torch.save({"layer": layer.cpu(), "one_by_one": one_by_one.cpu()}, sys.argv[3])
"""


def test_moe_operators_of_the_binding_without_the_python_package(cuda, tmp_path, monkeypatch):
    """torch_ipex::mixtral_moe_woq and deepseek_moe_woq as the C++ binding registers them (csrc/cpu/aten/MoE.cpp:260-328,
    455-472), in a process that loads only libwoq_torch.so -- what a TorchScript consumer has: equal, bit for bit, to
    the Python package's per-expert path on the same experts and routing."""
    import subprocess
    import sys

    from ipex_amd import _lib
    from ipex_amd.utils import synthetic

    E, H, I, G, T, topk = 4, 256, 384, 64, 9, 2
    layer = {"E": E, "H": H, "I": I, "G": G}
    for i, (name, n, k) in enumerate((("gate", I, H), ("up", I, H), ("down", H, I))):
        layer[name] = []
        for e in range(E):
            c = synthetic.make_int4_case(500 + 3 * e + i, 1, k, n, G)
            layer[name].append((c["qweight"], c["scales"], c["zeros"]))
    g = torch.Generator().manual_seed(77)
    layer["hidden"] = torch.randn(T, H, generator=g).to(torch.bfloat16)
    layer["ids"] = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(T)])
    layer["rw"] = torch.softmax(torch.randn(T, topk, generator=g), -1).to(torch.bfloat16)
    torch.save(layer, tmp_path / "layer.pt")
    (tmp_path / "alone.py").write_text(_BINDING_ALONE)
    run = subprocess.run([sys.executable, str(tmp_path / "alone.py"), _lib.TORCH_LIB_PATH, str(tmp_path / "layer.pt"),
                          str(tmp_path / "out.pt")], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-3000:]
    alone = torch.load(tmp_path / "out.pt")
    assert torch.equal(alone["layer"], alone["one_by_one"])

    ctx = lambda w, s, z, n, k: torch.ops.ipex_prepack.weight_only_qlinear_prepack(
        w.to(cuda), 2, [n, k], s.to(cuda), z.to(cuda), None, None, None, G, 2, -1, False)
    gate = [ctx(*layer["gate"][e], I, H) for e in range(E)]
    up = [ctx(*layer["up"][e], I, H) for e in range(E)]
    down = [ctx(*layer["down"][e], H, I) for e in range(E)]
    monkeypatch.setenv("IPEX_AMD_MOE_GROUPED", "0")
    want = torch.ops.torch_ipex.deepseek_moe_woq(layer["hidden"].to(cuda), layer["ids"].to(cuda), gate, up, down,
                                                 layer["rw"].to(cuda), False)
    assert torch.equal(alone["layer"], want.cpu())


def test_moe_route_against_the_oracle_token_lists(cuda):
    """woq_hip_moe_route: sorted positions, slots per compute type and per-token contribution order against the
    oracle's per-expert token lists (get_expert_topx_idx, MoE.cpp:64-81); ids outside the expert range drop out."""
    from ipex_amd import _lib
    from oracle import woq_oracle as O

    lib = _lib.load()
    g = torch.Generator().manual_seed(5)
    for T, topk, E, split in ((1, 8, 64, 5), (16, 8, 32, 5), (64, 6, 9, 5), (33, 4, 7, 0), (256, 8, 300, 5)):
        ids = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(T)])
        if T >= 16:
            ids[3, 1], ids[7, 0] = -1, E + 3  # not experts
        R = T * topk
        dev = ids.to(cuda)
        x_row = torch.full((R,), -7, dtype=torch.int64, device=cuda)
        row_of, slot_of = (torch.full((R,), -7, dtype=torch.int32, device=cuda) for _ in range(2))
        single = split > 1 and T != 33
        S = min(R, E) + (T == 16)  # also tables longer than needed
        slots = torch.full((4, 3, S), -7, dtype=torch.int32, device=cuda)
        assert lib.woq_hip_moe_route(dev.data_ptr(), T, topk, E, split, 16, int(single), min(R, E) - 1, x_row.data_ptr(),
                                     slots.data_ptr(), row_of.data_ptr(), slot_of.data_ptr(), None) != 0  # tables too short
        rc = lib.woq_hip_moe_route(dev.data_ptr(), T, topk, E, split, 16, int(single), S, x_row.data_ptr(),
                                   slots.data_ptr(), row_of.data_ptr(), slot_of.data_ptr(), None)
        assert rc == 0, lib.woq_hip_last_error()
        torch.cuda.synchronize()
        valid = (ids >= 0) & (ids < E)
        top_x, idx = O.expert_token_lists(torch.where(valid, ids, torch.full_like(ids, E)).numpy(), E + 1)
        pos, want_row, want = 0, [], [[], [], [], []]  # per class: (expert, first sorted position, rows)
        entry_pos = {}
        for e in range(E):
            n = len(top_x[e])
            if n:
                cls = 3 if single and n == 1 else 0 if n < split else 1 if n <= 16 else 2
                want[cls].append((e, pos, min(n, 64)))
            for t, j in zip(top_x[e], idx[e]):
                entry_pos[(int(t), int(j))] = pos
                want_row.append(int(t))
                pos += 1
        assert x_row.cpu().tolist()[:pos] == want_row
        got = slots.cpu()
        for cls in range(4):
            n = len(want[cls])
            assert [tuple(int(got[cls, i, k]) for i in range(3)) for k in range(n)] == want[cls], (T, cls)
            assert got[cls, 0, n:].eq(-1).all(), (T, cls)
        ro, so = row_of.cpu().view(T, topk), slot_of.cpu().view(T, topk)
        for t in range(T):
            order = sorted((int(ids[t, j]), j) for j in range(topk) if bool(valid[t, j]))
            for i in range(topk):
                if i < len(order):
                    assert int(ro[t, i]) == entry_pos[(t, order[i][1])] and int(so[t, i]) == order[i][1]
                else:
                    assert int(ro[t, i]) == -1


def test_moe_route_keeps_at_most_64_rows_of_an_expert(cuda):
    from ipex_amd import _lib

    lib = _lib.load()
    T, topk, E = 80, 2, 5
    ids = torch.stack([torch.tensor([2, 3 if t % 2 else 4]) for t in range(T)])  # expert 2 gets all 80 tokens
    R = T * topk
    x_row = torch.empty(R, dtype=torch.int64, device=cuda)
    row_of, slot_of = (torch.empty(R, dtype=torch.int32, device=cuda) for _ in range(2))
    slots = torch.empty((4, 3, E), dtype=torch.int32, device=cuda)
    rc = lib.woq_hip_moe_route(ids.to(cuda).data_ptr(), T, topk, E, 5, 16, 1, E, x_row.data_ptr(), slots.data_ptr(),
                               row_of.data_ptr(), slot_of.data_ptr(), None)
    assert rc == 0, lib.woq_hip_last_error()
    assert slots[2, :, 0].cpu().tolist() == [2, 0, 64] and x_row[:80].cpu().tolist() == list(range(80))
    assert slots[2, 0, 1:].cpu().tolist() == [3, 4, -1, -1] and slots[2, 1, 1:3].cpu().tolist() == [80, 120]
    ro = row_of.cpu().view(T, topk)
    assert ro[:64, 0].tolist() == list(range(64)) and bool((ro[64:, 0] == -1).all())
    assert bool((ro[:, 1] >= 80).all())  # the other contribution of every token is kept


@pytest.mark.parametrize("weight_dtype,lowp", [("INT4", "BF16"), ("INT8", "BF16"), ("INT4", "NONE")])
@pytest.mark.parametrize("T,topk", [(1, 4), (5, 3), (16, 4), (40, 2), (64, 6)])
def test_deepseek_moe_grouped_launches_equal_the_per_expert_path(cuda, monkeypatch, weight_dtype, lowp, T, topk):
    """The layer in grouped launches (routing sorted on the device, one launch per linear and compute type over all
    experts, contributions added in ascending expert order) against the per-expert path, which reads the routing on
    the host: bit for bit, with experts that get one, a few, many or no tokens."""
    from ipex_amd import _lib

    ipex = _ipex()
    # (K not a multiple of 256 in any linear: experts with few rows then run the dequantizing kernel on both paths)
    E, H, I = 9, 384, 640
    G = 64 if weight_dtype == "INT4" else -1
    mk = lambda k, n, s: _woq_module(ipex, k, n, weight_dtype, G, lowp, bias=False, seed=s)
    ctxs = [[mk(H, I, 300 + 3 * e)._op_context for e in range(E)], [mk(H, I, 301 + 3 * e)._op_context for e in range(E)],
            [mk(I, H, 302 + 3 * e)._op_context for e in range(E)]]
    g = torch.Generator().manual_seed(100 * T + topk)
    hidden = torch.randn(T, H, generator=g).to(torch.bfloat16).to(cuda)
    # skewed routing: expert 0 is popular, expert E - 1 never chosen
    ids = torch.stack([torch.cat([torch.zeros(1, dtype=torch.int64), 1 + torch.randperm(E - 2, generator=g)[:topk - 1]]) if t % 3 else
                       torch.randperm(E - 1, generator=g)[:topk] for t in range(T)]).to(cuda)
    rw = torch.softmax(torch.randn(T, topk, generator=g), -1).to(torch.bfloat16).to(cuda)
    op = torch.ops.torch_ipex.deepseek_moe_woq
    monkeypatch.setenv("IPEX_AMD_MOE_GROUPED", "0")
    want = op(hidden, ids, ctxs[0], ctxs[1], ctxs[2], rw, False)
    assert _lib.last_kernel() == "moe_scale_add_rows"
    monkeypatch.setenv("IPEX_AMD_MOE_GROUPED", "1")
    got = op(hidden, ids, ctxs[0], ctxs[1], ctxs[2], rw, False)
    assert _lib.last_kernel() == "moe_combine_rows"
    assert torch.equal(got, want)
    # again with other routing through the cached plan
    ids2 = ids.flip(0).contiguous()
    monkeypatch.setenv("IPEX_AMD_MOE_GROUPED", "0")
    want2 = op(hidden, ids2, ctxs[0], ctxs[1], ctxs[2], rw, False)
    monkeypatch.setenv("IPEX_AMD_MOE_GROUPED", "1")
    assert torch.equal(op(hidden, ids2, ctxs[0], ctxs[1], ctxs[2], rw, False), want2)


def test_moe_route_with_a_slot_per_position(cuda):
    """use_single = 2 (what a single token gets): every sorted position is a one-row slot of its own in class 3."""
    from ipex_amd import _lib

    lib = _lib.load()
    ids = torch.tensor([[5, 2, 5, 0, 7, 2]])  # experts 2 and 5 named twice
    T, topk, E, S = 1, 6, 8, 8
    x_row = torch.full((6,), -7, dtype=torch.int64, device=cuda)
    row_of, slot_of = (torch.full((6,), -7, dtype=torch.int32, device=cuda) for _ in range(2))
    slots = torch.full((4, 3, S), -7, dtype=torch.int32, device=cuda)
    args = (ids.to(cuda).data_ptr(), T, topk, E, 5, 16)
    assert lib.woq_hip_moe_route(*args, 2, 5, x_row.data_ptr(), slots.data_ptr(), row_of.data_ptr(), slot_of.data_ptr(), None) != 0
    assert lib.woq_hip_moe_route(*args, 3, S, x_row.data_ptr(), slots.data_ptr(), row_of.data_ptr(), slot_of.data_ptr(), None) != 0
    rc = lib.woq_hip_moe_route(*args, 2, S, x_row.data_ptr(), slots.data_ptr(), row_of.data_ptr(), slot_of.data_ptr(), None)
    assert rc == 0, lib.woq_hip_last_error()
    got = slots.cpu()
    assert got[3, 0].tolist() == [0, 2, 2, 5, 5, 7, -1, -1]
    assert got[3, 1, :6].tolist() == [0, 1, 2, 3, 4, 5] and got[3, 2, :6].tolist() == [1] * 6
    assert bool(got[:3, 0].eq(-1).all())
    assert row_of.cpu().tolist() == [0, 1, 2, 3, 4, 5] and slot_of.cpu().tolist() == [3, 1, 5, 0, 2, 4]


@pytest.mark.parametrize("G", [32, 64, 128])
@pytest.mark.parametrize("T,lowp", [(1, "BF16"), (3, "BF16"), (8, "BF16"), (16, "BF16"), (5, "FP16")])
def test_deepseek_moe_grouped_is_the_per_expert_result_up_to_16_rows(cuda, monkeypatch, G, T, lowp):
    """Experts with one row run the single-row decode kernel on both paths, those with two to four rows the other
    integer-weight decode kernel, those with five to sixteen the dequantizing one (groups of 32, 64 and 128, K a
    multiple of 256): bit for bit."""
    from ipex_amd import _lib

    ipex = _ipex()
    E, H, I, topk = 7, 512, 256, 4
    mk = lambda k, n, s: _woq_module(ipex, k, n, "INT4", G, lowp, bias=False, seed=s)
    ctxs = [[mk(H, I, 600 + 3 * e)._op_context for e in range(E)], [mk(H, I, 601 + 3 * e)._op_context for e in range(E)],
            [mk(I, H, 602 + 3 * e)._op_context for e in range(E)]]
    g = torch.Generator().manual_seed(G + T)
    xdt = torch.float16 if lowp == "FP16" else torch.bfloat16
    hidden = torch.randn(T, H, generator=g).to(xdt).to(cuda)
    ids = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(T)]).to(cuda)
    rw = torch.softmax(torch.randn(T, topk, generator=g), -1).to(xdt).to(cuda)
    op = torch.ops.torch_ipex.deepseek_moe_woq
    monkeypatch.setenv("IPEX_AMD_MOE_GROUPED", "0")
    want = op(hidden, ids, ctxs[0], ctxs[1], ctxs[2], rw, False)
    monkeypatch.setenv("IPEX_AMD_MOE_GROUPED", "1")
    got = op(hidden, ids, ctxs[0], ctxs[1], ctxs[2], rw, False)
    assert _lib.last_kernel() == "moe_combine_rows"
    assert torch.equal(got, want)


@pytest.mark.parametrize("lowp,G", [("BF16", 128), ("BF16", 64), ("FP16", 128), ("NONE", 64)])
@pytest.mark.parametrize("T", [1, 3])
def test_deepseek_moe_grouped_with_an_expert_named_twice(cuda, monkeypatch, lowp, G, T):
    """Top-k lists that name an expert twice: in the grouped launches both entries are rows of that expert, each with
    its own routing weight."""
    from ipex_amd import _lib

    ipex = _ipex()
    E, H, I, topk = 6, 256, 256, 4
    mk = lambda k, n, s: _woq_module(ipex, k, n, "INT4", G, lowp, bias=False, seed=s)
    ctxs = [[mk(H, I, 500 + 3 * e)._op_context for e in range(E)], [mk(H, I, 501 + 3 * e)._op_context for e in range(E)],
            [mk(I, H, 502 + 3 * e)._op_context for e in range(E)]]
    g = torch.Generator().manual_seed(T)
    xdt = torch.float16 if lowp == "FP16" else torch.bfloat16
    hidden = torch.randn(T, H, generator=g).to(xdt).to(cuda)
    ids = torch.tensor([[3, 1, 3, 5], [0, 0, 0, 0], [2, 4, 1, 2]][:T]).to(cuda)
    rw = torch.softmax(torch.randn(T, topk, generator=g), -1).to(xdt).to(cuda)
    op = torch.ops.torch_ipex.deepseek_moe_woq
    monkeypatch.setenv("IPEX_AMD_MOE_GROUPED", "1")
    got = op(hidden, ids, ctxs[0], ctxs[1], ctxs[2], rw, False)
    assert _lib.last_kernel() == "moe_combine_rows"
    # the same layer one top-k column at a time (no expert is named twice inside a column), summed in float
    want = torch.zeros(T, H)
    for j in range(topk):
        want += op(hidden, ids[:, j:j + 1].contiguous(), ctxs[0], ctxs[1], ctxs[2], rw[:, j:j + 1].contiguous(), False).float().cpu()
    assert float((got.float().cpu() - want).norm() / want.norm()) < 8e-3
    # the per-expert path runs the mentions of a token in rounds (its scatter adds one row per token)
    monkeypatch.setenv("IPEX_AMD_MOE_GROUPED", "0")
    per_expert = op(hidden, ids, ctxs[0], ctxs[1], ctxs[2], rw, False)
    assert _lib.last_kernel() == "moe_scale_add_rows"
    assert float((per_expert.float().cpu() - want).norm() / want.norm()) < 8e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("accumulate", [0, 1])
def test_moe_combine_rows_bit_exact(cuda, dtype, accumulate):
    """woq_hip_moe_combine_rows against the oracle's sequential weighted scatter applied expert by expert."""
    from ipex_amd import _kernels, _lib
    from oracle import woq_oracle as O

    lib = _lib.load()
    name = {torch.bfloat16: "bf16", torch.float16: "fp16", torch.float32: "fp32"}[dtype]
    g = torch.Generator().manual_seed(3)
    T, topk, E, H = 19, 10, 13, 100  # ten contributions: two groups of eight in the kernel; H not a multiple of 8
    ids = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(T)])
    ids[2, 3] = -1
    R = T * topk
    row_of, slot_of = (torch.empty(R, dtype=torch.int32, device=cuda) for _ in range(2))
    slots = torch.empty((4, 3, E), dtype=torch.int32, device=cuda)
    x_row = torch.empty(R, dtype=torch.int64, device=cuda)
    rc = lib.woq_hip_moe_route(ids.to(cuda).data_ptr(), T, topk, E, 5, 16, 0, E, x_row.data_ptr(), slots.data_ptr(),
                               row_of.data_ptr(), slot_of.data_ptr(), None)
    assert rc == 0, lib.woq_hip_last_error()
    expert_out = torch.randn(R, H, generator=g).to(dtype)
    rw = torch.rand(T, topk, generator=g).to(dtype)
    out0 = torch.randn(T, H, generator=g).to(dtype)
    out = out0.to(cuda).clone()
    rc = lib.woq_hip_moe_combine_rows(out.data_ptr(), _kernels._ACT_CODE[dtype], T, H, expert_out.to(cuda).data_ptr(),
                                      rw.to(cuda).data_ptr(), topk, row_of.data_ptr(), slot_of.data_ptr(), accumulate, None)
    assert rc == 0, lib.woq_hip_last_error()
    valid = (ids >= 0) & (ids < E)
    top_x, idx = O.expert_token_lists(torch.where(valid, ids, torch.full_like(ids, E)).numpy(), E + 1)
    want = out0.float().numpy() if accumulate else np.zeros((T, H), dtype=np.float32)
    pos = 0
    for e in range(E):
        n = len(top_x[e])
        want = O.moe_index_mul_index_add(want, expert_out[pos:pos + n].float().numpy(), rw.float().numpy(), top_x[e], idx[e], name)
        pos += n
    assert np.array_equal(out.float().cpu().numpy(), want)


def test_deepseek_moe_grouped_groups_of_128_and_rejections(cuda, monkeypatch):
    """Groups of 128: the per-expert path serves experts with fewer than five rows with the decode kernel that keeps the
    weights as integers, the grouped path dequantizes them -- two roundings of the same product, compared to tolerance
    and both against the float layer.  Then what the grouped entry point refuses."""
    import ctypes
    from ipex_amd import _lib

    ipex = _ipex()
    E, H, I, T, topk = 6, 512, 256, 3, 2
    mk = lambda k, n, s: _woq_module(ipex, k, n, "INT4", 128, "BF16", bias=False, seed=s)
    mods = [[mk(H, I, 400 + 3 * e) for e in range(E)], [mk(H, I, 401 + 3 * e) for e in range(E)], [mk(I, H, 402 + 3 * e) for e in range(E)]]
    ctxs = [[m._op_context for m in ms] for ms in mods]
    g = torch.Generator().manual_seed(9)
    hidden = torch.randn(T, H, generator=g).to(torch.bfloat16).to(cuda)
    ids = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(T)]).to(cuda)
    rw = torch.softmax(torch.randn(T, topk, generator=g), -1).to(torch.bfloat16).to(cuda)
    op = torch.ops.torch_ipex.deepseek_moe_woq
    monkeypatch.setenv("IPEX_AMD_MOE_GROUPED", "0")
    a = op(hidden, ids, ctxs[0], ctxs[1], ctxs[2], rw, False).float()
    monkeypatch.setenv("IPEX_AMD_MOE_GROUPED", "1")
    b = op(hidden, ids, ctxs[0], ctxs[1], ctxs[2], rw, False).float()
    assert _lib.last_kernel() == "moe_combine_rows"
    assert float((a - b).norm() / a.norm()) < 6e-3
    deq = lambda m: ipex.quantization.dequantize_per_block(
        m._op_context.to_public(m._op_context.get_weight()).cpu(), m._op_context.get_scales().cpu(),
        m._op_context.get_zero_points().cpu(), ipex.quantization.WoqWeightDtype.INT4, 128, [m.out_features, m.in_features])
    dense = torch.zeros(T, H)
    for t in range(T):
        for j in range(topk):
            e = int(ids[t, j])
            xc = hidden[t].float().cpu()
            ye = (torch.nn.functional.silu(deq(mods[0][e]) @ xc) * (deq(mods[1][e]) @ xc)) @ deq(mods[2][e]).t()
            dense[t] += ye * float(rw[t, j])
    for got in (a, b):
        assert float((got.cpu() - dense).norm() / dense.norm()) < 2e-2
    # the C entry point: what it refuses
    lib = _lib.load()
    p = _lib.LinearParams()
    p.struct_size = ctypes.sizeof(_lib.LinearParams)
    p.K, p.N, p.M, p.weight_dtype, p.group_size, p.lowp_mode = H, I, 16, 2, 128, 2
    p.x_dtype = p.out_dtype = 2
    p.x = p.out = hidden.data_ptr()
    table = torch.zeros(8, dtype=torch.int64, device=cuda)
    for change, text in ((dict(M=65), "rows per slot"), (dict(weight_dtype=3), "INT4 and INT8"), (dict(lowp_mode=3), "lowp_mode"),
                         (dict(fusion=_lib.FUSE_GELU_ERF), "post-op"), (dict(N=48), "even number"), (dict(K=H + 64), "multiple of the weight tile")):
        q = _lib.LinearParams.from_buffer_copy(p)
        for k, v in change.items():
            setattr(q, k, v)
        assert lib.woq_hip_linear_grouped(ctypes.byref(q), table.data_ptr(), 4) != 0
        assert text in lib.woq_hip_last_error().decode(), (change, lib.woq_hip_last_error())
    assert lib.woq_hip_linear_grouped(ctypes.byref(p), None, 4) != 0


def test_mixtral_moe_woq_single_expert_and_errors(cuda):
    ipex = _ipex()
    H, I, T = 128, 256, 6
    gate, up, down = _moe_layer(ipex, 1, H, I, 200)
    g = torch.Generator().manual_seed(5)
    hidden = torch.randn(T, H, generator=g).to(torch.bfloat16).to(cuda)
    rw = torch.rand(T, 2, generator=g).to(torch.bfloat16).to(cuda)
    top_x = torch.tensor([0, 2, 5])
    idx = torch.tensor([1, 0, 1])
    out = torch.zeros_like(hidden)
    handles = [m[0]._op_context.get_data_handle() for m in (gate, up, down)]
    ret = torch.ops.torch_ipex.mixtral_moe_woq(hidden, top_x.to(cuda), idx.to(cuda), *handles, rw, out, False)
    assert ret.data_ptr() == out.data_ptr()
    y = down[0](ipex.llm.modules.Linear2SiluMul(gate[0], up[0])(hidden[top_x.to(cuda)]))
    want = torch.zeros_like(hidden)
    want[top_x.to(cuda)] = (y.float() * rw[top_x.to(cuda), idx.to(cuda)].float().unsqueeze(-1)).to(torch.bfloat16)
    assert torch.equal(out, want)
    assert bool((out[[1, 3, 4]] == 0).all())
    # no tokens: output untouched
    before = out.clone()
    empty = torch.empty(0, dtype=torch.int64, device=cuda)
    torch.ops.torch_ipex.mixtral_moe_woq(hidden, empty, empty, *handles, rw, out, False)
    assert torch.equal(out, before)
    with pytest.raises(RuntimeError, match="all-reduce"):
        torch.ops.torch_ipex.mixtral_moe_woq(hidden, top_x.to(cuda), idx.to(cuda), *handles, rw, out, True)
    ctxs = [[m[0]._op_context] for m in (gate, up, down)]
    with pytest.raises(RuntimeError, match="expert ids"):
        torch.ops.torch_ipex.deepseek_moe_woq(hidden, torch.full((T, 1), 3), ctxs[0], ctxs[1], ctxs[2], rw, False)


# ---------------------------------------------------------------------------------------------
# the C++ binding: registered operators and the TorchScript custom class
# ---------------------------------------------------------------------------------------------
def test_custom_class_method_surface_and_pickle(cuda):
    """torch.classes.ipex_prepack.WoqLinearOpContext: the twelve methods of the reference's class
    (RegisterOpContextClass.cpp:127-173) and its pickle (plain format out, re-prepacked on load)."""
    from ipex_amd.utils import synthetic
    from helpers import make_context, make_torch_context

    case = synthetic.make_int4_case(60, 5, 512, 80, 128, bias=True)
    ctx = make_torch_context(case, 2)
    assert "WoqLinearOpContext" in str(type(ctx)) or "ScriptObject" in str(type(ctx))
    assert ctx.get_weight_shape() == [80, 512]
    assert torch.equal(ctx.to_public(ctx.get_weight()).cpu(), case["qweight"])
    assert torch.equal(ctx.pack(case["qweight"].to(cuda)), ctx.get_weight())
    assert torch.equal(ctx.get_scales().cpu(), case["scales"]) and ctx.get_scales().shape == (80, 4)
    assert torch.equal(ctx.get_zero_points().cpu(), case["zeros"])
    assert torch.equal(ctx.get_bias().cpu(), case["bias"])
    assert ctx.get_g_idx() is None and ctx.get_cached_weight() is None and ctx.get_cached_compensation() is None
    h = ctx.get_data_handle()
    assert h.dtype == torch.int64 and h.numel() == 1 and h.device.type == "cpu"
    x = case["x"].to(cuda)
    y0 = torch.ops.torch_ipex.ipex_woq_linear(x, h)
    # same kernels as the ctypes twin: bit-identical
    assert torch.equal(y0, make_context(case, 2).run(x))
    ctx2 = pickle.loads(pickle.dumps(ctx))
    assert ctx2.get_data_handle().item() != h.item()
    assert torch.equal(torch.ops.torch_ipex.ipex_woq_linear(x, ctx2.get_data_handle()), y0)
    # load_from_ctx: the state of another context under the old handle
    other = make_torch_context(synthetic.make_int4_case(61, 5, 512, 80, 128, bias=True), 2)
    y_other = torch.ops.torch_ipex.ipex_woq_linear(x, other.get_data_handle())
    ctx.load_from_ctx(other)
    assert ctx.get_data_handle().item() == h.item()
    assert torch.equal(torch.ops.torch_ipex.ipex_woq_linear(x, h), y_other)


@pytest.mark.parametrize("weight_dtype,bias", [("INT8", True), ("INT4", False)])
@pytest.mark.parametrize("M,K,N", [(3, 31 * 8, 31), (4, 4096, 4080), (70, 1024, 512)])
def test_jit_trace_save_load(cuda, tmp_path, weight_dtype, bias, M, K, N):
    """As the reference's test_weight_only_quantization_jit_save_load
    (tests/cpu/test_quantization_default_recipe.py:453-502): trace the converted model, freeze, save,
    load, compare.  The loaded module owns a context re-made from the pickled plain format."""
    import ipex_amd as ipex

    q = ipex.quantization
    torch.manual_seed(5)
    model = torch.nn.Sequential(torch.nn.Linear(K, N, bias=bias)).to(torch.bfloat16).eval().to(cuda)
    x = torch.rand(M, K, device=cuda).to(torch.bfloat16)
    qmap = q.get_weight_only_quant_qconfig_mapping(weight_dtype=getattr(q.WoqWeightDtype, weight_dtype),
                                                   lowp_mode=q.WoqLowpMode.BF16)
    with torch.no_grad():
        converted = q.convert(q.prepare(model, qmap, inplace=False), inplace=False)
        want = converted(x)
        traced = torch.jit.freeze(torch.jit.trace(converted, x))
        path = str(tmp_path / "woq.pt")
        traced.save(path)
        loaded = torch.jit.load(path)
        assert torch.equal(traced(x), want)
        assert torch.equal(loaded(x), want)
        # the loaded graph calls the operator with a handle taken at run time, not a baked-in one
        assert "ipex_woq_linear" in str(loaded.graph) or "ipex_woq_linear" in str(loaded.inlined_graph)
        del converted, traced
        assert torch.equal(loaded(x), want)


def test_autocast_casts_the_input_only(cuda):
    """AutocastCUDA (csrc/cpu/aten/Linear.cpp:874-883): fp32 rows under autocast(bf16) run as bf16 rows."""
    from ipex_amd.utils import synthetic
    from helpers import make_torch_context

    case = synthetic.make_int4_case(62, 9, 512, 96, 128, bias=True)
    ctx = make_torch_context(case, 2)
    h = ctx.get_data_handle()
    x32 = case["x"].to(cuda).float()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = torch.ops.torch_ipex.ipex_woq_linear(x32, h)
        ys = torch.ops.torch_ipex.woq_linear_silu(x32, h)
    assert y.dtype == torch.bfloat16
    assert torch.equal(y, torch.ops.torch_ipex.ipex_woq_linear(x32.bfloat16(), h))
    assert torch.equal(ys, torch.ops.torch_ipex.woq_linear_silu(x32.bfloat16(), h))
    # without autocast the fp32 rows are computed in fp32
    assert torch.ops.torch_ipex.ipex_woq_linear(x32, make_torch_context(case, 0).get_data_handle()).dtype == torch.float32


@pytest.mark.parametrize("N,K,G", [(64, 256, 64), (33, 512, 128), (16, 128, -1), (80, 1024, 32)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_dequantize_nf4_op(cuda, N, K, G, dtype):
    """torch_ipex::dequantize_nf4 (csrc/cpu/aten/Linear.cpp:804-811, test
    tests/cpu/test_quantization_default_recipe.py:2230-2261): table[code] * scale against the oracle's
    table, bit-exact in fp32 and after one rounding in the 16-bit types."""
    import numpy as np

    from oracle import woq_oracle as O

    g = torch.Generator().manual_seed(N + K)
    codes = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=g)
    KG = (K + G - 1) // G if G > 0 else 1
    scales = (0.02 + torch.rand(N, KG, generator=g)).float()
    got = torch.ops.torch_ipex.dequantize_nf4(codes.to(cuda), scales.to(cuda) if G > 0 else scales.reshape(N).to(cuda), G, dtype)
    assert got.dtype == dtype and tuple(got.shape) == (N, K)
    want = O.dequantize_woq_weight(codes.numpy(), N, K, scales.numpy(), None, O.WOQ_DTYPE_NF4, G)
    if dtype == torch.float32:
        assert np.array_equal(got.cpu().numpy(), want)
    else:
        assert torch.equal(got.cpu(), torch.from_numpy(want).to(dtype))
    with pytest.raises(RuntimeError, match="GPU"):
        torch.ops.torch_ipex.dequantize_nf4(codes, scales, G, dtype)


def test_moe_over_registered_contexts(cuda):
    """deepseek_moe_woq over lists of the registered custom class equals the same layer over the ctypes twins."""
    from ipex_amd.utils import synthetic
    from helpers import make_context, make_torch_context

    T, H, I, E, topk = 12, 256, 512, 4, 2
    g = torch.Generator().manual_seed(9)
    hidden = torch.randn(T, H, generator=g).bfloat16().to(cuda)
    ids = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(T)]).to(cuda)
    rw = torch.rand(T, topk, generator=g).bfloat16().to(cuda)
    cases = [[synthetic.make_int4_case(70 + 3 * e + j, 1, H if j < 2 else I, I if j < 2 else H, 128) for e in range(E)]
             for j in range(3)]
    py = [[make_context(c, 2) for c in row] for row in cases]
    cc = [[make_torch_context(c, 2) for c in row] for row in cases]
    want = torch.ops.torch_ipex.deepseek_moe_woq(hidden, ids, py[0], py[1], py[2], rw, False)
    got = torch.ops.torch_ipex.deepseek_moe_woq(hidden, ids, cc[0], cc[1], cc[2], rw, False)
    assert torch.equal(got, want)
