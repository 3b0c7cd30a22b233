"""CPU-side checks: the C ABI library loads and exports what include/woq_hip.h declares, the
recipe / enum surface matches the reference's values, the quantize helpers and checkpoint
converters implement the wire format, and the product refuses to run without a GPU."""
import os
import re

import numpy as np
import pytest
import torch

from oracle import woq_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from ipex_amd import _lib

    header = open(os.path.join(ROOT, "include", "woq_hip.h")).read()
    declared = set(re.findall(r"\b(woq_hip_[a-z0-9_]+)\s*\(", header))
    declared.discard("woq_hip_linear_params")
    assert declared == set(_lib.EXPORTS)
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.woq_hip_abi_version() == 3
    # pure host-side helpers can be called without a GPU
    assert lib.woq_hip_padded_n(500) == 512
    assert lib.woq_hip_padded_k(2, 4096) == 4096 and lib.woq_hip_padded_k(2, 4097) == 4224
    assert lib.woq_hip_padded_k(1, 100) == 128
    assert lib.woq_hip_packed_weight_bytes(2, 14336, 4096) == 14336 * 4096 // 2
    assert [lib.woq_hip_int8_block_k(g, 4096) for g in (-1, 32, 64, 128, 256)] == [128, 32, 64, 128, 128]
    # the dense bf16 copy of cache_weight_for_large_batch: two bytes per weight over the padded rows, none where K is
    # no multiple of 128 or the copy would reach 2 GiB
    assert lib.woq_hip_dense_weight_bytes(2, 14336, 4096) == 14336 * 4096 * 2
    assert lib.woq_hip_dense_weight_bytes(1, 500, 256) == 512 * 256 * 2
    assert lib.woq_hip_dense_weight_bytes(2, 64, 192) == 0 and lib.woq_hip_dense_weight_bytes(2, 65536, 16384) == 0
    assert lib.woq_hip_weight_cache_batch_threshold() == 64


def test_params_struct_size_is_checked():
    import ctypes

    from ipex_amd import _lib

    lib = _lib.load()
    p = _lib.LinearParams()
    p.struct_size = 8
    assert lib.woq_hip_linear(ctypes.byref(p)) != 0
    assert b"struct_size" in lib.woq_hip_last_error()
    p.struct_size = ctypes.sizeof(_lib.LinearParams)
    p.weight_dtype = 7
    assert lib.woq_hip_linear(ctypes.byref(p)) != 0
    assert b"weight dtype" in lib.woq_hip_last_error()


def test_enum_values_match_reference():
    from ipex_amd.quantization import WoqActQuantMode, WoqLowpMode, WoqWeightDtype, WoqWeightQScheme
    from ipex_amd.llm.quantization import QuantDtype, QuantMethod
    from ipex_amd.nn.modules.weight_only_quantization import WoqWeightFormat

    assert [int(v) for v in WoqLowpMode] == [0, 1, 2, 3]
    assert [int(v) for v in WoqActQuantMode] == [-1, 0, 1, 2, 3, 4, 5, 6, 7]
    assert (WoqWeightDtype.INT8, WoqWeightDtype.INT4, WoqWeightDtype.NF4, WoqWeightDtype.FP8) == (1, 2, 3, 4)
    assert (WoqWeightQScheme.UNDEFINED, WoqWeightQScheme.ASYMMETRIC, WoqWeightQScheme.SYMMETRIC) == (0, 1, 2)
    assert (QuantMethod.GPTQ_GEMM, QuantMethod.AWQ_GEMM, QuantDtype.INT4) == (0, 1, 0)
    assert (WoqWeightFormat.PLAIN_FORMAT, WoqWeightFormat.GPTQ_FORMAT, WoqWeightFormat.AWQ_FORMAT) == (0, 1, 2)


def test_qconfig_mapping_rules():
    from ipex_amd.quantization import (
        QConfigWoq, WoqActQuantMode, WoqLowpMode, WoqWeightDtype, WoqWeightQScheme,
        get_weight_only_quant_qconfig_mapping,
    )

    q = get_weight_only_quant_qconfig_mapping().global_qconfig
    assert isinstance(q, QConfigWoq)
    assert q.weight_dtype == WoqWeightDtype.INT8 and q.lowp_mode == WoqLowpMode.NONE and q.group_size == -1
    # act_quant_mode only survives with lowp_mode INT8
    assert q.act_quant_mode == WoqActQuantMode.NONE
    q = get_weight_only_quant_qconfig_mapping(weight_dtype=WoqWeightDtype.INT4, lowp_mode=WoqLowpMode.INT8).global_qconfig
    assert q.act_quant_mode == WoqActQuantMode.PER_BATCH_IC_BLOCK_SYM
    assert q.weight_qscheme == WoqWeightQScheme.ASYMMETRIC
    # INT8 x INT8 and NF4 resolve to symmetric and reject asymmetric
    q = get_weight_only_quant_qconfig_mapping(weight_dtype=WoqWeightDtype.INT8, lowp_mode=WoqLowpMode.INT8).global_qconfig
    assert q.weight_qscheme == WoqWeightQScheme.SYMMETRIC
    with pytest.raises(AssertionError):
        get_weight_only_quant_qconfig_mapping(
            weight_dtype=WoqWeightDtype.NF4, weight_qscheme=WoqWeightQScheme.ASYMMETRIC
        )
    with pytest.raises(AssertionError):
        get_weight_only_quant_qconfig_mapping(group_size=48)


@pytest.mark.parametrize("sym", [False, True])
@pytest.mark.parametrize("G", [-1, 32, 128, 48])
def test_quantize_dequantize_int4(sym, G):
    from ipex_amd.quantization import (
        WoqWeightDtype, dequantize_per_block, dequantize_per_channel, quantize_per_block, quantize_per_channel,
    )

    torch.manual_seed(0)
    N, K = 24, 200  # K % 48 != 0 and K % 128 != 0: trailing partial group
    w = torch.randn(N, K)
    if G == -1:
        qw, s, z = quantize_per_channel(w, WoqWeightDtype.INT4, None, None, sym)
        dq = dequantize_per_channel(qw, s, z, WoqWeightDtype.INT4, [N, K])
        assert s.shape == (N,)
    else:
        qw, s, z = quantize_per_block(w, WoqWeightDtype.INT4, G, None, None, sym)
        dq = dequantize_per_block(qw, s, z, WoqWeightDtype.INT4, G, [N, K])
        assert s.shape == (N, (K + G - 1) // G)
    assert qw.dtype == torch.uint8 and qw.shape == (N, K // 2)
    assert (z is None) == sym
    # the wire format is what the oracle decodes
    got = O.dequantize_woq_weight(qw.numpy(), N, K, s.numpy(), None if z is None else z.numpy(), 2, G)
    assert np.array_equal(got, dq.numpy())
    # quantization error is bounded by half a step (asym) / one step (sym, range -8..7 clamps +max)
    step = s.reshape(N, -1)
    g = (torch.arange(K) // G) if G > 0 else torch.zeros(K, dtype=torch.long)
    bound = step[:, g] * (1.001 if sym else 0.501)
    assert bool(((dq - w).abs() <= bound + 1e-6).all())
    if not sym:
        assert bool((z >= 0).all()) and bool((z <= 15).all())


def test_quantize_int8_per_channel_sym_and_asym():
    from ipex_amd.quantization import WoqWeightDtype, dequantize_per_channel, quantize_per_channel

    torch.manual_seed(1)
    w = torch.randn(16, 64)
    qw, s, z = quantize_per_channel(w, WoqWeightDtype.INT8, None, None, True)
    assert qw.dtype == torch.int8 and z is None
    assert torch.equal(s, w.abs().max(dim=1)[0] / 127)
    assert int(qw.abs().max()) == 127
    qw, s, z = quantize_per_channel(w, WoqWeightDtype.INT8, None, None, False)
    assert bool((z >= -128).all()) and bool((z <= 127).all())
    dq = dequantize_per_channel(qw, s, z, WoqWeightDtype.INT8)
    assert bool(((dq - w).abs() <= s.unsqueeze(1) * 0.501 + 1e-6).all())


def test_gptq_and_awq_converters_roundtrip():
    from ipex_amd.utils.weight_only_quantization import (
        AWQ_ORDER, _convert_awq_scales_qzeros, _convert_gptq_scales_qzeros, awq_to_plain, gptq_to_plain,
    )

    g = torch.Generator().manual_seed(0)
    K, N, G = 256, 64, 128
    q = torch.randint(0, 16, (N, K), generator=g)  # [N, K] codes
    zp = torch.randint(0, 16, (N, K // G), generator=g)
    plain = ((q[:, 1::2] << 4) | q[:, ::2]).to(torch.uint8)
    # GPTQ: word [j, n] nibble i = q[n, 8j + i]; zeros stored minus one
    qt = q.t().contiguous().view(K // 8, 8, N)
    gptq = torch.zeros(K // 8, N, dtype=torch.int64)
    for i in range(8):
        gptq |= qt[:, i, :] << (4 * i)
    gptq = gptq.to(torch.int32) if int(gptq.max()) < 2**31 else (gptq - (gptq >= 2**31) * 2**32).to(torch.int32)
    assert torch.equal(gptq_to_plain(gptq), plain)
    zt = ((zp - 1) % 16).t().contiguous().view(K // G, N // 8, 8)
    gz = torch.zeros(K // G, N // 8, dtype=torch.int64)
    for i in range(8):
        gz |= zt[:, :, i] << (4 * i)
    gz = (gz - (gz >= 2**31) * 2**32).to(torch.int32)
    s = torch.rand(K // G, N)
    s2, z2 = _convert_gptq_scales_qzeros(s, gz)
    assert torch.equal(s2, s.t()) and torch.equal(z2.long(), zp)
    # AWQ: word [k, j] nibble i = q[8j + ORDER[i], k]
    qa = q.t().contiguous().view(K, N // 8, 8)
    awq = torch.zeros(K, N // 8, dtype=torch.int64)
    for i in range(8):
        awq |= qa[:, :, AWQ_ORDER[i]] << (4 * i)
    awq = (awq - (awq >= 2**31) * 2**32).to(torch.int32)
    assert torch.equal(awq_to_plain(awq), plain)
    za = zp.t().contiguous().view(K // G, N // 8, 8)
    az = torch.zeros(K // G, N // 8, dtype=torch.int64)
    for i in range(8):
        az |= za[:, :, AWQ_ORDER[i]] << (4 * i)
    az = (az - (az >= 2**31) * 2**32).to(torch.int32)
    s3, z3 = _convert_awq_scales_qzeros(s, az)
    assert torch.equal(s3, s.t()) and torch.equal(z3.long(), zp)


def test_get_linear_parameters_per_checkpoint_kind():
    """utils/weight_only_quantization.py:_get_linear_parameters against checkpoints built from known codes."""
    import checkpoints as C
    from ipex_amd.nn.modules.weight_only_quantization import WoqWeightFormat
    from ipex_amd.utils import weight_only_quantization as W

    g = torch.Generator().manual_seed(1)
    N, K, G = 32, 256, 64
    q = torch.randint(0, 16, (N, K), generator=g)
    zp = torch.randint(0, 16, (N, K // G), generator=g)
    s = (0.01 * torch.rand(N, K // G, generator=g)).half()
    plain = ((q[:, 1::2] << 4) | q[:, ::2]).to(torch.uint8)
    # GPTQ without act-order: tensors stay in the GPTQ layout, parameters go to [N, groups]
    qw, sc, qz = C.gptq_layer(q, zp, s)
    sd = {"m.fc.qweight": qw, "m.fc.scales": sc, "m.fc.qzeros": qz, "m.fc.g_idx": torch.arange(K, dtype=torch.int32) // G,
          "m.fc.bias": torch.ones(N)}
    w, s2, z2, b, gs, gi, fmt = W._get_linear_parameters("m.fc", sd, W.GPTQ_LOWP_CHECKPOINT_CONFIG, {"quant_method": "gptq"})
    assert fmt == WoqWeightFormat.GPTQ_FORMAT and gs == G and gi is None and w is qw and torch.equal(b, torch.ones(N))
    assert torch.equal(s2, s) and torch.equal(z2.long(), zp)
    # ... with act-order: the plain layout (as int32 words along K) and g_idx kept
    perm = torch.randperm(K, generator=g)
    sd["m.fc.g_idx"] = (perm // G).to(torch.int32)
    w, s2, z2, _, gs, gi, fmt = W._get_linear_parameters("m.fc", sd, W.GPTQ_LOWP_CHECKPOINT_CONFIG, {"quant_method": "gptq"})
    assert fmt == WoqWeightFormat.PLAIN_FORMAT and gi is not None and gs == G
    assert torch.equal(w.contiguous().view(torch.uint8), plain) and torch.equal(z2.long(), zp)
    # ... and dropped when the config says there is none
    w, *_, gi, fmt = W._get_linear_parameters("m.fc", sd, dict(W.GPTQ_LOWP_CHECKPOINT_CONFIG, desc_act=False), {"quant_method": "gptq"})
    assert gi is None and fmt == WoqWeightFormat.GPTQ_FORMAT
    # AWQ
    qw, sc, qz = C.awq_layer(q, zp, s)
    sd = {"m.fc.qweight": qw, "m.fc.scales": sc, "m.fc.qzeros": qz}
    w, s2, z2, b, gs, gi, fmt = W._get_linear_parameters("m.fc", sd, W.AWQ_LOWP_CHECKPOINT_CONFIG, {"quant_method": "awq"})
    assert fmt == WoqWeightFormat.AWQ_FORMAT and gs == G and gi is None and b is None and w is qw
    assert torch.equal(s2, s) and torch.equal(z2.long(), zp)
    # DeepSeek FP8: one scale per 16 x 64 block -> one per row and block of 64 columns
    wf = torch.randn(40, 128, generator=g)
    q8, sinv, dq = C.fp8_layer(wf, 16, 64)
    sd = {"m.fc.weight": q8, "m.fc.weight_scale_inv": sinv}
    w, s2, z2, b, gs, gi, fmt = W._get_linear_parameters("m.fc", sd, W.FP8_LOWP_CHECKPOINT_CONFIG,
                                                        {"quant_method": "fp8", "weight_block_size": [16, 64]})
    assert w is q8 and z2 is None and gs == 64 and fmt == WoqWeightFormat.PLAIN_FORMAT and tuple(s2.shape) == (40, 2)
    assert torch.equal((q8.float().view(40, 2, 64) * s2[:, :, None]).view(40, 128), dq)
    # round to nearest, 8 bits: int8 along K four per word, zero points stored minus one as uint8
    q8i = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
    z8 = torch.randint(0, 256, (N, K // G), generator=g)
    sd = {"m.fc.qweight": q8i.contiguous().view(torch.int32).t().contiguous(),
          "m.fc.scales": s.t().contiguous().float(),
          "m.fc.qzeros": ((z8 - 1) % 256).to(torch.uint8).t().contiguous().view(torch.int32)}
    w, s2, z2, _, gs, gi, fmt = W._get_linear_parameters("m.fc", sd, W.RTN_LOWP_CHECKPOINT_CONFIG, {"quant_method": "rtn", "bits": 8})
    assert w.dtype == torch.int8 and torch.equal(w, q8i) and gs == G and gi is None
    assert torch.equal(z2.view(torch.uint8).long(), z8 % 256) and torch.equal(s2, s.float())
    # per-channel INT8 and a layer the checkpoint keeps in floating point
    sd = {"m.fc.weight": q8i, "m.fc.weight_scale": torch.rand(N, 1), "m.head.weight": torch.randn(8, N)}
    w, s2, z2, _, gs, _, _ = W._get_linear_parameters("m.fc", sd, W.INT8_LOWP_CHECKPOINT_CONFIG, {"quant_method": "int8"})
    assert w is q8i and gs == -1 and z2 is None and tuple(s2.shape) == (N, 1)
    w, s2, *_ = W._get_linear_parameters("m.head", sd, W.INT8_LOWP_CHECKPOINT_CONFIG, {"quant_method": "int8"})
    assert s2 is None and w is sd["m.head.weight"]


def test_c_port_of_oracle_matches_numpy_oracle():
    import ctypes

    so = os.path.join(ROOT, "oracle", "libwoq_oracle.so")
    if not os.path.exists(so):
        pytest.skip("oracle/libwoq_oracle.so not built")
    lib = ctypes.CDLL(so)
    rng = np.random.default_rng(0)
    M, K, N, G = 3, 512, 40, 128
    x = O.bf16_round(rng.standard_normal((M, K)).astype(np.float32))
    q = rng.integers(0, 16, (N, K)).astype(np.uint8)
    qw = O.pack_int4(q)
    sc = O.bf16_round((0.005 + 0.015 * rng.random((N, K // G))).astype(np.float32))
    zp = rng.integers(0, 16, (N, K // G)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    xb = O.f32_to_bf16_bits(x)
    acc = np.zeros((M, N), dtype=np.float32)
    vp, i64 = ctypes.c_void_p, ctypes.c_int64
    lib.woq_ref_linear_int4.argtypes = [vp, i64, i64, i64, vp, vp, vp, i64, vp, ctypes.c_int, i64, i64, vp]
    for regime, cd in ((1, "bf16"), (0, "fp16")):
        lib.woq_ref_linear_int4(xb.ctypes.data, M, K, N, qw.ctypes.data, sc.ctypes.data, zp.ctypes.data, G,
                                bias.ctypes.data, regime, 0, N, acc.ctypes.data)
        want, _ = O.woq_linear_ref(x, "bf16", qw, N, K, sc, zp, bias, 2, G, cd)
        assert np.max(np.abs(acc - want)) < 1e-4
    # the optimized fp16 kernel's chain of fp16 fused multiply-adds: the same bits as the numpy restatement
    lib.woq_ref_linear_int4_fp16_chain.argtypes = [vp, i64, i64, i64, vp, vp, vp, i64, i64, vp, i64, i64, vp]
    for b in (bias, None):
        lib.woq_ref_linear_int4_fp16_chain(xb.ctypes.data, M, K, N, qw.ctypes.data, sc.ctypes.data, zp.ctypes.data, G, 64,
                                           None if b is None else b.ctypes.data, 0, N, acc.ctypes.data)
        assert np.array_equal(O.bf16_round(acc), O.woq_linear_opt_fp16(x, qw, N, K, sc, zp, b, 2, G))
    # int8 path: quantization and block sums are exact, epilogue to fp32 rounding
    xq = np.zeros((M, K), dtype=np.int8)
    sa = np.zeros(M, dtype=np.float32)
    lib.woq_ref_quant_per_row.argtypes = [vp, i64, i64, vp, vp]
    lib.woq_ref_quant_per_row(xb.ctypes.data, M, K, xq.ctypes.data, sa.ctypes.data)
    r = O.woq_linear_opt_int8(x, "bf16", qw, N, K, sc, zp, bias, 2, G, 6)
    assert np.array_equal(xq, r["xq"]) and np.array_equal(sa, r["sa"])
    lib.woq_ref_linear_int4_int8.argtypes = [vp, vp, i64, i64, i64, vp, vp, vp, i64, i64, vp, i64, i64, vp]
    lib.woq_ref_linear_int4_int8(xq.ctypes.data, sa.ctypes.data, M, K, N, qw.ctypes.data, sc.ctypes.data,
                                 zp.ctypes.data, G, 128, bias.ctypes.data, 0, N, acc.ctypes.data)
    assert np.array_equal(acc, r["acc"])


def test_product_refuses_to_run_without_gpu():
    import ipex_amd  # noqa: F401
    from ipex_amd import _kernels, ops

    if torch.cuda.is_available():
        pytest.skip("GPU present")
    with pytest.raises(RuntimeError, match="GPU"):
        ops.WoqLinearOpContext(torch.zeros(16, 64, dtype=torch.uint8), 2, [16, 128], torch.ones(16), None, None,
                               None, None, -1, 2, -1)
    with pytest.raises(RuntimeError, match="GPU"):
        torch.ops.torch_ipex.ipex_woq_linear(torch.zeros(1, 128, dtype=torch.bfloat16), torch.tensor([1]))
    with pytest.raises(RuntimeError, match="GPU"):
        _kernels.pack_weight(torch.zeros(16, 64, dtype=torch.uint8), 2, 16, 128)


def test_ops_are_registered_with_reference_schemas():
    import ipex_amd  # noqa: F401

    s = str(torch.ops.torch_ipex.ipex_woq_linear.default._schema)
    assert s == "torch_ipex::ipex_woq_linear(Tensor input, Tensor W_prepack) -> Tensor"
    for name in ("woq_linear_gelu", "woq_linear_new_gelu", "woq_linear_relu", "woq_linear_silu"):
        assert "(Tensor input, Tensor W_prepack) -> Tensor" in str(getattr(torch.ops.torch_ipex, name).default._schema)
    for name in ("woq_linear_add", "woq_linear_add_add", "woq_linear_mul"):
        assert "(Tensor input, Tensor W_prepack, Tensor[] others) -> Tensor" in str(
            getattr(torch.ops.torch_ipex, name).default._schema
        )
    assert hasattr(torch.ops.torch_ipex, "woq_linear")
    assert "dequantize_nf4(Tensor t, Tensor scales, int group_size, ScalarType out_dtype) -> Tensor" in str(
        torch.ops.torch_ipex.dequantize_nf4.default._schema)
    # registered by the C++ binding, with the custom class the prepack operators return
    assert "__torch__.torch.classes.ipex_prepack.WoqLinearOpContext" in str(
        torch.ops.ipex_prepack.weight_only_qlinear_prepack.default._schema)
    assert torch.classes.ipex_prepack.WoqLinearOpContext is not None
    assert torch._C._dispatch_has_kernel_for_dispatch_key("torch_ipex::ipex_woq_linear", "CUDA")
    assert torch._C._dispatch_has_kernel_for_dispatch_key("torch_ipex::ipex_woq_linear", "AutocastCUDA")
    for name in ("weight_only_qlinear_prepack", "weight_only_qlinear_prepack_int4", "woq_linear_pack_weight",
                 "woq_linear_unpack_weight"):
        assert hasattr(torch.ops.ipex_prepack, name)


def test_auto_split_k_predicate_is_the_library_s():
    """The problems on which woq_hip_linear shares K between workgroups by itself, asked of the library (pure host
    arithmetic): few output tiles and a long K; everything else gets no scratch."""
    from ipex_amd import _lib

    lib = _lib.load()
    f = lib.woq_hip_linear_auto_split_k_workspace_bytes
    full = lib.woq_hip_linear_split_k_workspace_bytes
    BF16, INT8 = _lib.LOWP_BF16, _lib.LOWP_INT8
    assert f(16, 14336, 4096, BF16) == full(16, 4096) > 0  # down projection at decode
    assert f(16, 4096, 14336, BF16) == 0  # enough row-blocks
    assert f(16, 4096, 4096, BF16) == 0  # K too short
    assert f(4, 14336, 4096, BF16) == 0  # fewer than five rows: the integer-weight decode kernels never split
    assert f(33, 14336, 4096, BF16) == 0
    assert f(16, 14336, 4096, INT8) == 0  # the int8 decode kernel does not split
    assert f(128, 4096, 4096, BF16) == full(128, 4096) > 0
    assert f(128, 4096, 4096, INT8) == full(128, 4096)
    assert f(2048, 4096, 14336, BF16) == 0
    assert f(128, 2048, 4096, BF16) == 0


def test_environment_knobs_of_the_reference_are_read_by_the_library():
    """IPEX_WOQ_SMALL_BATCH_THRESHOLD (csrc/cpu/aten/utils/woq.h:24) and IPEX_WOQ_WEIGHT_CACHE_BATCH_THRESHOLD
    (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:17-18) are read once per process by the library; values that are
    not whole numbers leave the defaults (5 and 64).  Each setting in a process of its own."""
    import subprocess
    import sys

    code = (
        "import sys; sys.path.insert(0, %r); from ipex_amd import _lib; lib = _lib.load(); "
        "print(lib.woq_hip_small_batch_threshold(), lib.woq_hip_weight_cache_batch_threshold())"
    ) % os.path.join(ROOT, "intel-extension-for-pytorch_amd")

    def run(**env):
        e = {k: v for k, v in os.environ.items() if not k.startswith("IPEX_WOQ_")}
        e.update(env)
        out = subprocess.run([sys.executable, "-c", code], env=e, capture_output=True, text=True, timeout=120)
        assert out.returncode == 0, out.stderr[-2000:]
        return out.stdout.split()[-2:]

    assert run() == ["5", "64"]
    assert run(IPEX_WOQ_SMALL_BATCH_THRESHOLD="9", IPEX_WOQ_WEIGHT_CACHE_BATCH_THRESHOLD="256") == ["9", "256"]
    assert run(IPEX_WOQ_SMALL_BATCH_THRESHOLD="many", IPEX_WOQ_WEIGHT_CACHE_BATCH_THRESHOLD="-3") == ["5", "64"]
