"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on identical inputs.

Bars: integer results (pack / unpack, activation quantization, int32 block sums) bit-exact;
fp32 accumulators max-abs <= 1e-2; bf16 outputs relative-L2 <= 2e-3 (two correct
implementations with different summation orders can differ by one bf16 ulp, which at
|y| in [8, 16) is 0.0625, so the max-abs bar is applied to the accumulators).
"""
import pickle

import numpy as np
import pytest
import torch

from helpers import bf16_ulp_diff, case_np, make_context, make_torch_context, max_abs, rel_l2, to_np_f32
from oracle import woq_oracle as O

pytestmark = pytest.mark.gpu

MAX_ABS_ACC = 1e-2
REL_L2_OUT = 2e-3


def _kernels():
    from ipex_amd import _kernels

    return _kernels


def _lib_last_kernel():
    from ipex_amd import _lib

    return _lib.last_kernel()


def _synthetic():
    from ipex_amd.utils import synthetic

    return synthetic


def _lib_mod():
    from ipex_amd import _lib

    return _lib


# ---------------------------------------------------------------------------------------------
# prepack: integer-exact, invertible
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("N,K", [(16, 128), (4096, 4096), (500, 4096), (33, 200), (1, 2), (48, 4095)])
def test_int4_pack_unpack_roundtrip(cuda, N, K):
    k = _kernels()
    g = torch.Generator().manual_seed(N * 7 + K)
    plain = torch.randint(0, 256, (N, (K + 1) // 2), dtype=torch.uint8, generator=g)
    if K % 2:
        plain[:, -1] &= 0x0F  # the pad nibble of an odd K is zero in the format
    packed = k.pack_weight(plain.to(cuda), 2, N, K)
    assert packed.shape == ((N + 15) // 16, (K + 127) // 128, 1024)
    back = k.unpack_weight(packed, 2, N, K)
    assert torch.equal(back.cpu(), plain)


def test_int4_pack_layout_matches_definition(cuda):
    # lane l = r + 16c owns row r, K offsets 32c..32c+31; dword j holds offsets 8j..8j+7 with
    # element e in nibble (e even ? e/2 : 4 + e/2)
    k = _kernels()
    N, K = 32, 256
    q = torch.randint(0, 16, (N, K), dtype=torch.uint8, generator=torch.Generator().manual_seed(1))
    plain = (q[:, 1::2] << 4) | q[:, ::2]
    packed = k.pack_weight(plain.to(cuda), 2, N, K).cpu().numpy().view(np.uint32).reshape(2, 2, 64, 4)
    qn = q.numpy()
    for nt, kt, lane, j in [(0, 0, 0, 0), (1, 1, 37, 3), (0, 1, 63, 2), (1, 0, 16, 1)]:
        r, c = lane % 16, lane // 16
        word = int(packed[nt, kt, lane, j])
        for e in range(8):
            pos = e // 2 if e % 2 == 0 else 4 + e // 2
            assert (word >> (4 * pos)) & 0xF == qn[nt * 16 + r, kt * 128 + c * 32 + j * 8 + e]


@pytest.mark.parametrize("N,K", [(16, 64), (11008, 4096), (37, 100)])
def test_int8_pack_unpack_roundtrip(cuda, N, K):
    k = _kernels()
    plain = torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=torch.Generator().manual_seed(N + K))
    packed = k.pack_weight(plain.to(cuda), 1, N, K)
    assert torch.equal(k.unpack_weight(packed, 1, N, K).cpu(), plain)


def test_qparams_layout(cuda):
    k = _kernels()
    N, KG = 40, 3
    s = torch.rand(N, KG) + 0.5
    z = torch.randint(0, 16, (N, KG)).float()
    s32, s16, sb16, z8, sz, szb = k.pack_qparams(s.to(cuda), z.to(cuda), 2)
    assert s32.shape == (3, KG, 16)
    sp = torch.ones(48, KG)
    sp[:N] = s
    zp = torch.zeros(48, KG)
    zp[:N] = z
    assert torch.equal(s32.cpu(), sp.view(3, 16, KG).permute(0, 2, 1))
    assert torch.equal(s16.cpu(), sp.view(3, 16, KG).permute(0, 2, 1).half())
    assert torch.equal(sb16.cpu(), sp.view(3, 16, KG).permute(0, 2, 1).bfloat16())
    assert torch.equal(z8.cpu().float(), zp.view(3, 16, KG).permute(0, 2, 1))
    halves = sz.cpu().view(torch.float16).view(3, KG, 16, 2)
    assert torch.equal(halves[..., 0], s16.cpu())
    want_z = 128 + zp.view(3, 16, KG).permute(0, 2, 1)
    assert torch.equal(halves[..., 1].float(), want_z)
    # the bf16 kernels' dword: bf16 scale in the high half, the fp16 number 1024 + zero in the low half
    m = szb.cpu()
    assert torch.equal((m >> 16).to(torch.int16).view(torch.bfloat16), sb16.cpu())
    assert torch.equal((m & 0xFFFF).to(torch.int16).view(torch.float16).float(), 1024 + zp.view(3, 16, KG).permute(0, 2, 1))
    # symmetric 4-bit weights: the code of zero is 8; 8-bit weights: the stored byte (offset-binary), 128 when symmetric
    assert torch.equal((k.pack_qparams(s.to(cuda), None, 2)[5].cpu() & 0xFFFF)[:2], torch.full((2, KG, 16), 0x6408, dtype=torch.int32))
    z8b = torch.randint(-128, 128, (N, KG)).float()
    m8 = k.pack_qparams(s.to(cuda), z8b.to(cuda), 1)[5].cpu()
    zp8 = torch.zeros(48, KG)
    zp8[:N] = z8b
    assert torch.equal((m8 & 0xFFFF).to(torch.int16).view(torch.float16).float(), 128 + zp8.view(3, 16, KG).permute(0, 2, 1))
    assert torch.equal((k.pack_qparams(s.to(cuda), None, 1)[5].cpu() & 0xFFFF), torch.full((3, KG, 16), 0x5800, dtype=torch.int32))
    assert k.pack_qparams(s.to(cuda), None, 3)[5] is None  # NF4: no such table


def test_compressed_zero_points(cuda):
    k = _kernels()
    zp32 = torch.randint(-(2**31), 2**31 - 1, (9, 5), dtype=torch.int32, generator=torch.Generator().manual_seed(2))
    got = k.unpack_int4_zeros(zp32.to(cuda), 37).cpu().numpy()
    assert np.array_equal(got, O.unpack_compressed_zeros(zp32.numpy(), 37))


@pytest.mark.parametrize("G", [32, 128, -1])
def test_dequant_weight_bit_exact(cuda, G):
    syn, k = _synthetic(), _kernels()
    case = syn.make_int4_case(9, 1, 512, 80, G, scale_dtype=torch.float32)
    ctx = make_context(case, 2)
    c = case_np(case)
    want = O.dequantize_woq_weight(c["qw"], 80, 512, c["scales"], c["zps"], 2, G)
    got = k.dequant_weight(ctx.at_weight_, 2, 80, 512, ctx.scales_list_[0], ctx.zeros_u8_, G)
    assert np.array_equal(got.cpu().numpy(), want)
    got16 = k.dequant_weight(ctx.at_weight_, 2, 80, 512, ctx.scales_list_[0], ctx.zeros_u8_, G, torch.bfloat16)
    assert np.array_equal(to_np_f32(got16), O.bf16_round(want))


# ---------------------------------------------------------------------------------------------
# floating-point paths
# ---------------------------------------------------------------------------------------------
def _shipped_binding_output(case, lowp_mode, act_quant_mode=-1, g_idx=None):
    """The same call through what a user of the package gets: the registered prepack operator, the TorchScript custom
    class it returns and torch.ops.torch_ipex.ipex_woq_linear (lib/libwoq_torch.so)."""
    tctx = make_torch_context(case, lowp_mode, act_quant_mode, g_idx=g_idx)
    return torch.ops.torch_ipex.ipex_woq_linear(case["x"].cuda(), tctx.get_data_handle())


def _check_fp(case, lowp_mode, ctx=None, cols=None, force_kernel=0, label="", shipped=False):
    """Runs the HIP path twice (output dtype and fp32 accumulator) and checks both oracles.  ``shipped``: the output
    of the registered operator on the custom class must equal, bit for bit, the output of the ctypes twin that the
    oracle comparisons below are made on."""
    k = _kernels()
    ctx = ctx or make_context(case, lowp_mode)
    x = case["x"].cuda()
    N, K, G = case["N"], case["K"], case["group_size"]
    kw = dict(force_kernel=force_kernel)
    y_t = ctx.run(x, **kw)
    if shipped:
        assert force_kernel == 0
        y_s = _shipped_binding_output(case, lowp_mode)
        assert y_s.dtype == y_t.dtype and torch.equal(y_s, y_t), (label, "registered operator differs from the ctypes twin")
    y = to_np_f32(y_t)
    acc = ctx.run(x, out_fp32=True, **kw).cpu().numpy()
    c = case_np(case)
    M = c["x"].shape[0]
    cd = O.select_compute(lowp_mode, "bf16", M)
    qw, sc, zp, b = c["qw"], c["scales"], c["zps"], c["bias"]
    if cols is not None:  # check a subset of output columns against the oracle
        qw, sc = qw[cols], sc[cols]
        zp = None if zp is None else zp[cols]
        b = None if b is None else b[cols]
        y, acc = y[:, cols], acc[:, cols]
        N = len(cols)
    wd = case["weight_dtype"]
    # The optimized kernels read the scales in the compute dtype (ContextLinearWoq.h:104-106) and
    # so does the HIP path; the fallback keeps fp32 scales.  The fallback oracle is therefore
    # evaluated with the scales rounded the same way (a no-op for fp16 / bf16 checkpoints), and
    # the distance to the unrounded-scale fallback is reported.
    sc_cd = O._round_to(sc, cd)
    acc_ref, y_ref = O.woq_linear_ref(c["x"], "bf16", qw, N, K, sc_cd, zp, b, wd, G, cd)
    stats = {"max_abs_acc_vs_ref": max_abs(acc, acc_ref), "rel_l2_out_vs_ref": rel_l2(y, y_ref)}
    if not np.array_equal(sc_cd, sc):
        acc_f32s, _ = O.woq_linear_ref(c["x"], "bf16", qw, N, K, sc, zp, b, wd, G, cd)
        stats["max_abs_acc_vs_ref_fp32_scales"] = max_abs(acc, acc_f32s)
    assert stats["max_abs_acc_vs_ref"] <= MAX_ABS_ACC, (label, stats)
    # fp16 regime: the HIP path follows the fallback's rounding chain (fp16 result, fp16 bias add,
    # cast).  bf16 regime: it follows the optimized kernel (fp32 bias, one rounding), which the
    # fallback's extra bf16 rounding of a biased result does not match to 2e-3.
    if cd == "fp16" or b is None:
        assert stats["rel_l2_out_vs_ref"] <= REL_L2_OUT, (label, stats)
    if cd == "bf16":
        acc_opt, y_opt = O.woq_linear_opt_bf16(c["x"], "bf16", qw, N, K, sc, zp, b, wd, G)
        stats["max_abs_acc_vs_opt"] = max_abs(acc, acc_opt)
        stats["rel_l2_out_vs_opt"] = rel_l2(y, y_opt)
        ulps = bf16_ulp_diff(y, y_opt)
        stats["out_ulp_max_vs_opt"] = int(ulps.max())
        stats["out_exact_frac_vs_opt"] = float((ulps == 0).mean())
        assert stats["max_abs_acc_vs_opt"] <= MAX_ABS_ACC, (label, stats)
        assert stats["rel_l2_out_vs_opt"] <= REL_L2_OUT, (label, stats)
        # one bf16 ulp at most, except next to zero where an ulp is far below the accumulator bar
        assert bool(np.all((ulps <= 1) | (np.abs(y - y_opt) <= 1e-4))), (label, stats)
    elif wd in (2, 3) and M <= 4 and N * K <= 4096 * 4096:
        # the optimized fp16 kernel accumulates in fp16; its own rounding noise exceeds 1e-2 at
        # these magnitudes, so only the relative-L2 bar applies against it
        y_h = O.woq_linear_opt_fp16(c["x"], qw, N, K, sc, zp, b, wd, G)
        stats["rel_l2_out_vs_opt_fp16"] = rel_l2(y, y_h)
        stats["max_abs_out_vs_opt_fp16"] = max_abs(y, y_h)
        assert stats["rel_l2_out_vs_opt_fp16"] <= 6e-3, (label, stats)
    print(label, stats)
    return stats


@pytest.mark.parametrize(
    "kind,M,K,N,G,sym,bias",
    [("int4", 16, 1024, 272, 128, False, True), ("int4", 8, 512, 96, 32, False, False), ("int4", 32, 384, 48, -1, True, True),
     ("int4", 64, 1024, 544, 64, False, False), ("int4", 200, 1024, 512, 128, False, True), ("int4", 130, 512, 300, 32, True, False),
     ("int4", 2048, 512, 448, 256, False, False), ("int8", 32, 512, 176, -1, True, True), ("int8", 7, 256, 64, 64, False, False)],
)
def test_merged_scale_zero_table_changes_no_bit(cuda, kind, M, K, N, G, sym, bias):
    """The bf16 kernels read scale and zero point from one dword when the caller passes the merged table and from two
    arrays when it does not (the registered woq_linear operator of the reference's argument list): the same bits out."""
    syn = _synthetic()
    if kind == "int4":
        case = syn.make_int4_case(11, M, K, N, G, bias=bias)
        if sym:
            case["zeros"] = None
    else:
        case = syn.make_int8_case(11, M, K, N, group_size=G, bias=bias)
        if not sym:
            case["zeros"] = torch.randint(-128, 128, case["scales"].shape, generator=torch.Generator().manual_seed(5)).float()
    ctx = make_context(case, O.LOWP_BF16)
    assert ctx.scale_zero_bf16_ is not None
    x = case["x"].cuda()
    with_table = ctx.run(x, out_fp32=True)
    kernel = _lib_last_kernel()
    table, ctx.scale_zero_bf16_ = ctx.scale_zero_bf16_, None
    without = ctx.run(x, out_fp32=True)
    assert _lib_last_kernel() == kernel
    ctx.scale_zero_bf16_ = table
    assert torch.equal(with_table, without), (kernel, (with_table - without).abs().max().item())


# ---------------------------------------------------------------------------------------------
# cache_weight_for_large_batch: the dense bf16 copy and the kernel that runs on it
# ---------------------------------------------------------------------------------------------
def _dense_case(kind, M, K, N, G, sym=False, bias=False, seed=21):
    syn = _synthetic()
    if kind == "int4":
        case = syn.make_int4_case(seed, M, K, N, G, bias=bias)
        if sym:
            case["zeros"] = None
    elif kind == "int8":
        case = syn.make_int8_case(seed, M, K, N, group_size=G, bias=bias)
        if not sym:
            case["zeros"] = torch.randint(-128, 128, case["scales"].shape, generator=torch.Generator().manual_seed(5)).float()
    elif kind == "nf4":
        case = syn.make_nf4_case(seed, M, K, N, G, bias=bias)
    else:
        case = syn.make_fp8_case(seed, M, K, N, bias=bias, group_size=G)
    return case


def _dense_copy_as_matrix(dense, N, K, wbits):
    """[K / 128, NT, 4, 64, 8] fragments -> [padded N, K]: fragment (kt, nt, j, lane) holds row 16 nt + lane % 16 and
    the K values 128 kt + 8 chunk .. + 7 with chunk = 4 (lane / 16) + j for 4-bit codes and
    8 (j / 2) + 2 (lane / 16) + j % 2 for bytes."""
    d = dense.view(torch.int16).cpu().numpy().view(np.uint16)
    KT, NT = d.shape[0], d.shape[1]
    out = np.zeros((NT * 16, K), dtype=np.uint16)
    for j in range(4):
        for c in range(4):
            chunk = 4 * c + j if wbits == 4 else 8 * (j // 2) + 2 * c + (j % 2)
            for kt in range(KT):
                k0 = 128 * kt + 8 * chunk
                # lanes 16 c .. 16 c + 15 are rows 0..15 of every row-block
                out[:, k0:k0 + 8] = d[kt, :, j, 16 * c:16 * c + 16, :].reshape(NT * 16, 8)
    return out


@pytest.mark.parametrize(
    "kind,K,N,G,sym",
    [("int4", 512, 80, 128, False), ("int4", 256, 33, 32, True), ("int4", 384, 48, -1, False), ("int8", 256, 40, -1, True),
     ("int8", 512, 32, 128, False), ("nf4", 256, 48, 64, True), ("fp8", 384, 24, 128, True)],
)
def test_dense_copy_is_the_bf16_dequantized_weight(cuda, kind, K, N, G, sym):
    """The copy that cache_weight_for_large_batch keeps (LinearWoqPacked.cpp:430-486) against the oracle's
    dequantization with the bf16 scales, bit for bit, through the documented fragment layout."""
    case = _dense_case(kind, 4, K, N, G, sym=sym)
    ctx = make_context(case, O.LOWP_BF16, cache=True)
    dense = ctx.get_cached_weight()
    NT = (N + 15) // 16
    assert dense is not None and tuple(dense.shape) == (K // 128, NT, 4, 64, 8) and dense.dtype == torch.bfloat16
    c = case_np(case)
    w = O.dequantize_woq_weight(c["qw"], N, K, O._round_to(c["scales"], "bf16"), c["zps"], case["weight_dtype"], G)
    want = O.f32_to_bf16_bits(w)
    got = _dense_copy_as_matrix(dense, N, K, 8 if kind in ("int8", "fp8") else 4)
    assert np.array_equal(got[:N], want), kind


@pytest.mark.parametrize(
    "kind,M,K,N,G,sym,bias",
    [("int4", 130, 512, 448, 128, False, True), ("int4", 128, 1024, 500, 32, True, False),
     ("int4", 257, 384, 300, -1, False, True), ("int4", 64, 256, 1024, 64, False, False),
     ("int8", 96, 512, 272, 128, True, True), ("int8", 200, 256, 128, -1, False, False),
     ("int4", 70, 128, 176, 128, False, True), ("int4", 5, 256, 64, 32, False, False),
     # more than 256 workgroups of the narrowest shape (its variant without the deeper activation prefetch)
     ("int4", 2100, 256, 2064, 128, False, True), ("int4", 300, 640, 200, 128, False, False)],
)
@pytest.mark.parametrize("shape_kernels", [(24, 4), (25, 5), (26, 6)])
def test_dense_kernel_equals_the_dequantizing_prefill_kernel_bit_for_bit(cuda, kind, M, K, N, G, sym, bias, shape_kernels):
    """woq_gemm_dense_kernel on the copy feeds the MFMAs the operands that woq_gemm_w4_kernel dequantizes on the fly,
    in the same order: fp32 accumulators and rounded outputs are equal for every workgroup shape (ragged M, N and the
    row-blocks past N included), with and without bias."""
    dense_k, w4_k = shape_kernels
    if kind == "int8" and w4_k == 4:
        pytest.skip("8-bit weights have no 448-column shape in the dequantizing kernel")
    case = _dense_case(kind, M, K, N, G, sym=sym, bias=bias)
    ctx = make_context(case, O.LOWP_BF16, cache=True)
    x = case["x"].cuda()
    for fp32 in (True, False):
        y_dense = ctx.run(x, out_fp32=fp32, force_kernel=dense_k)
        assert _lib_last_kernel() == "woq_gemm_dense_kernel"
        y_w4 = ctx.run(x, out_fp32=fp32, force_kernel=w4_k)
        assert _lib_last_kernel() == "woq_gemm_w4_kernel"
        assert torch.equal(y_dense, y_w4), (kind, fp32, (y_dense.float() - y_w4.float()).abs().max().item())


@pytest.mark.parametrize("kind,G", [("nf4", 64), ("fp8", 128), ("int4", 128)])
def test_dense_kernel_against_the_oracle(cuda, kind, G):
    """Every weight format through the dense kernel (force_kernel 23) against the optimized bf16 oracle, to the bars
    of the other bf16 kernels; NF4 and FP8 have no dequantizing prefill kernel of the same accumulation order to be
    compared with bit for bit."""
    case = _dense_case(kind, 150, 512, 176, G, sym=True, bias=True)
    ctx = make_context(case, O.LOWP_BF16, cache=True)
    _check_fp(case, O.LOWP_BF16, ctx=ctx, force_kernel=23, label=f"dense {kind}")
    assert _lib_last_kernel() == "woq_gemm_dense_kernel"


def test_dense_kernel_post_ops_equal_the_dequantizing_kernel(cuda):
    lib = _lib_mod()
    case = _dense_case("int4", 160, 256, 144, 128, bias=True)
    ctx = make_context(case, O.LOWP_BF16, cache=True)
    x = case["x"].cuda()
    g = torch.Generator().manual_seed(3)
    o0 = torch.randn(160, 144, generator=g).to(torch.bfloat16).cuda()
    o1 = torch.randn(160, 144, generator=g).to(torch.bfloat16).cuda()
    for fusion, others in [(lib.FUSE_GELU_ERF, ()), (lib.FUSE_SILU, ()), (lib.FUSE_ADD, (o0,)), (lib.FUSE_MUL, (o0,)),
                           (lib.FUSE_ADD_ADD, (o0, o1))]:
        a = ctx.run(x, fusion=fusion, others=others, force_kernel=23)
        assert _lib_last_kernel() == "woq_gemm_dense_kernel"
        b = ctx.run(x, fusion=fusion, others=others, force_kernel=3)
        assert torch.equal(a, b), fusion


def test_weight_cache_serves_large_batches_only(cuda):
    """With the copy, lowp_mode BF16 runs batches of at least IPEX_WOQ_WEIGHT_CACHE_BATCH_THRESHOLD rows (64) on the
    dense kernel where the library's cost models make it the faster one (its 128-row tiles must fill the chip: here
    1536 rows on a wide layer); smaller ones and contexts without the flag stay on the kernels that read the packed
    weight.  Same bits either way."""
    lib = _lib_mod().load()
    assert lib.woq_hip_weight_cache_batch_threshold() == 64
    case = _dense_case("int4", 1536, 512, 7168, 128)
    cached, plain = make_context(case, O.LOWP_BF16, cache=True), make_context(case, O.LOWP_BF16)
    assert plain.get_cached_weight() is None
    x = case["x"].cuda()
    y = cached.run(x)
    assert _lib_last_kernel() == "woq_gemm_dense_kernel"
    y_plain = plain.run(x)
    assert _lib_last_kernel() == "woq_gemm_w4_kernel"
    assert torch.equal(y, y_plain)
    for rows in (1, 16, 63, 200):
        y = cached.run(x[:rows])
        assert _lib_last_kernel() != "woq_gemm_dense_kernel", rows
        assert torch.equal(y, plain.run(x[:rows])), rows
    # lowp_mode INT8 and K that is no multiple of 128 keep no copy (LinearWoqPacked.cpp:443-447 has its own conditions)
    assert make_context(case, O.LOWP_INT8, act_quant_mode=6, cache=True).get_cached_weight() is None
    odd = _dense_case("int4", 8, 192, 64, 64)
    assert make_context(odd, O.LOWP_BF16, cache=True).get_cached_weight() is None
    # a forced dense kernel without a copy is an error, not a fallback
    with pytest.raises(RuntimeError, match="dense"):
        plain.run(x, force_kernel=23)


def test_weight_cache_with_act_order(cuda):
    """GPTQ act-order with cache_weight_for_large_batch: the dense copy is made from the weight whose input channels
    are already sorted by group, and the activations are shuffled per call as without the copy -- same bits as the
    context without the flag, through the dense kernel."""
    from ipex_amd import ops

    M, K, N, G = 200, 512, 160, 128
    case = _synthetic().make_int4_case(33, M, K, N, G, bias=True)
    perm = torch.randperm(K, generator=torch.Generator().manual_seed(9))
    g_idx = (torch.arange(K) // G)[perm]
    make = lambda cache: ops.WoqLinearOpContext(
        case["qweight"].cuda(), 2, [N, K], case["scales"].cuda(), case["zeros"].cuda(), case["bias"].cuda(),
        g_idx, None, G, O.LOWP_BF16, -1, cache)
    cached, plain = make(True), make(False)
    assert cached.get_cached_weight() is not None and plain.get_cached_weight() is None
    x = case["x"].cuda()
    y = cached.run(x, force_kernel=23)
    assert _lib_last_kernel() == "woq_gemm_dense_kernel"
    assert torch.equal(y, plain.run(x, force_kernel=3))


def test_c3_prefill_bf16_with_weight_cache(cuda):
    """The named prefill configuration with cache_weight_for_large_batch: served by the dense kernel, equal bit for
    bit to the run without the flag, and within the bars of the oracle like that one."""
    case = _synthetic().make_int4_case(3, 2048, 4096, 14336, 128, outliers=True)
    ctx = make_context(case, O.LOWP_BF16, cache=True)
    x = case["x"].cuda()
    y = ctx.run(x)
    assert _lib_last_kernel() == "woq_gemm_dense_kernel"
    y_plain = make_context(case, O.LOWP_BF16).run(x)
    assert _lib_last_kernel() == "woq_gemm_w4_kernel"
    assert torch.equal(y, y_plain)
    _check_fp(case, O.LOWP_BF16, ctx=ctx, cols=np.arange(0, 14336, 29), label="C3 bf16 dense")
    assert _lib_last_kernel() == "woq_gemm_dense_kernel"
    # the same through the registered prepack operator, the custom class and torch.ops (the copy is made by the C++
    # binding at prepack time and handed to the library on every call)
    tctx = make_torch_context(case, O.LOWP_BF16, cache=True)
    y_shipped = torch.ops.torch_ipex.ipex_woq_linear(x, tctx.get_data_handle())
    assert _lib_last_kernel() == "woq_gemm_dense_kernel"
    assert y_shipped.dtype == y.dtype and torch.equal(y_shipped, y)
    cached = tctx.get_cached_weight()
    assert cached is not None and cached.dtype == torch.bfloat16 and cached.numel() == 14336 * 4096


def test_c0_int4_g128_m1(cuda):
    case = _synthetic().make_int4_case(0, 1, 4096, 4096, 128)
    _check_fp(case, O.LOWP_BF16, label="C0", shipped=True)


def test_single_row_kernel_converts_bf16_rows_toward_zero_outside_fp16_s_normal_range(cuda):
    """The one-row decode kernel turns its bf16 row into fp16 with round-toward-zero (v_cvt_pkrtz_f16_f32): exact for
    every bf16 value inside fp16's normal range, and a documented deviation from the reference's round-to-nearest
    outside it -- below 2^-14 a value between two fp16 subnormals goes to the smaller one, and beyond 65504 the row
    saturates at the largest finite fp16 instead of overflowing to infinity.  One planted activation at a time reads
    the converted value out of the fp32 accumulator: acc[n] = fp16(x_k) * (q[n, k] - z[n]) * s[n]."""
    K, N, G = 1024, 64, 128
    case = _synthetic().make_int4_case(41, 1, K, N, G)
    ctx = make_context(case, O.LOWP_BF16)
    q = O.unpack_int4(case["qweight"].numpy())[:, :K].astype(np.float64)
    s16 = case["scales"].numpy().astype(np.float16).astype(np.float64)  # fp16 scales in this regime
    z = case["zeros"].numpy().astype(np.float64)
    planted = [
        # (value, what the kernel's conversion gives, what round-to-nearest-even gives)
        (1.75 * 2.0 ** -24, 1.0 * 2.0 ** -24, 2.0 * 2.0 ** -24),    # between the first two subnormals
        (-1.75 * 2.0 ** -24, -1.0 * 2.0 ** -24, -2.0 * 2.0 ** -24),
        (1.5 * 2.0 ** -16, 1.5 * 2.0 ** -16, 1.5 * 2.0 ** -16),    # a subnormal that is exact: no deviation
        (1.0078125 * 2.0 ** -14, 1.0078125 * 2.0 ** -14, 1.0078125 * 2.0 ** -14),  # normal range: exact
        (99840.0, 65504.0, float("inf")),                            # beyond the largest finite fp16
        (-3.0e38, -65504.0, float("-inf")),
    ]
    for k, (value, rtz, rne) in zip((3, 200, 517, 640, 901, 1023), planted):
        x = torch.zeros(1, K, dtype=torch.bfloat16)
        x[0, k] = value
        assert float(x[0, k]) == value or abs(value) > 1e38  # representable in bf16 (the last one rounds, far beyond fp16)
        acc = ctx.run(x.cuda(), out_fp32=True).double().cpu().numpy()[0]
        assert _lib_last_kernel() == "woq_decode_m1_kernel"
        w = (q[:, k] - z[:, k // G]) * s16[:, k // G]
        want = rtz * w
        assert np.all(np.isfinite(acc))
        assert np.allclose(acc, want, rtol=1e-6, atol=0.0), (value, float(np.abs(acc - want).max()))
        if rne != rtz:  # and it is not what round-to-nearest would have given
            with np.errstate(invalid="ignore"):
                assert not np.allclose(acc[w != 0], (rne * w)[w != 0], rtol=1e-3, atol=0.0)


@pytest.mark.parametrize("M", [1, 4, 8, 16])
@pytest.mark.parametrize("K,N", [(4096, 14336), (14336, 4096)])
def test_c2_decode_sweep(cuda, M, K, N):
    case = _synthetic().make_int4_case(2, M, K, N, 128)
    cols = np.arange(0, N, 7)  # every 7th output column keeps the oracle in seconds
    _check_fp(case, O.LOWP_BF16, cols=cols, label=f"C2 M={M} K={K} N={N}", shipped=True)


def test_c1_int8_per_channel_bias(cuda):
    case = _synthetic().make_int8_case(1, 32, 4096, 11008)
    _check_fp(case, O.LOWP_BF16, cols=np.arange(0, 11008, 5), label="C1", shipped=True)


@pytest.mark.parametrize("K,N", [(4096, 6144), (4096, 4096), (4096, 28672), (14336, 4096)])
def test_c4_block_g32_m16(cuda, K, N):
    case = _synthetic().make_int4_case(4, 16, K, N, 32)
    _check_fp(case, O.LOWP_BF16, cols=np.arange(0, N, 9), label=f"C4 K={K} N={N}", shipped=True)


def test_c3_prefill_bf16(cuda):
    case = _synthetic().make_int4_case(3, 2048, 4096, 14336, 128, outliers=True)
    _check_fp(case, O.LOWP_BF16, cols=np.arange(0, 14336, 29), label="C3 bf16", shipped=True)


@pytest.mark.parametrize("M", [1, 3, 5, 17, 33, 64, 65, 130, 257])
def test_ragged_m_small_shapes(cuda, M):
    case = _synthetic().make_int4_case(11, M, 512, 272, 128, bias=True)
    _check_fp(case, O.LOWP_BF16, label=f"ragged M={M}")


@pytest.mark.parametrize("N,K,G", [(500, 1024, 128), (30, 384, 32), (100, 640, 64), (64, 1000, -1), (17, 136, -1)])
def test_ragged_n_k(cuda, N, K, G):
    case = _synthetic().make_int4_case(12, 6, K, N, G, bias=True)
    _check_fp(case, O.LOWP_BF16, label=f"ragged N={N} K={K} G={G}")
    case = _synthetic().make_int4_case(13, 2, K, N, G)
    _check_fp(case, O.LOWP_BF16, label=f"ragged fp16 N={N} K={K} G={G}")
    case = _synthetic().make_int4_case(14, 150, K, N, G, bias=True)
    _check_fp(case, O.LOWP_BF16, label=f"ragged gemm N={N} K={K} G={G}")


@pytest.mark.parametrize("M", [2, 40, 100])
def test_both_kernels_agree_on_mid_m(cuda, M):
    case = _synthetic().make_int4_case(15, M, 1024, 256, 128, bias=True)
    if M <= 64:
        _check_fp(case, O.LOWP_BF16, force_kernel=1, label=f"small-M kernel M={M}")
    _check_fp(case, O.LOWP_BF16, force_kernel=2, label=f"tiled kernel M={M}")


@pytest.mark.parametrize(
    "M,K,N,G,bias",
    [
        (128, 256, 448, 128, False),  # exactly one workgroup tile
        (300, 1024, 1000, 32, True),  # ragged M, last wave of the last workgroup partly outside N
        (129, 512, 464, 64, True),
        (200, 384, 96, -1, False),  # per-channel, fewer row-blocks than one wave owns
        (513, 2048, 912, 256, True),
        (70, 128, 16, 128, False),  # a single K step
        (150, 256, 450, 128, True),  # N not a multiple of 8: element-wise stores
    ],
)
@pytest.mark.parametrize("shape", [3, 4, 5, 6, 11, 12, 21])  # cost model, then 448 / 256 / 128 columns per workgroup, then 256 rows x 192, 64 x 128, then the kernel with the dequantized tile in LDS
def test_w4_prefill_kernel(cuda, M, K, N, G, bias, shape):
    case = _synthetic().make_int4_case(20, M, K, N, G, bias=bias)
    _check_fp(case, O.LOWP_BF16, force_kernel=shape, label=f"w4 prefill M={M} K={K} N={N} G={G} kernel={shape}")


def test_w4_prefill_kernel_shapes_agree_bit_for_bit(cuda):
    """Every workgroup shape sums the K products of an output in the same order.  M = 2048, N = 6144
    is the problem the 256 x 192 shape tiles into exactly 256 workgroups (the automatic choice)."""
    case = _synthetic().make_int4_case(22, 2048, 512, 6144, 32, bias=True)
    ctx = make_context(case, O.LOWP_BF16)
    x = case["x"].cuda()
    ys = [ctx.run(x, force_kernel=code) for code in (0, 4, 5, 6, 11, 12)]
    for y in ys[1:]:
        assert torch.equal(y, ys[0])
    cols = np.r_[0:64, 3000:3064, 6080:6144]
    _check_fp(case, O.LOWP_BF16, ctx=ctx, cols=cols, label="w4 prefill 2048 x 6144, automatic shape")


def test_w4_prefill_kernel_symmetric_and_close_to_tiled(cuda):
    case = _synthetic().make_int4_case(21, 260, 512, 464, 128, bias=True)
    case["zeros"] = None
    _check_fp(case, O.LOWP_BF16, force_kernel=3, label="w4 prefill, symmetric")
    # the two GEMM kernels sum the K products in different orders: same values up to the last bit
    ctx = make_context(case, O.LOWP_BF16)
    x = case["x"].cuda()
    a, b = to_np_f32(ctx.run(x, force_kernel=3)), to_np_f32(ctx.run(x, force_kernel=2))
    assert bool(np.all((bf16_ulp_diff(a, b) <= 1) | (np.abs(a - b) <= 1e-4)))


def test_w4_prefill_kernel_fp16_regime(cuda):
    """lowp_mode FP16 with fp16 activations: w = fp16((q - z) * s), fp16 result and bias add."""
    syn = _synthetic()
    M, K, N, G = 140, 512, 464, 128
    case = syn.make_int4_case(22, M, K, N, G, bias=True, scale_dtype=torch.float16)
    case["x"] = case["x"].to(torch.float16)
    ctx = make_context(case, O.LOWP_FP16)
    x = case["x"].cuda()
    y = to_np_f32(ctx.run(x, force_kernel=3))
    acc = ctx.run(x, out_fp32=True, force_kernel=3).cpu().numpy()
    c = case_np(case)
    acc_ref, y_ref = O.woq_linear_ref(c["x"], "fp16", c["qw"], N, K, c["scales"], c["zps"], c["bias"], 2, G, "fp16")
    assert max_abs(acc, acc_ref) <= MAX_ABS_ACC
    assert rel_l2(y, y_ref) <= REL_L2_OUT
    assert rel_l2(y, to_np_f32(ctx.run(x, force_kernel=2))) <= 1e-3


@pytest.mark.parametrize(
    "M,K,N,G,bias",
    [
        (65, 1024, 272, -1, True),
        (200, 384, 464, -1, False),  # three K steps, ragged M and N
        (300, 2048, 128, 128, True),  # one scale per 128 input channels
        (129, 512, 1040, 256, False),
        (2048, 256, 256, -1, True),
    ],
)
@pytest.mark.parametrize("kernel", [0, 5, 6, 12])  # automatic, 128 x 256, 128 x 128, 64 x 128 tiles
def test_prefill_kernel_int8_weights(cuda, M, K, N, G, bias, kernel):
    """8-bit weights through the prefill GEMM: two packed tiles per row-block and K step."""
    case = _synthetic().make_int8_case(26, M, K, N, bias=bias, group_size=G)
    _check_fp(case, O.LOWP_BF16, force_kernel=kernel, label=f"int8-weight prefill M={M} K={K} N={N} G={G} kernel={kernel}")


def test_prefill_kernel_int8_weights_fp16_and_rejections(cuda):
    syn = _synthetic()
    case = syn.make_int8_case(27, 150, 512, 272)
    case["x"] = case["x"].to(torch.float16)
    ctx = make_context(case, O.LOWP_FP16)
    x = case["x"].cuda()
    want = to_np_f32(ctx.run(x, force_kernel=2))
    for kernel in (3, 5, 6, 12):
        assert rel_l2(to_np_f32(ctx.run(x, force_kernel=kernel)), want) <= 1e-3, kernel
    with pytest.raises(RuntimeError, match="8-bit weights take"):
        ctx.run(x, force_kernel=4)  # 448 columns per workgroup: the tiles of a step would not fit the LDS
    small_groups = syn.make_int8_case(28, 100, 512, 64, group_size=64)
    with pytest.raises(RuntimeError, match="prefill kernel takes"):
        make_context(small_groups, O.LOWP_BF16).run(small_groups["x"].cuda(), force_kernel=3)
    _check_fp(small_groups, O.LOWP_BF16, label="int8 weights, groups of 64: general kernel")


@pytest.mark.parametrize("kind,M,K,N,G,bias", [("int4", 128, 4096, 512, 128, True), ("int4", 70, 2560, 272, 32, False),
                                               ("int8", 200, 4096, 256, -1, True), ("int4", 65, 8192, 1040, -1, False)])
@pytest.mark.parametrize("kernel", [0, 19, 20])  # automatic, K shared by two / four workgroups per tile
def test_prefill_kernel_split_k(cuda, kind, M, K, N, G, bias, kernel):
    """Few 64 x 128 tiles and a long K: the workgroups of a tile each take part of K, the last one to
    finish adds the partial tiles in order."""
    syn = _synthetic()
    case = syn.make_int8_case(29, M, K, N, bias=bias) if kind == "int8" else syn.make_int4_case(29, M, K, N, G, bias=bias)
    _check_fp(case, O.LOWP_BF16, force_kernel=kernel, label=f"prefill split K {kind} M={M} K={K} N={N} G={G} kernel={kernel}")
    ctx = make_context(case, O.LOWP_BF16)
    x = case["x"].cuda()
    first = ctx.run(x, force_kernel=kernel)
    runs = [ctx.run(x, force_kernel=kernel) for _ in range(100)]
    torch.cuda.synchronize()
    assert all(torch.equal(y, first) for y in runs)
    assert rel_l2(to_np_f32(first), to_np_f32(ctx.run(x, force_kernel=12))) <= 1e-3
    from ipex_amd import _kernels as kmod

    assert all(int(buf.abs().sum()) == 0 for buf in kmod._counter_cache.values())


def test_prefill_kernel_split_k_rejections(cuda):
    case = _synthetic().make_int4_case(30, 128, 512, 256, 128)  # four K steps: too few to share
    with pytest.raises(RuntimeError, match="too few"):
        make_context(case, O.LOWP_BF16).run(case["x"].cuda(), force_kernel=20)
    big = _synthetic().make_int4_case(31, 2048, 512, 2048, 128)  # 512 tiles: no scratch is offered
    with pytest.raises(RuntimeError, match="split K needs"):
        make_context(big, O.LOWP_BF16).run(big["x"].cuda(), force_kernel=19)


def test_w4_prefill_kernel_rejects_other_shapes(cuda):
    case = _synthetic().make_int4_case(23, 70, 1000, 64, -1)  # K is not a multiple of 128
    ctx = make_context(case, O.LOWP_BF16)
    with pytest.raises(RuntimeError, match="prefill kernel takes"):
        ctx.run(case["x"].cuda(), force_kernel=3)
    with pytest.raises(RuntimeError, match="dequantized tile in LDS takes"):
        ctx.run(case["x"].cuda(), force_kernel=21)
    int8 = _synthetic().make_int8_case(24, 70, 256, 64, 128)
    with pytest.raises(RuntimeError, match="dequantized tile in LDS takes"):
        make_context(int8, O.LOWP_BF16).run(int8["x"].cuda(), force_kernel=21)


def test_w4_prefill_kernel_with_the_tile_in_lds(cuda):
    """force_kernel 21 (256 x 224 workgroup tiles, weights dequantized once per workgroup into LDS): symmetric
    weights, the fp16 regime, post-ops through the staging tile, and agreement with the register-resident kernel
    (another order of the fp32 sums: the K values of an MFMA are grouped differently)."""
    from ipex_amd import _lib

    syn = _synthetic()
    case = syn.make_int4_case(21, 260, 512, 464, 128, bias=True)
    case["zeros"] = None
    _check_fp(case, O.LOWP_BF16, force_kernel=21, label="w4 prefill with the tile in LDS, symmetric")
    ctx = make_context(case, O.LOWP_BF16)
    x = case["x"].cuda()
    a, b = to_np_f32(ctx.run(x, force_kernel=21)), to_np_f32(ctx.run(x, force_kernel=3))
    assert bool(np.all((bf16_ulp_diff(a, b) <= 1) | (np.abs(a - b) <= 1e-4)))
    assert torch.equal(ctx.run(x, force_kernel=21), ctx.run(x, force_kernel=21))
    # post-ops and an fp32 output go through the per-wave staging tile
    other = torch.randn(260, 464, generator=torch.Generator().manual_seed(4)).bfloat16().cuda()
    base = ctx.run(x, out_fp32=True, force_kernel=21)
    assert max_abs(base.cpu().numpy(), ctx.run(x, out_fp32=True, force_kernel=3).cpu().numpy()) <= MAX_ABS_ACC
    y = ctx.run(x, force_kernel=21)
    assert torch.equal(ctx.run(x, fusion=_lib.FUSE_ADD, others=(other,), force_kernel=21), (y.float() + other.float()).bfloat16())
    assert torch.equal(ctx.run(x, fusion=_lib.FUSE_RELU, force_kernel=21), torch.relu(y))
    # fp16 regime
    M, K, N, G = 140, 512, 464, 128
    case = syn.make_int4_case(22, M, K, N, G, bias=True, scale_dtype=torch.float16)
    case["x"] = case["x"].to(torch.float16)
    ctx = make_context(case, O.LOWP_FP16)
    x = case["x"].cuda()
    y = to_np_f32(ctx.run(x, force_kernel=21))
    acc = ctx.run(x, out_fp32=True, force_kernel=21).cpu().numpy()
    c = case_np(case)
    acc_ref, y_ref = O.woq_linear_ref(c["x"], "fp16", c["qw"], N, K, c["scales"], c["zps"], c["bias"], 2, G, "fp16")
    assert max_abs(acc, acc_ref) <= MAX_ABS_ACC
    assert rel_l2(y, y_ref) <= REL_L2_OUT
    # groups of 32 (two groups inside a lane's K step) and per-channel scales, K = 128 (two K steps)
    for G2, K2 in ((32, 384), (-1, 128)):
        _check_fp(syn.make_int4_case(25, 257, K2, 240, G2, bias=False), O.LOWP_BF16, force_kernel=21,
                  label=f"w4 prefill with the tile in LDS, G={G2} K={K2}")


@pytest.mark.parametrize(
    "M,K,N,G,bias",
    [
        (5, 1024, 64, 128, False),
        (16, 4096, 1024, 32, True),  # eight waves, four rounds, one group per lane column
        (8, 512, 48, 64, True),  # fewer K tiles than waves
        (13, 1152, 96, -1, False),  # per-channel, nine K tiles: a partial last round
        (16, 128, 16, 128, False),  # a single K tile
        (3, 256, 80, 256, True),  # bf16 regime is forced below by lowp NONE
    ],
)
@pytest.mark.parametrize("kernel", [7, 8, 9, 10, 22])  # automatic, then 1 / 2 / 4 / 3 row-blocks per workgroup
def test_dequantizing_decode_kernel(cuda, M, K, N, G, bias, kernel):
    ntw = {7: 1, 8: 1, 9: 2, 10: 4, 22: 1}[kernel]  # three need not divide the row-blocks
    if (N // 16) % ntw:
        pytest.skip("row-blocks per workgroup must divide N / 16")
    case = _synthetic().make_int4_case(24, M, K, N, G, bias=bias)
    lowp = O.LOWP_NONE if M < 5 else O.LOWP_BF16  # bf16 compute at every M
    _check_fp(case, lowp, force_kernel=kernel, label=f"decode dq M={M} K={K} N={N} G={G} kernel={kernel}")


@pytest.mark.parametrize("M", [1, 7, 16, 17, 32])
@pytest.mark.parametrize("kernel", [7, 9, 10, 22])
def test_dequantizing_decode_kernel_int8_weights(cuda, M, kernel):
    """8-bit weights (64 K values per tile) and two row tiles (M > 16)."""
    case = _synthetic().make_int8_case(33, M, 704, 128)  # 11 K tiles: a partial last round
    lowp = O.LOWP_NONE if M < 5 else O.LOWP_BF16
    _check_fp(case, lowp, force_kernel=kernel, label=f"decode dq int8 weights M={M} kernel={kernel}")


@pytest.mark.parametrize("M,K,N,G", [(20, 1024, 96, 128), (32, 2048, 64, 32), (17, 384, 48, -1)])
def test_dequantizing_decode_kernel_two_row_tiles_int4(cuda, M, K, N, G):
    case = _synthetic().make_int4_case(34, M, K, N, G, bias=True)
    _check_fp(case, O.LOWP_BF16, force_kernel=7, label=f"decode dq int4 M={M} K={K} N={N} G={G}")


@pytest.mark.parametrize("M,K,N,G,bias", [(33, 1024, 96, 128, True), (64, 2048, 544, 32, False), (50, 384, 96, -1, True),
                                          (64, 512, 768, 128, False)])
@pytest.mark.parametrize("kernel", [0, 8, 9, 10])  # automatic, then one / two / four row-blocks per workgroup
def test_dequantizing_decode_kernel_four_row_tiles(cuda, M, K, N, G, bias, kernel):
    """33..64 rows: four row tiles per wave, 128 KiB of activation buffers per workgroup."""
    if kernel == 10 and (N // 16) % 4:
        pytest.skip("row-blocks per workgroup must divide N / 16")
    case = _synthetic().make_int4_case(35, M, K, N, G, bias=bias)
    _check_fp(case, O.LOWP_BF16, force_kernel=kernel, label=f"decode dq int4 M={M} K={K} N={N} G={G} kernel={kernel}")


@pytest.mark.parametrize("M,N,G", [(16, 4112, 128), (40, 4650, 32), (9, 10256, -1), (20, 13000, 64), (50, 9232, 128)])
def test_dequantizing_decode_kernel_row_blocks_that_do_not_divide(cuda, M, N, G):
    """The automatic choice of two (above 256 row-blocks) or four (from 640) row-blocks per workgroup with a
    count of row-blocks they do not divide: 257, 291, 641 and 813."""
    case = _synthetic().make_int4_case(59, M, 256, N, G, bias=True)
    _check_fp(case, O.LOWP_BF16, label=f"decode dq ragged row-blocks M={M} N={N} G={G}")
    assert _lib_last_kernel() == "woq_decode_dq_kernel"
    # one row-block per workgroup gives the same bits while the waves per workgroup agree (one or four row tiles)
    if M <= 16:
        ctx = make_context(case, O.LOWP_BF16)
        x = case["x"].cuda()
        assert torch.equal(ctx.run(x), ctx.run(x, force_kernel=8))


@pytest.mark.parametrize("M,N,G", [(6, 8200, 128), (16, 11008, -1), (17, 8208, 64), (32, 12288, 128)])
def test_dequantizing_decode_kernel_three_row_blocks_by_shape(cuda, M, N, G):
    """513..768 row-blocks: the automatic choice is three per workgroup, whose last workgroup may hold
    fewer (8200 columns: 513 row-blocks, the last one partial); the forced form gives the same bits."""
    case = _synthetic().make_int4_case(58, M, 256, N, G, bias=True)
    _check_fp(case, O.LOWP_BF16, label=f"decode dq three row-blocks M={M} N={N} G={G}")
    ctx = make_context(case, O.LOWP_BF16)
    x = case["x"].cuda()
    assert torch.equal(ctx.run(x), ctx.run(x, force_kernel=22))
    assert _lib_last_kernel() == "woq_decode_dq_kernel"


def test_dequantizing_decode_kernel_four_row_tiles_int8_weights_and_rejections(cuda):
    case = _synthetic().make_int8_case(36, 48, 704, 128)
    _check_fp(case, O.LOWP_BF16, force_kernel=7, label="decode dq int8 weights M=48")
    _check_fp(case, O.LOWP_BF16, force_kernel=10, label="decode dq int8 weights M=48, four row-blocks per workgroup")
    ctx = make_context(case, O.LOWP_BF16)
    with pytest.raises(RuntimeError, match="row-blocks"):
        ctx.run(case["x"].cuda(), force_kernel=22)
    fp8 = _synthetic().make_fp8_case(36, 48, 512, 128, bias=False, group_size=128)
    with pytest.raises(RuntimeError, match="row-blocks"):
        make_context(fp8, O.LOWP_BF16).run(fp8["x"].cuda(), force_kernel=10)
    nf4 = _synthetic().make_nf4_case(37, 40, 512, 64, 128)
    for kernel in (0, 7, 8, 9, 1):  # four row tiles of NF4 codes, then the small-M kernel
        _check_fp(nf4, O.LOWP_BF16, force_kernel=kernel, label=f"nf4 M=40 kernel={kernel}")
    with pytest.raises(RuntimeError, match="NF4"):
        make_context(nf4, O.LOWP_BF16).run(nf4["x"].cuda(), force_kernel=10)
    _check_fp(_synthetic().make_nf4_case(38, 64, 1024, 272, 64, bias=True), O.LOWP_BF16, label="nf4 M=64")


@pytest.mark.parametrize(
    "M,K,N,G,bias",
    [(1, 1024, 64, 32, False), (2, 4096, 1024, 64, True), (4, 1152, 96, -1, True), (3, 512, 128, 32, False),
     (4, 256, 64, 256, True)],
)
@pytest.mark.parametrize("kernel", [0, 8, 9, 10, 13, 14, 22])
def test_dequantizing_decode_kernel_bf16_rows_under_fp16_compute(cuda, M, K, N, G, bias, kernel):
    """lowp_mode BF16 with fewer than five bf16 rows computes in fp16 (the reference converts the rows
    per K block): group sizes the integer-weight decode kernel does not take go through this kernel,
    which converts the rows on the way into LDS."""
    ntw = {0: 1, 8: 1, 9: 2, 10: 4, 13: 1, 14: 2, 22: 1}[kernel]
    if (N // 16) % ntw:
        pytest.skip("row-blocks per workgroup must divide N / 16")
    case = _synthetic().make_int4_case(54, M, K, N, G, bias=bias)
    _check_fp(case, O.LOWP_BF16, force_kernel=kernel, label=f"decode dq bf16 rows, fp16 compute M={M} K={K} N={N} G={G} kernel={kernel}")


def test_dequantizing_decode_kernel_bf16_rows_under_fp16_compute_other_weights(cuda):
    syn = _synthetic()
    for M in (1, 4):
        _check_fp(syn.make_int8_case(55, M, 704, 128), O.LOWP_BF16, force_kernel=7, label=f"int8 weights M={M}")
        _check_fp(syn.make_nf4_case(56, M, 1024, 96, 64), O.LOWP_BF16, force_kernel=7, label=f"nf4 M={M}")
    # lowp_mode FP16 with bf16 activations: fp16 compute at any M; one row tile converts in the kernel
    case = syn.make_int4_case(57, 13, 1024, 96, 32, bias=True)
    _check_fp(case, O.LOWP_FP16, force_kernel=7, label="lowp FP16, bf16 rows, M=13")
    with pytest.raises(RuntimeError, match="dequantizing decode kernel"):
        big = syn.make_int4_case(58, 20, 1024, 96, 32)
        make_context(big, O.LOWP_FP16).run(big["x"].cuda(), force_kernel=7)


SPLIT_K_CODES = {13: (1, 2), 14: (2, 2), 15: (4, 2), 16: (2, 4), 17: (4, 4)}  # (row-blocks per workgroup, K splits)


@pytest.mark.parametrize(
    "M,K,N,G,bias",
    [
        (5, 1024, 64, 128, False),  # eight K tiles: two per workgroup with four splits
        (16, 4096, 1024, 32, True),
        (13, 1152, 96, -1, False),  # nine K tiles: with four splits the last workgroup has none
        (16, 128, 64, 128, False),  # a single K tile: every split but the first is empty
        (32, 2048, 64, 32, True),  # two row tiles
        (20, 1024, 96, 128, True),
        (3, 256, 128, 256, True),  # bf16 compute forced by lowp NONE
    ],
)
@pytest.mark.parametrize("kernel", sorted(SPLIT_K_CODES))
def test_dequantizing_decode_kernel_split_k(cuda, M, K, N, G, bias, kernel):
    """K shared between 2 or 4 workgroups; the one that finishes last adds the partial tiles."""
    if (N // 16) % SPLIT_K_CODES[kernel][0]:
        pytest.skip("row-blocks per workgroup must divide N / 16")
    case = _synthetic().make_int4_case(44, M, K, N, G, bias=bias)
    lowp = O.LOWP_NONE if M < 5 else O.LOWP_BF16
    _check_fp(case, lowp, force_kernel=kernel, label=f"decode dq split K M={M} K={K} N={N} G={G} kernel={kernel}")


@pytest.mark.parametrize("M", [2, 16, 27])
@pytest.mark.parametrize("kernel", [13, 14, 17])
def test_dequantizing_decode_kernel_split_k_int8_weights(cuda, M, kernel):
    case = _synthetic().make_int8_case(45, M, 704, 128)  # 11 K tiles
    lowp = O.LOWP_NONE if M < 5 else O.LOWP_BF16
    _check_fp(case, lowp, force_kernel=kernel, label=f"decode dq split K int8 weights M={M} kernel={kernel}")


def test_dequantizing_decode_kernel_split_k_nf4_and_fp16(cuda):
    syn = _synthetic()
    nf4 = syn.make_nf4_case(46, 12, 1024, 96, 64)
    for kernel in (13, 14, 16):
        _check_fp(nf4, O.LOWP_BF16, force_kernel=kernel, label=f"nf4 split K kernel={kernel}")
    with pytest.raises(RuntimeError, match="NF4"):
        make_context(nf4, O.LOWP_BF16).run(nf4["x"].cuda(), force_kernel=15)
    case = syn.make_int4_case(47, 11, 1024, 96, 32, bias=True, scale_dtype=torch.float16)
    case["x"] = case["x"].to(torch.float16)
    ctx = make_context(case, O.LOWP_FP16)
    want = to_np_f32(ctx.run(case["x"].cuda(), force_kernel=8))
    for kernel in (13, 14, 16):
        got = to_np_f32(ctx.run(case["x"].cuda(), force_kernel=kernel))
        assert rel_l2(got, want) <= 1e-3, kernel


# (16 x 125 and 2 x 61 row-block sets: the two workgroups of a set sit 125 / 61 places apart in the launch
# order, i.e. on different XCDs, whose L2 caches are not coherent with each other)
@pytest.mark.parametrize("M,K,N,G", [(16, 8192, 4096, 128), (8, 14336, 512, 128), (32, 8192, 2048, 32),
                                     (16, 8192, 2000, 128), (12, 16384, 1952, 64)])
def test_dequantizing_decode_kernel_splits_k_by_itself_for_long_k(cuda, M, K, N, G):
    """Few output columns and K >= 8192: the automatic choice shares K between two workgroups.  The
    result must not depend on which workgroup finishes last (the partial tiles are added in split
    order), the counters are zero again after every call, and a side stream has counters of its own."""
    case = _synthetic().make_int4_case(48, M, K, N, G, bias=True)
    cols = list(range(0, N, 37))
    _check_fp(case, O.LOWP_BF16, cols=cols, label=f"decode dq automatic split K M={M} K={K} N={N} G={G}")
    ctx = make_context(case, O.LOWP_BF16)
    x = case["x"].cuda()
    first = ctx.run(x)
    # another summation order shows in the fp32 sums: the split form ran
    assert not torch.equal(ctx.run(x, out_fp32=True), ctx.run(x, out_fp32=True, force_kernel=8))
    assert rel_l2(to_np_f32(first), to_np_f32(ctx.run(x, force_kernel=8))) <= 1e-3
    # many launches back to back, then compared: a partial tile read before it was complete, or a
    # counter left non-zero, would show as a differing result
    runs = [ctx.run(x) for _ in range(300)]
    torch.cuda.synchronize()
    assert all(torch.equal(y, first) for y in runs)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        other = ctx.run(x)
    side.synchronize()
    assert torch.equal(other, first)
    torch.cuda.synchronize()
    from ipex_amd import _kernels as kmod

    assert len(kmod._counter_cache) >= 2
    assert all(int(buf.abs().sum()) == 0 for buf in kmod._counter_cache.values())


def test_dequantizing_decode_kernel_split_k_needs_scratch(cuda):
    """Through the C ABI without the scratch: forced split-K codes are refused, code 0 runs unsplit."""
    import ctypes

    from ipex_amd import _lib

    lib = _lib.load()
    case = _synthetic().make_int4_case(49, 16, 8192, 256, 128)
    ctx = make_context(case, O.LOWP_BF16)
    x = case["x"].cuda()
    out = torch.empty(16, 256, dtype=torch.bfloat16, device="cuda")
    p = _lib.LinearParams()
    p.struct_size = ctypes.sizeof(_lib.LinearParams)
    p.x, p.x_dtype, p.M, p.K, p.N = x.data_ptr(), _lib.ACT_BF16, 16, 8192, 256
    p.qweight, p.weight_dtype = ctx.at_weight_.data_ptr(), 2
    p.scales_f32, p.scales_f16, p.scales_bf16 = (t.data_ptr() for t in ctx.scales_list_)
    p.zeros_u8 = ctx.zeros_u8_.data_ptr()
    p.group_size, p.lowp_mode, p.act_quant_mode = 128, 2, -1
    p.out, p.out_dtype = out.data_ptr(), _lib.ACT_BF16
    p.stream = torch.cuda.current_stream().cuda_stream
    p.force_kernel = 14
    assert lib.woq_hip_linear(ctypes.byref(p)) != 0
    assert b"split K needs" in lib.woq_hip_last_error()
    p.force_kernel = 0
    assert lib.woq_hip_linear(ctypes.byref(p)) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, ctx.run(x, force_kernel=8))
    assert lib.woq_hip_linear_split_k_workspace_bytes(16, 256) == 4 * 16 * 1024
    assert lib.woq_hip_linear_split_k_workspace_bytes(17, 256) == 4 * 16 * 2048
    assert lib.woq_hip_linear_split_k_workspace_bytes(33, 256) == 0


def test_dequantizing_decode_kernel_fp16_regime_and_symmetric(cuda):
    """fp16 regime with a group size the integer-weight decode kernel does not take, and weights
    without zero points."""
    syn = _synthetic()
    M, K, N, G = 11, 1024, 96, 32
    case = syn.make_int4_case(25, M, K, N, G, bias=True, scale_dtype=torch.float16)
    case["x"] = case["x"].to(torch.float16)
    ctx = make_context(case, O.LOWP_FP16)
    x = case["x"].cuda()
    y = to_np_f32(ctx.run(x, force_kernel=7))
    acc = ctx.run(x, out_fp32=True, force_kernel=7).cpu().numpy()
    c = case_np(case)
    acc_ref, y_ref = O.woq_linear_ref(c["x"], "fp16", c["qw"], N, K, c["scales"], c["zps"], c["bias"], 2, G, "fp16")
    assert max_abs(acc, acc_ref) <= MAX_ABS_ACC
    assert rel_l2(y, y_ref) <= REL_L2_OUT
    case = _synthetic().make_int4_case(26, 9, 768, 64, 128)
    case["zeros"] = None
    _check_fp(case, O.LOWP_BF16, force_kernel=7, label="decode dq, symmetric")


def test_dequantizing_decode_kernel_close_to_small_m_kernel(cuda):
    case = _synthetic().make_int4_case(27, 16, 2048, 1024, 128, bias=True)
    ctx = make_context(case, O.LOWP_BF16)
    x = case["x"].cuda()
    a, b = to_np_f32(ctx.run(x, force_kernel=7)), to_np_f32(ctx.run(x, force_kernel=1))
    assert bool(np.all((bf16_ulp_diff(a, b) <= 1) | (np.abs(a - b) <= 1e-4)))
    with pytest.raises(RuntimeError, match="dequantizing decode kernel"):
        ctx.run(torch.randn(65, 2048, device=cuda).bfloat16(), force_kernel=7)


def test_int8_weights_small_and_tiled(cuda):
    for M in (1, 8, 40, 200):
        case = _synthetic().make_int8_case(16, M, 512, 144)
        _check_fp(case, O.LOWP_BF16, label=f"int8 weights M={M}")


def test_lowp_none_and_fp16_modes(cuda):
    case = _synthetic().make_int4_case(17, 3, 512, 64, 128)
    _check_fp(case, O.LOWP_NONE, label="lowp NONE (bf16 compute at M=3)")
    _check_fp(case, O.LOWP_FP16, label="lowp FP16")
    case = _synthetic().make_int4_case(17, 70, 512, 64, 128)
    _check_fp(case, O.LOWP_FP16, label="lowp FP16 tiled")


@pytest.mark.parametrize("M,bias", [(20, True), (70, False), (200, True)])
def test_lowp_fp16_with_bf16_rows_beyond_one_row_tile(cuda, M, bias):
    """The op layer casts the rows to fp16 and the fp16 result back, as the reference's fp16 kernel does;
    the converting general kernel (reached through force_kernel) must agree."""
    case = _synthetic().make_int4_case(19, M, 1024, 272, 128, bias=bias)
    ctx = make_context(case, O.LOWP_FP16)
    x = case["x"].cuda()
    y = ctx.run(x)
    assert y.dtype == torch.bfloat16
    c = case_np(case)
    _, y_ref = O.woq_linear_ref(c["x"], "bf16", c["qw"], 272, 1024, O._round_to(c["scales"], "fp16"), c["zps"],
                                c["bias"], 2, 128, "fp16")
    assert rel_l2(to_np_f32(y), y_ref) <= REL_L2_OUT
    assert rel_l2(to_np_f32(y), to_np_f32(ctx.run(x, force_kernel=0))) <= 1e-3


def test_symmetric_int4(cuda):
    case = _synthetic().make_int4_case(18, 7, 512, 96, 128)
    case["zeros"] = None
    _check_fp(case, O.LOWP_BF16, label="sym int4")


# ---------------------------------------------------------------------------------------------
# NF4 weights (table lookups; floating-point regimes)
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("M", [1, 4, 5, 16, 40, 64, 65, 200])
@pytest.mark.parametrize("K,N,G", [(1024, 272, 128), (384, 48, 32), (1000, 100, -1)])
def test_nf4_linear(cuda, M, K, N, G):
    case = _synthetic().make_nf4_case(21, M, K, N, G, bias=(M % 2 == 0))
    _check_fp(case, O.LOWP_BF16, label=f"nf4 M={M} K={K} N={N} G={G}")


@pytest.mark.parametrize("M", [1, 4, 7, 16, 17, 32])
@pytest.mark.parametrize("kernel", [1, 7, 8, 9])  # small-M kernel, then the decode kernel: automatic, 1, 2 row-blocks
def test_nf4_decode_kernels(cuda, M, kernel):
    case = _synthetic().make_nf4_case(27, M, 1024, 544, 128, bias=(M == 7))
    # lowp_mode BF16 computes in fp16 below 5 rows, where bf16 activations need the converting
    # small-M kernel; lowp_mode NONE keeps them in bf16 for the decode kernel
    lowp = O.LOWP_NONE if (M < 5 and kernel >= 7) else O.LOWP_BF16
    _check_fp(case, lowp, force_kernel=kernel, label=f"nf4 kernel {kernel} M={M}")


def test_nf4_other_lowp_modes_and_fp16_activations(cuda):
    syn = _synthetic()
    for M in (3, 70):
        case = syn.make_nf4_case(22, M, 512, 96, 64, bias=True)
        _check_fp(case, O.LOWP_NONE, label=f"nf4 lowp NONE M={M}")
        _check_fp(case, O.LOWP_FP16, label=f"nf4 lowp FP16 M={M}")
    # fp16 activations, fp16 scales: w = fp16(table * s), fp32 accumulation
    case = syn.make_nf4_case(23, 9, 256, 64, 32, scale_dtype=torch.float16)
    ctx = make_context(case, O.LOWP_FP16)
    xh = case["x"].to(torch.float16)
    y = to_np_f32(ctx.run(xh.cuda()))
    c = case_np(case)
    _, y_ref = O.woq_linear_ref(to_np_f32(xh), "fp16", c["qw"], 64, 256, c["scales"], None, None, 3, 32, "fp16")
    assert rel_l2(y, y_ref) <= REL_L2_OUT


@pytest.mark.parametrize("G", [32, 128, -1])
def test_nf4_dequant_weight_bit_exact_and_pack_roundtrip(cuda, G):
    syn, k = _synthetic(), _kernels()
    case = syn.make_nf4_case(24, 1, 512, 80, G, scale_dtype=torch.float32)
    ctx = make_context(case, 2)
    c = case_np(case)
    want = O.dequantize_woq_weight(c["qw"], 80, 512, c["scales"], None, 3, G)
    got = k.dequant_weight(ctx.at_weight_, 3, 80, 512, ctx.scales_list_[0], None, G)
    assert np.array_equal(got.cpu().numpy(), want)
    got16 = k.dequant_weight(ctx.at_weight_, 3, 80, 512, ctx.scales_list_[0], None, G, torch.bfloat16)
    assert np.array_equal(to_np_f32(got16), O.bf16_round(want))
    assert torch.equal(k.unpack_weight(ctx.at_weight_, 3, 80, 512).cpu(), case["qweight"])


def test_nf4_rejections(cuda):
    syn = _synthetic()
    case = syn.make_nf4_case(25, 4, 256, 32, 64)
    bad = dict(case, zeros=torch.zeros(32, 4))
    with pytest.raises(RuntimeError, match="symmetric"):
        make_context(bad, O.LOWP_BF16)
    ctx = make_context(case, O.LOWP_BF16)
    with pytest.raises(RuntimeError, match="NF4"):
        ctx.run(case["x"].cuda(), force_kernel=3)
    with pytest.raises(RuntimeError, match="NF4"):
        ctx.run(case["x"].cuda(), force_kernel=10)


@pytest.mark.parametrize("mode", [6, 7, 2])
@pytest.mark.parametrize("M,K,N,G", [(1, 1024, 272, 128), (40, 512, 144, 32), (150, 1024, 272, 128), (20, 768, 80, -1),
                                     (16, 1024, 8208, 64), (9, 512, 144, 32), (4, 1152, 96, -1), (30, 1024, 272, 32), (32, 512, 1040, 128),
                                     (70, 2048, 528, 256), (100, 4096, 256, 128), (48, 1024, 144, 64)])
def test_nf4_lowp_int8(cuda, mode, M, K, N, G):
    """NF4 codes as int8 table values, scale / 127: int32 block sums bit-exact, fp32 epilogue to the bar."""
    case = _synthetic().make_nf4_case(28, M, K, N, G, bias=(M == 40))
    _check_int8(case, mode, label=f"nf4 int8 lowp mode={mode} M={M} K={K} N={N} G={G}")


def test_nf4_weight_cache_for_large_batch_matches_oracle(cuda):
    case = _synthetic().make_nf4_case(26, 1200, 256, 64, 64)
    ctx = make_context(case, O.LOWP_BF16, cache=True)
    y = to_np_f32(ctx.run(case["x"].cuda()))
    c = case_np(case)
    _, y_opt = O.woq_linear_opt_bf16(c["x"], "bf16", c["qw"], 64, 256, c["scales"], None, None, 3, 64)
    assert rel_l2(y, y_opt) <= REL_L2_OUT


# ---------------------------------------------------------------------------------------------
# float8 e4m3fn weights (WOQ_DTYPE_FP8): bytes converted as the reference's kernels convert them, times the scale
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("N,K", [(16, 64), (1024, 1024), (37, 100), (1, 1)])
def test_fp8_pack_unpack_roundtrip(cuda, N, K):
    k = _kernels()
    code = torch.randint(0, 256, (N, K), dtype=torch.int16, generator=torch.Generator().manual_seed(N + K)).to(torch.uint8)
    plain = code.view(torch.float8_e4m3fn)
    packed = k.pack_weight(plain.to(cuda), 4, N, K)
    back = k.unpack_weight(packed, 4, N, K)
    assert back.dtype == torch.float8_e4m3fn and torch.equal(back.view(torch.uint8).cpu(), code)
    # the bytes of a float8 tensor may also be handed over as uint8
    assert torch.equal(k.pack_weight(code.to(cuda), 4, N, K), packed)


@pytest.mark.parametrize("G", [128, -1])
def test_fp8_dequant_weight_bit_exact_on_every_byte(cuda, G):
    k = _kernels()
    N, K = 48, 512
    g = torch.Generator().manual_seed(77)
    code = torch.arange(N * K, dtype=torch.int32).reshape(N, K).remainder(256)
    code = code[:, torch.randperm(K, generator=g)].to(torch.uint8)  # all 256 bytes in every row, NaN codes included
    shape = (N, K // G) if G > 0 else (N,)
    scales = 0.0005 + 0.0015 * torch.rand(shape, generator=g)
    case = dict(x=torch.zeros(1, K, dtype=torch.bfloat16), qweight=code.view(torch.float8_e4m3fn), scales=scales,
                zeros=None, bias=None, M=1, K=K, N=N, group_size=G, weight_dtype=4)
    ctx = make_context(case, O.LOWP_BF16)
    want = O.dequantize_woq_weight(code.numpy(), N, K, scales.numpy(), None, 4, G)
    got = k.dequant_weight(ctx.at_weight_, 4, N, K, ctx.scales_list_[0], None, G)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    got16 = k.dequant_weight(ctx.at_weight_, 4, N, K, ctx.scales_list_[0], None, G, torch.bfloat16)
    assert np.array_equal(to_np_f32(got16), O.bf16_round(want))


@pytest.mark.parametrize("M", [1, 4, 5, 16, 40, 64, 65, 200])
@pytest.mark.parametrize("K,N,G", [(1024, 272, 128), (384, 48, 32), (1000, 100, -1)])
def test_fp8_linear(cuda, M, K, N, G):
    case = _synthetic().make_fp8_case(60, M, K, N, bias=(M % 2 == 0), group_size=G)
    _check_fp(case, O.LOWP_BF16, label=f"fp8 M={M} K={K} N={N} G={G}")


def test_fp8_other_lowp_modes_kernels_and_activations(cuda):
    syn = _synthetic()
    for M in (3, 70):
        case = syn.make_fp8_case(61, M, 512, 96, bias=True, group_size=64)
        _check_fp(case, O.LOWP_NONE, label=f"fp8 lowp NONE M={M}")
        _check_fp(case, O.LOWP_FP16, label=f"fp8 lowp FP16 M={M}")
    # the tiled kernel on few rows and the small-M kernel at its row limit agree with the oracle too
    case = syn.make_fp8_case(62, 48, 640, 144, bias=False, group_size=128)
    _check_fp(case, O.LOWP_BF16, force_kernel=2, label="fp8 tiled kernel M=48")
    _check_fp(case, O.LOWP_BF16, force_kernel=1, label="fp8 small-M kernel M=48")
    # fp16 activations: w = fp16(value * s), fp32 accumulation
    case = syn.make_fp8_case(63, 9, 256, 64, bias=False, group_size=128, x_dtype=torch.float16)
    ctx = make_context(case, O.LOWP_FP16)
    c = case_np(case)
    y = to_np_f32(ctx.run(case["x"].cuda()))
    _, y_ref = O.woq_linear_ref(c["x"], "fp16", c["qw"], 64, 256, O._round_to(c["scales"], "fp16"), None, None, 4, 128, "fp16")
    assert rel_l2(y, y_ref) <= REL_L2_OUT


@pytest.mark.parametrize("M,K,N,G,bias", [(4, 1024, 1024, 128, True), (300, 1024, 272, 128, False), (37, 1000, 100, -1, True)])
def test_fp8_fp32_compute(cuda, M, K, N, G, bias):
    """fp32 activations under lowp_mode NONE: w = fp32(value * s) (fp32 scales), fp32 matrix instructions."""
    case = _synthetic().make_fp8_case(64, M, K, N, bias=bias, group_size=G, x_dtype=torch.float32)
    ctx = make_context(case, O.LOWP_NONE)
    y = ctx.run(case["x"].cuda())
    assert y.dtype == torch.float32
    c = case_np(case)
    acc, _ = O.woq_linear_ref(c["x"], "fp32", c["qw"], N, K, c["scales"], None, c["bias"], 4, G, "fp32")
    assert rel_l2(y.cpu().numpy(), acc) <= 1e-5


@pytest.mark.parametrize("M,K,N,G,bias", [(1, 1024, 544, 128, False), (7, 1024, 544, 128, True), (16, 2048, 64, -1, False),
                                          (27, 1152, 96, 128, True), (50, 1024, 288, 256, False), (64, 2048, 544, 128, True)])
@pytest.mark.parametrize("kernel", [7, 8, 9, 13, 14])  # the dequantizing decode kernel: automatic, 1 / 2 row-blocks, K split in two
def test_fp8_decode_kernels(cuda, M, K, N, G, bias, kernel):
    if kernel in (13, 14) and M > 32:
        pytest.skip("split K takes at most 32 rows")
    case = _synthetic().make_fp8_case(66, M, K, N, bias=bias, group_size=G)
    # lowp_mode BF16 computes in fp16 below 5 rows (bf16 rows converted on the way in)
    _check_fp(case, O.LOWP_BF16, force_kernel=kernel, label=f"fp8 kernel {kernel} M={M}")
    assert _lib_last_kernel() == "woq_decode_dq_kernel"


@pytest.mark.parametrize("M,K,N,G,bias", [(128, 1024, 512, 128, True), (70, 2560, 272, -1, False), (300, 1024, 1040, 256, True),
                                          (65, 512, 144, 128, False)])
@pytest.mark.parametrize("kernel", [0, 5, 6, 12, 19])  # automatic, 128 x 256, 128 x 128, 64 x 128 tiles, K split in two
def test_fp8_prefill_kernel(cuda, M, K, N, G, bias, kernel):
    case = _synthetic().make_fp8_case(67, M, K, N, bias=bias, group_size=G)
    _check_fp(case, O.LOWP_BF16, force_kernel=kernel, label=f"fp8 prefill kernel {kernel} M={M}")
    assert _lib_last_kernel() == "woq_gemm_w4_kernel"


@pytest.mark.parametrize("regime", ["fp16", "bf16"])
@pytest.mark.parametrize("kernel", [1, 2, 8, 6])  # small-M, tiled, dequantizing decode, prefill
def test_fp8_unit_rows_read_out_the_dequantized_weight_bit_for_bit(cuda, regime, kernel):
    """Row m of the activations is the unit vector e_k(m): the fp32 accumulator is then the kernel's own
    dequantized weight w[n, k(m)] -- every byte (subnormal and NaN codes included) against the oracle's
    conversion and single rounding, bit for bit."""
    N, K, G = 64, 256, 128
    g = torch.Generator().manual_seed(91)
    code = torch.stack([torch.randperm(256, generator=g) for _ in range(N)]).to(torch.uint8)  # all bytes in every row
    scales = 0.0005 + 0.0015 * torch.rand((N, K // G), generator=g)
    xdt = torch.float16 if regime == "fp16" else torch.bfloat16
    case = dict(x=None, qweight=code.view(torch.float8_e4m3fn), scales=scales, zeros=None, bias=None, M=0, K=K, N=N,
                group_size=G, weight_dtype=4)
    ctx = make_context(case, O.LOWP_FP16 if regime == "fp16" else O.LOWP_BF16)
    want = O._round_to(O.dequantize_woq_weight(code.numpy(), N, K, O._round_to(scales.numpy(), regime), None, 4, G), regime)
    rows = 64 if kernel in (1, 8) else 256
    eye = torch.eye(K, dtype=xdt)
    for k0 in range(0, K, rows):
        acc = ctx.run(eye[k0:k0 + rows].cuda(), out_fp32=True, force_kernel=kernel).cpu().numpy()
        assert np.array_equal(acc, want[:, k0:k0 + rows].T), (regime, kernel, k0)


@pytest.mark.parametrize("regime", ["fp16", "bf16"])
@pytest.mark.parametrize("sym", [True, False])
@pytest.mark.parametrize("kernel", [1, 2, 8, 6])  # small-M, tiled, dequantizing decode, prefill
def test_int8_unit_rows_read_out_the_dequantized_weight_bit_for_bit(cuda, regime, sym, kernel):
    """As for FP8: unit-vector rows make the fp32 accumulator the kernel's own w[n, k] = cd((q - z) * s), here for
    every int8 code with and without zero points, against the oracle bit for bit."""
    N, K, G = 64, 256, 128
    g = torch.Generator().manual_seed(92)
    q = torch.stack([torch.randperm(256, generator=g) for _ in range(N)]).sub(128).to(torch.int8)  # every code in every row
    scales = 0.0005 + 0.0015 * torch.rand((N, K // G), generator=g)
    zeros = None if sym else torch.randint(-128, 128, (N, K // G), generator=g).float()
    xdt = torch.float16 if regime == "fp16" else torch.bfloat16
    case = dict(x=None, qweight=q, scales=scales, zeros=zeros, bias=None, M=0, K=K, N=N, group_size=G, weight_dtype=1)
    ctx = make_context(case, O.LOWP_FP16 if regime == "fp16" else O.LOWP_BF16)
    want = O._round_to(O.dequantize_woq_weight(q.numpy(), N, K, O._round_to(scales.numpy(), regime),
                                               None if sym else zeros.numpy(), 1, G), regime)
    rows = 64 if kernel in (1, 8) else 256
    eye = torch.eye(K, dtype=xdt)
    for k0 in range(0, K, rows):
        acc = ctx.run(eye[k0:k0 + rows].cuda(), out_fp32=True, force_kernel=kernel).cpu().numpy()
        assert np.array_equal(acc, want[:, k0:k0 + rows].T), (regime, sym, kernel, k0)


def test_fp8_rejections(cuda):
    syn = _synthetic()
    case = syn.make_fp8_case(65, 4, 256, 32, group_size=64)
    with pytest.raises(RuntimeError, match="no zero points"):
        make_context(dict(case, zeros=torch.zeros(32, 4)), O.LOWP_BF16)
    with pytest.raises(RuntimeError, match="INT8 does not take FP8"):
        make_context(case, O.LOWP_INT8, act_quant_mode=6)
    with pytest.raises(RuntimeError, match="float8_e4m3fn"):
        make_context(dict(case, qweight=case["qweight"].view(torch.uint8).view(torch.int8)), O.LOWP_BF16)


def test_empty_batch(cuda):
    case = _synthetic().make_int4_case(19, 1, 256, 32, 128)
    ctx = make_context(case, O.LOWP_BF16)
    y = ctx.run(torch.empty(0, 256, dtype=torch.bfloat16, device=cuda))
    assert y.shape == (0, 32)
    y = ctx.run(torch.randn(2, 3, 256, device=cuda).bfloat16())
    assert y.shape == (2, 3, 32)


# ---------------------------------------------------------------------------------------------
# lowp_mode INT8
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("mode", [0, 1, 2, 3, 4, 5, 6, 7])
@pytest.mark.parametrize("M,K", [(1, 512), (37, 4096), (300, 1024)])
def test_dynamic_quant_bit_exact(cuda, mode, M, K):
    k = _kernels()
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(M + K + mode))
    x[0, :5] = torch.tensor([0.5, -0.5, 1.5, 2.5, 1e-3])
    x = x.to(torch.bfloat16)
    q, s, zp = k.dynamic_quant(x.to(cuda), 128, mode)
    q_ref, s_ref, zp_ref = O.dynamic_quantize_per_block(to_np_f32(x), 128, mode)
    assert np.array_equal(s.cpu().numpy().reshape(-1), s_ref.reshape(-1))
    assert np.array_equal(q.cpu().numpy(), q_ref)
    if mode < 4:
        assert np.array_equal(zp.cpu().numpy().reshape(-1), zp_ref.reshape(-1))


@pytest.mark.parametrize("mode", [2, 3, 6, 7])
@pytest.mark.parametrize(
    "M,K,block,dtype",
    [
        (9, 8192, 64, torch.bfloat16),  # sixteen 512-element chunks per row
        (5, 14336, 512, torch.bfloat16),  # thirty-two chunks, a block per chunk
        (6, 1000, 32, torch.float16),  # K not a multiple of the block: a partial last block
        (3, 4096, 256, torch.float16),
        (4, 2048, 1024, torch.bfloat16),  # blocks wider than a chunk: the two-kernel form
        (4, 24576, 128, torch.bfloat16),  # rows too long for a wave's registers: the two-kernel form
        (7, 768, 128, torch.float32),  # fp32 activations: the two-kernel form
    ],
)
def test_dynamic_quant_rows_bit_exact(cuda, mode, M, K, block, dtype):
    """Per-row and per-(row, K block) scales over the row lengths, block sizes and activation types
    that select the one-pass kernel or the two-kernel form; one row is all zeros (scale 0)."""
    k = _kernels()
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(M * 7 + K + mode)) * 3.0
    x[1] = 0.0
    x[0, :5] = torch.tensor([0.5, -0.5, 1.5, 2.5, 1e-3])
    x = x.to(dtype)
    q, s, zp = k.dynamic_quant(x.to(cuda), block, mode)
    q_ref, s_ref, zp_ref = O.dynamic_quantize_per_block(x.float().numpy(), block, mode)
    assert np.array_equal(s.cpu().numpy().reshape(-1), s_ref.reshape(-1))
    assert np.array_equal(q.cpu().numpy(), q_ref)
    if mode < 4:
        assert np.array_equal(zp.cpu().numpy().reshape(-1), zp_ref.reshape(-1))


@pytest.mark.parametrize("mode", [0, 1, 4, 5])
@pytest.mark.parametrize(
    "M,K,block,dtype",
    [
        (2100, 4096, 128, torch.bfloat16),  # eight rows per workgroup, the last workgroup partly empty
        (9, 8192, 64, torch.bfloat16),
        (70, 14336, 512, torch.bfloat16),  # thirty-two chunks; more than 64 rows: a wave per row
        (6, 1000, 32, torch.float16),  # a partial last block
        (1, 4096, 128, torch.float16),  # one row: its statistics are the tensor's
        (4, 24576, 128, torch.bfloat16),  # rows too long for a wave's registers: the general form
    ],
)
def test_dynamic_quant_shared_scales_bit_exact(cuda, mode, M, K, block, dtype):
    """One scale per tensor or per K block (shared by all rows): statistics merged over workgroups,
    then quantization with the scales given; one K block is all zeros (scale 0 in the per-block modes)."""
    k = _kernels()
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(M * 5 + K + mode)) * 2.0
    x[:, block : 2 * block] = 0.0
    x[0, :5] = torch.tensor([0.5, -0.5, 1.5, 2.5, 1e-3])
    x[M // 2, K - 1] = 9.0
    x = x.to(dtype)
    q, s, zp = k.dynamic_quant(x.to(cuda), block, mode)
    q_ref, s_ref, zp_ref = O.dynamic_quantize_per_block(x.float().numpy(), block, mode)
    assert np.array_equal(s.cpu().numpy().reshape(-1), s_ref.reshape(-1))
    assert np.array_equal(q.cpu().numpy(), q_ref)
    if mode < 4:
        assert np.array_equal(zp.cpu().numpy().reshape(-1), zp_ref.reshape(-1))


def test_dynamic_quant_all_bf16_patterns(cuda):
    k = _kernels()
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    vals = bits.view(torch.bfloat16)
    vals = vals[torch.isfinite(vals.float()) & (vals.float().abs() < 3e4)]
    n = (vals.numel() // 1024) * 1024
    x = vals[torch.randperm(vals.numel(), generator=torch.Generator().manual_seed(0))][:n].reshape(-1, 1024)
    for mode in (6, 7):
        q, s, _ = k.dynamic_quant(x.to(cuda), 128, mode)
        q_ref, s_ref, _ = O.dynamic_quantize_per_block(to_np_f32(x), 128, mode)
        assert np.array_equal(s.cpu().numpy(), s_ref)
        assert np.array_equal(q.cpu().numpy(), q_ref)


def _check_int8(case, mode, cols=None, debug=True, label="", shipped=False):
    ctx = make_context(case, O.LOWP_INT8, mode)
    x = case["x"].cuda()
    N, K, G = case["N"], case["K"], case["group_size"]
    c = case_np(case)
    y_t = ctx.run(x)
    if shipped:  # the registered operator on the custom class: the same bits
        assert torch.equal(_shipped_binding_output(case, O.LOWP_INT8, mode), y_t), (label, "registered operator differs")
    y = to_np_f32(y_t)
    # the accumulators of the kernel that serves the call, and (debug) those of the general kernel with
    # its block sums
    acc = ctx.run(x, out_fp32=True).cpu().numpy()
    acc_dbg, sums = None, None
    if debug:
        acc_dbg, sums = ctx.run(x, out_fp32=True, debug_block_sums=True)
        acc_dbg, sums = acc_dbg.cpu().numpy(), sums.cpu().numpy()
    qw, sc, zp, b = c["qw"], c["scales"], c["zps"], c["bias"]
    if cols is not None:
        qw, sc = qw[cols], sc[cols]
        zp = None if zp is None else zp[cols]
        b = None if b is None else b[cols]
        y, acc = y[:, cols], acc[:, cols]
        sums = None if sums is None else sums[:, cols]
        acc_dbg = None if acc_dbg is None else acc_dbg[:, cols]
        N = len(cols)
    r = O.woq_linear_opt_int8(c["x"], "bf16", qw, N, K, sc, zp, b, case["weight_dtype"], G, mode)
    if sums is not None:
        assert np.array_equal(sums[:, :, : r["sums"].shape[2]], r["sums"]), label  # int32, bit-exact
    stats = {"max_abs_acc": max_abs(acc, r["acc"]), "rel_l2_out": rel_l2(y, r["y"])}
    if acc_dbg is not None:
        stats["max_abs_acc"] = max(stats["max_abs_acc"], max_abs(acc_dbg, r["acc"]))
    print(label, stats)
    assert stats["max_abs_acc"] <= MAX_ABS_ACC and stats["rel_l2_out"] <= REL_L2_OUT, (label, stats)
    return stats


@pytest.mark.parametrize("mode", [6, 7, 4, 5])
@pytest.mark.parametrize("M", [1, 4, 16, 48, 150])
def test_int8_lowp_int4_g128(cuda, mode, M):
    case = _synthetic().make_int4_case(20, M, 1024, 272, 128, bias=True, outliers=True)
    _check_int8(case, mode, label=f"int8 lowp mode={mode} M={M}")


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
@pytest.mark.parametrize("M,K,N,G", [(1, 1024, 272, 128), (37, 512, 144, 32), (150, 1024, 272, 128), (20, 768, 80, -1)])
def test_int8_lowp_asymmetric_activations(cuda, mode, M, K, N, G):
    """uint8 activations with a zero point: block sums bit-exact (as the reference defines them,
    unsigned activations times weights), compensation applied in integers."""
    case = _synthetic().make_int4_case(28, M, K, N, G, bias=True, outliers=True)
    case["x"] = (case["x"].float() + 0.5).to(torch.bfloat16)  # off-centre: zero points far from 128
    _check_int8(case, mode, label=f"int8 lowp asym mode={mode} M={M} K={K} N={N} G={G}")


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
@pytest.mark.parametrize(
    "M,K,N,G",
    [
        (1, 1024, 272, 128),
        (16, 4096, 1024, 128),
        (32, 2048, 1040, 256),  # two row tiles
        (25, 1024, 8208, -1),  # per channel; two row-blocks per workgroup
        (70, 2048, 528, -1),  # the 64-row tiles, ragged in both directions
        (150, 1024, 272, 128),
        (300, 4096, 256, 512),  # activation blocks of four tiles
    ],
)
def test_int8_lowp_asymmetric_activations_mfma_kernels(cuda, mode, M, K, N, G):
    """Asymmetric activations through the kernels that feed the stored codes to the int8 MFMA (groups
    of at least 128): the column sums of the weights come from MFMAs against rows of ones, the zero
    points enter in integers.  The general kernel (debug run) supplies the bit-exact block sums."""
    case = _synthetic().make_int4_case(33, M, K, N, G, bias=True, outliers=True)
    case["x"] = (case["x"].float() + 0.5).to(torch.bfloat16)  # off-centre: zero points far from 128
    cols = None if N < 4096 else list(range(0, N, 53)) + [N - 1]
    _check_int8(case, mode, cols=cols, debug=N < 4096 and M * N * (K // 128) < 1 << 24,
                label=f"int8 lowp asym mfma mode={mode} M={M} K={K} N={N} G={G}")


@pytest.mark.parametrize("mode", [2, 3])
def test_int8_lowp_asymmetric_activations_split_k(cuda, mode):
    """Asymmetric activations with the workgroups of a tile sharing K."""
    case = _synthetic().make_int4_case(34, 100, 4096, 256, 128, bias=True, outliers=True)
    case["x"] = (case["x"].float() - 0.7).to(torch.bfloat16)
    _check_int8(case, mode, debug=False, label=f"int8 lowp asym split K mode={mode}")


def test_int8_lowp_asymmetric_activations_int8_weights(cuda):
    case = _synthetic().make_int8_case(29, 70, 512, 80)
    _check_int8(case, 2, label="int8 lowp asym, int8 weights")


@pytest.mark.parametrize("G", [32, 64, -1, 256])
@pytest.mark.parametrize("M", [3, 130])
def test_int8_lowp_other_groups(cuda, G, M):
    case = _synthetic().make_int4_case(21, M, 1024, 144, G, bias=True)
    _check_int8(case, 7, label=f"int8 lowp G={G} M={M}")
    _check_int8(case, 6, label=f"int8 lowp G={G} M={M} per-M")


@pytest.mark.parametrize("mode", [4, 5, 6, 7])
@pytest.mark.parametrize("M,K,N,G", [(17, 1024, 272, 128), (32, 2048, 1040, 64), (9, 512, 144, 32), (16, 1152, 96, -1),
                                     (25, 1024, 8208, 256), (2, 384, 48, 64), (30, 1024, 272, 32), (64, 512, 144, 64),
                                     (41, 1024, 96, 64), (20, 512, 4128, 128), (1, 512, 8224, 128), (4, 256, 12320, -1)])
def test_int8_lowp_decode_kernel(cuda, mode, M, K, N, G):
    """The int8 MFMA decode kernel: one or two row tiles, groups of 32 / 64 as K blocks inside a tile,
    two row-blocks per workgroup for wide layers; the general kernel (debug run) supplies the bit-exact
    block sums, this one the outputs."""
    case = _synthetic().make_int4_case(22, M, K, N, G, bias=True, outliers=True)
    cols = None if N < 4096 else list(range(0, N, 53)) + [N - 1]
    _check_int8(case, mode, cols=cols, debug=N < 4096, label=f"int8 lowp decode mode={mode} M={M} K={K} N={N} G={G}")


@pytest.mark.parametrize("mode", [4, 5, 6, 7])
@pytest.mark.parametrize("M,K,N,G", [(33, 1024, 272, 32), (65, 1024, 272, 64), (150, 2048, 528, 32), (300, 1024, 1040, 64),
                                     (100, 4096, 256, 32)])
def test_int8_lowp_small_groups_mfma_tiles(cuda, mode, M, K, N, G):
    """Groups of 32 / 64 above the rows of the decode form: the 64 x 128 tiles with the K blocks of a
    packed tile computed one by one (B operand masked to the block's lane columns); the last shape shares
    K between workgroups.  The general kernel (debug run) supplies the bit-exact block sums."""
    case = _synthetic().make_int4_case(35, M, K, N, G, bias=True, outliers=True)
    _check_int8(case, mode, debug=M * N * (K // G) < 1 << 24,
                label=f"int8 lowp small groups tiles mode={mode} M={M} K={K} N={N} G={G}")


@pytest.mark.parametrize("mode", [6, 7])
@pytest.mark.parametrize("M,K,N,G", [(100, 4096, 256, 128), (200, 8192, 144, 256), (65, 14336, 512, -1)])
def test_int8_lowp_prefill_split_k(cuda, mode, M, K, N, G):
    """Few 64 x 128 tiles and a long K under lowp INT8: the workgroups of a tile share K (scratch behind
    the quantized activations); repeated launches must agree bit for bit."""
    case = _synthetic().make_int4_case(32, M, K, N, G, bias=True, outliers=True)
    _check_int8(case, mode, debug=False, label=f"int8 lowp split K mode={mode} M={M} K={K} N={N} G={G}")
    ctx = make_context(case, O.LOWP_INT8, mode)
    x = case["x"].cuda()
    first = ctx.run(x)
    runs = [ctx.run(x) for _ in range(100)]
    torch.cuda.synchronize()
    assert all(torch.equal(y, first) for y in runs)
    from ipex_amd import _kernels as kmod

    assert all(int(buf.abs().sum()) == 0 for buf in kmod._counter_cache.values())


def test_int8_lowp_int8_weights(cuda):
    for M in (2, 20, 140):
        case = _synthetic().make_int8_case(22, M, 512, 80)
        _check_int8(case, 6, label=f"int8 lowp int8 weights M={M}")


@pytest.mark.parametrize("mode", [4, 6, 7])
@pytest.mark.parametrize("M,K,N,G", [(1, 1024, 272, -1), (16, 4096, 8208, -1), (17, 1152, 96, 128), (32, 2048, 1040, 256)])
def test_int8_lowp_int8_weights_decode_kernel(cuda, mode, M, K, N, G):
    """Symmetric 8-bit weights in the int8 MFMA decode kernel: two packed tiles per round, the lane's
    bytes are the B operand as they are."""
    case = _synthetic().make_int8_case(23, M, K, N, group_size=G)
    cols = None if N < 4096 else list(range(0, N, 53)) + [N - 1]
    _check_int8(case, mode, cols=cols, debug=N < 4096, label=f"int8 lowp int8 weights decode mode={mode} M={M} K={K} N={N} G={G}")


@pytest.mark.parametrize("mode", [4, 5, 6, 7])
@pytest.mark.parametrize("M,K,N,G", [(33, 1024, 272, -1), (70, 2048, 528, 128), (150, 1152, 96, -1), (300, 1024, 1040, 256)])
def test_int8_lowp_int8_weights_mfma_tiles(cuda, mode, M, K, N, G):
    """Symmetric 8-bit weights above 32 rows: the 64 x 128 tiles of the int8 MFMA kernel with two packed
    tiles per row-block and K step; the general kernel (debug run) supplies the bit-exact block sums."""
    case = _synthetic().make_int8_case(24, M, K, N, group_size=G)
    _check_int8(case, mode, label=f"int8 lowp int8 weights tiles mode={mode} M={M} K={K} N={N} G={G}")


@pytest.mark.parametrize("mode", [6, 7])
def test_int8_lowp_int8_weights_split_k(cuda, mode):
    """8-bit weights with the workgroups of a tile sharing K; repeated launches agree bit for bit."""
    case = _synthetic().make_int8_case(25, 100, 4096, 256)
    _check_int8(case, mode, debug=False, label=f"int8 lowp int8 weights split K mode={mode}")
    ctx = make_context(case, O.LOWP_INT8, mode)
    x = case["x"].cuda()
    first = ctx.run(x)
    runs = [ctx.run(x) for _ in range(50)]
    torch.cuda.synchronize()
    assert all(torch.equal(y, first) for y in runs)


def test_c3_prefill_int8(cuda):
    case = _synthetic().make_int4_case(3, 2048, 4096, 14336, 128, outliers=True)
    _check_int8(case, 6, cols=np.arange(0, 14336, 61), debug=False, label="C3 int8 per-M", shipped=True)
    # bit-exact int32 block sums on a slice small enough to hold [M, N, K/128]
    small = dict(case)
    small["x"] = case["x"][:96]
    small["qweight"], small["scales"], small["zeros"] = case["qweight"][:512], case["scales"][:512], case["zeros"][:512]
    small["N"], small["M"] = 512, 96
    _check_int8(small, 6, label="C3 int8 block sums slice")


# ---------------------------------------------------------------------------------------------
# lowp INT8: the int32 block sums of the kernels that serve the calls (no debug path)
# ---------------------------------------------------------------------------------------------
# The debug_block_sums run above is served by the general int8 kernels.  The two checks below read the
# integers out of the kernels that serve a plain call, through their ordinary fp32 output:
#  * one K block at a time: with the activations of every other K block set to zero, the accumulator of
#    (m, n) is the block's integer times s_a[m] times s_w[n, g] with two or three fp32 roundings, so
#    rint(acc / (s_a s_w)) in float64 is the integer itself while |integer| * 3 * 2^-24 < 1/2
#    (|integer| <= 128 * 255 * 127 < 2^22);
#  * all K blocks at once: with weight scales that are powers of two (2^-7 or 2^-6) and activations laid
#    out so that every activation scale is a power of two, every product and every partial sum of the
#    epilogue is exact in fp32 in any order, so the fp32 accumulator must EQUAL the oracle's.
def _pow2_weight_scales(case, seed):
    out = dict(case)
    g = torch.Generator().manual_seed(seed)
    e = torch.randint(6, 8, case["scales"].shape, generator=g).float()
    out["scales"] = torch.pow(2.0, -e)
    out["bias"] = None
    return out


def _isolate_k_block(x, kb, bk):
    out = torch.zeros_like(x)
    out[:, kb * bk:(kb + 1) * bk] = x[:, kb * bk:(kb + 1) * bk]
    return out


def _plant_pow2_activation_scales(x, mode, qbk, seed):
    """Clamps every quantization group of x (bf16 [M, K]) into a range whose ends are planted in it, so
    that its scale is a power of two: symmetric modes max|x| = 127 * 2^e; asymmetric modes
    min = -a * 2^e, max = (255 - a) * 2^e (max - min = 255 * 2^e, zero point a)."""
    M, K = x.shape
    sym, per_m, per_k = mode >= 4, mode in (2, 3, 6, 7), mode in (1, 3, 5, 7)
    rng = np.random.default_rng(seed)
    xf = x.float().clone()
    row_groups = [slice(m, m + 1) for m in range(M)] if per_m else [slice(0, M)]
    col_groups = [slice(k, min(k + qbk, K)) for k in range(0, K, qbk)] if per_k else [slice(0, K)]
    for rs in row_groups:
        for cs in col_groups:
            e = float(2.0 ** int(rng.integers(-5, -2)))
            if sym:
                lo, hi = -127 * e, 127 * e
            else:
                a = int(rng.integers(40, 216))
                lo, hi = -a * e, (255 - a) * e
            blk = xf[rs, cs].clamp(lo, hi)
            flat = blk.reshape(-1).clone()
            i, j = rng.choice(flat.numel(), size=2, replace=False) if flat.numel() > 1 else (0, 0)
            if sym:
                flat[i] = hi if rng.integers(2) else lo
            else:
                flat[i], flat[j] = lo, hi
            xf[rs, cs] = flat.reshape(blk.shape)
    out = xf.to(torch.bfloat16)
    # the planted ends are bf16 values (integers below 256 times a power of two); rounding the rest to
    # bf16 cannot leave the range they span
    return out


def _served_by(want_kernel, label):
    from ipex_amd import _lib

    got = _lib.last_kernel()
    assert want_kernel is None or got == want_kernel, (label, got, want_kernel)
    return got


def _check_int8_block_integers(case, mode, blocks=None, rows=None, cols=None, want_kernel=None, label=""):
    """Bit-exact int32 block sums (after the zero-point compensation for the asymmetric modes) of the
    kernel that serves the call, one K block at a time (see above)."""
    case = _pow2_weight_scales(case, 7)
    ctx = make_context(case, O.LOWP_INT8, mode)
    N, K, G, wd = case["N"], case["K"], case["group_size"], case["weight_dtype"]
    c = case_np(case)
    bk = O.int8_block_k(G, K)
    qbk = G if G > 0 else bk
    M = case["x"].shape[0]
    rows = np.arange(M) if rows is None or mode in (0, 1, 4, 5) else np.asarray(rows)
    cols = np.arange(N) if cols is None else np.asarray(cols)
    qw, sc = c["qw"][cols], c["scales"].reshape(N, -1)[cols]
    zp = None if c["zps"] is None else c["zps"].reshape(N, -1)[cols]
    s_eff = (sc * (np.float32(1.0) / np.float32(127.0))).astype(np.float32) if wd == O.WOQ_DTYPE_NF4 else sc
    per_m, per_k, asym = mode in (2, 3, 6, 7), mode in (1, 3, 5, 7), mode < 4
    cols_t = torch.as_tensor(cols).cuda()
    rows_t = torch.as_tensor(rows).cuda()
    for kb in (range(K // bk) if blocks is None else blocks):
        xk = _isolate_k_block(case["x"], kb, bk)
        acc = ctx.run(xk.cuda(), out_fp32=True)
        kernel = _served_by(want_kernel, label)
        acc = acc[rows_t][:, cols_t].double().cpu().numpy()
        xs = to_np_f32(xk)[rows]
        xq, sa, za = O.dynamic_quantize_per_block(xs if per_m else to_np_f32(xk), qbk, mode)
        if not per_m:
            xq = xq[rows]
        Mr, Kc = len(rows), (K + qbk - 1) // qbk
        sa2 = np.asarray(sa, dtype=np.float32).reshape(Mr if per_m else 1, Kc if per_k else 1)
        kc = (kb * bk) // qbk if per_k else 0
        want = O.int8_block_sums(xq, qw, len(cols), K, zp, wd, G, bk)[:, :, kb].astype(np.int64)
        if asym:
            comp = O.int8_weight_block_sums(qw, len(cols), K, zp, wd, G, bk).astype(np.int64)
            za2 = np.asarray(za, dtype=np.int64).reshape(Mr if per_m else 1, Kc if per_k else 1)
            want = want - comp[:, kb][None, :] * za2[:, kc].reshape(-1, 1)
        assert np.abs(want).max() * 3 * 2.0 ** -24 < 0.5
        g = (kb * bk) // G if G > 0 else 0
        denom = sa2[:, kc].reshape(-1, 1).astype(np.float64) * s_eff[:, g][None, :].astype(np.float64)
        with np.errstate(divide="ignore", invalid="ignore"):
            got = np.rint(acc / denom)
        got = np.where(denom == 0, 0, got)  # an all-zero row: scale 0, accumulator 0
        want = np.where(denom == 0, 0, want)
        assert np.array_equal(got, want), (label, kernel, kb, int(np.abs(got - want).max()))
    return kernel


def _check_int8_exact_accumulator(case, mode, want_kernel=None, cols=None, label=""):
    """Power-of-two scales on both sides: the fp32 accumulator of the serving kernel equals the oracle's."""
    case = _pow2_weight_scales(case, 11)
    N, K, G, wd = case["N"], case["K"], case["group_size"], case["weight_dtype"]
    M = case["x"].shape[0]
    assert wd != O.WOQ_DTYPE_NF4  # its weight scale carries fp32(1 / 127): not a power of two
    bk = O.int8_block_k(G, K)
    case["x"] = _plant_pow2_activation_scales(case["x"], mode, G if G > 0 else bk, 5)
    ctx = make_context(case, O.LOWP_INT8, mode)
    acc = ctx.run(case["x"].cuda(), out_fp32=True)
    kernel = _served_by(want_kernel, label)
    c = case_np(case)
    cols = np.arange(N) if cols is None else np.asarray(cols)
    acc = acc[:, torch.as_tensor(cols).cuda()].cpu().numpy()
    sc = c["scales"].reshape(N, -1)[cols]
    zp = None if c["zps"] is None else c["zps"].reshape(N, -1)[cols]
    r = O.woq_linear_opt_int8(c["x"], "bf16", c["qw"][cols], len(cols), K, sc if G > 0 else sc.reshape(-1), zp, None, wd, G, mode)
    sa = np.asarray(r["sa"], dtype=np.float64)
    assert np.all(np.log2(sa) == np.rint(np.log2(sa))), "the planted activation scales are powers of two"
    # every term of the epilogue is an integer multiple of `unit`; while the sum of the terms' magnitudes
    # stays below 2^24 units every partial sum is exact in fp32, in any order
    per_m, per_k = mode in (2, 3, 6, 7), mode in (1, 3, 5, 7)
    qbk = G if G > 0 else bk
    KB, Kc = K // bk, (K + qbk - 1) // qbk
    sa2 = sa.reshape(M if per_m else 1, Kc if per_k else 1)
    sa_kb = sa2[:, [(kb * bk) // qbk if per_k else 0 for kb in range(KB)]]  # [M or 1, KB]
    sw_kb = sc.astype(np.float64)[:, [(kb * bk) // G if G > 0 else 0 for kb in range(KB)]]  # [cols, KB]
    unit = sa.min() * 2.0 ** -7
    mags = np.einsum("mnk,mk,nk->mn", np.abs(r["ints"]).astype(np.float64), np.broadcast_to(sa_kb, (M, KB)), sw_kb)
    assert mags.max() / unit < 2 ** 24, (label, mags.max() / unit)
    assert np.array_equal(acc, r["acc"]), (label, kernel, float(np.abs(acc - r["acc"]).max()))
    return kernel


@pytest.mark.parametrize("mode", [0, 1, 2, 3, 4, 5, 6, 7])
@pytest.mark.parametrize(
    "M,K,N,G,kernel",
    [
        (1, 1024, 272, 128, "woq_decode_w4i8_kernel"),
        (16, 2048, 1040, 256, "woq_decode_w4i8_kernel"),
        (32, 1024, 8208, -1, "woq_decode_w4i8_kernel"),  # two row tiles, two row-blocks per workgroup
        (64, 1024, 272, 128, "woq_gemm_w4i8_kernel"),
        (150, 1024, 272, 128, "woq_gemm_w4i8_kernel"),
        (100, 4096, 256, 128, "woq_gemm_w4i8_kernel"),  # K shared between the workgroups of a tile
        (300, 2048, 528, 512, "woq_gemm_w4i8_kernel"),  # activation blocks of four tiles
    ],
)
def test_int8_mfma_kernels_block_integers_bit_exact(cuda, mode, M, K, N, G, kernel):
    case = _synthetic().make_int4_case(41, M, K, N, G, outliers=True)
    if mode < 4:
        case["x"] = (case["x"].float() + 0.5).to(torch.bfloat16)
    cols = None if N < 4096 else list(range(0, N, 53)) + [N - 1]
    label = f"int8 block integers mode={mode} M={M} K={K} N={N} G={G}"
    blocks = None if K <= 2048 else [0, 1, 13, K // 128 - 1]
    _check_int8_block_integers(case, mode, blocks=blocks, cols=cols, want_kernel=kernel, label=label)
    _check_int8_exact_accumulator(case, mode, want_kernel=kernel, cols=cols, label=label)


@pytest.mark.parametrize("mode", [4, 5, 6, 7])
@pytest.mark.parametrize(
    "M,K,N,G,kernel",
    [
        (9, 512, 144, 32, "woq_decode_w4i8_kernel"),  # K blocks inside a packed tile: lane-column masking
        (32, 1024, 272, 32, "woq_decode_w4i8_kernel"),
        (2, 384, 48, 64, "woq_decode_w4i8_kernel"),
        (64, 512, 144, 64, "woq_decode_w4i8_kernel"),  # four row tiles
        (65, 1024, 272, 64, "woq_gemm_w4i8_kernel"),
        (150, 2048, 528, 32, None),  # per-(row, K block) scales stay on the general kernel, the others do not
        (100, 4096, 256, 32, None),
    ],
)
def test_int8_mfma_kernels_small_groups_block_integers_bit_exact(cuda, mode, M, K, N, G, kernel):
    case = _synthetic().make_int4_case(42, M, K, N, G, outliers=True)
    label = f"int8 block integers small groups mode={mode} M={M} K={K} N={N} G={G}"
    if kernel is None:
        kernel = "woq_gemm_i8_kernel" if (G == 32 and mode in (5, 7)) else "woq_gemm_w4i8_kernel"
    blocks = None if K // G <= 16 else sorted({0, 1, 2, 3, 4, 37 % (K // G), K // G - 1})
    _check_int8_block_integers(case, mode, blocks=blocks, want_kernel=kernel, label=label)
    _check_int8_exact_accumulator(case, mode, want_kernel=kernel, label=label)


@pytest.mark.parametrize("mode", [4, 6, 7])
@pytest.mark.parametrize(
    "M,K,N,G,kernel",
    [
        (1, 1024, 272, -1, "woq_decode_w4i8_kernel"),
        (17, 1152, 96, 128, "woq_decode_w4i8_kernel"),
        (70, 2048, 528, 128, "woq_gemm_w4i8_kernel"),
        (300, 1024, 1040, 256, "woq_gemm_w4i8_kernel"),
    ],
)
def test_int8_mfma_kernels_int8_weights_block_integers_bit_exact(cuda, mode, M, K, N, G, kernel):
    """Symmetric 8-bit weights: the stored bytes with the sign bit flipped are the MFMA operand."""
    case = _synthetic().make_int8_case(43, M, K, N, bias=False, group_size=G)
    label = f"int8 block integers int8 weights mode={mode} M={M} K={K} N={N} G={G}"
    _check_int8_block_integers(case, mode, want_kernel=kernel, label=label)
    _check_int8_exact_accumulator(case, mode, want_kernel=kernel, label=label)


@pytest.mark.parametrize("mode", [6, 7])
@pytest.mark.parametrize("M,K,N,G,kernel", [(1, 1024, 272, 128, "woq_decode_w4i8_kernel"), (40, 512, 144, 32, None),
                                            (150, 1024, 272, 128, "woq_gemm_w4i8_kernel")])
def test_int8_mfma_kernels_nf4_block_integers_bit_exact(cuda, mode, M, K, N, G, kernel):
    """NF4 codes as int8 table values through two byte permutes."""
    case = _synthetic().make_nf4_case(44, M, K, N, G)
    _check_int8_block_integers(case, mode, want_kernel=kernel,
                               label=f"int8 block integers nf4 mode={mode} M={M} K={K} N={N} G={G}")


@pytest.mark.parametrize("mode", [6, 7])
def test_c3_prefill_int8_block_integers_bit_exact(cuda, mode):
    """The named prefill configuration at full size (M = 2048, 4096 -> 14336, G = 128, 1 % outliers) on the
    kernel that serves it: K blocks 0, 1, 13 and 31 alone (every 61st column, every 8th row against the
    oracle), then all blocks with power-of-two scales: accumulators equal to the oracle's."""
    case = _synthetic().make_int4_case(3, 2048, 4096, 14336, 128, outliers=True)
    cols = np.arange(0, 14336, 61)
    _check_int8_block_integers(case, mode, blocks=[0, 1, 13, 31], rows=np.arange(0, 2048, 8), cols=cols,
                               want_kernel="woq_gemm_w4i8_kernel", label=f"C3 int8 block integers mode={mode}")
    _check_int8_exact_accumulator(case, mode, want_kernel="woq_gemm_w4i8_kernel", cols=cols,
                                  label=f"C3 int8 exact accumulator mode={mode}")


# ---------------------------------------------------------------------------------------------
# post-ops and size-independent properties
# ---------------------------------------------------------------------------------------------
def test_fused_post_ops(cuda):
    from ipex_amd import _lib

    case = _synthetic().make_int4_case(23, 9, 512, 96, 128, bias=True)
    ctx = make_context(case, O.LOWP_BF16)
    x = case["x"].cuda()
    base = ctx.run(x)
    o1 = torch.randn(9, 96, device=cuda).bfloat16()
    o2 = torch.randn(9, 96, device=cuda).bfloat16()
    F = torch.nn.functional
    checks = {
        _lib.FUSE_RELU: F.relu(base.float()),
        _lib.FUSE_SILU: F.silu(base.float()),
        _lib.FUSE_GELU_ERF: F.gelu(base.float()),
        _lib.FUSE_GELU_TANH: F.gelu(base.float(), approximate="tanh"),
    }
    for fusion, want in checks.items():
        got = ctx.run(x, fusion=fusion)
        assert torch.allclose(got.float(), want.bfloat16().float(), atol=2e-2, rtol=2e-2), fusion
    assert torch.equal(ctx.run(x, fusion=_lib.FUSE_ADD, others=(o1,)), (base.float() + o1.float()).bfloat16())
    assert torch.equal(ctx.run(x, fusion=_lib.FUSE_MUL, others=(o1,)), (base.float() * o1.float()).bfloat16())
    want = ((base.float() + o1.float()).bfloat16().float() + o2.float()).bfloat16()
    assert torch.equal(ctx.run(x, fusion=_lib.FUSE_ADD_ADD, others=(o1, o2)), want)


@pytest.mark.parametrize("K", [256, 384, 4096])
def test_output_rounding_chain_with_bias(cuda, K):
    """Hand-built sums (every weight is (q - z) * s = 1, so the GEMM result is the sum of the row) on which
    the number of roundings shows: the fp16 regime rounds the sum to fp16, adds the fp16 bias in fp16 and
    casts (as the fallback does, woq.h:3569-3576); the bf16 regime adds the fp32 bias before its single
    rounding (woq.h:3298-3310, 3452).  K = 256 / 4096: the integer-weight decode kernels, 384: the others."""
    from ipex_amd import ops

    N = 32
    qw = torch.full((N, K // 2), 0x99, dtype=torch.uint8)
    scales, zeros = torch.ones(N, 1), torch.full((N, 1), 8.0)
    # fp16 regime, fp16 rows: 1 + 2^-11 + 2^-13 -> fp16 1 + 2^-10; + 2^-11 -> tie -> 1 + 2^-9
    for M in (1, 3):
        x = torch.zeros(M, K, dtype=torch.float16)
        x[:, 0], x[:, K // 2], x[:, K - 1] = 1.0, 2.0 ** -11, 2.0 ** -13
        ctx = ops.WoqLinearOpContext(qw.cuda(), 2, [N, K], scales.cuda(), zeros.cuda(),
                                     torch.full((N,), 2.0 ** -11).cuda(), None, None, -1, O.LOWP_FP16, -1)
        y = ctx.run(x.cuda())
        assert torch.all(y.float() == 1 + 2.0 ** -9), (M, y.float().unique())
    # bf16 regime (M >= 5): 1 + 2^-8 + 2^-10 + bias 2^-8 = 1 + 2^-7 + 2^-10 -> 1 + 2^-7 in one rounding
    for M in (5, 70):
        x = torch.zeros(M, K, dtype=torch.bfloat16)
        x[:, 0], x[:, K // 2], x[:, K - 1] = 1.0, 2.0 ** -8, 2.0 ** -10
        ctx = ops.WoqLinearOpContext(qw.cuda(), 2, [N, K], scales.cuda(), zeros.cuda(),
                                     torch.full((N,), 2.0 ** -8).cuda(), None, None, -1, O.LOWP_BF16, -1)
        y = ctx.run(x.cuda())
        assert torch.all(y.float() == 1.0078125), (M, y.float().unique())
    # lowp_mode BF16 below five rows computes in fp16 on bf16 rows: fp16(1 + 2^-8 + 2^-10) is exact, the fp16 bias
    # 2^-8 gives 1 + 2^-7 + 2^-10 (exact in fp16), and the cast to bf16 rounds it to 1 + 2^-7
    x = torch.zeros(2, K, dtype=torch.bfloat16)
    x[:, 0], x[:, K // 2], x[:, K - 1] = 1.0, 2.0 ** -8, 2.0 ** -10
    y = ctx.run(x.cuda())
    assert torch.all(y.float() == 1.0078125)


def test_linearity_in_scales_at_full_size(cuda):
    # doubling every scale doubles the fp32 accumulator exactly (powers of two commute with
    # every rounding on the path); run at the full decode shape
    syn = _synthetic()
    case = syn.make_int4_case(2, 4, 4096, 14336, 128)
    a1 = make_context(case, O.LOWP_BF16).run(case["x"].cuda(), out_fp32=True)
    case2 = dict(case)
    case2["scales"] = case["scales"] * 2
    a2 = make_context(case2, O.LOWP_BF16).run(case["x"].cuda(), out_fp32=True)
    assert torch.equal(a2, a1 * 2)


def test_zero_point_equal_to_weight_gives_bias(cuda):
    # q == z everywhere -> every dequantized weight is 0 -> output is exactly the bias
    syn = _synthetic()
    case = syn.make_int4_case(24, 5, 1024, 272, 128, bias=True)
    q = torch.full((272, 1024), 7, dtype=torch.uint8)
    case["qweight"] = (q[:, 1::2] << 4) | q[:, ::2]
    case["zeros"] = torch.full_like(case["zeros"], 7.0)
    y = make_context(case, O.LOWP_BF16).run(case["x"].cuda())
    assert torch.equal(y.cpu(), case["bias"].unsqueeze(0).expand(5, -1))
    y = make_context(case, O.LOWP_INT8, 6).run(case["x"].cuda())
    assert torch.equal(y.cpu(), case["bias"].unsqueeze(0).expand(5, -1))


def test_determinism(cuda):
    case = _synthetic().make_int4_case(2, 8, 4096, 14336, 128)
    ctx = make_context(case, O.LOWP_BF16)
    x = case["x"].cuda()
    assert torch.equal(ctx.run(x), ctx.run(x))


# ---------------------------------------------------------------------------------------------
# GPTQ act-order (g_idx)
# ---------------------------------------------------------------------------------------------
def _g_idx_cases(K, G):
    n_groups = K // G
    yield "interleaved", torch.arange(n_groups).repeat(G)  # as the reference's tests build it
    perm = torch.randperm(K, generator=torch.Generator().manual_seed(K + G))
    yield "random", (torch.arange(K) // G)[perm]


class _Unshuffled:
    """Feeds a context built with g_idx the activations in checkpoint order when the caller holds
    them sorted by group."""

    def __init__(self, ctx, dst):
        self.ctx, self.dst = ctx, dst

    def run(self, x_sorted, **kw):
        return self.ctx.run(x_sorted[:, self.dst.to(x_sorted.device)].contiguous(), **kw)


@pytest.mark.parametrize("M", [3, 9, 80])
def test_g_idx_matches_the_group_sorted_problem(cuda, M):
    """w[n, k] = (q[n, k] - z[n, g_idx[k]]) * s[n, g_idx[k]]: sorting the channels by group with
    numpy gives an ordinary group-wise problem, which the oracle evaluates; the context built with
    g_idx must give the same result on the unsorted activations."""
    from ipex_amd import ops

    K, N, G = 512, 96, 128
    for name, g_idx in _g_idx_cases(K, G):
        case = _synthetic().make_int4_case(31, M, K, N, G, bias=True)
        src = np.argsort(g_idx.numpy(), kind="stable")
        dst = torch.from_numpy(np.argsort(src))
        q = O.unpack_int4(case["qweight"].numpy())[:, :K]
        sorted_case = dict(case)
        sorted_case["x"] = case["x"][:, torch.from_numpy(src)].contiguous()
        sorted_case["qweight"] = torch.from_numpy(O.pack_int4(np.ascontiguousarray(q[:, src])))
        ctx = ops.WoqLinearOpContext(
            case["qweight"].cuda(), 2, [N, K], case["scales"].cuda(), case["zeros"].cuda(), case["bias"].cuda(),
            g_idx, None, G, O.LOWP_BF16, -1,
        )
        _check_fp(sorted_case, O.LOWP_BF16, ctx=_Unshuffled(ctx, dst), label=f"g_idx {name} M={M}")
        # the checkpoint layout comes back bit-exactly, and the context pickles with its g_idx
        assert torch.equal(ctx.to_public(ctx.get_weight()).cpu(), case["qweight"])
        assert torch.equal(ctx.get_g_idx().cpu(), g_idx)
        ctx2 = pickle.loads(pickle.dumps(ctx))
        x = case["x"].cuda()
        assert torch.equal(ctx2.run(x), ctx.run(x))
        # the registered operator on the custom class built with the same g_idx: the same bits
        assert torch.equal(_shipped_binding_output(case, O.LOWP_BF16, g_idx=g_idx), ctx.run(x)), name
        assert torch.equal(_shipped_binding_output(case, O.LOWP_INT8, 6, g_idx=g_idx),
                           make_context(sorted_case, O.LOWP_INT8, 6).run(sorted_case["x"].cuda())), name
        # lowp INT8 goes through the same shuffles: identical to the context of the sorted problem
        ctx_i8 = ops.WoqLinearOpContext(
            case["qweight"].cuda(), 2, [N, K], case["scales"].cuda(), case["zeros"].cuda(), case["bias"].cuda(),
            g_idx, None, G, O.LOWP_INT8, 6,
        )
        ref_i8 = make_context(sorted_case, O.LOWP_INT8, 6)
        assert torch.equal(ctx_i8.run(x), ref_i8.run(sorted_case["x"].cuda()))


@pytest.mark.parametrize("M", [17, 200])
def test_g_idx_under_lowp_fp16_with_bf16_rows(cuda, M):
    """fp16 compute on bf16 rows beyond one row tile casts the rows around the call: the act-order
    shuffle must be applied once, not once per cast level.  Checked against the oracle on the
    group-sorted problem and bit for bit against the context of the sorted problem."""
    from ipex_amd import ops

    K, N, G = 512, 96, 128
    for name, g_idx in _g_idx_cases(K, G):
        case = _synthetic().make_int4_case(36, M, K, N, G, bias=True)
        src = np.argsort(g_idx.numpy(), kind="stable")
        dst = torch.from_numpy(np.argsort(src))
        q = O.unpack_int4(case["qweight"].numpy())[:, :K]
        sorted_case = dict(case)
        sorted_case["x"] = case["x"][:, torch.from_numpy(src)].contiguous()
        sorted_case["qweight"] = torch.from_numpy(O.pack_int4(np.ascontiguousarray(q[:, src])))
        ctx = ops.WoqLinearOpContext(
            case["qweight"].cuda(), 2, [N, K], case["scales"].cuda(), case["zeros"].cuda(), case["bias"].cuda(),
            g_idx, None, G, O.LOWP_FP16, -1,
        )
        ref = make_context(sorted_case, O.LOWP_FP16)
        y = ctx.run(case["x"].cuda())
        assert torch.equal(y, ref.run(sorted_case["x"].cuda())), name
        # the registered operator on the custom class: one shuffle there too
        assert torch.equal(_shipped_binding_output(case, O.LOWP_FP16, g_idx=g_idx), y), name
        c = case_np(sorted_case)
        _, want = O.woq_linear_ref(c["x"], "bf16", c["qw"], N, K, O._round_to(c["scales"], "fp16"), c["zps"], c["bias"],
                                   2, G, "fp16")
        assert rel_l2(to_np_f32(y), want) <= REL_L2_OUT, name


@pytest.mark.parametrize("M,K,N,G,bias", [(17, 512, 96, 128, True), (64, 1024, 272, 128, False), (200, 512, 96, 128, True),
                                          (300, 1024, 528, 64, False)])
def test_lowp_fp16_on_bf16_rows_beyond_one_tile(cuda, M, K, N, G, bias):
    """fp16 compute on a bf16 tensor of more than 16 rows: the library converts the rows to fp16 with its own
    kernel and the fp16 kernels write the bf16 output (no casts around the call).  Equal, bit for bit, to the
    same call on rows converted by torch with the fp16 result cast by torch; within the output gate of the
    fallback in fp16 arithmetic; the same through the C++ operator."""
    from ipex_amd import _kernels

    case = _synthetic().make_int4_case(61, M, K, N, G, bias=bias)
    ctx = make_context(case, O.LOWP_FP16)
    x = case["x"].cuda()
    xh = _kernels.convert_activations(x, torch.float16)
    assert torch.equal(xh, x.to(torch.float16))
    y = ctx.run(x)
    assert y.dtype == torch.bfloat16
    assert torch.equal(y, ctx.run(x.to(torch.float16)).to(torch.bfloat16))
    c = case_np(case)
    _, want = O.woq_linear_ref(c["x"], "bf16", c["qw"], N, K, O._round_to(c["scales"], "fp16"), c["zps"], c["bias"],
                               2, G, "fp16")
    assert rel_l2(to_np_f32(y), want) <= REL_L2_OUT
    tc = make_torch_context(case, O.LOWP_FP16)
    assert torch.equal(torch.ops.torch_ipex.ipex_woq_linear(x, tc.get_data_handle()), y)


def test_convert_activations_rounds_to_nearest_even(cuda):
    """Every dtype pair against torch's conversion, on every finite bf16 / fp16 bit pattern and on fp32 values
    that sit on and beside rounding ties; ragged counts and a pointer that is not 16-byte aligned."""
    from ipex_amd import _kernels

    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    for src in (torch.bfloat16, torch.float16):
        v = bits.view(src)
        v = v[torch.isfinite(v.float())].cuda()
        for dst in (torch.float16, torch.bfloat16, torch.float32):
            got = _kernels.convert_activations(v, dst)
            want = v.to(dst)
            assert torch.equal(got.view(torch.int16 if dst != torch.float32 else torch.int32),
                               want.view(torch.int16 if dst != torch.float32 else torch.int32)), (src, dst)
    g = torch.Generator().manual_seed(5)
    f = torch.randn(100003, generator=g) * 3.0
    ties = (torch.arange(0, 4096, dtype=torch.int32) << 12 | 0x3F800000).view(torch.float32)  # fp16 / bf16 ties
    f = torch.cat([f, ties, -ties, ties * (1 + 2.0 ** -20)]).cuda()
    for dst in (torch.float16, torch.bfloat16):
        assert torch.equal(_kernels.convert_activations(f, dst), f.to(dst)), dst
    odd = torch.randn(4099, generator=g).bfloat16().cuda()[3:]  # 4096 elements, 6 bytes past an aligned address
    assert torch.equal(_kernels.convert_activations(odd, torch.float16), odd.to(torch.float16))


def test_other_16_bit_output_type_rejections(cuda):
    """The other 16-bit output type is for plain calls only."""
    from ipex_amd import _kernels, _lib

    case = _synthetic().make_int4_case(62, 20, 256, 48, 128)
    ctx = make_context(case, O.LOWP_FP16)
    xh = case["x"].cuda().to(torch.float16)
    other = torch.zeros(20, 48, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="other 16-bit type"):
        ctx.run(xh, fusion=_lib.FUSE_ADD, others=(other,), out_dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="other 16-bit type"):
        ctx.run(case["x"].cuda().float(), out_dtype=torch.bfloat16)


def test_g_idx_validation(cuda):
    from ipex_amd import ops

    case = _synthetic().make_int4_case(32, 2, 256, 32, 128)
    args = lambda g: (case["qweight"].cuda(), 2, [32, 256], case["scales"].cuda(), case["zeros"].cuda(), None, g, None,
                      128, O.LOWP_BF16, -1)
    with pytest.raises(RuntimeError, match="mismatch"):
        ops.WoqLinearOpContext(*args(torch.zeros(100, dtype=torch.int64)))
    with pytest.raises(RuntimeError, match="exactly group_size"):
        ops.WoqLinearOpContext(*args(torch.zeros(256, dtype=torch.int64)))
    with pytest.raises(RuntimeError, match="must lie in"):
        ops.WoqLinearOpContext(*args(torch.full((256,), 5, dtype=torch.int64)))


# ---------------------------------------------------------------------------------------------
# seeded random shapes through the automatic dispatch
# ---------------------------------------------------------------------------------------------
def _random_cases(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        kind = ["int4", "int4", "int4", "int8", "nf4"][int(rng.integers(0, 5))]
        M = int(rng.choice([1, 2, 3, 4, 5, 7, 12, 16, 17, 29, 32, 33, 47, 64, 65, 90, 128, 150, 260]))
        G = int(rng.choice([-1, 32, 64, 128, 256]))
        if kind == "int8":
            G = -1
        kmul = 8 if rng.random() < 0.2 else (64 if kind == "int8" else 128)  # sometimes a ragged K
        K = int(rng.integers(1, 9)) * kmul * (1 if kmul > 8 else int(rng.integers(4, 40)))
        if G > 0:
            K = max(G, (K // G) * G) if rng.random() < 0.8 else K  # mostly whole groups
        K += K % 2  # two nibbles per byte
        N = int(rng.choice([16, 17, 48, 64, 100, 272, 500, 1024]))
        out.append((i, kind, M, K, N, G, bool(rng.random() < 0.5), bool(rng.random() < 0.3)))
    return out


@pytest.mark.parametrize("idx,kind,M,K,N,G,bias,sym", _random_cases(48, 2024))
def test_random_shapes_float_regimes(cuda, idx, kind, M, K, N, G, bias, sym):
    syn = _synthetic()
    if kind == "int8":
        case = syn.make_int8_case(100 + idx, M, K, N, bias=bias)
    elif kind == "nf4":
        case = syn.make_nf4_case(100 + idx, M, K, N, G, bias=bias)
    else:
        case = syn.make_int4_case(100 + idx, M, K, N, G, bias=bias)
        if sym:
            case["zeros"] = None
    _check_fp(case, O.LOWP_BF16, label=f"random {idx}: {kind} M={M} K={K} N={N} G={G} bias={bias} sym={sym}")


@pytest.mark.parametrize("idx,kind,M,K,N,G,bias,sym", [c for c in _random_cases(40, 777) if c[1] != "int8" or True][:32])
def test_random_shapes_lowp_int8(cuda, idx, kind, M, K, N, G, bias, sym):
    """lowp_mode INT8 with a random activation-quantization mode; shapes whose K blocks the int8
    kernels do not take run unquantized, as the reference's fallback does, and are checked as such."""
    syn = _synthetic()
    mode = [6, 7, 4, 5, 2, 3, 0, 1][idx % 8]
    if kind == "int8":
        case = syn.make_int8_case(200 + idx, M, K, N, bias=bias)
    elif kind == "nf4":
        case = syn.make_nf4_case(200 + idx, M, K, N, G, bias=bias)
    else:
        case = syn.make_int4_case(200 + idx, M, K, N, G, bias=bias)
        if sym:
            case["zeros"] = None
    bk = O.int8_block_k(G, K)
    label = f"random int8 {idx}: {kind} mode={mode} M={M} K={K} N={N} G={G}"
    if bk in (32, 64, 128):
        _check_int8(case, mode, label=label)
    else:
        ctx = make_context(case, O.LOWP_INT8, mode)
        y = to_np_f32(ctx.run(case["x"].cuda()))
        c = case_np(case)
        _, y_ref = O.woq_linear_ref(c["x"], "bf16", c["qw"], N, K, O.bf16_round(c["scales"]), c["zps"], c["bias"],
                                    case["weight_dtype"], G, "bf16")
        assert rel_l2(y, y_ref) <= (REL_L2_OUT if c["bias"] is None else 4e-3), label


def _activation_variants(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        act = ["bf16", "fp16", "fp32"][int(rng.integers(0, 3))]
        lowp = int(rng.choice([O.LOWP_NONE, O.LOWP_FP16, O.LOWP_BF16]))
        if act == "fp32" and lowp == O.LOWP_NONE:
            lowp = O.LOWP_BF16
        lead = [(1,), (3,), (2, 5), (1, 40), (4, 33), (2, 3, 7)][int(rng.integers(0, 6))]
        K = int(rng.choice([128, 256, 320, 1000, 1024]))
        G = int(rng.choice([-1, 32, 64, 128]))
        if G > 0 and K % G:
            G = -1
        N = int(rng.choice([16, 48, 100, 272]))
        layout = ["contiguous", "strided_rows", "transposed"][int(rng.integers(0, 3))]
        out.append((i, act, lowp, lead, K, N, G, layout))
    return out


@pytest.mark.parametrize("idx,act,lowp,lead,K,N,G,layout", _activation_variants(36, 99))
def test_activation_dtypes_shapes_and_layouts(cuda, idx, act, lowp, lead, K, N, G, layout):
    """fp16 / fp32 activations (converted inside the kernels), leading dimensions, and inputs that
    are views: the op takes what nn.Linear takes."""
    tdt = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[act]
    M = int(np.prod(lead))
    case = _synthetic().make_int4_case(300 + idx, M, K, N, G, bias=(idx % 2 == 0))
    x2 = case["x"].float().to(tdt)  # values representable in bf16 whatever the dtype
    ctx = make_torch_context(case, lowp)
    xg = x2.cuda()
    if layout == "strided_rows":
        wide = torch.zeros(M, K + 8, dtype=tdt, device=cuda)
        wide[:, :K] = xg
        xin = wide[:, :K]
    elif layout == "transposed":
        xin = xg.t().contiguous().t()
    else:
        xin = xg
    assert layout == "contiguous" or not xin.is_contiguous() or M == 1 or K == 1
    y = torch.ops.torch_ipex.ipex_woq_linear(xin.reshape(*lead, K) if layout == "contiguous" else xin, ctx.get_data_handle())
    assert y.dtype == tdt and tuple(y.shape) == ((*lead, N) if layout == "contiguous" else (M, N))
    y = to_np_f32(y).reshape(M, N)
    c = case_np(case)
    xs = to_np_f32(x2)
    cd = O.select_compute(lowp, act, M)
    if cd == "bf16":
        _, want = O.woq_linear_opt_bf16(xs, act, c["qw"], N, K, c["scales"], c["zps"], c["bias"], 2, G)
    else:
        _, want = O.woq_linear_ref(xs, act, c["qw"], N, K, O._round_to(c["scales"], cd), c["zps"], c["bias"], 2, G, cd)
    assert rel_l2(y, want) <= REL_L2_OUT, (idx, act, lowp, lead, K, N, G, layout, rel_l2(y, want))


# ---- fp32 compute: lowp_mode NONE with fp32 activations (WoqLinearKrnl.cpp:142-158) -----------
@pytest.mark.parametrize(
    "kind,M,K,N,G,bias",
    [
        ("int4", 1, 4096, 512, 128, False),
        ("int4", 130, 1000, 272, -1, True),   # ragged K, N and M; K % 4 == 0
        ("int4", 7, 250, 48, -1, False),      # K % 4 != 0: element-wise activation loads
        ("int4", 33, 640, 100, 32, True),
        ("int4sym", 5, 512, 80, 64, False),
        ("int8", 33, 512, 100, -1, True),
        ("int8", 3, 320, 272, 64, False),
        ("nf4", 40, 512, 80, 64, True),
    ],
)
def test_fp32_compute(cuda, kind, M, K, N, G, bias):
    """fp32 scales kept unrounded, w = (q - z) * s in fp32, fp32 products and sums, fp32 output:
    against the fallback oracle in fp32 (float64 sums), to fp32 summation accuracy."""
    syn = _synthetic()
    if kind == "int8":
        case = syn.make_int8_case(410, M, K, N, bias=bias, group_size=G)
    elif kind == "nf4":
        case = syn.make_nf4_case(411, M, K, N, G, bias=bias, scale_dtype=torch.float32)
    else:
        case = syn.make_int4_case(412, M, K, N, G, bias=bias, scale_dtype=torch.float32)
        if kind == "int4sym":
            case["zeros"] = None
    gen = torch.Generator().manual_seed(413)
    x = torch.randn(M, K, generator=gen)  # genuine fp32 values, not bf16-representable ones
    ctx = make_torch_context(case, O.LOWP_NONE)
    y = torch.ops.torch_ipex.ipex_woq_linear(x.cuda(), ctx.get_data_handle())
    assert y.dtype == torch.float32 and tuple(y.shape) == (M, N)
    c = case_np(case)
    assert O.select_compute(O.LOWP_NONE, "fp32", M) == "fp32"
    acc, want = O.woq_linear_ref(x.numpy(), "fp32", c["qw"], N, K, c["scales"], c["zps"], c["bias"],
                                 case["weight_dtype"], G, "fp32")
    got = y.cpu().numpy()
    assert rel_l2(got, acc) <= 1e-5, (kind, M, K, N, G, rel_l2(got, acc))
    assert max_abs(got, acc) <= 2e-4 * max(1.0, float(np.abs(acc).max())), (kind, M, K, N, G, max_abs(got, acc))
    # lowp_mode INT8 on fp32 activations runs unquantized in fp32 as well
    # (WoqInt8GemmAPerMKrnl.cpp:143-169): same kernel, same bits
    if kind in ("int4sym", "int8", "nf4"):
        ctx8 = make_context(case, O.LOWP_INT8, 6)
        assert torch.equal(ctx8.run(x.cuda()), y)


def test_fp32_compute_post_ops(cuda):
    from ipex_amd import _lib
    import torch.nn.functional as F

    case = _synthetic().make_int4_case(420, 9, 256, 64, 128, bias=True, scale_dtype=torch.float32)
    gen = torch.Generator().manual_seed(421)
    x = torch.randn(9, 256, generator=gen).cuda()
    o1, o2 = torch.randn(9, 64, generator=gen).cuda(), torch.randn(9, 64, generator=gen).cuda()
    ctx = make_context(case, O.LOWP_NONE)
    base = ctx.run(x)
    assert base.dtype == torch.float32
    assert torch.allclose(ctx.run(x, fusion=_lib.FUSE_SILU), F.silu(base), atol=1e-4, rtol=1e-4)
    assert torch.allclose(ctx.run(x, fusion=_lib.FUSE_GELU_ERF), F.gelu(base), atol=1e-4, rtol=1e-4)
    assert torch.equal(ctx.run(x, fusion=_lib.FUSE_RELU), F.relu(base))
    assert torch.equal(ctx.run(x, fusion=_lib.FUSE_ADD, others=(o1,)), base + o1)
    assert torch.equal(ctx.run(x, fusion=_lib.FUSE_MUL, others=(o1,)), base * o1)
    assert torch.equal(ctx.run(x, fusion=_lib.FUSE_ADD_ADD, others=(o1, o2)), base + o1 + o2)


@pytest.mark.parametrize("K,N", [(2048, 8192), (1024, 512), (512, 272), (4096, 512)])
def test_single_row_decode_with_four_k_tiles_per_wave(cuda, K, N):
    """M = 1 on layers small enough that the kernel gives every wave four K tiles instead of two."""
    from ipex_amd import _lib

    case = _synthetic().make_int4_case(77, 1, K, N, 128, bias=(N % 32 == 16))
    _check_fp(case, O.LOWP_BF16, label=f"M=1 K={K} N={N}")
    assert _lib.last_kernel() == "woq_decode_m1_kernel"
    case16 = dict(case)
    case16["x"] = case["x"].to(torch.float16)
    ctx = make_context(case16, O.LOWP_FP16)
    c = case_np(case16)
    y = to_np_f32(ctx.run(case16["x"].cuda()))
    _, want = O.woq_linear_ref(c["x"], "fp16", c["qw"], N, K, O._round_to(c["scales"], "fp16"), c["zps"], c["bias"], 2, 128, "fp16")
    assert rel_l2(y, want) <= REL_L2_OUT


@pytest.mark.parametrize(
    "K,N,bias",
    [
        (4096, 14336, False),  # two row-blocks per workgroup, 16 waves x two K tiles, one round
        (4096, 4096, False),   # one row-block per workgroup
        (14336, 4096, True),   # several rounds
        (2048, 8192, False),   # four K tiles per wave, two row-blocks
        (1024, 512, True),     # four K tiles per wave, one row-block
        (256, 48, False),      # a single wave
        (8192, 8192, True),    # several rounds with two row-blocks
    ],
)
@pytest.mark.parametrize("G", [32, 64])
def test_decode_kernels_with_groups_of_32_and_64(cuda, K, N, bias, G):
    """Up to four rows with groups of 32 or 64 input channels on the integer-weight decode kernels: the four or two
    groups of a K tile stay apart in rows of the MFMA's activation operand.  Symmetric weights and fp16 rows
    (lowp_mode FP16) as well; five and more rows keep the dequantizing kernel."""
    from ipex_amd import _lib

    syn = _synthetic()
    cols = None if N * K <= 4096 * 4096 else np.arange(0, N, 7)
    case = syn.make_int4_case(78, 1, K, N, G, bias=bias)
    _check_fp(case, O.LOWP_BF16, cols=cols, label=f"M=1 G={G} K={K} N={N}")
    assert _lib.last_kernel() == "woq_decode_m1_kernel"
    ctx = make_context(case, O.LOWP_BF16)
    x = case["x"].cuda()
    a, b = to_np_f32(ctx.run(x)), to_np_f32(ctx.run(x, force_kernel=1))
    assert rel_l2(a, b) <= 2e-3
    assert torch.equal(ctx.run(x), ctx.run(x))
    sym = dict(case, zeros=None)
    _check_fp(sym, O.LOWP_BF16, cols=cols, label=f"M=1 G={G} symmetric K={K} N={N}")
    case16 = dict(case)
    case16["x"] = case["x"].to(torch.float16)
    ctx16 = make_context(case16, O.LOWP_FP16)
    c = case_np(case16)
    y = to_np_f32(ctx16.run(case16["x"].cuda()))
    assert _lib.last_kernel() == "woq_decode_m1_kernel"
    if cols is None:
        _, want = O.woq_linear_ref(c["x"], "fp16", c["qw"], N, K, O._round_to(c["scales"], "fp16"), c["zps"], c["bias"], 2, G, "fp16")
        assert rel_l2(y, want) <= REL_L2_OUT
    # two to four rows: the same arrangement with row 4 g + m of the A operand for group g of activation row m
    for M in (2, 3, 4):
        more = syn.make_int4_case(79 + M, M, K, N, G, bias=bias)
        _check_fp(more, O.LOWP_BF16, cols=cols, label=f"M={M} G={G} K={K} N={N}")
        assert _lib.last_kernel() == "woq_decode_kernel"
        ctxm = make_context(more, O.LOWP_BF16)
        xm = more["x"].cuda()
        assert rel_l2(to_np_f32(ctxm.run(xm)), to_np_f32(ctxm.run(xm, force_kernel=1))) <= 2e-3
    five = syn.make_int4_case(85, 5, K, N, G, bias=bias)
    make_context(five, O.LOWP_BF16).run(five["x"].cuda())
    assert _lib.last_kernel() == "woq_decode_dq_kernel"
