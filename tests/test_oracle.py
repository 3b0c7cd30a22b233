"""Pins the CPU oracle: every function is checked against something the oracle did not
compute itself -- hand-built bytes, brute force in exact arithmetic, invariants of the
definition, or the AWQ tensors the reference's own test holds."""
import fractions
import os

import numpy as np
import pytest
import torch

from oracle import woq_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def test_nibble_order_closed_form():
    # byte j = q[2j] | q[2j+1] << 4
    q = np.array([[1, 2, 3, 4, 15, 0]], dtype=np.uint8)
    packed = O.pack_int4(q)
    assert packed.tolist() == [[0x21, 0x43, 0x0F]]
    assert O.unpack_int4(packed).tolist() == q.tolist()
    # odd K pads one zero element
    assert O.pack_int4(np.array([[7, 9, 5]], dtype=np.uint8)).tolist() == [[0x97, 0x05]]


def test_compressed_zero_points_closed_form():
    # 8 zero points per int32, value j in nibble j
    word = sum(((j + 3) % 16) << (4 * j) for j in range(8))
    zp32 = np.array([[word, 0x0000_00A5]], dtype=np.uint32).view(np.int32)
    out = O.unpack_compressed_zeros(zp32, 10)
    assert out.tolist() == [[(j + 3) % 16 for j in range(8)] + [5, 10]]
    # high bit set in the word must not sign-extend
    zp32 = np.array([[0xF000_0000]], dtype=np.uint32).view(np.int32)
    assert O.unpack_compressed_zeros(zp32, 8).tolist() == [[0, 0, 0, 0, 0, 0, 0, 15]]


def test_dequantize_brute_force_all_codes():
    # every code x every zero point, one group each: (q - z) * s in exact rationals
    codes = np.arange(16, dtype=np.uint8)
    K = 16
    for z in range(16):
        qw = O.pack_int4(codes[None, :])
        s = np.float32(0.0123)
        got = O.dequantize_woq_weight(qw, 1, K, np.array([[s]]), np.array([[float(z)]]), O.WOQ_DTYPE_INT4, 16)
        want = [float(fractions.Fraction(int(c) - z) * fractions.Fraction(float(s))) for c in codes]
        assert np.array_equal(got[0], np.array(want, dtype=np.float32))
    # symmetric int4 is stored +8
    got = O.dequantize_woq_weight(O.pack_int4(codes[None, :]), 1, K, np.array([2.0]), None, O.WOQ_DTYPE_INT4, -1)
    assert got[0].tolist() == [2.0 * (c - 8) for c in range(16)]


def test_nf4_table_is_the_normal_quantile_code_book():
    # The published construction of NormalFloat4 (QLoRA): 8 positive quantiles of N(0, 1) at
    # linspace(offset, 0.5, 9)[:-1], zero, 7 negative ones at linspace(offset, 0.5, 8)[:-1],
    # sorted and divided by the largest.  A mistyped or swapped entry misses it by far more than
    # the fp32 rounding of the published digits.
    from scipy.stats import norm

    off = 0.9677083
    pos = norm.ppf(np.linspace(off, 0.5, 9)[:-1])
    neg = -norm.ppf(np.linspace(off, 0.5, 8)[:-1])
    v = np.sort(np.concatenate([pos, [0.0], neg]))
    v /= v.max()
    t = O.NF4_DEQUANT_TABLE
    assert t.dtype == np.float32 and t.shape == (16,)
    assert np.abs(v - t).max() <= 2e-7
    assert t[0] == -1.0 and t[7] == 0.0 and t[15] == 1.0 and np.all(np.diff(t) > 0)


def test_nf4_dequantize_brute_force_and_groups():
    # every code in every group: table[code] * scale of that group, a single fp32 product
    N, K, G = 2, 64, 16
    codes = np.tile(np.arange(16, dtype=np.uint8), (N, K // 16))
    codes[1] = codes[1, ::-1]
    scales = np.array([[0.5, 0.031, 3.0, 0.0123], [1.0, 0.07, 0.25, 9.0]], dtype=np.float32)
    w = O.dequantize_woq_weight(O.pack_int4(codes), N, K, scales, None, O.WOQ_DTYPE_NF4, G)
    for n in range(N):
        for k in range(K):
            exact = fractions.Fraction(float(O.NF4_DEQUANT_TABLE[codes[n, k]])) * fractions.Fraction(float(scales[n, k // G]))
            assert w[n, k] == np.float32(float(exact)), (n, k)
    # per-channel
    w = O.dequantize_woq_weight(O.pack_int4(codes), N, K, np.array([2.0, 4.0], np.float32), None, O.WOQ_DTYPE_NF4, -1)
    assert np.array_equal(w[0], 2 * O.NF4_DEQUANT_TABLE[codes[0]]) and np.array_equal(w[1], 4 * O.NF4_DEQUANT_TABLE[codes[1]])
    with pytest.raises(AssertionError):
        O.dequantize_woq_weight(O.pack_int4(codes), N, K, scales, scales, O.WOQ_DTYPE_NF4, G)


def test_nf4_linear_paths_against_exact_rational_matmul():
    rng = np.random.default_rng(5)
    M, K, N, G = 3, 32, 4, 16
    codes = rng.integers(0, 16, (N, K)).astype(np.uint8)
    qw = O.pack_int4(codes)
    scales = O.bf16_round(rng.uniform(0.02, 0.08, (N, K // G)).astype(np.float32))
    x = O.bf16_round(rng.standard_normal((M, K)).astype(np.float32))
    w = O.bf16_round(O.dequantize_woq_weight(qw, N, K, scales, None, O.WOQ_DTYPE_NF4, G))
    exact = np.array(
        [[float(sum(fractions.Fraction(float(x[m, k])) * fractions.Fraction(float(w[n, k])) for k in range(K)))
          for n in range(N)] for m in range(M)]
    )
    acc, y = O.woq_linear_opt_bf16(x, "bf16", qw, N, K, scales, None, None, O.WOQ_DTYPE_NF4, G)
    assert np.abs(acc - exact).max() <= 1e-12
    assert np.array_equal(y, O.bf16_round(exact.astype(np.float32)))
    # the fp16 chain rounds the table to fp16 and accumulates in fp16: close to, not equal to, exact
    yh = O.woq_linear_opt_fp16(x, qw, N, K, scales, None, None, O.WOQ_DTYPE_NF4, G)
    assert np.abs(yh - exact).max() <= 2e-2 * max(1.0, np.abs(exact).max())
    # a zero scale row gives exact zeros whatever the codes (code 7 is 0, no implied offset)
    s0 = scales.copy()
    s0[2] = 0
    assert np.all(O.woq_linear_opt_fp16(x, qw, N, K, s0, None, None, O.WOQ_DTYPE_NF4, G)[:, 2] == 0)


def test_nf4_int8_table_and_lowp_int8_linear():
    # the int8 table is the float table times 127, rounded (closed form), and antisymmetric at the ends
    assert np.array_equal(O.NF4_TO_INT8_TABLE, np.rint(O.NF4_DEQUANT_TABLE.astype(np.float64) * 127).astype(np.int64))
    assert O.NF4_TO_INT8_TABLE[7] == 0 and O.NF4_TO_INT8_TABLE[0] == -127 and O.NF4_TO_INT8_TABLE[15] == 127
    rng = np.random.default_rng(8)
    M, K, N, G = 3, 256, 5, 128
    codes = rng.integers(0, 16, (N, K)).astype(np.uint8)
    qw = O.pack_int4(codes)
    scales = rng.uniform(0.02, 0.08, (N, K // G)).astype(np.float32)
    x = O.bf16_round(rng.standard_normal((M, K)).astype(np.float32))
    r = O.woq_linear_opt_int8(x, "bf16", qw, N, K, scales, None, None, O.WOQ_DTYPE_NF4, G, 6)
    # integer block sums: Python integers over the table values
    B = [[int(O.NF4_TO_INT8_TABLE[c]) for c in row] for row in codes]
    for m in range(M):
        for n in range(N):
            for kb in range(K // 128):
                want = sum(int(r["xq"][m, k]) * B[n][k] for k in range(kb * 128, (kb + 1) * 128))
                assert int(r["sums"][m, n, kb]) == want
    # the epilogue undoes both quantizations: close to the float product with table * scale weights
    w = O.dequantize_woq_weight(qw, N, K, scales, None, O.WOQ_DTYPE_NF4, G).astype(np.float64)
    exact = x.astype(np.float64) @ w.T
    assert np.abs(r["acc"] - exact).max() <= 0.02 * np.abs(exact).max() + 0.05
    # and it is exactly sum_kb (float(sum) * s_a) * (s_w * fp32(1 / 127)) in fp32
    f = np.float32
    for m in range(M):
        for n in range(N):
            c = f(0)
            for kb in range(K // 128):
                sw = f(scales[n, kb] * (f(1.0) / f(127.0)))
                c = f(c + f(f(f(r["sums"][m, n, kb]) * f(r["sa"][m])) * sw))
            assert r["acc"][m, n] == c


def test_nf4_quantize_dequantize_roundtrip_error_bound():
    # the package's quantizer picks the nearest table entry: error <= half the widest gap x scale
    from ipex_amd.quantization._qconfig import WoqWeightDtype
    from ipex_amd.quantization._quantize_utils import quantize_per_block

    torch.manual_seed(3)
    wt = torch.randn(8, 128) * 0.05
    qw, sc, zp = quantize_per_block(wt, WoqWeightDtype.NF4, 32, sym_quant=True)
    assert zp is None
    w = O.dequantize_woq_weight(qw.numpy(), 8, 128, sc.numpy(), None, O.WOQ_DTYPE_NF4, 32)
    half_gap = float(np.diff(O.NF4_DEQUANT_TABLE).max()) / 2
    bound = half_gap * np.repeat(sc.numpy(), 32, axis=1)
    assert np.all(np.abs(w - wt.numpy()) <= bound + 1e-7)
    # the group's extreme element is reproduced exactly (code 0 or 15)
    amax = wt.view(8, 4, 32).abs().max(dim=-1)[0].numpy()
    assert np.allclose(np.abs(w).reshape(8, 4, 32).max(axis=-1), amax, rtol=0, atol=1e-7)


def test_fp8_e4m3fn_tables():
    # the value table against an independent implementation: torch's float8_e4m3fn -> float32
    t = O.FP8_E4M3FN_TABLE
    want = torch.arange(256, dtype=torch.int16).to(torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert t.dtype == np.float32 and t.shape == (256,)
    assert np.array_equal(np.isnan(t), np.isnan(want)) and list(np.flatnonzero(np.isnan(t))) == [0x7F, 0xFF]
    ok = ~np.isnan(want)
    assert np.array_equal(t[ok].view(np.uint32), want[ok].view(np.uint32))  # bit for bit, -0.0 included
    # landmarks of the format
    assert t[0x7E] == 448.0 and t[0x08] == 2.0**-6 and t[0x01] == 2.0**-9 and t[0x07] == 7 * 2.0**-9
    assert t[0x38] == 1.0 and t[0xB8] == -1.0
    # the reference kernels' conversion: the same on +-0 and on every normal code ...
    k = O.FP8_E4M3FN_KERNEL_TABLE
    normal = np.array([b for b in range(256) if (b & 0x7F) == 0 or ((b >> 3) & 15) >= 1 and (b & 0x7F) != 0x7F])
    assert len(normal) == 256 - 16
    assert np.array_equal(k[normal].view(np.uint32), t[normal].view(np.uint32))
    # ... a subnormal code read as exponent -7 with a hidden one (0.0019..0.0137 "cannot be converted
    # correctly", vec512_fp8.h:94-98): m = 1 -> 1.125 / 128, m = 7 -> 1.875 / 128; NaN codes -> 1.875 * 2^8
    hand = {0x01: 0.0087890625, 0x02: 0.009765625, 0x03: 0.0107421875, 0x04: 0.01171875, 0x05: 0.0126953125,
            0x06: 0.013671875, 0x07: 0.0146484375, 0x7F: 480.0}
    for b, v in hand.items():
        assert k[b] == np.float32(v) and k[b | 0x80] == np.float32(-v), hex(b)
    # the largest deviation from the float8 value of a non-NaN code: code 0x01, 9 * 2^-10 - 2 * 2^-10
    assert np.nanmax(np.abs(k - t)) == 7 * 2.0**-10


def test_fp8_dequantize_and_linear_against_exact_rationals():
    # every byte, two scale groups: (table value) * scale in fp32, and the GEMM on top of it
    qw = np.arange(256, dtype=np.uint8).reshape(1, 256).repeat(2, 0)
    qw[1] = qw[1, ::-1]
    s = np.array([[0.5, 0.0078125], [3.0, 0.001953125]], dtype=np.float32)
    w = O.dequantize_woq_weight(qw, 2, 256, s, None, O.WOQ_DTYPE_FP8, 128)
    k = O.FP8_E4M3FN_KERNEL_TABLE
    for n in range(2):
        for c in range(256):
            assert w[n, c] == np.float32(k[qw[n, c]]) * s[n, c // 128]
    assert np.array_equal(O.dequantize_woq_weight(qw.view(np.int8), 2, 256, s, None, O.WOQ_DTYPE_FP8, 128), w)
    with pytest.raises(AssertionError):
        O.dequantize_woq_weight(qw, 2, 256, s, s, O.WOQ_DTYPE_FP8, 128)
    rng = np.random.default_rng(5)
    x = O.bf16_round(rng.standard_normal((3, 256)).astype(np.float32))
    acc, y = O.woq_linear_ref(x, "bf16", qw, 2, 256, s, None, None, O.WOQ_DTYPE_FP8, 128, "bf16")
    wb = O.bf16_round(w)
    for m in range(3):
        for n in range(2):
            exact = sum(fractions.Fraction(float(x[m, c])) * fractions.Fraction(float(wb[n, c])) for c in range(256))
            assert abs(float(exact) - acc[m, n]) <= 1e-9 * max(1.0, abs(float(exact)))
            assert y[m, n] == O.bf16_round(np.float32(float(exact)))


def test_moe_token_lists_and_weighted_scatter():
    rng = np.random.default_rng(11)
    T, topk, E, H = 9, 3, 5, 6
    ids = np.stack([rng.permutation(E)[:topk] for _ in range(T)])
    top_x, idx = O.expert_token_lists(ids, E)
    for e in range(E):  # independent formulation: row-major nonzero of the mask
        r, c = np.nonzero(ids == e)
        assert np.array_equal(top_x[e], r) and np.array_equal(idx[e], c)
    assert sum(len(t) for t in top_x) == T * topk
    # weighted scatter: exact rationals, rounded once (bf16 / fp32) or twice (fp16)
    for dtype in ("bf16", "fp16", "fp32"):
        rt = lambda a: O._round_to(np.asarray(a, dtype=np.float32), dtype)
        out0, rw = rt(rng.standard_normal((T, H))), rt(rng.uniform(0, 1, (T, topk)))
        e = int(np.argmax([len(t) for t in top_x]))
        cur = rt(rng.standard_normal((len(top_x[e]), H)))
        got = O.moe_index_mul_index_add(out0, cur, rw, top_x[e], idx[e], dtype)
        want = out0.copy()
        for i, (t, j) in enumerate(zip(top_x[e], idx[e])):
            for h in range(H):
                prod = fractions.Fraction(float(cur[i, h])) * fractions.Fraction(float(rw[t, j]))
                if dtype == "fp16":
                    prod = fractions.Fraction(float(np.float16(np.float32(float(prod)))))
                    # (the fp32 product of two fp16 values is exact, so this is the fp16 rounding of it)
                # fp32 rounding of the product, then of the sum, then the dtype
                p32 = np.float32(float(prod))
                want[t, h] = rt(np.float32(p32 + want[t, h]))
        assert np.array_equal(got, want), dtype
        untouched = np.setdiff1d(np.arange(T), top_x[e])
        assert np.array_equal(got[untouched], out0[untouched])


def test_dequantize_group_indexing():
    # group g of row n must use scales[n, g]: make each group's scale identify it
    N, K, G = 3, 96, 32
    q = np.full((N, K), 5, dtype=np.uint8)
    scales = np.arange(1, N * 3 + 1, dtype=np.float32).reshape(N, 3)
    zps = np.full((N, 3), 4.0, dtype=np.float32)
    w = O.dequantize_woq_weight(O.pack_int4(q), N, K, scales, zps, O.WOQ_DTYPE_INT4, G)
    for n in range(N):
        for k in range(K):
            assert w[n, k] == scales[n, k // G]
    # trailing partial group
    w = O.dequantize_woq_weight(O.pack_int4(q[:, :80]), N, 80, scales, zps, O.WOQ_DTYPE_INT4, G)
    assert w[1, 79] == scales[1, 2] and w.shape == (N, 80)


def test_bf16_round_matches_torch_on_all_halfway_cases():
    rng = np.random.default_rng(0)
    x = rng.standard_normal(200000).astype(np.float32) * rng.choice([1e-3, 1.0, 300.0], 200000).astype(np.float32)
    # exact ties: mantissa low 16 bits = 0x8000
    ties = (x.view(np.uint32) & 0xFFFF0000 | 0x8000).view(np.float32)
    for arr in (x, ties):
        want = torch.from_numpy(arr).to(torch.bfloat16).float().numpy()
        assert np.array_equal(O.bf16_round(arr), want)


def test_fma16_is_single_rounding():
    # a*b + c where the double rounding fp32->fp16 would differ from one rounding
    rng = np.random.default_rng(1)
    a = rng.standard_normal(20000).astype(np.float16)
    b = rng.integers(-15, 16, 20000).astype(np.float16)
    c = (rng.standard_normal(20000) * 30).astype(np.float16)
    got = O._fma16(a, b, c)
    want = np.array(
        [
            np.float16(float(fractions.Fraction(float(x)) * fractions.Fraction(float(y)) + fractions.Fraction(float(z))))
            for x, y, z in zip(a[:3000], b[:3000], c[:3000])
        ],
        dtype=np.float16,
    )
    assert np.array_equal(got[:3000], want)


def _tiny_case(M=3, N=5, K=64, G=32, seed=0, bias=True):
    rng = np.random.default_rng(seed)
    x = O.bf16_round(rng.standard_normal((M, K)).astype(np.float32))
    q = rng.integers(0, 16, (N, K)).astype(np.uint8)
    scales = O.bf16_round((0.005 + 0.015 * rng.random((N, K // G))).astype(np.float32))
    zps = rng.integers(0, 16, (N, K // G)).astype(np.float32)
    b = O.bf16_round((0.02 * rng.standard_normal(N)).astype(np.float32)) if bias else None
    return x, q, O.pack_int4(q), scales, zps, b


def test_gemm_paths_against_exact_rational_matmul():
    M, N, K, G = 3, 5, 64, 32
    x, q, qw, scales, zps, b = _tiny_case(M, N, K, G)
    F = fractions.Fraction
    exact = np.zeros((M, N))
    for m in range(M):
        for n in range(N):
            acc = F(0)
            for k in range(K):
                acc += F(float(x[m, k])) * F(int(q[n, k]) - int(zps[n, k // G])) * F(float(scales[n, k // G]))
            exact[m, n] = float(acc + F(float(b[n])))
    # fallback path with fp32 compute: no weight rounding -> equals the exact value to fp64 accuracy
    acc, _ = O.woq_linear_ref(x, "bf16", qw, N, K, scales, zps, b, O.WOQ_DTYPE_INT4, G, "fp32")
    assert np.max(np.abs(acc - exact)) < 1e-5
    # bf16 path: weights rounded to bf16 first -> within K * 2^-9 * |x||w| of exact, and equal to
    # an explicit per-element evaluation
    acc_b, y_b = O.woq_linear_opt_bf16(x, "bf16", qw, N, K, scales, zps, b, O.WOQ_DTYPE_INT4, G)
    manual = np.zeros((M, N))
    for m in range(M):
        for n in range(N):
            tot = F(float(b[n]))
            for k in range(K):
                w = np.float32(np.float32(int(q[n, k]) - zps[n, k // G]) * scales[n, k // G])
                w = torch.tensor(float(w)).to(torch.bfloat16).item()
                tot += F(float(x[m, k])) * F(w)
            manual[m, n] = float(tot)
    assert np.max(np.abs(acc_b - manual)) < 1e-9
    assert np.max(np.abs(acc_b - exact)) < 0.05
    assert np.array_equal(y_b, torch.from_numpy(acc_b.astype(np.float32)).to(torch.bfloat16).float().numpy())
    # fp16 chain: stays within the fp16 accumulation error of the exact value
    y_h = O.woq_linear_opt_fp16(x[:2], qw, N, K, scales, zps, b, O.WOQ_DTYPE_INT4, G)
    assert np.max(np.abs(y_h - exact[:2])) < 0.08


def test_ref_rounding_chain_with_bias_rounds_twice():
    """woq_gemm_ref_impl rounds the GEMM result to the compute dtype, adds the bias in that dtype (a second
    rounding) and casts to the activation dtype (csrc/cpu/aten/utils/woq.h:3569-3576, 3612).  Hand-built
    case where two roundings and one rounding of the exact sum differ: every weight is (q - z) * s = 1, so
    the exact GEMM result is the sum of the activations.
      bf16: sum = 1 + 2^-8 + 2^-10 -> bf16 1 + 2^-7 (above the tie); + bias 2^-8 = 1 + 2^-7 + 2^-8, a tie ->
            even mantissa 1 + 2^-6 = 1.015625.  One rounding of 1 + 2^-7 + 2^-10 would give 1.0078125.
      fp16: the same eight binades further down: 1 + 2^-11 + 2^-13 -> 1 + 2^-10; + 2^-11 -> tie -> 1 + 2^-9."""
    qw = O.pack_int4(np.full((1, 4), 9, dtype=np.uint8))
    scales, zps = np.ones((1, 1), dtype=np.float32), np.full((1, 1), 8, dtype=np.float32)
    x = np.array([[1.0, 2.0 ** -8, 2.0 ** -10, 0.0]], dtype=np.float32)
    acc, y = O.woq_linear_ref(x, "bf16", qw, 1, 4, scales, zps, np.array([2.0 ** -8], dtype=np.float32), 2, 4, "bf16")
    assert float(acc[0, 0]) == 1 + 2.0 ** -7 + 2.0 ** -10
    assert float(y[0, 0]) == 1.015625
    _, y_nobias = O.woq_linear_ref(x, "bf16", qw, 1, 4, scales, zps, None, 2, 4, "bf16")
    assert float(y_nobias[0, 0]) == 1.0078125
    x = np.array([[1.0, 2.0 ** -11, 2.0 ** -13, 0.0]], dtype=np.float32)
    _, y = O.woq_linear_ref(x, "fp16", qw, 1, 4, scales, zps, np.array([2.0 ** -11], dtype=np.float32), 2, 4, "fp16")
    assert float(y[0, 0]) == 1 + 2.0 ** -9
    # bf16 activations under fp16 compute (lowp_mode BF16 with M < 5): the fp16 result 1 + 2^-9 is then cast to
    # bf16, where it rounds to 1
    _, y = O.woq_linear_ref(x, "bf16", qw, 1, 4, scales, zps, np.array([2.0 ** -11], dtype=np.float32), 2, 4, "fp16")
    assert float(y[0, 0]) == 1.0
    # the optimized bf16 kernel adds the fp32 bias before its single rounding
    x = np.array([[1.0, 2.0 ** -8, 2.0 ** -10, 0.0]], dtype=np.float32)
    _, y = O.woq_linear_opt_bf16(x, "bf16", qw, 1, 4, scales, zps, np.array([2.0 ** -8], dtype=np.float32), 2, 4)
    assert float(y[0, 0]) == 1.0078125


def test_fp16_chain_order_matters_and_is_sequential():
    # one output, K = 4: ((x0*w0 + x1*w1) + x2*w2) + x3*w3 in fp16, chosen so that another order differs
    x = np.array([[1024.0, 0.25, 0.25, -1024.0]], dtype=np.float32)
    q = np.array([[9, 9, 9, 9]], dtype=np.uint8)  # z = 8 -> w = 1
    zps = np.array([[8.0]], dtype=np.float32)
    scales = np.array([[1.0]], dtype=np.float32)
    y = O.woq_linear_opt_fp16(x, O.pack_int4(q), 1, 4, scales, zps, None, O.WOQ_DTYPE_INT4, 4, block_k=4)
    # sequential: 1024 + .25 -> 1024 (fp16 ulp at 1024 is 1), again 1024, then 0
    assert y[0, 0] == 0.0
    # per-block scaling happens after the block sum: two blocks of 2
    y2 = O.woq_linear_opt_fp16(x, O.pack_int4(q), 1, 4, np.array([[1.0, 1.0]], np.float32),
                               np.array([[8.0, 8.0]], np.float32), None, O.WOQ_DTYPE_INT4, 2, block_k=2)
    # block0: 1024 (0.25 lost); block1: 0.25 - 1024 -> -1024 (fp16); C = 1024 + (-1024) = 0
    assert y2[0, 0] == 0.0


def test_select_compute_table():
    assert O.select_compute(O.LOWP_BF16, "bf16", 1) == "fp16"
    assert O.select_compute(O.LOWP_BF16, "bf16", 4) == "fp16"
    assert O.select_compute(O.LOWP_BF16, "bf16", 5) == "bf16"
    assert O.select_compute(O.LOWP_NONE, "bf16", 1) == "bf16"
    assert O.select_compute(O.LOWP_NONE, "fp16", 100) == "fp16"
    assert O.select_compute(O.LOWP_FP16, "bf16", 100) == "fp16"
    assert O.select_compute(O.LOWP_INT8, "bf16", 1) == "int8"
    assert O.select_compute(O.LOWP_NONE, "fp32", 1) == "fp32"
    assert [O.int8_block_k(g, 4096) for g in (-1, 32, 64, 128, 256)] == [128, 32, 64, 128, 128]
    assert O.int8_block_k(-1, 4160) == 64


def _all_bf16_values():
    bits = np.arange(65536, dtype=np.uint32)
    v = (bits << 16).view(np.float32)
    return v[np.isfinite(v)]


@pytest.mark.parametrize("mode", [4, 5, 6, 7, 0, 1, 2, 3])
def test_dynamic_quant_invariants_over_all_bf16_patterns(mode):
    vals = _all_bf16_values()
    vals = vals[np.abs(vals) < 1e4]
    rng = np.random.default_rng(3)
    x = rng.permutation(vals)[: 64 * 512].reshape(64, 512).astype(np.float32)
    qbk = 128
    q, s, zp = O.dynamic_quantize_per_block(x, qbk, mode)
    sym = mode >= 4
    per_m = mode in (2, 3, 6, 7)
    per_k = mode in (1, 3, 5, 7)
    assert q.dtype == (np.int8 if sym else np.uint8)
    for m in range(64):
        for kc in range(4 if per_k else 1):
            rows = slice(m, m + 1) if per_m else slice(0, 64)
            cols = slice(kc * qbk, (kc + 1) * qbk) if per_k else slice(0, 512)
            blk, qb = x[rows, cols], q[rows, cols].astype(np.float64)
            idx = tuple(([m] if per_m else []) + ([kc] if per_k else [])) or (0,)
            sc = float(s[idx])
            if sym:
                amax = np.abs(blk).max()
                # the definition: scale = absmax / 127 as an fp32 division
                assert sc == float(np.float32(amax) / np.float32(127))
                # the extreme element lands on +-127, nothing exceeds it
                assert np.abs(qb).max() == 127
                assert np.all(np.abs(blk - qb * sc) <= sc * 0.5 * (1 + 1e-4))
            else:
                z = float(zp[idx])
                assert sc == float(np.float32(blk.max() - blk.min()) / np.float32(255))
                assert qb.min() >= 0 and qb.max() <= 255
                inside = (qb > 0) & (qb < 255)
                assert np.all(np.abs(blk - (qb - z) * sc)[inside] <= sc * 0.5 * (1 + 1e-3))
        if not per_m:
            break


def test_dynamic_quant_rounds_half_to_even():
    # scale = 127/127 = 1 -> q = rint(x): halves go to the even neighbour
    x = np.array([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5]], dtype=np.float32)
    q, s, _ = O.dynamic_quantize_per_block(x, 8, 6)
    assert s.tolist() == [1.0]
    assert q.tolist() == [[127, 0, 2, 2, 0, -2, -2, 4]]
    # asymmetric: zp = -rint(min / s), q = rint(x / s + zp), clamped to 0..255
    x = np.array([[-1.0, 0.0, 1.0, 254.0]], dtype=np.float32)
    q, s, zp = O.dynamic_quantize_per_block(x, 4, 2)
    assert s.tolist() == [1.0] and zp.tolist() == [1]
    assert q.tolist() == [[0, 1, 2, 255]]
    # symmetric clamps at -128..127 only through rounding: -absmax maps to -127
    x = np.array([[-4.0, 4.0, 0.0, 2.0]], dtype=np.float32)
    q, _, _ = O.dynamic_quantize_per_block(x, 4, 6)
    assert q.tolist() == [[-127, 127, 0, 64]]  # 2 / (4/127) = 63.5 -> 64 (even)


def test_int8_block_sums_against_python_integers():
    rng = np.random.default_rng(5)
    M, N, K, G = 3, 4, 256, 128
    xq = rng.integers(-128, 128, (M, K)).astype(np.int8)
    q = rng.integers(0, 16, (N, K)).astype(np.uint8)
    zps = rng.integers(0, 16, (N, K // G)).astype(np.float32)
    sums = O.int8_block_sums(xq, O.pack_int4(q), N, K, zps, O.WOQ_DTYPE_INT4, G, 128)
    for m in range(M):
        for n in range(N):
            for kb in range(2):
                want = sum(int(xq[m, k]) * (int(q[n, k]) - int(zps[n, k // G])) for k in range(kb * 128, kb * 128 + 128))
                assert sums[m, n, kb] == want


def test_int8_linear_epilogue_close_to_exact():
    x, q, qw, scales, zps, b = _tiny_case(M=6, N=5, K=256, G=128, seed=7)
    r = O.woq_linear_opt_int8(x, "bf16", qw, 5, 256, scales, zps, b, O.WOQ_DTYPE_INT4, 128, 6)
    # against the unquantized product: int8 activations carry ~1/127 relative error per element
    acc_exact, _ = O.woq_linear_ref(x, "bf16", qw, 5, 256, scales, zps, b, O.WOQ_DTYPE_INT4, 128, "fp32")
    assert np.max(np.abs(r["acc"] - acc_exact)) < 0.1
    # and exactly the definition when re-evaluated in float64 from the integer sums
    sa = r["sa"].astype(np.float64).reshape(-1, 1)
    want = b.astype(np.float64)[None, :] + sum(
        r["sums"][:, :, kb].astype(np.float64) * sa * scales[:, kb].astype(np.float64)[None, :] for kb in range(2)
    )
    assert np.max(np.abs(r["acc"] - want)) < 1e-5


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_int8_linear_asymmetric_activations_is_the_dequantized_product(mode):
    """Pins the compensation term (its sign, its block index, which zero point multiplies it):
    sum_k (q_a - zp_a) s_a (q_w - z_w) s_w, evaluated exactly from the quantized tensors, must be
    what the integer-compensation form gives; a wrong sign or index is off by whole units."""
    x, q, qw, scales, zps, b = _tiny_case(M=6, N=5, K=256, G=128, seed=11)
    x = x + np.float32(0.75)  # an offset makes the zero points large
    r = O.woq_linear_opt_int8(x, "bf16", qw, 5, 256, scales, zps, b, O.WOQ_DTYPE_INT4, 128, mode)
    assert r["xq"].dtype == np.uint8 and r["za"] is not None
    per_m, per_k = mode in (2, 3), mode in (1, 3)
    sa = np.asarray(r["sa"], dtype=np.float64).reshape(6 if per_m else 1, 2 if per_k else 1)
    za = np.asarray(r["za"], dtype=np.float64).reshape(6 if per_m else 1, 2 if per_k else 1)
    kcol = (np.arange(256) // 128) if per_k else np.zeros(256, dtype=np.int64)
    xdq = (r["xq"].astype(np.float64) - za[:, kcol]) * sa[:, kcol]  # broadcasts over rows if not per_m
    g = np.arange(256) // 128
    wdq = (q.astype(np.float64) - zps.astype(np.float64)[:, g]) * scales.astype(np.float64)[:, g]
    want = xdq @ wdq.T + b.astype(np.float64)[None, :]
    assert np.max(np.abs(r["acc"] - want)) < 1e-4
    # and it approximates the unquantized product
    acc_exact, _ = O.woq_linear_ref(x, "bf16", qw, 5, 256, scales, zps, b, O.WOQ_DTYPE_INT4, 128, "fp32")
    assert np.max(np.abs(r["acc"] - acc_exact)) < 0.1


def test_int8_weight_block_sums_closed_form():
    rng = np.random.default_rng(12)
    N, K, G = 3, 256, 64
    q = rng.integers(0, 16, (N, K)).astype(np.uint8)
    zps = rng.integers(0, 16, (N, K // G)).astype(np.float32)
    comp = O.int8_weight_block_sums(O.pack_int4(q), N, K, zps, O.WOQ_DTYPE_INT4, G, 64)
    for n in range(N):
        for kb in range(K // 64):
            assert comp[n, kb] == sum(int(q[n, k]) - int(zps[n, k // G]) for k in range(kb * 64, kb * 64 + 64))


def _awq_decode_independent(qweight, qzeros, scales, group_size):
    """AutoAWQ GEMM packing, restated from its definition: word [k, j] holds column
    8j + ORDER[i] in nibble i, ORDER = [0, 2, 4, 6, 1, 3, 5, 7]."""
    order = [0, 2, 4, 6, 1, 3, 5, 7]
    K, N8 = qweight.shape
    w = np.zeros((K, N8 * 8), dtype=np.int64)
    z = np.zeros((qzeros.shape[0], N8 * 8), dtype=np.int64)
    qwu = qweight.astype(np.int64) & 0xFFFFFFFF
    qzu = qzeros.astype(np.int64) & 0xFFFFFFFF
    for i in range(8):
        w[:, order[i]::8] = (qwu >> (4 * i)) & 0xF
        z[:, order[i]::8] = (qzu >> (4 * i)) & 0xF
    g = np.arange(K) // group_size
    return ((w - z[g]) * scales[g].astype(np.float64)).T  # [N, K]


def test_awq_fixture_decode():
    p = os.path.join(GOLDEN, "awq_fixture.pt")
    d = torch.load(p, weights_only=True)
    qweight, qzeros, scales = d["qweight"].numpy(), d["qzeros"].numpy(), d["scales"].float().numpy()
    want = _awq_decode_independent(qweight, qzeros, scales, 128)
    # the product's converters + the oracle's dequantize must reproduce it
    from ipex_amd.utils.weight_only_quantization import _convert_awq_scales_qzeros, awq_to_plain

    plain = awq_to_plain(d["qweight"]).numpy()
    s2, z2 = _convert_awq_scales_qzeros(d["scales"], d["qzeros"])
    K, N = qweight.shape[0], qweight.shape[1] * 8
    got = O.dequantize_woq_weight(plain, N, K, s2.float().numpy(), z2.float().numpy(), O.WOQ_DTYPE_INT4, 128)
    assert np.max(np.abs(got - want)) < 1e-6
