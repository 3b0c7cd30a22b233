"""CPU restatement of the reference's weight-only-quantized linear -- TEST INFRASTRUCTURE ONLY.

Nothing in the product imports this file: it is the checker used by tests/, by
__graft_entry__.smoke() and by the cpu_baseline leg of bench.py.

It restates, in numpy, the arithmetic of intel/intel-extension-for-pytorch's WOQ linear
(paths relative to the reference tree):

  unpack_int4 / pack_int4            quantization/_quantize_utils.py:1184, 1247-1251;
                                     csrc/cpu/aten/utils/woq_utils.h:93-97
  unpack_compressed_zeros            csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:98-103
  dequantize_woq_weight              csrc/cpu/aten/utils/woq_utils.h:79-163
  woq_linear_ref                     woq_gemm_ref_impl, csrc/cpu/aten/utils/woq.h:3511-3613
  woq_linear_opt_fp16                GemmMicroKernel<half>, woq.h:775-951 under the driver
                                     qlinear_woq_affine_impl<bf16, half, half, bf16, half, half>
                                     (woq.h:3250-3477, kernels/WoqFp16GemmKrnl.cpp:98-121)
  woq_linear_opt_bf16                Dequantize<bfloat16> + BRGEMM, woq.h:1495-1581, 1847-1944,
                                     3298-3310, 3452
  dynamic_quantize_per_block         csrc/cpu/aten/utils/woq_dynamic_quant.h:1526-1750
  woq_linear_opt_int8                Dequantize<int8_t> + int8 BRGEMM + fp32 epilogue,
                                     woq.h:1664-1734, 2133-2199; driver woq.h:3298-3452
  expert_token_lists                 get_expert_topx_idx, csrc/cpu/aten/MoE.cpp:64-81
  moe_index_mul_index_add            fuse_index_mul_index_add, csrc/cpu/aten/kernels/MoEKrnl.cpp:31-121,
                                     and the generic branch :277-280
  select_compute                     qlinear_woq_affine, kernels/WoqLinearKrnl.cpp:56-161
  int8_block_k                       get_block_k, csrc/cpu/aten/Linear.cpp:362-376

How each function is pinned (see tests/test_oracle.py):
  * nibble order, compressed zero points: closed forms checked against hand-built bytes;
  * dequantize: brute force over all 16 codes x zero points, and the AWQ fixture the
    reference's own test holds (tests/cpu/data/awq/*.pt) against an independent decode;
  * GEMMs: exact rational / float64 brute force on tiny shapes;
  * dynamic quantization: properties the definition fixes (round-half-even at constructed ties,
    extreme element maps to +-127 / 0 / 255, |x - q*s| <= s/2) over all 65536 bf16 patterns;
  * int8 block sums: exact integer arithmetic against a Python big-int loop;
  * NF4 table: the published normal-quantile construction (scipy), codes by brute force;
  * float8 e4m3fn: the value table against torch's float8_e4m3fn -> float32 conversion on all 256 bytes
    and the format's landmarks (448 the largest, 2^-6 the smallest normal, 2^-9 the smallest subnormal);
    the reference kernels' conversion against that table on every normal code and +-0, and on the 16
    codes where it differs against the values the reference's own comment names
    (csrc/cpu/vec/vec512/vec512_fp8.h:94-98) worked out by hand;
  * MoE token lists / weighted scatter: an independent formulation (nonzero per expert) and exact
    rationals rounded once.
PARITY UNPINNED (no fixture or invariant can fix them; they are below the stated tolerances):
  * the fp32 accumulation order inside libxsmm BRGEMM / oneDNN (third_party/libxsmm, an
    un-vendored submodule whose pinned commit is not recoverable from the mount) -- the
    oracle accumulates in float64 instead;
  * whether the compiler contracted `C += (qC * s_a) * s_w` (woq.h:2172-2186) into an FMA --
    the oracle uses separate roundings;
  * whether the CPU compiler contracted `out + cs * rw` (MoEKrnl.cpp:107-108) into an FMA -- the
    oracle multiplies and adds separately;
  * the k order and chain structure of the fp16 micro-kernel are restated from the source
    text (woq.h:919-940) and could only be confirmed by running an AVX512-FP16 build.
"""
import numpy as np

WOQ_DTYPE_INT8, WOQ_DTYPE_INT4, WOQ_DTYPE_NF4, WOQ_DTYPE_FP8 = 1, 2, 3, 4  # csrc/cpu/aten/utils/woq_defines.h:6-9
LOWP_NONE, LOWP_FP16, LOWP_BF16, LOWP_INT8 = 0, 1, 2, 3
SMALL_BATCH_THRESHOLD = 5  # IPEX_WOQ_SMALL_BATCH_THRESHOLD, woq.h:24


# ---------------------------------------------------------------------------------------------
# bf16 helpers (numpy has no bfloat16): values are carried as float32 that are exactly bf16.
# ---------------------------------------------------------------------------------------------
def bf16_round(x):
    """float32 -> nearest bf16 (ties to even), returned as float32."""
    x = np.asarray(x, dtype=np.float32)
    bits = x.view(np.uint32).astype(np.uint64)
    lsb = (bits >> 16) & 1
    rounded = ((bits + 0x7FFF + lsb) >> 16) << 16
    out = rounded.astype(np.uint32).view(np.float32)
    nan = np.isnan(x)
    if np.any(nan):
        out = np.where(nan, np.float32(np.nan), out)
    return out.reshape(x.shape)


def bf16_bits_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(x):
    return (bf16_round(x).view(np.uint32) >> 16).astype(np.uint16)


def f16_round(x):
    """float -> nearest fp16 (ties to even), returned as float32."""
    return np.asarray(x).astype(np.float16).astype(np.float32)


# ---------------------------------------------------------------------------------------------
# wire format
# ---------------------------------------------------------------------------------------------
def pack_int4(q):
    """codes 0..15 [N, K] -> bytes [N, ceil(K/2)]; element 2j in the low nibble of byte j."""
    q = np.asarray(q, dtype=np.uint8)
    if q.shape[1] % 2:
        q = np.pad(q, ((0, 0), (0, 1)))
    return ((q[:, 1::2] << 4) | (q[:, ::2] & 0xF)).astype(np.uint8)


def unpack_int4(qw):
    qw = np.asarray(qw, dtype=np.uint8)
    out = np.empty((qw.shape[0], qw.shape[1] * 2), dtype=np.uint8)
    out[:, ::2] = qw & 0xF
    out[:, 1::2] = qw >> 4
    return out


def unpack_compressed_zeros(zp32, cols):
    """zp[i, j] = (zp32[i, j // 8] >> (4 * (j % 8))) & 0xf"""
    z = np.asarray(zp32).view(np.uint32) if np.asarray(zp32).dtype == np.int32 else np.asarray(zp32, dtype=np.uint32)
    j = np.arange(cols)
    return ((z[:, j // 8] >> ((j % 8) * 4).astype(np.uint32)) & 0xF).astype(np.float32)


# The NormalFloat4 code book (csrc/cpu/aten/utils/woq_utils.h:34-51): 16 values in [-1, 1], code 7
# is exactly zero.
NF4_DEQUANT_TABLE = np.array(
    [
        -1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453,
        -0.28444138169288635, -0.18477343022823334, -0.09105003625154495, 0.0,
        0.07958029955625534, 0.16093020141124725, 0.24611230194568634, 0.33791524171829224,
        0.44070982933044434, 0.5626170039176941, 0.7229568362236023, 1.0,
    ],
    dtype=np.float32,
)


def _fp8_e4m3fn_table():
    """All 256 float8 e4m3fn values (the dtype of the reference's FP8 weights, torch.float8_e4m3fn:
    weight_only_quantization.py:238, tests/cpu/test_quantization_default_recipe.py:2155-2226): 1 sign bit,
    4 exponent bits with bias 7, 3 mantissa bits, no infinities, exponent 15 with mantissa 7 is NaN;
    exponent 0 is subnormal (mantissa * 2^-9)."""
    t = np.zeros(256, dtype=np.float32)
    for b in range(256):
        e, m = (b >> 3) & 15, b & 7
        if e == 15 and m == 7:
            v = np.nan
        elif e == 0:
            v = m * 2.0 ** -9
        else:
            v = (1.0 + m / 8.0) * 2.0 ** (e - 7)
        t[b] = -v if b & 0x80 else v
    return t


FP8_E4M3FN_TABLE = _fp8_e4m3fn_table()


def _fp8_e4m3fn_kernel_table():
    """What the reference's weight-only kernels make of each float8 e4m3fn byte
    (convert_fp8_e4m3_to_fp32, csrc/cpu/aten/utils/woq.h:465-485, restated on the integers): mantissa
    << 20 | (exponent + 120) << 23, zeroed when the 7 low bits are zero, | sign << 24.  Equal to the
    float8 value on +-0 and every normal code; the subnormal codes 0x01..0x07 come out as
    (8 + m) * 2^-10 (float8: m * 2^-9) and the NaN codes 0x7F / 0xFF as +-480 (the conversion "without
    denorm behavior" that csrc/cpu/vec/vec512/vec512_fp8.h:94-98 describes)."""
    x = np.arange(256, dtype=np.uint32)
    nonsign = np.where((x & 127) != 0, ((x & 7) << 20) | ((((x >> 3) & 15) + 120) << 23), 0).astype(np.uint32)
    return (nonsign | ((x & 128) << 24)).astype(np.uint32).view(np.float32)


FP8_E4M3FN_KERNEL_TABLE = _fp8_e4m3fn_kernel_table()


def dequantize_woq_weight(qw, N, K, scales, zps, weight_dtype, group_size):
    """fp32 (q - z) * s; q - z first, then the scale, both in fp32.  zps None: symmetric (INT4
    codes stand for code - 8).  FP8: qw holds float8 e4m3fn bytes, each converted as the reference's kernels convert it, times s.  NF4: table[code] * s, no zero point
    (csrc/cpu/aten/utils/woq_utils.h:64-77, 108-131).  scales / zps: [N] or
    [N, ceil(K / group_size)]."""
    if weight_dtype == WOQ_DTYPE_NF4:
        assert zps is None, "NF4 is symmetric"
        q = NF4_DEQUANT_TABLE[unpack_int4(qw)[:, :K]]
    elif weight_dtype == WOQ_DTYPE_INT4:
        q = unpack_int4(qw)[:, :K].astype(np.float32)
        if zps is None:
            q = q - np.float32(8)
    elif weight_dtype == WOQ_DTYPE_INT8:
        q = np.asarray(qw, dtype=np.int8).astype(np.float32)
    elif weight_dtype == WOQ_DTYPE_FP8:
        # the byte converted to the compute type (exactly: 4 significant bits) times the scale
        # (load_dequant_fp8, csrc/cpu/aten/utils/woq.h:728-741); no zero points
        assert zps is None, "FP8 weights are symmetric"
        q = FP8_E4M3FN_KERNEL_TABLE[np.asarray(qw).view(np.uint8)]
    else:
        raise NotImplementedError("oracle: weight dtype")
    s = np.asarray(scales, dtype=np.float32).reshape(N, -1)
    z = None if zps is None else np.asarray(zps, dtype=np.float32).reshape(N, -1)
    if group_size > 0:
        g = np.arange(K) // group_size
        s_full = s[:, g]
        z_full = None if z is None else z[:, g]
    else:
        s_full = np.broadcast_to(s[:, :1], (N, K))
        z_full = None if z is None else np.broadcast_to(z[:, :1], (N, K))
    if z_full is not None:
        q = q - z_full
    return (q * s_full).astype(np.float32)


# ---------------------------------------------------------------------------------------------
# kernel selection
# ---------------------------------------------------------------------------------------------
def select_compute(lowp_mode, act_dtype, M):
    """'fp16' | 'bf16' | 'int8' | 'fp32' as qlinear_woq_affine picks it."""
    if lowp_mode == LOWP_FP16 or (lowp_mode == LOWP_NONE and act_dtype == "fp16") or (
        lowp_mode == LOWP_BF16 and M < SMALL_BATCH_THRESHOLD
    ):
        return "fp16"
    if (lowp_mode == LOWP_NONE and act_dtype == "bf16") or (lowp_mode == LOWP_BF16 and M >= SMALL_BATCH_THRESHOLD):
        return "bf16"
    if lowp_mode == LOWP_INT8:
        return "int8"
    return "fp32"


def int8_block_k(group_size, K):
    bk = min(group_size, 128) if group_size > 0 else 128
    while K % bk != 0:
        bk //= 2
    return bk


def _round_to(x, dt):
    if dt == "bf16":
        return bf16_round(x)
    if dt == "fp16":
        return f16_round(x)
    return np.asarray(x, dtype=np.float32)


# ---------------------------------------------------------------------------------------------
# fallback implementation (what the reference runs without AVX512-FP16)
# ---------------------------------------------------------------------------------------------
def woq_linear_ref(x, act_dtype, qw, N, K, scales, zps, bias, weight_dtype, group_size, compute_dtype):
    """w = ((q - z) * s).to(cd); y = linear(x.to(cd), w) (result in cd); y += bias.to(cd) (in cd);
    y.to(act dtype).  x: float32 array holding act_dtype values.  Returns (acc, y): acc is the
    float64 dot product plus bias before any output rounding, y the final values as float32."""
    w = _round_to(dequantize_woq_weight(qw, N, K, scales, zps, weight_dtype, group_size), compute_dtype)
    xc = _round_to(x, compute_dtype)
    acc = xc.astype(np.float64) @ w.astype(np.float64).T
    y = _round_to(acc.astype(np.float32), compute_dtype)
    acc_b = acc
    if bias is not None:
        b = _round_to(np.asarray(bias, dtype=np.float32), compute_dtype)
        y = _round_to(y + b, compute_dtype)
        acc_b = acc + np.asarray(bias, dtype=np.float64)
    return acc_b, _round_to(y, act_dtype)


# ---------------------------------------------------------------------------------------------
# optimized kernels
# ---------------------------------------------------------------------------------------------
def _fma16(a, b, c):
    """fp16 fused multiply-add: a * b + c rounded once to fp16.  float64 holds a * b exactly
    (22 bits) and the sum exactly unless |c| dwarfs |ab| by more than 2**30, in which case the
    result rounds to c either way."""
    return (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(np.float16)


def woq_linear_opt_fp16(x, qw, N, K, scales, zps, bias, weight_dtype, group_size, block_k=None):
    """The M < 5 path with bf16 activations: everything in fp16, including the accumulators.
    Per output: C = fp16(bias) or 0; per K block of Kb = min(group_size, 64):
    vc = 0; for k ascending: vc = fma(x_k, q_k - z, vc); then C = fma(s, vc, C); y = bf16(C).
    NF4: q_k is the table value rounded to fp16 and there is no z (the fp16 lookup table of
    csrc/cpu/aten/utils/woq.h:827-836)."""
    assert weight_dtype in (WOQ_DTYPE_INT4, WOQ_DTYPE_NF4)
    nf4 = weight_dtype == WOQ_DTYPE_NF4
    assert not (nf4 and zps is not None), "NF4 is symmetric"
    M = x.shape[0]
    if block_k is None:
        block_k = min(group_size, 64) if group_size > 0 else 64
        while K % block_k:
            block_k //= 2
    q = unpack_int4(qw)[:, :K]
    q = NF4_DEQUANT_TABLE[q].astype(np.float16) if nf4 else q.astype(np.float16)
    s = np.asarray(scales, dtype=np.float32).reshape(N, -1).astype(np.float16)
    z = None if zps is None else np.asarray(zps, dtype=np.float32).reshape(N, -1).astype(np.float16)
    xh = np.asarray(x, dtype=np.float32).astype(np.float16)
    C = np.zeros((M, N), dtype=np.float16)
    if bias is not None:
        C[:] = np.asarray(bias, dtype=np.float32).astype(np.float16)[None, :]
    for kb in range(K // block_k):
        g = (kb * block_k) // group_size if group_size > 0 else 0
        zg = z[:, g] if z is not None else np.float16(0 if nf4 else 8)
        vc = np.zeros((M, N), dtype=np.float16)
        for k in range(kb * block_k, (kb + 1) * block_k):
            w = (q[:, k] - zg).astype(np.float16)  # exact small integers
            vc = _fma16(xh[:, k : k + 1], w[None, :], vc)
        C = _fma16(s[:, g][None, :], vc, C)
    return bf16_round(C.astype(np.float32))


def woq_linear_opt_bf16(x, act_dtype, qw, N, K, scales, zps, bias, weight_dtype, group_size):
    """The M >= 5 path: scales / zero points read as bf16, w = bf16((q - z) * s) with the
    subtraction and the product each in fp32; bf16 x bf16 products accumulated in fp32 on top of
    the fp32 bias; one rounding to the output dtype.  Returns (acc, y)."""
    s = bf16_round(np.asarray(scales, dtype=np.float32))
    z = None if zps is None else bf16_round(np.asarray(zps, dtype=np.float32))
    w = bf16_round(dequantize_woq_weight(qw, N, K, s, z, weight_dtype, group_size))
    xb = bf16_round(x)
    acc = xb.astype(np.float64) @ w.astype(np.float64).T
    if bias is not None:
        acc = acc + np.asarray(bias, dtype=np.float32).astype(np.float64)[None, :]
    return acc, _round_to(acc.astype(np.float32), act_dtype)


def dynamic_quantize_per_block(x, quant_block_k, mode):
    """x: float32 [M, K] holding the activation values.  Modes 0..3 asymmetric (uint8 + zero
    point), 4..7 symmetric (int8): per tensor, per K block, per row, per row x K block.
    scale = max(|max|, |min|) / 127 or (max - min) / 255 in fp32; q = clamp(rint(x / scale + zp))
    with an IEEE fp32 division and round-half-even.  Returns (q, scales, zps)."""
    x = np.asarray(x, dtype=np.float32)
    M, K = x.shape
    sym = mode >= 4
    per_m = mode in (2, 3, 6, 7)
    per_k = mode in (1, 3, 5, 7)
    qbk = quant_block_k if (per_k and quant_block_k > 0) else K
    Kc = (K + qbk - 1) // qbk
    Mg = M if per_m else 1
    scales = np.zeros((Mg, Kc), dtype=np.float32)
    zps = np.zeros((Mg, Kc), dtype=np.int32)
    q = np.zeros((M, K), dtype=np.int8 if sym else np.uint8)
    for mg in range(Mg):
        rows = slice(mg, mg + 1) if per_m else slice(0, M)
        for kc in range(Kc):
            cols = slice(kc * qbk, min((kc + 1) * qbk, K))
            blk = x[rows, cols]
            mn, mx = np.float32(blk.min()), np.float32(blk.max())
            if sym:
                s = np.float32(max(abs(mx), abs(mn))) / np.float32(127.0)
                zp = np.float32(0)
                lo, hi = -128.0, 127.0
            else:
                s = np.float32(mx - mn) / np.float32(255.0)
                with np.errstate(divide="ignore", invalid="ignore"):
                    zp = np.float32(-np.rint(mn / s))
                zps[mg, kc] = np.int32(zp) if np.isfinite(zp) else 0
                lo, hi = 0.0, 255.0
            scales[mg, kc] = s
            with np.errstate(divide="ignore", invalid="ignore"):
                t = (blk / np.float32(s)).astype(np.float32) + zp
            t = np.clip(np.rint(t), lo, hi)
            # an all-zero block gives 0 / 0 in the reference; the product with its zero scale
            # is 0 whatever q holds, so q is pinned to the zero point here
            t = np.where(np.isnan(t), zp if np.isfinite(zp) else 0, t)
            q[rows, cols] = t.astype(q.dtype)
    shape = ([M] if per_m else []) + ([Kc] if per_k else [])
    scales = scales.reshape(shape if shape else [1])
    zps = zps.reshape(shape if shape else [1])
    return q, scales, (None if sym else zps)


# NF4 codes as int8 for the lowp-INT8 kernels: round(127 * table) (the lookup table of
# load_nf4_as_int8, csrc/cpu/aten/utils/woq.h:628-669); the weight scale is multiplied by
# fp32(1 / 127) to make up for it (woq.h:1006-1009, 2174-2176).
NF4_TO_INT8_TABLE = np.array([-127, -88, -67, -50, -36, -23, -12, 0, 10, 20, 31, 43, 56, 71, 92, 127], dtype=np.int64)


def _int8_weights(qw, N, K, zps, weight_dtype, group_size):
    """B[n, k] = q - z as integers (the int8 operand of the lowp-INT8 kernels, woq.h:1701-1704,
    614-625); NF4: the int8 table value of the code."""
    if weight_dtype == WOQ_DTYPE_NF4:
        assert zps is None, "NF4 is symmetric"
        return NF4_TO_INT8_TABLE[unpack_int4(qw)[:, :K]]
    if weight_dtype == WOQ_DTYPE_INT4:
        q = unpack_int4(qw)[:, :K].astype(np.int64)
        if zps is None:
            return q - 8
        z = np.asarray(zps).reshape(N, -1).astype(np.int64)
        g = (np.arange(K) // group_size) if group_size > 0 else np.zeros(K, dtype=np.int64)
        return q - z[:, g]
    return np.asarray(qw, dtype=np.int8).astype(np.int64)


def int8_weight_block_sums(qw, N, K, zps, weight_dtype, group_size, block_k):
    """compensation[n, kb] = sum_{k in block kb} (q[n, k] - z[n, g(k)]) (woq.h:1679-1727)."""
    B = _int8_weights(qw, N, K, zps, weight_dtype, group_size)
    KB = K // block_k
    return B[:, : KB * block_k].reshape(N, KB, block_k).sum(axis=2).astype(np.int32)


def int8_block_sums(xq, qw, N, K, zps, weight_dtype, group_size, block_k):
    """Exact int32 sums qC[m, n, kb] = sum_{k in block kb} xq[m, k] * (q[n, k] - z[n, g(k)])."""
    B = _int8_weights(qw, N, K, zps, weight_dtype, group_size)
    A = np.asarray(xq).astype(np.int64)
    KB = K // block_k
    out = np.empty((A.shape[0], N, KB), dtype=np.int64)
    for kb in range(KB):
        sl = slice(kb * block_k, (kb + 1) * block_k)
        out[:, :, kb] = A[:, sl] @ B[:, sl].T
    assert np.abs(out).max() < 2**31
    return out.astype(np.int32)


def woq_linear_opt_int8(x, act_dtype, qw, N, K, scales, zps, bias, weight_dtype, group_size, act_quant_mode):
    """lowp_mode INT8.  C = fp32 bias or 0; for each K block kb ascending:
    C += (float(qC[kb]) * s_a) * s_w[n, g(kb)] for the symmetric activation modes 4..7, and
    C += (float(qC[kb] - compensation[n, kb] * zp_a) * s_a) * s_w[n, g(kb)] for the asymmetric
    modes 0..3 (integer subtraction first, woq.h:2172-2186).  Returns dict(xq, sa, za, sums, ints
    (the integer that is converted to fp32 per block: sums, minus the compensation term for the
    asymmetric modes), acc (fp32), y)."""
    M = x.shape[0]
    asym = act_quant_mode < 4
    bk = int8_block_k(group_size, K)
    qbk = group_size if group_size > 0 else bk
    xq, sa, za = dynamic_quantize_per_block(x, qbk, act_quant_mode)
    sums = int8_block_sums(xq, qw, N, K, zps, weight_dtype, group_size, bk)
    s = np.asarray(scales, dtype=np.float32).reshape(N, -1)
    if weight_dtype == WOQ_DTYPE_NF4:
        s = (s * (np.float32(1.0) / np.float32(127.0))).astype(np.float32)
    per_m = act_quant_mode in (2, 3, 6, 7)
    per_k = act_quant_mode in (1, 3, 5, 7)
    Kc = (K + qbk - 1) // qbk
    sa2 = np.asarray(sa, dtype=np.float32).reshape(M if per_m else 1, Kc if per_k else 1)
    if asym:
        comp = int8_weight_block_sums(qw, N, K, zps, weight_dtype, group_size, bk).astype(np.int64)
        za2 = np.asarray(za, dtype=np.int64).reshape(M if per_m else 1, Kc if per_k else 1)
    C = np.zeros((M, N), dtype=np.float32)
    if bias is not None:
        C[:] = np.asarray(bias, dtype=np.float32)[None, :]
    ints = sums if not asym else np.empty_like(sums)
    for kb in range(K // bk):
        g = (kb * bk) // group_size if group_size > 0 else 0
        kc = (kb * bk) // qbk if per_k else 0
        sa_col = sa2[:, kc].reshape(-1, 1)
        qv = sums[:, :, kb].astype(np.int64)
        if asym:
            qv = qv - comp[:, kb][None, :] * za2[:, kc].reshape(-1, 1)
            assert np.abs(qv).max() < 2**31
            ints[:, :, kb] = qv
        c = (qv.astype(np.float32) * sa_col).astype(np.float32)
        c = (c * s[:, g][None, :]).astype(np.float32)
        C = (C + c).astype(np.float32)
    return {"xq": xq, "sa": sa, "za": za, "sums": sums, "ints": ints, "acc": C, "y": _round_to(C, act_dtype)}


def woq_linear(x, act_dtype, qw, N, K, scales, zps, bias, weight_dtype, group_size, lowp_mode, act_quant_mode=-1,
               numerics="opt"):
    """Dispatch as the reference does.  numerics 'ref' = fallback implementation,
    'opt' = optimized kernels.  Returns (acc or None, y)."""
    M = x.shape[0]
    cd = select_compute(lowp_mode, act_dtype, M)
    if numerics == "ref":
        if cd == "int8":
            cd = act_dtype  # the fallback does not quantize activations
        return woq_linear_ref(x, act_dtype, qw, N, K, scales, zps, bias, weight_dtype, group_size, cd)
    if cd == "fp16":
        return None, woq_linear_opt_fp16(x, qw, N, K, scales, zps, bias, weight_dtype, group_size)
    if cd == "bf16":
        return woq_linear_opt_bf16(x, act_dtype, qw, N, K, scales, zps, bias, weight_dtype, group_size)
    if cd == "int8":
        r = woq_linear_opt_int8(x, act_dtype, qw, N, K, scales, zps, bias, weight_dtype, group_size, act_quant_mode)
        return r["acc"], r["y"]
    raise NotImplementedError(cd)


# ---------------------------------------------------------------------------------------------
# mixture of experts around the WOQ linears
# ---------------------------------------------------------------------------------------------
def expert_token_lists(topk_ids, num_experts):
    """Per expert: (tokens routed to it, their slot in the top-k), tokens ascending, slots ascending
    inside a token -- the order get_expert_topx_idx builds by walking topk_ids row by row."""
    ids = np.asarray(topk_ids)
    top_x = [[] for _ in range(num_experts)]
    idx = [[] for _ in range(num_experts)]
    for i in range(ids.shape[0]):
        for j in range(ids.shape[1]):
            top_x[int(ids[i, j])].append(i)
            idx[int(ids[i, j])].append(j)
    return [np.asarray(t, dtype=np.int64) for t in top_x], [np.asarray(t, dtype=np.int64) for t in idx]


def moe_index_mul_index_add(output, cur, routing_weights, top_x, idx, dtype):
    """output[top_x[i], :] += routing_weights[top_x[i], idx[i]] * cur[i, :], sequentially in i.
    All arrays float32 holding `dtype` values.  bf16 / fp32: product and sum in fp32, one rounding
    to dtype; fp16: the product is rounded to fp16 before the add."""
    out = np.array(output, dtype=np.float32, copy=True)
    cur = np.asarray(cur, dtype=np.float32)
    rw = np.asarray(routing_weights, dtype=np.float32)
    for i in range(len(top_x)):
        t = int(top_x[i])
        p = (cur[i] * rw[t, int(idx[i])]).astype(np.float32)
        if dtype == "fp16":
            p = f16_round(p)
        out[t] = _round_to((out[t] + p).astype(np.float32), dtype)
    return out
