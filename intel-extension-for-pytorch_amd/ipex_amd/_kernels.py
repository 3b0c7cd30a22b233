"""Tensor-level wrappers over the C ABI: every function takes CUDA (HIP) tensors, passes
their device pointers and the current torch stream to libwoq_hip.so and returns tensors.
PyTorch is used for device memory and stream plumbing only.
"""
import ctypes

import torch

from . import _lib

_ACT_CODE = {torch.float32: _lib.ACT_FP32, torch.float16: _lib.ACT_FP16, torch.bfloat16: _lib.ACT_BF16}


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _require_cuda(t, name):
    if not t.is_cuda:
        raise RuntimeError(
            f"{name} must live on the GPU (got device {t.device}); this build runs the WOQ linear "
            "on MI355X only and has no CPU path"
        )


def padded_n(N):
    return _lib.load().woq_hip_padded_n(N)


def padded_k(weight_dtype, K):
    return _lib.load().woq_hip_padded_k(weight_dtype, K)


def pack_weight(plain, weight_dtype, N, K):
    """Plain [N, ceil(K/2)] uint8 (4-bit), [N, K] int8, or [N, K] float8_e4m3fn / uint8 bytes (FP8) -> packed tiles
    [NT, KT, 1024] uint8."""
    lib = _lib.load()
    _require_cuda(plain, "qweight")
    plain = plain.contiguous()
    if weight_dtype == _lib.DTYPE_FP8 and plain.dtype != torch.uint8:
        plain = plain.view(torch.uint8)
    tk = _lib.TILE_K_INT8 if weight_dtype in _lib.DTYPES_8BIT else _lib.TILE_K_INT4
    nt, kt = padded_n(N) // _lib.TILE_N, padded_k(weight_dtype, K) // tk
    packed = torch.empty((nt, kt, _lib.TILE_BYTES), dtype=torch.uint8, device=plain.device)
    with torch.cuda.device(plain.device):
        _lib.check(lib.woq_hip_pack_weight(_ptr(plain), weight_dtype, N, K, _ptr(packed), _stream()), "pack_weight")
    return packed


def unpack_weight(packed, weight_dtype, N, K):
    lib = _lib.load()
    _require_cuda(packed, "packed weight")
    if weight_dtype == _lib.DTYPE_FP8:
        plain = torch.empty((N, K), dtype=torch.float8_e4m3fn, device=packed.device)
    elif weight_dtype == _lib.DTYPE_INT8:
        plain = torch.empty((N, K), dtype=torch.int8, device=packed.device)
    else:
        plain = torch.empty((N, (K + 1) // 2), dtype=torch.uint8, device=packed.device)
    with torch.cuda.device(packed.device):
        _lib.check(
            lib.woq_hip_unpack_weight(_ptr(packed), weight_dtype, N, K, _ptr(plain), _stream()), "unpack_weight"
        )
    return plain


def pack_qparams(scales, zeros, weight_dtype):
    """scales / zeros: fp32 [N, KG] -> ([NT, KG, 16] fp32, fp16, bf16, uint8-or-None, packed
    (fp16 scale, fp16 128 + zero) dwords-or-None, packed (bf16 scale, fp16 zero code) dwords-or-None: the
    last for INT4 and INT8 weights, which the bf16 kernels then read with one load per (row, group))."""
    lib = _lib.load()
    _require_cuda(scales, "scales")
    scales = scales.to(torch.float32).contiguous()
    N, KG = scales.shape
    nt = padded_n(N) // _lib.TILE_N
    dev = scales.device
    s32 = torch.empty((nt, KG, _lib.TILE_N), dtype=torch.float32, device=dev)
    s16 = torch.empty((nt, KG, _lib.TILE_N), dtype=torch.float16, device=dev)
    sb16 = torch.empty((nt, KG, _lib.TILE_N), dtype=torch.bfloat16, device=dev)
    z8 = None
    if zeros is not None:
        zeros = zeros.to(torch.float32).contiguous()
        assert zeros.shape == scales.shape
        z8 = torch.empty((nt, KG, _lib.TILE_N), dtype=torch.uint8, device=dev)
    sz = None
    if weight_dtype not in _lib.DTYPES_8BIT:
        sz = torch.empty((nt, KG, _lib.TILE_N), dtype=torch.int32, device=dev)
    szb = None
    if weight_dtype in (_lib.DTYPE_INT4, _lib.DTYPE_INT8):
        szb = torch.empty((nt, KG, _lib.TILE_N), dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        _lib.check(
            lib.woq_hip_pack_qparams(
                _ptr(scales), _ptr(zeros), weight_dtype, N, KG, _ptr(s32), _ptr(s16), _ptr(sb16), _ptr(z8), _ptr(sz),
                _ptr(szb), _stream()
            ),
            "pack_qparams",
        )
    return s32, s16, sb16, z8, sz, szb


def dense_weight(qweight, weight_dtype, N, K, scales_bf16, zeros_u8, group_size):
    """Dense bf16 copy of a packed weight in the operand layout of the dense kernel
    ([K / 128, padded N / 16, 4, 64, 8] bf16), or None where none can be made (K % 128 != 0)."""
    lib = _lib.load()
    _require_cuda(qweight, "weight")
    nbytes = lib.woq_hip_dense_weight_bytes(weight_dtype, N, K)
    if nbytes == 0:
        return None
    nt = padded_n(N) // _lib.TILE_N
    out = torch.empty((K // 128, nt, 4, 64, 8), dtype=torch.bfloat16, device=qweight.device)
    assert out.numel() * 2 == nbytes
    with torch.cuda.device(qweight.device):
        _lib.check(
            lib.woq_hip_dense_weight(
                _ptr(qweight), weight_dtype, N, K, _ptr(scales_bf16), _ptr(zeros_u8), group_size, _ptr(out), _stream()
            ),
            "dense_weight",
        )
    return out


def unpack_int4_zeros(zp32, cols):
    """int32-compressed zero points [rows, ceil(cols/8)] -> fp32 [rows, cols]."""
    lib = _lib.load()
    _require_cuda(zp32, "zero points")
    zp32 = zp32.contiguous()
    rows, cols_zp = zp32.shape
    out = torch.empty((rows, cols), dtype=torch.float32, device=zp32.device)
    with torch.cuda.device(zp32.device):
        _lib.check(lib.woq_hip_unpack_int4_zeros(_ptr(zp32), rows, cols, cols_zp, _ptr(out), _stream()), "unpack_int4_zeros")
    return out


def dynamic_quant(x, quant_block_k, act_quant_mode):
    """Returns (q, scales, zps) as dynamic_quantize_per_block does; zps is None for symmetric modes."""
    lib = _lib.load()
    _require_cuda(x, "x")
    K = x.shape[-1]
    x2 = x.reshape(-1, K).contiguous()
    M = x2.shape[0]
    sym = act_quant_mode >= 4
    per_m = act_quant_mode in (2, 3, 6, 7)
    per_k = act_quant_mode in (1, 3, 5, 7)
    qbk = quant_block_k if quant_block_k > 0 else K
    Kc = (K + qbk - 1) // qbk
    shape = []
    if per_m:
        shape.append(M)
    if per_k:
        shape.append(Kc)
    if not shape:
        shape = [1]
    q = torch.empty((M, K), dtype=torch.int8 if sym else torch.uint8, device=x.device)
    scales = torch.empty(shape, dtype=torch.float32, device=x.device)
    zps = None if sym else torch.empty(shape, dtype=torch.int32, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(
            lib.woq_hip_dynamic_quant(
                _ptr(x2), _ACT_CODE[x.dtype], M, K, qbk, act_quant_mode, _ptr(q), _ptr(scales), _ptr(zps), _stream()
            ),
            "dynamic_quant",
        )
    return q, scales, zps


def int8_block_k(group_size, K):
    return _lib.load().woq_hip_int8_block_k(group_size, K)


_counter_cache = {}


def _split_k_counters(device):
    """The zeroed counter array the split-K decode kernel needs, one per (device, stream): launches
    on one stream run in order and every launch leaves the counters at zero.  None while a HIP graph
    is being captured on a stream that has no array yet (an allocation made during capture belongs to
    the graph's memory pool and must not outlive it): the call then runs without splitting K."""
    with torch.cuda.device(device):
        key = (torch.cuda.current_device(), torch.cuda.current_stream().cuda_stream)
        buf = _counter_cache.get(key)
        if buf is None:
            if torch.cuda.is_current_stream_capturing():
                return None
            buf = torch.zeros(512, dtype=torch.int32, device=device)
            _counter_cache[key] = buf
    return buf


def linear(
    x,
    qweight,
    weight_dtype,
    N,
    K,
    scales_f32,
    scales_f16,
    scales_bf16,
    zeros_u8,
    group_size,
    bias_f32,
    lowp_mode,
    act_quant_mode,
    scale_zero_f16x2=None,
    fusion=_lib.FUSE_NONE,
    others=(),
    out_fp32=False,
    force_kernel=0,
    debug_block_sums=False,
    noalloc=False,
    out_dtype=None,
    scale_zero_bf16=None,
    dense_bf16=None,
):
    """y = x @ dequant(W)^T (+ bias, post-op).  x: [..., K]; returns [..., N] in x.dtype, or the
    fp32 accumulator when ``out_fp32``.  With ``debug_block_sums`` also returns the int32 sum of
    every (m, n, K block) of the int8 path.  ``noalloc``: through ``woq_hip_linear_noalloc``, which
    takes no workspace (the output tensor is still made here).  ``out_dtype``: without a post-op, the other
    16-bit type than x's (fp16 rows converted from a bf16 tensor, bf16 output)."""
    lib = _lib.load()
    _require_cuda(x, "input")
    if x.dtype not in _ACT_CODE:
        raise RuntimeError(f"woq_linear: unsupported activation dtype {x.dtype}")
    if x.shape[-1] != K:
        raise RuntimeError(
            f"WOQ linear: input and weight shapes do not match, got k = {x.shape[-1]} and {K} respectively."
        )
    x2 = x.reshape(-1, K).contiguous()
    if x2.data_ptr() % 16:
        x2 = x2.clone()  # the kernels read activation rows with 16-byte loads
    M = x2.shape[0]
    out_dtype = torch.float32 if out_fp32 else (out_dtype or x.dtype)
    out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    p = _lib.LinearParams()
    p.struct_size = ctypes.sizeof(_lib.LinearParams)
    p.x = x2.data_ptr()
    p.x_dtype = _ACT_CODE[x.dtype]
    p.M, p.K, p.N = M, K, N
    p.qweight = qweight.data_ptr()
    p.weight_dtype = weight_dtype
    p.scales_f32 = scales_f32.data_ptr()
    p.scales_f16 = scales_f16.data_ptr()
    p.scales_bf16 = scales_bf16.data_ptr()
    p.zeros_u8 = zeros_u8.data_ptr() if zeros_u8 is not None else None
    p.scale_zero_f16x2 = scale_zero_f16x2.data_ptr() if scale_zero_f16x2 is not None else None
    p.scale_zero_bf16 = scale_zero_bf16.data_ptr() if scale_zero_bf16 is not None else None
    p.dense_bf16 = dense_bf16.data_ptr() if dense_bf16 is not None else None
    p.group_size = group_size
    p.bias = bias_f32.data_ptr() if bias_f32 is not None else None
    p.lowp_mode = lowp_mode
    p.act_quant_mode = act_quant_mode
    p.fusion = fusion
    keep = []
    for i, o in enumerate(others):
        o2 = o.reshape(-1, N)
        if o2.shape[0] != M:
            raise RuntimeError("woq_linear: post-op operand must have the output's shape")
        o2 = o2.to(x.dtype).contiguous()
        keep.append(o2)
        p.others[i] = o2.data_ptr()
    p.out = out.data_ptr()
    p.out_dtype = _ACT_CODE[out_dtype]
    ws = None
    wbytes = 0 if noalloc else lib.woq_hip_linear_workspace_bytes(M, K, lowp_mode, act_quant_mode, group_size)
    counters = None
    if wbytes > 0 and lowp_mode == 3 and M > 64:
        # lowp INT8 at prefill sizes: room behind the quantized activations lets the int8 GEMM share a
        # long K between the workgroups of its few tiles
        extra = lib.woq_hip_linear_split_k_workspace_bytes(M, N)
        counters = _split_k_counters(x.device) if extra > 0 else None
        if counters is not None:
            p.split_k_counters = counters.data_ptr()
            wbytes = (wbytes + 255) // 256 * 256 + extra
    if wbytes == 0 and lowp_mode != 3 and not noalloc:
        # scratch that lets the decode kernel split K across workgroups (small M, few output columns)
        wbytes = lib.woq_hip_linear_split_k_workspace_bytes(M, N)
        counters = _split_k_counters(x.device) if wbytes > 0 else None
        if counters is not None:
            p.split_k_counters = counters.data_ptr()
        else:
            wbytes = 0
    if wbytes > 0:
        ws = torch.empty((wbytes,), dtype=torch.uint8, device=x.device)
        p.workspace = ws.data_ptr()
        p.workspace_bytes = wbytes
    sums = None
    if debug_block_sums:
        bk = lib.woq_hip_int8_block_k(group_size, K)
        kp = padded_k(weight_dtype, K)
        sums = torch.zeros((M, N, kp // bk), dtype=torch.int32, device=x.device)
        p.debug_block_sums = sums.data_ptr()
    p.force_kernel = force_kernel
    with torch.cuda.device(x.device):
        p.stream = torch.cuda.current_stream().cuda_stream
        entry = lib.woq_hip_linear_noalloc if noalloc else lib.woq_hip_linear
        _lib.check(entry(ctypes.byref(p)), "woq_linear")
    out = out.reshape(*x.shape[:-1], N)
    if debug_block_sums:
        return out, sums
    return out


def dequant_weight(qweight, weight_dtype, N, K, scales_f32, zeros_u8, group_size, dtype=torch.float32):
    lib = _lib.load()
    out = torch.empty((N, K), dtype=dtype, device=qweight.device)
    with torch.cuda.device(qweight.device):
        _lib.check(
            lib.woq_hip_dequant_weight(
                _ptr(qweight), weight_dtype, N, K, _ptr(scales_f32), _ptr(zeros_u8), group_size, _ptr(out),
                _ACT_CODE[dtype], _stream()
            ),
            "dequant_weight",
        )
    return out


def convert_activations(x, dtype):
    """x converted to ``dtype`` (round to nearest even) by the library's own kernel."""
    lib = _lib.load()
    _require_cuda(x, "input")
    if x.dtype not in _ACT_CODE or dtype not in _ACT_CODE:
        raise RuntimeError(f"convert_activations: unsupported dtype {x.dtype} -> {dtype}")
    x2 = x.contiguous()
    out = torch.empty(x2.shape, dtype=dtype, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(
            lib.woq_hip_convert_activations(_ptr(x2), _ACT_CODE[x.dtype], _ptr(out), _ACT_CODE[dtype], x2.numel(), _stream()),
            "convert_activations",
        )
    return out


def shuffle_activations(x, src):
    """out[..., p] = x[..., src[p]] (GPTQ act-order: channels sorted by group)."""
    lib = _lib.load()
    _require_cuda(x, "input")
    if x.dtype not in _ACT_CODE:
        raise RuntimeError(f"shuffle_activations: unsupported dtype {x.dtype}")
    K = x.shape[-1]
    x2 = x.reshape(-1, K).contiguous()
    out = torch.empty_like(x2)
    with torch.cuda.device(x.device):
        _lib.check(
            lib.woq_hip_shuffle_activations(_ptr(x2), _ACT_CODE[x.dtype], x2.shape[0], K, _ptr(src), _ptr(out), _stream()),
            "shuffle_activations",
        )
    return out.reshape(x.shape)


def shuffle_int4_weight(plain, N, K, src):
    """Plain int4 rows [N, (K + 1) // 2] with nibble p taken from nibble src[p]."""
    lib = _lib.load()
    _require_cuda(plain, "weight")
    plain = plain.contiguous()
    out = torch.empty_like(plain)
    with torch.cuda.device(plain.device):
        _lib.check(lib.woq_hip_shuffle_int4_weight(_ptr(plain), N, K, _ptr(src), _ptr(out), _stream()), "shuffle_int4_weight")
    return out


def moe_gather_rows(x, rows):
    """out[i, :] = x[rows[i], :]; x [T, H] on the GPU, rows int64 on the same device."""
    lib = _lib.load()
    _require_cuda(x, "hidden_states")
    _require_cuda(rows, "top_x")
    if x.dtype not in _ACT_CODE or x.dim() != 2:
        raise RuntimeError(f"moe_gather_rows: expected a 2-D bf16 / fp16 / fp32 tensor, got {x.dtype} {tuple(x.shape)}")
    x = x.contiguous()
    rows = rows.to(torch.int64).contiguous()
    out = torch.empty((rows.numel(), x.shape[1]), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(
            lib.woq_hip_moe_gather_rows(_ptr(x), _ACT_CODE[x.dtype], x.shape[0], x.shape[1], _ptr(rows), rows.numel(),
                                        _ptr(out), _stream()),
            "moe_gather_rows",
        )
    return out


def moe_scale_add_rows(output, expert_out, routing_weights, top_x, idx):
    """output[top_x[i], :] += routing_weights[top_x[i], idx[i]] * expert_out[i, :], in place."""
    lib = _lib.load()
    for t, name in ((output, "output"), (expert_out, "expert output"), (routing_weights, "routing_weights"),
                    (top_x, "top_x"), (idx, "idx")):
        _require_cuda(t, name)
    if output.dtype not in _ACT_CODE or expert_out.dtype != output.dtype or routing_weights.dtype != output.dtype:
        raise RuntimeError("moe_scale_add_rows: output, expert output and routing_weights must share one float dtype")
    if not output.is_contiguous() or output.dim() != 2:
        raise RuntimeError("moe_scale_add_rows: output must be a contiguous [tokens, hidden] tensor")
    n, H = top_x.numel(), output.shape[1]
    expert_out = expert_out.reshape(-1, H).contiguous()
    if expert_out.shape[0] != n or idx.numel() != n or routing_weights.dim() != 2 or routing_weights.shape[0] != output.shape[0]:
        raise RuntimeError("moe_scale_add_rows: shape mismatch between top_x / idx / expert output / routing_weights")
    routing_weights = routing_weights.contiguous()
    top_x = top_x.to(torch.int64).contiguous()
    idx = idx.to(torch.int64).contiguous()
    with torch.cuda.device(output.device):
        _lib.check(
            lib.woq_hip_moe_scale_add_rows(_ptr(output), _ACT_CODE[output.dtype], output.shape[0], H, _ptr(expert_out),
                                           _ptr(routing_weights), routing_weights.shape[1], _ptr(top_x), _ptr(idx), n,
                                           _stream()),
            "moe_scale_add_rows",
        )
    return output
