"""Operator boundary: the ``torch_ipex`` / ``ipex_prepack`` ops and the prepack context.

The operators and the TorchScript custom class ``torch.classes.ipex_prepack.WoqLinearOpContext`` are
registered by the C++ binding (csrc/torch_binding.cpp -> lib/libwoq_torch.so), loaded by ``register()``:
same op names, argument order and error behaviour as the reference
(csrc/cpu/aten/Linear.cpp:1013-1112, csrc/cpu/jit/cpu/kernels/RegisterOpContextClass.cpp:127-223),
for tensors that live on the GPU:

    torch.ops.torch_ipex.ipex_woq_linear(x, ctx.get_data_handle())
    torch.ops.torch_ipex.woq_linear_{gelu,new_gelu,relu,silu}(x, handle)
    torch.ops.torch_ipex.woq_linear_{add,add_add,mul}(x, handle, others)
    torch.ops.torch_ipex.woq_linear(x, packed_w, "int4", [N, K], scales, zeros, bias, g_idx, G, lowp, aq, comp)
    torch.ops.ipex_prepack.weight_only_qlinear_prepack(...)      -> WoqLinearOpContext
    torch.ops.ipex_prepack.weight_only_qlinear_prepack_int4(...) -> WoqLinearOpContext
    torch.ops.ipex_prepack.woq_linear_pack_weight(...) / woq_linear_unpack_weight(...)

This module adds the mixture-of-experts ops on top of them, and keeps ``WoqLinearOpContext``, a
Python twin of the custom class over the same C ABI through ctypes: the vehicle of the C-ABI tests
(``run`` takes the library's debugging options: fp32 accumulators, forced kernels, block sums).  Its
handles name Python objects and are understood by the functions of this module only, not by
``torch.ops``.
"""
import contextlib
import ctypes
import os
import threading
import weakref
from typing import List, Optional

import torch

from . import _kernels, _lib

_NO_GUARD = contextlib.nullcontext()
_current_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None) or (
    lambda index: torch.cuda.current_stream(index).cuda_stream
)
_current_device = getattr(torch._C, "_cuda_getDevice", None) or torch.cuda.current_device

WOQ_DTYPE_MAP = {"int8": _lib.DTYPE_INT8, "int4": _lib.DTYPE_INT4, "nf4": _lib.DTYPE_NF4, "fp8": _lib.DTYPE_FP8}
PLAIN_WEIGHT_FORMAT, GPTQ_WEIGHT_FORMAT, AWQ_WEIGHT_FORMAT = 0, 1, 2

_contexts = {}
_contexts_lock = threading.Lock()
# Bumped whenever a context of this module changes or frees its device arrays (load_from_ctx, destruction): whoever
# caches device addresses of contexts (the grouped mixture-of-experts plans) compares it before every use.
_context_epoch = [0]
# Handles of this ctypes twin are negative, those of the registered custom class (torch_binding.cpp) positive:
# a handle of one kind given to an operator of the other kind raises instead of naming some live context there.
_next_handle = [-1]


def _to_gpu(t, device=None):
    if t is None:
        return None
    if t.is_cuda:
        return t
    if not torch.cuda.is_available():
        raise RuntimeError(
            "WOQ linear: no GPU is available; this build runs on MI355X only and has no CPU path"
        )
    return t.to(device if device is not None else torch.device("cuda", torch.cuda.current_device()))


def _check_integral_zeros(zeros, weight_dtype):
    lo, hi = (-128, 127) if weight_dtype == _lib.DTYPE_INT8 else (0, 127)
    z = zeros.to(torch.float32)
    ok = torch.equal(z, z.round()) and bool((z >= lo).all()) and bool((z <= hi).all())
    if not ok:
        raise RuntimeError(
            f"WOQ linear: zero points must be integers in [{lo}, {hi}] for this weight dtype"
        )


class WoqLinearOpContext:
    """Prepacked weight + quantization parameters of one linear layer
    (ContextLinearWoq / IpexWoqLinearOpContext of the reference,
    csrc/cpu/jit/cpu/kernels/ContextLinearWoq.h:12-139, OpContext.cpp:364-507).

    ``weight`` is the plain checkpoint format: uint8 [N, ceil(K/2)] for 4-bit, int8 [N, K] for
    8-bit weights.
    """

    def __init__(
        self,
        weight,
        weight_dtype,
        weight_shape,
        scales,
        zero_points=None,
        bias=None,
        g_idx=None,
        batch_size=None,
        group_size=-1,
        lowp_mode=0,
        act_quant_mode=0,
        cache_weight_for_large_batch=False,
    ):
        weight_dtype = int(weight_dtype)
        if weight_dtype not in (_lib.DTYPE_INT8, _lib.DTYPE_INT4, _lib.DTYPE_NF4, _lib.DTYPE_FP8):
            raise RuntimeError(f"WOQ linear: unsupported weight dtype {weight_dtype}")
        if weight_dtype == _lib.DTYPE_NF4 and zero_points is not None:
            raise RuntimeError("WOQ: symmetric quantization is required for NF4 or INT8 with lowp-mode INT8")
        if weight_dtype == _lib.DTYPE_FP8 and zero_points is not None:
            raise RuntimeError("WOQ: FP8 weights take no zero points")
        if weight_dtype == _lib.DTYPE_FP8 and int(lowp_mode) == _lib.LOWP_INT8:
            raise RuntimeError("WOQ: lowp-mode INT8 does not take FP8 weights")
        N, K = int(weight_shape[0]), int(weight_shape[1])
        weight = _to_gpu(weight)
        dev = weight.device
        if weight_dtype == _lib.DTYPE_FP8:
            # float8 e4m3fn values, or their bytes
            if weight.dtype not in (torch.float8_e4m3fn, torch.uint8) or tuple(weight.shape) != (N, K):
                raise RuntimeError(f"WOQ linear: fp8 weight must be float8_e4m3fn [{N}, {K}]")
            weight = weight.view(torch.uint8)
        elif weight_dtype != _lib.DTYPE_INT8:
            weight = weight.view(torch.uint8) if weight.dtype != torch.uint8 else weight
            if tuple(weight.shape) != (N, (K + 1) // 2):
                raise RuntimeError(
                    f"WOQ linear: 4-bit weight has shape {tuple(weight.shape)}, expected {(N, (K + 1) // 2)}"
                )
        else:
            if weight.dtype != torch.int8 or tuple(weight.shape) != (N, K):
                raise RuntimeError(f"WOQ linear: int8 weight must be int8 [{N}, {K}]")
        scales = _to_gpu(scales, dev).to(torch.float32)
        group_size = int(group_size)
        if group_size > 0:
            KG = (K + group_size - 1) // group_size
            scales = scales.reshape(N, -1)
            if scales.shape[1] != KG:
                raise RuntimeError(
                    f"WOQ linear: scales have {scales.shape[1]} groups, expected {KG} for group_size {group_size}"
                )
        else:
            scales = scales.reshape(N, 1)
        if zero_points is not None:
            zero_points = _to_gpu(zero_points, dev).to(torch.float32).reshape(scales.shape)
            _check_integral_zeros(zero_points, weight_dtype)
        if weight_dtype == _lib.DTYPE_INT8 and int(lowp_mode) == _lib.LOWP_INT8 and zero_points is not None:
            raise RuntimeError("WOQ: symmetric quantization is required for NF4 or INT8 with lowp-mode INT8")

        self.weight_dtype_ = weight_dtype
        self.weight_shape_ = [N, K]
        self.group_size_ = group_size
        self.lowp_mode_ = int(lowp_mode)
        self.act_quant_mode_ = int(act_quant_mode)
        self.batch_size_ = batch_size
        self.cache_weight_for_large_batch_ = bool(cache_weight_for_large_batch)
        # GPTQ act-order: input channel k belongs to group g_idx[k].  As the reference does for
        # 4-bit group-wise weights (LinearWoqPacked.cpp:306-316, 407-421), the weight's input channels
        # are sorted by group once here and the activations are shuffled the same way per call.
        self.g_idx_ = None
        self.g_src_ = None  # position -> source channel
        self.g_dst_ = None  # inverse permutation
        if g_idx is not None and weight_dtype == _lib.DTYPE_INT4 and group_size > 0:
            g = _to_gpu(g_idx, dev).to(torch.int64).reshape(-1)
            KG = (K + group_size - 1) // group_size
            if g.numel() != K:
                raise RuntimeError("g_idx size and weight shape mismatch")
            if int(g.min()) < 0 or int(g.max()) >= KG:
                raise RuntimeError(f"WOQ linear: g_idx values must lie in [0, {KG})")
            want = torch.full((KG,), group_size, dtype=torch.int64, device=dev)
            want[-1] = K - (KG - 1) * group_size
            if not torch.equal(torch.bincount(g, minlength=KG), want):
                raise RuntimeError("WOQ linear: g_idx must assign exactly group_size channels to every group")
            src = torch.argsort(g, stable=True)
            self.g_idx_ = g_idx
            self.g_src_ = src.to(torch.int32).contiguous()
            self.g_dst_ = torch.argsort(src).to(torch.int32).contiguous()
            weight = _kernels.shuffle_int4_weight(weight, N, K, self.g_src_)
        self.at_bias_ = _to_gpu(bias, dev)
        self.bias_f32_ = self.at_bias_.to(torch.float32).contiguous() if self.at_bias_ is not None else None
        self.at_weight_ = _kernels.pack_weight(weight, weight_dtype, N, K)
        s32, s16, sb16, z8, sz, szb = _kernels.pack_qparams(scales, zero_points, weight_dtype)
        self.scales_list_ = [s32, s16, sb16]
        self.zeros_u8_ = z8
        self.scale_zero_f16x2_ = sz
        self.scale_zero_bf16_ = szb
        # cache_weight_for_large_batch under lowp_mode BF16 (LinearWoqPacked.cpp:430-486): the dense bf16 copy, made
        # at prepack time so that a forward call mutates nothing; None where the flag is off or K % 128 != 0
        self.cached_weight_ = None
        if self.cache_weight_for_large_batch_ and self.lowp_mode_ == _lib.LOWP_BF16:
            self.cached_weight_ = _kernels.dense_weight(
                self.at_weight_, weight_dtype, N, K, sb16, z8, group_size
            )
        self.scales_plain_ = scales if group_size > 0 else scales.reshape(N)
        self.zero_points_plain_ = (
            None if zero_points is None else (zero_points if group_size > 0 else zero_points.reshape(N))
        )
        self.cached_compensation_ = None
        with _contexts_lock:
            self._handle = _next_handle[0]
            _next_handle[0] -= 1
            _contexts[self._handle] = weakref.ref(self)

    def __del__(self):
        try:
            _context_epoch[0] += 1
            with _contexts_lock:
                _contexts.pop(self._handle, None)
        except Exception:
            pass

    # ---- reference method surface ----
    def get_weight(self):
        if self.weight_dtype_ == _lib.DTYPE_FP8:
            return self.at_weight_.view(torch.float8_e4m3fn)
        return self.at_weight_

    def get_bias(self):
        return self.at_bias_

    def get_scales(self):
        return self.scales_plain_

    def get_zero_points(self):
        return self.zero_points_plain_

    def get_weight_shape(self):
        return list(self.weight_shape_)

    def get_g_idx(self):
        return self.g_idx_

    def get_cached_weight(self):
        """The dequantized bf16 copy of the weight that ``cache_weight_for_large_batch`` asks for under lowp_mode
        BF16 (LinearWoqPacked.cpp:430-486), in the operand layout of the dense kernel; None otherwise."""
        return self.cached_weight_

    def get_cached_compensation(self):
        return self.cached_compensation_

    def pack(self, tensor):
        return tensor

    def to_public(self, tensor):
        """Packed tensor -> plain [N, K/2] (or [N, K]) checkpoint layout."""
        N, K = self.weight_shape_
        plain = _kernels.unpack_weight(tensor, self.weight_dtype_, N, K)
        if self.g_dst_ is not None:  # back to the checkpoint's channel order (LinearWoqPacked.cpp:755-765)
            plain = _kernels.shuffle_int4_weight(plain, N, K, self.g_dst_)
        return plain

    def get_data_handle(self):
        return torch.tensor([self._handle], dtype=torch.int64)

    def load_from_ctx(self, other):
        _context_epoch[0] += 1
        self.__dict__.pop("_tls", None)  # cached parameter blocks point at the old tensors
        self.__dict__.update({k: v for k, v in other.__dict__.items() if k not in ("_handle", "_tls")})

    # ---- pickling: always the plain format, re-prepacked on load (OpContext.h:363-403) ----
    def __getstate__(self):
        cpu = lambda t: None if t is None else t.detach().cpu()
        weight = cpu(self.to_public(self.at_weight_))
        if weight.dtype == torch.float8_e4m3fn:
            # float8 tensors do not pickle with every torch version: the state carries their bytes,
            # which the constructor takes as well
            weight = weight.view(torch.uint8)
        return (
            weight,
            self.weight_dtype_,
            list(self.weight_shape_),
            cpu(self.scales_plain_),
            cpu(self.zero_points_plain_),
            cpu(self.at_bias_),
            cpu(self.g_idx_),
            self.batch_size_,
            self.group_size_,
            self.lowp_mode_,
            self.act_quant_mode_,
            self.cache_weight_for_large_batch_,
        )

    def __setstate__(self, state):
        self.__init__(*state)

    # ---- execution ----
    def _run_planned(self, x, M, fusion, others):
        """The common call (no debugging options) through a parameter block that is filled once per
        context and thread: per call only the activation / output pointers, M, the post-op, the
        workspace and the stream change."""
        N, K = self.weight_shape_
        tl = self.__dict__.get("_tls")
        if tl is None:
            tl = self.__dict__.setdefault("_tls", threading.local())
        p = getattr(tl, "plan", None)
        if p is None:
            p = _lib.LinearParams()
            p.struct_size = ctypes.sizeof(_lib.LinearParams)
            p.K, p.N = K, N
            p.qweight = self.at_weight_.data_ptr()
            p.weight_dtype = self.weight_dtype_
            p.scales_f32 = self.scales_list_[0].data_ptr()
            p.scales_f16 = self.scales_list_[1].data_ptr()
            p.scales_bf16 = self.scales_list_[2].data_ptr()
            p.zeros_u8 = self.zeros_u8_.data_ptr() if self.zeros_u8_ is not None else None
            p.scale_zero_f16x2 = self.scale_zero_f16x2_.data_ptr() if self.scale_zero_f16x2_ is not None else None
            p.scale_zero_bf16 = self.scale_zero_bf16_.data_ptr() if self.scale_zero_bf16_ is not None else None
            p.dense_bf16 = self.cached_weight_.data_ptr() if self.cached_weight_ is not None else None
            p.group_size = self.group_size_
            p.bias = self.bias_f32_.data_ptr() if self.bias_f32_ is not None else None
            p.lowp_mode = self.lowp_mode_
            p.act_quant_mode = self.act_quant_mode_
            p.others[0] = p.others[1] = None
            tl.plan = p
            tl.plan_ref = ctypes.byref(p)
            tl.had_others = tl.had_scratch = False
        x2 = x if x.is_contiguous() else x.contiguous()
        if x2.data_ptr() % 16:
            x2 = x2.clone()  # the kernels read activation rows with 16-byte loads
        out = torch.empty((*x.shape[:-1], N), dtype=x.dtype, device=x.device)
        code = _kernels._ACT_CODE[x.dtype]
        p.x, p.x_dtype, p.M = x2.data_ptr(), code, M
        p.out, p.out_dtype = out.data_ptr(), code
        p.fusion = fusion
        keep = []
        if others or tl.had_others:
            for i in range(2):
                if i < len(others):
                    o = others[i]
                    if o.numel() != M * N:
                        raise RuntimeError("woq_linear: post-op operand must have the output's shape")
                    o = o.to(x.dtype).contiguous()
                    keep.append(o)
                    p.others[i] = o.data_ptr()
                else:
                    p.others[i] = None
            tl.had_others = bool(others)
        lib = _lib._lib or _lib.load()
        dev_index = x.device.index
        with _NO_GUARD if dev_index == _current_device() else torch.cuda.device(x.device):
            # the raw handle of the current stream: torch.cuda.current_stream() builds a Stream object
            # around it, 2.8 us of a call whose kernel takes 5-8 us
            p.stream = _current_raw_stream(dev_index)
            ws = counters = None
            wbytes = 0
            int8 = self.lowp_mode_ == _lib.LOWP_INT8
            if int8:  # the quantized activations and their scales
                wbytes = lib.woq_hip_linear_workspace_bytes(M, K, _lib.LOWP_INT8, self.act_quant_mode_, self.group_size_)
            # long K and few output tiles: scratch with which the decode kernel or the prefill GEMMs share K
            # between workgroups, and the zeroed counters of this stream (the library says for which problems)
            extra = lib.woq_hip_linear_auto_split_k_workspace_bytes(M, K, N, self.lowp_mode_)
            if extra > 0:
                counters = _kernels._split_k_counters(x.device)
                if counters is not None:
                    wbytes = (wbytes + 255) // 256 * 256 + extra
            if wbytes > 0:
                ws = torch.empty(wbytes, dtype=torch.uint8, device=x.device)
                p.workspace, p.workspace_bytes = ws.data_ptr(), wbytes
                p.split_k_counters = counters.data_ptr() if counters is not None else None
                tl.had_scratch = True
            elif tl.had_scratch:
                p.workspace, p.workspace_bytes, p.split_k_counters = None, 0, None
                tl.had_scratch = False
            rc = lib.woq_hip_linear(tl.plan_ref)
        if rc:
            _lib.check(rc, "woq_linear")
        return out

    def run(self, x, fusion=_lib.FUSE_NONE, others=(), **kw):
        N, K = self.weight_shape_
        if x.shape[-1] != K:
            raise RuntimeError(
                f"WOQ linear: input and weight shapes do not match, got k = {x.shape[-1]} and {K} respectively."
            )
        M = x.numel() // K if x.numel() > 0 else 0
        if M == 0:
            return x.new_empty(*x.shape[:-1], N)
        if self.g_src_ is not None:
            x = _kernels.shuffle_activations(x, self.g_src_)
        return self._run_sorted(x, M, fusion, others, kw)

    def _run_sorted(self, x, M, fusion, others, kw):
        """``run`` behind the act-order shuffle: the input channels of ``x`` are already in the order of
        the stored weight."""
        N, K = self.weight_shape_
        if (
            self.lowp_mode_ == _lib.LOWP_FP16
            and x.dtype == torch.bfloat16
            and M > 16
            and fusion == _lib.FUSE_NONE
            and not kw
        ):
            # fp16 compute on bf16 activations beyond one row tile: the reference converts the rows to
            # fp16 and casts the fp16 result to bf16 (csrc/cpu/aten/utils/woq.h:3076-3085).  The library
            # converts the rows once and its fp16 kernels write the bf16 output themselves
            # (M = 2048, 4096 -> 14336: 430 us through the converting general kernel otherwise)
            x = _kernels.convert_activations(x, torch.float16)
            kw = {"out_dtype": torch.bfloat16}
        if not kw and x.dtype in _kernels._ACT_CODE and x.is_cuda:
            return self._run_planned(x, M, fusion, others)
        return _kernels.linear(
            x,
            self.at_weight_,
            self.weight_dtype_,
            N,
            K,
            self.scales_list_[0],
            self.scales_list_[1],
            self.scales_list_[2],
            self.zeros_u8_,
            self.group_size_,
            self.bias_f32_,
            self.lowp_mode_,
            self.act_quant_mode_,
            scale_zero_f16x2=self.scale_zero_f16x2_,
            scale_zero_bf16=self.scale_zero_bf16_,
            dense_bf16=self.cached_weight_,
            fusion=fusion,
            others=others,
            **kw,
        )


def _context_from_handle(handle):
    if handle.dtype != torch.int64 or handle.numel() != 1:
        raise RuntimeError("ipex_woq_linear: W_prepack must be the 1-element int64 tensor of get_data_handle()")
    key = handle.item()
    if key > 0:
        raise RuntimeError(
            "ipex_woq_linear: this handle belongs to a torch.classes.ipex_prepack.WoqLinearOpContext; pass it to "
            "torch.ops.torch_ipex.*, not to the ctypes twin in ipex_amd.ops"
        )
    ref = _contexts.get(key)  # a single dict read: atomic under the interpreter lock
    ctx = ref() if ref is not None else None
    if ctx is None:
        raise RuntimeError("ipex_woq_linear: the prepack context behind this handle no longer exists")
    return ctx


# ---- prepack entry points -----------------------------------------------------------------------
def weight_only_qlinear_prepack(
    W,
    W_dtype,
    W_shape,
    scales,
    zero_points,
    B,
    g_idx,
    batch_size,
    group_size,
    lowp_mode,
    act_quant_mode,
    cache_weight_for_large_batch=False,
):
    """createWoqLinearPrePackOpContext (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:20-51)."""
    return WoqLinearOpContext(
        W, W_dtype, list(W_shape), scales, zero_points, B, g_idx, batch_size, group_size, lowp_mode,
        act_quant_mode, cache_weight_for_large_batch,
    )


def weight_only_qlinear_prepack_int4(
    W,
    scales,
    zeros,
    B,
    g_idx,
    batch_size,
    group_size,
    lowp_mode,
    act_quant_mode,
    cache_weight_for_large_batch=False,
    weight_format=PLAIN_WEIGHT_FORMAT,
):
    """INT4 checkpoint ingest (createWoqLinearPrePackOpContextInt4,
    csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:53-202): scales -> fp32, int32-compressed
    zero points -> one value per group, int32 / uint8 weight viewed as bytes, or a float weight
    re-quantized with the given parameters."""
    from .utils.weight_only_quantization import gptq_to_plain, awq_to_plain

    W = _to_gpu(W)
    dev = W.device
    scales_f32 = _to_gpu(scales, dev).squeeze().to(torch.float32)
    zp_f32 = None
    if zeros is not None:
        zeros = _to_gpu(zeros, dev)
        if zeros.dtype == torch.int32 and zeros.numel() != scales_f32.numel():
            if scales_f32.dim() != 2 or zeros.dim() != 2 or scales_f32.size(0) != zeros.size(0):
                raise RuntimeError("IPEX WOQ INT4: unexpected zero points size")
            zp_f32 = _kernels.unpack_int4_zeros(zeros, scales_f32.size(1))
        elif zeros.numel() == scales_f32.numel():
            zp_f32 = zeros.squeeze().to(torch.float32)
        else:
            raise RuntimeError("IPEX WOQ INT4: unexpected zero points size")
    if W.dtype in (torch.int32, torch.uint8):
        if weight_format == GPTQ_WEIGHT_FORMAT:
            plain = gptq_to_plain(W)
        elif weight_format == AWQ_WEIGHT_FORMAT:
            plain = awq_to_plain(W)
        else:
            plain = W.contiguous().view(torch.uint8)
        N, K = plain.shape[0], plain.shape[1] * 2
    elif W.dtype in (torch.bfloat16, torch.float32, torch.float16):
        N, K = W.shape
        w = W.to(torch.float32)
        if group_size > 0:
            wv = w.view(N, K // group_size, group_size)
            q = wv / scales_f32.unsqueeze(2)
            if zp_f32 is not None:
                q = q + zp_f32.unsqueeze(2)
        else:
            q = w / scales_f32.unsqueeze(1)
            if zp_f32 is not None:
                q = q + zp_f32.unsqueeze(1)
        q = torch.round(q).to(torch.uint8).view(N, K)
        plain = (q[:, 1::2] << 4).bitwise_or(q[:, ::2])
    else:
        raise RuntimeError(f"IPEX WOQ INT4: unexpected weight data type: {W.dtype}")
    return WoqLinearOpContext(
        plain, _lib.DTYPE_INT4, [N, K], scales_f32, zp_f32, B, g_idx, batch_size, group_size, lowp_mode,
        act_quant_mode, cache_weight_for_large_batch,
    )


def woq_linear_pack_weight(W, W_dtype, W_shape, scales, zero_points, B, g_idx, group_size, lowp_mode):
    """packWoqLinearWeight (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:212-256): returns
    (packed weight, [scales fp32, fp16, bf16], zeros list or None, bias list or None, compensation)."""
    ctx = WoqLinearOpContext(
        W, WOQ_DTYPE_MAP[W_dtype], list(W_shape), scales, zero_points, B, g_idx, None, group_size, lowp_mode, 0
    )
    zeros = None
    if ctx.zeros_u8_ is not None:
        zf = ctx.zeros_u8_.to(torch.float32)
        if ctx.weight_dtype_ == _lib.DTYPE_INT8:
            zf = zf - 128
        zeros = [zf, zf.to(torch.float16), zf.to(torch.bfloat16), ctx.zeros_u8_]
    bias = None
    if ctx.at_bias_ is not None:
        b = ctx.at_bias_
        bias = [b.to(torch.float32), b.to(torch.float16), b.to(torch.bfloat16)]
    return ctx.at_weight_, list(ctx.scales_list_), zeros, bias, None


def woq_linear_unpack_weight(W, W_dtype, W_shape, lowp_mode):
    """unpackWoqLinearWeight (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:258-275)."""
    return _kernels.unpack_weight(W, WOQ_DTYPE_MAP[W_dtype], int(W_shape[0]), int(W_shape[1]))


# ---- forward ops --------------------------------------------------------------------------------
def _require_gpu_input(x, name):
    if not x.is_cuda:
        raise RuntimeError(
            f"{name}: the input must be on the GPU (got {x.device}); there is no CPU implementation in this build"
        )


def ipex_woq_linear(input, W_prepack):
    _require_gpu_input(input, "torch_ipex::ipex_woq_linear")
    return _context_from_handle(W_prepack).run(input)


def _unary(fusion, name):
    def op(input, W_prepack):
        _require_gpu_input(input, f"torch_ipex::{name}")
        return _context_from_handle(W_prepack).run(input, fusion=fusion)

    op.__name__ = name
    return op


def _binary(fusion, name, n_others):
    def op(input, W_prepack, others):
        _require_gpu_input(input, f"torch_ipex::{name}")
        if len(others) < n_others:
            raise RuntimeError(f"torch_ipex::{name}: expected {n_others} extra input(s), got {len(others)}")
        return _context_from_handle(W_prepack).run(input, fusion=fusion, others=tuple(others[:n_others]))

    op.__name__ = name
    return op


woq_linear_gelu = _unary(_lib.FUSE_GELU_ERF, "woq_linear_gelu")
woq_linear_new_gelu = _unary(_lib.FUSE_GELU_TANH, "woq_linear_new_gelu")
woq_linear_relu = _unary(_lib.FUSE_RELU, "woq_linear_relu")
woq_linear_silu = _unary(_lib.FUSE_SILU, "woq_linear_silu")
woq_linear_add = _binary(_lib.FUSE_ADD, "woq_linear_add", 1)
woq_linear_add_add = _binary(_lib.FUSE_ADD_ADD, "woq_linear_add_add", 2)
woq_linear_mul = _binary(_lib.FUSE_MUL, "woq_linear_mul", 1)


def woq_linear(
    input,
    qweight,
    weight_dtype: str,
    weight_shape: List[int],
    weight_scales: List[torch.Tensor],
    weight_zeros: Optional[List[torch.Tensor]],
    bias: Optional[List[torch.Tensor]],
    g_idx: Optional[torch.Tensor],
    group_size: int,
    lowp_mode: int,
    act_quant_mode: int,
    compensation: Optional[torch.Tensor] = None,
):
    """Context-free forward (woq_linear_forward_v2, csrc/cpu/aten/Linear.cpp:556-617); the
    tensor arguments are the outputs of ``woq_linear_pack_weight``."""
    _require_gpu_input(input, "torch_ipex::woq_linear")
    if weight_dtype not in WOQ_DTYPE_MAP:
        raise RuntimeError(f"Unsupported weight dtype: {weight_dtype}")
    if g_idx is not None and WOQ_DTYPE_MAP[weight_dtype] == _lib.DTYPE_INT4 and group_size > 0:
        # the packed weight from woq_linear_pack_weight is already sorted by group
        src = torch.argsort(g_idx.to(input.device).to(torch.int64).reshape(-1), stable=True).to(torch.int32)
        input = _kernels.shuffle_activations(input, src.contiguous())
    if weight_zeros is not None and len(weight_zeros) != 4:
        raise RuntimeError("IPEX WOQ: expect list of zeros has length 4")
    if bias is not None and len(bias) != 3:
        raise RuntimeError("IPEX WOQ: expect list of bias has length 3")
    if len(weight_scales) != 3:
        raise RuntimeError("IPEX WOQ: expect list of scales has length 3")
    N, K = int(weight_shape[0]), int(weight_shape[1])
    return _kernels.linear(
        input,
        qweight,
        WOQ_DTYPE_MAP[weight_dtype],
        N,
        K,
        weight_scales[0],
        weight_scales[1],
        weight_scales[2],
        weight_zeros[3] if weight_zeros is not None else None,
        group_size,
        bias[0].contiguous() if bias is not None else None,
        lowp_mode,
        act_quant_mode,
    )


# ---- mixture of experts over WOQ linears ---------------------------------------------------------
def _is_python_context(ctx):
    return isinstance(ctx, WoqLinearOpContext)


def _run_context(ctx, x, fusion=_lib.FUSE_NONE, others=()):
    """One linear of an expert: ``ctx`` is a ``torch.classes.ipex_prepack.WoqLinearOpContext`` (the
    registered operators, by handle) or the ctypes twin of this module."""
    if isinstance(ctx, torch.Tensor) and ctx.numel() == 1 and ctx.dtype == torch.int64 and ctx.item() < 0:
        ctx = _context_from_handle(ctx)  # a handle of the ctypes twin (negative), resolved here
    if _is_python_context(ctx):
        return ctx.run(x, fusion=fusion, others=others)
    h = ctx if isinstance(ctx, torch.Tensor) else ctx.get_data_handle()
    if fusion == _lib.FUSE_NONE:
        return torch.ops.torch_ipex.ipex_woq_linear(x, h)
    if fusion == _lib.FUSE_SILU:
        return torch.ops.torch_ipex.woq_linear_silu(x, h)
    if fusion == _lib.FUSE_MUL:
        return torch.ops.torch_ipex.woq_linear_mul(x, h, list(others))
    raise RuntimeError(f"unexpected post-op 0x{fusion:x} in an expert")


def _moe_expert(hidden_states, top_x, idx, gate, up, down, routing_weights, output):
    """One expert: gather its tokens, down(up(x) * silu(gate(x))), weighted accumulation
    (mixtral_moe_woq_kernl_impl, csrc/cpu/aten/kernels/MoEKrnl.cpp:254-284)."""
    cur = _kernels.moe_gather_rows(hidden_states, top_x)
    act = _run_context(gate, cur, _lib.FUSE_SILU)
    cur = _run_context(down, _run_context(up, cur, _lib.FUSE_MUL, (act,)))
    return _kernels.moe_scale_add_rows(output, cur, routing_weights, top_x, idx)


def _no_all_reduce(is_distributed, name):
    if is_distributed:
        raise RuntimeError(f"torch_ipex::{name}: is_distributed=True needs an all-reduce, which this one-GPU build does not have")


def mixtral_moe_woq(hidden_states, top_x, idx, gate_wei, up_wei, down_wei, routing_weights, output, is_distributed):
    """One expert of a Mixtral-style layer (csrc/cpu/aten/MoE.cpp:260-288): ``gate_wei`` / ``up_wei`` /
    ``down_wei`` are context handles, ``top_x`` the tokens routed to the expert and ``idx`` their
    slot in the top-k; accumulates into ``output`` and returns it."""
    _require_gpu_input(hidden_states, "torch_ipex::mixtral_moe_woq")
    _no_all_reduce(is_distributed, "mixtral_moe_woq")
    if top_x.shape[0] == 0:
        return output
    dev = hidden_states.device
    return _moe_expert(hidden_states, top_x.to(dev), idx.to(dev), gate_wei, up_wei, down_wei, routing_weights, output)


# ---- a whole layer in grouped launches (decode sizes) -----------------------------------------------
# (identities of the experts' contexts, device, stream) -> plan.  A plan snapshots device addresses of its contexts and
# holds none of them alive; it is valid while no context anywhere has changed or freed its arrays since the snapshot
# (_context_epochs), which is checked before every use.  One plan per stream: its routing buffers are reused from call
# to call, and calls on one stream follow each other.
_MOE_PLANS = {}
_MOE_PLAN_LIMIT = 128
# (device, stream, dtype, intermediate width, hidden width) -> (act, inter, y) rows for the largest routing the grouped
# path takes, allocated once and never moved, so that a HIP graph captured over a layer keeps valid addresses; shared
# by all layers of those widths (calls on one stream follow each other).
_MOE_ROWS = {}


def _context_epochs():
    """(epoch of this module's contexts, epoch of the registered custom class's contexts)."""
    return _context_epoch[0], int(torch.ops.ipex_prepack.woq_context_epoch())


def _context_pointers(ctx):
    """[qweight, fp16 scales, bf16 scales, zero points or 0, fp32 bias or 0, N, K, group size, weight dtype,
    lowp_mode, has g_idx, device index, (scale, zero) dword table or 0] of a context of either binding."""
    if _is_python_context(ctx):
        ptr = lambda t: 0 if t is None else t.data_ptr()
        N, K = ctx.weight_shape_
        return [ctx.at_weight_.data_ptr(), ctx.scales_list_[1].data_ptr(), ctx.scales_list_[2].data_ptr(),
                ptr(ctx.zeros_u8_), ptr(ctx.bias_f32_), N, K, ctx.group_size_, ctx.weight_dtype_, ctx.lowp_mode_,
                0 if ctx.g_idx_ is None else 1, ctx.at_weight_.device.index, ptr(ctx.scale_zero_f16x2_)]
    return list(ctx.kernel_pointers())


class _MoeGroupedPlan:
    """What the grouped launches of one layer reuse from call to call: per linear (gate, up, down) the experts'
    pointer tables and the woq_hip_moe_group structs on the device (one per size class of the experts: fewer than five
    rows, which lowp_mode BF16 computes in fp16, up to 16 rows, up to 64), the routing buffers they point to and the
    intermediate rows."""

    def __init__(self, gate_ctx, up_ctx, down_ctx, device):
        self.epochs = _context_epochs()  # before the snapshot: a change during it makes the plan stale, not wrong
        self.ok = False
        infos = [[_context_pointers(c) for c in lst] for lst in (gate_ctx, up_ctx, down_ctx)]
        self.shapes = []
        for rows in infos:
            first = rows[0]
            same = all(r[5:11] == first[5:11] and (r[3] == 0) == (first[3] == 0) and (r[4] == 0) == (first[4] == 0)
                       and (r[12] == 0) == (first[12] == 0) and r[11] == device.index for r in rows)
            if not same or first[10] or first[8] not in (_lib.DTYPE_INT4, _lib.DTYPE_INT8) or first[9] not in (0, 1, 2):
                return
            self.shapes.append(dict(N=first[5], K=first[6], G=first[7], wd=first[8], lowp=first[9]))
        g, u, d = self.shapes
        if (g["N"], g["K"]) != (u["N"], u["K"]) or d["K"] != g["N"] or d["N"] != g["K"] or len({x["lowp"] for x in self.shapes}) != 1:
            return
        if any((-(-x["N"] // 16)) % 2 for x in self.shapes):  # the grouped kernel takes two 16-column blocks per workgroup
            return
        R = _lib.MOE_ROUTE_MAX
        i32 = lambda: torch.empty(R, dtype=torch.int32, device=device)
        self.x_row = torch.empty(R, dtype=torch.int64, device=device)
        # slot tables [class][expert, first row, rows][S]: experts with few / up to 16 / up to 64 rows / exactly one row
        self.S = len(gate_ctx)
        self.slots = torch.empty((4, 3, self.S), dtype=torch.int32, device=device)
        self.row_of, self.slot_of = i32(), i32()
        self.tables = []
        for rows in infos:
            col = lambda k: torch.tensor([r[k] for r in rows], dtype=torch.int64, device=device)
            self.tables.append(dict(qweight=col(0), s16=col(1), sb16=col(2), z8=col(3) if rows[0][3] else None,
                                    bias=col(4) if rows[0][4] else None, sz=col(12) if rows[0][12] else None))
        # the single-row decode kernel serves the experts with one row where all three linears have its
        # (scale, zero) tables: 4-bit weights in groups of 32, 64 or 128 x 2^k, K a multiple of 256
        self.single_row = all(t["sz"] is not None for t in self.tables) and all(
            x["wd"] == _lib.DTYPE_INT4 and x["K"] % 256 == 0 and (x["G"] in (32, 64) or (
                x["G"] % 128 == 0 and (x["G"] // 128) & (x["G"] // 128 - 1) == 0))
            for x in self.shapes)
        self.structs = {}
        self.device = device
        self.ok = True

    def buffers(self, dtype, stream):
        N1, H = self.shapes[0]["N"], self.shapes[0]["K"]
        key = (self.device.index, stream, dtype, N1, H)
        have = _MOE_ROWS.get(key)
        if have is None:
            mk = lambda n: torch.empty((_lib.MOE_ROUTE_MAX, n), dtype=dtype, device=self.device)
            have = _MOE_ROWS[key] = (mk(N1), mk(N1), mk(H))
        return have

    def group_struct(self, linear, cls, f16_scales, gather, sz=False):
        """Device copy of the woq_hip_moe_group of one launch (built once).  ``sz``: for the integer-weight decode
        kernels, with the (scale, zero) dword tables in place of the scales."""
        key = (linear, cls, f16_scales, gather, sz)
        st = self.structs.get(key)
        if st is None:
            t = self.tables[linear]
            ptr = lambda x: 0 if x is None else x.data_ptr()
            tab = [ptr(self.slots[cls, i]) for i in range(3)] + [ptr(self.x_row) if gather else 0]
            if sz:
                fields = tab + [ptr(t["qweight"]), ptr(t["sz"]), 0, ptr(t["bias"])]
            else:
                fields = tab + [ptr(t["qweight"]), ptr(t["s16"] if f16_scales else t["sb16"]), ptr(t["z8"]), ptr(t["bias"])]
            st = torch.tensor(fields, dtype=torch.int64, device=self.device)
            self.structs[key] = st
        return st


def _moe_plan(gate_ctx, up_ctx, down_ctx, device, stream):
    # the contexts themselves, not the lists that hold them: a caller may build the lists anew for every call, or
    # replace an expert inside a list
    key = (tuple(map(id, gate_ctx)), tuple(map(id, up_ctx)), tuple(map(id, down_ctx)), device.index, stream)
    plan = _MOE_PLANS.get(key)
    if plan is None or plan.epochs != _context_epochs():
        if len(_MOE_PLANS) >= _MOE_PLAN_LIMIT:
            _MOE_PLANS.clear()
        plan = _MoeGroupedPlan(gate_ctx, up_ctx, down_ctx, device)
        _MOE_PLANS[key] = plan
    return plan


def _small_batch_threshold():
    """Rows below which lowp_mode BF16 computes in fp16: the library's reading of IPEX_WOQ_SMALL_BATCH_THRESHOLD."""
    return (_lib._lib or _lib.load()).woq_hip_small_batch_threshold()


def _f16_regime(lowp, x_dtype, rows):
    return lowp == 1 or (lowp == 0 and x_dtype == torch.float16) or (lowp == 2 and rows < _small_batch_threshold())


def _deepseek_moe_grouped(hidden_states, topk_ids, gate_ctx, up_ctx, down_ctx, routing_weights):
    """The layer in five to fourteen launches and without reading the routing on the host: the routing is sorted on the
    device, every linear runs once per compute type over all experts that have tokens (woq_hip_linear_grouped), and
    the contributions of a token are added in ascending expert order.  Returns None when the layer does not fit
    (more than 64 tokens, mixed experts, act-order, NF4 / FP8 / lowp INT8 ...): the caller then takes the per-expert path."""
    x = hidden_states
    if x.dim() != 2 or x.dtype not in (torch.bfloat16, torch.float16) or not x.is_contiguous() or x.data_ptr() % 16:
        return None
    if _small_batch_threshold() != 5:  # the size classes below are cut for the default threshold
        return None
    T, H = x.shape
    if topk_ids.dim() != 2 or topk_ids.shape[0] != T or not topk_ids.is_cuda or topk_ids.device != x.device:
        return None
    topk = topk_ids.shape[1]
    if T == 0 or T > 64 or T * topk > _lib.MOE_ROUTE_MAX or T * H * 2 >= 2**31:
        return None
    if routing_weights.dtype != x.dtype or routing_weights.dim() != 2 or tuple(routing_weights.shape) != (T, topk) or not routing_weights.is_cuda:
        return None
    raw_stream = _current_raw_stream(x.device.index)
    plan = _moe_plan(gate_ctx, up_ctx, down_ctx, x.device, raw_stream)
    if not plan.ok or plan.shapes[0]["K"] != H:
        return None
    lowp = plan.shapes[0]["lowp"]
    # experts with fewer than five rows on the integer-weight decode kernels, as woq_hip_linear serves them, where
    # such rows compute in fp16 and the layer has the kernels' tables; those with exactly one row (most of them in a
    # layer with many experts and few tokens) on the single-row kernel
    single = plan.single_row and _f16_regime(lowp, x.dtype, 1)
    # lowp_mode BF16: experts with fewer than five rows compute in fp16, a class of their own
    split = 5 if (lowp == 2 or single) else 0
    # (size class, bound on its slots' rows): an expert has at most T * topk entries (a token may name it in several of
    # its slots), so the larger classes are empty while that bound is small
    # a single token: every (token, slot) entry is a slot of its own (an expert named twice included)
    each = single and T == 1 and topk <= plan.S
    most = T * topk
    launches = [(3, 1)] if each else ([(3, 1)] if single else []) + ([(0, 4)] if split else []) + \
               ([(1, 16)] if most >= split else []) + ([(2, 64)] if most > 16 else [])
    for cls, bound in launches:
        f16 = _f16_regime(lowp, x.dtype, bound)
        # rows must be in the compute type; bf16 rows under fp16 compute are converted for up to 16 rows per slot
        if f16 and x.dtype == torch.bfloat16 and bound > 16:
            return None
        if not f16 and x.dtype == torch.float16:
            return None
    lib = _lib.load()
    ids = topk_ids.to(torch.int64).contiguous()
    rw = routing_weights.contiguous()
    R = T * topk
    N1 = plan.shapes[0]["N"]
    act, inter, y = plan.buffers(x.dtype, raw_stream)  # calls on one stream follow each other
    out = torch.empty_like(x)
    code = _kernels._ACT_CODE[x.dtype]
    with torch.cuda.device(x.device):
        stream = _kernels._stream()
        _lib.check(lib.woq_hip_moe_route(ids.data_ptr(), T, topk, len(gate_ctx), split, 16, 2 if each else int(single), plan.S,
                                         plan.x_row.data_ptr(), plan.slots.data_ptr(), plan.row_of.data_ptr(),
                                         plan.slot_of.data_ptr(), stream), "moe_route")
        nslots = R if each else min(R, plan.S)  # experts that can have tokens: the tables are dense
        p = _lib.LinearParams()
        p.struct_size = ctypes.sizeof(_lib.LinearParams)
        p.x_dtype = p.out_dtype = code
        p.stream = torch.cuda.current_stream().cuda_stream
        p.lowp_mode = lowp
        p.act_quant_mode = -1
        steps = ((0, x, act, _lib.FUSE_SILU, None, True), (1, x, inter, _lib.FUSE_MUL, act, True),
                 (2, inter, y, _lib.FUSE_NONE, None, False))
        for li, src, dst, fusion, other, gather in steps:
            sh = plan.shapes[li]
            p.K, p.N, p.weight_dtype, p.group_size = sh["K"], sh["N"], sh["wd"], sh["G"]
            p.x, p.out, p.fusion = src.data_ptr(), dst.data_ptr(), fusion
            p.others[0] = other.data_ptr() if other is not None else None
            for cls, bound in launches:
                p.M = bound
                # (a non-null value tells the entry point that the group's scales are (scale, zero) dword tables)
                sz = cls == 3 or (cls == 0 and single)
                p.scale_zero_f16x2 = plan.tables[li]["sz"].data_ptr() if sz else None
                g = plan.group_struct(li, cls, _f16_regime(lowp, x.dtype, bound), gather, sz)
                _lib.check(lib.woq_hip_linear_grouped(ctypes.byref(p), g.data_ptr(), nslots), "woq_linear_grouped")
        _lib.check(lib.woq_hip_moe_combine_rows(out.data_ptr(), code, T, H, y.data_ptr(), rw.data_ptr(), topk,
                                                plan.row_of.data_ptr(), plan.slot_of.data_ptr(), 0, stream), "moe_combine_rows")
    return out


def deepseek_moe_woq(hidden_states, topk_ids, gate_ctx, up_ctx, down_ctx, routing_weights, is_distributed):
    """All experts of a layer (csrc/cpu/aten/MoE.cpp:290-328): ``topk_ids`` [tokens, top-k] names the
    experts of every token, the three lists hold one WoqLinearOpContext per expert.  Experts are
    visited in ascending order and, inside an expert, tokens in ascending order (get_expert_topx_idx,
    MoE.cpp:64-81), which fixes the order of the additions into a token's row.
    The routing table is read on the host (one synchronizing copy of [tokens, top-k] int64) to size
    the per-expert launches."""
    _require_gpu_input(hidden_states, "torch_ipex::deepseek_moe_woq")
    _no_all_reduce(is_distributed, "deepseek_moe_woq")
    num_experts = len(gate_ctx)
    if len(up_ctx) != num_experts or len(down_ctx) != num_experts:
        raise RuntimeError("torch_ipex::deepseek_moe_woq: gate / up / down lists differ in length")
    if topk_ids.numel() and os.environ.get("IPEX_AMD_MOE_GROUPED", "1") != "0":
        grouped = _deepseek_moe_grouped(hidden_states, topk_ids, gate_ctx, up_ctx, down_ctx, routing_weights)
        if grouped is not None:
            return grouped
    output = torch.zeros_like(hidden_states)
    ids = topk_ids.detach().to("cpu", torch.int64)
    if ids.numel() == 0:
        return output
    if int(ids.min()) < 0 or int(ids.max()) >= num_experts:
        raise RuntimeError(f"torch_ipex::deepseek_moe_woq: expert ids must lie in [0, {num_experts})")
    topk = ids.shape[1]
    order = torch.argsort(ids.reshape(-1), stable=True)  # by expert, then token, then slot
    counts = torch.bincount(ids.reshape(-1), minlength=num_experts).tolist()
    tokens = order // topk
    routed = torch.stack([tokens, order % topk]).to(hidden_states.device)
    start = 0
    for e, n in enumerate(counts):
        if n:
            tok = tokens[start:start + n]
            if n > 1 and bool((tok[1:] == tok[:-1]).any()):
                # a token names this expert more than once: the scatter adds one row per token, so the entries go in
                # rounds, the k-th mention of every token in round k
                first = torch.cat([torch.ones(1, dtype=torch.bool), tok[1:] != tok[:-1]])
                pos = torch.arange(n)
                mention = pos - torch.cummax(torch.where(first, pos, torch.zeros_like(pos)), 0).values
                for k in range(int(mention.max()) + 1):
                    sel = (start + torch.nonzero(mention == k).flatten()).to(hidden_states.device)
                    _moe_expert(hidden_states, routed[0].index_select(0, sel), routed[1].index_select(0, sel), gate_ctx[e],
                                up_ctx[e], down_ctx[e], routing_weights, output)
            else:
                _moe_expert(hidden_states, routed[0, start:start + n], routed[1, start:start + n], gate_ctx[e], up_ctx[e],
                            down_ctx[e], routing_weights, output)
        start += n
    return output


_registered = False
_libs = []


def register():
    """Loads the C++ binding, which registers the operators and the custom class under
    ``torch.ops.torch_ipex`` / ``torch.ops.ipex_prepack`` / ``torch.classes.ipex_prepack``, and adds the
    mixture-of-experts ops (idempotent).  Raises if the binding has not been built."""
    global _registered
    if _registered:
        return
    _lib.load_torch_binding()
    # The binding defines mixtral_moe_woq / deepseek_moe_woq over the registered custom class (per-expert launches,
    # routing read on the host).  In front of them: a kernel for mixtral_moe_woq that also resolves the handles of this
    # module's ctypes contexts, and deepseek_moe_woq as a function that takes contexts of either binding and runs small
    # batches in grouped launches without reading the routing on the host.
    tl = torch.library.Library("torch_ipex", "IMPL")
    _libs.append(tl)
    tl.impl("mixtral_moe_woq", mixtral_moe_woq, "CUDA")
    setattr(torch.ops.torch_ipex, "deepseek_moe_woq", deepseek_moe_woq)
    _registered = True
