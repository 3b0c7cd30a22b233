"""WeightOnlyQuantizedLinear: the module users get from ``convert`` or build from a checkpoint.

Same constructors, attributes and forward call as the reference module
(intel_extension_for_pytorch/nn/modules/weight_only_quantization.py:40-533); the prepack
context and the op behind ``forward`` run on MI355X.  The tensor-parallel subclasses of the
reference (IpexWoqLinearAllreduce, IpexWoqLmHeadLinearAllreduce) wrap a collective around
this module and are not part of a one-GPU build.
"""
from enum import IntEnum
from typing import Optional

import torch
from torch import nn

from .. import utils as _nn_utils  # noqa: F401  (package marker)
from ... import ops as _ops
from ...llm.quantization.utils import QuantDtype, QuantMethod
from ...quantization import (
    QConfigWoq,
    WoqActQuantMode,
    WoqLowpMode,
    WoqWeightDtype,
    WoqWeightQScheme,
    quantize_per_block,
    quantize_per_channel,
)
from ...quantization._qconfig import (
    WOQ_ACT_QUANT_MODE_TO_STR,
    WOQ_DTYPE_TO_STR,
    WOQ_LOWP_MODE_TO_STR,
    WOQ_QSCHEME_TO_STR,
)
from ...utils.weight_only_quantization import (
    _convert_awq_scales_qzeros,
    _convert_gptq_scales_qzeros,
    _convert_optimum_format_to_desired,
)


class WoqWeightFormat(IntEnum):
    PLAIN_FORMAT = 0
    GPTQ_FORMAT = 1
    AWQ_FORMAT = 2


def _target_device(t):
    if t.is_cuda:
        return t.device
    if not torch.cuda.is_available():
        raise RuntimeError("WeightOnlyQuantizedLinear needs a GPU: this build has no CPU path for the WOQ linear")
    return torch.device("cuda", torch.cuda.current_device())


class WeightOnlyQuantizedLinear(nn.Module):
    r"""A weight-only quantized linear layer: floating-point activations in and out, weights
    stored as INT4 / INT8 and dequantized inside the GEMM kernel."""

    def __init__(self, in_features, out_features, bias_=True, dtype=WoqWeightDtype.INT8):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.bias = bias_
        self.dtype = dtype
        # Reference to the packed weight held by the context, for dtype / device queries only;
        # its shape is the tile layout, not [out_features, in_features].
        self.weight = None
        self._op_context = None
        self._lowp_mode = 0
        self._act_quant_mode = 0
        self._group_size = -1
        self._cache_weight_for_large_batch = False
        self._weight_qscheme = WoqWeightQScheme.ASYMMETRIC

    def pre_ipex_gemm(self, input):
        return input

    def post_ipex_gemm(self, output):
        return output

    def forward(self, x):
        x = self.pre_ipex_gemm(x)
        Y = torch.ops.torch_ipex.ipex_woq_linear(x, self._op_context.get_data_handle())
        return self.post_ipex_gemm(Y)

    def _get_name(self):
        return "WeightOnlyQuantizedLinear"

    def extra_repr(self):
        return (
            "in_features={}, out_features={}, dtype={}, bias={}, lowp_mode={}, act_quant_mode={}, "
            "group_size={}, cache_weight_for_large_batch={}, weight_qscheme={}"
        ).format(
            self.in_features,
            self.out_features,
            WOQ_DTYPE_TO_STR[self.dtype],
            self.bias,
            WOQ_LOWP_MODE_TO_STR[self._lowp_mode],
            WOQ_ACT_QUANT_MODE_TO_STR[self._act_quant_mode],
            self._group_size,
            self._cache_weight_for_large_batch,
            WOQ_QSCHEME_TO_STR[self._weight_qscheme],
        )

    # ---- construction from a float module -----------------------------------------------------
    @classmethod
    def from_float(cls, mod, scales=None, zero_points=None):
        r"""Quantizes ``mod.weight`` according to ``mod.qconfig`` (a QConfigWoq).  With ``scales``
        (and ``zero_points`` unless symmetric) given they are used as is, otherwise they come
        from the min / max of each channel or block."""
        assert isinstance(mod, torch.nn.Linear), (
            "WeightOnlyQuantizedLinear.from_float only works for nn.Linear or its subclasses, "
            f"but found {type(mod)}"
        )
        assert hasattr(mod, "qconfig"), "Input float module must have qconfig defined"
        qconfig = mod.qconfig
        if qconfig is None or not isinstance(qconfig, QConfigWoq):
            return mod
        lowp_mode = qconfig.lowp_mode
        act_quant_mode = qconfig.act_quant_mode
        dtype = qconfig.weight_dtype
        group_size = qconfig.group_size
        sym_quant = qconfig.weight_qscheme == WoqWeightQScheme.SYMMETRIC
        # INT8 weights under lowp_mode INT8 need zero points of 0: the int8 kernel subtracts
        # them from int8 values and would overflow otherwise.
        if dtype == WoqWeightDtype.NF4 or (dtype == WoqWeightDtype.INT8 and lowp_mode == WoqLowpMode.INT8):
            assert sym_quant is True, "WOQ NF4 and INT8 with lowp-mode 3 must use symmetric quantization"
        w = mod.weight.detach()
        if group_size == -1:
            qweight, scales, zero_points = quantize_per_channel(w.cpu().float(), dtype, scales, zero_points, sym_quant)
        else:
            qweight, scales, zero_points = quantize_per_block(
                w.cpu().float(), dtype, group_size, scales, zero_points, sym_quant
            )
        if not hasattr(mod, "in_features"):
            mod.in_features = mod.weight.size()[1]
        if not hasattr(mod, "out_features"):
            mod.out_features = mod.weight.size()[0]
        cache_weight_for_large_batch = qconfig.cache_weight_for_large_batch and lowp_mode in (2, 3)
        qlinear = cls._init_cls(
            mod,
            dtype,
            qweight,
            scales,
            zero_points,
            None,  # bias: taken from mod
            None,  # g_idx
            group_size,
            lowp_mode,
            act_quant_mode,
            cache_weight_for_large_batch,
            False,
            device=_target_device(mod.weight),
        )
        del qweight
        mod.weight = torch.nn.Parameter()
        return qlinear

    @classmethod
    def from_float_and_qweight(
        cls,
        mod,
        qweight,
        dtype,
        scales,
        zero_points,
        bias=None,
        group_size=-1,
        g_idx=None,
        weight_format=WoqWeightFormat.PLAIN_FORMAT,
    ):
        r"""Builds the module from a float module (for shapes, bias and recipe) and an already
        quantized weight."""
        assert isinstance(mod, torch.nn.Linear), (
            f"WeightOnlyQuantizedLinear.from_float_and_qweight needs an nn.Linear, but found {type(mod)}"
        )
        assert hasattr(mod, "qconfig"), "Input float module must have qconfig defined"
        lowp_mode = 0
        act_quant_mode = 0
        cache_weight_for_large_batch = False
        if mod.qconfig is not None:
            lowp_mode = getattr(mod.qconfig, "lowp_mode", lowp_mode)
            act_quant_mode = getattr(mod.qconfig, "act_quant_mode", act_quant_mode)
            if hasattr(mod.qconfig, "cache_weight_for_large_batch"):
                cache_weight_for_large_batch = mod.qconfig.cache_weight_for_large_batch and lowp_mode in (2, 3)
        supported = [torch.int32, torch.uint8, torch.int8, torch.quint4x2, torch.bfloat16, torch.float32, torch.float8_e4m3fn]
        assert qweight.dtype in supported, "Data type of quantized weight should be in {}, but got: {}".format(
            supported, qweight.dtype
        )
        if not hasattr(mod, "in_features"):
            mod.in_features = mod.weight.size()[1]
        if not hasattr(mod, "out_features"):
            mod.out_features = mod.weight.size()[0]
        if group_size < 0:
            scales = scales.squeeze()
            if zero_points is not None:
                zero_points = zero_points.squeeze()
        qlinear = cls._init_cls(
            mod,
            dtype,
            qweight,
            scales,
            zero_points,
            bias,
            g_idx,
            group_size,
            lowp_mode,
            act_quant_mode,
            cache_weight_for_large_batch,
            dtype == WoqWeightDtype.INT4,
            weight_format,
            device=_target_device(qweight),
        )
        del qweight
        mod.weight = torch.nn.Parameter()
        return qlinear

    @classmethod
    def from_float_and_int4_weight(
        cls, mod, qweight, scales, zero_points, bias=None, group_size=-1, g_idx=None,
        weight_format=WoqWeightFormat.PLAIN_FORMAT,
    ):
        print("[WARNING] from_float_and_int4_weight() is deprecated. Please use from_float_and_qweight() instead.")
        return cls.from_float_and_qweight(
            mod, qweight, WoqWeightDtype.INT4, scales, zero_points, bias, group_size, g_idx, weight_format
        )

    # ---- construction from an INT4 checkpoint ---------------------------------------------------
    @classmethod
    def from_int4_weight(
        cls,
        qweight,
        scales,
        zero_points,
        in_features,
        out_features,
        quant_method,
        qconfig=None,
        bias=None,
        group_size=-1,
        g_idx=None,
    ):
        r"""Builds the module from AutoGPTQ / AutoAWQ INT4 tensors (qweight int32 or uint8)."""
        lowp_mode = WoqLowpMode.BF16
        act_quant_mode = WoqActQuantMode.PER_IC_BLOCK
        cache_weight_for_large_batch = False
        if qconfig is not None and hasattr(qconfig, "global_qconfig"):
            g = qconfig.global_qconfig
            lowp_mode = getattr(g, "lowp_mode", lowp_mode)
            act_quant_mode = getattr(g, "act_quant_mode", act_quant_mode)
            if hasattr(g, "cache_weight_for_large_batch"):
                cache_weight_for_large_batch = g.cache_weight_for_large_batch and lowp_mode in (
                    WoqLowpMode.BF16,
                    WoqLowpMode.INT8,
                )
        supported = [torch.int32, torch.uint8, torch.quint4x2]
        assert qweight.dtype in supported, "Data type of int4 weight should be in {}, but got: {}".format(
            supported, qweight.dtype
        )
        qlinear = cls(in_features, out_features, dtype=WoqWeightDtype.INT4)
        weight_format = WoqWeightFormat.PLAIN_FORMAT
        if quant_method == QuantMethod.AWQ_GEMM:
            scales, zero_points = _convert_awq_scales_qzeros(scales, zero_points)
            weight_format = WoqWeightFormat.AWQ_FORMAT
        elif quant_method == QuantMethod.GPTQ_GEMM:
            if g_idx is not None:
                qweight, scales, zero_points = _convert_optimum_format_to_desired(
                    qweight, scales, zero_points, inplace=False
                )
            else:
                scales, zero_points = _convert_gptq_scales_qzeros(scales, zero_points)
                weight_format = WoqWeightFormat.GPTQ_FORMAT
        if bias is not None and torch.count_nonzero(bias) == 0:
            bias = None
        qlinear._op_context = torch.ops.ipex_prepack.weight_only_qlinear_prepack_int4(
            qweight,
            scales,
            zero_points,
            bias,
            g_idx,
            None,
            group_size,
            int(lowp_mode),
            act_quant_mode,
            cache_weight_for_large_batch,
            weight_format,
        )
        qlinear._finish_init(bias, zero_points, lowp_mode, act_quant_mode, group_size, cache_weight_for_large_batch)
        del qweight
        return qlinear

    @classmethod
    def from_weight(
        cls,
        qweight: torch.Tensor,
        scales: torch.Tensor,
        zero_points: torch.Tensor,
        in_features: int,
        out_features: int,
        qconfig=None,
        bias: Optional[torch.Tensor] = None,
        group_size: int = -1,
        g_idx: Optional[torch.Tensor] = None,
        quant_method: QuantMethod = QuantMethod.GPTQ_GEMM,
        dtype: QuantDtype = QuantDtype.INT4,
        **kwargs,
    ):
        if quant_method in [QuantMethod.GPTQ_GEMM, QuantMethod.AWQ_GEMM] and dtype == QuantDtype.INT4:
            return cls.from_int4_weight(
                qweight, scales, zero_points, in_features, out_features, quant_method, qconfig, bias, group_size, g_idx
            )
        raise AssertionError(
            "Currently ipex.llm.quantization.IPEXWeightOnlyQuantizedLinear.from_weight() supports 4bits with AWQ or GPTQ."
        )

    def _finish_init(self, bias, zero_points, lowp_mode, act_quant_mode, group_size, cache_weight_for_large_batch):
        self.weight = self._op_context.get_weight()
        self.bias = bias is not None
        self._lowp_mode = lowp_mode
        self._act_quant_mode = act_quant_mode
        self._group_size = group_size
        self._cache_weight_for_large_batch = cache_weight_for_large_batch
        self._weight_qscheme = (
            WoqWeightQScheme.ASYMMETRIC if zero_points is not None else WoqWeightQScheme.SYMMETRIC
        )

    @classmethod
    def _init_cls(
        cls,
        mod,
        dtype,
        qweight,
        scales,
        zero_points,
        bias,
        g_idx,
        group_size,
        lowp_mode,
        act_quant_mode,
        cache_weight_for_large_batch,
        is_from_int4_weight,
        weight_format=WoqWeightFormat.PLAIN_FORMAT,
        device=None,
    ):
        if bias is None and mod.bias is not None:
            bias = mod.bias.detach()
        if bias is not None and torch.count_nonzero(bias) == 0:
            bias = None  # an all-zero bias is dropped
        qlinear = cls(mod.in_features, mod.out_features, bias is not None, dtype=dtype)
        if device is not None:
            qweight = qweight.to(device)
        if is_from_int4_weight:
            qlinear._op_context = torch.ops.ipex_prepack.weight_only_qlinear_prepack_int4(
                qweight,
                scales,
                zero_points,
                bias,
                g_idx,
                None,  # batch size
                group_size,
                int(lowp_mode),
                act_quant_mode,
                cache_weight_for_large_batch,
                weight_format,
            )
        else:
            qlinear._op_context = torch.ops.ipex_prepack.weight_only_qlinear_prepack(
                qweight,
                dtype,
                [mod.out_features, mod.in_features],
                scales,
                zero_points,
                bias,
                g_idx,
                None,  # batch size
                group_size,
                int(lowp_mode),
                act_quant_mode,
                cache_weight_for_large_batch,
            )
        qlinear._finish_init(bias, zero_points, lowp_mode, act_quant_mode, group_size, cache_weight_for_large_batch)
        return qlinear
