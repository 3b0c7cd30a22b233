"""Weight-only-quantization recipe objects.

Mirrors the public names and values of the reference
(intel_extension_for_pytorch/quantization/_qconfig.py:106-307) so that a recipe written for
the reference configures this build unchanged.
"""
import warnings
from collections import namedtuple
from enum import IntEnum

import torch
from torch.ao.quantization import PerChannelMinMaxObserver, PlaceholderObserver, QConfig, QConfigMapping


class WoqLowpMode(IntEnum):
    NONE = 0
    FP16 = 1
    BF16 = 2
    INT8 = 3


class WoqActQuantMode(IntEnum):
    NONE = -1
    PER_TENSOR = 0
    PER_IC_BLOCK = 1  # IC = input channel
    PER_BATCH = 2
    PER_BATCH_IC_BLOCK = 3
    PER_TENSOR_SYM = 4
    PER_IC_BLOCK_SYM = 5
    PER_BATCH_SYM = 6
    PER_BATCH_IC_BLOCK_SYM = 7


class WoqWeightDtype(IntEnum):
    # values start at 1 to match the kernel-side codes
    INT8 = 1
    INT4 = 2
    NF4 = 3
    FP8 = 4


class WoqWeightQScheme(IntEnum):
    UNDEFINED = 0
    ASYMMETRIC = 1
    SYMMETRIC = 2


WOQ_LOWP_MODE_TO_STR = {m: m.name.lower() for m in WoqLowpMode}
WOQ_ACT_QUANT_MODE_TO_STR = {
    WoqActQuantMode.NONE: "none",
    WoqActQuantMode.PER_TENSOR: "per_tensor",
    WoqActQuantMode.PER_IC_BLOCK: "per_ic_block",
    WoqActQuantMode.PER_BATCH: "per_batch",
    WoqActQuantMode.PER_BATCH_IC_BLOCK: "per_batch_ic_block",
    WoqActQuantMode.PER_TENSOR_SYM: "per_tensor_sym",
    WoqActQuantMode.PER_IC_BLOCK_SYM: "per_ic_block_sym",
    WoqActQuantMode.PER_BATCH_SYM: "per_batch_sym",
    WoqActQuantMode.PER_BATCH_IC_BLOCK_SYM: "per_batch_ic_block_sym",
}
WOQ_DTYPE_TO_STR = {d: d.name.lower() for d in WoqWeightDtype}
WOQ_QSCHEME_TO_STR = {
    WoqWeightQScheme.UNDEFINED: "undefined",
    WoqWeightQScheme.ASYMMETRIC: "asymmetric",
    WoqWeightQScheme.SYMMETRIC: "symmetric",
}

QConfigWoq = namedtuple(
    "QConfigWoq",
    [
        *QConfig._fields,
        "lowp_mode",
        "act_quant_mode",
        "weight_dtype",
        "group_size",
        "cache_weight_for_large_batch",
        "weight_qscheme",
    ],
)


def get_weight_only_quant_qconfig_mapping(
    *,
    weight_dtype: int = WoqWeightDtype.INT8,
    lowp_mode: int = WoqLowpMode.NONE,
    act_quant_mode: int = WoqActQuantMode.PER_BATCH_IC_BLOCK_SYM,
    group_size: int = -1,
    weight_qscheme: int = WoqWeightQScheme.UNDEFINED,
):
    """Builds the QConfigMapping that selects weight-only quantization.

    weight_dtype   : WoqWeightDtype.INT8 / INT4 / NF4.
    lowp_mode      : lowest precision the GEMM may compute in.  NONE: activation dtype;
                     FP16; BF16 (fp16 below 5 rows, as the reference does); INT8: activations
                     are quantized to int8 on the fly.
    act_quant_mode : granularity of that on-the-fly quantization; ignored (forced to NONE)
                     unless lowp_mode is INT8.
    group_size     : -1 for one scale per output channel, else a positive power of two: the
                     number of input channels that share a scale / zero point.
    weight_qscheme : UNDEFINED resolves to SYMMETRIC for NF4 and for INT8 weights with
                     lowp_mode INT8, ASYMMETRIC otherwise; those two cases reject ASYMMETRIC.
    """
    assert group_size == -1 or (
        group_size > 0 and (group_size & (group_size - 1)) == 0
    ), "Group size must be -1 or a positive power of 2, but got {}".format(group_size)
    if weight_dtype in (torch.qint8, torch.quint4x2):
        weight_dtype = WoqWeightDtype.INT8 if weight_dtype == torch.qint8 else WoqWeightDtype.INT4
        warnings.warn(
            "torch.qint8 and torch.quint4x2 are deprecated for weight only quantization. "
            "Please use WoqWeightDtype.INT8 / WoqWeightDtype.INT4."
        )
    assert weight_dtype in [d.value for d in WoqWeightDtype], (
        f"Invalid weight data type for weight only quantization: {weight_dtype}"
    )
    if lowp_mode != WoqLowpMode.INT8:
        act_quant_mode = WoqActQuantMode.NONE
    must_be_sym = weight_dtype == WoqWeightDtype.NF4 or (
        weight_dtype == WoqWeightDtype.INT8 and lowp_mode == WoqLowpMode.INT8
    )
    if must_be_sym:
        assert weight_qscheme != WoqWeightQScheme.ASYMMETRIC, (
            "Asymmetric quantization of weight is not supported when "
            "(1) weight_dtype is NF4 or (2) weight_dtype is INT8 and lowp_mode is INT8."
        )
    if weight_qscheme == WoqWeightQScheme.UNDEFINED:
        weight_qscheme = WoqWeightQScheme.SYMMETRIC if must_be_sym else WoqWeightQScheme.ASYMMETRIC
    qconfig = QConfigWoq(
        activation=PlaceholderObserver.with_args(dtype=torch.float, is_dynamic=False),
        weight=PerChannelMinMaxObserver(),
        lowp_mode=lowp_mode,
        act_quant_mode=act_quant_mode,
        weight_dtype=weight_dtype,
        group_size=group_size,
        cache_weight_for_large_batch=False,
        weight_qscheme=weight_qscheme,
    )
    return QConfigMapping().set_global(qconfig)
