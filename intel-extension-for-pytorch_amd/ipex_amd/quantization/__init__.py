from ._qconfig import (
    QConfigWoq,
    WoqActQuantMode,
    WoqLowpMode,
    WoqWeightDtype,
    WoqWeightQScheme,
    WOQ_ACT_QUANT_MODE_TO_STR,
    WOQ_DTYPE_TO_STR,
    WOQ_LOWP_MODE_TO_STR,
    WOQ_QSCHEME_TO_STR,
    get_weight_only_quant_qconfig_mapping,
)
from ._quantize_utils import (
    dequantize_per_block,
    dequantize_per_channel,
    quantize_per_block,
    quantize_per_channel,
)
from ._quantize import convert, prepare
