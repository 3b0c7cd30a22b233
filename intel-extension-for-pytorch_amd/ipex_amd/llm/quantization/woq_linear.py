"""``ipex.llm.quantization.IPEXWeightOnlyQuantizedLinear``: the device-agnostic front door
serving frameworks use to build a WOQ linear straight from checkpoint tensors
(intel_extension_for_pytorch/llm/quantization/woq_linear.py:9-80)."""
from importlib import import_module
from typing import Optional

import torch
import torch.nn as nn

from .utils import QuantDtype, QuantMethod


class IPEXWeightOnlyQuantizedLinear(nn.Module):
    r"""Wraps the device implementation selected from the device of ``qweight``."""

    module_mapping = {
        "cuda": "ipex_amd.nn.modules.weight_only_quantization",
        # checkpoint tensors still on the host are moved to the GPU by the prepack
        "cpu": "ipex_amd.nn.modules.weight_only_quantization",
    }
    impl_name = "WeightOnlyQuantizedLinear"

    def __init__(self, woq_linear_impl):
        super().__init__()
        self.woq_linear_impl = woq_linear_impl

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
        r"""qweight / scales / zero_points in AutoGPTQ (default) or AutoAWQ layout; see
        ``WeightOnlyQuantizedLinear.from_weight``."""
        device_type = qweight.device.type
        assert device_type in cls.module_mapping, "Device type not supported."
        impl_cls = getattr(import_module(cls.module_mapping[device_type]), cls.impl_name)
        impl = impl_cls.from_weight(
            qweight, scales, zero_points, in_features, out_features, qconfig, bias, group_size, g_idx,
            quant_method, dtype, **kwargs,
        )
        return cls(impl)

    def forward(self, x, **kwargs):
        return self.woq_linear_impl(x, **kwargs)
