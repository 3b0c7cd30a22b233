"""prepare / convert for the weight-only-quantization recipe.

The reference routes WOQ through its general quantization front end
(intel_extension_for_pytorch/quantization/_quantize.py:24, 407-451): ``prepare`` records the
recipe on the model, ``convert`` swaps every ``nn.Linear`` for ``WeightOnlyQuantizedLinear``.
Only that recipe is handled here; static / dynamic INT8 recipes are rejected.
"""
import copy

import torch
from torch.ao.quantization import QConfigMapping

from ._qconfig import QConfigWoq


def prepare(model, configure, example_inputs=None, inplace=False, bn_folding=True, example_kwarg_inputs=None):
    assert isinstance(model, torch.nn.Module), "Only support nn.Module prepare for quantization path"
    if isinstance(configure, QConfigMapping):
        configure = configure.global_qconfig
    if not isinstance(configure, QConfigWoq):
        raise NotImplementedError(
            "prepare: only the weight-only quantization recipe "
            "(get_weight_only_quant_qconfig_mapping) is supported by this build"
        )
    prepared = model if inplace else copy.deepcopy(model)
    prepared.q_config = configure
    return prepared


def convert(model, inplace=False):
    assert isinstance(model, torch.nn.Module), "Only support nn.Module convert for quantization path"
    assert hasattr(model, "q_config"), "Please do prepare the model before doing convert"
    from ..nn.modules.weight_only_quantization import WeightOnlyQuantizedLinear

    converted = model if inplace else copy.deepcopy(model)
    qconfig = converted.q_config

    def swap(module):
        for name, child in list(module.named_children()):
            if type(child) is torch.nn.Linear:
                child.qconfig = qconfig
                setattr(module, name, WeightOnlyQuantizedLinear.from_float(child))
            else:
                swap(child)

    if type(converted) is torch.nn.Linear:
        converted.qconfig = qconfig
        return WeightOnlyQuantizedLinear.from_float(converted)
    swap(converted)
    return converted
