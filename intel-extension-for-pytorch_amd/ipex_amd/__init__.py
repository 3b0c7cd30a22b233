"""MI355X-native weight-only-quantized linear, behind the Intel Extension for PyTorch API
for that path: ``quantization`` (recipe, quantize helpers, prepare / convert),
``nn.modules.WeightOnlyQuantizedLinear``, ``llm.quantization.IPEXWeightOnlyQuantizedLinear``
and the ``torch.ops.torch_ipex`` / ``torch.ops.ipex_prepack`` operators."""
from . import ops as _ops

_ops.register()

from . import llm, nn, quantization  # noqa: E402

__version__ = "0.1.0"
