from . import modules, quantization
