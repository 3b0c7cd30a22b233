from . import quantization
