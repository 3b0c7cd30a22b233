from . import modules
from .modules import WeightOnlyQuantizedLinear
