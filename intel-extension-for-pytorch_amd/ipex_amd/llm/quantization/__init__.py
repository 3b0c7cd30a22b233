from .utils import QuantDtype, QuantMethod
from .woq_linear import IPEXWeightOnlyQuantizedLinear
