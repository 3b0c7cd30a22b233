from .linear_fusion import (  # noqa: F401
    ConcatLinear,
    Linear2SiluMul,
    LinearAdd,
    LinearAddAdd,
    LinearGelu,
    LinearMul,
    LinearNewGelu,
    LinearRelu,
    LinearSilu,
    LinearSiluMul,
)
