from .quant_linear import QuantLinear, UniformQuantizer, QuantizerMap  # noqa: F401
