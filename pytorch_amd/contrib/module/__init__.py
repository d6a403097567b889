"""Quantized linear layers with the constructor arguments, parameter names and argument
marshalling of torch_npu.contrib.module.{LinearQuant, LinearA8W8Quant, LinearWeightQuant}."""
from .linear_quant import LinearQuant, LinearA8W8Quant
from .linear_weight_quant import LinearWeightQuant

__all__ = ["LinearQuant", "LinearA8W8Quant", "LinearWeightQuant"]
