"""bitween_amd: MI355X (gfx950) implementation of Bitween's quantized-linear
hot path behind the reference's Python names."""
from .functional import dequantize_rtn, quantize_rtn
from .modules import QuantizedLinear, QuantizedLinearFunction
from .quantizer.quantizer import Bitween

__all__ = ["Bitween", "QuantizedLinear", "QuantizedLinearFunction", "quantize_rtn", "dequantize_rtn"]
