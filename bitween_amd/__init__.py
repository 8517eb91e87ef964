"""bitween_amd: MI355X (gfx950) implementation of Bitween's quantized-linear
hot path behind the reference's Python names."""
from .functional import dequantize_rtn, quantize_rtn, quantize_rtn_perturbed
from .modules import QuantizedLinear, QuantizedLinearFunction, fuse_sibling_linears
from .quantizer.quantizer import Bitween, apply_precision_map

__all__ = ["Bitween", "QuantizedLinear", "QuantizedLinearFunction", "quantize_rtn", "dequantize_rtn",
           "quantize_rtn_perturbed", "apply_precision_map", "fuse_sibling_linears"]
