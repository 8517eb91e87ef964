"""bitween_amd: MI355X (gfx950) implementation of Bitween's quantized-linear
hot path behind the reference's Python names."""
from .functional import dequantize_rtn, get_scale_division, quantize_rtn, quantize_rtn_perturbed, set_scale_division
from .modules import QuantizedLinear, QuantizedLinearFunction, fuse_sibling_linears
from .quantizer.quantizer import Bitween, apply_precision_map

__all__ = ["Bitween", "QuantizedLinear", "QuantizedLinearFunction", "quantize_rtn", "dequantize_rtn",
           "quantize_rtn_perturbed", "apply_precision_map", "fuse_sibling_linears", "set_scale_division", "get_scale_division"]
