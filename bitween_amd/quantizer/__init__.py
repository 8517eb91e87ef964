from .quantizer import Bitween, apply_precision_map
