from .quantizer import Bitween
