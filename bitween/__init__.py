"""Alias of bitween_amd under the reference's package name.

Models pickled by the reference name their classes by module path
(`bitween.modules.QuantizedLinear`, written by torch.save(model) as in main.py:134-145);
with this alias on the path torch.load resolves them to the MI355X implementation, and
scripts that say `from bitween import Bitween` or `from bitween.functional import quantize_rtn`
run unchanged.  Every submodule name below IS the bitween_amd module of the same name.
"""
import importlib
import sys

import bitween_amd
from bitween_amd import *  # noqa: F401,F403
from bitween_amd import __all__  # noqa: F401

for _name in ("functional", "modules", "quantizer", "quantizer.quantizer", "quantizer.func", "kernels",
              "kernels.hip_loader"):
    _mod = importlib.import_module("bitween_amd." + _name)
    sys.modules[__name__ + "." + _name] = _mod
    if "." not in _name:
        setattr(sys.modules[__name__], _name, _mod)
