def _set_module(model, submodule_key, module):
    """Replace the submodule named by a dotted key (bitween/quantizer/func.py:1-14)."""
    parent = model
    *path, leaf = submodule_key.split(".")
    for part in path:
        parent = getattr(parent, part)
    setattr(parent, leaf, module)
