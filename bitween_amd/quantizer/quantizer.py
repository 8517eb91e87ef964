"""Bitween: the model-level quantiser (bitween/quantizer/quantizer.py:11-118).

Only the RTN branch is on this package's path: every nn.Linear not listed in
ignore_layers is replaced by QuantizedLinear.from_float.  Trainable
quantisation and perplexity / KL evaluation belong to other subsystems of the
reference (calibration data, training loop, downloaded datasets) and raise
NotImplementedError here.
"""
import copy

import torch.nn as nn

from ..modules import QuantizedLinear, fuse_sibling_linears
from .func import _set_module


def _precision_for(name, layer_config, default):
    """(bits, group_size) for the layer `name`: its own entry, else the entry of the longest enclosing
    block ("model.layers.3" covers "model.layers.3.mlp.up_proj"), else `default`."""
    best, best_len = default, -1
    for key, value in layer_config.items():
        if (name == key or name.startswith(key + ".")) and len(key) > best_len:
            best, best_len = value, len(key)
    if best is None:
        return None
    if isinstance(best, dict):                            # the reference's saved form: {'bits': .., 'group_size': ..}
        return int(best["bits"]), int(best["group_size"])
    bits, group_size = best
    return int(bits), int(group_size)


def apply_precision_map(model, layer_config, default=None, ignore_layers=None, verbose=False):
    """RTN-quantise `model` IN PLACE with a per-layer or per-block precision: what the gradual search's
    RTNWrapper does for one block (bitween/gradual/base_wrapper.py:290-315) and what
    PrecisionOptimizer.finalize leaves behind (bitween/gradual/precision_optimizer.py:1832-1858), given the
    finished {name: (bits, group_size)} map instead of the search.  Layers without an entry keep `default`
    (None = stay nn.Linear).  Returns the model."""
    ignore = set(ignore_layers) if ignore_layers else set()
    targets = [(name, module) for name, module in model.named_modules() if isinstance(module, nn.Linear)]
    for name, module in targets:
        if name in ignore:
            continue
        precision = _precision_for(name, layer_config, default)
        if precision is None:
            continue
        if verbose:
            print(f"  - Quantizing layer: {name} ({precision[0]}-bit, group_size={precision[1]})")
        _set_module(model, name, QuantizedLinear.from_float(module, precision[0], precision[1]))
    return model


class Bitween:
    def __init__(self, model, tokenizer=None, bits=8, group_size=32, iters=1, lr=0.005, enable_minmax_tuning=True,
                 seqlen=2048, cache_to_disk=False, max_memory_mb=512, ignore_layers=None, batch_size=32):
        self.model = model
        self.tokenizer = tokenizer
        self.bits = bits
        self.group_size = group_size
        self.iters = iters
        self.lr = lr
        self.enable_minmax_tuning = enable_minmax_tuning
        self.seqlen = seqlen
        self.cache_to_disk = cache_to_disk
        self.max_memory_mb = max_memory_mb
        self.ignore_layers = set(ignore_layers) if ignore_layers else set()
        self.batch_size = batch_size
        assert group_size > 0, "Group size must be greater than 0."

    def quantize(self, evaluate_perplexity=False, eval_samples=100, rtn=False, trainable=False, calib_dataset="pile-10k",
                 nsamples=None, cache_to_disk=None, max_memory_mb=None, ignore_layers=None, batch_size=None,
                 verbose=True, layer_config=None, fuse_siblings=False, **eval_kwargs):
        """Returns a deep copy of the model with its linear layers RTN-quantised.  As in the reference,
        trainable=False selects RTN whatever `rtn` says (quantizer.py:67).  `layer_config` (not in the
        reference's signature) overrides bits / group_size per layer or block, see apply_precision_map;
        `fuse_siblings=True` (also not in the reference) groups q/k/v and gate/up children so that they share
        one launch, see modules.fuse_sibling_linears."""
        if trainable:
            raise NotImplementedError("trainable quantisation is outside this package (RTN only)")
        if evaluate_perplexity and self.tokenizer is not None and eval_samples > 0:
            raise NotImplementedError("perplexity / KL evaluation needs the reference's dataset pipeline")
        saved_ignore = self.ignore_layers
        if ignore_layers is not None:
            self.ignore_layers = set(ignore_layers)
        if batch_size is not None:
            self.batch_size = batch_size
        try:
            # The reference deep-copies the model and then replaces the copies of the linear layers
            # (quantizer.py:69-80).  Same result without ever copying the weights that are about to be replaced:
            # quantise from the original layers and hand deepcopy the replacements through its memo.
            memo = {}
            targets = [(name, module) for name, module in self.model.named_modules() if isinstance(module, nn.Linear)]
            for name, module in targets:
                if name in self.ignore_layers:
                    if verbose:
                        print(f"  - Skipping ignored layer: {name}")
                    continue
                if verbose:
                    print(f"  - Quantizing layer: {name}")
                bits, group_size = _precision_for(name, layer_config or {}, (self.bits, self.group_size))
                memo[id(module)] = QuantizedLinear.from_float(module, bits, group_size)
            quantized_model = copy.deepcopy(self.model, memo)
            if fuse_siblings:
                fuse_sibling_linears(quantized_model)
            if verbose:
                print("--- Quantization complete ---")
        finally:
            self.ignore_layers = saved_ignore
        return quantized_model
