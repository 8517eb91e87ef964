"""quantize_rtn / dequantize_rtn with the reference's signatures
(bitween/functional.py:4,48), executed by the HIP kernels of
libbitween_hip.so.  Tensors that live on the CPU are staged through the GPU
and the results returned on the input's device; without a GPU these
functions raise (there is no CPU implementation in this package).
"""
import os

import torch

from .kernels import hip_loader as _hip


# How `(w_max - w_min) / Qmax` (bitween/functional.py:25) is rounded.  Eager torch divides a tensor by a Python
# scalar exactly on the CPU and multiplies by the float32 reciprocal on a GPU; the two differ in the last bit of
# most float32 scales.  "auto" (default) follows the device of the tensor being quantised, which is what the
# reference's own call yields: a CPU tensor gets the true division, a GPU tensor the reciprocal.  "ieee" forces
# the CPU arithmetic (the source as written), "torch_device" the GPU's, wherever the tensor lives.
# BITWEEN_SCALE_DIVISION sets the initial choice.
_SCALE_DIVISIONS = ("auto", "ieee", "torch_device")
_scale_division = os.environ.get("BITWEEN_SCALE_DIVISION", "auto")
if _scale_division not in _SCALE_DIVISIONS:
    raise ValueError(f"BITWEEN_SCALE_DIVISION must be one of {_SCALE_DIVISIONS}, got {_scale_division!r}")


def set_scale_division(mode: str) -> str:
    """Choose the rounding of the scale division for quantize_rtn and QuantizedLinear.from_float: "auto" (follow the
    tensor's device), "ieee" or "torch_device".  Returns the previous choice."""
    global _scale_division
    if mode not in _SCALE_DIVISIONS:
        raise ValueError(f"scale division must be one of {_SCALE_DIVISIONS}, got {mode!r}")
    previous, _scale_division = _scale_division, mode
    return previous


def get_scale_division() -> str:
    return _scale_division


def scale_reciprocal_for(tensor, mode=None) -> bool:
    """True when the scale of `tensor` is to be formed as (max - min) * fl(1 / Qmax): the current mode (or `mode`)
    says "torch_device", or it says "auto" and the tensor lives on a GPU - where the reference's eager division by
    a Python scalar is that multiplication."""
    mode = _scale_division if mode is None else mode
    if mode not in _SCALE_DIVISIONS:
        raise ValueError(f"scale division must be one of {_SCALE_DIVISIONS}, got {mode!r}")
    return mode == "torch_device" or (mode == "auto" and tensor.is_cuda)


def _gpu_for(t):
    if t.is_cuda:
        return t.device
    if not torch.cuda.is_available():
        raise _hip.BitweenHipError("bitween_amd needs a ROCm GPU: there is no CPU implementation of this operator")
    return torch.device("cuda", torch.cuda.current_device())


@torch.no_grad()
def quantize_rtn_perturbed(weight: torch.Tensor, value: torch.Tensor, bits: int = 8, group_size: int = 32):
    """quantize_rtn(weight + value, bits, group_size) in one kernel: the hand-off of a tuned layer to its
    inference form (WrapperLinear.to_quantized_linear, bitween/wrapper.py:222-232).  `value` must have the
    shape and dtype of `weight`; the sum is rounded once to that dtype, as the eager add is."""
    return _quantize(weight, bits, group_size, value)


@torch.no_grad()
def quantize_rtn(weight: torch.Tensor, bits: int = 8, group_size: int = 32):
    """Round-to-nearest asymmetric per-group quantisation and packing.

    Returns (q_packed int32 [N, K*bits/32], scale [N, K/group_size] in
    weight.dtype, zero_point int32 [N, K/group_size], group_size) - the tuple
    of bitween/functional.py:45.  Arithmetic is carried out in weight.dtype,
    as the reference's eager ops do.
    """
    return _quantize(weight, bits, group_size, None)


def _quantize(weight, bits, group_size, value):
    assert bits in [2, 4, 8], "Only 2, 4, or 8-bit quantization supported."
    if weight.dim() != 2:
        raise ValueError("weight must be [out_features, in_features]")
    out_features, in_features = weight.shape
    pad = (group_size - in_features % group_size) % group_size
    if pad > 0:
        raise ValueError(f"Padding {pad} columns to {in_features} to make it a multiple of {group_size}")
    if in_features % (32 // bits):
        raise ValueError(f"in_features={in_features} does not fill whole int32 words at {bits} bits")
    if weight.dtype not in (torch.float32, torch.float16, torch.bfloat16, torch.float64):
        raise NotImplementedError(f"quantize_rtn: weight dtype {weight.dtype} is not supported")
    dev = _gpu_for(weight)
    w = weight.to(dev)
    qweight, scale, zp = _hip.quantize_pack(w, bits, group_size, math_dtype=weight.dtype, scale_dtype=weight.dtype,
                                            zp_dtype=torch.int32, delta=None if value is None else value.to(dev),
                                            scale_reciprocal=scale_reciprocal_for(weight))
    if not weight.is_cuda:
        qweight, scale, zp = qweight.to(weight.device), scale.to(weight.device), zp.to(weight.device)
    return qweight, scale, zp, group_size


@torch.no_grad()
def dequantize_rtn(q_packed: torch.Tensor, scale: torch.Tensor, zero_point: torch.Tensor, group_size: int,
                   bits: int = 8):
    """scale * (q - zero_point) as float32 [N, K] (bitween/functional.py:47-71); float64 for a float64 scale, as
    the reference's product promotes."""
    assert bits in [2, 4, 8], "Only 2, 4, or 8-bit quantization supported."
    dev = _gpu_for(q_packed)
    s = scale.to(dev)
    z = zero_point.to(dev)
    if s.dtype == torch.bfloat16:
        s = s.float()                       # exact widening; the product is float32 either way
    if z.dtype not in (torch.int32, torch.float16):
        z = z.to(torch.int32) if not z.is_floating_point() else z.float().to(torch.int32)
    n = q_packed.shape[0]
    out_dtype = torch.float64 if s.dtype == torch.float64 else torch.float32
    out = _hip.dequantize(q_packed.to(dev), s.reshape(n, -1), z.reshape(n, -1), group_size, bits, out_dtype)
    return out if q_packed.is_cuda else out.to(q_packed.device)
