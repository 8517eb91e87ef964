"""QuantizedLinear and its autograd function with the reference's interface
(bitween/modules.py:60-217): same constructor, buffers (qweight int32,
scale / zero_point / bias float16), from_float, forward and repr.  The
forward is one fused dequantise+matmul HIP kernel instead of the reference's
dequantise-to-HBM, BLAS matmul and bias add.
"""
import weakref

import torch
import torch.nn as nn

from . import functional as _functional
from .kernels import hip_loader as _hip


FUSED_DGRAD_MAX_ROWS = 512       # measured on MI355X, Llama-shaped layers: the 128-row fused kernel wins up to here (3x at 128 rows)
FUSED_DGRAD_LARGE_MAX_ROWS = 2048  # ... and the 256 x 256 kernel, where the library plans it (large layers), up to here


class QuantizedLinearFunction(torch.autograd.Function):
    """apply(x, qweight, scale, zero_point, bias, bits, group_size) -> float16 [..., N]
    (bitween/modules.py:62-106).  backward returns grad_input only
    (bitween/modules.py:108-141)."""

    @staticmethod
    def forward(ctx, x, qweight, scale, zero_point, bias, bits, group_size):
        ctx.save_for_backward(x, qweight, scale, zero_point, bias)
        ctx.bits = bits
        ctx.group_size = group_size
        original_shape = x.shape
        x2 = x.reshape(-1, original_shape[-1]).to(torch.float16)
        n = qweight.shape[0]
        y = _hip.quantized_matmul_hip(x2, qweight, scale, zero_point, bias, bits, group_size)
        return y.reshape(*original_shape[:-1], n)

    @staticmethod
    def backward(ctx, grad_output):
        x, qweight, scale, zero_point, bias = ctx.saved_tensors
        grad_input = None
        if ctx.needs_input_grad[0]:
            # float16 / bfloat16 gradients: one fused kernel, the weights are never materialised - up to
            # FUSED_DGRAD_MAX_ROWS rows always, up to FUSED_DGRAD_LARGE_MAX_ROWS where the library runs its 256 x 256
            # kernel (large layers); otherwise the library GEMM on dequantised weights is faster.
            go2 = grad_output.reshape(-1, grad_output.shape[-1])
            if grad_output.dtype in (torch.float16, torch.bfloat16) and grad_output.is_cuda and _hip.input_grad_prefers_fused(
                    go2.shape[0], qweight.shape[0], x.shape[-1], ctx.bits, ctx.group_size, FUSED_DGRAD_MAX_ROWS, FUSED_DGRAD_LARGE_MAX_ROWS):
                gx = _hip.quantized_input_grad(go2, qweight, scale, zero_point, ctx.bits, ctx.group_size)
                if gx is not None:
                    return gx.view(*grad_output.shape[:-1], gx.shape[-1]), None, None, None, None, None, None
            # W = scale * (q - zp) in float32, cast to grad_output.dtype: the float32 product is exact,
            # so dequantising straight to that dtype gives the same bits.
            gdt = grad_output.dtype if grad_output.dtype in (torch.float16, torch.bfloat16, torch.float32) else torch.float32
            weight = _hip.dequantize(qweight, scale, zero_point, ctx.group_size, ctx.bits, gdt)
            grad_input = grad_output @ weight.to(grad_output.dtype)
        return grad_input, None, None, None, None, None, None


class BitweenShapeError(RuntimeError):
    pass


class QuantizedLinear(nn.Module):
    """Linear layer holding 2/4/8-bit group-quantised weights."""

    def __init__(self, in_features, out_features, bits=8, group_size=32, bias=True, dtype=torch.float16):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.bits = bits
        self.group_size = group_size
        self.requires_grad = False
        if self.bits not in [2, 4, 8]:
            raise ValueError("Only 2, 4, or 8 bits are supported.")
        if group_size < 1:
            raise ValueError("Group size must be at least 1.")
        self.dtype = torch.float16          # the reference forces float16 whatever is asked (modules.py:167)
        values_per_int32 = 32 // self.bits
        self.register_buffer("qweight", torch.zeros((out_features, in_features // values_per_int32), dtype=torch.int32))
        meta_shape = (out_features, in_features // group_size)
        self.register_buffer("scale", torch.zeros(meta_shape, dtype=self.dtype))
        self.register_buffer("zero_point", torch.zeros(meta_shape, dtype=self.dtype))
        if bias:
            self.register_buffer("bias", torch.zeros(out_features, dtype=self.dtype))
        else:
            self.bias = None

    def forward(self, x):
        if x.requires_grad and torch.is_grad_enabled():
            return QuantizedLinearFunction.apply(x, self.qweight, self.scale, self.zero_point, self.bias, self.bits,
                                                 self.group_size)
        group = self.__dict__.get("_sibling_group")
        if group is not None:
            y = group.forward(self, x)
            if y is not None:
                return y
        # nothing to differentiate (the buffers never require grad): same arithmetic without the autograd node
        shape = x.shape
        x2 = x.reshape(-1, shape[-1])
        m = x2.shape[0]
        if 0 < m <= 48:
            # decode: the buffers were validated once; they are looked at again only when one of them has been
            # replaced (module.to(), load with assign, sibling fusion) or moved
            plan = self.__dict__.get("_decode_plan")
            b = self._buffers
            if plan is None or plan[0] is not b["qweight"] or plan[1] is not b["scale"] or \
                    plan[2] is not b["zero_point"] or plan[3] is not b.get("bias") or plan[4] != plan[0].data_ptr() or \
                    plan[5] != plan[1].data_ptr() or plan[6] != plan[2].data_ptr() or \
                    (plan[3] is not None and plan[7] != plan[3].data_ptr()):
                plan = _hip.make_decode_plan(b["qweight"], b["scale"], b["zero_point"], b.get("bias"), self.bits,
                                             self.group_size) if b["qweight"].is_cuda else None
                self.__dict__["_decode_plan"] = plan
            if plan is not None:
                y = _hip.decode_with_plan(plan, x2, m)
                if y is not None:
                    return y.view(*shape[:-1], self.out_features)
        if x2.dtype is not torch.float16 and x2.dtype is not torch.bfloat16:    # bfloat16 is converted by the kernel
            x2 = x2.to(torch.float16)
        y = _hip.quantized_matmul_hip(x2, self.qweight, self.scale, self.zero_point, self.bias, self.bits, self.group_size)
        return y.view(*shape[:-1], self.out_features)

    def __getstate__(self):                                # the validated-buffers cache holds device addresses
        state = self.__dict__.copy()
        state.pop("_decode_plan", None)
        return state

    @classmethod
    def from_float(cls, float_layer: nn.Linear, bits=8, group_size=32):
        """RTN-quantise an nn.Linear.  The reference upcasts the layer to float32, quantises, and stores
        scale / zero_point as float16 (modules.py:189-213); here the upcast, the quantiser and the stores
        are one kernel reading the layer's own dtype."""
        if bits not in [2, 4, 8]:
            raise AssertionError("Only 2, 4, or 8-bit quantization supported.")
        weight = float_layer.weight.data
        if weight.shape[1] % group_size:
            pad = group_size - weight.shape[1] % group_size
            raise ValueError(f"Padding {pad} columns to {weight.shape[1]} to make it a multiple of {group_size}")
        device = weight.device
        if weight.dtype not in (torch.float16, torch.bfloat16, torch.float32):
            weight = weight.to(torch.float32)
        if not weight.is_cuda:
            if not torch.cuda.is_available():
                raise _hip.BitweenHipError("QuantizedLinear.from_float needs a ROCm GPU (no CPU implementation)")
            weight = weight.to("cuda")
        qweight, scale, zero_point = _hip.quantize_pack(weight, bits, group_size, math_dtype=torch.float32,
                                                        scale_dtype=torch.float16, zp_dtype=torch.float16,
                                                        scale_reciprocal=_functional.scale_reciprocal_for(float_layer.weight))
        # the constructor's zero buffers are built on the meta device (no memory, no host-to-device copy) and
        # replaced by the kernel's outputs, which already have the buffers' shapes and dtypes
        with torch.device("meta"):
            q_layer = cls(float_layer.in_features, float_layer.out_features, bits, group_size,
                          bias=float_layer.bias is not None, dtype=torch.float16)
        new = {"qweight": qweight, "scale": scale, "zero_point": zero_point}
        if float_layer.bias is not None:
            new["bias"] = float_layer.bias.data.to(device="cuda", dtype=torch.float16, copy=True)
        for name, value in new.items():
            if value.shape != q_layer._buffers[name].shape or value.dtype != q_layer._buffers[name].dtype:
                raise BitweenShapeError(f"{name}: kernel produced {tuple(value.shape)} {value.dtype}, the module "
                                        f"declares {tuple(q_layer._buffers[name].shape)} {q_layer._buffers[name].dtype}")
            q_layer._buffers[name] = value if device.type == "cuda" else value.to(device)
        return q_layer

    def __repr__(self):
        return (f"QuantizedLinear(in_features={self.in_features}, out_features={self.out_features}, "
                f"bias={self.bias is not None}, bits={self.bits}, group_size={self.group_size})")


class _SiblingGroup:
    """Linears that read the same input (q/k/v, gate/up) as one launch.

    The members' buffers are re-pointed at row slices of concatenated tensors (names, shapes and values are
    unchanged, so state_dict and stand-alone use are unaffected).  The first member called with an input
    tensor runs one kernel over the concatenated weights; a sibling called next with the very same tensor
    (same object, same version counter) gets its slice of that result.  Anything unexpected - grad mode, a
    member whose buffers were moved or replaced since - falls back to the member's own forward."""

    def __init__(self, members):
        first = members[0]
        for m in members:
            if (m.in_features, m.bits, m.group_size) != (first.in_features, first.bits, first.group_size):
                raise ValueError("sibling linears must share in_features, bits and group_size")
            if (m.bias is None) != (first.bias is None) or m.qweight.device != first.qweight.device:
                raise ValueError("sibling linears must all have a bias or none, and live on one device")
        self.bits, self.group_size = first.bits, first.group_size
        self.qweight = torch.cat([m.qweight for m in members], 0)
        self.scale = torch.cat([m.scale for m in members], 0)
        self.zero_point = torch.cat([m.zero_point for m in members], 0)
        self.bias = None if first.bias is None else torch.cat([m.bias for m in members], 0)
        self.size = len(members)
        self.wasted = 0                                   # launches in a row that served a single member
        row = 0
        for index, m in enumerate(members):
            a, b = row, row + m.out_features
            m.__dict__["_sibling_rows"] = (a, b)
            m.__dict__["_sibling_index"] = index
            m._buffers["qweight"] = self.qweight[a:b]
            m._buffers["scale"] = self.scale[a:b]
            m._buffers["zero_point"] = self.zero_point[a:b]
            if self.bias is not None:
                m._buffers["bias"] = self.bias[a:b]
            m.__dict__["_sibling_group"] = self
            row = b
        self._x = None
        self._version = -1
        self._y = None
        self._served = 0
        self._served_mask = 0

    def __getstate__(self):                                # copies and pickles drop the one-call cache
        state = dict(self.__dict__)
        state["_x"], state["_version"], state["_y"], state["_served"], state["_served_mask"] = None, -1, None, 0, 0
        return state

    def _views_fused_buffers(self, member, row):
        """Every buffer of `member` still starts at its row of the concatenated tensors (a buffer replaced through
        `.data = ...` or `.set_()` keeps its Python object but not its address)."""
        b = member._buffers
        if b["qweight"].data_ptr() != self.qweight.data_ptr() + row * self.qweight.stride(0) * 4 or \
                b["scale"].data_ptr() != self.scale.data_ptr() + row * self.scale.stride(0) * 2 or \
                b["zero_point"].data_ptr() != self.zero_point.data_ptr() + row * self.zero_point.stride(0) * 2:
            return False
        bias = b.get("bias")
        if (bias is None) != (self.bias is None):
            return False
        return bias is None or bias.data_ptr() == self.bias.data_ptr() + row * 2

    def forward(self, member, x):
        rng = member.__dict__.get("_sibling_rows")
        if rng is None or not self._views_fused_buffers(member, rng[0]):
            return None                                    # the member no longer views the fused buffers
        if self.wasted >= 4:
            return None                                    # the members do not share inputs after all: stop grouping
        seen = self._x() if self._x is not None else None
        bit = 1 << member.__dict__["_sibling_index"]
        # The cached result serves each member once: a member that comes back with the very same tensor object and
        # version (an input rewritten in place through .data or by a kernel writing to its address) gets a new launch.
        if seen is not x or self._version != x._version or self._y is None or self._served_mask & bit:
            self.wasted = self.wasted + 1 if self._served == 1 else 0
            shape = x.shape
            x2 = x.reshape(-1, shape[-1])
            if x2.dtype is not torch.float16 and x2.dtype is not torch.bfloat16:
                x2 = x2.to(torch.float16)
            y = _hip.quantized_matmul_hip(x2, self.qweight, self.scale, self.zero_point, self.bias, self.bits, self.group_size)
            self._y = y.view(*shape[:-1], y.shape[-1])
            self._x = weakref.ref(x)
            self._version = x._version
            self._served = 0
            self._served_mask = 0
        out = self._y[..., rng[0]:rng[1]]
        self._served += 1
        self._served_mask |= bit
        if self._served == self.size:
            self._y = None                                 # everyone has its slice: do not keep the result alive
        return out


def fuse_sibling_linears(model, sibling_names=(("q_proj", "k_proj", "v_proj"), ("gate_proj", "up_proj"))):
    """Make QuantizedLinear children that consume the same input share one launch (decode spends about 2.5 us
    per launch before a byte moves).  For every module of `model` that has all the children named in one
    tuple of `sibling_names` as QuantizedLinear layers of equal in_features / bits / group_size, those
    children are grouped.  The model's code is unchanged: it still calls each child.  Returns the number of
    groups formed.  Not part of the reference's interface.
    A group computes all its members' outputs when the first of them is called with a tensor and hands the others
    their slices when they are called with that same tensor (same object, same version counter); a member that
    asks twice gets a new launch.  An input that is rewritten in place without a version bump (through .data, or
    by a kernel writing to its address) between the calls of two different members is not noticed: change inputs
    through ordinary torch ops."""
    formed = 0
    for parent in list(model.modules()):
        for names in sibling_names:
            kids = [getattr(parent, n, None) for n in names]
            if not all(isinstance(k, QuantizedLinear) for k in kids):
                continue
            if any("_sibling_group" in k.__dict__ for k in kids):
                continue
            try:
                _SiblingGroup(kids)
            except ValueError:
                continue
            formed += 1
    return formed
