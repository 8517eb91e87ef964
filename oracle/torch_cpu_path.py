"""The reference's CPU path, restated in eager torch ops (TEST INFRASTRUCTURE: checker and timed CPU baseline).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may use this module; nothing in the
shipped package imports it.  It exists because the reference's own files do not travel to the GPU box: this
is the same sequence of eager torch operations, written out from the reference lines cited per function
(paths relative to the reference checkout), so that timing it on the box's host cores times what the
reference would execute there:

    quantize_rtn     bitween/functional.py:3-45
    dequantize_rtn   bitween/functional.py:47-71
    module_buffers   bitween/modules.py:191,207-209   (float32 upcast, float16 stores)
    forward          main.py:462-466                  (dequantize -> .half() -> matmul (+ bias))

Pinned by tests/test_oracle_pins.py::test_torch_cpu_path_matches_exact_vectors (every output bit for bit
against the exact-rational vectors; the matmul against their exactly evaluated products).
"""
import torch


@torch.no_grad()
def quantize_rtn(weight, bits=8, group_size=32):
    """functional.py:3-45: per-group min / max, scale = (max - min) / Qmax clamped at 1e-8, zero point =
    round(-min / scale), q = round(w / scale + zp), all clamped to [0, Qmax]; values packed little-endian
    into int32 words by strided slices."""
    weight = weight.contiguous()
    assert bits in [2, 4, 8], "Only 2, 4, or 8-bit quantization supported."
    qmax = (1 << bits) - 1
    out_features, in_features = weight.shape
    pad = (group_size - in_features % group_size) % group_size
    if pad > 0:
        raise ValueError(f"Padding {pad} columns to {in_features} to make it a multiple of {group_size}")
    groups = in_features // group_size
    w = weight.view(out_features, groups, group_size)
    lo = w.amin(dim=-1, keepdim=True)
    hi = w.amax(dim=-1, keepdim=True)
    scale = ((hi - lo) / qmax).clamp(min=1e-8)
    zero_point = torch.round(-lo / scale).clamp(0, qmax).to(torch.int32)
    q = torch.round(w / scale + zero_point).clamp(0, qmax).to(torch.int32)
    vpi = 32 // bits
    flat = q.reshape(-1)
    packed = torch.zeros(flat.numel() // vpi, dtype=torch.int32, device=weight.device)
    for i in range(vpi):
        packed |= flat[i::vpi] << (i * bits)
    return packed.view(out_features, in_features // vpi), scale.squeeze(-1), zero_point.squeeze(-1), group_size


@torch.no_grad()
def dequantize_rtn(q_packed, scale, zero_point, group_size, bits=8):
    """functional.py:47-71: unpack by strided scatters, then scale * (q.float() - zero_point.float())."""
    assert bits in [2, 4, 8], "Only 2, 4, or 8-bit quantization supported."
    vpi = 32 // bits
    out_features, words = q_packed.shape
    groups = (words * vpi) // group_size
    flat = torch.empty(out_features * groups * group_size, dtype=torch.int32, device=q_packed.device)
    mask = (1 << bits) - 1
    for i in range(vpi):
        flat[i::vpi] = (q_packed.view(-1) >> (i * bits)) & mask
    q = flat.view(out_features, groups, group_size)
    w = scale.view(out_features, groups, 1) * (q.float() - zero_point.view(out_features, groups, 1).float())
    return w.view(out_features, groups * group_size)


@torch.no_grad()
def module_buffers(weight16, bits, group_size):
    """QuantizedLinear.from_float, modules.py:191-211: upcast the layer to float32, quantise, keep scale and zero
    point as float16."""
    qw, scale, zp, _ = quantize_rtn(weight16.float(), bits, group_size)
    return qw, scale.to(torch.float16), zp.to(torch.float16)


@torch.no_grad()
def forward(x16, qweight, scale16, zp16, bias16, bits, group_size):
    """main.py:462-466 / modules.py:85-101: dequantise to float16 weights, matmul, separate bias add."""
    w16 = dequantize_rtn(qweight, scale16, zp16, group_size, bits).half()
    y = torch.matmul(x16, w16.T)
    if bias16 is not None:
        y = y + bias16
    return y
