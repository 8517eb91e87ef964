"""The quantiser against torch's own arithmetic.

bitween/functional.py:22-29 is a sequence of eager torch ops; torch (un-vendored, unpinned by the reference) is
what defines their rounding.  This file runs that sequence, written out below, in torch itself - on the CPU and on
the device - and compares scale, zero point and packed values bit for bit with the HIP kernel in the matching mode:
  * on the CPU the division of a tensor by the Python scalar Qmax is a true IEEE division  -> mode "ieee";
  * on a GPU torch multiplies by the float32 reciprocal of a scalar divisor                -> mode "torch_device".
The package's default mode, "auto", picks between the two by the device of the tensor it is handed, so that the same
call on the same tensor gives what the reference's call gives: the `default_scale_division` tests check that, for
quantize_rtn and for QuantizedLinear.from_float, with nothing set.
Groups whose scale rounds to zero in a 16-bit type divide by zero in the reference and are left out."""
import numpy as np
import pytest
import torch

from oracle import rtn_oracle as orc

pytestmark = pytest.mark.gpu


def eager_rtn(weight, bits, group_size):
    """The arithmetic of quantize_rtn up to q, op for op (amin / amax, sub, div by Qmax, clamp, neg, div, round,
    clamp, div, add of the int32 zero point, round, clamp)."""
    qmax = (1 << bits) - 1
    n, k = weight.shape
    w = weight.contiguous().view(n, k // group_size, group_size)
    w_min = w.amin(dim=-1, keepdim=True)
    w_max = w.amax(dim=-1, keepdim=True)
    scale = ((w_max - w_min) / qmax).clamp(min=1e-8)
    zero_point = torch.round(-w_min / scale).clamp(0, qmax).to(torch.int32)
    q = torch.round(w / scale + zero_point).clamp(0, qmax).to(torch.int32)
    return q.view(n, k), scale.squeeze(-1), zero_point.squeeze(-1)


def _bits(t):
    t = t.contiguous().cpu()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype is torch.float64:
        return t.view(torch.int64).numpy().view(np.uint64)
    return t.view(torch.int32).numpy().view(np.uint32)


def _weights(dtype, outliers, seed):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(384, 1024, generator=g, dtype=torch.float64 if dtype is torch.float64 else torch.float32) * 0.02
    if outliers:
        w = torch.where(torch.rand(384, 1024, generator=g) < 0.001, w * 10, w)
    return w.to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.float64])
@pytest.mark.parametrize("bits,group", [(2, 32), (4, 128), (4, 64), (8, 128)])
@pytest.mark.parametrize("where,mode", [("cpu", "ieee"), ("cuda", "torch_device")])
def test_kernel_matches_eager_torch(dtype, bits, group, where, mode):
    import bitween_amd
    w = _weights(dtype, outliers=bits != 4, seed=bits * 100 + group)
    q_t, s_t, z_t = eager_rtn(w.to(where), bits, group)
    previous = bitween_amd.set_scale_division(mode)
    try:
        qw, s, z, _ = bitween_amd.quantize_rtn(w.cuda(), bits, group)
    finally:
        bitween_amd.set_scale_division(previous)
    valid = (s_t.float() != 0).cpu().numpy()
    assert valid.mean() > 0.99
    assert np.array_equal(_bits(s)[valid], _bits(s_t)[valid])
    assert np.array_equal(z.cpu().numpy()[valid], z_t.cpu().numpy()[valid])
    q = orc.unpack_words(qw.cpu().numpy(), bits)
    vq = np.repeat(valid, group, axis=1)
    assert np.array_equal(q[vq], q_t.cpu().numpy()[vq])


def test_the_two_modes_are_not_the_same_function():
    """On float32 weights torch's CPU and device results differ in most scales (one ulp): the mode matters."""
    w = _weights(torch.float32, False, 1)
    _, s_c, _ = eager_rtn(w, 4, 128)
    _, s_d, _ = eager_rtn(w.cuda(), 4, 128)
    assert (_bits(s_c) != _bits(s_d)).mean() > 0.3


@pytest.mark.default_scale_division
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.float64])
@pytest.mark.parametrize("bits,group", [(2, 32), (4, 128), (8, 128)])
@pytest.mark.parametrize("where", ["cpu", "cuda"])
def test_default_mode_follows_the_device_of_the_tensor(dtype, bits, group, where):
    """quantize_rtn with the default mode on a tensor on `where` against eager torch on that very device."""
    import bitween_amd
    assert bitween_amd.get_scale_division() == "auto"
    w = _weights(dtype, outliers=bits != 4, seed=bits * 100 + group + 7).to(where)
    q_t, s_t, z_t = eager_rtn(w, bits, group)
    qw, s, z, _ = bitween_amd.quantize_rtn(w, bits, group)
    assert qw.device == w.device and s.device == w.device and z.device == w.device
    valid = (s_t.float() != 0).cpu().numpy()
    assert valid.mean() > 0.99
    assert np.array_equal(_bits(s)[valid], _bits(s_t)[valid])
    assert np.array_equal(z.cpu().numpy()[valid], z_t.cpu().numpy()[valid])
    q = orc.unpack_words(qw.cpu().numpy(), bits)
    vq = np.repeat(valid, group, axis=1)
    assert np.array_equal(q[vq], q_t.cpu().numpy()[vq])


@pytest.mark.default_scale_division
@pytest.mark.parametrize("bits,group", [(2, 32), (4, 128), (8, 128)])
@pytest.mark.parametrize("where", ["cpu", "cuda"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_from_float_default_mode_follows_the_layer(dtype, bits, group, where):
    """QuantizedLinear.from_float with nothing set, on a layer living on `where`: the reference upcasts the layer to
    float32 on its own device, runs the eager sequence there and stores scale / zero point as float16
    (bitween/modules.py:189-213)."""
    import bitween_amd
    assert bitween_amd.get_scale_division() == "auto"
    w = _weights(dtype, outliers=True, seed=bits + group)
    lin = torch.nn.Linear(w.shape[1], w.shape[0], bias=False)
    lin.weight.data = w.clone()
    lin = lin.to(where)
    q_t, s_t, z_t = eager_rtn(lin.weight.data.to(torch.float32), bits, group)
    layer = bitween_amd.QuantizedLinear.from_float(lin, bits, group)
    assert layer.qweight.device == lin.weight.device
    assert np.array_equal(_bits(layer.scale), _bits(s_t.to(torch.float16)))
    assert np.array_equal(_bits(layer.zero_point), _bits(z_t.to(torch.float16)))
    assert np.array_equal(orc.unpack_words(layer.qweight.cpu().numpy(), bits), q_t.cpu().numpy())
