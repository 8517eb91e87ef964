"""The decode kernels for 2-16 activation rows that keep a workgroup's requests in flight (several 16-row tiles of
N per workgroup, or rounds of a long K): shapes chosen to reach every variant - 1 to 4 tiles per workgroup, grids
of more workgroups than fit the chip, the last tile partly empty, bias, bfloat16 x, K that is not a multiple of a
wave's slice, the round kernel's straight and ring forms - against the oracle on sampled rows."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import rtn_oracle as orc
from gpu_util import check_matmul, make_weight, to_gpu

pytestmark = pytest.mark.gpu


def _layer_rows(n, k, bits, g, seed, rows):
    """Quantise only the sampled rows on the host (the oracle); the device gets the whole layer from the kernel."""
    import bitween_amd
    gen = torch.Generator(device="cuda").manual_seed(seed)
    w = (torch.randn(n, k, device="cuda", generator=gen) * 0.02).half()
    lin = torch.nn.Linear(k, n, bias=True, device="cuda", dtype=torch.float16)
    lin.weight.data = w
    lin.bias.data = (torch.randn(n, device="cuda", generator=gen) * 0.1).half()
    q = bitween_amd.QuantizedLinear.from_float(lin, bits, g)
    qw_o, s_o, z_o, _ = orc.quantize_rtn(w[rows].float().cpu().numpy(), bits, g)
    s16, z16 = orc.store_module_buffers(s_o, z_o)
    assert np.array_equal(q.qweight[rows].cpu().numpy(), qw_o)
    return q, qw_o, s16, z16, lin.bias.data[rows].cpu().numpy()


def _gemv(q, x, bits, g, bias=True):
    from bitween_amd.kernels import hip_loader as hip
    return hip.quantized_gemv_hip(x, q.qweight, q.scale, q.zero_point, q.bias if bias else None, bits, g)


@pytest.mark.parametrize("bits,g", [(4, 128), (4, 32), (2, 32), (2, 128), (8, 64)])
@pytest.mark.parametrize("n", [16400, 36870, 70002])            # 2, 3 and 4 tiles per workgroup at K = 1024 (4 waves each)
def test_several_tiles_per_workgroup(bits, g, n):
    k = 1024
    rows = np.unique(np.concatenate([np.arange(0, n, n // 30), [15, 16, n - 17, n - 2, n - 1]]))
    q, qw_o, s16, z16, b16 = _layer_rows(n, k, bits, g, seed=bits + g + n, rows=rows)
    for m in (2, 3, 4, 7, 8, 13, 16):
        x = torch.randn(m, k, device="cuda", dtype=torch.float16)
        y = _gemv(q, x, bits, g)
        check_matmul(y[:, rows], x.cpu().numpy(), qw_o, s16, z16, b16, bits, g)
    xb = torch.randn(5, k, device="cuda").to(torch.bfloat16)
    y = _gemv(q, xb, bits, g)
    check_matmul(y[:, rows], xb.to(torch.float16).cpu().numpy(), qw_o, s16, z16, b16, bits, g)


@pytest.mark.parametrize("bits,g,k", [(4, 128, 4096), (4, 64, 2944), (2, 32, 4096), (2, 64, 3840), (8, 128, 4096), (4, 32, 896)])
@pytest.mark.parametrize("n", [4096, 11008, 5000])
def test_one_round_shapes_with_and_without_bias(bits, g, k, n):
    rows = np.unique(np.concatenate([np.arange(0, n, n // 24), [n - 1]]))
    q, qw_o, s16, z16, b16 = _layer_rows(n, k, bits, g, seed=k + n + bits, rows=rows)
    for m in (3, 6, 11, 16):
        x = torch.randn(m, k, device="cuda", dtype=torch.float16)
        check_matmul(_gemv(q, x, bits, g)[:, rows], x.cpu().numpy(), qw_o, s16, z16, b16, bits, g)
        check_matmul(_gemv(q, x, bits, g, bias=False)[:, rows], x.cpu().numpy(), qw_o, s16, z16, None, bits, g)


@pytest.mark.parametrize("bits,g,k", [(2, 32, 11008), (2, 32, 8192), (2, 128, 14336), (2, 64, 28672), (4, 32, 11008), (4, 32, 16384)])
def test_rounds_of_a_long_k(bits, g, k):
    """2, 3 and more rounds (the ring form where the registers allow it)."""
    n = 1040
    rows = np.arange(0, n, 13)
    q, qw_o, s16, z16, b16 = _layer_rows(n, k, bits, g, seed=k + bits, rows=rows)
    for m in (1, 2, 3, 4, 8, 9, 16):
        x = torch.randn(m, k, device="cuda", dtype=torch.float16)
        check_matmul(_gemv(q, x, bits, g)[:, rows], x.cpu().numpy(), qw_o, s16, z16, b16, bits, g)


def test_one_hot_rows_return_w16_columns_through_the_tile_kernels():
    from bitween_amd.kernels import hip_loader as hip
    for bits, g, k, n in ((4, 128, 4096, 11008), (2, 32, 4096, 11008), (4, 32, 2048, 20000), (2, 32, 11008, 2048)):
        rows = np.arange(0, n, 97)
        q, *_ = _layer_rows(n, k, bits, g, seed=9, rows=rows)
        w16 = hip.dequantize(q.qweight, q.scale, q.zero_point, g, bits, torch.float16)
        for m in (3, 8, 16):
            cols = [0, 5, k // 2 + 1, k - 1][:min(4, m)]
            x = torch.zeros(m, k, device="cuda", dtype=torch.float16)
            for i, c in enumerate(cols):
                x[m - 1 - i, c] = 1.0
            y = _gemv(q, x, bits, g, bias=False)
            for i, c in enumerate(cols):
                assert torch.equal(y[m - 1 - i], w16[:, c])
            assert (y[: m - len(cols)] == 0).all()


def test_layouts_the_tile_kernels_do_not_take_fall_back():
    """An odd number of groups per row, scale arrays at 2-byte alignment, an odd N with a bias: the earlier kernels run."""
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for bits, g, k, n, off in ((4, 128, 128 * 13, 301, 0), (4, 128, 4096, 4096, 1), (2, 32, 4096, 333, 0)):
        w = make_weight(n, k, seed=n)
        qw, s, z, _ = orc.quantize_rtn(w, bits, g)
        s16, z16 = orc.store_module_buffers(s, z)
        b16 = (np.random.default_rng(1).standard_normal(n) * 0.1).astype(np.float16)
        x = np.random.default_rng(2).standard_normal((9, k)).astype(np.float16)
        sbuf = torch.zeros(s16.size + off, dtype=torch.float16, device="cuda")
        zbuf = torch.zeros(s16.size + off, dtype=torch.float16, device="cuda")
        sbuf[off:] = to_gpu(s16).reshape(-1)
        zbuf[off:] = to_gpu(z16).reshape(-1)
        xg, qg, bg = to_gpu(x), to_gpu(qw), to_gpu(b16)
        y = torch.empty((9, n), dtype=torch.float16, device="cuda")
        st = lib.bw_qgemv(xg.data_ptr(), 0, 9, k, k, qg.data_ptr(), sbuf.data_ptr() + 2 * off, zbuf.data_ptr() + 2 * off,
                          bg.data_ptr(), n, bits, g, y.data_ptr(), n, stream)
        assert st == 0
        torch.cuda.synchronize()
        check_matmul(y, x, qw, s16, z16, b16, bits, g)
