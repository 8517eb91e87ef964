"""Seeded sweep over ragged shapes: N that is not a multiple of the 16-row tile, K that ends inside a chunk,
every M from 1 to past the decode / prefill switch, padded activation rows, bias on and off.  Each case goes
through the C ABI (bw_qlinear picks the kernel) and is checked against the oracle."""
import ctypes

import numpy as np
import pytest
import torch

from gpu_util import check_matmul, quantized_layer, to_gpu
from oracle import rtn_oracle as orc

pytestmark = pytest.mark.gpu


def _cases():
    rng = np.random.default_rng(2024)
    out = []
    for i in range(48):
        bits = int(rng.choice([2, 4, 8]))
        g = int(rng.choice([32, 64, 128]))
        k = g * int(rng.integers(1, 20))
        n = int(rng.integers(1, 200))
        m = int(rng.choice([1, 2, 3, 4, 5, 8, 9, 15, 16, 17, 31, 33, 64, 129]))
        pad = int(rng.choice([0, 0, 8, 24]))
        out.append((i, bits, g, k, n, m, pad, bool(rng.integers(0, 2))))
    return out


@pytest.mark.parametrize("case", _cases(), ids=lambda c: "b%d_g%d_K%d_N%d_M%d_pad%d_%s" % (c[1:7] + ("bias" if c[7] else "nobias",)))
def test_ragged_shapes_through_the_abi(case):
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    i, bits, g, k, n, m, pad, use_bias = case
    _, qw, s16, z16, b16 = quantized_layer(n, k, bits, g, seed=900 + i, outliers=True)
    x = np.random.default_rng(i).standard_normal((m, k)).astype(np.float16)
    ldx = k + pad
    xbuf = torch.full((m, ldx), float("nan"), dtype=torch.float16, device="cuda")      # the padding must never be read
    xbuf[:, :k] = to_gpu(x)
    d = [to_gpu(a) for a in (qw, s16, z16, b16)]
    ldy = n + 3
    y = torch.full((m, ldy), 7.0, dtype=torch.float16, device="cuda")
    st = lib.bw_qlinear(xbuf.data_ptr(), 0, m, k, ldx, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(),
                        d[3].data_ptr() if use_bias else None, n, bits, g, y.data_ptr(), ldy,
                        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert st == 0
    torch.cuda.synchronize()
    assert (y[:, n:] == 7.0).all()                        # nothing written past a row's N outputs
    check_matmul(y[:, :n], x, qw, s16, z16, b16 if use_bias else None, bits, g)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("groups,offset", [(12, 0), (12, 1), (13, 0), (14, 2), (14, 3), (43, 0)])
def test_prefill_scale_rows_at_every_alignment(bits, groups, offset):
    """The 128-group prefill kernel fetches the scales of four K steps in one request when a row of scales
    starts on a 4-byte boundary; an odd number of groups or a base address off by one element must take the
    per-step requests and give the same result.  K steps that are not a multiple of four end in a short run."""
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    g, n, m = 128, 300, 192
    k = g * groups
    _, qw, s16, z16, _ = quantized_layer(n, k, bits, g, seed=77 + groups, outliers=True)
    x = np.random.default_rng(groups).standard_normal((m, k)).astype(np.float16)
    sbuf = torch.zeros(n * groups + offset, dtype=torch.float16, device="cuda")
    zbuf = torch.zeros(n * groups + offset, dtype=torch.float16, device="cuda")
    sbuf[offset:] = to_gpu(s16).reshape(-1)
    zbuf[offset:] = to_gpu(z16).reshape(-1)
    xg, qg = to_gpu(x), to_gpu(qw)
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")
    st = lib.bw_qgemm(xg.data_ptr(), 0, m, k, k, qg.data_ptr(), sbuf.data_ptr() + 2 * offset, zbuf.data_ptr() + 2 * offset,
                      None, n, bits, g, y.data_ptr(), n, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert st == 0
    torch.cuda.synchronize()
    check_matmul(y, x, qw, s16, z16, None, bits, g)


@pytest.mark.parametrize("bits,g,groups", [(4, 64, 24), (8, 64, 12), (2, 128, 8), (2, 32, 16), (2, 32, 24)])
@pytest.mark.parametrize("offset", [0, 1, 2, 3])
def test_prefill_wide_scale_requests_at_every_alignment(bits, g, groups, offset):
    """The other formats with wide scale requests - one 8-byte request per two K steps (4 and 8 bits at g64, 2 bits at
    g128), one 4-byte request for a lane's two groups (2 bits at g32): a base address off by one element must take
    the 2-byte requests and give the same result."""
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    n, m = 300, 192
    k = g * groups
    _, qw, s16, z16, _ = quantized_layer(n, k, bits, g, seed=177 + groups, outliers=True)
    x = np.random.default_rng(groups + offset).standard_normal((m, k)).astype(np.float16)
    sbuf = torch.zeros(n * groups + offset, dtype=torch.float16, device="cuda")
    zbuf = torch.zeros(n * groups + offset, dtype=torch.float16, device="cuda")
    sbuf[offset:] = to_gpu(s16).reshape(-1)
    zbuf[offset:] = to_gpu(z16).reshape(-1)
    xg, qg = to_gpu(x), to_gpu(qw)
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")
    st = lib.bw_qgemm(xg.data_ptr(), 0, m, k, k, qg.data_ptr(), sbuf.data_ptr() + 2 * offset, zbuf.data_ptr() + 2 * offset,
                      None, n, bits, g, y.data_ptr(), n, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert st == 0
    torch.cuda.synchronize()
    check_matmul(y, x, qw, s16, z16, None, bits, g)


@pytest.mark.parametrize("m", [1, 2, 16, 130])
@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("groups", [13, 14, 15, 16])
def test_rows_do_not_see_their_neighbours_scales(bits, groups, m):
    """The K loops run in steps of several groups and pad with zero steps; a row whose scale or zero point
    is Inf / NaN (its own outputs are then not finite, as in the reference) must leave every other row as it was."""
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    g, n = 128, 64
    k = g * groups
    _, qw, s16, z16, _ = quantized_layer(n, k, bits, g, seed=5 + groups)
    x = to_gpu(np.random.default_rng(groups).standard_normal((m, k)).astype(np.float16))
    qg = to_gpu(qw)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def run(s, z):
        sg, zg = to_gpu(s), to_gpu(z)
        y = torch.empty((m, n), dtype=torch.float16, device="cuda")
        assert lib.bw_qlinear(x.data_ptr(), 0, m, k, k, qg.data_ptr(), sg.data_ptr(), zg.data_ptr(), None, n, bits, g,
                              y.data_ptr(), n, stream) == 0
        torch.cuda.synchronize()
        return y

    clean = run(s16, z16)
    assert torch.isfinite(clean).all()
    bad_rows = [7, 20, 63]
    s_bad, z_bad = s16.copy(), z16.copy()
    s_bad[7, :] = np.inf
    z_bad[20, :] = np.nan
    s_bad[63, 0] = np.nan
    dirty = run(s_bad, z_bad)
    keep = [r for r in range(n) if r not in bad_rows]
    assert torch.equal(dirty[:, keep], clean[:, keep])
    assert not torch.isfinite(dirty[:, bad_rows]).all()


@pytest.mark.parametrize("bits,g,n,k", [(4, 128, 5, 256), (8, 32, 33, 96), (2, 64, 17, 192), (4, 32, 1, 32)])
def test_quantize_dequantize_ragged(bits, g, n, k):
    """Row counts that leave waves partly empty, with a padded row pitch on the way in and out."""
    from bitween_amd.kernels import hip_loader as hip
    lib = hip.load()
    rng = np.random.default_rng(n * k)
    w = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    ldw = k + 16
    wbuf = torch.full((n, ldw), float("nan"), dtype=torch.float32, device="cuda")
    wbuf[:, :k] = to_gpu(w)
    vpi = 32 // bits
    qw = torch.empty((n, k // vpi), dtype=torch.int32, device="cuda")
    sc = torch.empty((n, k // g), dtype=torch.float32, device="cuda")
    zp = torch.empty((n, k // g), dtype=torch.int32, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.bw_quantize_pack(wbuf.data_ptr(), 2, 2, n, k, ldw, bits, g, qw.data_ptr(), sc.data_ptr(), 2, zp.data_ptr(), 3, st) == 0
    qw_o, s_o, z_o, _ = orc.quantize_rtn(w, bits, g)
    assert np.array_equal(qw.cpu().numpy(), qw_o) and np.array_equal(zp.cpu().numpy(), z_o)
    assert np.array_equal(sc.cpu().numpy().view(np.uint32), s_o.view(np.uint32))
    ldo = k + 5
    out = torch.full((n, ldo), 3.0, dtype=torch.float32, device="cuda")
    assert lib.bw_dequantize(qw.data_ptr(), sc.data_ptr(), 2, zp.data_ptr(), 3, n, k, bits, g, out.data_ptr(), 2, ldo, st) == 0
    torch.cuda.synchronize()
    assert (out[:, k:] == 3.0).all()
    expect = (s_o.repeat(g, axis=1) * (orc.unpack_words(qw_o, bits).astype(np.float32) - z_o.repeat(g, axis=1).astype(np.float32)))
    assert np.array_equal(out[:, :k].cpu().numpy().view(np.uint32), expect.astype(np.float32).view(np.uint32))


@pytest.mark.parametrize("bits,g", [(4, 128), (8, 64), (2, 32)])
@pytest.mark.parametrize("m,n,k,ypad", [(300, 320, 512, 8), (300, 330, 640, 16), (129, 64, 256, 8), (256 * 52 + 5, 1000, 384, 8)])
def test_prefill_padded_rows_of_x_and_y(bits, g, m, n, k, ypad):
    """Prefill through the C ABI with padded rows on both sides: x rows K + 8 apart with NaN in the padding (never
    read: the activations go to LDS by buffer loads of whole 16-byte pieces), y rows N + ypad apart (a multiple of 8,
    so the whole-row stores of the LDS epilogue run where a wave's 64 columns lie inside N, the piecewise stores
    elsewhere) - nothing may be written past a row's N outputs.  Both tile heights (the last case has 53 row tiles)."""
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    _, qw, s16, z16, b16 = quantized_layer(n, k, bits, g, seed=m + n + k + bits, outliers=True)
    gen = torch.Generator(device="cuda").manual_seed(m + k)
    x = torch.randn(m, k, device="cuda", generator=gen).half()
    ldx, ldy = k + 8, n + ypad
    xbuf = torch.full((m, ldx), float("nan"), dtype=torch.float16, device="cuda")
    xbuf[:, :k] = x
    d = [to_gpu(a) for a in (qw, s16, z16, b16)]
    need = lib.bw_qgemm_workspace_bytes(m, n, k, bits, g)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    y = torch.full((m, ldy), 7.0, dtype=torch.float16, device="cuda")
    st = lib.bw_qgemm_ws(xbuf.data_ptr(), 0, m, k, ldx, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), n, bits, g,
                         y.data_ptr(), ldy, ws.data_ptr() if need else None, need, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert st == 0
    torch.cuda.synchronize()
    assert (y[:, n:] == 7.0).all()
    rows = np.unique(np.concatenate([np.arange(0, m, max(1, m // 40)), np.arange(max(0, m - 6), m)]))
    idx = torch.from_numpy(rows).cuda()
    check_matmul(y[idx][:, :n], x[idx].cpu().numpy(), qw, s16, z16, b16, bits, g)
    w16 = to_gpu(orc.dequantize_f16(qw, s16, z16, g, bits))
    ref = (x @ w16.T).float() + to_gpu(b16).float()
    assert ((y[:, :n].float() - ref).abs().max() <= 2.0 ** -8 * ref.abs().max()).item()


@pytest.mark.parametrize("bits,g", [(4, 128), (4, 32), (8, 64), (8, 128), (2, 32), (2, 128)])
@pytest.mark.parametrize("k", [128, 256, 384])
def test_prefill_one_to_three_k_steps(bits, g, k):
    """K of one, two and three steps of the prefill loop (its prologue requests two steps and the loop runs them in
    pairs, so these are the shapes where most of what is requested lies past the end of a row), at both tile heights:
    300 rows (128-row tiles) and 53 x 256 - 3 rows against N = 1000 (256-row tiles, the last row tile and the last
    column tile ragged)."""
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    for m, n in ((300, 200), (256 * 53 - 3, 1000)):
        _, qw, s16, z16, b16 = quantized_layer(n, k, bits, g, seed=m + n + k + bits, outliers=True)
        gen = torch.Generator(device="cuda").manual_seed(m + k + bits)
        x = torch.randn(m, k, device="cuda", generator=gen).half()
        d = [to_gpu(a) for a in (qw, s16, z16, b16)]
        need = lib.bw_qgemm_workspace_bytes(m, n, k, bits, g)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        y = torch.full((m, n), 7.0, dtype=torch.float16, device="cuda")
        st = lib.bw_qgemm_ws(x.data_ptr(), 0, m, k, k, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), n, bits, g,
                             y.data_ptr(), n, ws.data_ptr() if need else None, need, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert st == 0
        torch.cuda.synchronize()
        rows = np.unique(np.concatenate([np.arange(0, m, max(1, m // 30)), np.arange(max(0, m - 6), m)]))
        idx = torch.from_numpy(rows).cuda()
        check_matmul(y[idx], x[idx].cpu().numpy(), qw, s16, z16, b16, bits, g)
        w16 = to_gpu(orc.dequantize_f16(qw, s16, z16, g, bits))
        ref = (x @ w16.T).float() + to_gpu(b16).float()
        assert ((y.float() - ref).abs().max() <= 2.0 ** -8 * ref.abs().max()).item()
