"""bw_qdgrad (grad_x = grad_y @ W16, dequantisation fused) through the C ABI against the oracle's
qlinear_backward (bitween/modules.py:108-141 of the reference).

Bars: max |g - ref| <= 1e-2 * max |ref| and mean |g - ref| < 1e-2 * mean |ref| (the forward's tolerance,
main.py:471-477: the reference states none for the backward); elementwise one float16 rounding of the result plus
float32 accumulation slack; a one-hot grad_y row returns a ROW of W16 bit for bit."""
import ctypes

import numpy as np
import pytest
import torch

from gpu_util import quantized_layer, to_gpu
from oracle import rtn_oracle as orc

pytestmark = pytest.mark.gpu

COMBOS = [(b, g) for b in (2, 4, 8) for g in (32, 64, 128)]


def _call(lib, go, d, m, n, k, bits, g, use_ws=True, ldg=None):
    ldg = n if ldg is None else ldg
    need = lib.bw_qdgrad_workspace_bytes(m, n, k, bits, g) if use_ws else 0
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    gx = torch.full((m, k), float("nan"), dtype=torch.float16, device="cuda")
    st = lib.bw_qdgrad(go.data_ptr(), 0, m, n, ldg, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), k, bits, g,
                       gx.data_ptr(), k, ws.data_ptr() if need else None, need,
                       ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return st, gx, need


def _check(gx, go16, qw, s16, z16, bits, g):
    ref = orc.qlinear_backward(go16, qw, s16, z16, bits, g)                  # float64
    got = gx.double().cpu().numpy()
    assert np.isfinite(got).all()
    w16 = np.abs(orc.dequantize_f16(qw, s16, z16, g, bits).astype(np.float64))
    mag = np.abs(go16.astype(np.float64)) @ w16
    bound = 2.0 ** -10 * np.abs(ref) + 2e-6 * mag + 1e-7
    assert (np.abs(got - ref) <= bound).all(), float((np.abs(got - ref) / bound).max())
    assert np.abs(got - ref).max() <= 1e-2 * np.abs(ref).max()
    assert np.abs(got - ref).mean() < 1e-2 * np.abs(ref).mean()


@pytest.mark.parametrize("bits,g", COMBOS)
def test_dgrad_vs_oracle(bits, g):
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    for (n, k) in ((256, 384), (1024, 128), (96, 768), (32, 128)):
        _, qw, s16, z16, _ = quantized_layer(n, k, bits, g, seed=n + k + bits + g, outliers=True, bias=False)
        d = [to_gpu(a) for a in (qw, s16, z16)]
        rng = np.random.default_rng(n * 7 + k)
        for m in (1, 17, 128, 200, 513):
            go16 = rng.standard_normal((m, n)).astype(np.float16)
            for use_ws in (True, False):
                st, gx, need = _call(lib, to_gpu(go16), d, m, n, k, bits, g, use_ws)
                assert st == 0
                _check(gx, go16, qw, s16, z16, bits, g)


@pytest.mark.parametrize("bits,g,n,k", [(4, 128, 11008, 4096), (8, 128, 4096, 4096), (2, 32, 4096, 11008), (4, 64, 14336, 4096)])
def test_dgrad_full_size_one_hot_rows_and_split(bits, g, n, k):
    """Full-size layers: the reduction over N is cut into slices (workspace) at small M; a one-hot grad_y row
    returns a row of the reference's W16 exactly; random rows meet the oracle on a sample of columns."""
    from bitween_amd.kernels import hip_loader
    hip = hip_loader
    lib = hip.load()
    gen = torch.Generator(device="cuda").manual_seed(bits * 17 + g)
    w = (torch.randn(n, k, device="cuda", generator=gen) * 0.02).half()
    qw, sc, zp = hip.quantize_pack(w, bits, g, math_dtype=torch.float32, scale_dtype=torch.float16, zp_dtype=torch.float16)
    w16 = hip.dequantize(qw, sc, zp, g, bits, torch.float16)
    d = [qw, sc, zp]
    rows = [0, 1, 31, 32, n // 2 + 5, n - 1]
    go = torch.zeros(len(rows), n, device="cuda", dtype=torch.float16)
    for i, r in enumerate(rows):
        go[i, r] = 1.0
    st, gx, need = _call(lib, go, d, len(rows), n, k, bits, g)
    assert st == 0 and need > 0, "small M on a full-size layer is meant to split"
    for i, r in enumerate(rows):
        assert torch.equal(gx[i], w16[r])
    for m in (64, 300, 700):                                  # 700: the 256-row tile variant, last tile ragged
        go = torch.randn(m, n, device="cuda", dtype=torch.float16, generator=gen)
        st, gx, _ = _call(lib, go, d, m, n, k, bits, g)
        assert st == 0
        ref = go.float() @ w16.float()
        err = (gx.float() - ref).abs()
        assert (err <= 2.0 ** -9 * ref.abs() + 2e-5 * (go.float().abs() @ w16.float().abs()) + 1e-6).all()


def test_dgrad_refusals_and_padding():
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    n, k, bits, g = 64, 256, 4, 64
    _, qw, s16, z16, _ = quantized_layer(n, k, bits, g, seed=3, bias=False)
    d = [to_gpu(a) for a in (qw, s16, z16)]
    go16 = np.random.default_rng(0).standard_normal((5, n)).astype(np.float16)
    # padded grad_y rows: the padding is never read
    buf = torch.full((5, n + 8), float("nan"), dtype=torch.float16, device="cuda")
    buf[:, :n] = to_gpu(go16)
    st, gx, _ = _call(lib, buf, d, 5, n, k, bits, g, ldg=n + 8)
    assert st == 0
    _check(gx, go16, qw, s16, z16, bits, g)
    # shapes outside the fused kernel are refused, nothing is launched
    assert lib.bw_qdgrad_workspace_bytes(5, 40, 256, 4, 64) == 0
    go = to_gpu(go16)
    gx = torch.full((5, k), 7.0, dtype=torch.float16, device="cuda")
    st = lib.bw_qdgrad(go.data_ptr(), 0, 5, n, n, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), k, bits, g,
                       gx.data_ptr(), k, None, 0, None)
    assert st == 0
    assert lib.bw_qdgrad(go.data_ptr(), 2, 5, n, n, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), k, bits, g,
                         gx.data_ptr(), k, None, 0, None) == -2          # float32 gradients: BW_EUNSUPPORTED
    assert lib.bw_qdgrad(go.data_ptr(), 0, 5, n, n, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), k, 3, g,
                         gx.data_ptr(), k, None, 0, None) == -1          # BW_EINVAL
    assert lib.bw_qdgrad(None, 0, 5, n, n, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), k, bits, g,
                         gx.data_ptr(), k, None, 0, None) == -1


def test_module_backward_uses_fused_kernel_and_falls_back():
    """autograd through QuantizedLinear: float16 gradients take bw_qdgrad; float32 gradients and odd shapes take
    the dequantise + library GEMM path; both meet the oracle."""
    import bitween_amd
    torch.manual_seed(4)
    for (k, n, gdt) in ((256, 512, torch.float16), (256, 512, torch.float32), (96, 40, torch.float16)):
        lin = torch.nn.Linear(k, n, bias=True, device="cuda", dtype=torch.float16)
        q = bitween_amd.QuantizedLinear.from_float(lin, 4, 32)
        x = torch.randn(3, 7, k, device="cuda", dtype=torch.float16, requires_grad=True)
        y = q(x)
        go = torch.randn(3, 7, n, device="cuda", dtype=torch.float16)
        if gdt is torch.float32:
            (y.float() * go.float()).sum().backward()
        else:
            y.backward(go)
        ref = orc.qlinear_backward(go.reshape(21, n).cpu().numpy(), q.qweight.cpu().numpy(), q.scale.cpu().numpy(),
                                   q.zero_point.cpu().numpy(), 4, 32)
        got = x.grad.reshape(21, k).double().cpu().numpy()
        assert x.grad.dtype == torch.float16
        assert np.abs(got - ref).max() <= 1e-2 * np.abs(ref).max()


def _sweep():
    rng = np.random.default_rng(77)
    out = []
    for i in range(24):
        bits = int(rng.choice([2, 4, 8]))
        g = int(rng.choice([32, 64, 128]))
        k = 128 * int(rng.integers(1, 7))
        n = 32 * int(rng.integers(1, 13))
        m = int(rng.choice([1, 2, 15, 16, 33, 127, 128, 129, 255, 300, 513, 600]))
        pad = int(rng.choice([0, 8, 40]))
        out.append((i, bits, g, k, n, m, pad))
    return out


@pytest.mark.parametrize("case", _sweep(), ids=lambda c: "b%d_g%d_K%d_N%d_M%d_pad%d" % c[1:])
def test_dgrad_seeded_sweep(case):
    """Random supported shapes (K % 128 == 0, N % 32 == 0), both tile variants, ragged last m tile, padded grad_y
    rows, sliced and unsliced reduction."""
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    i, bits, g, k, n, m, pad = case
    _, qw, s16, z16, _ = quantized_layer(n, k, bits, g, seed=500 + i, outliers=True, bias=False)
    d = [to_gpu(a) for a in (qw, s16, z16)]
    go16 = np.random.default_rng(i).standard_normal((m, n)).astype(np.float16)
    buf = torch.full((m, n + pad), float("nan"), dtype=torch.float16, device="cuda")
    buf[:, :n] = to_gpu(go16)
    for use_ws in (True, False):
        st, gx, _ = _call(lib, buf, d, m, n, k, bits, g, use_ws, ldg=n + pad)
        assert st == 0
        _check(gx, go16, qw, s16, z16, bits, g)


def _bf16_values(a):
    """float32 array rounded to bfloat16 values (what a bfloat16 tensor holds)."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16)


@pytest.mark.parametrize("bits,g", COMBOS)
def test_dgrad_bfloat16_vs_oracle(bits, g):
    """bfloat16 gradients: the kernel multiplies with W32.to(bfloat16) (bitween/modules.py:134-139) on the bfloat16
    matrix core and returns bfloat16.  Against qlinear_backward(dtype="bf16"): one bfloat16 rounding of the result
    (2^-8 relative) plus float32 accumulation slack; one-hot rows return rows of the bfloat16 weight bit for bit."""
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for (n, k) in ((256, 384), (96, 768), (1024, 128)):
        _, qw, s16, z16, _ = quantized_layer(n, k, bits, g, seed=n + k + bits + g + 1, outliers=True, bias=False)
        d = [to_gpu(a) for a in (qw, s16, z16)]
        wbf = orc.dequantize_bf16(qw, s16, z16, g, bits)                 # float32 holding bfloat16 values
        rng = np.random.default_rng(n + 3 * k)
        for m in (1, 17, 130, 600):
            go = _bf16_values(rng.standard_normal((m, n))).cuda()
            for use_ws in (True, False):
                need = lib.bw_qdgrad_workspace_bytes(m, n, k, bits, g) if use_ws else 0
                ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
                gx = torch.full((m, k), float("nan"), dtype=torch.bfloat16, device="cuda")
                st = lib.bw_qdgrad(go.data_ptr(), 1, m, n, n, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), k, bits, g,
                                   gx.data_ptr(), k, ws.data_ptr() if need else None, need, stream)
                torch.cuda.synchronize()
                assert st == 0
                go32 = go.float().cpu().numpy()
                ref = orc.qlinear_backward(go32, qw, s16, z16, bits, g, dtype="bf16")
                got = gx.double().cpu().numpy()
                mag = np.abs(go32.astype(np.float64)) @ np.abs(wbf.astype(np.float64))
                bound = 2.0 ** -8 * np.abs(ref) + 2e-6 * mag + 1e-7
                assert (np.abs(got - ref) <= bound).all(), float((np.abs(got - ref) / bound).max())
                assert np.abs(got - ref).max() <= 1e-2 * np.abs(ref).max()
        # one-hot rows: rows of the bfloat16 weight, bit for bit
        rows = [0, 1, n // 2 + 1, n - 1]
        go = torch.zeros((len(rows), n), dtype=torch.bfloat16, device="cuda")
        for i, r in enumerate(rows):
            go[i, r] = 1.0
        gx = torch.empty((len(rows), k), dtype=torch.bfloat16, device="cuda")
        st = lib.bw_qdgrad(go.data_ptr(), 1, len(rows), n, n, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), k, bits, g,
                           gx.data_ptr(), k, None, 0, stream)
        torch.cuda.synchronize()
        assert st == 0
        assert np.array_equal(gx.float().cpu().numpy(), wbf[rows])


def test_module_backward_takes_the_fused_kernel_for_bfloat16_gradients():
    """QuantizedLinearFunction.backward with a bfloat16 grad_output: the fused kernel's result equals the reference's
    own sequence - dequantise to float32, cast to bfloat16, matmul (bitween/modules.py:125-139) - to bfloat16 rounding."""
    import bitween_amd
    torch.manual_seed(4)
    lin = torch.nn.Linear(512, 384, bias=False, device="cuda", dtype=torch.float16)
    q = bitween_amd.QuantizedLinear.from_float(lin, 4, 128)
    go = torch.randn(40, 384, device="cuda", dtype=torch.bfloat16)
    from bitween_amd.kernels import hip_loader as hip
    got = hip.quantized_input_grad(go, q.qweight, q.scale, q.zero_point, 4, 128)
    assert got is not None and got.dtype is torch.bfloat16
    w = bitween_amd.dequantize_rtn(q.qweight, q.scale, q.zero_point, 128, 4).to(torch.bfloat16)
    want = go.float() @ w.float()
    assert (got.float() - want).abs().max().item() <= 2.0 ** -7 * want.abs().max().item()


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("bits,g", COMBOS)
def test_dgrad_256_tiles_vs_oracle(bits, g, dtype):
    """Large problems run the 256 x 256 kernel (bw_qdgrad_tile_rows == 257; 129 = its variant with 128 rows of m per tile,
    up to 512 rows of grad_y): grad_y tile memory -> LDS by buffer loads, the dequantised weight tile read transposed from
    LDS, steps of 64 rows of n.  Ragged M (1100 rows: five row tiles, the last 76 rows high; 300 rows: three 128-row tiles;
    64 rows: half a tile), rows of grad_y and grad_x padded, N sliced through the workspace (20 tiles on 256 CUs) and, where
    the grid is large enough without one, unsliced; sampled rows against the oracle, one-hot rows return rows of the
    weight in the gradient's type bit for bit, the whole result against the library GEMM on the dequantised weight."""
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    tdt, code = (torch.float16, 0) if dtype == "f16" else (torch.bfloat16, 1)
    for (m, n, k, plan) in ((1100, 64 * 154, 1024, 257), (300, 64 * 800, 512, 129), (256 * 160 + 9, 64 * 6, 1024, 257), (64, 64 * 640, 1024, 129)):
        assert lib.bw_qdgrad_tile_rows(m, n, k, bits, g) == plan
        _, qw, s16, z16, _ = quantized_layer(n, k, bits, g, seed=n + k + bits + g + 5, outliers=True, bias=False)
        d = [to_gpu(a) for a in (qw, s16, z16)]
        wt = orc.dequantize_f16(qw, s16, z16, g, bits).astype(np.float32) if dtype == "f16" else orc.dequantize_bf16(qw, s16, z16, g, bits)
        gen = torch.Generator(device="cuda").manual_seed(m + n + bits)
        ldg, ldx = n + 8, k + 4
        gobuf = torch.full((m, ldg), float("nan"), dtype=tdt, device="cuda")
        go = torch.randn(m, n, device="cuda", generator=gen).to(tdt)
        hot = {0: 0, 1: n - 1, m // 2: n // 2 + 1, m - 1: 63}
        for r, c in hot.items():
            go[r] = 0
            go[r, c] = 1.0
        gobuf[:, :n] = go
        need = lib.bw_qdgrad_workspace_bytes(m, n, k, bits, g)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        wg = torch.from_numpy(np.ascontiguousarray(wt)).cuda().to(tdt)
        ref_all = (go @ wg).float()
        tiles = -(-m // 256) * (k // 256)
        for use_ws in ((True, False) if tiles > 128 else (True,)):     # without a workspace small grids stay on the other kernel
            gx = torch.full((m, ldx), 7.0, dtype=tdt, device="cuda")
            st = lib.bw_qdgrad(gobuf.data_ptr(), code, m, n, ldg, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), k, bits, g,
                               gx.data_ptr(), ldx, ws.data_ptr() if (use_ws and need) else None, need if use_ws else 0, stream)
            torch.cuda.synchronize()
            assert st == 0
            assert (gx[:, k:] == 7.0).all()                          # nothing written past a row's K outputs
            got_all = gx[:, :k].float()
            assert torch.isfinite(got_all).all()
            assert ((got_all - ref_all).abs().max() <= 2.0 ** -7 * ref_all.abs().max()).item()
            rows = np.unique(np.concatenate([np.arange(0, m, max(1, m // 24)), np.arange(max(0, m - 5), m), np.array(list(hot))]))
            go_np = go[torch.from_numpy(rows).cuda()].float().cpu().numpy()
            ref = orc.qlinear_backward(go_np if dtype == "bf16" else go_np.astype(np.float16), qw, s16, z16, bits, g,
                                       **({"dtype": "bf16"} if dtype == "bf16" else {}))
            got = gx[torch.from_numpy(rows).cuda()][:, :k].double().cpu().numpy()
            mag = np.abs(go_np.astype(np.float64)) @ np.abs(wt.astype(np.float64))
            bound = (2.0 ** -10 if dtype == "f16" else 2.0 ** -8) * np.abs(ref) + 2e-6 * mag + 1e-7
            assert (np.abs(got - ref) <= bound).all(), float((np.abs(got - ref) / bound).max())
            for r, c in hot.items():
                assert np.array_equal(gx[r, :k].float().cpu().numpy(), wt[c].astype(np.float32))
