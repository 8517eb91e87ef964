"""GPU parity: the HIP kernels (through the C ABI / the Python boundary)
against the CPU oracle and the committed exact vectors.  Bit-exact for packed
weights, scales, zero points and dequantised weights; matmul outputs to the
tolerance stated in gpu_util.check_matmul."""
import os

import numpy as np
import pytest
import torch

from oracle import rtn_oracle as orc
from gpu_util import check_matmul, make_weight, quantized_layer, to_gpu

pytestmark = pytest.mark.gpu

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "rtn_exact_vectors.npz"))
ALL_CASES = [str(s) for s in GOLD["names"]]
CASES = [c for c in ALL_CASES if not c.endswith(":recip")]          # scale by true division (eager torch on the CPU)
RECIP_CASES = [c for c in ALL_CASES if c.endswith(":recip")]        # scale by the float32 reciprocal (eager torch on a GPU)
TORCH_DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
COMBOS = [(b, g) for b in (2, 4, 8) for g in (32, 64, 128)]


def _hip():
    from bitween_amd.kernels import hip_loader
    return hip_loader


def _bits_of(t):
    """Raw bit pattern of a GPU tensor as a numpy integer array."""
    t = t.contiguous().cpu()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.float32:
        return t.view(torch.int32).numpy().view(np.uint32)
    return t.numpy()


def _bf16_bits(a32):
    return (np.ascontiguousarray(a32, np.float32).view(np.uint32) >> 16).astype(np.uint16)


@pytest.mark.parametrize("name", CASES)
def test_quantize_matches_exact_vectors(name):
    import bitween_amd
    key, fmt, bits, g, _ = name.split(":")
    bits, g = int(bits), int(g)
    w = torch.from_numpy(GOLD[key + "_w"]).to(TORCH_DT[fmt]).cuda()
    qw, scale, zp, gs = bitween_amd.quantize_rtn(w, bits, g)
    assert gs == g and qw.dtype == torch.int32 and zp.dtype == torch.int32 and scale.dtype == TORCH_DT[fmt]
    valid = GOLD[key + "_valid"]
    assert np.array_equal(zp.cpu().numpy()[valid], GOLD[key + "_zp"][valid])
    exp_scale = GOLD[key + "_scale"]
    if fmt == "f32":
        assert np.array_equal(_bits_of(scale)[valid], exp_scale.view(np.uint32)[valid])
    elif fmt == "f16":
        assert np.array_equal(_bits_of(scale)[valid], exp_scale.astype(np.float16).view(np.uint16)[valid])
    else:
        assert np.array_equal(_bits_of(scale)[valid], _bf16_bits(exp_scale)[valid])
    q = orc.unpack_words(qw.cpu().numpy(), bits)
    vq = np.repeat(valid, g, axis=1)
    assert np.array_equal(q[vq], GOLD[key + "_q"][vq])
    if valid.all():
        assert np.array_equal(qw.cpu().numpy(), GOLD[key + "_qweight"])


GOLD64 = np.load(os.path.join(os.path.dirname(__file__), "golden", "rtn_exact_vectors_f64.npz"))


@pytest.mark.parametrize("name", [str(n) for n in GOLD64["names"]])
def test_quantize_float64_tensor_matches_exact_vectors(name):
    """functional.py:3-71 is dtype-agnostic: a float64 weight is quantised in float64 arithmetic, returns a float64
    scale, and dequantises to float64 - bit for bit, in both scale-division modes."""
    import bitween_amd
    key, _, bits, g, _, scale_div = name.split(":")
    bits, g = int(bits), int(g)
    w = torch.from_numpy(GOLD64[key + "_w"]).cuda()
    previous = bitween_amd.set_scale_division("ieee" if scale_div == "ieee" else "torch_device")
    try:
        qw, scale, zp, group = bitween_amd.quantize_rtn(w, bits, g)
    finally:
        bitween_amd.set_scale_division(previous)
    assert group == g and scale.dtype == torch.float64 and zp.dtype == torch.int32 and qw.dtype == torch.int32
    assert np.array_equal(qw.cpu().numpy(), GOLD64[key + "_qweight"])
    assert np.array_equal(zp.cpu().numpy(), GOLD64[key + "_zp"])
    assert np.array_equal(scale.cpu().numpy().view(np.uint64), GOLD64[key + "_scale"].view(np.uint64))
    w64 = bitween_amd.dequantize_rtn(qw, scale, zp, g, bits)
    assert w64.dtype == torch.float64
    assert np.array_equal(w64.cpu().numpy().view(np.uint64), GOLD64[key + "_w64"].view(np.uint64))
    # the perturbed form: w = a + b with the sum rounded once to float64
    a = w * 0.75
    qw2, s2, z2, _ = bitween_amd.quantize_rtn_perturbed(a, w - a, bits, g)
    qw3, s3, z3, _ = bitween_amd.quantize_rtn(a + (w - a), bits, g)
    assert torch.equal(qw2, qw3) and torch.equal(s2, s3) and torch.equal(z2, z3)


@pytest.mark.parametrize("name", RECIP_CASES)
def test_quantize_with_reciprocal_scale_matches_exact_vectors(name):
    """set_scale_division("torch_device"): the scale as eager torch forms it on a GPU, (max - min) * fl32(1 / Qmax)."""
    import bitween_amd
    key, fmt, bits, g = name.split(":")[:4]
    bits, g = int(bits), int(g)
    w = torch.from_numpy(GOLD[key + "_w"]).to(TORCH_DT[fmt]).cuda()
    previous = bitween_amd.set_scale_division("torch_device")
    try:
        qw, scale, zp, _ = bitween_amd.quantize_rtn(w, bits, g)
        if fmt == "f32":
            lin = torch.nn.Linear(w.shape[1], w.shape[0], bias=False)
            lin.weight.data = w.clone()
            layer = bitween_amd.QuantizedLinear.from_float(lin, bits, g)
    finally:
        bitween_amd.set_scale_division(previous)
    valid = GOLD[key + "_valid"]
    assert np.array_equal(zp.cpu().numpy()[valid], GOLD[key + "_zp"][valid])
    exp_scale = GOLD[key + "_scale"]
    if fmt == "f32":
        assert np.array_equal(_bits_of(scale)[valid], exp_scale.view(np.uint32)[valid])
        assert np.array_equal(layer.qweight.cpu().numpy(), GOLD[key + "_qweight"])
        assert np.array_equal(_bits_of(layer.scale), GOLD[key + "_scale16"].view(np.uint16))
    elif fmt == "f16":
        assert np.array_equal(_bits_of(scale)[valid], exp_scale.astype(np.float16).view(np.uint16)[valid])
    else:
        assert np.array_equal(_bits_of(scale)[valid], _bf16_bits(exp_scale)[valid])
    q = orc.unpack_words(qw.cpu().numpy(), bits)
    vq = np.repeat(valid, g, axis=1)
    assert np.array_equal(q[vq], GOLD[key + "_q"][vq])


@pytest.mark.parametrize("name", [c for c in CASES if c.split(":")[1] == "f32"])
def test_from_float_and_dequantize_match_exact_vectors(name):
    import bitween_amd
    key, _, bits, g, kind = name.split(":")
    bits, g = int(bits), int(g)
    w = GOLD[key + "_w"]
    n, k = w.shape
    layer = torch.nn.Linear(k, n, bias=False)
    layer.weight.data = torch.from_numpy(w)
    if kind in ("normal_f16", "outliers"):                       # exactly representable: exercise the f16-input kernel
        layer = layer.half()
    q = bitween_amd.QuantizedLinear.from_float(layer.cuda(), bits, g)
    assert q.qweight.dtype == torch.int32 and q.scale.dtype == torch.float16 and q.zero_point.dtype == torch.float16
    assert np.array_equal(q.qweight.cpu().numpy(), GOLD[key + "_qweight"])
    assert np.array_equal(_bits_of(q.scale), GOLD[key + "_scale16"].view(np.uint16))
    assert np.array_equal(q.zero_point.float().cpu().numpy(), GOLD[key + "_zp"].astype(np.float32))
    hip = _hip()
    w16 = hip.dequantize(q.qweight, q.scale, q.zero_point, g, bits, torch.float16)
    assert np.array_equal(_bits_of(w16), GOLD[key + "_w16"].view(np.uint16))
    qw32, s32, z32, _ = bitween_amd.quantize_rtn(torch.from_numpy(w).cuda(), bits, g)
    w32 = bitween_amd.dequantize_rtn(qw32, s32, z32, g, bits)
    assert w32.dtype == torch.float32
    assert np.array_equal(_bits_of(w32), GOLD[key + "_w32"].view(np.uint32))
    # forward on the exact vectors' activations (M = 3)
    x = GOLD[key + "_x"]
    y = q(torch.from_numpy(x).cuda())
    ref = GOLD[key + "_y64"]
    yv = y.float().cpu().numpy().astype(np.float64)
    over = np.abs(ref) > 65519.0                              # beyond float16: the reference overflows too
    assert (np.isinf(yv[over]) & (np.sign(yv[over]) == np.sign(ref[over]))).all()
    w16a = np.abs(GOLD[key + "_w16"].astype(np.float64))
    mag = np.abs(x.astype(np.float64)) @ w16a.T
    rss = np.sqrt((x.astype(np.float64) ** 2) @ (w16a ** 2).T)
    ok = np.abs(ref) < 65000.0
    assert (np.abs(yv - ref)[ok] <= (2.0 ** -10 * np.abs(ref) + 6 * 2.0 ** -11 * rss + 2e-6 * mag + 1e-7)[ok]).all()


@pytest.mark.parametrize("bits,g", COMBOS)
@pytest.mark.parametrize("wdtype", ["f32", "f16", "bf16"])
def test_quantize_random_vs_oracle(bits, g, wdtype):
    """from_float-style quantisation (float32 math) of f32 / f16 / bf16 weights, with outliers."""
    hip = _hip()
    w = make_weight(64, 768, seed=bits * 1000 + g, outliers=True, dtype=np.float32)
    wt = torch.from_numpy(w).to(TORCH_DT[wdtype])
    w_eff = wt.float().numpy()
    qw_o, s_o, z_o, _ = orc.quantize_rtn(w_eff, bits, g)
    qw, s, z = hip.quantize_pack(wt.cuda(), bits, g, math_dtype=torch.float32, scale_dtype=torch.float32,
                                 zp_dtype=torch.int32)
    assert np.array_equal(qw.cpu().numpy(), qw_o)
    assert np.array_equal(_bits_of(s), s_o.view(np.uint32))
    assert np.array_equal(z.cpu().numpy(), z_o)
    # dequantise to every output type
    s16, z16 = orc.store_module_buffers(s_o, z_o)
    for odt, expect in ((torch.float16, orc.dequantize_f16(qw_o, s16, z16, g, bits).view(np.uint16)),
                        (torch.float32, orc.dequantize_rtn_f32(qw_o, s16, z16, g, bits).view(np.uint32)),
                        (torch.bfloat16, _bf16_bits(orc.dequantize_bf16(qw_o, s16, z16, g, bits)))):
        got = hip.dequantize(to_gpu(qw_o), to_gpu(s16), to_gpu(z16), g, bits, odt)
        assert np.array_equal(_bits_of(got), expect)


def _tie_heavy_weights(n, k, bits, g, seed):
    """float32 weights whose quotient w / scale + zp sits on, or within a few ulps of, a half-integer: the
    inputs where a quotient that is off by one ulp changes the rounded integer."""
    rng = np.random.default_rng(seed)
    qmax = np.float32(2 ** bits - 1)
    w = np.empty((n, k), dtype=np.float32)
    for r in range(n):
        for c in range(k // g):
            mag = np.float32(10.0 ** rng.uniform(-6, 4))
            lo = np.float32(-mag * rng.uniform(0.05, 1.0))
            hi = np.float32(mag * rng.uniform(0.05, 1.0))
            s = max(np.float32(np.float32(hi - lo) / qmax), np.float32(1e-8))
            zf = np.float32(min(max(np.rint(np.float32(-lo / s)), 0), qmax))
            j = rng.integers(0, int(qmax), size=g).astype(np.float32)
            vals = (s * (j + np.float32(0.5) - zf)).astype(np.float32)       # quotient + zp = j + 0.5 (up to rounding)
            for _ in range(3):                                               # walk up to 3 ulps either way
                step = rng.integers(-1, 2, size=g)
                vals = np.where(step > 0, np.nextafter(vals, np.float32(np.inf)),
                                np.where(step < 0, np.nextafter(vals, np.float32(-np.inf)), vals)).astype(np.float32)
            vals = np.clip(vals, lo, hi)
            vals[0], vals[1] = lo, hi                                        # pin the group's extrema, hence its scale
            w[r, c * g:(c + 1) * g] = vals
    return w


@pytest.mark.parametrize("bits,g", COMBOS)
def test_quantize_near_ties_vs_oracle(bits, g):
    """The quantiser's short division is only taken away from rounding ties; this feeds it ties."""
    hip = _hip()
    w = _tie_heavy_weights(48, 1024, bits, g, seed=17 * bits + g)
    for wt in (torch.from_numpy(w), torch.from_numpy(w).half()):
        w_eff = wt.float().numpy()
        finite = np.isfinite(w_eff).all(axis=1)
        qw_o, s_o, z_o, _ = orc.quantize_rtn(w_eff, bits, g)
        qw, sc, z = hip.quantize_pack(wt.cuda(), bits, g, math_dtype=torch.float32, scale_dtype=torch.float32,
                                      zp_dtype=torch.int32)
        assert finite.sum() >= 40
        assert np.array_equal(qw.cpu().numpy()[finite], qw_o[finite])
        assert np.array_equal(_bits_of(sc)[finite], s_o.view(np.uint32)[finite])
        assert np.array_equal(z.cpu().numpy()[finite], z_o[finite])


GEMV_SHAPES = [(768, 3072), (256, 40), (4096, 512), (11008, 64), (2048, 16), (1024, 1000)]


@pytest.mark.parametrize("bits,g", COMBOS)
@pytest.mark.parametrize("k,n", GEMV_SHAPES)
def test_gemv_vs_oracle(bits, g, k, n):
    hip = _hip()
    _, qw, s16, z16, b16 = quantized_layer(n, k, bits, g, seed=k + n + bits, outliers=True)
    d = [to_gpu(a) for a in (qw, s16, z16, b16)]
    rng = np.random.default_rng(k * 3 + n)
    for m in (1, 2, 3, 4, 7, 8, 16):
        x = rng.standard_normal((m, k)).astype(np.float16)
        use_bias = m % 2 == 1
        y = hip.quantized_gemv_hip(to_gpu(x), d[0], d[1], d[2], d[3] if use_bias else None, bits, g)
        assert y.shape == (m, n) and y.dtype == torch.float16
        check_matmul(y, x, qw, s16, z16, b16 if use_bias else None, bits, g)


@pytest.mark.parametrize("bits,g", COMBOS)
def test_gemm_vs_oracle(bits, g):
    hip = _hip()
    for (k, n) in ((2048, 1024), (768, 200)):
        _, qw, s16, z16, b16 = quantized_layer(n, k, bits, g, seed=k + n + bits + 7, outliers=True)
        d = [to_gpu(a) for a in (qw, s16, z16, b16)]
        rng = np.random.default_rng(k + n)
        for m in (17, 128, 200, 512):
            x = rng.standard_normal((m, k)).astype(np.float16)
            y = hip.quantized_gemm_hip(to_gpu(x), d[0], d[1], d[2], d[3], bits, g)
            check_matmul(y, x, qw, s16, z16, b16, bits, g)


@pytest.mark.parametrize("bits,g,m,k,n", [(4, 128, 128, 14336, 512), (4, 64, 200, 4096, 768), (8, 128, 96, 4096, 300),
                                          (2, 32, 128, 8192, 256), (4, 32, 17, 2048 + 128, 40)])
def test_gemm_split_k_vs_unsplit_and_oracle(bits, g, m, k, n):
    """bw_qgemm_ws through the C ABI: with a workspace K is cut into parallel slices, without one it is
    bw_qgemm; both must meet the oracle, and a workspace that is too small is refused before any launch."""
    import ctypes
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    _, qw, s16, z16, b16 = quantized_layer(n, k, bits, g, seed=m + k + n, outliers=True)
    x = np.random.default_rng(k + m).standard_normal((m, k)).astype(np.float16)
    d = [to_gpu(a) for a in (x, qw, s16, z16, b16)]
    need = lib.bw_qgemm_workspace_bytes(m, n, k, bits, g)
    assert need >= 2 * 128 * 256 * 4, "case is meant to split"
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def run(ws_ptr, ws_bytes, y):
        return lib.bw_qgemm_ws(d[0].data_ptr(), 0, m, k, k, d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(),
                               d[4].data_ptr(), n, bits, g, y.data_ptr(), n, ws_ptr, ws_bytes, st)

    y_split = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
    y_plain = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
    y_small = torch.full((m, n), 7.0, dtype=torch.float16, device="cuda")
    assert run(ws.data_ptr(), need, y_split) == 0
    assert run(None, 0, y_plain) == 0
    # bw_qgemm_workspace_bytes covers every plan a call of this shape may get (the 128-row plan also where the call
    # itself runs 64-row tiles, whose blocks are half as large): there only less than two 64-row blocks is surely short
    short = need - 4 if lib.bw_qgemm_tile_rows(m, n, k, bits, g) != 64 else 2 * 64 * 256 * 4 - 16
    assert run(ws.data_ptr(), short, y_small) == -5             # BW_EWORKSPACE, nothing launched
    assert run(ws.data_ptr() + 4, need, y_small) == -3          # BW_EALIGN
    torch.cuda.synchronize()
    assert (y_small == 7.0).all()
    check_matmul(y_split, x, qw, s16, z16, b16, bits, g)
    check_matmul(y_plain, x, qw, s16, z16, b16, bits, g)
    # the two differ only in the float32 summation order
    diff = (y_split.float() - y_plain.float()).abs().max().item()
    assert diff <= 2.0 ** -9 * y_plain.float().abs().max().item()


def test_gemm_short_last_round_is_split():
    """258 tiles on 256 CUs: the two tiles of the last round are cut along K (partial tiles + reduce kernel), the
    other 256 are not.  Checked against the un-split run everywhere and against the oracle on rows of both kinds."""
    import ctypes
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    bits, g, m, k, n = 4, 128, 128 * 86, 2048, 768
    need = lib.bw_qgemm_workspace_bytes(m, n, k, bits, g)
    if need == 0:
        pytest.skip("this device's CU count leaves no short last round for 258 tiles")
    assert need % (128 * 256 * 4) == 0 and need < 64 * 128 * 256 * 4      # a few tiles' worth, not the whole matrix
    _, qw, s16, z16, b16 = quantized_layer(n, k, bits, g, seed=77, outliers=True)
    x = np.random.default_rng(78).standard_normal((m, k)).astype(np.float16)
    d = [to_gpu(a) for a in (x, qw, s16, z16, b16)]
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ys = []
    for ws_ptr, ws_bytes in ((ws.data_ptr(), need), (None, 0)):
        y = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
        assert lib.bw_qgemm_ws(d[0].data_ptr(), 0, m, k, k, d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), d[4].data_ptr(),
                               n, bits, g, y.data_ptr(), n, ws_ptr, ws_bytes, st) == 0
        ys.append(y)
    torch.cuda.synchronize()
    assert torch.isfinite(ys[0]).all()
    diff = (ys[0].float() - ys[1].float()).abs().max().item()
    assert diff <= 2.0 ** -9 * ys[1].float().abs().max().item()
    rows = np.r_[0:40, m - 300:m - 260, m - 40:m]                           # first tile, and both tiles of the last round
    check_matmul(ys[0][torch.from_numpy(rows).cuda()], x[rows], qw, s16, z16, b16, bits, g)


def test_reference_acceptance_recipe():
    """main.py:394-477: M=512, N=1024, K=2048, 8-bit g128, nn.Linear default init, mean-relative error < 1 %."""
    import bitween_amd
    torch.manual_seed(0)
    layer = torch.nn.Linear(2048, 1024, bias=True, dtype=torch.float32).cuda()
    qweight, scale, zp, _ = bitween_amd.quantize_rtn(layer.weight.data, bits=8, group_size=128)
    scale, zp, bias = scale.half(), zp.half(), layer.bias.data.half()
    x = torch.randn(512, 2048, device="cuda", dtype=torch.float16)
    out = _hip().quantized_matmul_hip(x, qweight, scale, zp, bias, 8, 128)
    w16 = orc.dequantize_f16(qweight.cpu().numpy(), scale.cpu().numpy(), zp.cpu().numpy(), 128, 8)
    ref = torch.nn.functional.linear(x.float().cpu(), torch.from_numpy(w16).float(), bias.float().cpu())
    rel = (out.float().cpu() - ref).abs().mean() / ref.abs().mean()
    assert rel < 0.01
    check_matmul(out, x.cpu().numpy(), qweight.cpu().numpy(), scale.cpu().numpy(), zp.cpu().numpy(), bias.cpu().numpy(), 8, 128)


def test_generic_shapes_any_group():
    """Group sizes / K outside the fast layouts take the shape-generic kernels."""
    hip = _hip()
    for bits, g, k, n in ((4, 48, 96, 20), (8, 20, 40, 33), (2, 16, 48, 7)):
        w, qw, s16, z16, b16 = quantized_layer(n, k, bits, g, seed=g + k)
        # quantiser: any group size the reference accepts, bit-exact
        qw_g, s_g, z_g = hip.quantize_pack(to_gpu(w), bits, g, math_dtype=torch.float32, scale_dtype=torch.float16,
                                           zp_dtype=torch.float16)
        assert np.array_equal(qw_g.cpu().numpy(), qw)
        assert np.array_equal(_bits_of(s_g), s16.view(np.uint16)) and np.array_equal(_bits_of(z_g), z16.view(np.uint16))
        x = np.random.default_rng(g).standard_normal((5, k)).astype(np.float16)
        y = hip.quantized_matmul_hip(to_gpu(x), to_gpu(qw), to_gpu(s16), to_gpu(z16), to_gpu(b16), bits, g)
        check_matmul(y, x, qw, s16, z16, b16, bits, g)
        w16 = hip.dequantize(to_gpu(qw), to_gpu(s16), to_gpu(z16), g, bits, torch.float16)
        assert np.array_equal(_bits_of(w16), orc.dequantize_f16(qw, s16, z16, g, bits).view(np.uint16))


def test_module_forward_backward_and_model_walk():
    import bitween_amd
    torch.manual_seed(1)
    model = torch.nn.Sequential()
    model.add_module("fc1", torch.nn.Linear(768, 3072))
    model.add_module("act", torch.nn.GELU())
    model.add_module("fc2", torch.nn.Linear(3072, 768, bias=False))
    model.add_module("lm_head", torch.nn.Linear(768, 100))
    model = model.half().cuda()
    qm = bitween_amd.Bitween(model, bits=4, group_size=128, ignore_layers=["lm_head"]).quantize(rtn=True, verbose=False)
    assert isinstance(qm.fc1, bitween_amd.QuantizedLinear) and isinstance(qm.fc2, bitween_amd.QuantizedLinear)
    assert isinstance(qm.lm_head, torch.nn.Linear) and isinstance(model.fc1, torch.nn.Linear)
    assert repr(qm.fc1) == "QuantizedLinear(in_features=768, out_features=3072, bias=True, bits=4, group_size=128)"
    w = model.fc1.weight.data.float().cpu().numpy()
    qw, s, z, _ = orc.quantize_rtn(w, 4, 128)
    s16, z16 = orc.store_module_buffers(s, z)
    assert np.array_equal(qm.fc1.qweight.cpu().numpy(), qw)
    assert np.array_equal(_bits_of(qm.fc1.scale), s16.view(np.uint16))
    x = torch.randn(2, 5, 768, device="cuda", dtype=torch.float32, requires_grad=True)   # any dtype in, float16 out
    y = qm.fc1(x)
    assert y.shape == (2, 5, 3072) and y.dtype == torch.float16
    x16 = x.detach().half().cpu().numpy().reshape(10, 768)
    b16 = model.fc1.bias.data.cpu().numpy()
    check_matmul(y.reshape(10, 3072), x16, qw, s16, z16, b16, 4, 128)
    go = torch.randn_like(y)
    y.backward(go)
    gref = orc.qlinear_backward(go.reshape(10, 3072).cpu().numpy(), qw, s16, z16, 4, 128)
    got = x.grad.reshape(10, 768).double().cpu().numpy()
    assert np.abs(got - gref).max() <= 1e-2 * np.abs(gref).max()
    # state_dict round trip keeps the reference's buffer names
    assert set(qm.fc1.state_dict().keys()) == {"qweight", "scale", "zero_point", "bias"}


def test_precision_map_and_perturbed_quantize():
    """The "next" rows either side of the path: a per-layer (bits, group_size) map applied in place, and
    quantize_rtn(orig_weight + value) fused into the quantiser (bitween/wrapper.py:222-232)."""
    import bitween_amd
    torch.manual_seed(3)
    model = torch.nn.ModuleDict({"blk0": torch.nn.ModuleDict({"a": torch.nn.Linear(256, 64), "b": torch.nn.Linear(256, 64)}),
                                 "blk1": torch.nn.ModuleDict({"a": torch.nn.Linear(256, 64)}),
                                 "head": torch.nn.Linear(256, 10)}).half().cuda()
    ref = {n: m.weight.data.float().cpu().numpy() for n, m in model.named_modules() if isinstance(m, torch.nn.Linear)}
    bitween_amd.apply_precision_map(model, {"blk0": (8, 128), "blk0.b": {"bits": 2, "group_size": 32}, "blk1.a": (4, 64)})
    for name, (bits, g) in (("blk0.a", (8, 128)), ("blk0.b", (2, 32)), ("blk1.a", (4, 64))):
        q = model.get_submodule(name)
        assert isinstance(q, bitween_amd.QuantizedLinear) and (q.bits, q.group_size) == (bits, g)
        qw, s, z, _ = orc.quantize_rtn(ref[name], bits, g)
        s16, z16 = orc.store_module_buffers(s, z)
        assert np.array_equal(q.qweight.cpu().numpy(), qw) and np.array_equal(_bits_of(q.scale), s16.view(np.uint16))
        assert np.array_equal(_bits_of(q.zero_point), z16.view(np.uint16))
    assert isinstance(model["head"], torch.nn.Linear)
    # perturbed quantise, in float32 and in float16 (where the sum is rounded to float16 first)
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((24, 384)) * 0.02).astype(np.float32)
    v = (rng.standard_normal((24, 384)) * 0.002).astype(np.float32)
    for bits, g in ((4, 128), (8, 32), (2, 64), (4, 48)):
        qw, s, z, _ = bitween_amd.quantize_rtn_perturbed(torch.from_numpy(w).cuda(), torch.from_numpy(v).cuda(), bits, g)
        qw_o, s_o, z_o, _ = orc.quantize_rtn((w + v).astype(np.float32), bits, g)
        assert np.array_equal(qw.cpu().numpy(), qw_o) and np.array_equal(_bits_of(s), s_o.view(np.uint32))
        assert np.array_equal(z.cpu().numpy(), z_o)
        w16, v16 = torch.from_numpy(w).half(), torch.from_numpy(v).half()
        qw, s, z, _ = bitween_amd.quantize_rtn_perturbed(w16.cuda(), v16.cuda(), bits, g)
        summed = (w16 + v16)                                            # eager float16 add on the host
        qw_o, s_o, z_o, _ = orc.quantize_rtn(summed.float().numpy(), bits, g, math="f16")
        assert np.array_equal(qw.cpu().numpy(), qw_o) and np.array_equal(z.cpu().numpy(), z_o)
        assert np.array_equal(_bits_of(s), s_o.astype(np.float16).view(np.uint16))


def test_sibling_linears_share_a_launch():
    """fuse_sibling_linears: q/k/v (and gate/up) read one input; grouped, the first call computes all of them and
    the siblings return slices.  Results, state_dict and behaviour after copies / in-place input edits must not change."""
    import copy
    import io
    import bitween_amd
    torch.manual_seed(11)

    model = _QkvBlock().half().cuda()
    qm = bitween_amd.Bitween(model, bits=4, group_size=128).quantize(verbose=False)
    x = torch.randn(3, 256, device="cuda", dtype=torch.float16)
    with torch.no_grad():
        before = [t.clone() for t in qm(x)]
        sd_before = {k: v.clone() for k, v in qm.state_dict().items()}
        assert bitween_amd.fuse_sibling_linears(qm) == 1
        calls = []
        real = bitween_amd.kernels.hip_loader.quantized_matmul_hip
        bitween_amd.modules._hip.quantized_matmul_hip = lambda *a, **k: (calls.append(a[1].shape[0]), real(*a, **k))[1]
        try:
            after = qm(x)
            assert calls == [256]                                   # one launch over the 128 + 64 + 64 rows
            for a, b in zip(after, before):
                assert torch.equal(a, b)
            x2 = x.clone()
            r1 = qm.q_proj(x2)
            x2.mul_(2.0)                                            # same tensor object, new contents
            r2 = qm.k_proj(x2)
            assert torch.equal(r2, real(x2, qm.k_proj.qweight, qm.k_proj.scale, qm.k_proj.zero_point, qm.k_proj.bias, 4, 128))
            assert calls[-2:] == [256, 256] and r1.shape == (3, 128)
        finally:
            bitween_amd.modules._hip.quantized_matmul_hip = real
        # siblings fed different inputs (cross-attention style) stop being grouped after a few wasted launches
        cross = copy.deepcopy(qm)
        outs = []
        for i in range(8):
            xa, xb = torch.randn_like(x), torch.randn_like(x)
            outs.append((cross.q_proj(xa), cross.k_proj(xb), xa, xb))
        assert cross.q_proj.__dict__["_sibling_group"].wasted >= 4
        qa, kb, xa, xb = outs[-1]
        assert torch.equal(qa, real(xa, qm.q_proj.qweight, qm.q_proj.scale, qm.q_proj.zero_point, qm.q_proj.bias, 4, 128))
        assert torch.equal(kb, real(xb, qm.k_proj.qweight, qm.k_proj.scale, qm.k_proj.zero_point, qm.k_proj.bias, 4, 128))
        sd_after = qm.state_dict()
        assert set(sd_after) == set(sd_before) and all(torch.equal(sd_after[k], sd_before[k]) for k in sd_before)
        # copies and pickles keep working (fused when the views survive, per layer otherwise)
        for clone in (copy.deepcopy(qm), torch.load(io.BytesIO(_saved(qm)), weights_only=False)):
            for a, b in zip(clone(x), before):
                assert torch.equal(a, b)
        # gradients bypass the group
        xg = x.clone().requires_grad_(True)
    y = qm.q_proj(xg)
    y.float().sum().backward()
    assert xg.grad is not None and xg.grad.shape == x.shape


class _QkvBlock(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.q_proj = torch.nn.Linear(256, 128)
        self.k_proj = torch.nn.Linear(256, 64)
        self.v_proj = torch.nn.Linear(256, 64)
        self.o_proj = torch.nn.Linear(128, 256)

    def forward(self, x):
        return self.q_proj(x), self.k_proj(x), self.v_proj(x)


def _saved(model):
    import io
    buf = io.BytesIO()
    torch.save(model, buf)
    return buf.getvalue()


def test_error_conventions_on_gpu():
    import bitween_amd
    w = torch.zeros(4, 100, device="cuda")
    with pytest.raises(ValueError):
        bitween_amd.quantize_rtn(w, 4, 32)
    with pytest.raises(AssertionError):
        bitween_amd.quantize_rtn(torch.zeros(4, 96, device="cuda"), 3, 32)
    with pytest.raises(ValueError):
        bitween_amd.QuantizedLinear(64, 64, bits=3)
    with pytest.raises(ValueError):
        bitween_amd.QuantizedLinear(64, 64, bits=4, group_size=0)
    # CPU tensors are staged through the GPU and come back on the CPU
    qw, s, z, _ = bitween_amd.quantize_rtn(torch.randn(8, 128), 4, 32)
    assert qw.device.type == "cpu" and s.device.type == "cpu"


@pytest.mark.parametrize("bits,g,k,n", [(4, 128, 4096, 11008), (4, 128, 11008, 4096), (8, 128, 4096, 11008),
                                        (4, 64, 4096, 11008), (2, 32, 4096, 11008), (4, 128, 4096, 4096),
                                        (4, 32, 11008, 4096), (4, 64, 11008, 4096), (2, 32, 11008, 4096),
                                        # the attention linears of the mixed recipe: 8-bit on 4096 x 4096 and on the fused
                                        # q/k/v launch (N = 12288); 8-bit on a long K and at the smaller groups
                                        (8, 128, 4096, 4096), (8, 128, 4096, 12288), (8, 128, 11008, 4096),
                                        (8, 64, 4096, 4096), (8, 32, 4096, 11008)])
def test_full_size_properties(bits, g, k, n):
    """Full-size layers (Llama-2-7B shapes), checked through size-independent properties:
      * a one-hot activation row returns a column of W16 bit-for-bit (the fused kernels reproduce the
        reference's dequantised weights exactly), for the decode and the prefill kernel;
      * quantise -> dequantise stays within half a step of the input for unclamped elements;
      * a strided sample of rows matches the oracle (quantiser bit-exact, GEMV to tolerance)."""
    hip = _hip()
    g_t = torch.Generator(device="cuda").manual_seed(bits * 131 + g)
    w = (torch.randn(n, k, device="cuda", generator=g_t) * 0.02)
    w = torch.where(torch.rand(n, k, device="cuda", generator=g_t) < 0.001, w * 10, w).half()
    layer = torch.nn.Linear(k, n, bias=False, device="cuda", dtype=torch.float16)
    layer.weight.data = w
    import bitween_amd
    q = bitween_amd.QuantizedLinear.from_float(layer, bits, g)
    w16 = hip.dequantize(q.qweight, q.scale, q.zero_point, g, bits, torch.float16)
    # one-hot rows
    cols = [0, 1, 7, 8, 31, k // 2 + 3, k - 1]
    for m_pad, fn in ((len(cols), hip.quantized_gemv_hip), (130, hip.quantized_gemm_hip)):
        x = torch.zeros(m_pad, k, device="cuda", dtype=torch.float16)
        for i, c in enumerate(cols):
            x[i, c] = 1.0
        y = fn(x, q.qweight, q.scale, q.zero_point, None, bits, g)
        for i, c in enumerate(cols):
            assert torch.equal(y[i], w16[:, c])              # value compare: the accumulator turns -0 into +0
        assert (y[len(cols):] == 0).all()
    # the same through the one- and two-row decode kernels (W4: the subnormal-operand kernel)
    for i in range(0, len(cols) - 1, 2):
        x = torch.zeros(2, k, device="cuda", dtype=torch.float16)
        x[0, cols[i]] = 1.0
        x[1, cols[i + 1]] = 1.0
        y2 = hip.quantized_gemv_hip(x, q.qweight, q.scale, q.zero_point, None, bits, g)
        y1 = hip.quantized_gemv_hip(x[1:], q.qweight, q.scale, q.zero_point, None, bits, g)
        assert torch.equal(y2[0], w16[:, cols[i]]) and torch.equal(y2[1], w16[:, cols[i + 1]])
        assert torch.equal(y1[0], w16[:, cols[i + 1]])
    # and through the three- and four-row forms (4-bit groups of 128 and 8-bit: still the subnormal-operand kernels)
    for m in (3, 4):
        x = torch.zeros(m, k, device="cuda", dtype=torch.float16)
        for i in range(m):
            x[i, cols[(i + m) % len(cols)]] = 1.0
        y = hip.quantized_gemv_hip(x, q.qweight, q.scale, q.zero_point, None, bits, g)
        for i in range(m):
            assert torch.equal(y[i], w16[:, cols[(i + m) % len(cols)]])
    # reconstruction bound
    w32 = hip.dequantize(q.qweight, q.scale, q.zero_point, g, bits, torch.float32)
    qmax = (1 << bits) - 1
    rows = np.arange(0, n, max(1, n // 24))
    qs = orc.unpack_words(q.qweight[rows].cpu().numpy(), bits)
    inner = torch.from_numpy((qs > 0) & (qs < qmax)).cuda()
    step = q.scale[rows].float().repeat_interleave(g, dim=1)
    # scale was rounded to f16 on store: allow its relative 2^-11 on |q - z| <= qmax steps
    err = (w32[rows] - w[rows].float()).abs()
    assert (err[inner] <= (0.5 + qmax * 2.0 ** -11) * step[inner] * 1.001).all()
    # sampled rows against the oracle
    w_rows = w[rows].float().cpu().numpy()
    qw_o, s_o, z_o, _ = orc.quantize_rtn(w_rows, bits, g)
    s16, z16 = orc.store_module_buffers(s_o, z_o)
    assert np.array_equal(q.qweight[rows].cpu().numpy(), qw_o)
    assert np.array_equal(_bits_of(q.scale[rows]), s16.view(np.uint16))
    assert np.array_equal(q.zero_point[rows].float().cpu().numpy(), z_o.astype(np.float32))
    for m in (1, 2, 4, 8, 16):
        x = torch.randn(m, k, device="cuda", dtype=torch.float16, generator=g_t)
        y = q(x)
        check_matmul(y[:, rows], x.cpu().numpy(), qw_o, s16, z16, None, bits, g)
    # one-hot rows through the 16-row decode kernels as well (rows 7..15 stay zero)
    x = torch.zeros(16, k, device="cuda", dtype=torch.float16)
    for i, c in enumerate(cols):
        x[2 * i, c] = 1.0
    y = hip.quantized_gemv_hip(x, q.qweight, q.scale, q.zero_point, None, bits, g)
    for i, c in enumerate(cols):
        assert torch.equal(y[2 * i], w16[:, c])
    assert (y[1::2] == 0).all()
    x = torch.randn(256, k, device="cuda", dtype=torch.float16, generator=g_t)
    y = q(x)
    check_matmul(y[:, rows], x.cpu().numpy(), qw_o, s16, z16, None, bits, g)


@pytest.mark.parametrize("bits,g", COMBOS)
def test_bfloat16_activations_are_rounded_to_float16_in_the_kernel(bits, g):
    """x.to(float16) of the reference's forward (bitween/modules.py:74) fused into the decode kernels: a bfloat16 x
    gives bit for bit what its float16 rounding gives, for every decode kernel variant, through bw_qlinear's 16-row
    slices and (cast on the host side) through the prefill kernel; tiny and huge values included."""
    hip = _hip()
    k, n = 1024, 272
    _, qw, s16, z16, b16 = quantized_layer(n, k, bits, g, seed=bits * 31 + g, outliers=True)
    d = [to_gpu(a) for a in (qw, s16, z16, b16)]
    gen = torch.Generator(device="cuda").manual_seed(bits + g)
    for m in (1, 2, 3, 8, 16, 17, 48, 64):
        xb = torch.randn(m, k, device="cuda", generator=gen).to(torch.bfloat16)
        xb[0, 0] = 3.0e-6          # below the float16 normal range: rounds to a subnormal
        xb[0, 1] = 1.0e-9          # rounds to zero
        xb[0, 2] = 60000.0
        xh = xb.to(torch.float16)
        y_b = hip.quantized_matmul_hip(xb, d[0], d[1], d[2], d[3], bits, g)
        y_h = hip.quantized_matmul_hip(xh, d[0], d[1], d[2], d[3], bits, g)
        assert y_b.dtype == torch.float16 and torch.equal(y_b, y_h)
        if m <= 16:
            assert torch.equal(hip.quantized_gemv_hip(xb, d[0], d[1], d[2], d[3], bits, g), y_h)
    check_matmul(y_b, xh.cpu().numpy(), qw, s16, z16, b16, bits, g)
    import bitween_amd
    q = bitween_amd.QuantizedLinear(k, n, bits=bits, group_size=g, bias=True).cuda()
    q.qweight.copy_(d[0]); q.scale.copy_(d[1]); q.zero_point.copy_(d[2]); q.bias.copy_(d[3])
    xb = torch.randn(2, 3, k, device="cuda", generator=gen).to(torch.bfloat16)
    assert torch.equal(q(xb), q(xb.to(torch.float16)))


def test_bfloat16_activations_on_a_shape_only_the_generic_kernel_takes():
    """Group size 48 is outside the fast layouts: the C ABI answers BW_EUNSUPPORTED for bfloat16 there and the
    Python forward casts to float16 and calls again."""
    import bitween_amd
    torch.manual_seed(3)
    lin = torch.nn.Linear(96, 40, bias=True, device="cuda", dtype=torch.float16)
    q = bitween_amd.QuantizedLinear.from_float(lin, 4, 48)
    xb = torch.randn(5, 96, device="cuda").to(torch.bfloat16)
    y = q(xb)
    assert y.dtype == torch.float16 and torch.equal(y, q(xb.to(torch.float16)))
    check_matmul(y, xb.to(torch.float16).cpu().numpy(), q.qweight.cpu().numpy(), q.scale.cpu().numpy(),
                 q.zero_point.cpu().numpy(), q.bias.cpu().numpy(), 4, 48)


def test_validated_buffer_cache_follows_replaced_buffers():
    """The decode path validates a layer's buffers once and afterwards only checks that they are still the same
    tensors at the same address.  Every way of changing them must be seen: in-place load, a replaced buffer, a
    deep copy, a pickle round trip, a move off the GPU and back."""
    import copy
    import io
    import bitween_amd
    torch.manual_seed(11)
    k, n = 256, 96
    lin_a = torch.nn.Linear(k, n, bias=True, device="cuda", dtype=torch.float16)
    lin_b = torch.nn.Linear(k, n, bias=True, device="cuda", dtype=torch.float16)
    qa = bitween_amd.QuantizedLinear.from_float(lin_a, 4, 64)
    qb = bitween_amd.QuantizedLinear.from_float(lin_b, 4, 64)
    x = torch.randn(3, k, device="cuda", dtype=torch.float16)
    hip = _hip()

    def direct(q):
        return hip.quantized_matmul_hip(x, q.qweight, q.scale, q.zero_point, q.bias, q.bits, q.group_size)

    ya, yb = direct(qa), direct(qb)
    assert not torch.equal(ya, yb)
    assert torch.equal(qa(x), ya) and "_decode_plan" in qa.__dict__
    qa.load_state_dict(qb.state_dict())                       # in place: same tensors, new contents
    assert torch.equal(qa(x), yb)
    qa.qweight = qa.qweight.clone()                           # a replaced buffer
    qa.scale = torch.zeros_like(qa.scale)
    assert torch.equal(qa(x), direct(qa)) and (qa(x) == qa.bias).all()
    qc = copy.deepcopy(qb)
    assert "_decode_plan" not in qc.__dict__ and torch.equal(qc(x), yb)
    buf = io.BytesIO()
    torch.save(qb, buf)
    buf.seek(0)
    qd = torch.load(buf, weights_only=False)                  # our own file
    assert torch.equal(qd(x), yb)
    qe = qb.to("cpu").to("cuda")                              # new tensors at new addresses
    assert torch.equal(qe(x), yb)
    lin_c = torch.nn.Linear(k, n, bias=False, device="cuda", dtype=torch.float16)
    qf = bitween_amd.QuantizedLinear.from_float(lin_c, 8, 32)
    assert torch.equal(qf(x), direct(qf))
    assert torch.equal(qf(x.to(torch.bfloat16)), qf(x.to(torch.bfloat16).to(torch.float16)))
    xs = torch.randn(3, 2 * k, device="cuda", dtype=torch.float16)[:, ::2]     # strided x falls back to the general path
    assert torch.equal(qf(xs), qf(xs.contiguous()))
    # same Python objects, new storage: `.data = ...` and `.set_()` on scale, zero_point and bias
    qg = bitween_amd.QuantizedLinear.from_float(lin_a, 4, 64)
    assert torch.equal(qg(x), ya)
    keep = [qg.scale.data, qg.zero_point.data, qg.bias.data]  # the old blocks stay allocated: the test must not depend on reuse
    scale_obj, zp_obj, bias_obj = qg.scale, qg.zero_point, qg.bias
    qg.scale.data = qb.scale.clone()
    assert qg.scale is scale_obj and torch.equal(qg(x), direct(qg)) and not torch.equal(qg(x), ya)
    qg.zero_point.set_(qb.zero_point.clone())
    assert qg.zero_point is zp_obj and torch.equal(qg(x), direct(qg))
    qg.bias.data = torch.zeros_like(qg.bias)
    assert qg.bias is bias_obj and torch.equal(qg(x), direct(qg))
    qg.qweight.data = qb.qweight.clone()
    assert torch.equal(qg(x), hip.quantized_matmul_hip(x, qb.qweight, qb.scale, qb.zero_point, None, 4, 64))
    del keep
    # and in a sibling group: a member whose scale was re-pointed leaves the group and answers for itself
    blk = torch.nn.Module()
    blk.gate_proj = bitween_amd.QuantizedLinear.from_float(lin_a, 4, 64)
    blk.up_proj = bitween_amd.QuantizedLinear.from_float(lin_b, 4, 64)
    assert bitween_amd.fuse_sibling_linears(blk) == 1
    with torch.no_grad():
        assert torch.equal(blk.gate_proj(x), ya) and torch.equal(blk.up_proj(x), yb)
        blk.up_proj.scale.data = qa.scale.clone()
        x2 = x.clone()
        assert torch.equal(blk.gate_proj(x2), ya)
        assert torch.equal(blk.up_proj(x2), hip.quantized_matmul_hip(x, qb.qweight, qa.scale, qb.zero_point, qb.bias, 4, 64))


def test_bf16_cast_matches_tensor_cast_bit_for_bit():
    """bw_cast_bf16_f16 is the x.to(float16) of the reference's forward (bitween/modules.py:74): every bfloat16 bit
    pattern, through a padded row pitch on both sides, against torch's own cast."""
    import ctypes
    from bitween_amd.kernels import hip_loader as hip
    lib = hip.load()
    allbits = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16).cuda().view(torch.bfloat16)   # 65536 patterns
    rows, cols, ldx, ldy = 64, 1024, 1024 + 8, 1024 + 24
    xbuf = torch.zeros((rows, ldx), dtype=torch.bfloat16, device="cuda")
    xbuf[:, :cols] = allbits.view(rows, cols)
    ybuf = torch.full((rows, ldy), 7.0, dtype=torch.float16, device="cuda")
    st = lib.bw_cast_bf16_f16(xbuf.data_ptr(), rows, cols, ldx, ybuf.data_ptr(), ldy,
                              ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert st == 0
    torch.cuda.synchronize()
    want = xbuf[:, :cols].to(torch.float16)
    assert torch.equal(ybuf[:, :cols].view(torch.int16), want.view(torch.int16))
    assert (ybuf[:, cols:] == 7.0).all()
    # layouts the kernel does not take are refused, and the Python forward falls back to the tensor cast
    assert lib.bw_cast_bf16_f16(xbuf.data_ptr(), rows, 1020, ldx, ybuf.data_ptr(), ldy, None) == -2
    assert lib.bw_cast_bf16_f16(xbuf.data_ptr() + 2, rows, cols, ldx, ybuf.data_ptr(), ldy, None) == -3
    for shape in ((200, 1020), (64, 4096), (2048, 4096)):      # odd K, below and above the size where the kernel takes over
        x = torch.randn(*shape, device="cuda").to(torch.bfloat16)
        assert torch.equal(hip._bf16_to_f16(x), x.to(torch.float16))


@pytest.mark.parametrize("m,dtype", [(1, torch.float16), (16, torch.bfloat16), (64, torch.float16), (160, torch.float16),
                                      (2048, torch.bfloat16)])
def test_forward_under_graph_capture_replays_like_eager(m, dtype):
    """A captured forward of two QuantizedLinear layers (decode, 16-row launches, prefill with its split-K workspace
    and, for bfloat16 prefill input, the cast kernel) replayed with new inputs gives what the eager call gives,
    bit for bit, on every replay; eager work and synchronisations sit between the replays."""
    from bitween_amd import QuantizedLinear
    torch.manual_seed(m)
    k, h = 2048, 1024
    lin1 = torch.nn.Linear(k, h, bias=True, dtype=torch.float16, device="cuda")
    lin2 = torch.nn.Linear(h, k, bias=False, dtype=torch.float16, device="cuda")
    q1 = QuantizedLinear.from_float(lin1, bits=4, group_size=128)
    q2 = QuantizedLinear.from_float(lin2, bits=8, group_size=64)

    def net(x):
        return q2(torch.nn.functional.silu(q1(x)).to(dtype))

    static_x = torch.randn(m, k, device="cuda").to(dtype)
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                net(static_x)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_y = net(static_x)
        for i in range(4):
            x = torch.randn(m, k, device="cuda").to(dtype) * (1 + i)
            want = net(x)
            torch.cuda.synchronize()
            static_x.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_y, want), f"replay {i}"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits,switch,ms", [(4, 32, (32, 33, 40, 48)), (8, 16, (16, 17, 32, 33))])
def test_rows_33_to_48_on_a_large_layer_take_the_prefill_kernel(dtype, bits, switch, ms):
    """For a layer of 10 MiB of packed weights and more bw_qlinear hands 33-48 rows to the prefill kernel, from 40 MiB on
    (4096 -> 11008 at 8 bits) 17-32 rows too; the module forward (validated-buffer path, bfloat16 cast included) must
    follow it and agree with the C entry point."""
    import ctypes
    from bitween_amd import QuantizedLinear
    from bitween_amd.kernels import hip_loader as hip
    lib = hip.load()
    k, n, g = 4096, 11008, 128
    assert lib.bw_qlinear_decode_rows(n, k, bits) == switch
    lin = torch.nn.Linear(k, n, bias=True, dtype=torch.float16, device="cuda")
    q = QuantizedLinear.from_float(lin, bits=bits, group_size=g)
    w16 = hip.dequantize(q.qweight, q.scale, q.zero_point, g, bits, torch.float16)
    for m in ms:
        x = torch.randn(m, k, device="cuda").to(dtype)
        with torch.no_grad():
            y = q(x)
        x16 = x.to(torch.float16)
        ref = x16.double() @ w16.double().T + q.bias.double()
        mag = x16.double().abs() @ w16.double().abs().T + 1.0
        assert ((y.double() - ref).abs() <= 2.0 ** -10 * ref.abs() + 2.0 ** -12 * mag).all()
        yc = torch.empty_like(y)
        st = lib.bw_qlinear(x16.data_ptr(), 0, m, k, k, q.qweight.data_ptr(), q.scale.data_ptr(), q.zero_point.data_ptr(),
                            q.bias.data_ptr(), n, bits, g, yc.data_ptr(), n, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert st == 0
        torch.cuda.synchronize()
        if m <= switch:
            assert torch.equal(y, yc)                            # same decode launches either way
        else:
            assert ((y.double() - yc.double()).abs() <= 2.0 ** -9 * ref.abs() + 2.0 ** -12 * mag).all()   # split-K or not


@pytest.mark.parametrize("k,n", [(4096, 14336), (14336, 4096)])
@pytest.mark.parametrize("m", [128, 512, 2048])
@pytest.mark.parametrize("xdtype", [torch.float16, torch.bfloat16])
def test_prefill_llama3_8b_mlp_shapes_at_full_size(k, n, m, xdtype):
    """The prefill configuration at its own shapes (Llama-3-8B MLP, 4-bit g128, 128 / 512 / 2048 rows, float16 and
    bfloat16 activations): through the split and the unsplit plan, one-hot rows return columns of W16 bit for bit and
    random rows meet the matmul bars on a strided sample of output columns whose weights the oracle quantised
    (main.py:444-466 is the formula, x.to(float16) of modules.py:74 for bfloat16)."""
    import ctypes
    hip = _hip()
    lib = hip.load()
    bits, g = 4, 128
    g_t = torch.Generator(device="cuda").manual_seed(k // 7 + m)
    w = (torch.randn(n, k, device="cuda", generator=g_t) * 0.02).half()
    layer = torch.nn.Linear(k, n, bias=False, device="cuda", dtype=torch.float16)
    layer.weight.data = w
    import bitween_amd
    q = bitween_amd.QuantizedLinear.from_float(layer, bits, g)
    w16 = hip.dequantize(q.qweight, q.scale, q.zero_point, g, bits, torch.float16)
    rows = np.unique(np.concatenate([np.arange(0, n, n // 40), [255, 256, n - 257, n - 1]]))
    qw_o, s_o, z_o, _ = orc.quantize_rtn(w[rows].float().cpu().numpy(), bits, g)
    s16, z16 = orc.store_module_buffers(s_o, z_o)
    assert np.array_equal(q.qweight[rows].cpu().numpy(), qw_o)
    x = torch.randn(m, k, device="cuda", generator=g_t).to(xdtype)
    hot = {0: 0, 1: k - 1, 5: 129, m // 2 + 1: k // 2, m - 1: 4095}            # row -> column of its single 1
    for r, c in hot.items():
        x[r] = 0
        x[r, c] = 1.0
    x16 = x.to(torch.float16)
    # the forward as the module runs it (bfloat16 cast + split-K workspace where the plan wants one)
    y_split = hip.quantized_matmul_hip(x, q.qweight, q.scale, q.zero_point, None, bits, g)
    # the same kernel without a workspace: nothing is split
    y_plain = torch.empty((m, n), dtype=torch.float16, device="cuda")
    st = lib.bw_qgemm(x16.data_ptr(), 0, m, k, k, q.qweight.data_ptr(), q.scale.data_ptr(), q.zero_point.data_ptr(), None, n,
                      bits, g, y_plain.data_ptr(), n, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert st == 0
    torch.cuda.synchronize()
    x_np = x16.cpu().numpy()
    for y in (y_split, y_plain):
        for r, c in hot.items():
            assert torch.equal(y[r], w16[:, c])
        check_matmul(y[:, rows], x_np, qw_o, s16, z16, None, bits, g)


@pytest.mark.parametrize("bits,g", [(4, 64), (8, 64), (2, 128)])
@pytest.mark.parametrize("groups", [8, 10, 12, 20])
@pytest.mark.parametrize("m", [40, 200])
def test_prefill_formats_with_two_groups_per_k_step(bits, g, groups, m):
    """Formats whose K step spans two groups (4 and 8 bits at g64, 2 bits at g128): with a multiple of four groups the
    prefill kernel fetches the scales of two steps in one 8-byte request per tile, else per step and lane - both
    against the oracle, split and unsplit, one-hot rows bit for bit, and the two plans on shapes that differ only in
    taking one or the other."""
    import ctypes
    hip = _hip()
    lib = hip.load()
    k, n = g * groups, 300
    _, qw, s16, z16, b16 = quantized_layer(n, k, bits, g, seed=bits * 1000 + groups, outliers=True)
    rng = np.random.default_rng(groups + m)
    x = rng.standard_normal((m, k)).astype(np.float16)
    hot = {0: 0, 3: k - 1, m - 1: k // 2 + 1}
    for r, c in hot.items():
        x[r] = 0
        x[r, c] = 1
    d = [to_gpu(a) for a in (x, qw, s16, z16, b16)]
    w16 = orc.dequantize_f16(qw, s16, z16, g, bits)
    y_ws = hip.quantized_gemm_hip(d[0], d[1], d[2], d[3], None, bits, g)
    y_plain = torch.empty((m, n), dtype=torch.float16, device="cuda")
    assert lib.bw_qgemm(d[0].data_ptr(), 0, m, k, k, d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), d[4].data_ptr(), n, bits, g,
                        y_plain.data_ptr(), n, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
    torch.cuda.synchronize()
    check_matmul(y_ws, x, qw, s16, z16, None, bits, g)
    check_matmul(y_plain, x, qw, s16, z16, b16, bits, g)
    for r, c in hot.items():
        assert np.array_equal(y_ws[r].cpu().numpy().view(np.uint16), w16[:, c].view(np.uint16))


def test_sibling_group_does_not_serve_a_member_twice_from_its_cache():
    """An input rewritten in place without a version bump (.data) and handed to the same member again gets a new
    launch, not the cached slice."""
    import bitween_amd
    torch.manual_seed(0)
    blk = torch.nn.Module()
    for name in ("q_proj", "k_proj", "v_proj"):
        lin = torch.nn.Linear(256, 128, bias=False, device="cuda", dtype=torch.float16)
        setattr(blk, name, bitween_amd.QuantizedLinear.from_float(lin, 4, 128))
    assert bitween_amd.fuse_sibling_linears(blk) == 1
    x = torch.randn(1, 256, device="cuda", dtype=torch.float16)
    with torch.no_grad():
        y1 = blk.q_proj(x).clone()
        version = x._version
        x.data.mul_(2.0)
        assert x._version == version                      # the rewrite is invisible to the version counter
        y2 = blk.q_proj(x)
        k2 = blk.k_proj(x)
    assert torch.allclose(y2.float(), 2 * y1.float(), rtol=2e-3, atol=1e-3)
    ref_k = bitween_amd.kernels.hip_loader.quantized_matmul_hip(x, blk.k_proj.qweight, blk.k_proj.scale, blk.k_proj.zero_point, None, 4, 128)
    assert torch.equal(k2, ref_k)


@pytest.mark.parametrize("bits,g", [(4, 128), (4, 64), (4, 32), (8, 128), (8, 64), (8, 32), (2, 128), (2, 64), (2, 32)])
@pytest.mark.parametrize("k", [768, 896, 1024])
def test_prefill_256_row_tiles_vs_oracle(bits, g, k):
    """Shapes whose grid of 256-row tiles fills the device take the 256-row variant of the prefill kernel (same
    arithmetic as bitween/modules.py:85-97, twice the rows per unpacked weight): ragged in M and N, an even and an odd
    number of K steps (with and without the wide scale requests; 768 = six steps: a run of four and two steps after
    the loop), with and without bias - sampled rows from every part
    of the row range against the oracle, one-hot rows bit for bit, and the workspace plan against the plain one."""
    import ctypes
    hip = _hip()
    lib = hip.load()
    m, n = 256 * 52 + 37, 1000
    if lib.bw_qgemm_tile_rows(m, n, k, bits, g) != 256:
        pytest.skip("this device's CU count does not put the shape on 256-row tiles")
    _, qw, s16, z16, b16 = quantized_layer(n, k, bits, g, seed=bits * 100 + g + k, outliers=True)
    w16 = orc.dequantize_f16(qw, s16, z16, g, bits)
    gen = torch.Generator(device="cuda").manual_seed(k + bits)
    x = torch.randn(m, k, device="cuda", generator=gen).half()
    hot = {0: 0, 255: k - 1, 256: 129, 4001: k // 2, m - 38: 31, m - 1: k - 2}       # row -> column of its single 1
    for r, c in hot.items():
        x[r] = 0
        x[r, c] = 1.0
    d = [to_gpu(a) for a in (qw, s16, z16, b16)]
    y_ws = hip.quantized_gemm_hip(x, d[0], d[1], d[2], d[3], bits, g)
    y_plain = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
    assert lib.bw_qgemm(x.data_ptr(), 0, m, k, k, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), None, n, bits, g,
                        y_plain.data_ptr(), n, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
    torch.cuda.synchronize()
    rows = np.unique(np.concatenate([np.arange(0, m, 997), np.arange(250, 262), np.arange(m - 40, m)]))
    x_np = x[torch.from_numpy(rows).cuda()].cpu().numpy()
    check_matmul(y_ws[torch.from_numpy(rows).cuda()], x_np, qw, s16, z16, b16, bits, g)
    check_matmul(y_plain[torch.from_numpy(rows).cuda()], x_np, qw, s16, z16, None, bits, g)
    for r, c in hot.items():
        assert np.array_equal(y_plain[r].cpu().numpy().view(np.uint16), w16[:, c].view(np.uint16))
    # every row of the full result: finite, and equal to the library GEMM on the dequantised weights to float16 rounding
    ref = x @ to_gpu(w16).T
    assert torch.isfinite(y_plain).all()
    assert ((y_plain.float() - ref.float()).abs().max() <= 2.0 ** -8 * ref.float().abs().max()).item()


@pytest.mark.parametrize("bits,g", [(4, 128), (4, 64), (4, 32), (8, 128), (8, 64), (8, 32), (2, 128), (2, 64), (2, 32)])
def test_prefill_64_row_tiles_vs_oracle(bits, g):
    """Calls of at most 64 rows - and up to 128 rows where N is at most 16 tiles wide - run the prefill kernel with 64-row
    tiles (same arithmetic as bitween/modules.py:85-97): 17, 33, 64, 100 and 128 rows (one and two row tiles), ragged N, K of one / six / seven / 32 steps, split along K through the workspace and un-split,
    with and without bias - every row against the oracle, one-hot rows bit for bit."""
    import ctypes
    hip = _hip()
    lib = hip.load()
    n = 1000
    for k in (128, 768, 896, 4096):
        _, qw, s16, z16, b16 = quantized_layer(n, k, bits, g, seed=bits * 10 + g + k, outliers=True)
        w16 = orc.dequantize_f16(qw, s16, z16, g, bits)
        d = [to_gpu(a) for a in (qw, s16, z16, b16)]
        for m in (17, 33, 64, 100, 128):
            assert lib.bw_qgemm_tile_rows(m, n, k, bits, g) == 64
            gen = torch.Generator(device="cuda").manual_seed(k + bits + m)
            x = torch.randn(m, k, device="cuda", generator=gen).half()
            hot = {0: k - 1, m - 1: k // 2}
            for r, c in hot.items():
                x[r] = 0
                x[r, c] = 1.0
            y_ws = hip.quantized_gemm_hip(x, d[0], d[1], d[2], d[3], bits, g)          # with the split-K workspace
            y_plain = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
            assert lib.bw_qgemm(x.data_ptr(), 0, m, k, k, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), None, n, bits, g,
                                y_plain.data_ptr(), n, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
            torch.cuda.synchronize()
            x_np = x.cpu().numpy()
            check_matmul(y_ws, x_np, qw, s16, z16, b16, bits, g)
            check_matmul(y_plain, x_np, qw, s16, z16, None, bits, g)
            for r, c in hot.items():
                assert np.array_equal(y_plain[r].cpu().numpy().view(np.uint16), w16[:, c].view(np.uint16))


def test_prefill_256_row_tiles_split_the_short_last_round():
    """778 tiles of 256 rows on 256 CUs: three rounds and ten tiles, which are cut in two along K into partial tiles of
    256 x 256 floats that the reduce kernel adds up; against the un-split run everywhere and the oracle on rows of both
    kinds of tile."""
    import ctypes
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    bits, g, m, k, n = 4, 128, 256 * 389, 1024, 512
    need = lib.bw_qgemm_workspace_bytes(m, n, k, bits, g)
    if lib.bw_qgemm_tile_rows(m, n, k, bits, g) != 256 or need == 0:
        pytest.skip("this device's CU count leaves no short last round of 256-row tiles for this shape")
    assert need % (256 * 256 * 4) == 0 and need <= 64 * 256 * 256 * 4
    _, qw, s16, z16, b16 = quantized_layer(n, k, bits, g, seed=79, outliers=True)
    gen = torch.Generator(device="cuda").manual_seed(80)
    x = torch.randn(m, k, device="cuda", generator=gen).half()
    d = [to_gpu(a) for a in (qw, s16, z16, b16)]
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ys = []
    for ws_ptr, ws_bytes in ((ws.data_ptr(), need), (None, 0)):
        y = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
        assert lib.bw_qgemm_ws(x.data_ptr(), 0, m, k, k, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(),
                               n, bits, g, y.data_ptr(), n, ws_ptr, ws_bytes, st) == 0
        ys.append(y)
    torch.cuda.synchronize()
    assert torch.isfinite(ys[0]).all()
    diff = (ys[0].float() - ys[1].float()).abs().max().item()
    assert diff <= 2.0 ** -9 * ys[1].float().abs().max().item()
    rows = np.r_[0:20, m - 1300:m - 1280, m - 20:m]                      # a whole tile, and split tiles of the last round
    idx = torch.from_numpy(rows).cuda()
    check_matmul(ys[0][idx], x[idx].cpu().numpy(), qw, s16, z16, b16, bits, g)
