"""Pins the CPU oracle (oracle/rtn_oracle.py and oracle/rtn_oracle.c).

The reference holds no vectors for this path, so the oracle is pinned by:
  * tests/golden/rtn_exact_vectors.npz - expected values computed in exact
    rational arithmetic with explicit IEEE rounding (no float arithmetic);
  * hand-derived known answers written out literally below;
  * closed forms / invariants of the domain;
  * agreement between two independently written restatements (numpy, C).
"""
import os

import numpy as np
import pytest

from oracle import c_oracle, rtn_oracle as orc

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "rtn_exact_vectors.npz"))
ALL_CASES = [str(s) for s in GOLD["names"]]
CASES = [c for c in ALL_CASES if not c.endswith(":recip")]          # scale by true division (eager torch on the CPU)
RECIP_CASES = [c for c in ALL_CASES if c.endswith(":recip")]        # scale by the float32 reciprocal (eager torch on a GPU)


def _case(name):
    key, fmt, bits, g, kind = name.split(":")[:5]
    return key, fmt, int(bits), int(g), kind


@pytest.mark.parametrize("name", CASES)
def test_numpy_oracle_matches_exact_vectors(name):
    key, fmt, bits, g, _ = _case(name)
    w = GOLD[key + "_w"]
    valid = GOLD[key + "_valid"]
    qw, scale, zp, q = orc.quantize_rtn(w, bits, g, math=fmt)
    vq = np.repeat(valid, g, axis=1)
    assert np.array_equal(scale.view(np.uint32)[valid], GOLD[key + "_scale"].view(np.uint32)[valid])
    assert np.array_equal(zp[valid], GOLD[key + "_zp"][valid])
    assert np.array_equal(q[vq], GOLD[key + "_q"][vq])
    if valid.all():
        assert np.array_equal(qw, GOLD[key + "_qweight"])
        s16, z16 = orc.store_module_buffers(scale, zp)
        assert np.array_equal(s16.view(np.uint16), GOLD[key + "_scale16"].view(np.uint16))
        w16 = orc.dequantize_f16(qw, s16, z16, g, bits)
        assert np.array_equal(w16.view(np.uint16), GOLD[key + "_w16"].view(np.uint16))
        w32 = orc.dequantize_rtn_f32(qw, scale, zp, g, bits)
        assert np.array_equal(w32.view(np.uint32), GOLD[key + "_w32"].view(np.uint32))
        y, y64 = orc.qlinear_forward(GOLD[key + "_x"], qw, s16, z16, None, bits, g)
        ref = GOLD[key + "_y64"]
        assert np.allclose(y64, ref, rtol=1e-12, atol=1e-12 * np.abs(ref).max())


@pytest.mark.parametrize("name", RECIP_CASES)
def test_oracles_match_exact_vectors_with_reciprocal_scale(name):
    """scale = RN(RN32((max - min) * RN32(1 / Qmax))): the arithmetic of eager torch on a GPU for functional.py:25."""
    key, fmt, bits, g, _ = _case(name)
    w = GOLD[key + "_w"]
    valid = GOLD[key + "_valid"]
    qw, scale, zp, q = orc.quantize_rtn(w, bits, g, math=fmt, scale_div="reciprocal")
    vq = np.repeat(valid, g, axis=1)
    assert np.array_equal(scale.view(np.uint32)[valid], GOLD[key + "_scale"].view(np.uint32)[valid])
    assert np.array_equal(zp[valid], GOLD[key + "_zp"][valid])
    assert np.array_equal(q[vq], GOLD[key + "_q"][vq])
    if valid.all():
        assert np.array_equal(qw, GOLD[key + "_qweight"])
    if fmt == "f32":
        qw_c, s_c, z_c = c_oracle.quantize_rtn_f32(w, bits, g, scale_div="reciprocal")
        assert np.array_equal(qw_c, GOLD[key + "_qweight"]) and np.array_equal(z_c, GOLD[key + "_zp"])
        assert np.array_equal(s_c.view(np.uint32), GOLD[key + "_scale"].view(np.uint32))


def test_reciprocal_scale_differs_from_true_division_where_expected():
    """The two roundings are different functions: on random float32 ranges most scales differ by one ulp (the
    flag is not a no-op), while zero points and packed values move only in a few groups."""
    w = (np.random.default_rng(5).standard_normal((64, 1024)) * 0.02).astype(np.float32)
    _, s_a, z_a, q_a = orc.quantize_rtn(w, 4, 128)
    _, s_b, z_b, q_b = orc.quantize_rtn(w, 4, 128, scale_div="reciprocal")
    differ = (s_a.view(np.uint32) != s_b.view(np.uint32)).mean()
    assert 0.3 < differ < 0.95
    assert np.abs(s_a.view(np.int32).astype(np.int64) - s_b.view(np.int32).astype(np.int64)).max() <= 1
    assert (q_a != q_b).mean() < 0.01


@pytest.mark.parametrize("name", [c for c in CASES if c.split(":")[1] == "f32"])
def test_c_oracle_matches_exact_vectors(name):
    key, _, bits, g, _ = _case(name)
    w = GOLD[key + "_w"]
    qw, scale, zp = c_oracle.quantize_rtn_f32(w, bits, g)
    assert np.array_equal(qw, GOLD[key + "_qweight"])
    assert np.array_equal(scale.view(np.uint32), GOLD[key + "_scale"].view(np.uint32))
    assert np.array_equal(zp, GOLD[key + "_zp"])
    s16 = GOLD[key + "_scale16"]
    z16 = zp.astype(np.float16)
    assert np.array_equal(c_oracle.dequantize_f16(qw, s16, z16, g, bits).view(np.uint16), GOLD[key + "_w16"].view(np.uint16))
    assert np.array_equal(c_oracle.dequantize_f32(qw, scale, zp, g, bits).view(np.uint32), GOLD[key + "_w32"].view(np.uint32))
    y = c_oracle.qlinear_forward(GOLD[key + "_x"], qw, s16, z16, None, bits, g)
    with np.errstate(over="ignore"):
        ref = GOLD[key + "_y64"].astype(np.float32).astype(np.float16)
    assert np.array_equal(y.view(np.uint16), ref.view(np.uint16))


def test_c_f16_conversion_is_rne_for_every_half_and_midpoint():
    lib = c_oracle.load()
    import ctypes
    lib.orc_f32_to_f16.restype = ctypes.c_uint16
    lib.orc_f32_to_f16.argtypes = [ctypes.c_float]
    lib.orc_f16_to_f32.restype = ctypes.c_float
    lib.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
    halves = np.arange(0, 0x7C00, dtype=np.uint16)
    vals = halves.view(np.float16).astype(np.float32)
    for h in range(0, 0x7C00, 7):
        assert lib.orc_f16_to_f32(h) == vals[h]
        assert lib.orc_f32_to_f16(float(vals[h])) == h
    rng = np.random.default_rng(5)
    probe = np.concatenate([(vals[:-1] + vals[1:]) / 2,                      # exact midpoints
                            rng.standard_normal(4000).astype(np.float32) * 1e-4,
                            rng.standard_normal(4000).astype(np.float32) * 100,
                            np.array([1e-8, 6e-8, 2.98e-8, 2.9802322e-8, 65504, 65519.9, 65520, 1e30], np.float32)])
    with np.errstate(over="ignore"):
        expect = probe.astype(np.float16).view(np.uint16)
    got = np.array([lib.orc_f32_to_f16(float(v)) for v in probe], np.uint16)
    assert np.array_equal(got, expect)


# ---- hand-derived known answers -------------------------------------------------

def test_kat_identity_ramp_4bit():
    # min 0, max 15 -> scale (15-0)/15 = 1, zp = round(-0/1) = 0, q = w.
    w = np.arange(16, dtype=np.float32).reshape(1, 16)
    qw, s, z, q = orc.quantize_rtn(w, 4, 16)
    assert s.tolist() == [[1.0]] and z.tolist() == [[0]]
    assert q.tolist() == [list(range(16))]
    # nibble k sits at bits 4*(k%8): 0x76543210, 0xFEDCBA98 (sign bit set)
    assert qw.tolist() == [[0x76543210, 0xFEDCBA98 - (1 << 32)]]
    cq, cs, cz = c_oracle.quantize_rtn_f32(w, 4, 16)
    assert cq.tolist() == qw.tolist() and cs.tolist() == [[1.0]] and cz.tolist() == [[0]]


def test_kat_negative_min_gives_zero_point():
    # -8..7: scale 1, zp = round(8/1) = 8, q = w + 8
    w = np.arange(-8, 8, dtype=np.float32).reshape(1, 16)
    _, s, z, q = orc.quantize_rtn(w, 4, 16)
    assert s.tolist() == [[1.0]] and z.tolist() == [[8]] and q.tolist() == [list(range(16))]


def test_kat_ties_round_half_to_even():
    # scale 1, zp 0: 0.5->0, 1.5->2, 2.5->2, 3.5->4, 4.5->4 (round half away would give 1,2,3,4,5)
    w = np.array([[0, 15, 0.5, 1.5, 2.5, 3.5, 4.5, 13.5, 14.5, 7, 7, 7, 7, 7, 7, 7]], np.float32)
    _, _, _, q = orc.quantize_rtn(w, 4, 16)
    assert q[0, :9].tolist() == [0, 15, 0, 2, 2, 4, 4, 14, 14]
    cq, _, _ = c_oracle.quantize_rtn_f32(w, 4, 16)
    assert orc.unpack_words(cq, 4)[0, :9].tolist() == [0, 15, 0, 2, 2, 4, 4, 14, 14]


def test_kat_constant_groups_hit_the_scale_floor():
    # max == min -> scale = 1e-8 (float32); +c: zp = clamp(round(-c/1e-8)) = 0, q = clamp(c/1e-8) = qmax
    #                                      -c: zp = qmax, q = clamp(-c/1e-8 + qmax) = 0;  0: zp 0, q 0
    w = np.concatenate([np.full((1, 32), 0.3), np.full((1, 32), -0.3), np.zeros((1, 32))], axis=1).astype(np.float32)
    for bits in (2, 4, 8):
        qmax = (1 << bits) - 1
        qw, s, z, q = orc.quantize_rtn(w, bits, 32)
        assert s.view(np.uint32).tolist() == [[int(np.float32(1e-8).view(np.uint32))] * 3]
        assert z.tolist() == [[0, qmax, 0]]
        assert (q[0, :32] == qmax).all() and (q[0, 32:] == 0).all()
        s16, z16 = orc.store_module_buffers(s, z)
        assert (s16 == 0).all()                      # 1e-8 is below half the smallest float16 subnormal
        assert (orc.dequantize_f16(qw, s16, z16, 32, bits) == 0).all()
        assert np.array_equal(orc.dequantize_rtn_f32(qw, s, z, 32, bits)[0, :32], np.full(32, np.float32(1e-8) * np.float32(qmax)))


def test_kat_pack_words_literal():
    # 8-bit: 255 in the top byte sets the sign bit: 255 << 24 == -16777216 as int32
    assert orc.pack_words(np.array([[0, 0, 0, 255]]), 8).tolist() == [[-16777216]]
    assert orc.pack_words(np.array([[1, 2, 3, 4]]), 8).tolist() == [[0x04030201]]
    # 2-bit: 0,1,2,3 repeated -> every byte 0b11100100 = 0xE4
    assert orc.pack_words(np.array([[0, 1, 2, 3] * 4]), 2).tolist() == [[0xE4E4E4E4 - (1 << 32)]]
    # 4-bit: value k of the row is nibble k % 8 of word k // 8
    q = np.zeros((1, 24), np.int64)
    q[0, 13] = 0xA
    assert orc.pack_words(q, 4).tolist() == [[0, 0xA << 20, 0]]


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_pack_closed_form_and_round_trip(bits):
    from ieee_exact import pack_exact
    rng = np.random.default_rng(bits)
    q = rng.integers(0, 1 << bits, size=(5, 256))
    q[0, :] = (1 << bits) - 1                        # every slot saturated: all words 0xFFFFFFFF = -1
    words = orc.pack_words(q, bits)
    assert (words[0] == -1).all()
    for r in range(5):
        assert words[r].tolist() == pack_exact(list(q[r]), bits)
    assert np.array_equal(orc.unpack_words(words, bits), q)


@pytest.mark.parametrize("bits,g", [(2, 32), (4, 64), (4, 128), (8, 128)])
def test_invariants_and_two_restatements_agree(bits, g):
    rng = np.random.default_rng(100 + bits + g)
    w = (rng.standard_normal((64, 8 * g)) * 0.02).astype(np.float32)
    w = np.where(rng.random(w.shape) < 0.001, w * 10, w).astype(np.float32)
    qmax = (1 << bits) - 1
    qw, s, z, q = orc.quantize_rtn(w, bits, g)
    cq, cs, cz = c_oracle.quantize_rtn_f32(w, bits, g)
    assert np.array_equal(qw, cq) and np.array_equal(s.view(np.uint32), cs.view(np.uint32)) and np.array_equal(z, cz)
    assert q.min() >= 0 and q.max() <= qmax and z.min() >= 0 and z.max() <= qmax and (s >= np.float32(1e-8)).all()
    # reconstruction error of an unclamped element is at most half a step (plus rounding slack)
    deq = orc.dequantize_rtn_f32(qw, s, z, g, bits)
    step = np.repeat(s, g, axis=1)
    inner = (q > 0) & (q < qmax)
    assert (np.abs(deq - w)[inner] <= 0.5 * step[inner] * (1 + 1e-5)).all()
    # the group minimum maps to q <= 1 and the maximum to q >= qmax - 1
    wg, qg = w.reshape(64, -1, g), q.reshape(64, -1, g)
    assert (np.take_along_axis(qg, wg.argmin(-1)[..., None], -1) <= 1).all()
    assert (np.take_along_axis(qg, wg.argmax(-1)[..., None], -1) >= qmax - 1).all()
    # forward: C restatement (double accumulate, f16 out) equals numpy restatement
    s16, z16 = orc.store_module_buffers(s, z)
    x = rng.standard_normal((4, 8 * g)).astype(np.float16)
    b = (rng.standard_normal(64) * 0.1).astype(np.float16)
    y_np, _ = orc.qlinear_forward(x, qw, s16, z16, b, bits, g)
    y_c = c_oracle.qlinear_forward(x, qw, s16, z16, b, bits, g)
    assert np.array_equal(y_np.astype(np.float16).view(np.uint16), y_c.view(np.uint16))


def test_error_conventions():
    w = np.zeros((2, 100), np.float32)
    with pytest.raises(ValueError):
        orc.quantize_rtn(w, 4, 32)                   # bitween/functional.py:12-17
    with pytest.raises(AssertionError):
        orc.quantize_rtn(np.zeros((2, 96), np.float32), 3, 32)   # bitween/functional.py:6


def test_backward_is_the_adjoint_of_the_forward_and_matches_brute_force():
    """qlinear_backward (bitween/modules.py:108-141): grad_x[m][k] = sum_n grad_y[m][n] * W16[n][k].  Pinned by
    plain loops over a tiny layer (an index or transposition slip fails), by one-hot rows returning rows of W16,
    and by <grad_y, x W^T> == <grad_y W, x> in float64."""
    rng = np.random.default_rng(12)
    n, k, bits, g = 6, 64, 4, 32
    w = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    qw, s, z, _ = orc.quantize_rtn(w, bits, g)
    s16, z16 = orc.store_module_buffers(s, z)
    w16 = orc.dequantize_f16(qw, s16, z16, g, bits)
    # the float32 dequantised weight cast to float16 is the same W16 (what backward multiplies with)
    assert np.array_equal(orc.dequantize_rtn_f32(qw, s16, z16, g, bits).astype(np.float16).view(np.uint16), w16.view(np.uint16))
    go = rng.standard_normal((3, n)).astype(np.float16)
    got = orc.qlinear_backward(go, qw, s16, z16, bits, g)
    want = np.zeros((3, k))
    for m in range(3):
        for kk in range(k):
            acc = 0.0
            for nn in range(n):
                acc += float(go[m, nn]) * float(w16[nn, kk])
            want[m, kk] = acc
    assert got.shape == (3, k) and np.allclose(got, want, rtol=1e-12, atol=1e-15)
    eye = np.eye(n, dtype=np.float16)
    assert np.array_equal(orc.qlinear_backward(eye, qw, s16, z16, bits, g), w16.astype(np.float64))
    x = rng.standard_normal((3, k)).astype(np.float16)
    _, y64 = orc.qlinear_forward(x, qw, s16, z16, None, bits, g)
    lhs = (go.astype(np.float64) * y64).sum()
    rhs = (got * x.astype(np.float64)).sum()
    assert abs(lhs - rhs) <= 1e-9 * max(1.0, abs(lhs))


@pytest.mark.parametrize("name", CASES)
def test_torch_cpu_path_matches_exact_vectors(name):
    """oracle/torch_cpu_path.py (the eager-torch restatement that bench.py times as the CPU baseline) against the
    exact-rational vectors, in every dtype the vectors cover: packed words, scale, zero point, the module's
    float16 buffers, both dequantisations bit for bit; the matmul against the exactly evaluated products."""
    import torch
    from oracle import torch_cpu_path as tcp
    key, fmt, bits, g, _ = _case(name)
    dt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[fmt]
    w = torch.from_numpy(GOLD[key + "_w"]).to(dt)
    valid = GOLD[key + "_valid"]
    qw, scale, zp, _ = tcp.quantize_rtn(w, bits, g)
    assert scale.dtype == dt and zp.dtype == torch.int32 and qw.dtype == torch.int32
    assert np.array_equal(zp.numpy()[valid], GOLD[key + "_zp"][valid])
    assert np.array_equal(scale.float().numpy().view(np.uint32)[valid], GOLD[key + "_scale"].view(np.uint32)[valid])
    vq = np.repeat(valid, g, axis=1)
    assert np.array_equal(orc.unpack_words(qw.numpy(), bits)[vq], GOLD[key + "_q"][vq])
    if fmt != "f32" or not valid.all():
        return
    assert np.array_equal(qw.numpy(), GOLD[key + "_qweight"])
    qw2, s16, z16 = tcp.module_buffers(w.half() if np.array_equal(w.half().float().numpy(), w.numpy()) else w, bits, g)
    assert np.array_equal(qw2.numpy(), GOLD[key + "_qweight"])
    assert np.array_equal(s16.numpy().view(np.uint16), GOLD[key + "_scale16"].view(np.uint16))
    w16 = tcp.dequantize_rtn(qw, s16, z16, g, bits).half()
    assert np.array_equal(w16.numpy().view(np.uint16), GOLD[key + "_w16"].view(np.uint16))
    w32 = tcp.dequantize_rtn(qw, scale, zp, g, bits)
    assert np.array_equal(w32.numpy().view(np.uint32), GOLD[key + "_w32"].view(np.uint32))
    y = tcp.forward(torch.from_numpy(GOLD[key + "_x"]), qw, s16, z16, None, bits, g).float().numpy()
    ref = GOLD[key + "_y64"]
    with np.errstate(over="ignore", invalid="ignore"):
        finite = np.isfinite(ref.astype(np.float32).astype(np.float16))
    assert np.abs(y - ref)[finite].max() <= 1e-2 * max(np.abs(ref[finite]).max(), 1e-30)


GOLD64 = np.load(os.path.join(os.path.dirname(__file__), "golden", "rtn_exact_vectors_f64.npz"))


@pytest.mark.parametrize("name", [str(n) for n in GOLD64["names"]])
def test_f64_oracle_matches_exact_vectors(name):
    """quantize_rtn on a float64 tensor (the reference is dtype-agnostic): 53-bit rounding per operation, both
    roundings of the scale division; the torch restatement run on a float64 tensor agrees in the IEEE mode."""
    key, _, bits, g, _, scale_div = name.split(":")
    bits, g = int(bits), int(g)
    w = GOLD64[key + "_w"]
    qw, scale, zp, q = orc.quantize_rtn_f64(w, bits, g, scale_div)
    assert np.array_equal(q, GOLD64[key + "_q"])
    assert np.array_equal(qw, GOLD64[key + "_qweight"])
    assert np.array_equal(zp, GOLD64[key + "_zp"])
    assert np.array_equal(scale.view(np.uint64), GOLD64[key + "_scale"].view(np.uint64))
    w64 = orc.dequantize_rtn_f64(qw, scale, zp, g, bits)
    assert np.array_equal(w64.view(np.uint64), GOLD64[key + "_w64"].view(np.uint64))
    if scale_div == "ieee":
        import torch
        from oracle import torch_cpu_path as tcp
        qw_t, s_t, z_t, _ = tcp.quantize_rtn(torch.from_numpy(w), bits, g)
        assert s_t.dtype == torch.float64
        assert np.array_equal(qw_t.numpy(), qw) and np.array_equal(s_t.numpy(), scale) and np.array_equal(z_t.numpy(), zp)
        w_t = tcp.dequantize_rtn(qw_t, s_t, z_t, g, bits)
        assert w_t.dtype == torch.float64 and np.array_equal(w_t.numpy().view(np.uint64), w64.view(np.uint64))


def test_bfloat16_weights_of_the_backward_match_exact_rational_rounding():
    """For bfloat16 gradients the reference multiplies with W32.to(bfloat16) (bitween/modules.py:134-139): the float32
    product scale16 * (q - zp) - exact - rounded once to bfloat16, ties to even.  dequantize_bf16 against that rounding
    carried out on exact fractions (tests/ieee_exact.py), over every (q, zp) difference and scales that put the product
    on, just below and just above bfloat16 ties; then qlinear_backward(dtype="bf16") against plain loops."""
    from fractions import Fraction
    import ieee_exact as ex
    rng = np.random.default_rng(21)
    bits, g = 8, 32
    n, k = 24, 64
    q = rng.integers(0, 256, size=(n, k)).astype(np.int32)
    qw = orc.pack_words(q, bits)
    # scales: random float16 values, plus values with few significant bits (products that are exact ties in bfloat16)
    s16 = np.abs(rng.standard_normal((n, k // g)).astype(np.float16) * np.float16(0.01)) + np.float16(1e-4)
    s16[::3] = np.float16(0.0078125) * (1 + rng.integers(0, 8, size=s16[::3].shape) / 8).astype(np.float16)
    z16 = rng.integers(0, 256, size=(n, k // g)).astype(np.float16)
    got = orc.dequantize_bf16(qw, s16, z16, g, bits)
    for i in range(n):
        for j in range(k):
            exact = Fraction(float(s16[i, j // g])) * (int(q[i, j]) - int(z16[i, j // g]))
            want = ex.rn(exact, "bf16")
            assert Fraction(float(got[i, j])) == want, (i, j)
    go = orc._round_to(rng.standard_normal((3, n)).astype(np.float32), "bf16")
    out = orc.qlinear_backward(go, qw, s16, z16, bits, g, dtype="bf16")
    want = np.zeros((3, k))
    for m in range(3):
        for kk in range(k):
            acc = 0.0
            for nn in range(n):
                acc += float(go[m, nn]) * float(got[nn, kk])
            want[m, kk] = acc
    assert np.allclose(out, want, rtol=1e-12, atol=1e-15)
    eye = np.eye(n, dtype=np.float32)
    assert np.array_equal(orc.qlinear_backward(eye, qw, s16, z16, bits, g, dtype="bf16"), got.astype(np.float64))
    with pytest.raises(AssertionError):
        orc.qlinear_backward(np.full((1, n), 1.001, np.float32), qw, s16, z16, bits, g, dtype="bf16")   # not a bfloat16 value
