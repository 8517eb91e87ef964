"""Writes tests/golden/rtn_exact_vectors.npz.

The reference (pure Python/torch) holds no golden vectors for its
quantize/pack/dequantize path, so these are derived from first principles:
every expected value is computed with exact rational arithmetic and one
explicit round-to-nearest-even per IEEE operation (tests/ieee_exact.py), in
the operation order of bitween/functional.py:22-29,35-40,70 and
bitween/modules.py:55-58.  Neither the oracle nor numpy float arithmetic is
used to produce an expected value.

Run from the repo root:  python tests/golden/make_exact_vectors.py
"""
import os
import sys
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from ieee_exact import pack_exact, quantize_group_exact, rn  # noqa: E402


def _to_bf16(a):
    u = np.ascontiguousarray(a, np.float32).view(np.uint32)
    r = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) & np.uint32(0xFFFF0000)
    return r.view(np.float32)


def make_weight(kind, rng, n, k, g, bits):
    qmax = (1 << bits) - 1
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    if kind == "normal_f32":
        pass
    elif kind == "normal_f16":                       # an fp16 checkpoint upcast by from_float
        w = w.astype(np.float16).astype(np.float32)
    elif kind == "outliers":
        mask = rng.random((n, k)) < 0.01
        w = np.where(mask, w * 10, w).astype(np.float16).astype(np.float32)
    elif kind == "edge":
        w[0, :] = 0.0                                # all-zero row
        w[1, :g] = 0.3                               # constant positive group
        w[1, g:2 * g] = -0.3 if k >= 2 * g else 0.3  # constant negative group
        w[2, :g] = 0.0
        w[2, 3] = 1.0                                # one-hot group
        w[3, :g] = 0.0
        w[3, 5] = -1.0                               # negative one-hot
    elif kind == "ties":
        # min 0, max qmax*2^j -> scale exactly 2^j, zp 0; values (i+0.5)*2^j are exact ties
        for r in range(n):
            j = float(2.0 ** (r - 3))
            for gi in range(k // g):
                vals = (rng.integers(0, qmax, size=g) + 0.5) * j
                vals[0], vals[1] = 0.0, qmax * j
                if gi % 2:                           # shifted: min -3*2^j -> zp 3
                    vals = vals - 3 * j
                    vals[0], vals[1] = -3 * j, (qmax - 3) * j
                w[r, gi * g:(gi + 1) * g] = vals
    elif kind == "denormal":
        w = (w * np.float32(1e-36)).astype(np.float32)        # float32 subnormals and tiny normals
        w[0, :g] *= np.float32(1e-3)
    elif kind == "large":
        w = (w * np.float32(5e5)).astype(np.float32)          # |w| up to ~4e4
    else:
        raise ValueError(kind)
    return np.ascontiguousarray(w, np.float32)


def exact_case(w, bits, g, fmt, scale_div="ieee"):
    n, k = w.shape
    groups = k // g
    q = np.zeros((n, k), np.int32)
    scale = np.zeros((n, groups), np.float64)
    zp = np.zeros((n, groups), np.int32)
    valid = np.ones((n, groups), bool)
    w16 = np.zeros((n, k), np.float64)
    w32 = np.zeros((n, k), np.float64)
    for r in range(n):
        for gi in range(groups):
            vals = [float(v) for v in w[r, gi * g:(gi + 1) * g]]
            try:
                s, z, qq = quantize_group_exact(vals, bits, fmt, scale_div)
            except ZeroDivisionError:
                valid[r, gi] = False                 # reference divides by zero here: unpinned
                continue
            scale[r, gi] = float(s)                  # exact: s is representable in fmt
            zp[r, gi] = z
            q[r, gi * g:(gi + 1) * g] = qq
            s16 = rn(s, "f16")                       # module buffer, bitween/modules.py:208
            for i, qi in enumerate(qq):
                neg_zero = -0.0 if qi < z else 0.0     # IEEE: (+s) * (negative) that rounds to 0 is -0
                w16[r, gi * g + i] = float(rn(s16 * (qi - z), "f16")) or neg_zero
                w32[r, gi * g + i] = float(rn(s * (qi - z), "f32")) or neg_zero
    words = np.array([pack_exact(list(q[r]), bits) for r in range(n)], np.int64).astype(np.int32)
    return dict(q=q, qweight=words, scale=scale.astype(np.float32), zp=zp, valid=valid,
                scale16=np.array([[float(rn(Fraction(float(v)), "f16")) for v in row] for row in scale], np.float32).astype(np.float16),
                w16=w16.astype(np.float16), w32=w32.astype(np.float32))


def main():
    out = {}
    names = []
    idx = 0
    for fmt, kinds in (("f32", ["normal_f32", "normal_f16", "outliers", "edge", "ties", "denormal", "large"]),
                       ("f16", ["normal_f16", "outliers"]), ("bf16", ["normal_f16"])):
        for bits in (2, 4, 8):
            for g in (32, 64, 128):
                for kind in kinds:
                    if fmt != "f32" and g == 64:
                        continue
                    rng = np.random.default_rng(1000 * bits + g + len(kind))
                    n, k = (6, 2 * g if g == 128 else 4 * g)
                    w = make_weight(kind, rng, n, k, g, bits)
                    if fmt == "f16":
                        w = w.astype(np.float16).astype(np.float32)
                    if fmt == "bf16":
                        w = _to_bf16(w)
                    case = exact_case(w, bits, g, fmt)
                    key = f"c{idx:03d}"
                    names.append(f"{key}:{fmt}:{bits}:{g}:{kind}")
                    out[key + "_w"] = w
                    for name, arr in case.items():
                        out[f"{key}_{name}"] = arr
                    # activations and an exactly evaluated product for M = 3
                    x = rng.standard_normal((3, k)).astype(np.float16)
                    y = np.zeros((3, n), np.float64)
                    for m in range(3):
                        for r in range(n):
                            y[m, r] = float(sum(Fraction(float(a)) * Fraction(float(b)) for a, b in zip(x[m], case["w16"][r])))
                    out[key + "_x"] = x
                    out[key + "_y64"] = y
                    idx += 1
    # the same path with the scale formed by the float32 reciprocal (eager torch on a GPU): names end in ":recip"
    for fmt, kinds in (("f32", ["normal_f32", "normal_f16", "outliers", "ties", "large"]), ("f16", ["normal_f16"]), ("bf16", ["normal_f16"])):
        for bits in (2, 4, 8):
            for g in (32, 128):
                for kind in kinds:
                    rng = np.random.default_rng(77000 + 1000 * bits + g + len(kind))
                    n, k = 4, 2 * g
                    w = make_weight(kind, rng, n, k, g, bits)
                    if fmt == "f16":
                        w = w.astype(np.float16).astype(np.float32)
                    if fmt == "bf16":
                        w = _to_bf16(w)
                    case = exact_case(w, bits, g, fmt, "reciprocal")
                    key = f"c{idx:03d}"
                    names.append(f"{key}:{fmt}:{bits}:{g}:{kind}:recip")
                    out[key + "_w"] = w
                    for name, arr in case.items():
                        if name not in ("w16", "w32"):
                            out[f"{key}_{name}"] = arr
                    idx += 1
    out["names"] = np.array(names)
    path = os.path.join(HERE, "rtn_exact_vectors.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {idx} cases, {os.path.getsize(path) / 1024:.0f} KiB")


def main_f64():
    """float64 tensors (functional.py is dtype-agnostic): every operation rounded to 53 bits; a file of its own."""
    out, names, idx = {}, [], 0
    for scale_div in ("ieee", "reciprocal"):
        for bits in (2, 4, 8):
            for g in (32, 128):
                for kind in ("normal_f64", "ties_f64"):
                    rng = np.random.default_rng(91000 + 1000 * bits + g + len(kind) + (7 if scale_div == "ieee" else 0))
                    n, k = 3, 2 * g
                    w = rng.standard_normal((n, k)) * 0.02
                    if kind == "ties_f64":
                        # values on a grid of the group's range: many exact x.5 ties after w / scale + zp
                        qmax = (1 << bits) - 1
                        step = 2.0 ** -10
                        w = rng.integers(0, 2 * qmax + 1, size=(n, k)).astype(np.float64) * (step / 2)
                        w[:, ::g] = 0.0
                        w[:, 1::g] = qmax * step
                    groups = k // g
                    q = np.zeros((n, k), np.int32)
                    scale = np.zeros((n, groups), np.float64)
                    zp = np.zeros((n, groups), np.int32)
                    w64 = np.zeros((n, k), np.float64)
                    for r in range(n):
                        for gi in range(groups):
                            s, z, qq = quantize_group_exact([float(v) for v in w[r, gi * g:(gi + 1) * g]], bits, "f64", scale_div)
                            scale[r, gi], zp[r, gi] = float(s), z
                            q[r, gi * g:(gi + 1) * g] = qq
                            for i, qi in enumerate(qq):
                                w64[r, gi * g + i] = float(rn(s * (qi - z), "f64")) or (-0.0 if qi < z else 0.0)
                    words = np.array([pack_exact(list(q[r]), bits) for r in range(n)], np.int64).astype(np.int32)
                    key = f"d{idx:03d}"
                    names.append(f"{key}:f64:{bits}:{g}:{kind}:{scale_div}")
                    for name, arr in dict(w=w, q=q, qweight=words, scale=scale, zp=zp, w64=w64).items():
                        out[f"{key}_{name}"] = arr
                    idx += 1
    out["names"] = np.array(names)
    path = os.path.join(HERE, "rtn_exact_vectors_f64.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {idx} cases, {os.path.getsize(path) / 1024:.0f} KiB")


if __name__ == "__main__":
    import sys
    if "--f64" in sys.argv:
        main_f64()
    else:
        main()
