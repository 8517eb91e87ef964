"""Helpers shared by the GPU parity tests (oracle side runs on the host)."""
import numpy as np
import torch

from oracle import rtn_oracle as orc


def make_weight(n, k, seed, outliers=False, dtype=np.float16):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    if outliers:
        w = np.where(rng.random((n, k)) < 0.001, w * 10, w)
    return w.astype(dtype).astype(np.float32)


def quantized_layer(n, k, bits, g, seed, outliers=False, bias=True):
    """Oracle-side module buffers for a random layer: (qweight, scale16, zp16, bias16)."""
    w = make_weight(n, k, seed, outliers)
    qw, s, z, _ = orc.quantize_rtn(w, bits, g)
    s16, z16 = orc.store_module_buffers(s, z)
    rng = np.random.default_rng(seed + 1)
    b = (rng.standard_normal(n) * 0.1).astype(np.float16) if bias else None
    return w, qw, s16, z16, b


def to_gpu(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()


def check_matmul(y_gpu, x16, qw, s16, z16, b16, bits, g, tol_rel=1e-2):
    """Compare a float16 kernel result with the oracle.

    Bars (written out as the north star asks):
      * max |y - ref| / max |ref| <= 1e-2            (max relative error, fp32 accumulate)
      * mean |y - ref| / mean |ref| < 1e-2           (main.py:471-477)
      * elementwise: |y - y64| <= 2^-10 |y64| + 6 * 2^-11 * sqrt(x^2 @ (W16^2)^T) + 2e-6 * (|x| @ |W16|^T) + 1e-7:
        one float16 rounding of the result, float32 accumulation slack, and - where a kernel applies the
        group scale to the exact integer dot product instead of rounding every weight to float16 first -
        the reference's own per-weight float16 rounding (relative 2^-11 each, independent, 6 sigma).
    """
    y_ref, y64 = orc.qlinear_forward(x16, qw, s16, z16, b16, bits, g)
    y = y_gpu.detach().float().cpu().numpy().astype(np.float64)
    assert np.isfinite(y).all()
    w16 = np.abs(orc.dequantize_f16(qw, s16, z16, g, bits).astype(np.float64))
    mag = np.abs(x16.astype(np.float64)) @ w16.T
    err = np.abs(y - y64)
    rss = np.sqrt((x16.astype(np.float64) ** 2) @ (w16 ** 2).T)
    bound = 2.0 ** -10 * np.abs(y64) + 6 * 2.0 ** -11 * rss + 2e-6 * mag + 1e-7
    if b16 is not None:
        bound = bound + 2.0 ** -10 * np.abs(b16.astype(np.float64))
    worst = (err / bound).max()
    assert worst <= 1.0, f"elementwise bound exceeded by {worst:.3f}x"
    ref = y_ref.astype(np.float64)
    assert np.abs(y - ref).max() / max(np.abs(ref).max(), 1e-30) <= tol_rel
    assert np.abs(y - ref).mean() / max(np.abs(ref).mean(), 1e-30) < tol_rel
