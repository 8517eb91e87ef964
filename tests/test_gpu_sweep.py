"""Seeded sweep of the forward over formats, shapes that end inside tiles and chunks, row counts on both sides of
every kernel switch (1, 2, 16, 32 / 48, split-K or not), bias on and off, float16 and bfloat16 activations.

The expected value is a float64 matmul on the GPU over the library's own bit-exact dequantisation (which
tests/test_gpu_parity.py pins against the oracle and the exact vectors, and every tenth case here compares with
the oracle's again), so hundreds of cases run in seconds; the
bound is elementwise: one float16 rounding of the result plus float32 accumulation error on sum |x| |w|."""
import numpy as np
import pytest
import torch

from oracle import rtn_oracle as orc

pytestmark = pytest.mark.gpu

ROWS = [1, 2, 3, 7, 16, 17, 32, 33, 40, 48, 49, 64, 100, 128, 129, 200, 256, 300, 513, 1024, 1300, 2048]


def _run(seed, cases, max_groups, max_n):
    from bitween_amd.kernels import hip_loader as hip
    rng = np.random.default_rng(seed)
    for it in range(cases):
        bits = int(rng.choice([2, 4, 8]))
        g = int(rng.choice([32, 64, 128]))
        groups = int(rng.integers(1, max_groups))
        k = g * groups
        n = int(rng.integers(1, max_n))
        m = int(rng.choice(ROWS))
        qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (n, k * bits // 32), device="cuda", dtype=torch.int64).to(torch.int32)
        s = (torch.rand(n, groups, device="cuda") * 0.02 + 0.001).half()
        z = torch.randint(0, 2 ** bits, (n, groups), device="cuda").half()
        bias = (torch.randn(n, device="cuda") * 0.1).half() if rng.integers(0, 2) else None
        dt = torch.bfloat16 if rng.integers(0, 4) == 0 else torch.float16
        x = torch.randn(m, k, device="cuda").to(dt)
        y = hip.quantized_matmul_hip(x, qw, s, z, bias, bits, g)
        w16 = hip.dequantize(qw, s, z, g, bits, torch.float16)
        if it % 10 == 0:
            # every tenth case: the expected weights straight from the oracle, so the sweep does not rest on the
            # library's own dequantisation alone
            w16_o = orc.dequantize_f16(qw.cpu().numpy(), s.cpu().numpy(), z.cpu().numpy(), g, bits)
            assert np.array_equal(w16.cpu().numpy().view(np.uint16) & 0x7FFF | ((w16.cpu().numpy() != 0) * (w16.cpu().numpy().view(np.uint16) & 0x8000)),
                                  w16_o.view(np.uint16) & 0x7FFF | ((w16_o != 0) * (w16_o.view(np.uint16) & 0x8000)))
        w16 = w16.double()
        x64 = x.to(torch.float16).double()
        ref = x64 @ w16.T
        if bias is not None:
            ref = ref + bias.double()
        mag = x64.abs() @ w16.abs().T
        worst = ((y.double() - ref).abs() / (2.0 ** -10 * ref.abs() + 2.0 ** -12 * mag + 1e-6)).max().item()
        assert torch.isfinite(y).all() and worst <= 1.0, \
            f"case {it}: bits {bits} group {g} K {k} N {n} M {m} {dt} bias {bias is not None}: {worst:.2f}x the bound"


def test_forward_sweep_small_layers():
    _run(seed=1, cases=300, max_groups=48, max_n=700)


def test_forward_sweep_long_rows_and_wide_layers():
    _run(seed=2, cases=150, max_groups=130, max_n=3000)
