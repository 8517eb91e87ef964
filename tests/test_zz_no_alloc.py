"""bw_qgemm_static: the prefill entry point that allocates nothing (its split-K partial tiles go to a device
array of the library) against bw_qgemm_ws with a caller's workspace - same kernels, same plan, so bit for bit -
and against the oracle.  Two calls in a row share the array; the second is smaller."""
import ctypes

import numpy as np
import pytest
import torch

from gpu_util import check_matmul, quantized_layer, to_gpu

pytestmark = pytest.mark.gpu


def _call(lib, fn, x, qw, s, z, b, n, bits, g, ws=None):
    m, k = x.shape
    y = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    args = [x.data_ptr(), 0, m, k, k, qw.data_ptr(), s.data_ptr(), z.data_ptr(), None if b is None else b.data_ptr(),
            n, bits, g, y.data_ptr(), n]
    if ws is not None:
        args += [ws.data_ptr(), ws.numel()]
    st = fn(*args, stream)
    torch.cuda.synchronize()
    return st, y


def test_static_scratch_matches_caller_workspace_twice_in_a_row():
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    cases = [(128, 4096, 2048, 4, 128, 11), (48, 2048, 512, 8, 64, 12)]     # (M, K, N, bits, group, seed): large, then smaller
    outs = []
    for m, k, n, bits, g, seed in cases:
        _, qw, s16, z16, b16 = quantized_layer(n, k, bits, g, seed=seed)
        x = np.random.default_rng(seed).standard_normal((m, k)).astype(np.float16)
        xg, qg, sg, zg, bg = to_gpu(x), to_gpu(qw), to_gpu(s16), to_gpu(z16), to_gpu(b16)
        need = lib.bw_qgemm_workspace_bytes(m, n, k, bits, g)
        assert need > 0, "the case is meant to take the split-K path"
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        st_ws, y_ws = _call(lib, lib.bw_qgemm_ws, xg, qg, sg, zg, bg, n, bits, g, ws)
        assert st_ws == 0
        outs.append((xg, qg, sg, zg, bg, n, bits, g, y_ws, x, qw, s16, z16, b16))
    # the two calls back to back on the library's own array, nothing allocated in between
    before = torch.cuda.memory_allocated()
    for xg, qg, sg, zg, bg, n, bits, g, y_ws, x, qw, s16, z16, b16 in outs:
        st, y = _call(lib, lib.bw_qgemm_static, xg, qg, sg, zg, bg, n, bits, g)
        assert st == 0
        assert torch.equal(y, y_ws)
        check_matmul(y, x, qw, s16, z16, b16, bits, g)
    assert torch.cuda.memory_allocated() - before <= 2 * 128 * 2048 * 2 + 4096     # only the test's own y tensors


def test_static_scratch_takes_unsplit_and_generic_shapes():
    """Shapes that need no partial tiles (and the shape-generic kernel) run through the same entry point."""
    from bitween_amd.kernels import hip_loader
    lib = hip_loader.load()
    for m, k, n, bits, g in ((300, 512, 768, 4, 128), (5, 96, 33, 8, 32)):
        _, qw, s16, z16, b16 = quantized_layer(n, k, bits, g, seed=3)
        x = np.random.default_rng(4).standard_normal((m, k)).astype(np.float16)
        st, y = _call(lib, lib.bw_qgemm_static, to_gpu(x), to_gpu(qw), to_gpu(s16), to_gpu(z16), to_gpu(b16), n, bits, g)
        assert st == 0
        check_matmul(y, x, qw, s16, z16, b16, bits, g)
