"""ctypes binding of libbitween_hip.so (the C ABI in include/bitween_hip.h).

This module takes the place of the reference's absent
`bitween.kernels.cuda_loader` (main.py:401): `quantized_matmul_hip` has the
signature and meaning of `quantized_matmul_cuda(x, qweight, scale, zero_point,
bias, bits, group_size)` (main.py:433).

There is no CPU path: a missing library or a missing GPU raises.
"""
import ctypes
import os

import torch

_LIB_PATH = os.environ.get("BITWEEN_HIP_LIB") or os.path.join(
    os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc", "libbitween_hip.so")
_lib = None

BW_F16, BW_BF16, BW_F32, BW_I32, BW_F64 = 0, 1, 2, 3, 4
BW_SCALE_RECIPROCAL = 0x100   # flag for math_dtype: scale = (max - min) * fl32(1 / Qmax), as eager torch computes it on a GPU
_DTYPE_CODE = {torch.float16: BW_F16, torch.bfloat16: BW_BF16, torch.float32: BW_F32, torch.int32: BW_I32, torch.float64: BW_F64}

ABI_VERSION = 10           # what bw_abi_version() of a matching library returns
ENTRY_POINTS = ("bw_abi_version", "bw_strerror", "bw_quantize_pack", "bw_quantize_pack_add", "bw_dequantize", "bw_qgemv", "bw_qgemm",
                "bw_qgemm_ws", "bw_qgemm_static", "bw_qgemm_workspace_bytes", "bw_qgemm_tile_rows", "bw_qlinear", "bw_qdgrad", "bw_qdgrad_workspace_bytes", "bw_qdgrad_tile_rows", "bw_cast_bf16_f16", "bw_qlinear_decode_rows", "bw_qgemv_last_kernel")


class BitweenHipError(RuntimeError):
    pass


def library_path():
    return _LIB_PATH


def load():
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise BitweenHipError(
            f"{_LIB_PATH} is missing: build it with `python -m bitween_amd.csrc.build` "
            "(bitween_amd has no CPU or eager fallback)")
    lib = ctypes.CDLL(_LIB_PATH)
    vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    lib.bw_abi_version.restype = i32
    if lib.bw_abi_version() != ABI_VERSION:
        raise BitweenHipError(f"{_LIB_PATH} has ABI version {lib.bw_abi_version()}, this package expects {ABI_VERSION}: "
                              "rebuild it with `python -m bitween_amd.csrc.build`")
    lib.bw_strerror.restype = ctypes.c_char_p
    lib.bw_strerror.argtypes = [i32]
    lib.bw_quantize_pack.argtypes = [vp, i32, i32, i64, i64, i64, i32, i32, vp, vp, i32, vp, i32, vp]
    lib.bw_quantize_pack_add.argtypes = [vp, vp, i32, i32, i64, i64, i64, i64, i32, i32, vp, vp, i32, vp, i32, vp]
    lib.bw_dequantize.argtypes = [vp, vp, i32, vp, i32, i64, i64, i32, i32, vp, i32, i64, vp]
    mm = [vp, i32, i64, i64, i64, vp, vp, vp, vp, i64, i32, i32, vp, i64, vp]
    for name in ("bw_qgemv", "bw_qgemm", "bw_qlinear", "bw_qgemm_static"):
        getattr(lib, name).argtypes = mm
    lib.bw_qgemm_ws.argtypes = mm[:-1] + [vp, ctypes.c_size_t, vp]
    lib.bw_qgemm_workspace_bytes.argtypes = [i64, i64, i64, i32, i32]
    lib.bw_qgemm_workspace_bytes.restype = ctypes.c_size_t
    lib.bw_qgemm_tile_rows.argtypes = [i64, i64, i64, i32, i32]
    lib.bw_qgemm_tile_rows.restype = i32
    lib.bw_qdgrad_workspace_bytes.argtypes = [i64, i64, i64, i32, i32]
    lib.bw_qdgrad_workspace_bytes.restype = ctypes.c_size_t
    lib.bw_qdgrad_tile_rows.argtypes = [i64, i64, i64, i32, i32]
    lib.bw_qdgrad_tile_rows.restype = i32
    lib.bw_qdgrad.argtypes = [vp, i32, i64, i64, i64, vp, vp, vp, i64, i32, i32, vp, i64, vp, ctypes.c_size_t, vp]
    lib.bw_qdgrad.restype = i32
    lib.bw_cast_bf16_f16.argtypes = [vp, i64, i64, i64, vp, i64, vp]
    lib.bw_cast_bf16_f16.restype = i32
    lib.bw_qlinear_decode_rows.argtypes = [i64, i64, i32]
    lib.bw_qlinear_decode_rows.restype = i32
    lib.bw_qgemv_last_kernel.argtypes = []
    lib.bw_qgemv_last_kernel.restype = ctypes.c_char_p
    for name in ("bw_quantize_pack", "bw_quantize_pack_add", "bw_dequantize", "bw_qgemv", "bw_qgemm", "bw_qgemm_ws", "bw_qgemm_static", "bw_qlinear"):
        getattr(lib, name).restype = i32
    for name in ("bw_qgemv", "bw_qgemm", "bw_qlinear"):
        _ENTRY[name] = getattr(lib, name)
    _lib = lib
    return lib


_ENTRY = {}


def _check(status, what):
    if status == 0:
        return
    msg = load().bw_strerror(status).decode()
    if status == -2:
        raise NotImplementedError(f"{what}: {msg}")
    raise BitweenHipError(f"{what}: {msg} (status {status})")


def require_gpu(t, what):
    if not t.is_cuda:
        raise BitweenHipError(f"{what}: expected a tensor on the ROCm GPU, got device {t.device} "
                              "(bitween_amd has no CPU path)")


def _stream(device):
    return torch._C._cuda_getCurrentRawStream(device.index if device.index is not None else torch.cuda.current_device())


def quantize_pack(weight, bits, group_size, math_dtype, scale_dtype, zp_dtype, delta=None, scale_reciprocal=False):
    """weight [N,K] on GPU (f16/bf16/f32, or f64 with f64 math and scale) -> (qweight int32, scale, zero_point) per bw_quantize_pack; with
    `delta` (same shape and dtype) the kernel quantises weight + delta (bw_quantize_pack_add).
    `scale_reciprocal`: the scale as eager torch forms it on a GPU (BW_SCALE_RECIPROCAL)."""
    require_gpu(weight, "quantize_pack")
    if weight.stride(-1) != 1:
        weight = weight.contiguous()
    n, k = weight.shape
    vpi = 32 // bits
    dev = weight.device
    if delta is not None:
        require_gpu(delta, "quantize_pack")
        if delta.shape != weight.shape or delta.dtype != weight.dtype:
            raise ValueError("delta must have the shape and dtype of weight")
        if delta.stride(-1) != 1:
            delta = delta.contiguous()
    qweight = torch.empty((n, k // vpi), dtype=torch.int32, device=dev)
    scale = torch.empty((n, k // group_size), dtype=scale_dtype, device=dev)
    zp = torch.empty((n, k // group_size), dtype=zp_dtype, device=dev)
    with torch.cuda.device(dev):
        st = load().bw_quantize_pack_add(weight.data_ptr(), None if delta is None else delta.data_ptr(),
                                         _DTYPE_CODE[weight.dtype], _DTYPE_CODE[math_dtype] | (BW_SCALE_RECIPROCAL if scale_reciprocal else 0), n, k, weight.stride(0),
                                         0 if delta is None else delta.stride(0), bits, group_size, qweight.data_ptr(),
                                         scale.data_ptr(), _DTYPE_CODE[scale_dtype], zp.data_ptr(),
                                         _DTYPE_CODE[zp_dtype], _stream(dev))
    _check(st, "bw_quantize_pack")
    return qweight, scale, zp


def dequantize(qweight, scale, zero_point, group_size, bits, out_dtype):
    """(qweight, scale f32|f16, zero_point i32|f16) on GPU -> weight [N,K] of out_dtype per bw_dequantize; a float64
    scale goes with out_dtype float64."""
    require_gpu(qweight, "dequantize")
    qweight, scale, zero_point = qweight.contiguous(), scale.contiguous(), zero_point.contiguous()
    n, words = qweight.shape
    k = words * (32 // bits)
    out = torch.empty((n, k), dtype=out_dtype, device=qweight.device)
    with torch.cuda.device(qweight.device):
        st = load().bw_dequantize(qweight.data_ptr(), scale.data_ptr(), _DTYPE_CODE[scale.dtype], zero_point.data_ptr(),
                                  _DTYPE_CODE[zero_point.dtype], n, k, bits, group_size, out.data_ptr(),
                                  _DTYPE_CODE[out_dtype], k, _stream(qweight.device))
    _check(st, "bw_dequantize")
    return out


def _raw_stream(index):
    return torch._C._cuda_getCurrentRawStream(index)


class _on_device:
    """torch.cuda.device(), skipped when the device is already current (the common case: saves microseconds
    on a call whose kernel runs for a few)."""
    __slots__ = ("index", "ctx")

    def __init__(self, device):
        self.index = device.index if device.index is not None else torch.cuda.current_device()
        self.ctx = None

    def __enter__(self):
        if torch.cuda.current_device() != self.index:
            self.ctx = torch.cuda.device(self.index)
            self.ctx.__enter__()
        return self.index

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)
        return False


_CAST_MIN_NUMEL = 1 << 22     # below this the tensor cast's shorter host path wins (5 vs 9 us per eager call)


def _bf16_to_f16(x):
    """x.to(float16) for a 2-D bfloat16 activation matrix through bw_cast_bf16_f16 (a streaming kernel of the
    library: 19 us against 50 us for 2048 x 14336); the tensor cast for small inputs and when the layout does
    not qualify."""
    if (x.dim() == 2 and x.numel() >= _CAST_MIN_NUMEL and x.stride(1) == 1 and x.shape[1] % 8 == 0 and x.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0):
        y = torch.empty(x.shape, dtype=torch.float16, device=x.device)
        with _on_device(x.device) as index:
            st = load().bw_cast_bf16_f16(x.data_ptr(), x.shape[0], x.shape[1], x.stride(0), y.data_ptr(), y.stride(0), _raw_stream(index))
        if st == 0:
            return y
        if st not in (-2, -3):                            # unsupported layout or alignment: tensor cast
            _check(st, "bw_cast_bf16_f16")
    return x.to(torch.float16)


def _matmul(entry, x, qweight, scale, zero_point, bias, bits, group_size):
    if not x.is_cuda:
        require_gpu(x, entry)
    if x.dim() != 2:
        raise ValueError("x must be [M, K]")
    if qweight.dtype is not torch.int32 or scale.dtype is not torch.float16 or zero_point.dtype is not torch.float16:
        raise TypeError("qweight must be int32 and scale / zero_point float16 (the QuantizedLinear buffers)")
    m = x.shape[0]
    # rows that bw_qlinear keeps on the decode kernel: always 16, and 32 or 48 for layers that are not too large
    decode_rows = 16 if m <= 16 or entry != "bw_qlinear" else load().bw_qlinear_decode_rows(qweight.shape[0], x.shape[1], bits)
    act = BW_F16
    if x.dtype is torch.bfloat16:
        # the decode kernels round bfloat16 to float16 as they stage x (the reference's x.to(float16),
        # bitween/modules.py:74, without the extra kernel); the prefill kernel wants float16 in memory
        if entry == "bw_qgemv" or (entry == "bw_qlinear" and m <= decode_rows):
            act = BW_BF16
        else:
            x = _bf16_to_f16(x)
    elif x.dtype is not torch.float16:
        raise TypeError("x must be float16 or bfloat16")
    if bias is not None and bias.dtype is not torch.float16:
        raise TypeError("bias must be float16")
    ldx = x.stride(0)
    if x.stride(1) != 1 or (ldx * 2) % 16 or x.data_ptr() % 16:
        x = x.contiguous().clone()
        ldx = x.stride(0)
    if not qweight.is_contiguous():
        qweight = qweight.contiguous()
    if not scale.is_contiguous():
        scale = scale.contiguous()
    if not zero_point.is_contiguous():
        zero_point = zero_point.contiguous()
    m, k = x.shape
    n, words = qweight.shape
    if words * (32 // bits) != k:
        raise ValueError(f"x has K={k} but qweight packs K={words * (32 // bits)}")
    groups = k // group_size
    if scale.shape != (n, groups) or zero_point.shape != (n, groups):
        raise ValueError("scale / zero_point must be [N, K // group_size]")
    y = torch.empty((m, n), dtype=torch.float16, device=x.device)
    if m == 0:
        return y
    lib = load()
    bias_ptr = None
    if bias is not None:
        bias_ptr = (bias if bias.is_contiguous() else bias.contiguous()).data_ptr()
    with _on_device(x.device) as index:
        if (entry == "bw_qgemm" and m > 16) or (entry == "bw_qlinear" and m > decode_rows):
            # prefill (bw_qlinear itself keeps fewer rows on the decode kernel): give the library a split-K
            # workspace when the shape wants one
            nbytes = lib.bw_qgemm_workspace_bytes(m, n, k, bits, group_size)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device) if nbytes else None
            st = lib.bw_qgemm_ws(x.data_ptr(), BW_F16, m, k, ldx, qweight.data_ptr(), scale.data_ptr(),
                                 zero_point.data_ptr(), bias_ptr, n, bits, group_size, y.data_ptr(), n,
                                 None if ws is None else ws.data_ptr(), nbytes, _raw_stream(index))
            entry = "bw_qgemm_ws"
        else:
            st = _ENTRY[entry](x.data_ptr(), act, m, k, ldx, qweight.data_ptr(), scale.data_ptr(),
                               zero_point.data_ptr(), bias_ptr, n, bits, group_size, y.data_ptr(), n, _raw_stream(index))
            if st == -2 and act == BW_BF16:                # a shape only the generic kernel takes: float16 in memory
                x = x.to(torch.float16)
                st = _ENTRY[entry](x.data_ptr(), BW_F16, m, k, x.stride(0), qweight.data_ptr(), scale.data_ptr(),
                                   zero_point.data_ptr(), bias_ptr, n, bits, group_size, y.data_ptr(), n, _raw_stream(index))
    if st:
        _check(st, entry)
    return y


def make_decode_plan(qweight, scale, zero_point, bias, bits, group_size):
    """Validate a layer's buffers once for decode_with_plan: returns a tuple holding the tensors (so that the
    caller can tell by identity whether they are still the ones validated), their device addresses and the
    layer's sizes - or None when the buffers do not qualify and the general path has to look at them."""
    if not qweight.is_cuda or qweight.dtype is not torch.int32 or scale.dtype is not torch.float16 or \
            zero_point.dtype is not torch.float16 or (bias is not None and bias.dtype is not torch.float16):
        return None
    if not (qweight.is_contiguous() and scale.is_contiguous() and zero_point.is_contiguous()) or \
            (bias is not None and not bias.is_contiguous()):
        return None
    n, words = qweight.shape
    k = words * (32 // bits)
    if k % group_size or scale.shape != (n, k // group_size) or zero_point.shape != scale.shape or \
            (bias is not None and bias.shape != (n,)):
        return None
    load()
    index = qweight.device.index if qweight.device.index is not None else torch.cuda.current_device()
    return (qweight, scale, zero_point, bias, qweight.data_ptr(), scale.data_ptr(), zero_point.data_ptr(),
            None if bias is None else bias.data_ptr(), n, k, bits, group_size, index,
            load().bw_qlinear_decode_rows(n, k, bits))


def decode_with_plan(plan, x, m):
    """bw_qlinear on its decode path with buffers validated by make_decode_plan: only x is looked at.  Returns None
    when x does not qualify (layout, device, dtype, more rows than the decode path takes for this layer) - the
    caller then takes quantized_matmul_hip."""
    if m > plan[13]:
        return None
    dt = x.dtype
    if dt is torch.float16:
        act = BW_F16
    elif dt is torch.bfloat16:
        act = BW_BF16
    else:
        return None
    ldx = x.stride(0)
    xp = x.data_ptr()
    index = plan[12]
    if not x.is_cuda or x.stride(1) != 1 or (ldx * 2) % 16 or xp % 16 or x.shape[1] != plan[9] or \
            torch.cuda.current_device() != index:
        return None
    n = plan[8]
    y = torch.empty((m, n), dtype=torch.float16, device=x.device)
    st = _ENTRY["bw_qlinear"](xp, act, m, plan[9], ldx, plan[4], plan[5], plan[6], plan[7], n, plan[10], plan[11],
                              y.data_ptr(), n, _raw_stream(index))
    if st:
        if st == -2:
            return None
        _check(st, "bw_qlinear")
    return y


def input_grad_prefers_fused(m, n, k, bits, group_size, max_rows, large_max_rows):
    """Whether the backward should take the fused kernel for an m-row gradient: up to `max_rows` rows always (the
    kernel that walks N in steps of 32 rows); up to `large_max_rows` where the library's plan is its 256 x 256 kernel,
    which beats dequantise + library GEMM there (measured on Llama-shaped layers: 0.45-1.0 of its time up to 2048
    rows, 1.0-1.13 at 4096)."""
    return m <= max_rows or (m <= large_max_rows and load().bw_qdgrad_tile_rows(m, n, k, bits, group_size) == 257)


def quantized_input_grad(grad_y, qweight, scale, zero_point, bits, group_size):
    """grad_x[M,K] = grad_y[M,N] @ W[N,K] with the dequantisation fused in (bw_qdgrad), W being the dequantised weight
    in grad_y's dtype (float16 or bfloat16); None when the library has no fused kernel for this shape / dtype - the
    caller then dequantises and calls the library GEMM."""
    if grad_y.dtype not in (torch.float16, torch.bfloat16) or not grad_y.is_cuda or grad_y.dim() != 2:
        return None
    if qweight.dtype is not torch.int32 or scale.dtype is not torch.float16 or zero_point.dtype is not torch.float16:
        return None
    m, n = grad_y.shape
    k = qweight.shape[1] * (32 // bits)
    if m == 0 or qweight.shape[0] != n:
        return None
    if grad_y.stride(1) != 1 or grad_y.stride(0) % 8 or grad_y.data_ptr() % 16:
        grad_y = grad_y.contiguous()
        if grad_y.data_ptr() % 16:                         # contiguous already, but at an odd offset of its storage
            grad_y = grad_y.clone()
        if grad_y.stride(0) % 8:
            return None
    qweight, scale, zero_point = qweight.contiguous(), scale.contiguous(), zero_point.contiguous()
    lib = load()
    grad_x = torch.empty((m, k), dtype=grad_y.dtype, device=grad_y.device)
    with _on_device(grad_y.device) as index:
        nbytes = lib.bw_qdgrad_workspace_bytes(m, n, k, bits, group_size)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=grad_y.device) if nbytes else None
        st = lib.bw_qdgrad(grad_y.data_ptr(), _DTYPE_CODE[grad_y.dtype], m, n, grad_y.stride(0), qweight.data_ptr(), scale.data_ptr(),
                           zero_point.data_ptr(), k, bits, group_size, grad_x.data_ptr(), k,
                           None if ws is None else ws.data_ptr(), nbytes, _raw_stream(index))
    if st in (-2, -3):                                     # BW_EUNSUPPORTED / BW_EALIGN: the caller's unfused path
        return None
    _check(st, "bw_qdgrad")
    return grad_x


def last_decode_kernel():
    """Name of the decode kernel this thread's last bw_qgemv / bw_qlinear launch ran (a diagnostic for benchmarks)."""
    return load().bw_qgemv_last_kernel().decode()


def quantized_matmul_hip(x, qweight, scale, zero_point, bias, bits, group_size):
    """y[M,N] = x[M,K] @ dequant(qweight, scale, zero_point)^T + bias, float16 (main.py:433's operator)."""
    return _matmul("bw_qlinear", x, qweight, scale, zero_point, bias, bits, group_size)


def quantized_gemv_hip(x, qweight, scale, zero_point, bias, bits, group_size):
    """Decode kernel only (M <= 16)."""
    return _matmul("bw_qgemv", x, qweight, scale, zero_point, bias, bits, group_size)


def quantized_gemm_hip(x, qweight, scale, zero_point, bias, bits, group_size):
    """Prefill kernel only (any M)."""
    return _matmul("bw_qgemm", x, qweight, scale, zero_point, bias, bits, group_size)
