"""CPU restatement (numpy) of Bitween's quantized-linear hot path.

TEST INFRASTRUCTURE ONLY.  This module is the checker that the HIP kernels are
compared against; nothing in the shipped package imports it.  Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may use it.

Every function names the reference lines it restates (paths relative to the
reference checkout).  All arithmetic is IEEE-754 binary32 unless a function
says otherwise; numpy's float32 +,-,*,/ are correctly rounded and np.rint is
round-half-to-even, which is what torch.round does.

How each function is pinned (see tests/test_oracle_pins.py):
  pack_words / unpack_words   closed form sum(q_i << (i*bits)) mod 2**32 in
                              Python integers, hand-written words, round trip
  quantize_rtn (f32 math)     (both scale_div modes) exact-rational evaluation with explicit
                              round-to-nearest-even per operation, hand-derived
                              known answers, invariants, C restatement
  quantize_rtn (f16/bf16)     same exact-rational check with binary16/bfloat16
                              rounding after every operation; groups whose
                              scale rounds to zero are "parity unpinned"
                              (the reference divides by zero there)
  quantize_rtn_f64 / dequantize_rtn_f64   exact-rational evaluation with 53-bit rounding per operation
  store_module_buffers        numpy float16 cast is RNE (library routine)
  dequantize_f16              closed form RNE_f16(s16*(q-z)); product exact
  dequantize_rtn_f32          single binary32 multiply
  qlinear_forward             float64 dot of the fp16 operands, tolerance 1e-2
  qlinear_backward            float64 product with the same W16 (the float32
                              weight cast to float16 equals dequantize_f16:
                              the product is exact); brute-force loops on a
                              tiny case, one-hot rows, adjointness with the
                              forward
"""
import numpy as np

SUPPORTED_BITS = (2, 4, 8)


def _round_to(x32, math):
    """Round binary32 values to the storage type of a math mode, back in f32."""
    if math == "f32":
        return x32.astype(np.float32)
    if math == "f16":
        return x32.astype(np.float32).astype(np.float16).astype(np.float32)
    if math == "bf16":
        u = np.ascontiguousarray(x32, dtype=np.float32).view(np.uint32)
        nan = np.isnan(x32)
        r = ((u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) & np.uint32(0xFFFF0000))
        out = r.view(np.float32).copy()
        out[nan] = np.nan
        return out
    raise ValueError(math)


def pack_words(q, bits):
    """q int [N,K] in [0,2^bits) -> int32 [N, K*bits/32].

    bitween/functional.py:31-43: value k of a row sits in word k // vpi at bit
    offset (k % vpi) * bits (vpi = 32 // bits); the top slot may set the sign
    bit of the int32 word.
    """
    vpi = 32 // bits
    n, k = q.shape
    if k % vpi:
        raise ValueError("in_features must be a multiple of 32 // bits")
    lanes = q.astype(np.uint32).reshape(n, k // vpi, vpi)
    shifts = (np.arange(vpi, dtype=np.uint32) * np.uint32(bits))
    words = np.bitwise_or.reduce(lanes << shifts, axis=-1)
    return words.astype(np.uint32).view(np.int32)


def unpack_words(qweight, bits):
    """int32 [N,P] -> int32 [N, P*32/bits]; bitween/functional.py:56-64."""
    vpi = 32 // bits
    u = np.ascontiguousarray(qweight).view(np.uint32)
    shifts = (np.arange(vpi, dtype=np.uint32) * np.uint32(bits))
    vals = (u[:, :, None] >> shifts) & np.uint32((1 << bits) - 1)
    return vals.reshape(u.shape[0], -1).astype(np.int32)


def quantize_rtn(weight, bits=8, group_size=32, math="f32", scale_div="ieee"):
    """bitween/functional.py:3-45.

    scale_div: how the division of a tensor by the Python scalar Qmax (:25) is
    carried out.  "ieee" = a correctly rounded division, what eager torch does
    on the CPU.  "reciprocal" = what eager torch does on a GPU for a scalar
    divisor: a multiplication by float32(1) / float32(Qmax), the product
    rounded to float32 and then to the tensor's type (pinned on the GPU box
    against torch itself, tests/test_gpu_eager_torch.py, and by exact-rational
    vectors).

    Returns (qweight int32 [N,K*bits/32], scale [N,G], zero_point int32 [N,G],
    q int32 [N,K]).  `math` is the dtype the reference would compute in, i.e.
    the dtype of the tensor handed to it: "f32" is what
    QuantizedLinear.from_float uses (bitween/modules.py:191); "f16"/"bf16"
    round every intermediate to that type, as eager torch ops on a half tensor
    do.  scale is returned as float32 holding values of the math type.
    """
    assert bits in SUPPORTED_BITS, "Only 2, 4, or 8-bit quantization supported."
    w = _round_to(np.asarray(weight, dtype=np.float32), math)
    n, k = w.shape
    if k % group_size:
        pad = group_size - k % group_size
        raise ValueError(f"Padding {pad} columns to {k} to make it a multiple of {group_size}")
    qmax = np.float32((1 << bits) - 1)
    groups = k // group_size
    wg = w.reshape(n, groups, group_size)
    w_min = wg.min(axis=-1, keepdims=True)                       # :22
    w_max = wg.max(axis=-1, keepdims=True)                       # :23
    with np.errstate(all="ignore"):
        rng = _round_to(w_max - w_min, math)
        if scale_div == "ieee":
            scale = _round_to(rng / qmax, math)                  # :25
        elif scale_div == "reciprocal":
            scale = _round_to((rng * (np.float32(1.0) / qmax)).astype(np.float32), math)
        else:
            raise ValueError(scale_div)
        floor = _round_to(np.float32(1e-8).reshape(1), math)[0]  # 1e-8 is 0 in f16
        scale = np.maximum(scale, floor)
        zp_f = _round_to((-w_min) / scale, math)                 # :26
        zp_f = np.clip(np.rint(zp_f), np.float32(0), qmax)
        zero_point = zp_f.astype(np.int32)
        t = _round_to(wg / scale, math)                          # :29 divide ...
        t = _round_to(t + zp_f.astype(np.float32), math)         # ... then add
        q = np.clip(np.rint(t), np.float32(0), qmax).astype(np.int32)
    q = q.reshape(n, k)
    return pack_words(q, bits), scale.reshape(n, groups), zero_point.reshape(n, groups), q


def quantize_rtn_f64(weight, bits=8, group_size=32, scale_div="ieee"):
    """bitween/functional.py:3-45 on a float64 tensor: the same sequence in IEEE double arithmetic (numpy float64
    operations are correctly rounded), a float64 scale.  "reciprocal": the scalar division as a multiplication by
    1.0 / Qmax in double, what eager torch does on a GPU.  Pinned by exact-rational vectors with 53-bit rounding."""
    assert bits in SUPPORTED_BITS, "Only 2, 4, or 8-bit quantization supported."
    w = np.asarray(weight, dtype=np.float64)
    n, k = w.shape
    if k % group_size:
        pad = group_size - k % group_size
        raise ValueError(f"Padding {pad} columns to {k} to make it a multiple of {group_size}")
    qmax = np.float64((1 << bits) - 1)
    groups = k // group_size
    wg = w.reshape(n, groups, group_size)
    w_min = wg.min(axis=-1, keepdims=True)
    w_max = wg.max(axis=-1, keepdims=True)
    with np.errstate(all="ignore"):
        rng = w_max - w_min
        scale = rng / qmax if scale_div == "ieee" else rng * (np.float64(1.0) / qmax)
        scale = np.maximum(scale, np.float64(1e-8))
        zp_f = np.clip(np.rint((-w_min) / scale), 0.0, qmax)
        q = np.clip(np.rint(wg / scale + zp_f), 0.0, qmax).astype(np.int32)
    q = q.reshape(n, k)
    return pack_words(q, bits), scale.reshape(n, groups), zp_f.astype(np.int32).reshape(n, groups), q


def dequantize_rtn_f64(qweight, scale64, zero_point, group_size, bits=8):
    """bitween/functional.py:70 with a float64 scale: scale * (q.float() - zp.float()) promotes to float64; the
    difference is an exact small integer."""
    q = unpack_words(qweight, bits)
    n, k = q.shape
    groups = k // group_size
    d = q.reshape(n, groups, group_size).astype(np.float32) - np.asarray(zero_point).astype(np.float32).reshape(n, groups, 1)
    return (np.asarray(scale64, np.float64).reshape(n, groups, 1) * d.astype(np.float64)).reshape(n, k)


def store_module_buffers(scale, zero_point):
    """bitween/modules.py:174-178,207-209: the module keeps scale and
    zero_point as float16 (copy_ rounds to nearest even; zp <= 255 is exact)."""
    return np.asarray(scale, np.float32).astype(np.float16), np.asarray(zero_point).astype(np.float16)


def dequantize_rtn_f32(qweight, scale, zero_point, group_size, bits=8):
    """bitween/functional.py:47-71: scale * (q.float() - zp.float()) in float32.
    scale / zero_point may be the float32/int32 outputs of quantize_rtn or the
    float16 module buffers (promotion makes the arithmetic float32 either way)."""
    assert bits in SUPPORTED_BITS, "Only 2, 4, or 8-bit quantization supported."
    q = unpack_words(qweight, bits)
    n, k = q.shape
    groups = k // group_size
    qf = q.reshape(n, groups, group_size).astype(np.float32)
    s = np.asarray(scale).astype(np.float32).reshape(n, groups, 1)
    z = np.asarray(zero_point).astype(np.float32).reshape(n, groups, 1)
    return (s * (qf - z)).reshape(n, k)


def dequantize_f16(qweight, scale16, zp16, group_size, bits):
    """bitween/modules.py:10-58 (the live dequantize kernel): float16 result of
    the float32 product s16 * (q - z16); the product is exact in float32, so
    this is one rounding of the true value."""
    w32 = dequantize_rtn_f32(qweight, np.asarray(scale16, np.float16), np.asarray(zp16, np.float16), group_size, bits)
    return w32.astype(np.float16)


def dequantize_bf16(qweight, scale16, zp16, group_size, bits):
    """bfloat16 variant of dequantize_f16 (the reference is float16 only; this
    is the additive dtype option used for bf16 prefill activations).  Returned
    as float32 holding bfloat16 values."""
    w32 = dequantize_rtn_f32(qweight, np.asarray(scale16, np.float16), np.asarray(zp16, np.float16), group_size, bits)
    return _round_to(w32, "bf16")


def qlinear_forward(x16, qweight, scale16, zp16, bias16, bits, group_size):
    """bitween/modules.py:62-106 and main.py:444-466: y = x16 @ W16.T (+ bias),
    float16 out.  The dot product is taken in float64 here; the reference's
    BLAS accumulates in float32, so agreement is to tolerance (1e-2 relative,
    main.py:471-477), not bit-exact.  Returns (y as float16-valued float32,
    y64 before any output rounding)."""
    w = dequantize_f16(qweight, scale16, zp16, group_size, bits).astype(np.float64)
    xa = np.asarray(x16, np.float16).astype(np.float64)
    y64 = xa @ w.T
    y = _round_to(y64.astype(np.float32), "f16")
    if bias16 is not None:
        b = np.asarray(bias16).astype(np.float32)
        y64 = y64 + b.astype(np.float64)
        y = _round_to(y + b, "f16")                    # second rounding, modules.py:100-101
    return y, y64


def qlinear_backward(grad_out, qweight, scale16, zp16, bits, group_size, dtype="f16"):
    """bitween/modules.py:108-141: grad_input = grad_output @ W, W being the
    float32 dequantized weight cast to grad_output's dtype: float16 (default)
    or bfloat16 (`grad_out` is then a float32 array holding bfloat16 values).
    Float64 accumulate, tolerance as for the forward."""
    w32 = dequantize_rtn_f32(qweight, scale16, zp16, group_size, bits)
    if dtype == "f16":
        w = w32.astype(np.float16).astype(np.float64)
        go = np.asarray(grad_out, np.float16).astype(np.float64)
    elif dtype == "bf16":
        w = _round_to(w32, "bf16").astype(np.float64)
        go = np.asarray(grad_out, np.float32)
        assert np.array_equal(go, _round_to(go, "bf16")), "grad_out must hold bfloat16 values"
        go = go.astype(np.float64)
    else:
        raise ValueError("dtype must be 'f16' or 'bf16'")
    return go @ w
