// RTN per-group quantise + pack, and the stand-alone dequantise.
//
// bw_quantize_pack restates bitween/functional.py:3-45 as ONE kernel: a
// thread owns one packed output word (32/bits consecutive weights), the
// group/(32/bits) threads of a group agree on min and max with cross-lane
// shuffles, and every thread then forms scale, zero point and its own
// quantised values with the same sequence of correctly rounded IEEE
// operations eager torch performs: (max-min)/Qmax, clamp(1e-8), -min/scale,
// round-half-even, clamp; then w/scale, a separate add of the zero point,
// round-half-even, clamp.  Divisions are true IEEE divisions (x/15 differs
// from x*(1/15)), nothing is contracted into FMAs, denormals are kept.
// The weights are read once (2 or 4 bytes each) and bits/8 + 4/group bytes are
// written: HBM-bound, with the divide sequence as the ALU cost.
#include "bw_common.h"

namespace {

// Rounding of every intermediate to the "math" dtype (float32: identity).
template <int MATH> BW_DEV float rnd(float v);
template <> BW_DEV float rnd<BW_F32>(float v) { return v; }
template <> BW_DEV float rnd<BW_F16>(float v) { return (float)(_Float16)v; }
template <> BW_DEV float rnd<BW_BF16>(float v) { return bf16_to_f32(f32_to_bf16(v)); }

template <int DT> struct Elem;
template <> struct Elem<BW_F32> { typedef float T; static BW_DEV float load(const void* p, int64_t i) { return ((const float*)p)[i]; } };
template <> struct Elem<BW_F16> { typedef _Float16 T; static BW_DEV float load(const void* p, int64_t i) { return (float)((const _Float16*)p)[i]; } };
template <> struct Elem<BW_BF16> { typedef uint16_t T; static BW_DEV float load(const void* p, int64_t i) { return bf16_to_f32(((const uint16_t*)p)[i]); } };

BW_DEV void store_meta(void* p, int dtype, int64_t i, float v) {
    if (dtype == BW_F32) ((float*)p)[i] = v;
    else if (dtype == BW_F16) ((_Float16*)p)[i] = (_Float16)v;
    else if (dtype == BW_BF16) ((uint16_t*)p)[i] = f32_to_bf16(v);
    else ((int32_t*)p)[i] = (int32_t)v;
}

// Load the VPI consecutive weights of one output word as float32.
template <int WDT, int VPI>
BW_DEV void load_vals(const void* w, int64_t off, float* v) {
    if constexpr (WDT == BW_F32) {
        const f4* p = reinterpret_cast<const f4*>((const float*)w + off);
#pragma unroll
        for (int i = 0; i < VPI / 4; i++) { f4 t = p[i]; v[4 * i] = t[0]; v[4 * i + 1] = t[1]; v[4 * i + 2] = t[2]; v[4 * i + 3] = t[3]; }
    } else if constexpr (VPI == 4) {
        const u2 t = *reinterpret_cast<const u2*>((const uint16_t*)w + off);
        const uint16_t h[4] = {(uint16_t)t[0], (uint16_t)(t[0] >> 16), (uint16_t)t[1], (uint16_t)(t[1] >> 16)};
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] = WDT == BW_F16 ? (float)__builtin_bit_cast(_Float16, h[i]) : bf16_to_f32(h[i]);
    } else {
        const u4* p = reinterpret_cast<const u4*>((const uint16_t*)w + off);
#pragma unroll
        for (int i = 0; i < VPI / 8; i++) {
            const u4 t = p[i];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint16_t lo = (uint16_t)t[j], hi = (uint16_t)(t[j] >> 16);
                v[8 * i + 2 * j] = WDT == BW_F16 ? (float)__builtin_bit_cast(_Float16, lo) : bf16_to_f32(lo);
                v[8 * i + 2 * j + 1] = WDT == BW_F16 ? (float)__builtin_bit_cast(_Float16, hi) : bf16_to_f32(hi);
            }
        }
    }
}

// One thread per packed word; LPG = group / VPI threads (a power of two <= 64,
// aligned inside the wave) cooperate on one group.
template <int BITS, int WDT, int MATH>
__global__ __launch_bounds__(256) void quantize_pack_kernel(const void* __restrict__ w, int64_t N, int K, int64_t ldw,
                                                            int group, int lpg, int32_t* __restrict__ qweight,
                                                            void* __restrict__ scale, int scale_dtype,
                                                            void* __restrict__ zp, int zp_dtype) {
    constexpr int VPI = 32 / BITS;
    constexpr float QMAX = (float)((1 << BITS) - 1);
    const int words = K / VPI;
    const int64_t total = N * (int64_t)words;
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const bool live = idx < total;
    if (!live) idx = total - 1;          // keep the whole wave in the shuffles; stores are masked
    const int64_t row = idx / words;
    const int wcol = (int)(idx - row * words);
    float v[VPI];
    load_vals<WDT, VPI>(w, row * ldw + (int64_t)wcol * VPI, v);
    float lo = v[0], hi = v[0];
#pragma unroll
    for (int i = 0; i < VPI; i++) { v[i] = rnd<MATH>(v[i]); }
    lo = hi = v[0];
#pragma unroll
    for (int i = 1; i < VPI; i++) { lo = fminf(lo, v[i]); hi = fmaxf(hi, v[i]); }
    for (int d = 1; d < lpg; d <<= 1) {
        lo = fminf(lo, __shfl_xor(lo, d));
        hi = fmaxf(hi, __shfl_xor(hi, d));
    }
    float s = rnd<MATH>(__fdiv_rn(rnd<MATH>(__fsub_rn(hi, lo)), QMAX));          // functional.py:25
    s = fmaxf(s, rnd<MATH>(1e-8f));
    float zf = rintf(rnd<MATH>(__fdiv_rn(-lo, s)));                                // functional.py:26
    zf = fminf(fmaxf(zf, 0.f), QMAX);
    uint32_t word = 0;
#pragma unroll
    for (int i = 0; i < VPI; i++) {
        float t = rnd<MATH>(__fdiv_rn(v[i], s));                                   // functional.py:29: divide,
        t = rnd<MATH>(__fadd_rn(t, zf));                                           // then a separate add
        t = fminf(fmaxf(rintf(t), 0.f), QMAX);
        word |= (uint32_t)(int)t << (i * BITS);
    }
    if (live) {
        qweight[idx] = (int32_t)word;
        const int k = wcol * VPI;
        if (k % group == 0) {
            const int64_t gi = row * (K / group) + k / group;
            store_meta(scale, scale_dtype, gi, s);
            store_meta(zp, zp_dtype, gi, zf);
        }
    }
}

// Any group size (including ones that are not a power-of-two multiple of the
// word width): one thread per group, two passes over its values.
template <int WDT, int MATH>
__global__ void quantize_group_generic_kernel(const void* __restrict__ w, int64_t N, int K, int64_t ldw, int bits, int group,
                                              uint8_t* __restrict__ qtmp, void* __restrict__ scale, int scale_dtype,
                                              void* __restrict__ zp, int zp_dtype) {
    const int groups = K / group;
    const int64_t gi = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gi >= N * groups) return;
    const int64_t row = gi / groups;
    const int64_t base = row * ldw + (gi - row * groups) * group;
    const float qmax = (float)((1 << bits) - 1);
    float lo = rnd<MATH>(Elem<WDT>::load(w, base)), hi = lo;
    for (int i = 1; i < group; i++) { const float t = rnd<MATH>(Elem<WDT>::load(w, base + i)); lo = fminf(lo, t); hi = fmaxf(hi, t); }
    float s = rnd<MATH>(__fdiv_rn(rnd<MATH>(__fsub_rn(hi, lo)), qmax));
    s = fmaxf(s, rnd<MATH>(1e-8f));
    float zf = fminf(fmaxf(rintf(rnd<MATH>(__fdiv_rn(-lo, s))), 0.f), qmax);
    store_meta(scale, scale_dtype, gi, s);
    store_meta(zp, zp_dtype, gi, zf);
    for (int i = 0; i < group; i++) {
        float t = rnd<MATH>(__fdiv_rn(rnd<MATH>(Elem<WDT>::load(w, base + i)), s));
        t = rnd<MATH>(__fadd_rn(t, zf));
        qtmp[row * K + (gi - row * groups) * group + i] = (uint8_t)(int)fminf(fmaxf(rintf(t), 0.f), qmax);
    }
}

// out[n][k] = scale * (q - zp): float32 product, rounded once to the output type.
template <int BITS, int ODT>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint32_t* __restrict__ qweight, const void* __restrict__ scale,
                                                         int scale_dtype, const void* __restrict__ zp, int zp_dtype,
                                                         int64_t N, int K, int group, void* __restrict__ out, int64_t ldo) {
    constexpr int VPI = 32 / BITS;
    const int words = K / VPI, groups = K / group;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= N * (int64_t)words) return;
    const int64_t row = idx / words;
    const int wcol = (int)(idx - row * words);
    const uint32_t w = qweight[idx];
    float r[VPI];
    int gprev = -1;
    float s = 0.f, z = 0.f;
#pragma unroll
    for (int i = 0; i < VPI; i++) {
        const int g = (wcol * VPI + i) / group;
        if (g != gprev) {
            const int64_t gi = row * groups + g;
            s = scale_dtype == BW_F32 ? ((const float*)scale)[gi] : (float)((const _Float16*)scale)[gi];
            z = zp_dtype == BW_I32 ? (float)((const int32_t*)zp)[gi] : (float)((const _Float16*)zp)[gi];
            gprev = g;
        }
        const float q = (float)((w >> (i * BITS)) & ((1u << BITS) - 1));
        r[i] = __fmul_rn(s, __fsub_rn(q, z));                                      // functional.py:70, modules.py:55
    }
    const int64_t o = row * ldo + (int64_t)wcol * VPI;
    if constexpr (ODT == BW_F32) {
        float* p = (float*)out + o;
#pragma unroll
        for (int i = 0; i < VPI; i++) p[i] = r[i];
    } else {
        uint16_t* p = (uint16_t*)out + o;
#pragma unroll
        for (int i = 0; i < VPI; i++)
            p[i] = ODT == BW_F16 ? __builtin_bit_cast(uint16_t, (_Float16)r[i]) : f32_to_bf16(r[i]);
    }
}

template <int BITS, int WDT, int MATH>
int launch_quantize(const void* w, int64_t N, int64_t K, int64_t ldw, int group, int32_t* qweight, void* scale, int sdt,
                    void* zp, int zdt, hipStream_t st) {
    const int vpi = 32 / BITS;
    const int64_t total = N * (K / vpi);
    hipLaunchKernelGGL((quantize_pack_kernel<BITS, WDT, MATH>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, w, N,
                       (int)K, ldw, group, group / vpi, qweight, scale, sdt, zp, zdt);
    return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
}

template <int WDT, int MATH>
int dispatch_bits(int bits, const void* w, int64_t N, int64_t K, int64_t ldw, int group, int32_t* qweight, void* scale,
                  int sdt, void* zp, int zdt, hipStream_t st) {
    if (bits == 2) return launch_quantize<2, WDT, MATH>(w, N, K, ldw, group, qweight, scale, sdt, zp, zdt, st);
    if (bits == 4) return launch_quantize<4, WDT, MATH>(w, N, K, ldw, group, qweight, scale, sdt, zp, zdt, st);
    return launch_quantize<8, WDT, MATH>(w, N, K, ldw, group, qweight, scale, sdt, zp, zdt, st);
}

}  // namespace

extern "C" int bw_quantize_pack(const void* w, int w_dtype, int math_dtype, int64_t N, int64_t K, int64_t ldw, int bits,
                                int group, int32_t* qweight, void* scale, int scale_dtype, void* zp, int zp_dtype,
                                void* stream) {
    if (!w || !qweight || !scale || !zp) return BW_EINVAL;
    if (!bw_shape_ok(N, K, bits, group) || ldw < K) return BW_EINVAL;
    if (w_dtype != BW_F16 && w_dtype != BW_BF16 && w_dtype != BW_F32) return BW_EINVAL;
    if (scale_dtype != BW_F32 && scale_dtype != BW_F16 && scale_dtype != BW_BF16) return BW_EINVAL;
    if (zp_dtype != BW_I32 && zp_dtype != BW_F16 && zp_dtype != BW_BF16) return BW_EINVAL;
    // math in a 16-bit type only makes sense on weights of that type (eager torch never mixes them)
    if (math_dtype != BW_F32 && math_dtype != w_dtype) return BW_EINVAL;
    const int vpi = 32 / bits;
    const int lpg = group / vpi;
    const bool pow2 = group % vpi == 0 && lpg >= 1 && lpg <= 64 && (lpg & (lpg - 1)) == 0;
    // vector loads of one word's worth of weights: 16-byte (or 8-byte for 4 halves) alignment
    const size_t esz = w_dtype == BW_F32 ? 4 : 2;
    const size_t need = (vpi * esz >= 16) ? 16 : vpi * esz;
    if (!pow2) return BW_EUNSUPPORTED;   // needs a byte scratch plane; see bw_quantize_pack in the header
    if (!bw_aligned(w, need) || (ldw * esz) % need) return BW_EALIGN;
    hipStream_t st = (hipStream_t)stream;
#define BW_Q(WD, MD) \
    if (w_dtype == WD && math_dtype == MD) return dispatch_bits<WD, MD>(bits, w, N, K, ldw, group, qweight, scale, scale_dtype, zp, zp_dtype, st);
    BW_Q(BW_F32, BW_F32) BW_Q(BW_F16, BW_F32) BW_Q(BW_BF16, BW_F32) BW_Q(BW_F16, BW_F16) BW_Q(BW_BF16, BW_BF16)
#undef BW_Q
    return BW_EINVAL;
}

extern "C" int bw_dequantize(const int32_t* qweight, const void* scale, int scale_dtype, const void* zp, int zp_dtype,
                             int64_t N, int64_t K, int bits, int group, void* w_out, int out_dtype, int64_t ldo,
                             void* stream) {
    if (!qweight || !scale || !zp || !w_out) return BW_EINVAL;
    if (!bw_shape_ok(N, K, bits, group) || ldo < K) return BW_EINVAL;
    if (scale_dtype != BW_F32 && scale_dtype != BW_F16) return BW_EINVAL;
    if (zp_dtype != BW_I32 && zp_dtype != BW_F16) return BW_EINVAL;
    if (out_dtype != BW_F32 && out_dtype != BW_F16 && out_dtype != BW_BF16) return BW_EINVAL;
    const int vpi = 32 / bits;
    const int64_t total = N * (K / vpi);
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    hipStream_t st = (hipStream_t)stream;
#define BW_D(B, OD)                                                                                                     \
    if (bits == B && out_dtype == OD) {                                                                                 \
        hipLaunchKernelGGL((dequantize_kernel<B, OD>), grid, block, 0, st, (const uint32_t*)qweight, scale, scale_dtype, zp, \
                           zp_dtype, N, (int)K, group, w_out, ldo);                                                     \
        return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;                                                    \
    }
    BW_D(2, BW_F32) BW_D(4, BW_F32) BW_D(8, BW_F32) BW_D(2, BW_F16) BW_D(4, BW_F16) BW_D(8, BW_F16)
    BW_D(2, BW_BF16) BW_D(4, BW_BF16) BW_D(8, BW_BF16)
#undef BW_D
    return BW_EINVAL;
}

extern "C" int bw_abi_version(void) { return 1; }

extern "C" const char* bw_strerror(int status) {
    switch (status) {
        case BW_OK: return "ok";
        case BW_EINVAL: return "invalid argument (bits must be 2/4/8, K % group == 0, K % (32/bits) == 0, pointers non-null)";
        case BW_EUNSUPPORTED: return "combination not implemented by this library";
        case BW_EALIGN: return "pointer or row pitch not aligned for vector access";
        case BW_ELAUNCH: return "HIP kernel launch failed";
        case BW_EWORKSPACE: return "workspace missing or too small";
        default: return "unknown status";
    }
}
