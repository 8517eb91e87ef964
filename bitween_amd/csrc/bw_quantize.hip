// RTN per-group quantise + pack, and the stand-alone dequantise.
//
// bw_quantize_pack restates bitween/functional.py:3-45 as ONE kernel: a
// thread owns a few packed output words, the threads of a group agree on min
// and max with cross-lane shuffles, and every thread then forms scale, zero
// point and its own quantised values with the results of the same sequence
// of correctly rounded IEEE operations eager torch performs: (max-min)/Qmax,
// clamp(1e-8), -min/scale, round-half-even, clamp; then w/scale, a separate
// add of the zero point, round-half-even, clamp.  Divisions are true IEEE
// divisions (x/15 differs from x*(1/15)) or provably give the same rounded
// integer, nothing else is contracted into FMAs, denormals are kept.
// The weights are read once (2 or 4 bytes each) and bits/8 + 4/group bytes are
// written: HBM-bound.
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

// scale and zero point of one group from its extrema, exactly as functional.py:25-26.  The division by the
// Python scalar Qmax is a true division in eager torch on the CPU; on a GPU torch multiplies by the float32
// reciprocal of a scalar divisor instead (one float32 rounding of the product, then the tensor's type), which
// differs in the last bit of most float32 scales: `recip` selects that arithmetic.
template <int MATH>
BW_DEV void group_params(float lo, float hi, float qmax, bool recip, float& s, float& zf) {
    const float range = rnd<MATH>(__fsub_rn(hi, lo));
    s = rnd<MATH>(recip ? __fmul_rn(range, __fdiv_rn(1.0f, qmax)) : __fdiv_rn(range, qmax));
    s = fmaxf(s, rnd<MATH>(1e-8f));
    zf = rintf(rnd<MATH>(__fdiv_rn(-lo, s)));
    zf = fminf(fmaxf(zf, 0.f), qmax);
}

// round(w / s + zf) before the clamp, exactly as functional.py:29: an IEEE divide, then a separate add
template <int MATH>
BW_DEV float quant_exact(float w, float s, float zf) {
    return rintf(rnd<MATH>(__fadd_rn(rnd<MATH>(__fdiv_rn(w, s)), zf)));
}

// A thread owns WPT consecutive packed words (VPT = WPT * 32/bits weights, 32 bytes of 16-bit input where
// the shape allows); the lpg = group / VPT threads of a group (a power of two <= 64, aligned inside the
// wave) agree on min and max with cross-lane shuffles.
//
// float32 math takes a short cut that cannot change a result.  With x = w / s, r = 1/s refined once (relative
// error <= 2^-23), F = fma(w, r, zf) and the reference's A = fl(fl(x) + zf):
//     |F - (x + zf)| <= |x| 2^-23 + |F| 2^-24,      |A - (x + zf)| <= |x| 2^-24 + |A| 2^-24,
// so |F - A| <= 2^-23 (1.5 |x| + max(|F|, |A|)) <= 2.5 * 2^-23 * B with B = max|x| of the group + Qmax + 3 (an upper
// bound of |x|, |F| and |A|, with room for the rounding of B itself).  Unless F lies within 2^-21 B (> 2.5 * 2^-23 B)
// of a half-integer, round(F) is therefore the reference's value.  B is formed once per group from its extrema: a
// group of 4-bit weights that straddles zero has B ~ 20, a window of 1e-5 around the ties instead of a fixed one
// sized for the worst case - the exact path, which a wave enters when any of its lanes needs it, was what a third
// of the kernel's arithmetic went into.  Values inside the window (and infinities, NaN, groups so lopsided that the
// window exceeds 1/2) are redone with the true IEEE divide.
template <int BITS, int WDT, int MATH, int WPT>
__global__ __launch_bounds__(256) void quantize_pack_kernel(const void* __restrict__ w, const void* __restrict__ delta,
                                                            int64_t N, int K, int64_t ldw, int64_t ldd,
                                                            int group, int lpg, int32_t* __restrict__ qweight,
                                                            void* __restrict__ scale, int scale_dtype,
                                                            void* __restrict__ zp, int zp_dtype, int recip) {
    constexpr int VPI = 32 / BITS, VPT = VPI * WPT;
    constexpr float QMAX = (float)((1 << BITS) - 1);
    const int tpr = K / VPT;                             // threads per row; grid.x covers them, grid.y the rows
    int tcol = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    const bool live = tcol < tpr;
    if (!live) tcol = tpr - 1;           // keep the whole wave in the shuffles; stores are masked
    const int groups = K / group;
    for (int64_t row = blockIdx.y; row < N; row += gridDim.y) {
        float v[VPT];
        load_vals<WDT, VPT>(w, row * ldw + (int64_t)tcol * VPT, v);
        if (delta) {                                     // w + delta, one rounding to the weights' own type
            float dv[VPT];
            load_vals<WDT, VPT>(delta, row * ldd + (int64_t)tcol * VPT, dv);
#pragma unroll
            for (int i = 0; i < VPT; i++) v[i] = rnd<WDT>(__fadd_rn(v[i], dv[i]));
        }
#pragma unroll
        for (int i = 0; i < VPT; i++) { v[i] = rnd<MATH>(v[i]); }
        float lo = v[0], hi = v[0];
#pragma unroll
        for (int i = 1; i < VPT; i++) { lo = fminf(lo, v[i]); hi = fmaxf(hi, v[i]); }
        for (int d = 1; d < lpg; d <<= 1) {
            lo = fminf(lo, __shfl_xor(lo, d));
            hi = fmaxf(hi, __shfl_xor(hi, d));
        }
        float s, zf;
        group_params<MATH>(lo, hi, QMAX, recip != 0, s, zf);
        float t[VPT];
        if constexpr (MATH == BW_F32) {
            const float r0 = __builtin_amdgcn_rcpf(s);
            const float r = __builtin_fmaf(__builtin_fmaf(-s, r0, 1.0f), r0, r0);
            const float bound = __builtin_fmaf(fmaxf(fabsf(lo), fabsf(hi)), r, QMAX + 3.0f);
            const float safe = __builtin_fmaf(-0x1p-21f, bound, 0.5f);   // NaN extrema: every comparison below fails
#pragma unroll
            for (int i = 0; i < VPT; i++) {
                const float sum = __builtin_fmaf(v[i], r, zf);
                t[i] = rintf(sum);
                // far enough from a tie?  (an infinite sum gives NaN here and fails the test.)  Else redo with the true divide.
                if (!(fabsf(__fsub_rn(sum, t[i])) < safe)) t[i] = quant_exact<MATH>(v[i], s, zf);
            }
        } else {
#pragma unroll
            for (int i = 0; i < VPT; i++) t[i] = quant_exact<MATH>(v[i], s, zf);
        }
        // pack: the clamped values are small integers, so 16 bits' worth of fields add up exactly in float32
        constexpr int FPH = 16 / BITS;                    // fields per 16-bit half word
        uint32_t word[WPT];
#pragma unroll
        for (int j = 0; j < WPT; j++) {
            float half[2] = {0.f, 0.f};
#pragma unroll
            for (int i = 0; i < VPI; i++)
                half[i / FPH] = __builtin_fmaf(__builtin_amdgcn_fmed3f(t[j * VPI + i], 0.f, QMAX), (float)(1 << ((i % FPH) * BITS)), half[i / FPH]);
            word[j] = (uint32_t)half[0] | ((uint32_t)half[1] << 16);
        }
        if (live) {
            uint32_t* dst = reinterpret_cast<uint32_t*>(qweight) + (row * tpr + tcol) * WPT;
            if constexpr (WPT == 8) {
                reinterpret_cast<u4*>(dst)[0] = u4{word[0], word[1], word[2], word[3]};
                reinterpret_cast<u4*>(dst)[1] = u4{word[4], word[5], word[6], word[7]};
            } else if constexpr (WPT == 4) *reinterpret_cast<u4*>(dst) = u4{word[0], word[1], word[2], word[3]};
            else if constexpr (WPT == 2) *reinterpret_cast<u2*>(dst) = u2{word[0], word[1]};
            else dst[0] = word[0];
            const int k = tcol * VPT;
            if (k % group == 0) {
                const int64_t gi = row * groups + k / group;
                store_meta(scale, scale_dtype, gi, s);
                store_meta(zp, zp_dtype, gi, zf);
            }
        }
    }
}

// Any group size: one thread per packed word, which scans the whole group of each of its values for the
// extrema (re-using them while consecutive values share a group).  Slow, exact, no scratch memory.
template <int WDT, int MATH>
__global__ __launch_bounds__(256) void quantize_pack_generic_kernel(const void* __restrict__ w, const void* __restrict__ delta,
                                                                    int64_t N, int K, int64_t ldw, int64_t ldd,
                                                                    int bits, int group, int32_t* __restrict__ qweight,
                                                                    void* __restrict__ scale, int scale_dtype,
                                                                    void* __restrict__ zp, int zp_dtype, int recip) {
    const int vpi = 32 / bits, words = K / vpi, groups = K / group;
    const float qmax = (float)((1 << bits) - 1);
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= N * (int64_t)words) return;
    const int64_t row = idx / words;
    const int wcol = (int)(idx - row * words);
    uint32_t word = 0;
    int gprev = -1;
    float s = 0.f, zf = 0.f;
    auto value = [&](int k) {
        float x = Elem<WDT>::load(w, row * ldw + k);
        if (delta) x = rnd<WDT>(__fadd_rn(x, Elem<WDT>::load(delta, row * ldd + k)));
        return rnd<MATH>(x);
    };
    for (int i = 0; i < vpi; i++) {
        const int k = wcol * vpi + i, g = k / group;
        if (g != gprev) {
            float lo = value(g * group), hi = lo;
            for (int e = 1; e < group; e++) {
                const float x = value(g * group + e);
                lo = fminf(lo, x);
                hi = fmaxf(hi, x);
            }
            group_params<MATH>(lo, hi, qmax, recip != 0, s, zf);
            gprev = g;
            if (k == g * group) {                        // the thread holding a group's first value stores its parameters
                store_meta(scale, scale_dtype, row * groups + g, s);
                store_meta(zp, zp_dtype, row * groups + g, zf);
            }
        }
        const float t = quant_exact<MATH>(value(k), s, zf);
        word |= (uint32_t)(int)fminf(fmaxf(t, 0.f), qmax) << (i * bits);
    }
    qweight[idx] = (int32_t)word;
}

// float64 weights (functional.py:3-45 is dtype-agnostic: a float64 tensor is quantised in float64 arithmetic and
// returns a float64 scale).  Rare, so the simple layout: one thread per packed word scanning the group(s) of its
// values; every operation is the IEEE double operation the reference's eager ops perform.
__global__ __launch_bounds__(256) void quantize_pack_f64_kernel(const double* __restrict__ w, const double* __restrict__ delta,
                                                                int64_t N, int K, int64_t ldw, int64_t ldd, int bits, int group,
                                                                int32_t* __restrict__ qweight, double* __restrict__ scale,
                                                                int32_t* __restrict__ zp, int recip) {
    const int vpi = 32 / bits, words = K / vpi, groups = K / group;
    const double qmax = (double)((1 << bits) - 1);
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= N * (int64_t)words) return;
    const int64_t row = idx / words;
    const int wcol = (int)(idx - row * words);
    uint32_t word = 0;
    int gprev = -1;
    double s = 0.0, zf = 0.0;
    auto value = [&](int k) {
        double x = w[row * ldw + k];
        if (delta) x = __dadd_rn(x, delta[row * ldd + k]);
        return x;
    };
    for (int i = 0; i < vpi; i++) {
        const int k = wcol * vpi + i, g = k / group;
        if (g != gprev) {
            double lo = value(g * group), hi = lo;
            for (int e = 1; e < group; e++) {
                const double x = value(g * group + e);
                lo = fmin(lo, x);
                hi = fmax(hi, x);
            }
            const double range = __dsub_rn(hi, lo);
            s = recip ? __dmul_rn(range, __ddiv_rn(1.0, qmax)) : __ddiv_rn(range, qmax);
            s = fmax(s, 1e-8);
            zf = fmin(fmax(rint(__ddiv_rn(-lo, s)), 0.0), qmax);
            gprev = g;
            if (k == g * group) {
                scale[row * groups + g] = s;
                zp[row * groups + g] = (int32_t)zf;
            }
        }
        const double t = rint(__dadd_rn(__ddiv_rn(value(k), s), zf));
        word |= (uint32_t)(int)fmin(fmax(t, 0.0), qmax) << (i * bits);
    }
    qweight[idx] = (int32_t)word;
}

// functional.py:70 with a float64 scale: scale * (q.float() - zp.float()) promotes to float64; q - zp is exact.
__global__ __launch_bounds__(256) void dequantize_f64_kernel(const uint32_t* __restrict__ qweight, const double* __restrict__ scale,
                                                             const void* __restrict__ zp, int zp_dtype, int64_t N, int K, int bits,
                                                             int group, double* __restrict__ out, int64_t ldo) {
    const int vpi = 32 / bits, words = K / vpi, groups = K / group;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= N * (int64_t)words) return;
    const int64_t row = idx / words;
    const int wcol = (int)(idx - row * words);
    const uint32_t word = qweight[idx], mask = (1u << bits) - 1;
    for (int i = 0; i < vpi; i++) {
        const int k = wcol * vpi + i;
        const int64_t gi = row * groups + k / group;
        const float z = zp_dtype == BW_I32 ? (float)((const int32_t*)zp)[gi] : (float)((const _Float16*)zp)[gi];
        const float d = __fsub_rn((float)((word >> (i * bits)) & mask), z);
        out[row * ldo + k] = __dmul_rn(scale[gi], (double)d);
    }
}

// out[n][k] = scale * (q - zp): float32 product, rounded once to the output type.  A thread owns one packed word
// (32 / BITS weights); grid.x runs along the row, grid.y over rows.  VEC: the row pitch and base of `out` allow
// 16-byte stores (8-byte for the 8 bytes an 8-bit word becomes in a 16-bit type).
template <int BITS, int ODT, bool VEC>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint32_t* __restrict__ qweight, const void* __restrict__ scale,
                                                         int scale_dtype, const void* __restrict__ zp, int zp_dtype,
                                                         int64_t N, int K, int group, void* __restrict__ out, int64_t ldo) {
    constexpr int VPI = 32 / BITS;
    const int words = K / VPI, groups = K / group;
    const int wcol = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (wcol >= words) return;
    for (int64_t row = blockIdx.y; row < N; row += gridDim.y) {
        const uint32_t w = qweight[row * words + wcol];
        float r[VPI];
        auto load_sz = [&](int g, float& s, float& z) {
            const int64_t gi = row * groups + g;
            s = scale_dtype == BW_F32 ? ((const float*)scale)[gi] : (float)((const _Float16*)scale)[gi];
            z = zp_dtype == BW_I32 ? (float)((const int32_t*)zp)[gi] : (float)((const _Float16*)zp)[gi];
        };
        const int g_first = (wcol * VPI) / group, g_last = (wcol * VPI + VPI - 1) / group;
        float s = 0.f, z = 0.f;
        load_sz(g_first, s, z);
#pragma unroll
        for (int i = 0; i < VPI; i++) {
            if (g_first != g_last && i > 0 && (wcol * VPI + i) % group == 0) load_sz((wcol * VPI + i) / group, s, z);   // rare: groups narrower than a word
            const float q = (float)((w >> (i * BITS)) & ((1u << BITS) - 1));
            r[i] = __fmul_rn(s, __fsub_rn(q, z));                                  // functional.py:70, modules.py:55
            // keep the product a value of its own: folded into a mixed-precision multiply-add with a +0 addend
            // (what the compiler makes of multiply + narrowing conversion) 0 * -3 would lose its sign
            asm volatile("" : "+v"(r[i]));
        }
        const int64_t o = row * ldo + (int64_t)wcol * VPI;
        if constexpr (ODT == BW_F32) {
            float* p = (float*)out + o;
            if constexpr (VEC) {
#pragma unroll
                for (int i = 0; i < VPI; i += 4) *reinterpret_cast<f4*>(p + i) = f4{r[i], r[i + 1], r[i + 2], r[i + 3]};
            } else {
#pragma unroll
                for (int i = 0; i < VPI; i++) p[i] = r[i];
            }
        } else {
            uint16_t h[VPI];
#pragma unroll
            for (int i = 0; i < VPI; i++) h[i] = ODT == BW_F16 ? __builtin_bit_cast(uint16_t, (_Float16)r[i]) : f32_to_bf16(r[i]);
            uint16_t* p = (uint16_t*)out + o;
            if constexpr (VEC) {
                uint32_t d[VPI / 2];
#pragma unroll
                for (int i = 0; i < VPI / 2; i++) d[i] = (uint32_t)h[2 * i] | ((uint32_t)h[2 * i + 1] << 16);
                if constexpr (VPI == 4) {
                    *reinterpret_cast<u2*>(p) = u2{d[0], d[1]};
                } else {
#pragma unroll
                    for (int i = 0; i < VPI / 2; i += 4) *reinterpret_cast<u4*>(p + 2 * i) = u4{d[i], d[i + 1], d[i + 2], d[i + 3]};
                }
            } else {
#pragma unroll
                for (int i = 0; i < VPI; i++) p[i] = h[i];
            }
        }
    }
}

// The same for the usual layouts, four words per thread, 256 words apart so that every load and store instruction of
// a wave stays contiguous.  All four words and their (scale, zero point) are requested before the first is used: with
// one 4-byte load per thread the kernel waits a memory round trip per 16 bytes it writes.  The group is a power of
// two and at least a word wide, so a shift finds it; scale / zero point float16 (the module buffers) or float32 /
// int32 (what quantize_rtn returns) are told apart once per thread, not per value.
template <int BITS, int ODT>
__global__ __launch_bounds__(256) void dequantize_x4_kernel(const uint32_t* __restrict__ qweight, const void* __restrict__ scale,
                                                            const void* __restrict__ zp, int module_buffers, int64_t N, int K,
                                                            int group_shift, void* __restrict__ out, int64_t ldo) {
    constexpr int VPI = 32 / BITS;
    const int words = K / VPI, groups = K >> group_shift;
    const int w0 = (int)(blockIdx.x * 1024 + threadIdx.x);
    for (int64_t row = blockIdx.y; row < N; row += gridDim.y) {
        uint32_t w[4];
        float s[4], z[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int wc = w0 + 256 * j;
            if (wc < words) {
                w[j] = qweight[row * words + wc];
                const int64_t gi = row * groups + ((wc * VPI) >> group_shift);
                if (module_buffers) {
                    s[j] = (float)((const _Float16*)scale)[gi];
                    z[j] = (float)((const _Float16*)zp)[gi];
                } else {
                    s[j] = ((const float*)scale)[gi];
                    z[j] = (float)((const int32_t*)zp)[gi];
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int wc = w0 + 256 * j;
            if (wc >= words) break;
            float r[VPI];
#pragma unroll
            for (int i = 0; i < VPI; i++) {
                const float q = (float)((w[j] >> (i * BITS)) & ((1u << BITS) - 1));
                r[i] = __fmul_rn(s[j], __fsub_rn(q, z[j]));                        // functional.py:70, modules.py:55
                asm volatile("" : "+v"(r[i]));                                     // see dequantize_kernel
            }
            const int64_t o = row * ldo + (int64_t)wc * VPI;
            if constexpr (ODT == BW_F32) {
                float* p = (float*)out + o;
#pragma unroll
                for (int i = 0; i < VPI; i += 4) *reinterpret_cast<f4*>(p + i) = f4{r[i], r[i + 1], r[i + 2], r[i + 3]};
            } else {
                uint32_t d[VPI / 2];
#pragma unroll
                for (int i = 0; i < VPI / 2; i++) {
                    const uint16_t lo = ODT == BW_F16 ? __builtin_bit_cast(uint16_t, (_Float16)r[2 * i]) : f32_to_bf16(r[2 * i]);
                    const uint16_t hi = ODT == BW_F16 ? __builtin_bit_cast(uint16_t, (_Float16)r[2 * i + 1]) : f32_to_bf16(r[2 * i + 1]);
                    d[i] = (uint32_t)lo | ((uint32_t)hi << 16);
                }
                uint16_t* p = (uint16_t*)out + o;
                if constexpr (VPI == 4) {
                    *reinterpret_cast<u2*>(p) = u2{d[0], d[1]};
                } else {
#pragma unroll
                    for (int i = 0; i < VPI / 2; i += 4) *reinterpret_cast<u4*>(p + 2 * i) = u4{d[i], d[i + 1], d[i + 2], d[i + 3]};
                }
            }
        }
    }
}

// Can a launch with WPT words per thread take this shape?  Vector loads / stores need their alignment, the
// threads of a group must be a power of two inside one wave.
template <int BITS, int WDT, int WPT>
bool quantize_fits(const void* w, const void* delta, int64_t K, int64_t ldw, int64_t ldd, int group, const void* qweight) {
    constexpr int VPT = 32 / BITS * WPT;
    constexpr size_t esz = WDT == BW_F32 ? 4 : 2;
    constexpr size_t need = (VPT * esz >= 16) ? 16 : VPT * esz;
    const int lpg = group / VPT;
    return group % VPT == 0 && K % VPT == 0 && lpg >= 1 && lpg <= 64 && (lpg & (lpg - 1)) == 0 && bw_aligned(w, need) &&
           (ldw * esz) % need == 0 && bw_aligned(qweight, 4 * WPT) &&
           (!delta || (bw_aligned(delta, need) && (ldd * esz) % need == 0));
}

template <int BITS, int WDT, int MATH, int WPT>
int launch_quantize(const void* w, const void* delta, int64_t N, int64_t K, int64_t ldw, int64_t ldd, int group,
                    int32_t* qweight, void* scale, int sdt, void* zp, int zdt, int recip, hipStream_t st) {
    constexpr int VPT = 32 / BITS * WPT;
    const int tpr = (int)(K / VPT);
    const int block = tpr >= 256 ? 256 : ((tpr + 63) / 64) * 64;
    dim3 grid((unsigned)((tpr + block - 1) / block), (unsigned)(N < 65535 ? N : 65535));
    hipLaunchKernelGGL((quantize_pack_kernel<BITS, WDT, MATH, WPT>), grid, dim3(block), 0, st, w, delta, N, (int)K, ldw, ldd,
                       group, group / VPT, qweight, scale, sdt, zp, zdt, recip);
    return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
}

template <int BITS, int WDT, int MATH>
int launch_quantize_bits(const void* w, const void* delta, int64_t N, int64_t K, int64_t ldw, int64_t ldd, int group,
                         int32_t* qweight, void* scale, int sdt, void* zp, int zdt, int recip, hipStream_t st) {
    // 64 bytes of 16-bit input per thread (32 weights) where the shape allows - everything a thread does once per
    // group share (extrema exchange, the two divisions of the group's parameters, addressing, the stores) then costs
    // half as much per weight as with 32 bytes, and the kernel is bound by arithmetic, not memory: 28.6 -> see the
    // benchmark - else 32 bytes, else one word per thread, else the generic kernel
    constexpr int VPI = 32 / BITS;
    constexpr int WIDE = (WDT == BW_F32 ? 8 : 16) / VPI;
    if constexpr (WDT != BW_F32) {
        constexpr int WIDER = 32 / VPI;
        if (quantize_fits<BITS, WDT, WIDER>(w, delta, K, ldw, ldd, group, qweight))
            return launch_quantize<BITS, WDT, MATH, WIDER>(w, delta, N, K, ldw, ldd, group, qweight, scale, sdt, zp, zdt, recip, st);
    }
    if constexpr (WIDE > 1) {
        if (quantize_fits<BITS, WDT, WIDE>(w, delta, K, ldw, ldd, group, qweight))
            return launch_quantize<BITS, WDT, MATH, WIDE>(w, delta, N, K, ldw, ldd, group, qweight, scale, sdt, zp, zdt, recip, st);
    }
    if (quantize_fits<BITS, WDT, 1>(w, delta, K, ldw, ldd, group, qweight))
        return launch_quantize<BITS, WDT, MATH, 1>(w, delta, N, K, ldw, ldd, group, qweight, scale, sdt, zp, zdt, recip, st);
    const int64_t total = N * (K / VPI);
    hipLaunchKernelGGL((quantize_pack_generic_kernel<WDT, MATH>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, w,
                       delta, N, (int)K, ldw, ldd, BITS, group, qweight, scale, sdt, zp, zdt, recip);
    return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
}

template <int WDT, int MATH>
int dispatch_bits(int bits, const void* w, const void* delta, int64_t N, int64_t K, int64_t ldw, int64_t ldd, int group,
                  int32_t* qweight, void* scale, int sdt, void* zp, int zdt, int recip, hipStream_t st) {
    if (bits == 2) return launch_quantize_bits<2, WDT, MATH>(w, delta, N, K, ldw, ldd, group, qweight, scale, sdt, zp, zdt, recip, st);
    if (bits == 4) return launch_quantize_bits<4, WDT, MATH>(w, delta, N, K, ldw, ldd, group, qweight, scale, sdt, zp, zdt, recip, st);
    return launch_quantize_bits<8, WDT, MATH>(w, delta, N, K, ldw, ldd, group, qweight, scale, sdt, zp, zdt, recip, st);
}

}  // namespace

extern "C" int bw_quantize_pack_add(const void* w, const void* delta, int w_dtype, int math_dtype, int64_t N, int64_t K,
                                    int64_t ldw, int64_t ldd, int bits, int group, int32_t* qweight, void* scale,
                                    int scale_dtype, void* zp, int zp_dtype, void* stream) {
    if (!w || !qweight || !scale || !zp) return BW_EINVAL;
    const int recip = (math_dtype & BW_SCALE_RECIPROCAL) != 0;
    math_dtype &= ~BW_SCALE_RECIPROCAL;
    if (!bw_shape_ok(N, K, bits, group) || ldw < K || (delta && ldd < K)) return BW_EINVAL;
    if (w_dtype == BW_F64) {
        // float64 in, float64 arithmetic, float64 scale, int32 zero point: what the reference returns for such a tensor
        if (math_dtype != BW_F64 || scale_dtype != BW_F64 || zp_dtype != BW_I32) return BW_EINVAL;
        if (!bw_aligned(w, 8) || !bw_aligned(qweight, 4) || !bw_aligned(scale, 8) || !bw_aligned(zp, 4) || (delta && !bw_aligned(delta, 8)))
            return BW_EALIGN;
        const int64_t total = N * (K / (32 / bits));
        hipLaunchKernelGGL(quantize_pack_f64_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                           (const double*)w, (const double*)delta, N, (int)K, ldw, ldd, bits, group, qweight, (double*)scale,
                           (int32_t*)zp, recip);
        return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
    }
    if (w_dtype != BW_F16 && w_dtype != BW_BF16 && w_dtype != BW_F32) return BW_EINVAL;
    if (scale_dtype != BW_F32 && scale_dtype != BW_F16 && scale_dtype != BW_BF16) return BW_EINVAL;
    if (zp_dtype != BW_I32 && zp_dtype != BW_F16 && zp_dtype != BW_BF16) return BW_EINVAL;
    // math in a 16-bit type only makes sense on weights of that type (eager torch never mixes them)
    if (math_dtype != BW_F32 && math_dtype != w_dtype) return BW_EINVAL;
    // every element needs its natural alignment; the kernels pick their own vector widths
    const size_t esz = w_dtype == BW_F32 ? 4 : 2;
    if (!bw_aligned(w, esz) || !bw_aligned(qweight, 4) || (delta && !bw_aligned(delta, esz))) return BW_EALIGN;
    hipStream_t st = (hipStream_t)stream;
#define BW_Q(WD, MD) \
    if (w_dtype == WD && math_dtype == MD) \
        return dispatch_bits<WD, MD>(bits, w, delta, N, K, ldw, ldd, group, qweight, scale, scale_dtype, zp, zp_dtype, recip, st);
    BW_Q(BW_F32, BW_F32) BW_Q(BW_F16, BW_F32) BW_Q(BW_BF16, BW_F32) BW_Q(BW_F16, BW_F16) BW_Q(BW_BF16, BW_BF16)
#undef BW_Q
    return BW_EINVAL;
}

extern "C" int bw_quantize_pack(const void* w, int w_dtype, int math_dtype, int64_t N, int64_t K, int64_t ldw, int bits,
                                int group, int32_t* qweight, void* scale, int scale_dtype, void* zp, int zp_dtype,
                                void* stream) {
    return bw_quantize_pack_add(w, nullptr, w_dtype, math_dtype, N, K, ldw, 0, bits, group, qweight, scale, scale_dtype, zp,
                                zp_dtype, stream);
}

extern "C" int bw_dequantize(const int32_t* qweight, const void* scale, int scale_dtype, const void* zp, int zp_dtype,
                             int64_t N, int64_t K, int bits, int group, void* w_out, int out_dtype, int64_t ldo,
                             void* stream) {
    if (!qweight || !scale || !zp || !w_out) return BW_EINVAL;
    if (!bw_shape_ok(N, K, bits, group) || ldo < K) return BW_EINVAL;
    if (scale_dtype == BW_F64 || out_dtype == BW_F64) {
        if (scale_dtype != BW_F64 || out_dtype != BW_F64 || (zp_dtype != BW_I32 && zp_dtype != BW_F16)) return BW_EINVAL;
        if (!bw_aligned(scale, 8) || !bw_aligned(w_out, 8)) return BW_EALIGN;
        const int64_t total = N * (K / (32 / bits));
        hipLaunchKernelGGL(dequantize_f64_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                           (const uint32_t*)qweight, (const double*)scale, zp, zp_dtype, N, (int)K, bits, group, (double*)w_out, ldo);
        return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
    }
    if (scale_dtype != BW_F32 && scale_dtype != BW_F16) return BW_EINVAL;
    if (zp_dtype != BW_I32 && zp_dtype != BW_F16) return BW_EINVAL;
    if (out_dtype != BW_F32 && out_dtype != BW_F16 && out_dtype != BW_BF16) return BW_EINVAL;
    const int vpi = 32 / bits;
    const int64_t words = K / vpi;
    const size_t esz = out_dtype == BW_F32 ? 4 : 2;
    const bool vec = bw_aligned(w_out, 16) && (ldo * esz) % 16 == 0;
    hipStream_t st = (hipStream_t)stream;
    const bool module_buffers = scale_dtype == BW_F16 && zp_dtype == BW_F16, returned = scale_dtype == BW_F32 && zp_dtype == BW_I32;
    if (vec && (module_buffers || returned) && words >= 512 && (group & (group - 1)) == 0 && group >= vpi) {
        int shift = 0;
        while ((1 << shift) < group) shift++;
        const int bsz = 256;
        dim3 g4((unsigned)((words + 1023) / 1024), (unsigned)(N < 65535 ? N : 65535));
#define BW_D4(B, OD)                                                                                                    \
    if (bits == B && out_dtype == OD) {                                                                                 \
        hipLaunchKernelGGL((dequantize_x4_kernel<B, OD>), g4, dim3(bsz), 0, st, (const uint32_t*)qweight, scale, zp,    \
                           (int)module_buffers, N, (int)K, shift, w_out, ldo);                                          \
        return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;                                                    \
    }
        BW_D4(2, BW_F32) BW_D4(4, BW_F32) BW_D4(8, BW_F32) BW_D4(2, BW_F16) BW_D4(4, BW_F16) BW_D4(8, BW_F16)
        BW_D4(2, BW_BF16) BW_D4(4, BW_BF16) BW_D4(8, BW_BF16)
#undef BW_D4
    }
    dim3 grid((unsigned)((words + 255) / 256), (unsigned)(N < 65535 ? N : 65535)), block(256);
#define BW_D(B, OD)                                                                                                     \
    if (bits == B && out_dtype == OD) {                                                                                 \
        if (vec)                                                                                                        \
            hipLaunchKernelGGL((dequantize_kernel<B, OD, true>), grid, block, 0, st, (const uint32_t*)qweight, scale,   \
                               scale_dtype, zp, zp_dtype, N, (int)K, group, w_out, ldo);                                \
        else                                                                                                            \
            hipLaunchKernelGGL((dequantize_kernel<B, OD, false>), grid, block, 0, st, (const uint32_t*)qweight, scale,  \
                               scale_dtype, zp, zp_dtype, N, (int)K, group, w_out, ldo);                                \
        return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;                                                    \
    }
    BW_D(2, BW_F32) BW_D(4, BW_F32) BW_D(8, BW_F32) BW_D(2, BW_F16) BW_D(4, BW_F16) BW_D(8, BW_F16)
    BW_D(2, BW_BF16) BW_D(4, BW_BF16) BW_D(8, BW_BF16)
#undef BW_D
    return BW_EINVAL;
}

extern "C" int bw_abi_version(void) { return 10; }

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
