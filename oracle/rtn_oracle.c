/* Scalar C restatement of Bitween's quantized-linear hot path.
 *
 * TEST INFRASTRUCTURE ONLY: the checker the HIP kernels are compared with and
 * the CPU baseline that bench.py times.  Nothing in the shipped library links
 * or loads this file.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off -fno-fast-math, so
 * every float operation below is one correctly rounded IEEE-754 binary32
 * operation, as in eager torch on CPU).
 *
 * Reference lines restated (paths relative to the reference checkout):
 *   orc_quantize_rtn_f32   bitween/functional.py:3-45
 *   orc_dequantize_f32     bitween/functional.py:47-71
 *   orc_dequantize_f16     bitween/modules.py:10-58
 *   orc_qlinear_forward    bitween/modules.py:62-106, main.py:444-466
 * Pinned by tests/test_oracle_pins.py (exact-rational evaluation, hand-derived
 * known answers, agreement with the independent numpy restatement).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* binary32 -> binary16 bits, round to nearest even, subnormals kept. */
static uint16_t f32_to_f16_bits(float f) {
    uint32_t x; memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u, mant = x & 0x7FFFFFu;
    int32_t exp = (int32_t)((x >> 23) & 0xFF);
    if (exp == 0xFF) return (uint16_t)(sign | 0x7C00u | (mant ? 0x200u : 0));
    int32_t e = exp - 127 + 15;
    if (e >= 0x1F) return (uint16_t)(sign | 0x7C00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        mant |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t half = mant >> shift, rem = mant & ((1u << shift) - 1), mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1))) half++;
        return (uint16_t)(sign | half);
    }
    uint32_t half = ((uint32_t)e << 10) | (mant >> 13), rem = mant & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1))) half++;
    return (uint16_t)(sign | half);
}

static float f16_bits_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16, exp = (h >> 10) & 0x1F, mant = h & 0x3FFu, x;
    if (exp == 0) {
        if (!mant) x = sign;
        else { int e = -1; do { e++; mant <<= 1; } while (!(mant & 0x400u)); x = sign | ((uint32_t)(127 - 15 - e) << 23) | ((mant & 0x3FFu) << 13); }
    } else if (exp == 0x1F) x = sign | 0x7F800000u | (mant << 13);
    else x = sign | ((exp - 15 + 127) << 23) | (mant << 13);
    float f; memcpy(&f, &x, 4); return f;
}

uint16_t orc_f32_to_f16(float f) { return f32_to_f16_bits(f); }
float orc_f16_to_f32(uint16_t h) { return f16_bits_to_f32(h); }

/* w [n][k] float32 -> qweight int32 [n][k*bits/32], scale f32 [n][k/g],
 * zero_point int32 [n][k/g].  Returns 0, or -1 for bad arguments. */
int orc_quantize_rtn_f32_div(const float* w, int64_t n, int64_t k, int bits, int g, int reciprocal,
                             int32_t* qweight, float* scale, int32_t* zero_point);
int orc_quantize_rtn_f32(const float* w, int64_t n, int64_t k, int bits, int g,
                         int32_t* qweight, float* scale, int32_t* zero_point) {
    return orc_quantize_rtn_f32_div(w, n, k, bits, g, 0, qweight, scale, zero_point);
}

/* reciprocal != 0: the scale as eager torch forms it on a GPU, (hi - lo) * (1.0f / qmax); else the true
 * division of the CPU path. */
int orc_quantize_rtn_f32_div(const float* w, int64_t n, int64_t k, int bits, int g, int reciprocal,
                             int32_t* qweight, float* scale, int32_t* zero_point) {
    if (!(bits == 2 || bits == 4 || bits == 8) || g < 1 || k % g || k % (32 / bits)) return -1;
    const float qmax = (float)((1 << bits) - 1);
    const int vpi = 32 / bits;
    const int64_t groups = k / g, words = k / vpi;
    memset(qweight, 0, (size_t)(n * words) * sizeof(int32_t));
    #pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < n; r++) {
        uint32_t* qrow = (uint32_t*)(qweight + r * words);
        for (int64_t gi = 0; gi < groups; gi++) {
            const float* p = w + r * k + gi * g;
            float lo = p[0], hi = p[0];
            for (int i = 1; i < g; i++) { if (p[i] < lo) lo = p[i]; if (p[i] > hi) hi = p[i]; }
            const float range = hi - lo;
            float s = reciprocal ? range * (1.0f / qmax) : range / qmax;   /* functional.py:25 */
            if (s < 1e-8f) s = 1e-8f;
            float zf = clampf(rintf(-lo / s), 0.0f, qmax); /* functional.py:26 */
            scale[r * groups + gi] = s;
            zero_point[r * groups + gi] = (int32_t)zf;
            for (int i = 0; i < g; i++) {
                float t = p[i] / s;                        /* functional.py:29: divide, */
                t = t + zf;                                /* then a separate add      */
                uint32_t q = (uint32_t)(int32_t)clampf(rintf(t), 0.0f, qmax);
                int64_t col = gi * g + i;
                qrow[col / vpi] |= q << ((col % vpi) * bits);   /* functional.py:35-40 */
            }
        }
    }
    return 0;
}

/* scale/zero_point given as float32 arrays (callers widen f16 / int32 first). */
int orc_dequantize_f32(const int32_t* qweight, const float* scale, const float* zp, int64_t n, int64_t k,
                       int bits, int g, float* w) {
    if (!(bits == 2 || bits == 4 || bits == 8) || g < 1 || k % g || k % (32 / bits)) return -1;
    const int vpi = 32 / bits; const uint32_t mask = (1u << bits) - 1; const int64_t groups = k / g, words = k / vpi;
    #pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < n; r++)
        for (int64_t c = 0; c < k; c++) {
            uint32_t word = (uint32_t)qweight[r * words + c / vpi];
            float q = (float)((word >> ((c % vpi) * bits)) & mask);
            w[r * k + c] = scale[r * groups + c / g] * (q - zp[r * groups + c / g]);   /* functional.py:70 */
        }
    return 0;
}

int orc_dequantize_f16(const int32_t* qweight, const uint16_t* scale16, const uint16_t* zp16, int64_t n, int64_t k,
                       int bits, int g, uint16_t* w16) {
    if (!(bits == 2 || bits == 4 || bits == 8) || g < 1 || k % g || k % (32 / bits)) return -1;
    const int vpi = 32 / bits; const uint32_t mask = (1u << bits) - 1; const int64_t groups = k / g, words = k / vpi;
    #pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < n; r++)
        for (int64_t c = 0; c < k; c++) {
            uint32_t word = (uint32_t)qweight[r * words + c / vpi];
            float q = (float)((word >> ((c % vpi) * bits)) & mask);
            float s = f16_bits_to_f32(scale16[r * groups + c / g]), z = f16_bits_to_f32(zp16[r * groups + c / g]);
            w16[r * k + c] = f32_to_f16_bits(s * (q - z));                              /* modules.py:55-58 */
        }
    return 0;
}

/* y16[m][n] = f16( sum_k x16[m][k] * W16[n][k] ) (+ bias16, a second f16 rounding).
 * Accumulates in double; W16 is dequantized row by row, never stored whole. */
int orc_qlinear_forward(const uint16_t* x16, int64_t m, int64_t k, const int32_t* qweight, const uint16_t* scale16,
                        const uint16_t* zp16, const uint16_t* bias16, int64_t n, int bits, int g, uint16_t* y16) {
    if (!(bits == 2 || bits == 4 || bits == 8) || g < 1 || k % g || k % (32 / bits)) return -1;
    const int vpi = 32 / bits; const uint32_t mask = (1u << bits) - 1; const int64_t groups = k / g, words = k / vpi;
    float* xf = (float*)malloc((size_t)(m * k) * sizeof(float));
    if (!xf) return -2;
    for (int64_t i = 0; i < m * k; i++) xf[i] = f16_bits_to_f32(x16[i]);
    #pragma omp parallel
    {
        float* wrow = (float*)malloc((size_t)k * sizeof(float));
        #pragma omp for schedule(static)
        for (int64_t r = 0; r < n; r++) {
            for (int64_t c = 0; c < k; c++) {
                uint32_t word = (uint32_t)qweight[r * words + c / vpi];
                float q = (float)((word >> ((c % vpi) * bits)) & mask);
                float s = f16_bits_to_f32(scale16[r * groups + c / g]), z = f16_bits_to_f32(zp16[r * groups + c / g]);
                wrow[c] = f16_bits_to_f32(f32_to_f16_bits(s * (q - z)));
            }
            for (int64_t i = 0; i < m; i++) {
                double acc = 0.0;
                for (int64_t c = 0; c < k; c++) acc += (double)xf[i * k + c] * (double)wrow[c];
                uint16_t y = f32_to_f16_bits((float)acc);
                if (bias16) y = f32_to_f16_bits(f16_bits_to_f32(y) + f16_bits_to_f32(bias16[r]));   /* modules.py:100-101 */
                y16[i * n + r] = y;
            }
        }
        free(wrow);
    }
    free(xf);
    return 0;
}
