// Prefill path: y[M][N] = x[M][K] @ W16[N][K]^T (+ bias) for any M, built for
// M >= 128 where the matrix cores are the bound.
//
// A workgroup of 4 waves owns a 128 (M) x 256 (N) output tile; each wave owns
// 128 x 64 of it (8 x 4 MFMA 16x16 tiles, 128 accumulator registers).  Per K
// step of one chunk (64 packed bytes per weight row):
//   * weights go global -> registers with one 128-bit load per lane per 16
//     rows, already in MFMA B-operand layout, and are unpacked in registers
//     to the float16 values the reference's dequantize kernel would store
//     (bitween/modules.py:55-58).  No wave unpacks a weight another wave of
//     the workgroup also unpacks; each weight is unpacked M/128 times overall.
//   * activations go global -> LDS once per workgroup (double buffered,
//     permuted into the k order the unpack emits) and every A fragment read
//     from LDS feeds 4 MFMAs.
// Also holds the shape-generic fallback used when the fast layouts do not
// apply (odd K or group size): correct for everything the reference accepts.
#include "bw_common.h"

bool bw_fast_shape(int64_t M, int64_t N, int64_t K, int64_t ldx, int bits, int group);

namespace {

constexpr int BM = 128, WAVES = 4, NT = 4, MT = BM / 16, BN = WAVES * NT * 16;

template <int BITS, int GROUP>
struct GemmCfg {
    static constexpr int VPL = 128 / BITS, CHUNK_K = 4 * VPL, MF = VPL / 8;
    static constexpr int NG = (VPL > GROUP) ? VPL / GROUP : 1;
    static constexpr int PITCH = CHUNK_K + 8;                 // halves per LDS row
    static constexpr int STAGE_BYTES = BM * PITCH * 2;
};

template <int BITS>
BW_DEV void permute16(const uint32_t* r, uint32_t* o) {
    if constexpr (BITS == 8) {
#pragma unroll
        for (int j = 0; j < 8; j++) o[j] = r[j];
    } else if constexpr (BITS == 4) {
#pragma unroll
        for (int b = 0; b < 2; b++) {
            o[4 * b + 0] = __builtin_amdgcn_perm(r[4 * b + 2], r[4 * b + 0], 0x05040100u);
            o[4 * b + 1] = __builtin_amdgcn_perm(r[4 * b + 2], r[4 * b + 0], 0x07060302u);
            o[4 * b + 2] = __builtin_amdgcn_perm(r[4 * b + 3], r[4 * b + 1], 0x05040100u);
            o[4 * b + 3] = __builtin_amdgcn_perm(r[4 * b + 3], r[4 * b + 1], 0x07060302u);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++)
            o[j] = __builtin_amdgcn_perm(r[4 + j / 2], r[j / 2], (j & 1) ? 0x07060302u : 0x05040100u);
    }
}

template <int BITS, int GROUP>
__global__ __launch_bounds__(WAVES * 64) void qgemm_kernel(
    const _Float16* __restrict__ x, int M, int K, int64_t ldx, const uint32_t* __restrict__ qweight,
    const _Float16* __restrict__ scale, const _Float16* __restrict__ zp, const _Float16* __restrict__ bias, int N,
    _Float16* __restrict__ y, int64_t ldy) {
    using C = GemmCfg<BITS, GROUP>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nl = lane & 15, kq = lane >> 4;
    const int m0 = blockIdx.y * BM;
    const int n0 = blockIdx.x * BN + wave * (NT * 16);
    const int row_bytes = K * BITS / 8, groups = K / GROUP;
    const int nchunks = (K + C::CHUNK_K - 1) / C::CHUNK_K;

    const char* wrow[NT];
    const _Float16 *srow[NT], *zrow[NT];
#pragma unroll
    for (int j = 0; j < NT; j++) {
        const int row = min(n0 + 16 * j + nl, N - 1);
        wrow[j] = reinterpret_cast<const char*>(qweight) + (int64_t)row * row_bytes;
        srow[j] = scale + (int64_t)row * groups;
        zrow[j] = zp + (int64_t)row * groups;
    }

    // x tile staging: 16 halves per thread step
    constexpr int BLK_PER_ROW = C::CHUNK_K / 16, STEPS = BM * BLK_PER_ROW / (WAVES * 64);
    static_assert(BM * BLK_PER_ROW % (WAVES * 64) == 0, "tile must split evenly over the workgroup");
    auto stage = [&](int chunk, _Float16* xs) {
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            const int i = tid + s * WAVES * 64;
            const int m = i / BLK_PER_ROW, kb = (i % BLK_PER_ROW) * 16;
            const int k = chunk * C::CHUNK_K + kb;
            uint32_t r[8], o[8];
            if (m0 + m < M && k < K) {
                const u4* src = reinterpret_cast<const u4*>(x + (int64_t)(m0 + m) * ldx + k);
                u4 lo = src[0], hi = src[1];
                r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
                r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
            } else {
#pragma unroll
                for (int j = 0; j < 8; j++) r[j] = 0;
            }
            permute16<BITS>(r, o);
            u4* dst = reinterpret_cast<u4*>(xs + m * C::PITCH + kb);
            dst[0] = u4{o[0], o[1], o[2], o[3]};
            dst[1] = u4{o[4], o[5], o[6], o[7]};
        }
    };

    u4 wreg[NT];
    _Float16 sv[NT][C::NG], zv[NT][C::NG];
    auto load_w = [&](int chunk) {
        int kbyte = chunk * 64 + kq * 16;
        kbyte = kbyte < row_bytes ? kbyte : 0;            // masked lanes: their x is staged as zero
        const int g0 = (kbyte * 8 / BITS) / GROUP;
#pragma unroll
        for (int j = 0; j < NT; j++) {
            wreg[j] = *reinterpret_cast<const u4*>(wrow[j] + kbyte);
#pragma unroll
            for (int g = 0; g < C::NG; g++) { sv[j][g] = srow[j][g0 + g]; zv[j][g] = zrow[j][g0 + g]; }
        }
    };

    f4 acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < NT; j++) acc[i][j] = f4{0.f, 0.f, 0.f, 0.f};

    _Float16* buf0 = reinterpret_cast<_Float16*>(smem);
    _Float16* buf1 = reinterpret_cast<_Float16*>(smem + C::STAGE_BYTES);
    stage(0, buf0);
    load_w(0);
    __syncthreads();
    for (int c = 0; c < nchunks; c++) {
        _Float16* cur = (c & 1) ? buf1 : buf0;
        _Float16* nxt = (c & 1) ? buf0 : buf1;
        // unpack this chunk's weights, then refill the weight registers for the next one
        h2 wp[NT][C::VPL / 2];
#pragma unroll
        for (int j = 0; j < NT; j++) {
            GroupConst<BITS> gc[C::NG];
#pragma unroll
            for (int g = 0; g < C::NG; g++) gc[g].set(sv[j][g], zv[j][g]);
            dequant_lane16<BITS, C::NG>(wreg[j], gc, wp[j]);
        }
        if (c + 1 < nchunks) { load_w(c + 1); stage(c + 1, nxt); }
        const _Float16* xp = cur + nl * C::PITCH + kq * C::VPL;
#pragma unroll
        for (int t = 0; t < C::MF; t++) {
            h8 b[NT];
#pragma unroll
            for (int j = 0; j < NT; j++) b[j] = pack_h8(wp[j] + 4 * t);
#pragma unroll
            for (int i = 0; i < MT; i++) {
                const h8 a = *reinterpret_cast<const h8*>(xp + i * 16 * C::PITCH + 8 * t);
#pragma unroll
                for (int j = 0; j < NT; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b[j], acc[i][j], 0, 0, 0);
            }
        }
        __syncthreads();
    }
    // acc[i][j][r] = y[m0 + 16 i + 4 kq + r][n0 + 16 j + nl]
#pragma unroll
    for (int j = 0; j < NT; j++) {
        const int n = n0 + 16 * j + nl;
        if (n >= N) continue;
        const float bv = bias ? (float)bias[n] : 0.f;
#pragma unroll
        for (int i = 0; i < MT; i++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int m = m0 + 16 * i + 4 * kq + r;
                if (m < M) y[(int64_t)m * ldy + n] = (_Float16)(acc[i][j][r] + bv);
            }
    }
}

template <int BITS, int GROUP>
int launch_gemm(const void* x, int64_t M, int64_t K, int64_t ldx, const int32_t* qweight, const void* scale,
                const void* zp, const void* bias, int64_t N, void* y, int64_t ldy, hipStream_t stream) {
    using C = GemmCfg<BITS, GROUP>;
    const size_t lds = 2 * (size_t)C::STAGE_BYTES;
    auto kern = qgemm_kernel<BITS, GROUP>;
    if (lds > 64 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) !=
            hipSuccess)
            return BW_ELAUNCH;
    }
    dim3 grid((unsigned)((N + BN - 1) / BN), (unsigned)((M + BM - 1) / BM)), block(WAVES * 64);
    hipLaunchKernelGGL(kern, grid, block, lds, stream, (const _Float16*)x, (int)M, (int)K, ldx, (const uint32_t*)qweight,
                       (const _Float16*)scale, (const _Float16*)zp, (const _Float16*)bias, (int)N, (_Float16*)y, ldy);
    return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
}

// Shape-generic fallback: one thread per output element, any group size and
// any K the reference accepts.  Same arithmetic: W16 = fp16(s * (q - z)) from
// the float32 product, float32 accumulation, one rounding of the result.
__global__ void qgemm_generic_kernel(const _Float16* __restrict__ x, int M, int K, int64_t ldx,
                                     const uint32_t* __restrict__ qweight, const _Float16* __restrict__ scale,
                                     const _Float16* __restrict__ zp, const _Float16* __restrict__ bias, int N, int bits,
                                     int group, _Float16* __restrict__ y, int64_t ldy) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)M * N) return;
    const int n = (int)(idx % N), m = (int)(idx / N);
    const int vpi = 32 / bits, words = K / vpi, groups = K / group;
    const uint32_t mask = (1u << bits) - 1;
    float acc = 0.f;
    for (int wi = 0; wi < words; wi++) {
        const uint32_t w = qweight[(int64_t)n * words + wi];
        for (int i = 0; i < vpi; i++) {
            const int k = wi * vpi + i;
            const float q = (float)((w >> (i * bits)) & mask);
            const float s = (float)scale[(int64_t)n * groups + k / group], z = (float)zp[(int64_t)n * groups + k / group];
            const _Float16 w16 = (_Float16)(s * (q - z));
            acc = __builtin_fmaf((float)x[(int64_t)m * ldx + k], (float)w16, acc);
        }
    }
    if (bias) acc += (float)bias[n];
    y[(int64_t)m * ldy + n] = (_Float16)acc;
}

}  // namespace

int bw_qgemm_generic(const void* x, int act_dtype, int64_t M, int64_t K, int64_t ldx, const int32_t* qweight,
                     const void* scale16, const void* zp16, const void* bias, int64_t N, int bits, int group, void* y,
                     int64_t ldy, void* stream) {
    if (act_dtype != BW_F16) return BW_EUNSUPPORTED;
    const int64_t total = M * N;
    hipLaunchKernelGGL(qgemm_generic_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const _Float16*)x, (int)M, (int)K, ldx, (const uint32_t*)qweight, (const _Float16*)scale16,
                       (const _Float16*)zp16, (const _Float16*)bias, (int)N, bits, group, (_Float16*)y, ldy);
    return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
}

extern "C" int bw_qgemm(const void* x, int act_dtype, int64_t M, int64_t K, int64_t ldx, const int32_t* qweight,
                        const void* scale16, const void* zp16, const void* bias, int64_t N, int bits, int group,
                        void* y, int64_t ldy, void* stream) {
    if (!x || !qweight || !scale16 || !zp16 || !y) return BW_EINVAL;
    if (!bw_shape_ok(N, K, bits, group) || M < 1 || M >= ((int64_t)1 << 31) || ldx < K || ldy < N) return BW_EINVAL;
    if (act_dtype != BW_F16) return BW_EUNSUPPORTED;
    if (!bw_fast_shape(M, N, K, ldx, bits, group) || !bw_aligned(x, 16) || (ldx * 2) % 16 || !bw_aligned(qweight, 16))
        return bw_qgemm_generic(x, act_dtype, M, K, ldx, qweight, scale16, zp16, bias, N, bits, group, y, ldy, stream);
    hipStream_t st = (hipStream_t)stream;
#define BW_CASE(B, G) \
    if (bits == B && group == G) return launch_gemm<B, G>(x, M, K, ldx, qweight, scale16, zp16, bias, N, y, ldy, st);
    BW_CASE(4, 128) BW_CASE(4, 64) BW_CASE(4, 32)
    BW_CASE(8, 128) BW_CASE(8, 64) BW_CASE(8, 32)
    BW_CASE(2, 128) BW_CASE(2, 64) BW_CASE(2, 32)
#undef BW_CASE
    return BW_EUNSUPPORTED;
}

extern "C" int bw_qlinear(const void* x, int act_dtype, int64_t M, int64_t K, int64_t ldx, const int32_t* qweight,
                          const void* scale16, const void* zp16, const void* bias, int64_t N, int bits, int group,
                          void* y, int64_t ldy, void* stream) {
    if (M >= 1 && M <= 16) return bw_qgemv(x, act_dtype, M, K, ldx, qweight, scale16, zp16, bias, N, bits, group, y, ldy, stream);
    return bw_qgemm(x, act_dtype, M, K, ldx, qweight, scale16, zp16, bias, N, bits, group, y, ldy, stream);
}
