// Decode path: y[M][N] = x[M][K] @ W16[N][K]^T (+ bias), 1 <= M <= 16.
//
// HBM-bound: every packed weight byte is read exactly once with 128-bit
// loads, straight into the lane that feeds it to the matrix core.
//
// Work split.  A workgroup owns 16 consecutive output rows (one MFMA column
// tile) and the whole K extent; its waves split K.  The unit of work is a
// "chunk": 64 bytes of every one of the 16 rows (512/BITS weights per row).
// Lane l of a wave loads 16 bytes of row (l & 15) at byte 16*(l >> 4) of the
// chunk - exactly the B-operand layout of v_mfma_f32_16x16x32_f16 (column
// l & 15, k-group l >> 4), so no shuffle or LDS hop is needed for weights.
// The lane unpacks its nibbles/crumbs in registers to the same float16 values
// the reference's dequantize kernel would store (bitween/modules.py:55-58)
// and issues MFMAs against the activations, which the workgroup staged once
// in LDS in the k order the unpack emits.  M < 16 leaves MFMA rows idle,
// which costs nothing here: the matrix pipe has >5x headroom at HBM speed.
//
// Partial sums of the waves are reduced through LDS; the epilogue adds the
// bias in float32 and rounds once.
#include "bw_common.h"

namespace {

constexpr int kXBudgetBytes = 48 * 1024;   // LDS for the staged activations
constexpr int kBatch = 4;                  // chunks a wave keeps in flight

template <int BITS, int GROUP>
struct GemvCfg {
    static constexpr int VPI = 32 / BITS;            // values per int32 word
    static constexpr int VPL = 128 / BITS;           // values per 16-byte lane load
    static constexpr int CHUNK_K = 4 * VPL;          // k extent of one chunk
    static constexpr int MF = VPL / 8;               // MFMAs per lane load
    static constexpr int NG = (VPL > GROUP) ? VPL / GROUP : 1;   // groups per lane load
    static_assert(GROUP % VPI == 0, "a packed word must not straddle groups");
};

// Stage x[0:M][k0:k0+kn] (zero beyond K) into LDS, permuted inside every block
// of VPI values into the order dequant_word* emits them.  16 values per thread
// step, so the global reads are two 128-bit loads.
template <int BITS>
BW_DEV void stage_x(const _Float16* __restrict__ x, int M, int K, int64_t ldx, int k0, int kn, _Float16* xs, int pitch,
                    int tid, int nthreads) {
    const int blocks_per_row = kn / 16;
    for (int i = tid; i < M * blocks_per_row; i += nthreads) {
        const int m = i / blocks_per_row, kb = (i - m * blocks_per_row) * 16;
        uint32_t r[8];
        if (k0 + kb < K) {   // K % 16 == 0, so a block is entirely in or out
            const u4* src = reinterpret_cast<const u4*>(x + (int64_t)m * ldx + k0 + kb);
            u4 lo = src[0], hi = src[1];
            r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
            r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) r[j] = 0;
        }
        uint32_t o[8];
        if constexpr (BITS == 8) {
#pragma unroll
            for (int j = 0; j < 8; j++) o[j] = r[j];
        } else if constexpr (BITS == 4) {
            // block of 8 halves in r[0..3]: (h0,h4)(h1,h5)(h2,h6)(h3,h7)
#pragma unroll
            for (int b = 0; b < 2; b++) {
                o[4 * b + 0] = __builtin_amdgcn_perm(r[4 * b + 2], r[4 * b + 0], 0x05040100u);
                o[4 * b + 1] = __builtin_amdgcn_perm(r[4 * b + 2], r[4 * b + 0], 0x07060302u);
                o[4 * b + 2] = __builtin_amdgcn_perm(r[4 * b + 3], r[4 * b + 1], 0x05040100u);
                o[4 * b + 3] = __builtin_amdgcn_perm(r[4 * b + 3], r[4 * b + 1], 0x07060302u);
            }
        } else {
            // block of 16 halves: (h_j, h_{j+8}) for j = 0..7
#pragma unroll
            for (int j = 0; j < 8; j++)
                o[j] = __builtin_amdgcn_perm(r[4 + j / 2], r[j / 2], (j & 1) ? 0x07060302u : 0x05040100u);
        }
        u4* dst = reinterpret_cast<u4*>(xs + m * pitch + kb);
        dst[0] = u4{o[0], o[1], o[2], o[3]};
        dst[1] = u4{o[4], o[5], o[6], o[7]};
    }
}

template <int BITS, int GROUP, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void qgemv_kernel(
    const _Float16* __restrict__ x, int M, int K, int64_t ldx, const uint32_t* __restrict__ qweight,
    const _Float16* __restrict__ scale, const _Float16* __restrict__ zp, const _Float16* __restrict__ bias, int N,
    _Float16* __restrict__ y, int64_t ldy, int slice_chunks) {
    using C = GemvCfg<BITS, GROUP>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nl = lane & 15, kq = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int row = min(n0 + nl, N - 1);                 // clamp: out-of-range rows are computed and dropped
    const int row_bytes = K * BITS / 8, groups = K / GROUP;
    const int nchunks = (K + C::CHUNK_K - 1) / C::CHUNK_K;
    const int pitch = slice_chunks * C::CHUNK_K + 8;      // +8 halves: rows land on different LDS banks
    _Float16* xs = reinterpret_cast<_Float16*>(smem);
    float* red = reinterpret_cast<float*>(smem + (size_t)M * pitch * 2);   // rows >= M are never read

    const char* wrow = reinterpret_cast<const char*>(qweight) + (int64_t)row * row_bytes;
    const _Float16* srow = scale + (int64_t)row * groups;
    const _Float16* zrow = zp + (int64_t)row * groups;

    f4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < nchunks; s0 += slice_chunks) {
        const int s_chunks = min(slice_chunks, nchunks - s0);
        if (s0) __syncthreads();
        stage_x<BITS>(x, M, K, ldx, s0 * C::CHUNK_K, s_chunks * C::CHUNK_K, xs, pitch, tid, WAVES * 64);
        __syncthreads();
        for (int c0 = wave * kBatch; c0 < s_chunks; c0 += WAVES * kBatch) {
            u4 wreg[kBatch];
            _Float16 sv[kBatch][C::NG], zv[kBatch][C::NG];
#pragma unroll
            for (int b = 0; b < kBatch; b++) {
                const int chunk = s0 + c0 + b;
                int kbyte = chunk * 64 + kq * 16;
                const bool ok = (c0 + b < s_chunks) && kbyte < row_bytes;
                kbyte = ok ? kbyte : 0;                   // masked lanes re-read byte 0; their x is zero
                wreg[b] = __builtin_nontemporal_load(reinterpret_cast<const u4*>(wrow + kbyte));
                const int g0 = (kbyte * 8 / BITS) / GROUP;
#pragma unroll
                for (int g = 0; g < C::NG; g++) { sv[b][g] = srow[g0 + g]; zv[b][g] = zrow[g0 + g]; }
            }
#pragma unroll
            for (int b = 0; b < kBatch; b++) {
                if (c0 + b >= s_chunks) break;            // wave-uniform
                GroupConst<BITS> gc[C::NG];
#pragma unroll
                for (int g = 0; g < C::NG; g++) gc[g].set(sv[b][g], zv[b][g]);
                h2 wp[C::VPL / 2];
                dequant_lane16<BITS, C::NG>(wreg[b], gc, wp);
                const _Float16* xp = xs + nl * pitch + (c0 + b) * C::CHUNK_K + kq * C::VPL;
#pragma unroll
                for (int t = 0; t < C::MF; t++) {
                    h8 a = {0, 0, 0, 0, 0, 0, 0, 0};
                    if (nl < M) a = *reinterpret_cast<const h8*>(xp + 8 * t);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, pack_h8(wp + 4 * t), acc, 0, 0, 0);
                }
            }
        }
    }
    // acc[r] = partial y[m = 4*kq + r][n = nl]
#pragma unroll
    for (int r = 0; r < 4; r++) red[(wave * 16 + 4 * kq + r) * 16 + nl] = acc[r];
    __syncthreads();
    if (tid < 256) {
        const int m = tid >> 4, n = n0 + (tid & 15);
        if (m < M && n < N) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; w++) v += red[(w * 16 + m) * 16 + (tid & 15)];
            if (bias) v += (float)bias[n];
            y[(int64_t)m * ldy + n] = (_Float16)v;
        }
    }
}

template <int BITS, int GROUP>
int launch_gemv(const void* x, int64_t M, int64_t K, int64_t ldx, const int32_t* qweight, const void* scale,
                const void* zp, const void* bias, int64_t N, void* y, int64_t ldy, hipStream_t stream) {
    using C = GemvCfg<BITS, GROUP>;
    constexpr int WAVES = 8;
    const int nchunks = (int)((K + C::CHUNK_K - 1) / C::CHUNK_K);
    // chunks per LDS slice: M rows of (slice + 8) halves must fit the budget
    int slice_chunks = (kXBudgetBytes / ((int)M * 2) - 8) / C::CHUNK_K;
    if (slice_chunks < 1) slice_chunks = 1;
    if (slice_chunks > nchunks) slice_chunks = nchunks;
    const size_t lds = (size_t)M * (slice_chunks * C::CHUNK_K + 8) * 2 + (size_t)WAVES * 256 * 4;
    dim3 grid((unsigned)((N + 15) / 16)), block(WAVES * 64);
    hipLaunchKernelGGL((qgemv_kernel<BITS, GROUP, WAVES>), grid, block, lds, stream, (const _Float16*)x, (int)M, (int)K,
                       ldx, (const uint32_t*)qweight, (const _Float16*)scale, (const _Float16*)zp,
                       (const _Float16*)bias, (int)N, (_Float16*)y, ldy, slice_chunks);
    return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
}

}  // namespace

// Shapes the MFMA path takes: 16-byte lane loads need K*bits/8 % 16 == 0 and
// group in {32, 64, 128}.
bool bw_fast_shape(int64_t K, int bits, int group) {
    return (group == 32 || group == 64 || group == 128) && (K * bits / 8) % 16 == 0 && K % 16 == 0;
}

int bw_qgemm_generic(const void* x, int act_dtype, int64_t M, int64_t K, int64_t ldx, const int32_t* qweight,
                     const void* scale16, const void* zp16, const void* bias, int64_t N, int bits, int group, void* y,
                     int64_t ldy, void* stream);

extern "C" int bw_qgemv(const void* x, int act_dtype, int64_t M, int64_t K, int64_t ldx, const int32_t* qweight,
                        const void* scale16, const void* zp16, const void* bias, int64_t N, int bits, int group,
                        void* y, int64_t ldy, void* stream) {
    if (!x || !qweight || !scale16 || !zp16 || !y) return BW_EINVAL;
    if (!bw_shape_ok(N, K, bits, group) || M < 1 || M > 16 || ldx < K || ldy < N) return BW_EINVAL;
    if (act_dtype != BW_F16) return BW_EUNSUPPORTED;
    if (!bw_fast_shape(K, bits, group) || !bw_aligned(x, 16) || (ldx * 2) % 16 || !bw_aligned(qweight, 16))
        return bw_qgemm_generic(x, act_dtype, M, K, ldx, qweight, scale16, zp16, bias, N, bits, group, y, ldy, stream);
    hipStream_t st = (hipStream_t)stream;
#define BW_CASE(B, G) \
    if (bits == B && group == G) return launch_gemv<B, G>(x, M, K, ldx, qweight, scale16, zp16, bias, N, y, ldy, st);
    BW_CASE(4, 128) BW_CASE(4, 64) BW_CASE(4, 32)
    BW_CASE(8, 128) BW_CASE(8, 64) BW_CASE(8, 32)
    BW_CASE(2, 128) BW_CASE(2, 64) BW_CASE(2, 32)
#undef BW_CASE
    return BW_EUNSUPPORTED;
}
