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

constexpr int kWaves = 8;

template <int BITS, int GROUP, int MT>
struct GemvCfg {
    static constexpr int VPI = 32 / BITS;            // values per int32 word
    static constexpr int VPL = 128 / BITS;           // values per 16-byte lane load
    static constexpr int CHUNK_K = 4 * VPL;          // k extent of one chunk
    static constexpr int MF = VPL / 8;               // MFMAs per lane load
    static constexpr int NG = (VPL > GROUP) ? VPL / GROUP : 1;   // groups per lane load
    // chunks a wave takes per batch: its private x tile (MT rows x KB*CHUNK_K halves) stays near 16 KB
    static constexpr int KB = (8192 / (MT * CHUNK_K) >= 4) ? 4 : ((8192 / (MT * CHUNK_K) >= 2) ? 2 : 1);
    static constexpr int BK = KB * CHUNK_K;          // k extent of a batch
    static constexpr int PITCH = BK + 8;             // halves; +8 spreads the rows over the LDS banks
    static constexpr int UNIT = VPI > 8 ? VPI : 8;   // halves permuted together when staging x
    static constexpr int UPR = BK / UNIT;            // staging units per x row
    static constexpr int XL = (MT * UPR + 63) / 64;  // staging units per lane
    static constexpr int GPB = BK / GROUP > 0 ? BK / GROUP : 1;   // groups per batch per row
    static constexpr int GL = (GPB + 3) / 4;         // groups each of a row's 4 lanes fetches
    static constexpr int X_BYTES = MT * PITCH * 2;
    static constexpr int META_BYTES = 16 * GPB * 2 * 2;
    static constexpr int WAVE_LDS = X_BYTES + META_BYTES;
    // A chunk that lies inside one quantisation group can be unpacked to the exact integers q - z and
    // the group's partial dot product scaled by s afterwards (4 FMAs per chunk instead of a multiply
    // per weight pair).  Smaller groups scale every weight, reproducing the reference's W16 bit for bit.
    static constexpr bool POST = GROUP % CHUNK_K == 0;
    static_assert(GROUP % VPI == 0, "a packed word must not straddle groups");
};

template <int BITS>
BW_DEV void permute_unit(const uint32_t* r, uint32_t* o) {
    if constexpr (BITS == 8) {
#pragma unroll
        for (int j = 0; j < 4; j++) o[j] = r[j];
    } else if constexpr (BITS == 4) {
        // 8 halves in r[0..3] -> (h0,h4)(h1,h5)(h2,h6)(h3,h7)
        o[0] = __builtin_amdgcn_perm(r[2], r[0], 0x05040100u);
        o[1] = __builtin_amdgcn_perm(r[2], r[0], 0x07060302u);
        o[2] = __builtin_amdgcn_perm(r[3], r[1], 0x05040100u);
        o[3] = __builtin_amdgcn_perm(r[3], r[1], 0x07060302u);
    } else {
        // 16 halves in r[0..7] -> (h_j, h_{j+8}) for j = 0..7
#pragma unroll
        for (int j = 0; j < 8; j++)
            o[j] = __builtin_amdgcn_perm(r[4 + j / 2], r[j / 2], (j & 1) ? 0x07060302u : 0x05040100u);
    }
}

// One wave = 16 rows x (its share of K).  Nothing is shared between the waves of a workgroup until the
// final reduction, so there is no barrier on the load path: every wave stages the activations and the
// scales / zero points of its own batch in its own LDS region.
template <int BITS, int GROUP, int MT>
__global__ __launch_bounds__(kWaves * 64) void qgemv_kernel(
    const _Float16* __restrict__ x, int M, int K, int64_t ldx, const uint32_t* __restrict__ qweight,
    const _Float16* __restrict__ scale, const _Float16* __restrict__ zp, const _Float16* __restrict__ bias, int N,
    _Float16* __restrict__ y, int64_t ldy) {
    using C = GemvCfg<BITS, GROUP, MT>;
    constexpr int UW = C::UNIT / 8;                       // 16-byte loads per staging unit
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nl = lane & 15, kq = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int row = min(n0 + nl, N - 1);                 // clamp: out-of-range rows are computed and dropped
    const int row_bytes = K * BITS / 8, groups = K / GROUP;
    const int nchunks = (K + C::CHUNK_K - 1) / C::CHUNK_K;
    _Float16* xs = reinterpret_cast<_Float16*>(smem + wave * C::WAVE_LDS);
    _Float16* s_lds = reinterpret_cast<_Float16*>(smem + wave * C::WAVE_LDS + C::X_BYTES);
    _Float16* z_lds = s_lds + 16 * C::GPB;
    float* red = reinterpret_cast<float*>(smem + kWaves * C::WAVE_LDS);

    const char* wrow = reinterpret_cast<const char*>(qweight) + (int64_t)row * row_bytes;
    const _Float16* srow = scale + (int64_t)row * groups;
    const _Float16* zrow = zp + (int64_t)row * groups;

    // Two register sets (ping-pong): while one batch is being unpacked and multiplied, the loads of the
    // wave's next batch are in flight into the other set.  The sets are never copied - a register move of
    // an outstanding load would stall on it.
    struct Regs {
        u4 x[C::XL * UW];
        _Float16 s[C::GL], z[C::GL];
        u4 w[C::KB];
    };
    // Loads return in order, so activations and scales (cache hits) are requested before the weights
    // (HBM) and can be staged while the weights are still in flight.
    auto issue = [&](int c0, Regs& r) {
        const int k0 = c0 * C::CHUNK_K;
#pragma unroll
        for (int i = 0; i < C::XL; i++) {
            const int u = lane + 64 * i, m = u / C::UPR, k = k0 + (u - m * C::UPR) * C::UNIT;
            const bool ok = m < M && k < K;               // K % UNIT == 0: a unit is entirely in or out
            const u4* src = reinterpret_cast<const u4*>(x + (int64_t)(ok ? m : 0) * ldx + (ok ? k : 0));
#pragma unroll
            for (int j = 0; j < UW; j++) { r.x[i * UW + j] = src[j]; if (!ok) r.x[i * UW + j] = u4{0, 0, 0, 0}; }
        }
        const int g0 = k0 / GROUP + kq * C::GL;
#pragma unroll
        for (int j = 0; j < C::GL; j++) {
            const int gi = min(g0 + j, groups - 1);
            r.s[j] = srow[gi];
            r.z[j] = zrow[gi];
        }
        asm volatile("" ::: "memory");                    // keep the weight loads behind the small ones
#pragma unroll
        for (int b = 0; b < C::KB; b++) {
            int kbyte = (c0 + b) * 64 + kq * 16;
            kbyte = kbyte < row_bytes ? kbyte : 0;        // masked lanes re-read byte 0; their x is zero
            r.w[b] = *reinterpret_cast<const u4*>(wrow + kbyte);
        }
        asm volatile("" ::: "memory");
    };

    f4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    const int arow = nl < MT ? nl : MT - 1;              // MFMA rows >= MT repeat a valid row; never stored

    // stage the batch's activations (permuted to the unpack order) and scales into the wave's LDS
    auto stage = [&](Regs& r) {
#pragma unroll
        for (int i = 0; i < C::XL; i++) {
            const int u = lane + 64 * i, m = u / C::UPR, ku = u - m * C::UPR;
            if (m < MT) {
                uint32_t in[4 * UW], o[4 * UW];
#pragma unroll
                for (int j = 0; j < UW; j++) { in[4 * j] = r.x[i * UW + j][0]; in[4 * j + 1] = r.x[i * UW + j][1]; in[4 * j + 2] = r.x[i * UW + j][2]; in[4 * j + 3] = r.x[i * UW + j][3]; }
                permute_unit<BITS>(in, o);
                u4* dst = reinterpret_cast<u4*>(xs + m * C::PITCH + ku * C::UNIT);
#pragma unroll
                for (int j = 0; j < UW; j++) dst[j] = u4{o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]};
            }
        }
#pragma unroll
        for (int j = 0; j < C::GL; j++) {
            if (kq * C::GL + j < C::GPB) { s_lds[nl * C::GPB + kq * C::GL + j] = r.s[j]; z_lds[nl * C::GPB + kq * C::GL + j] = r.z[j]; }
        }
        __builtin_amdgcn_wave_barrier();
    };

    auto compute = [&](Regs& r) {
#pragma unroll
        for (int b = 0; b < C::KB; b++) {
            // chunks past the end of K are not skipped: their activations were staged as zeros, and
            // straight-line code lets the four chunks' unpack and MFMA chains interleave
            const int gb = (b * C::CHUNK_K + kq * C::VPL) / GROUP;   // group index inside the batch
            GroupConst<BITS> gc[C::NG];
#pragma unroll
            for (int g = 0; g < C::NG; g++) gc[g].set(s_lds[nl * C::GPB + gb + g], z_lds[nl * C::GPB + gb + g]);
            h2 wp[C::VPL / 2];
            dequant_lane16<BITS, C::NG, !C::POST>(r.w[b], gc, wp);
            const _Float16* xp = xs + arow * C::PITCH + b * C::CHUNK_K + kq * C::VPL;
            if constexpr (C::POST) {
                f4 part = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < C::MF; t++)
                    part = __builtin_amdgcn_mfma_f32_16x16x32_f16(*reinterpret_cast<const h8*>(xp + 8 * t),
                                                                  pack_h8(wp + 4 * t), part, 0, 0, 0);
                const float sf = (float)s_lds[nl * C::GPB + (b * C::CHUNK_K) / GROUP];
#pragma unroll
                for (int q = 0; q < 4; q++) acc[b & 1][q] = __builtin_fmaf(sf, part[q], acc[b & 1][q]);
            } else {
#pragma unroll
                for (int t = 0; t < C::MF; t++)
                    acc[t & 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(*reinterpret_cast<const h8*>(xp + 8 * t),
                                                                        pack_h8(wp + 4 * t), acc[t & 1], 0, 0, 0);
            }
        }
        __builtin_amdgcn_wave_barrier();
    };

    constexpr int kStride = kWaves * C::KB;
    Regs ra, rb;
    int c0 = wave * C::KB;
    if (c0 < nchunks) {
        issue(c0, ra);
        // The "more to come" and "last batch" paths are separate code so that each path's wait counts
        // are exact: after a branch merge the compiler would have to wait for the prefetch as well.
        while (true) {
            stage(ra);
            const int c1 = c0 + kStride;
            if (c1 >= nchunks) { compute(ra); break; }
            issue(c1, rb);
            compute(ra);
            stage(rb);
            c0 = c1 + kStride;
            if (c0 >= nchunks) { compute(rb); break; }
            issue(c0, ra);
            compute(rb);
        }
    }
    // acc[r] = partial y[m = 4*kq + r][n = nl]
#pragma unroll
    for (int r = 0; r < 4; r++) red[(wave * 16 + 4 * kq + r) * 16 + nl] = acc[0][r] + acc[1][r];
    __syncthreads();
    if (tid < 256) {
        const int m = tid >> 4, n = n0 + (tid & 15);
        if (m < M && n < N) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < kWaves; w++) v += red[(w * 16 + m) * 16 + (tid & 15)];
            if (bias) v += (float)bias[n];
            y[(int64_t)m * ldy + n] = (_Float16)v;
        }
    }
}

template <int BITS, int GROUP, int MT>
int launch_gemv_mt(const void* x, int64_t M, int64_t K, int64_t ldx, const int32_t* qweight, const void* scale,
                   const void* zp, const void* bias, int64_t N, void* y, int64_t ldy, hipStream_t stream) {
    using C = GemvCfg<BITS, GROUP, MT>;
    const size_t lds = (size_t)kWaves * C::WAVE_LDS + (size_t)kWaves * 256 * 4;
    auto kern = qgemv_kernel<BITS, GROUP, MT>;
    static bool attr_set = false;                          // per instantiation; benign if raced
    if (lds > 64 * 1024 && !attr_set) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return BW_ELAUNCH;
        attr_set = true;
    }
    dim3 grid((unsigned)((N + 15) / 16)), block(kWaves * 64);
    hipLaunchKernelGGL(kern, grid, block, lds, stream, (const _Float16*)x, (int)M, (int)K, ldx, (const uint32_t*)qweight,
                       (const _Float16*)scale, (const _Float16*)zp, (const _Float16*)bias, (int)N, (_Float16*)y, ldy);
    return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
}

template <int BITS, int GROUP>
int launch_gemv(const void* x, int64_t M, int64_t K, int64_t ldx, const int32_t* qweight, const void* scale,
                const void* zp, const void* bias, int64_t N, void* y, int64_t ldy, hipStream_t stream) {
    if (M == 1) return launch_gemv_mt<BITS, GROUP, 1>(x, M, K, ldx, qweight, scale, zp, bias, N, y, ldy, stream);
    if (M <= 4) return launch_gemv_mt<BITS, GROUP, 4>(x, M, K, ldx, qweight, scale, zp, bias, N, y, ldy, stream);
    if (M <= 8) return launch_gemv_mt<BITS, GROUP, 8>(x, M, K, ldx, qweight, scale, zp, bias, N, y, ldy, stream);
    return launch_gemv_mt<BITS, GROUP, 16>(x, M, K, ldx, qweight, scale, zp, bias, N, y, ldy, stream);
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
