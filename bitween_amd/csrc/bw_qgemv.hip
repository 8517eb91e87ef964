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
// A wave takes KB consecutive chunks per round, all of whose loads are issued
// before anything is waited for; each chunk is unpacked in registers as soon
// as its 16 bytes per lane land and is multiplied against the activations,
// which the wave staged in its own LDS tile in the k order the unpack emits.
// M < 16 leaves MFMA rows idle, which costs nothing: the matrix pipe has >5x
// headroom at HBM speed.
//
// Scales and zero points of the 16 rows are one contiguous block of the
// [N][K/group] arrays; the workgroup copies it to LDS once (one barrier).
// All global reads are buffer loads: the hardware range check returns zero
// for lanes past the end of a row block or of x, so no lane is predicated.
//
// Partial sums of the waves are reduced through LDS; the epilogue adds the
// bias in float32 and rounds once.
#include "bw_common.h"

#include <cstdlib>

namespace {

template <int BITS, int GROUP, int MT>
struct GemvCfg {
    static constexpr int VPI = 32 / BITS;            // values per int32 word
    static constexpr int VPL = 128 / BITS;           // values per 16-byte lane load
    static constexpr int CHUNK_K = 4 * VPL;          // k extent of one chunk
    static constexpr int MF = VPL / 8;               // MFMAs per lane load
    static constexpr int NG = (VPL > GROUP) ? VPL / GROUP : 1;   // groups per lane load
    static constexpr int UNIT = VPI > 8 ? VPI : 8;   // halves permuted together when staging x
    // A chunk that lies inside one quantisation group is unpacked to the exact integers q - z and the
    // group's partial dot product scaled by s afterwards (4 FMAs per chunk instead of a multiply per
    // weight pair).  Smaller groups scale every weight, reproducing the reference's W16 bit for bit.
    static constexpr bool POST = GROUP % CHUNK_K == 0;
    // 16 activation rows need 64 registers for the staged x alone: cap the workgroup at 8 waves there so
    // that every wave may use 256 VGPRs
    static constexpr int MAX_WAVES = MT > 8 ? 8 : 16;
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

struct GemvArgs {
    const void* x;
    const void* qweight;
    const void* scale;
    const void* zp;
    const _Float16* bias;
    _Float16* y;
    uint32_t x_bytes, w_bytes, meta_bytes;   // extents for the buffer range checks
    int M, N, K, ldx, ldy;
    int groups, nchunks, row_bytes;
};

BW_DEV __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), (short)0, (int)bytes, 0x00020000);
}

// blockDim.x = 64 * nwaves; wave w takes chunks [w*KB + r*nwaves*KB, +KB) for r = 0, 1, ...
template <int BITS, int GROUP, int MT, int KB>
__global__ __launch_bounds__((64 * GemvCfg<BITS, GROUP, MT>::MAX_WAVES)) void qgemv_kernel(const GemvArgs a) {
    using C = GemvCfg<BITS, GROUP, MT>;
    constexpr int BK = KB * C::CHUNK_K, PITCH = BK + 8, UPR = BK / C::UNIT, XL = (MT * UPR + 63) / 64;
    constexpr int X_BYTES = MT * PITCH * 2, UW = C::UNIT / 8;
    constexpr uint32_t kOob = 0x80000000u;               // any offset >= the buffer size reads as zero
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const int nl = lane & 15, kq = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int groups = a.groups;
    // LDS: [(scale, zero point) pairs 16 x GP uint32][x tile of wave 0] ... [x tile of wave n-1][partial sums]
    const int GP = groups | 1;                            // odd row pitch: the 16 rows hit different banks
    uint32_t* meta = reinterpret_cast<uint32_t*>(smem);
    char* after_meta = smem + ((16 * GP * 4 + 15) & ~15);
    _Float16* xs = reinterpret_cast<_Float16*>(after_meta + wave * X_BYTES);
    float* red = reinterpret_cast<float*>(after_meta + nwaves * X_BYTES);

    const __amdgpu_buffer_rsrc_t rw = make_rsrc(a.qweight, a.w_bytes), rx = make_rsrc(a.x, a.x_bytes),
                                 rs = make_rsrc(a.scale, a.meta_bytes), rz = make_rsrc(a.zp, a.meta_bytes);

    // ---- request everything of the first round, small things first (loads return in order) ----
    // scales / zero points: thread t fetches pair index t (and t + blockDim, ...) of the 16 x groups block
    const uint32_t meta_base = (uint32_t)n0 * groups * 2;
    uint16_t ms = 0, mz = 0;
    if (tid < 16 * groups) {
        ms = __builtin_amdgcn_raw_buffer_load_b16(rs, meta_base + tid * 2, 0, 0);
        mz = __builtin_amdgcn_raw_buffer_load_b16(rz, meta_base + tid * 2, 0, 0);
    }
    u4 xr[XL * UW];
    u4 wr[KB];
    const uint32_t w_lane = (uint32_t)(n0 + nl) * a.row_bytes + kq * 16;
    auto issue = [&](int c0) {
        const int k0 = c0 * C::CHUNK_K;
#pragma unroll
        for (int i = 0; i < XL; i++) {
            const int u = lane + 64 * i, m = u / UPR, k = k0 + (u - m * UPR) * C::UNIT;
            const uint32_t off = (m < a.M && k < a.K) ? (uint32_t)(m * a.ldx + k) * 2 : kOob;
#pragma unroll
            for (int j = 0; j < UW; j++) xr[i * UW + j] = __builtin_amdgcn_raw_buffer_load_b128(rx, off + j * 16, 0, 0);
        }
        asm volatile("" ::: "memory");                    // keep the weight loads behind the small ones
        const uint32_t off = c0 * 64 < a.row_bytes ? w_lane + c0 * 64 : kOob;
#pragma unroll
        for (int b = 0; b < KB; b++) wr[b] = __builtin_amdgcn_raw_buffer_load_b128(rw, off + b * 64, 0, 0);
        asm volatile("" ::: "memory");
    };
    int c0 = wave * KB;
    issue(c0);

    // ---- scales / zero points to LDS, once per workgroup ----
    if (tid < 16 * groups) {
        const int r = tid / groups, c = tid - r * groups;
        meta[r * GP + c] = (uint32_t)ms | ((uint32_t)mz << 16);
    }
    for (int e = tid + blockDim.x; e < 16 * groups; e += blockDim.x) {   // more pairs than threads
        const int r = e / groups, c = e - r * groups;
        const uint32_t s2 = __builtin_amdgcn_raw_buffer_load_b16(rs, meta_base + e * 2, 0, 0);
        const uint32_t z2 = __builtin_amdgcn_raw_buffer_load_b16(rz, meta_base + e * 2, 0, 0);
        meta[r * GP + c] = s2 | (z2 << 16);
    }
    __syncthreads();

    f4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    const int arow = nl < MT ? nl : MT - 1;              // MFMA rows >= MT repeat a valid row; never stored
    const uint32_t* mrow = meta + nl * GP;
    while (true) {
        // stage the round's activations, permuted to the unpack order, into this wave's LDS tile
#pragma unroll
        for (int i = 0; i < XL; i++) {
            const int u = lane + 64 * i, m = u / UPR, ku = u - m * UPR;
            if (m < MT) {
                uint32_t in[4 * UW], o[4 * UW];
#pragma unroll
                for (int j = 0; j < UW; j++) { in[4 * j] = xr[i * UW + j][0]; in[4 * j + 1] = xr[i * UW + j][1]; in[4 * j + 2] = xr[i * UW + j][2]; in[4 * j + 3] = xr[i * UW + j][3]; }
                permute_unit<BITS>(in, o);
                u4* dst = reinterpret_cast<u4*>(xs + m * PITCH + ku * C::UNIT);
#pragma unroll
                for (int j = 0; j < UW; j++) dst[j] = u4{o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]};
            }
        }
        __builtin_amdgcn_wave_barrier();
        const int k0 = c0 * C::CHUNK_K;
#pragma unroll
        for (int b = 0; b < KB; b++) {
            // chunks past the end of K are not skipped: their activations were staged as zeros
            const int gb = min((k0 + b * C::CHUNK_K + kq * C::VPL) / GROUP, groups - C::NG);
            GroupConst<BITS> gc[C::NG];
#pragma unroll
            for (int g = 0; g < C::NG; g++) {
                const uint32_t sz = mrow[gb + g];
                gc[g].set(__builtin_bit_cast(_Float16, (uint16_t)sz), __builtin_bit_cast(_Float16, (uint16_t)(sz >> 16)));
            }
            h2 wp[C::VPL / 2];
            dequant_lane16<BITS, C::NG, !C::POST>(wr[b], gc, wp);
            const _Float16* xp = xs + arow * PITCH + b * C::CHUNK_K + kq * C::VPL;
            if constexpr (C::POST) {
                f4 part = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < C::MF; t++)
                    part = __builtin_amdgcn_mfma_f32_16x16x32_f16(*reinterpret_cast<const h8*>(xp + 8 * t), pack_h8(wp + 4 * t), part, 0, 0, 0);
                const float sf = (float)gc[0].s[0];
#pragma unroll
                for (int q = 0; q < 4; q++) acc[b & 1][q] = __builtin_fmaf(sf, part[q], acc[b & 1][q]);
            } else {
#pragma unroll
                for (int t = 0; t < C::MF; t++)
                    acc[t & 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(*reinterpret_cast<const h8*>(xp + 8 * t), pack_h8(wp + 4 * t), acc[t & 1], 0, 0, 0);
            }
        }
        c0 += nwaves * KB;
        if (c0 >= a.nchunks) break;                       // wave-uniform
        __builtin_amdgcn_wave_barrier();
        issue(c0);
    }

    // acc[r] = partial y[m = 4*kq + r][n = nl]; only rows < MT are kept
    if (4 * kq < MT) {
#pragma unroll
        for (int r = 0; r < 4; r++)
            if (4 * kq + r < MT) red[(wave * MT + 4 * kq + r) * 16 + nl] = acc[0][r] + acc[1][r];
    }
    __syncthreads();
    for (int o = tid; o < 16 * MT; o += blockDim.x) {
        const int m = o >> 4, n = n0 + (o & 15);
        if (m < a.M && n < a.N) {
            float v = 0.f;
            for (int w = 0; w < nwaves; w++) v += red[(w * MT + m) * 16 + (o & 15)];
            if (a.bias) v += (float)a.bias[n];
            a.y[(int64_t)m * a.ldy + n] = (_Float16)v;
        }
    }
}

constexpr int kLdsBudget = 150 * 1024;

template <int BITS, int GROUP, int MT, int KB>
int launch_gemv_kb(const GemvArgs& a, hipStream_t stream) {
    using C = GemvCfg<BITS, GROUP, MT>;
    constexpr int BK = KB * C::CHUNK_K, X_BYTES = MT * (BK + 8) * 2;
    const size_t fixed = (size_t)((16 * (a.groups | 1) * 4 + 15) & ~15);
    int nwaves = (a.nchunks + KB - 1) / KB;
    if (nwaves > C::MAX_WAVES) nwaves = C::MAX_WAVES;
    while (nwaves > 1 && fixed + (size_t)nwaves * (X_BYTES + MT * 64) > (size_t)kLdsBudget) nwaves--;
    const size_t lds = fixed + (size_t)nwaves * (X_BYTES + MT * 64);
    if (lds > (size_t)kLdsBudget) return BW_EUNSUPPORTED;
    auto kern = qgemv_kernel<BITS, GROUP, MT, KB>;
    static bool attr_set = false;                          // per instantiation; benign if raced
    if (lds > 64 * 1024 && !attr_set) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
            return BW_ELAUNCH;
        attr_set = true;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)((a.N + 15) / 16)), dim3(nwaves * 64), lds, stream, a);
    return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
}

template <int BITS, int GROUP, int MT>
int launch_gemv_mt(const GemvArgs& a, hipStream_t stream) {
    using C = GemvCfg<BITS, GROUP, MT>;
    static const int force_kb = getenv("BW_GEMV_KB") ? atoi(getenv("BW_GEMV_KB")) : 0;
    // Chunks per wave and round, from timing Llama-shaped layers on MI355X: short rows want many small
    // waves (more requests in flight early), wide activation tiles want small batches (LDS, registers);
    // never more than ~16 KB of staged activations per wave.
    constexpr int fit = 8192 / (MT * C::CHUNK_K);
    int kb;
    if (MT >= 8) kb = a.nchunks <= 32 ? 1 : 2;
    else kb = (a.nchunks <= 32 && a.N < 8192) ? 2 : 4;
    if (kb > fit) kb = fit >= 4 ? 4 : (fit >= 2 ? 2 : 1);
    if (force_kb) kb = force_kb;
    if (kb >= 8) return launch_gemv_kb<BITS, GROUP, MT, 8>(a, stream);
    if (kb >= 4) return launch_gemv_kb<BITS, GROUP, MT, 4>(a, stream);
    if (kb >= 2) return launch_gemv_kb<BITS, GROUP, MT, 2>(a, stream);
    return launch_gemv_kb<BITS, GROUP, MT, 1>(a, stream);
}

template <int BITS, int GROUP>
int launch_gemv(const GemvArgs& a, hipStream_t stream) {
    if (a.M == 1) return launch_gemv_mt<BITS, GROUP, 1>(a, stream);
    if (a.M <= 4) return launch_gemv_mt<BITS, GROUP, 4>(a, stream);
    if (a.M <= 8) return launch_gemv_mt<BITS, GROUP, 8>(a, stream);
    return launch_gemv_mt<BITS, GROUP, 16>(a, stream);
}

}  // namespace

// Shapes the MFMA kernels take: 16-byte lane loads need K*bits/8 % 16 == 0, group in {32, 64, 128}, and
// every extent must fit the 32-bit offsets of buffer addressing.
bool bw_fast_shape(int64_t M, int64_t N, int64_t K, int64_t ldx, int bits, int group) {
    if (!((group == 32 || group == 64 || group == 128) && (K * bits / 8) % 16 == 0 && K % 16 == 0)) return false;
    const int64_t lim = (int64_t)1 << 31;
    return N * (K * bits / 8) < lim && M * ldx * 2 < lim && N * (K / group) * 2 < lim;
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
    if (!bw_fast_shape(M, N, K, ldx, bits, group) || !bw_aligned(x, 16) || (ldx * 2) % 16 || !bw_aligned(qweight, 16))
        return bw_qgemm_generic(x, act_dtype, M, K, ldx, qweight, scale16, zp16, bias, N, bits, group, y, ldy, stream);
    GemvArgs a;
    a.x = x; a.qweight = qweight; a.scale = scale16; a.zp = zp16; a.bias = (const _Float16*)bias; a.y = (_Float16*)y;
    a.M = (int)M; a.N = (int)N; a.K = (int)K; a.ldx = (int)ldx; a.ldy = (int)ldy;
    a.groups = (int)(K / group);
    a.row_bytes = (int)(K * bits / 8);
    a.nchunks = (a.row_bytes + 63) / 64;
    a.x_bytes = (uint32_t)(((M - 1) * ldx + K) * 2);
    a.w_bytes = (uint32_t)(N * a.row_bytes);
    a.meta_bytes = (uint32_t)(N * a.groups * 2);
    hipStream_t st = (hipStream_t)stream;
#define BW_CASE(B, G) \
    if (bits == B && group == G) return launch_gemv<B, G>(a, st);
    BW_CASE(4, 128) BW_CASE(4, 64) BW_CASE(4, 32)
    BW_CASE(8, 128) BW_CASE(8, 64) BW_CASE(8, 32)
    BW_CASE(2, 128) BW_CASE(2, 64) BW_CASE(2, 32)
#undef BW_CASE
    return BW_EUNSUPPORTED;
}
