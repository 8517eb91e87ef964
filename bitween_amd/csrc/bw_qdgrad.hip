// bw_qdgrad.hip - input gradient of the quantised linear layer, fused with the dequantisation:
//
//     grad_x[M][K] = grad_y[M][N] @ W16[N][K],      W16 = fp16(scale * (q - zp))   (or bfloat16 for bfloat16 gradients)
//
// (QuantizedLinearFunction.backward, bitween/modules.py:108-141: it unpacks, forms W32 = scale * (q - zp),
// casts to grad_output's dtype and calls matmul; for float16 gradients that cast gives exactly W16, for bfloat16
// gradients the float32 product - exact: an 11-bit scale times an integer below 256 - rounded to nearest even, which
// is what the kernel forms with the hardware's packed float32 -> bfloat16 conversion before a bfloat16 MFMA.)
//
// The reduction runs over N, the dimension the packed words do NOT run along, so a weight tile has to be
// transposed on its way to the matrix core.  A workgroup owns a 128 or 256 (m) x 128 (k) tile of grad_x and walks
// N in steps of 32 rows:
//   * 256 threads each take 16 consecutive k of one row n (one group: groups are >= 32 wide), dequantise them to
//     the reference's W16 in natural k order (magic-number unpack, exact q - z, one multiply by the scale) and write
//     them as they are - 32 bytes - into an LDS tile stored n-major (row n holds the 128 k of the tile; the 32-byte
//     pieces of a row XOR-swizzled by the row number);
//   * the matrix core wants, per lane, 8 consecutive n of one k: ds_read_b64_tr_b16 is that transposition - the 16
//     lanes of a quarter wave point at 4 rows x 4 pieces of 4 halves and each receives one column of the 4 x 16 block
//     (element e of lane i = element i % 4 of the piece lane 4 e + i / 4 points at), two reads per operand;
//   * the 128 / 256 x 32 slice of grad_y goes to a second LDS tile as it is;
//   * v_mfma_f32_16x16x32_f16 with A = those columns (8 consecutive n per lane) and B = rows of the
//     grad_y tile: D[k][m], so a lane ends up with 4 consecutive k of one m.
// LDS is double buffered and filled one step ahead, in the shadow of the current step's MFMAs; global loads run
// two steps ahead; one barrier per step.  Three (two with the 256-row tile) workgroups share a CU and cover each
// other's barriers.
// Small M * K leaves the chip idle, so N is cut into slices whose float32 partial tiles a second kernel adds up.
#include <hip/hip_runtime.h>

#include "bw_common.h"

namespace {

constexpr int DK = 128, DN = 32, DTHREADS = 256;
constexpr int DPITCH = 80;                           // bytes per LDS row of the grad_y tile: 32 halves + 16 (rows stay 16-byte aligned)
constexpr int B_BYTES = DN * DK * 2;                 // n-major weight tile: 32 rows of 128 halves, unpadded
// MT = 16-row m tiles per wave (the workgroup's 2 x 2 waves cover 32 MT rows of m).  MT = 4 (161 registers, three
// workgroups per CU) up to 512 rows of grad_y; MT = 8 (251 registers, two per CU, a quarter fewer LDS reads per MFMA)
// beyond: 15-20 % faster there, slower below.
template <int MT> struct DgradTile {
    static constexpr int DM = 32 * MT;
    static constexpr int A_BYTES = DM * DPITCH;      // grad_y tile
    static constexpr int STAGE = A_BYTES + B_BYTES;
};

struct DgradArgs {
    const _Float16* go;
    const char* qweight;
    const _Float16* scale;
    const _Float16* zp;
    _Float16* gx;
    float* ws;
    int M, N, K, ldg, ldx, groups, row_bytes;
    int tiles_k, splits, steps_per_split;
};

// 32-byte piece p of row n of the weight tile sits at piece p ^ w_swizzle(n): the rows a transposing read touches
// (n = 8 q + 4 h + 0..3 for the four quarter waves q) then fall into different banks, 8 distinct pieces per half wave
BW_DEV int w_swizzle(int n) { return (n & 3) | (((n >> 3) & 1) << 2); }

typedef short s4 __attribute__((ext_vector_type(4)));

template <int BITS> struct WLoad;
template <> struct WLoad<4> { typedef u2 type; };
template <> struct WLoad<8> { typedef u4 type; };
template <> struct WLoad<2> { typedef uint32_t type; };

// 16 values of one row -> 8 float16 pairs in natural k order.  SCALE = false: the exact integers q - z (the caller
// multiplies by the scale in float32).
template <int BITS, bool SCALE>
BW_DEV void dequant16(const typename WLoad<BITS>::type& w, const GroupConstNat<BITS>& gc, h2* out) {
    if constexpr (BITS == 4) {
        dequant_word4_nat<SCALE>(w[0], gc, out);
        dequant_word4_nat<SCALE>(w[1], gc, out + 4);
    } else if constexpr (BITS == 8) {
#pragma unroll
        for (int j = 0; j < 4; j++) dequant_word8_nat<SCALE>(w[j], gc, out + 2 * j);
    } else {
        dequant_halfword2_nat<SCALE>(w, 0, gc, out);
        dequant_halfword2_nat<SCALE>(w, 1, gc, out + 4);
    }
}

typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
typedef float f2 __attribute__((ext_vector_type(2)));

// two float32 -> two 16-bit values of the gradient's type, round to nearest even, as one dword
template <int DT>
BW_DEV uint32_t pack2(float a, float b) {
    if constexpr (DT == BW_F16) return as_u32(h2{(_Float16)a, (_Float16)b});
    else return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2{a, b}, bf2));
}

template <int DT>
BW_DEV f4 mfma16(const h8& a, const h8& b, const f4& c) {
    if constexpr (DT == BW_F16) return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8, a), __builtin_bit_cast(bf8, b), c, 0, 0, 0);
}
template <int BITS, int GROUP, int MT, int DT>
__global__ __launch_bounds__(DTHREADS, MT == 4 ? 3 : 2) void qdgrad_kernel(const DgradArgs a) {   // workgroups per CU: 3 (<= 168 registers) or 2
    constexpr int DM = DgradTile<MT>::DM, A_BYTES = DgradTile<MT>::A_BYTES, STAGE = DgradTile<MT>::STAGE;
    constexpr int GR = DM / 128;                                      // grad_y rows a thread stages
    constexpr int PD = 2;                                             // steps of global loads in flight (even)
    extern __shared__ __attribute__((aligned(16))) char smem[];
    typedef typename WLoad<BITS>::type wload_t;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tile = blockIdx.x / a.splits, split = blockIdx.x % a.splits;
    const int m0 = (tile / a.tiles_k) * DM, k0 = (tile % a.tiles_k) * DK;
    const int nsteps = a.N / DN;
    const int s_begin = split * a.steps_per_split;
    const int s_end = min(s_begin + a.steps_per_split, nsteps);

    // loader roles
    const int wn = tid >> 3, wks = tid & 7;                           // weight: row of the step, 16-value segment
    const int gm = tid >> 1, gpart = tid & 1;                         // grad_y: row of the tile, 32-byte half
    const char* wp = a.qweight + (int64_t)wn * a.row_bytes + (int64_t)(k0 + wks * 16) * BITS / 8;
    const int gcol = (k0 + wks * 16) / GROUP;
    const _Float16* sp = a.scale + (int64_t)wn * a.groups + gcol;
    const _Float16* zp = a.zp + (int64_t)wn * a.groups + gcol;
    // rows past M repeat the last row: every output row depends on its own grad_y row only, and rows >= M are
    // never stored
    const _Float16* gp[GR];
#pragma unroll
    for (int r = 0; r < GR; r++) gp[r] = a.go + (int64_t)min(m0 + gm + 128 * r, a.M - 1) * a.ldg + gpart * 16;
    // a thread's 16 values are one 32-byte piece of row wn of the weight tile
    const int b_dst = wn * (DK * 2) + ((wks ^ w_swizzle(wn)) * 32);

    // PD steps of loads are in flight (a step's MFMAs take a fraction of a memory round trip).  Requests are
    // unconditional - past the slice's end they repeat its last step - so the wait counts stay exact.
    wload_t wreg[PD];
    _Float16 sreg[PD], zreg[PD];
    u4 greg[PD][2 * GR];
    auto issue = [&](int step, int slot) {
        const int64_t n0 = (int64_t)min(step, s_end - 1) * DN;
        wreg[slot] = *reinterpret_cast<const wload_t*>(wp + n0 * a.row_bytes);
        sreg[slot] = sp[n0 * a.groups];
        zreg[slot] = zp[n0 * a.groups];
#pragma unroll
        for (int r = 0; r < GR; r++) {
            greg[slot][2 * r] = *reinterpret_cast<const u4*>(gp[r] + n0);
            greg[slot][2 * r + 1] = *reinterpret_cast<const u4*>(gp[r] + n0 + 8);
        }
    };

    f4 acc[4][MT];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < MT; j++) acc[i][j] = f4{0.f, 0.f, 0.f, 0.f};

    const int wk = (wave & 1) * 64, wm = (wave >> 1) * (16 * MT);     // this wave's quarter of the tile
    const int l16 = lane & 15, q = lane >> 4;
    // rows of the weight tile this lane points the transposing reads at (h = 0, 1) and their swizzle (the same for both)
    const int tr_row[2] = {(8 * q + (l16 >> 2)) * (DK * 2), (8 * q + 4 + (l16 >> 2)) * (DK * 2)};
    const int tr_swz = w_swizzle(8 * q + (l16 >> 2));

    // slot -> LDS stage: dequantise the 16 weights and scatter them transposed; copy the grad_y rows
    auto fill = [&](int slot, int stage, bool live) {
        char* As = smem + stage * STAGE;
        char* Bs = As + A_BYTES;
        GroupConstNat<BITS> gc;
        gc.set(live ? sreg[slot] : (_Float16)0.f, zreg[slot]);        // past the slice's end: weights of zero
        h2 w16[8];
        uint32_t wd[8];                                               // the 8 pairs in the gradient's type
        if constexpr (DT == BW_F16) {
            dequant16<BITS, true>(wreg[slot], gc, w16);
#pragma unroll
            for (int i = 0; i < 8; i++) wd[i] = as_u32(w16[i]);
        } else {
            dequant16<BITS, false>(wreg[slot], gc, w16);              // exact q - z; the product with the scale is exact in float32
            const float sf = (float)gc.s[0];
#pragma unroll
            for (int i = 0; i < 8; i++) wd[i] = pack2<DT>(__fmul_rn((float)w16[i][0], sf), __fmul_rn((float)w16[i][1], sf));
        }
        *reinterpret_cast<u4*>(Bs + b_dst) = u4{wd[0], wd[1], wd[2], wd[3]};
        *reinterpret_cast<u4*>(Bs + b_dst + 16) = u4{wd[4], wd[5], wd[6], wd[7]};
#pragma unroll
        for (int r = 0; r < GR; r++) {
            u4* dst = reinterpret_cast<u4*>(As + (gm + 128 * r) * DPITCH + gpart * 32);
            dst[0] = greg[slot][2 * r];
            dst[1] = greg[slot][2 * r + 1];
        }
    };

    // Step s: read the fragments of stage s & 1, then - in the shadow of the step's MFMAs - fill the other
    // stage with step s + 1 and request step s + 1 + PD.  One barrier per step: everybody has read the
    // fragments of stage s & 1 before the next step overwrites it, and has written step s + 1 before it is read.
    if (s_begin < s_end) {
#pragma unroll
        for (int d = 0; d < PD; d++) issue(s_begin + d, d);
        fill(0, 0, true);
        issue(s_begin + PD, 0);
        __syncthreads();
    }
    // whole passes of PD steps, no early exit (the steps past the end multiply by zero weights): the loop body
    // is one straight block, which keeps the compiler's count of outstanding loads exact
    for (int base = s_begin; base < s_end; base += PD) {
#pragma unroll
        for (int d = 0; d < PD; d++) {
            const int step = base + d;
            const char* As = smem + (d & 1) * STAGE;                  // PD is even: stages alternate across passes too
            const char* Bs = As + A_BYTES;
            h8 af[4], bf[MT];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                // operand of k-tile i: n = 8 q .. 8 q + 7 of column k = wk + 16 i + l16 - two transposing reads of 4 n each
                const int piece = (wk >> 4) + i;
                s4 v[2];
#pragma unroll
                for (int h = 0; h < 2; h++)
                    v[h] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) s4*)(Bs + tr_row[h] + ((piece ^ tr_swz) * 32) + (l16 & 3) * 8));
                af[i] = __builtin_bit_cast(h8, __builtin_shufflevector(v[0], v[1], 0, 1, 2, 3, 4, 5, 6, 7));
            }
#pragma unroll
            for (int j = 0; j < MT; j++) bf[j] = *reinterpret_cast<const h8*>(As + (wm + 16 * j + l16) * DPITCH + q * 16);
            fill((d + 1) % PD, (d + 1) & 1, step + 1 < s_end);
            issue(step + 1 + PD, (d + 1) % PD);
#pragma unroll
            for (int j = 0; j < MT; j++)
#pragma unroll
                for (int i = 0; i < 4; i++)
                    acc[i][j] = mfma16<DT>(af[i], bf[j], acc[i][j]);
            __syncthreads();
        }
    }

    // acc[i][j][r] = grad_x[m0 + wm + 16 j + l16][k0 + wk + 16 i + 4 q + r]
    if (a.splits > 1) {
        float* dst = a.ws + (size_t)blockIdx.x * (DM * DK);
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < MT; j++)
                *reinterpret_cast<f4*>(dst + (wm + 16 * j + l16) * DK + wk + 16 * i + 4 * q) = acc[i][j];
    } else {
#pragma unroll
        for (int j = 0; j < MT; j++) {
            const int m = m0 + wm + 16 * j + l16;
            if (m >= a.M) continue;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const f4 v = acc[i][j];
                _Float16* dst = a.gx + (int64_t)m * a.ldx + k0 + wk + 16 * i + 4 * q;
                *reinterpret_cast<u2*>(dst) = u2{pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
            }
        }
    }
}

// grad_x tile = sum of its slices' partial tiles, rounded once
template <int DM, int DT>
__global__ __launch_bounds__(256) void qdgrad_reduce_kernel(const DgradArgs a) {
    const int tile = blockIdx.y;
    const int quad = (int)(blockIdx.x * blockDim.x + threadIdx.x);    // < DM * DK / 4
    const int ml = quad / (DK / 4), kl = (quad % (DK / 4)) * 4;
    const int m = (tile / a.tiles_k) * DM + ml, k = (tile % a.tiles_k) * DK + kl;
    if (m >= a.M) return;
    const float* src = a.ws + (size_t)tile * a.splits * (DM * DK) + ml * DK + kl;
    f4 v = {0.f, 0.f, 0.f, 0.f};
    for (int z = 0; z < a.splits; z++) {
        const f4 t = *reinterpret_cast<const f4*>(src + (size_t)z * (DM * DK));
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] += t[i];
    }
    *reinterpret_cast<u2*>(a.gx + (int64_t)m * a.ldx + k) = u2{pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
}

struct DgradPlan {
    int mt, tiles_k, tiles, splits, steps_per_split;
    size_t ws_bytes;
};

inline int dgrad_cus() {
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
            n = 0;
        return n > 0 ? n : 256;
    }();
    return cus;
}

// Three workgroups fit a CU and hide each other's barriers.  With fewer tiles than two per CU N is cut into slices:
// to two workgroups per CU (three measured slower: more partial-tile traffic) when a slice keeps at least 24 steps,
// else to one per CU with at least 8 (short slices pay their prologue and the partial tiles' traffic).
inline DgradPlan dgrad_plan(int64_t M, int64_t N, int64_t K, bool have_workspace) {
    DgradPlan p;
    p.mt = M > 512 ? 8 : 4;
    const int DM = 32 * p.mt;
    p.tiles_k = (int)(K / DK);
    p.tiles = p.tiles_k * (int)((M + DM - 1) / DM);
    const int nsteps = (int)(N / DN);
    p.splits = 1;
    p.steps_per_split = nsteps;
    p.ws_bytes = 0;
    if (!have_workspace) return p;
    const int cus = dgrad_cus();
    int s = (2 * cus + p.tiles - 1) / p.tiles;
    if (s < 2 || nsteps / s < 24) {
        s = (cus + p.tiles - 1) / p.tiles;
        if (s > nsteps / 8) s = nsteps / 8;
    }
    if (s > 32) s = 32;
    if (s < 2) return p;
    const int sps = (nsteps + s - 1) / s;
    s = (nsteps + sps - 1) / sps;
    if (s < 2) return p;
    p.splits = s;
    p.steps_per_split = sps;
    p.ws_bytes = (size_t)p.tiles * s * DM * DK * sizeof(float);
    return p;
}

inline bool dgrad_fast_shape(int64_t M, int64_t N, int64_t K, int64_t ldg, int64_t ldx, int bits, int group) {
    return (group == 32 || group == 64 || group == 128) && K % DK == 0 && N % DN == 0 && ldg % 8 == 0 && ldx % 4 == 0 &&
           M >= 1 && M < ((int64_t)1 << 24) && N * (K * bits / 8) < ((int64_t)1 << 40);
}

template <int BITS, int GROUP, int MT, int DT>
int launch_dgrad_mt(const DgradArgs& a, const DgradPlan& p, hipStream_t stream) {
    constexpr int DM = DgradTile<MT>::DM;
    auto kern = qdgrad_kernel<BITS, GROUP, MT, DT>;
    static uint64_t big_lds_devices = 0;                   // per instantiation
    if (2 * DgradTile<MT>::STAGE > 64 * 1024 && !bw_allow_big_lds(reinterpret_cast<const void*>(kern), big_lds_devices)) return BW_ELAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)(p.tiles * p.splits)), dim3(DTHREADS), 2 * DgradTile<MT>::STAGE, stream, a);
    if (hipGetLastError() != hipSuccess) return BW_ELAUNCH;
    if (p.splits > 1) {
        hipLaunchKernelGGL((qdgrad_reduce_kernel<DM, DT>), dim3(DM * DK / 4 / 256, (unsigned)p.tiles), dim3(256), 0, stream, a);
        if (hipGetLastError() != hipSuccess) return BW_ELAUNCH;
    }
    return BW_OK;
}

template <int BITS, int GROUP, int DT>
int launch_dgrad(DgradArgs a, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    const DgradPlan p = dgrad_plan(a.M, a.N, a.K, workspace != nullptr);
    if (p.ws_bytes > workspace_bytes) return BW_EWORKSPACE;
    a.ws = (float*)workspace;
    a.tiles_k = p.tiles_k;
    a.splits = p.splits;
    a.steps_per_split = p.steps_per_split;
    return p.mt == 8 ? launch_dgrad_mt<BITS, GROUP, 8, DT>(a, p, stream) : launch_dgrad_mt<BITS, GROUP, 4, DT>(a, p, stream);
}

}  // namespace

extern "C" size_t bw_qdgrad_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits, int group) {
    if (!bw_shape_ok(N, K, bits, group) || !dgrad_fast_shape(M, N, K, N, K, bits, group)) return 0;
    return dgrad_plan(M, N, K, true).ws_bytes;
}

extern "C" int bw_qdgrad(const void* grad_y, int act_dtype, int64_t M, int64_t N, int64_t ldg, const int32_t* qweight,
                         const void* scale16, const void* zp16, int64_t K, int bits, int group, void* grad_x,
                         int64_t ldx, void* workspace, size_t workspace_bytes, void* stream) {
    if (!grad_y || !qweight || !scale16 || !zp16 || !grad_x) return BW_EINVAL;
    if (!bw_shape_ok(N, K, bits, group) || M < 1 || ldg < N || ldx < K) return BW_EINVAL;
    if (act_dtype != BW_F16 && act_dtype != BW_BF16) return BW_EUNSUPPORTED;
    if (!dgrad_fast_shape(M, N, K, ldg, ldx, bits, group)) return BW_EUNSUPPORTED;
    if (!bw_aligned(grad_y, 16) || !bw_aligned(grad_x, 8) || !bw_aligned(qweight, 16)) return BW_EALIGN;
    if (workspace && !bw_aligned(workspace, 16)) return BW_EALIGN;
    DgradArgs a;
    a.go = (const _Float16*)grad_y; a.qweight = (const char*)qweight; a.scale = (const _Float16*)scale16;
    a.zp = (const _Float16*)zp16; a.gx = (_Float16*)grad_x; a.ws = nullptr;
    a.M = (int)M; a.N = (int)N; a.K = (int)K; a.ldg = (int)ldg; a.ldx = (int)ldx;
    a.groups = (int)(K / group); a.row_bytes = (int)(K * bits / 8);
    hipStream_t st = (hipStream_t)stream;
#define BW_CASE(B, G)                                                                                                    \
    if (bits == B && group == G)                                                                                         \
        return act_dtype == BW_F16 ? launch_dgrad<B, G, BW_F16>(a, workspace, workspace_bytes, st)                       \
                                   : launch_dgrad<B, G, BW_BF16>(a, workspace, workspace_bytes, st);
    BW_CASE(4, 128) BW_CASE(4, 64) BW_CASE(4, 32)
    BW_CASE(8, 128) BW_CASE(8, 64) BW_CASE(8, 32)
    BW_CASE(2, 128) BW_CASE(2, 64) BW_CASE(2, 32)
#undef BW_CASE
    return BW_EUNSUPPORTED;
}
