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
//
// Two kernels share that scheme.  qdgrad_kernel (the "stepping" kernel, described above) serves small layers.  Large
// problems run qdgrad256_kernel further down: 256 columns of k per tile and 256 or 128 rows of m, one wave per SIMD,
// steps of 64 rows of n with the side work dealt out between the wave's own MFMAs - the forward kernel's natural-order
// schedule turned around.  dgrad256_rows() holds the measured rule that picks between them.
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
    uint32_t go_bytes, w_bytes, meta_bytes;          // extents for the buffer descriptors of the 256 x 256 kernel
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
template <int DM, int DT, int DKT = DK>
__global__ __launch_bounds__(256) void qdgrad_reduce_kernel(const DgradArgs a) {
    const int tile = blockIdx.y;
    const int quad = (int)(blockIdx.x * blockDim.x + threadIdx.x);    // < DM * DKT / 4
    const int ml = quad / (DKT / 4), kl = (quad % (DKT / 4)) * 4;
    const int m = (tile / a.tiles_k) * DM + ml, k = (tile % a.tiles_k) * DKT + kl;
    if (m >= a.M) return;
    const float* src = a.ws + (size_t)tile * a.splits * (DM * DKT) + ml * DKT + kl;
    f4 v = {0.f, 0.f, 0.f, 0.f};
    for (int z = 0; z < a.splits; z++) {
        const f4 t = *reinterpret_cast<const f4*>(src + (size_t)z * (DM * DKT));
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] += t[i];
    }
    *reinterpret_cast<u2*>(a.gx + (int64_t)m * a.ldx + k) = u2{pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
}


// ---- 256 (m) x 256 (k) tiles: one wave per SIMD, the side work dealt out between the wave's own MFMAs ----------------
//
// The kernel above keeps 16-32 MFMAs of a wave between two workgroup barriers and lets its four waves dequantise in
// lockstep; large problems run this one instead.  A wave owns 256 m x 64 k of the tile (all 256 accumulation
// registers); a step covers 64 rows of n: 128 MFMAs per wave between barriers.
//   * grad_y tile (256 rows x 128 bytes) memory -> LDS by buffer loads with LDS destination, 8 rows per instruction, the
//     16-byte pieces of a row XOR-swizzled by (row >> 1) & 7 (through the lane's source address) so that the fragment
//     reads of 16 rows spread over the banks; read through a ring of 8 fragments, one read per four MFMAs;
//   * weights: a thread owns two units of a step - 32 consecutive k of one row n each - requested two steps ahead,
//     dequantised to natural k order during the step before they are needed (48 pieces of one to three instructions per
//     unit, one piece per MFMA gap) and written n-major into the weight tile (64 rows x 512 bytes, 32-byte pieces
//     swizzled as above); every wave reads its 4 k-tiles back transposed (ds_read_b64_tr_b16, 16 reads per step);
//   * the step's barrier waits for LDS only and for the grad_y loads (explicit count: the weight requests made after them
//     stay in flight).
// Slices of N for small grids as above (float32 partial tiles + qdgrad_reduce_kernel).  Needs K % 256 == 0, N % 64 == 0.
constexpr int QM = 256, QK = 256, QN = 64;

template <int OFF>
BW_DEV void lds_read_b128_asm(h8& dst, uint32_t addr) {       // (assembly: an LDS read the compiler would order behind the loads to LDS in flight)
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
template <int OFF>
BW_DEV void lds_read_tr_asm(u2& dst, uint32_t addr) {
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
template <int DT>
BW_DEV void mfma_acc_agpr(f4& acc, const h8& a, const h8& b) {  // accumulators in the AGPR file: all 256 VGPRs stay free for operands
    if constexpr (DT == BW_F16) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
    else asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
BW_DEV __amdgpu_buffer_rsrc_t dgrad_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), (short)0, (int)bytes, 0x00020000);
}

template <int BITS, int GROUP, int DT, int MT>     // MT = 16: 256 rows of m per tile; MT = 8: 128 rows (twice the dequantisation per MFMA)
__global__ __launch_bounds__(256) void qdgrad256_kernel(const DgradArgs a) {
    constexpr int QMv = MT * 16, NT = 4, XRING = 8, MF = QN / 32;
    constexpr int WR = QMv / 4, UNITS = WR / 8;            // rows of grad_y a wave brings in, 8 per instruction
    constexpr int PPG = 48 / (3 * MT);                     // dequantisation pieces per gap: a unit's 48 over the first three gaps of MT slots
    constexpr int WL = BITS == 8 ? 2 : 1;                  // 16-byte (8-byte at 2 bits) loads per unit
    constexpr int REQ = 2 * (WL + 2);                      // requests of one step per thread: two units' words, scale, zero point
    constexpr int G_BYTES = QMv * QN * 2, W_BYTES = QN * QK * 2;
    constexpr uint32_t kOob = 0x80000000u;
    static_assert(MF == 2 && XRING <= MT && (MT == 16 || MT == 8), "schedule below: two MFMA steps, a ring no longer than a step");
    extern __shared__ __attribute__((aligned(16))) char smem[];
    char* gbuf[2] = {smem, smem + G_BYTES};
    char* wbuf[2] = {smem + 2 * G_BYTES, smem + 2 * G_BYTES + W_BYTES};
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nl = lane & 15, kq = lane >> 4;
    const int tile = (int)blockIdx.x / a.splits, split = (int)blockIdx.x % a.splits;
    const int m0 = (tile / a.tiles_k) * QMv, k0 = (tile % a.tiles_k) * QK;
    const int s_begin = split * a.steps_per_split, s_end = min(s_begin + a.steps_per_split, a.N / QN);
    const __amdgpu_buffer_rsrc_t rw = dgrad_rsrc(a.qweight, a.w_bytes), rg = dgrad_rsrc(a.go, a.go_bytes);
    const __amdgpu_buffer_rsrc_t rs = dgrad_rsrc(a.scale, a.meta_bytes), rz = dgrad_rsrc(a.zp, a.meta_bytes);
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);

    // weight units of a thread: unit e: row n = tid / 8 + 32 e of the step, the 32 k at block tid % 8 of the tile's 256
    const int un = tid >> 3, ub = tid & 7;
    uint32_t w_off[2], m_off[2], w_dst[2];
#pragma unroll
    for (int e = 0; e < 2; e++) {
        const int n = un + 32 * e;
        w_off[e] = (uint32_t)n * a.row_bytes + (uint32_t)(k0 + 32 * ub) * BITS / 8;
        m_off[e] = ((uint32_t)n * a.groups + (uint32_t)(k0 + 32 * ub) / GROUP) * 2;
        // 32-byte pieces 2 ub and 2 ub + 1 of row n; the swizzle touches the low 3 bits of the piece index, so the second
        // piece sits at the first one's address ^ 32
        w_dst[e] = n * (QK * 2) + (((2 * ub) ^ w_swizzle(n)) * 32);
    }
    struct WSet { u4 w[2][WL]; uint32_t s[2], z[2]; };
    WSet set0, set1;
    auto w_req = [&](int step, WSet& ws) {                 // past the slice's end: offsets beyond every buffer read as zero
        const uint32_t so = step < s_end ? (uint32_t)step * QN * a.row_bytes : kOob;
        const uint32_t mo = step < s_end ? (uint32_t)step * QN * a.groups * 2 : kOob;
#pragma unroll
        for (int e = 0; e < 2; e++) {
            if constexpr (BITS == 2) {
                const u2 v = __builtin_amdgcn_raw_buffer_load_b64(rw, w_off[e] + so, 0, 0);
                ws.w[e][0][0] = v[0];
                ws.w[e][0][1] = v[1];
            } else {
#pragma unroll
                for (int l = 0; l < WL; l++) ws.w[e][l] = __builtin_amdgcn_raw_buffer_load_b128(rw, w_off[e] + so + 16 * l, 0, 0);
            }
            ws.s[e] = __builtin_amdgcn_raw_buffer_load_b16(rs, m_off[e] + mo, 0, 0);
            ws.z[e] = __builtin_amdgcn_raw_buffer_load_b16(rz, m_off[e] + mo, 0, 0);
        }
    };
    // grad_y tile: a wave brings in rows WR wave .. + WR - 1, unit u = 8 rows; lane L: row L / 8, LDS piece L % 8 holds source
    // piece (L % 8) ^ s, s = (row >> 1) & 7 = (4 (u & 1) + (L >> 4)) & 7
    uint32_t gd_base[2];
#pragma unroll
    for (int par = 0; par < 2; par++) {
        const int sw = (4 * par + (lane >> 4)) & 7;
        gd_base[par] = (uint32_t)((m0 + WR * wave + (lane >> 3)) * a.ldg) * 2 + (((lane & 7) ^ sw) * 16);
    }
    auto g_dma = [&](int u, int step, char* buf) {
        uint32_t so = step < s_end ? (uint32_t)(u * 8 * a.ldg) * 2 + (uint32_t)step * QN * 2 : kOob;
        asm("" : "+s"(so));                                   // one scalar sum, one VALU add
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rg, (__attribute__((address_space(3))) void*)(buf + (WR * wave_u + 8 * u) * 128), 16,
                                                 gd_base[u & 1] + so, 0, 0, 0);
    };
    // grad_y fragment (m-tile i, MFMA step t) of the lane: row 16 i + nl, source piece 4 t + kq
    uint32_t fa[MF];
#pragma unroll
    for (int t = 0; t < MF; t++) fa[t] = (uint32_t)(nl * 128 + (((4 * t + kq) ^ (nl >> 1)) * 16));
    // weight fragment (k-tile j of the wave, step t, half h): the lane points at row 32 t + 8 kq + 4 h + (nl >> 2), piece
    // 4 wave + j, 8 (nl & 3) bytes in; the swizzle of those rows is the same for both h and both t
    const int tsw = w_swizzle(8 * kq + (nl >> 2));
    uint32_t ta[2], tp[NT];
#pragma unroll
    for (int h = 0; h < 2; h++) ta[h] = (uint32_t)((8 * kq + 4 * h + (nl >> 2)) * (QK * 2) + (nl & 3) * 8);
#pragma unroll
    for (int j = 0; j < NT; j++) tp[j] = (uint32_t)(((4 * wave + j) ^ tsw) * 32);

    f4 acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < NT; j++) acc[i][j] = f4{0.f, 0.f, 0.f, 0.f};
    h8 xf[XRING];
    u2 wfr[MF][NT][2];                                     // [t][j][h]
    uint32_t od[2][16];                                    // a unit's 16 pairs in the gradient's type, natural k order
    h2 ot[2][16];
    GroupConstNat<BITS> gcn[2];

    // Piece P (0 .. 47) of the dequantisation of unit e of `ws`: extract (1-3 instructions), exact q - z, times the scale.
    auto piece = [&](auto ec, auto pc, const WSet& ws) {
        constexpr int e = decltype(ec)::value, P = decltype(pc)::value;
        if constexpr (P == 0) gcn[e].set(__builtin_bit_cast(_Float16, (uint16_t)ws.s[e]), __builtin_bit_cast(_Float16, (uint16_t)ws.z[e]));
        auto finish = [&](int idx) {                          // ot[e][idx] = exact q - z  ->  od[e][idx]
            if constexpr (DT == BW_F16) od[e][idx] = as_u32(ot[e][idx] * gcn[e].s);
            else {
                const float sf = (float)gcn[e].s[0];
                od[e][idx] = pack2<DT>(__fmul_rn((float)ot[e][idx][0], sf), __fmul_rn((float)ot[e][idx][1], sf));
            }
        };
        if constexpr (BITS == 4) {
            constexpr int wd = P / 12, v = P % 12;
            const uint32_t word = ws.w[e][0][wd];
            const h2 kk = h2{(_Float16)1.0f, (_Float16)0.0625f};
            if constexpr (v < 4) {
                const uint32_t pq = v < 2 ? __builtin_amdgcn_perm(word, word, 0x01000100u) : __builtin_amdgcn_perm(word, word, 0x03020302u);
                ot[e][4 * wd + v] = as_h2(and_or((v & 1) ? pq >> 8 : pq, 0x00F0000Fu, kMagic));
            } else if constexpr (v < 8) {
                ot[e][4 * wd + v - 4] = __builtin_elementwise_fma(ot[e][4 * wd + v - 4], kk, gcn[e].zz);
            } else {
                finish(4 * wd + v - 8);
            }
        } else if constexpr (BITS == 2) {
            constexpr int hw = P / 12, v = P % 12;             // half-word hw of the unit's two words
            const uint32_t word = ws.w[e][0][hw / 2];
            const h2 ka = h2{(_Float16)1.0f, (_Float16)0.25f}, kb = h2{(_Float16)0.0625f, (_Float16)0.015625f};
            if constexpr (v < 4) {
                const uint32_t p = (hw & 1) ? __builtin_amdgcn_perm(word, word, 0x03020302u) : __builtin_amdgcn_perm(word, word, 0x01000100u);
                ot[e][4 * hw + v] = as_h2(and_or(v < 2 ? p : p >> 8, (v & 1) ? 0x00C00030u : 0x000C0003u, kMagic));
            } else if constexpr (v < 8) {
                ot[e][4 * hw + v - 4] = __builtin_elementwise_fma(ot[e][4 * hw + v - 4], (v & 1) ? kb : ka, (v & 1) ? gcn[e].zz2 : gcn[e].zz);
            } else {
                finish(4 * hw + v - 8);
            }
        } else {
            constexpr int pr = P / 3, op = P % 3;              // pair pr: bytes 2 (pr % 2), + 1 of word pr / 2
            const uint32_t word = ws.w[e][pr / 8][(pr / 2) % 4];
            if constexpr (op == 0) ot[e][pr] = as_h2(__builtin_amdgcn_perm(0x64646464u, word, (pr & 1) ? 0x04030402u : 0x04010400u));
            else if constexpr (op == 1) ot[e][pr] = ot[e][pr] + gcn[e].zz;
            else finish(pr);
        }
    };
    auto w_store = [&](auto ec, auto qc, char* wt) {          // 16-byte quarter q (pairs 4 q .. 4 q + 3) of unit e
        constexpr int e = decltype(ec)::value, q = decltype(qc)::value;
        char* d = wt + ((q & 2) ? (w_dst[e] ^ 32) : w_dst[e]) + (q & 1) * 16;
        *reinterpret_cast<u4*>(d) = u4{od[e][4 * q], od[e][4 * q + 1], od[e][4 * q + 2], od[e][4 * q + 3]};
    };

    auto step = [&](int s, const char* gcur, char* gnxt, const char* wcur, char* wnxt, WSet& ws, const WSet& wsn) {
        // ws: the words that became wcur a step ago - free, so the requests of step s + 2 land there; wsn: the words of
        // step s + 1, dequantised into wnxt during this step
        __builtin_amdgcn_sched_barrier(0);
        const uint32_t g_a = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) char*)gcur;
        const uint32_t w_a = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) char*)wcur;
        static_for<0, MF>([&](auto tc) {                       // the step's weight fragments, t = 0 first
            constexpr int t = decltype(tc)::value;
            static_for<0, NT>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                lds_read_tr_asm<t * 32 * QK * 2>(wfr[t][j][0], w_a + ta[0] + tp[j]);
                lds_read_tr_asm<t * 32 * QK * 2>(wfr[t][j][1], w_a + ta[1] + tp[j]);
            });
        });
        auto frag_read = [&](auto tc, auto ic) {
            constexpr int t = decltype(tc)::value, i = decltype(ic)::value;
            lds_read_b128_asm<i * 16 * 128>(xf[(MT * t + i) % XRING], g_a + fa[t]);
        };
        static_for<0, XRING>([&](auto Sc) {
            constexpr int S0 = decltype(Sc)::value;
            frag_read(std::integral_constant<int, S0 / MT>{}, std::integral_constant<int, S0 % MT>{});
        });
        static_for<0, MF>([&](auto tc) {
            constexpr int t = decltype(tc)::value;
            static_for<0, NT * MT>([&](auto gcnt) {
                constexpr int g = decltype(gcnt)::value, i = g / NT, j = g % NT;
                constexpr int S = MT * t + i, SLAST = MT * MF - 1 - XRING;
                __builtin_amdgcn_sched_barrier(0);
                // (the 16 weight-fragment reads were issued before the ring reads and return first)
                if constexpr (j == 0) __builtin_amdgcn_s_waitcnt(0xC07F | ((XRING - 1 - (S > SLAST + 1 ? S - SLAST - 1 : 0)) << 8));
                mfma_acc_agpr<DT>(acc[i][j], __builtin_bit_cast(h8, u4{wfr[t][j][0][0], wfr[t][j][0][1], wfr[t][j][1][0], wfr[t][j][1][1]}), xf[S % XRING]);
                __builtin_amdgcn_sched_barrier(0);
                // ---- side work: the first three gaps of a slot take PPG dequantisation pieces each (unit t: MT slots x 3
                // gaps = its 48 pieces), the fourth belongs to the slot's ring read
                if constexpr (j < 3)
                    static_for<0, PPG>([&](auto pp) { piece(std::integral_constant<int, t>{}, std::integral_constant<int, PPG * (3 * i + j) + decltype(pp)::value>{}, wsn); });
                if constexpr (j == 3 && i >= MT - 4) w_store(std::integral_constant<int, t>{}, std::integral_constant<int, i - (MT - 4)>{}, wnxt);
                if constexpr (t == 0 && j == 1 && i < UNITS) g_dma(i, s + 1, gnxt);
                if constexpr (j == NT - 1) {
                    constexpr int S2 = S + XRING;
                    if constexpr (S2 < MT * MF) frag_read(std::integral_constant<int, S2 / MT>{}, std::integral_constant<int, S2 % MT>{});
                }
                asm volatile("" ::: "memory");
            });
        });
        __builtin_amdgcn_sched_barrier(0);
        w_req(s + 2, ws);
        asm volatile("" ::: "memory");
        wait_loads<REQ>();                                    // the next grad_y tile has landed: only the requests just made are out
        lds_barrier();
    };

    // prologue: grad_y tile of the first step, the words of the first two steps, the first weight tile
#pragma unroll
    for (int u = 0; u < UNITS; u++) g_dma(u, s_begin, gbuf[0]);
    w_req(s_begin, set0);
    w_req(s_begin + 1, set1);
    asm volatile("" ::: "memory");
    static_for<0, 2>([&](auto ec) {
        static_for<0, 48>([&](auto pc) { piece(ec, pc, set0); });
        static_for<0, 4>([&](auto qc) { w_store(ec, qc, wbuf[0]); });
    });
    asm volatile("" ::: "memory");
    wait_loads<REQ>();
    lds_barrier();
    // whole passes of two steps (a step past the slice's end multiplies zeros)
    for (int s = s_begin; s < s_end; s += 2) {
        step(s, gbuf[0], gbuf[1], wbuf[0], wbuf[1], set0, set1);
        step(s + 1, gbuf[1], gbuf[0], wbuf[1], wbuf[0], set1, set0);
    }
    // acc[i][j][r] = grad_x[m0 + 16 i + nl][k0 + 64 wave + 16 j + 4 kq + r]
    if (a.splits > 1) {
        float* dst = a.ws + (size_t)blockIdx.x * (QMv * QK) + 64 * wave + 4 * kq;
#pragma unroll
        for (int i = 0; i < MT; i++) {
            if (m0 + 16 * i + nl >= a.M) continue;
#pragma unroll
            for (int j = 0; j < NT; j++) *reinterpret_cast<f4*>(dst + (16 * i + nl) * QK + 16 * j) = acc[i][j];
        }
        return;
    }
    // the wave's QMv x 64 block leaves through its quarter of LDS as whole 128-byte rows
    __builtin_amdgcn_s_waitcnt(0xC07F);
    char* ob = smem + wave * (QMv * 128);
#pragma unroll
    for (int j = 0; j < NT; j++) {
        const int ch = 4 * j + kq;
#pragma unroll
        for (int i = 0; i < MT; i++) {
            const int row = 16 * i + nl;
            const f4 v = acc[i][j];
            *reinterpret_cast<u2*>(ob + row * 128 + (((ch >> 1) ^ (row & 7)) * 16) + (ch & 1) * 8) = u2{pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const bool wide = a.ldx % 8 == 0 && (((uintptr_t)a.gx) & 15) == 0;
#pragma unroll
    for (int q = 0; q < QMv / 8; q++) {
        const int row = 8 * q + (lane >> 3), unit = lane & 7;
        const u4 v = *reinterpret_cast<const u4*>(ob + row * 128 + ((unit ^ (row & 7)) * 16));
        if (m0 + row >= a.M) continue;
        _Float16* dst = a.gx + (int64_t)(m0 + row) * a.ldx + k0 + 64 * wave + unit * 8;
        if (wide) *reinterpret_cast<u4*>(dst) = v;
        else {
            *reinterpret_cast<u2*>(dst) = u2{v[0], v[1]};
            *reinterpret_cast<u2*>(dst + 4) = u2{v[2], v[3]};
        }
    }
}

struct DgradPlan {
    int mt, tiles_k, tiles, splits, steps_per_split;   // mt = 16: the 256 x 256 kernel
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
// The 256 x 256 kernel takes a problem when it is large enough, counted in tile-steps (tiles x steps of 64 rows of n),
// K in whole tiles, N in whole steps, extents that fit the 32-bit offsets of buffer addressing - and, below one
// workgroup per CU, a workspace: N is then cut into slices of at least 8 steps so that every CU has one.  Measured
// against the stepping kernel on 4096 x 4096, 4096 -> 11008 / 14336 and 14336 -> 4096 at 64 ... 4096 rows:
//   256 rows of m per tile: beyond 384 rows from 3072 tile-steps (0.63-0.88 of the stepping kernel's time; at 512 rows
//   level with the 128-row variant for float16 and ahead for bfloat16, whose dequantisation is twice as long);
//   128 rows of m per tile (twice the dequantisation per MFMA, half the padding): up to 512 rows from 2560 tile-steps
//   (0.66-0.96; 4096 x 4096 up to 256 rows - 1024 and 2048 tile-steps - is 1.07-1.11 and stays on the stepping kernel).
// Returns the rows of m per tile (256 or 128), 0 = the stepping kernel.
inline int dgrad256_rows(int64_t M, int64_t N, int64_t K, int64_t ldg, int bits, int group) {
    const int64_t lim = (int64_t)1 << 31;
    if (K % QK || N % QN || N * (K * bits / 8) >= lim || (M + QM) * ldg * 2 >= lim || N * (K / group) * 2 >= lim) return 0;
    const int64_t col_steps = (K / QK) * (N / QN);
    if (M > 384 && ((M + QM - 1) / QM) * col_steps >= 3072) return QM;
    if (M <= 512 && ((M + 127) / 128) * col_steps >= 2560) return 128;
    return 0;
}

inline DgradPlan dgrad256_plan(int64_t M, int64_t N, int64_t K, bool have_workspace, int qm = QM) {
    DgradPlan p;
    p.mt = qm / 16;
    p.tiles_k = (int)(K / QK);
    p.tiles = p.tiles_k * (int)((M + qm - 1) / qm);
    const int nsteps = (int)(N / QN);
    p.splits = 1;
    p.steps_per_split = nsteps;
    p.ws_bytes = 0;
    const int cus = dgrad_cus();
    if (!have_workspace || p.tiles > cus / 2) return p;
    int s = cus / p.tiles;
    if (s > nsteps / 8) s = nsteps / 8;
    if (s > 16) s = 16;
    if (s < 2) return p;
    int sps = (nsteps + s - 1) / s;
    sps += sps & 1;                                          // the loop runs two steps per pass
    s = (nsteps + sps - 1) / sps;
    if (s < 2) return p;
    p.splits = s;
    p.steps_per_split = sps;
    p.ws_bytes = (size_t)p.tiles * s * qm * QK * sizeof(float);
    return p;
}

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

template <int BITS, int GROUP, int DT, int MT = 16>
int launch_dgrad256(DgradArgs a, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    constexpr int QMv = MT * 16;
    const DgradPlan p = dgrad256_plan(a.M, a.N, a.K, workspace != nullptr, QMv);
    if (p.ws_bytes > workspace_bytes) return BW_EWORKSPACE;
    a.ws = (float*)workspace;
    a.tiles_k = p.tiles_k;
    a.splits = p.splits;
    a.steps_per_split = p.steps_per_split;
    a.go_bytes = (uint32_t)((((int64_t)a.M - 1) * a.ldg + a.N) * 2);
    a.w_bytes = (uint32_t)((int64_t)a.N * a.row_bytes);
    a.meta_bytes = (uint32_t)((int64_t)a.N * a.groups * 2);
    auto kern = qdgrad256_kernel<BITS, GROUP, DT, MT>;
    constexpr int lds = 2 * (QMv * QN * 2) + 2 * (QN * QK * 2);
    static uint64_t big_lds_devices = 0;                   // per instantiation
    if (!bw_allow_big_lds(reinterpret_cast<const void*>(kern), big_lds_devices)) return BW_ELAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)(p.tiles * p.splits)), dim3(256), lds, stream, a);
    if (hipGetLastError() != hipSuccess) return BW_ELAUNCH;
    if (p.splits > 1) {
        hipLaunchKernelGGL((qdgrad_reduce_kernel<QMv, DT, QK>), dim3(QMv * QK / 4 / 256, (unsigned)p.tiles), dim3(256), 0, stream, a);
        if (hipGetLastError() != hipSuccess) return BW_ELAUNCH;
    }
    return BW_OK;
}

// which kernel a call gets: the 256 x 256 one (with 256 or 128 rows of m) when the problem is large enough and, where its
// grid would leave CUs idle, a workspace is on offer; 0 = the stepping kernel
inline int dgrad_use256(int64_t M, int64_t N, int64_t K, int64_t ldg, int bits, int group, bool have_workspace) {
    const int rows = dgrad256_rows(M, N, K, ldg, bits, group);
    if (!rows) return 0;
    const int64_t tiles = ((M + rows - 1) / rows) * (K / QK);
    return (have_workspace || tiles > dgrad_cus() / 2) ? rows : 0;
}

#ifdef BW_TUNE
static int g_dgrad_force = 0;                              // measurement builds: 1 = stepping kernel, 16 / 8 = the 256 x 256 kernel with 256 / 128 rows
extern "C" void bw_tune_dgrad_kernel(int kind) { g_dgrad_force = kind; }
#endif

template <int BITS, int GROUP, int DT>
int launch_dgrad(DgradArgs a, void* workspace, size_t workspace_bytes, hipStream_t stream) {
#ifdef BW_TUNE
    if (g_dgrad_force == 16) return launch_dgrad256<BITS, GROUP, DT, 16>(a, workspace, workspace_bytes, stream);
    if (g_dgrad_force == 8) return launch_dgrad256<BITS, GROUP, DT, 8>(a, workspace, workspace_bytes, stream);
    if (g_dgrad_force != 1)
#endif
    if (const int rows = dgrad_use256(a.M, a.N, a.K, a.ldg, BITS, GROUP, workspace != nullptr))
        return rows == QM ? launch_dgrad256<BITS, GROUP, DT, 16>(a, workspace, workspace_bytes, stream)
                          : launch_dgrad256<BITS, GROUP, DT, 8>(a, workspace, workspace_bytes, stream);
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
    // enough for either kernel (the call's own leading dimensions decide between them)
    const size_t a = dgrad_plan(M, N, K, true).ws_bytes;
    const int rows = dgrad256_rows(M, N, K, N, bits, group);
    const size_t b = rows ? dgrad256_plan(M, N, K, true, rows).ws_bytes : 0;
    return a > b ? a : b;
}

// Rows of grad_x a workgroup owns for this shape (with a workspace on offer): 128 or 256 for the kernel that walks N in
// steps of 32 rows, 129 or 257 for the 256 x 256 kernel with 128 or 256 rows of m, 0 where the fused path does not apply.  A diagnostic, and what the
// Python backward asks before it chooses between this kernel and dequantise + library GEMM.
extern "C" int bw_qdgrad_tile_rows(int64_t M, int64_t N, int64_t K, int bits, int group) {
    if (!bw_shape_ok(N, K, bits, group) || !dgrad_fast_shape(M, N, K, N, K, bits, group)) return 0;
    if (const int rows = dgrad_use256(M, N, K, N, bits, group, true)) return rows + 1;
    return M > 512 ? 256 : 128;
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
