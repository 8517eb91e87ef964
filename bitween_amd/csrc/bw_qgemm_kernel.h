// bw_qgemm_kernel.h - the prefill kernel template, its split-K plan and its launcher, shared by the two translation
// units that instantiate it (bw_qgemm.hip: 128-row tiles and the entry points; bw_qgemm_rows.hip: 64- and 256-row
// tiles), so that the instantiations compile in parallel.  Not an interface: everything but GemmArgs and
// bw_launch_gemm_rows has internal linkage.
#pragma once
#include "bw_common.h"

struct GemmArgs {
    const void* x;
    const void* qweight;
    const _Float16* scale;
    const _Float16* zp;
    const _Float16* bias;
    _Float16* y;
    uint32_t x_bytes, w_bytes, meta_bytes;
    int M, N, K, ldx, ldy;
    int groups, nchunks, row_bytes;
    // Grid plan: workgroup ids [0, full_tiles) each own a whole output tile; the remaining ids come in runs of
    // `splits`, each run sharing one tile and cutting K into slices of chunks_per_split chunks whose float32
    // partial tiles go to ws (one BM x BN block per id) for qgemm_reduce_kernel to add up.
    float* ws;
    int tiles_n, full_tiles, splits, chunks_per_split;
    int bm;                                        // rows of a tile: 128 or 256
    // Order of the tiles.  Tile t sits in panel t / (panel * tiles_n) of `panel` m-tiles, n-major inside the panel, so
    // consecutive tiles form blocks a few m-tiles high.  Workgroup ids go to the 8 XCDs round-robin; id i < xcd_tiles (a
    // multiple of 8) takes tile (i % 8) * xcd_tiles / 8 + i / 8: an XCD works through one contiguous eighth of the tile
    // order, and the 32 workgroups it runs together share `panel` activation tiles and 32 / panel weight tiles in its L2
    // instead of every activation tile (plain row-major ids give an XCD every 8th tile: all m-tiles and few n-tiles
    // whenever tiles_n is a multiple of 8).
    int tiles_m, panel, xcd_tiles;
#ifdef BW_TUNE   // measurement builds only: where workgroups 0..255 leave (core-clock ticks, real-time ticks) of their K loop
    unsigned long long* clk;
#endif
};

// 64- and 256-row tiles of the natural-order schedule (bw_qgemm_rows.hip); BW_EUNSUPPORTED for any other `rows`
int bw_launch_gemm_rows(int bits, int group, int rows, const GemmArgs& a, void* workspace, size_t workspace_bytes, hipStream_t stream);

namespace {


constexpr int WAVES = 4, NT = 4, BN = WAVES * NT * 16;   // a wave owns MT x NT MFMA tiles; MT = 8 or 16 (128 or 256 rows)

template <int BITS, int GROUP, int MT = 8, bool NAT = false>
struct GemmCfg {
    static constexpr int BM = MT * 16;
    // A lane takes WL adjacent 16-byte loads of a weight row per K step: VPL consecutive values.  Two loads
    // at 8 bits, so that every format runs 4 or 8 MFMA steps per K step (the per-step costs - barrier,
    // first fragments, scale and zero-point requests - are spread equally thin) and a lane's values never
    // span more than one group of 32.
    static constexpr int WL = BITS == 8 ? 2 : 1;
    // bytes of a lane load: 16, except 8 at 2 bits with 256-row tiles - there a K step is 128 values like at the other
    // widths (a 256-value step of 256 rows of activations would not fit LDS twice)
    static constexpr int LB = (BITS == 2 && NAT) ? 8 : 16;
    static constexpr int VPI = 32 / BITS, VPL = WL * LB * 8 / BITS, CHUNK_K = 4 * VPL, MF = VPL / 8;
    static constexpr int SPL = MF / WL;                          // MFMA steps per lane load
    static constexpr int CHUNK_BYTES = 4 * LB * WL;              // of a packed weight row
    static constexpr int NG = (VPL > GROUP) ? VPL / GROUP : 1;   // groups inside a lane's values
    static constexpr int WPG = 4 * WL / NG;                      // words of a lane's values per group
    // One K step = one group, or two: the scales (zero points) of four (two) consecutive steps are 8 adjacent bytes
    // and can come in one request per tile instead of one per step and lane group (kernel parameter META4; needs rows
    // of scales that start on 4-byte boundaries, i.e. an even number of groups).  SPR = steps per request.
    static constexpr bool CAN_META4 = (CHUNK_K == GROUP || CHUNK_K == 2 * GROUP) && VPL <= GROUP;
    static constexpr int SPR = 4 * GROUP / CHUNK_K, GPS = CHUNK_K / GROUP;   // groups per step (1 or 2)
    // Where the per-step side work sits (each placement measured per format, M = 512 and 2048):
    // EARLY_W: the first weight fragments of a K step are unpacked under the last MFMA step of the step
    // before (else at the start of the step, with the matrix pipe idle);
    // T_STAGE: the MFMA step whose slots move the next chunk's activations to LDS and re-request them.
    // 4 bits: early, last step (3-9 % over start-of-step / first step); 2 bits at group 32: early, last but
    // one (5 %); 8 bits and 2 bits at larger groups were fastest as they were.
    static constexpr bool EARLY_W = BITS == 4 || (BITS == 2 && GROUP == 32);
    static constexpr int T_STAGE = BITS == 4 ? MF - 1 : (BITS == 2 && GROUP == 32) ? MF - 2 : 0;
    static constexpr int PITCH = CHUNK_K + 8;                    // halves per LDS row
    // 128 rows: padded rows written by the staging threads; 256 rows: 256-byte rows written by buffer loads with LDS
    // destination, unpadded, the 16-byte slots of a row XOR-swizzled by the row number instead
    static constexpr int STAGE_BYTES = NAT ? BM * CHUNK_K * 2 : BM * PITCH * 2;
    static constexpr int UNIT = VPI > 8 ? VPI : 8;               // halves permuted together when staging x
    static constexpr int UW = UNIT / 8;
    static constexpr int UPR = CHUNK_K / UNIT;                   // staging units per x row
    static constexpr int XL = BM * UPR / (WAVES * 64);           // staging units per thread (128-row tiles)
    static_assert(BM * UPR % (WAVES * 64) == 0, "tile must split evenly over the workgroup");
    // Activation fragments in registers: 128 rows - two sets of MT, the set of MFMA step t+1 read during step t;
    // 256 rows - a ring of 8, the fragment of slot i + 8 read when slot i has issued its MFMAs.
    static constexpr int XSETS = NAT ? 1 : 2, XRING = NAT ? 8 : MT;
};

template <int BITS>
BW_DEV void permute_unit(const uint32_t* r, uint32_t* o) {
    if constexpr (BITS == 8) {
#pragma unroll
        for (int j = 0; j < 4; j++) o[j] = r[j];
    } else if constexpr (BITS == 4) {
        o[0] = __builtin_amdgcn_perm(r[2], r[0], 0x05040100u);
        o[1] = __builtin_amdgcn_perm(r[2], r[0], 0x07060302u);
        o[2] = __builtin_amdgcn_perm(r[3], r[1], 0x05040100u);
        o[3] = __builtin_amdgcn_perm(r[3], r[1], 0x07060302u);
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++)
            o[j] = __builtin_amdgcn_perm(r[4 + j / 2], r[j / 2], (j & 1) ? 0x07060302u : 0x05040100u);
    }
}

// Unpack word t of a lane load (8 values for MFMA step t at 4 bits; two steps' worth at 2 bits, half a
// step at 8 bits is handled by the caller) - thin wrappers so the K loop can unpack just in time.
template <int BITS>
BW_DEV h8 unpack_step(const u4& w, int t, const GroupConst<BITS>* gc, int ng_words) {
    h2 o[8];
    if constexpr (BITS == 4) {
        dequant_word4<true>(w[t], gc[t / ng_words], o);
        return pack_h8(o);
    } else if constexpr (BITS == 8) {
        dequant_word8<true>(w[2 * t], gc[(2 * t) / ng_words], o);
        dequant_word8<true>(w[2 * t + 1], gc[(2 * t + 1) / ng_words], o + 2);
        return pack_h8(o);
    } else {
        dequant_word2<true>(w[t / 2], gc[(t / 2) / ng_words], o);
        return pack_h8(o + 4 * (t & 1));
    }
}

// The 128 accumulator registers of a wave live in the accumulation register file (AGPRs), leaving all 256
// architectural VGPRs for operands and prefetch.  The compiler only selects the AGPR form of an MFMA when
// asked through the operand constraint, hence the inline assembly.  Software-visible hazards of this
// instruction on gfx950 concern reads of the result by non-MFMA instructions; the only such reads are in
// the epilogue, hundreds of cycles (an LDS staging pass and a barrier) after the last MFMA.
BW_DEV void mfma_acc(f4& acc, const h8& a, const h8& b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

// 16 bytes per lane from LDS byte address `addr` + OFF, as an instruction the compiler does not know to be an LDS read
// (its result is ready only after an s_waitcnt lgkmcnt the caller places).
template <int OFF>
BW_DEV void lds_read_b128(h8& dst, uint32_t addr) {
    static_assert(OFF >= 0 && OFF < 65536, "16-bit offset field");
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}

BW_DEV void tile_coords(int tile, const GemmArgs& a, int& tm, int& tn) {
    const int per_panel = a.panel * a.tiles_n;
    const int p = tile / per_panel, within = tile - p * per_panel;
    const int rows = min(a.panel, a.tiles_m - p * a.panel);
    tn = within / rows;
    tm = p * a.panel + (within - tn * rows);
}

BW_DEV __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), (short)0, (int)bytes, 0x00020000);
}

// Software pipeline, one K step = one chunk:
//   step c computes from LDS buffer c&1 and the weight register set c&1 (two sets, used alternately and
//   never copied);
//   the activations of chunk c+1 were requested one step earlier and are written to buffer (c+1)&1 during
//   step c, then re-requested for chunk c+2; the weights of chunk c+2 are requested into step c's own set
//   once its last fragment is unpacked.  Every global load has a full K step (~2000 MFMA cycles) to land.
template <int BITS, int GROUP, bool WIDE_META, int MT, bool NAT>
__global__ __launch_bounds__(WAVES * 64) void qgemm_kernel(const GemmArgs a) {
    static_assert(MT == 8 || (NAT && (MT == 4 || MT == 16)), "64- and 256-row tiles exist with the natural-order schedule only");
    using C = GemmCfg<BITS, GROUP, MT, NAT>;
    constexpr int BM = C::BM;
    // WIDE_META (rows of scales on 4-byte boundaries): META4 = 8-byte requests over runs of K steps; PAIR = a lane whose
    // values span two groups fetches both scales (zero points) with one 4-byte request instead of two 2-byte ones
    constexpr bool META4 = WIDE_META && C::CAN_META4, PAIR = WIDE_META && !C::CAN_META4 && C::NG == 2;
    constexpr uint32_t kOob = 0x80000000u;
    extern __shared__ __attribute__((aligned(16))) char smem[];
#ifdef BW_TUNE
    const unsigned long long clk_c0 = clock64(), clk_r0 = wall_clock64();
#endif
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nl = lane & 15, kq = lane >> 4;
    const int id = (int)blockIdx.x;
    const bool partial = id >= a.full_tiles;
    const int run = partial ? id - a.full_tiles : 0;
    const int tile = partial ? a.full_tiles + run / a.splits : id < a.xcd_tiles ? (id & 7) * (a.xcd_tiles >> 3) + (id >> 3) : id;
    int tm, tn;
    tile_coords(tile, a, tm, tn);
    const int m0 = tm * BM;
    const int n0 = tn * BN + wave * (NT * 16);
    const int groups = a.groups;
    // a partial workgroup takes chunks [c_begin, c_end); requests beyond c_end read as zero
    const int c_begin = partial ? (run % a.splits) * a.chunks_per_split : 0;
    const int c_end = partial ? min(a.nchunks, c_begin + a.chunks_per_split) : a.nchunks;
    const __amdgpu_buffer_rsrc_t rw = make_rsrc(a.qweight, a.w_bytes), rx = make_rsrc(a.x, a.x_bytes);

    const __amdgpu_buffer_rsrc_t rs = make_rsrc(a.scale, a.meta_bytes), rz = make_rsrc(a.zp, a.meta_bytes);
    uint32_t w_off[NT], m_off[NT];
#pragma unroll
    for (int j = 0; j < NT; j++) {
        const int row = n0 + 16 * j + nl;
        // (256-row tiles add a scalar chunk offset that is itself "out of range" past the last chunk: rows past N then
        // read the last row's bytes instead of relying on a sum that could wrap; their outputs are never stored)
        w_off[j] = row < a.N ? (uint32_t)row * a.row_bytes + kq * C::LB * C::WL : NAT ? (uint32_t)(a.N - 1) * a.row_bytes + kq * C::LB * C::WL : kOob;
        m_off[j] = (uint32_t)min(row, a.N - 1) * groups * 2;
    }
    // 128-row tiles: byte offsets of the staging units of a thread
    uint32_t x_off[C::XL];
#pragma unroll
    for (int i = 0; i < C::XL; i++) {
        const int u = tid + i * WAVES * 64, m = u / C::UPR, ku = u - m * C::UPR;
        x_off[i] = (m0 + m < a.M) ? (uint32_t)((m0 + m) * a.ldx + ku * C::UNIT) * 2 : kOob;
    }

    u4 xr[C::XL * C::UW];
    // Two weight register sets, used alternately by even and odd K steps and never copied: a register move
    // of an outstanding load would stall on it.
    struct WSet { u4 w[NT][C::WL]; uint32_t s[NT][C::NG], z[NT][C::NG]; };   // 16-bit values, one register each
    WSet set0, set1;
    u2 m_cur[NT][2], m_next[NT][2];                               // META4: [tile][scales, zero points] of 4 steps

    f4 acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < NT; j++) acc[i][j] = f4{0.f, 0.f, 0.f, 0.f};

    // Pieces of the staging / issue work, one per m-tile index, so they can be slotted between MFMA groups.
    auto stage_unit = [&](int i, _Float16* xs) {
        const int u = tid + i * WAVES * 64, m = u / C::UPR, ku = u - m * C::UPR;
        uint32_t in[4 * C::UW], o[4 * C::UW];
#pragma unroll
        for (int j = 0; j < C::UW; j++) { in[4 * j] = xr[i * C::UW + j][0]; in[4 * j + 1] = xr[i * C::UW + j][1]; in[4 * j + 2] = xr[i * C::UW + j][2]; in[4 * j + 3] = xr[i * C::UW + j][3]; }
        permute_unit<BITS>(in, o);
        u4* dst = reinterpret_cast<u4*>(xs + m * C::PITCH + ku * C::UNIT);
#pragma unroll
        for (int j = 0; j < C::UW; j++) dst[j] = u4{o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]};
    };
    auto issue_x_unit = [&](int i, int c) {
        const int ku = (tid + i * WAVES * 64) % C::UPR;
        const uint32_t off = (c < c_end && c * C::CHUNK_K + ku * C::UNIT < a.K) ? x_off[i] + (uint32_t)c * C::CHUNK_K * 2 : kOob;
#pragma unroll
        for (int j = 0; j < C::UW; j++) xr[i * C::UW + j] = __builtin_amdgcn_raw_buffer_load_b128(rx, off + j * 16, 0, 0);
    };
    auto issue_w_load = [&](int j, int l, int c, WSet& ws) {
        const int b = c * C::CHUNK_BYTES + l * 16;
        const bool in = c < c_end && b + kq * 16 * C::WL < a.row_bytes;
        ws.w[j][l] = __builtin_amdgcn_raw_buffer_load_b128(rw, in ? w_off[j] + b : kOob, 0, 0);
    };
    auto issue_meta = [&](int j, int which, int c, WSet& ws) {   // which: 0 = scales, 1 = zero points
        const int g0 = min((c * C::CHUNK_K + kq * C::VPL) / GROUP, groups - C::NG);
        if constexpr (PAIR) {                                       // g0 is even: both entries in one aligned word
            if (which == 0) ws.s[j][0] = __builtin_amdgcn_raw_buffer_load_b32(rs, m_off[j] + g0 * 2, 0, 0);
            else ws.z[j][0] = __builtin_amdgcn_raw_buffer_load_b32(rz, m_off[j] + g0 * 2, 0, 0);
            return;
        }
#pragma unroll
        for (int g = 0; g < C::NG; g++) {
            if (which == 0) ws.s[j][g] = __builtin_amdgcn_raw_buffer_load_b16(rs, m_off[j] + (g0 + g) * 2, 0, 0);
            else ws.z[j][g] = __builtin_amdgcn_raw_buffer_load_b16(rz, m_off[j] + (g0 + g) * 2, 0, 0);
        }
    };
    // Scales (zero points) of steps c .. c+3.  Past the row's last group this reads the next row's (or zero past
    // the buffer); no step that runs ever uses those: a META4 launch has an even group count and even slices, so
    // the K loop below never pads with a zero step, and what the last step prepares for its successor is dropped.
    auto issue_meta4 = [&](int j, int which, int c, u2 (*m)[2]) {
        m[j][which] = __builtin_amdgcn_raw_buffer_load_b64(which == 0 ? rs : rz, m_off[j] + c * (2 * C::GPS), 0, 0);
    };
    // Weight fragment of MFMA step t: values [8 t, 8 t + 8) of the lane's VPL, from lane load t / SPL.
    auto unpack = [&](const WSet& ws, int j, int t, const auto* gcj) {
        static_assert(C::WL == 1 || C::NG == 1, "two lane loads share one group");
        if constexpr (NAT) {                                  // natural k order
            h2 o[4];
            if constexpr (BITS == 4) {
                dequant_word4_nat(ws.w[j][0][t], gcj[0], o);
            } else if constexpr (BITS == 2) {
                dequant_halfword2_nat(ws.w[j][0][t / 2], t % 2, gcj[0], o);
            } else {
#pragma unroll
                for (int e = 0; e < 2; e++) {
                    const uint32_t w = ws.w[j][t / C::SPL][2 * (t % C::SPL) + e];
                    o[2 * e] = (as_h2(__builtin_amdgcn_perm(0x64646464u, w, 0x04010400u)) + gcj[0].zz) * gcj[0].s;
                    o[2 * e + 1] = (as_h2(__builtin_amdgcn_perm(0x64646464u, w, 0x04030402u)) + gcj[0].zz) * gcj[0].s;
                }
            }
            return pack_h8(o);
        } else {
            return unpack_step<BITS>(ws.w[j][t / C::SPL], t % C::SPL, gcj, C::WPG);
        }
    };

    // One K step.  The 32 MFMAs of MFMA step t are issued in groups of 4 (one m-tile); between two groups
    // sits one slice of other work, fenced so the compiler keeps it there: the LDS read of one activation
    // fragment and (every other slot) the unpack of one weight fragment of MFMA step t+1 - with EARLY_W the last
    // MFMA step prepares the first fragment of the NEXT K step, from the other register set, so that a step starts
    // with its weight fragments ready - plus the staging and global requests listed at slot_requests below.
    // Requests past the last chunk are range-checked to zero by the hardware; no branches, so every wait
    // count is exact.
    // `ph` (META4 only): position of the step in its run of four, a constant after inlining.
    static_assert(C::MF % 2 == 0, "the fragment double buffer returns to slot 0 at the end of a step");
    using GC = std::conditional_t<NAT, GroupConstNat<BITS>, GroupConst<BITS>>;
    h8 xf[C::XSETS][C::XRING];
    h2 wf[2][NT][4];                                      // weight fragments as 4 register pairs each
    // group constants of tile j for the step that reads `from` (META4: half `half` of m_cur / m_next)
    auto set_consts = [&](GC* gj, int j, const WSet& from, const u2 (*m)[2], int half) {
#pragma unroll
        for (int g = 0; g < C::NG; g++) {
            if constexpr (META4 && C::GPS == 1)
                gj[g].set(__builtin_bit_cast(_Float16, (uint16_t)(m[j][0][half >> 1] >> (16 * (half & 1)))),
                          __builtin_bit_cast(_Float16, (uint16_t)(m[j][1][half >> 1] >> (16 * (half & 1)))));
            else if constexpr (META4)                            // two groups per step: lanes kq >= 2 take the second
                gj[g].set(__builtin_bit_cast(_Float16, (uint16_t)(m[j][0][half] >> (16 * (kq >> 1)))),
                          __builtin_bit_cast(_Float16, (uint16_t)(m[j][1][half] >> (16 * (kq >> 1)))));
            else if constexpr (PAIR)
                gj[g].set(__builtin_bit_cast(_Float16, (uint16_t)(from.s[j][0] >> (16 * g))), __builtin_bit_cast(_Float16, (uint16_t)(from.z[j][0] >> (16 * g))));
            else
                gj[g].set(__builtin_bit_cast(_Float16, (uint16_t)from.s[j][g]), __builtin_bit_cast(_Float16, (uint16_t)from.z[j][g]));
        }
    };
    auto step8 = [&](int c, const _Float16* cur, _Float16* nxt, WSet& ws, const WSet& wsn, auto& gc, auto& gn, const int ph) {
        static_assert(C::XL <= MT && NT * 2 == MT, "at most one staging unit and half a weight tile per m-tile slot");
        __builtin_amdgcn_sched_barrier(0);
        const _Float16* xp = cur + nl * C::PITCH + kq * C::VPL;
#pragma unroll
        for (int i = 0; i < MT; i++) xf[0][i] = *reinterpret_cast<const h8*>(xp + i * 16 * C::PITCH);
        if constexpr (!C::EARLY_W) {
#pragma unroll
            for (int j = 0; j < NT; j++) {
                set_consts(gc[j], j, ws, m_cur, ph);
                const h8 f = unpack(ws, j, 0, gc[j]);
#pragma unroll
                for (int e = 0; e < 4; e++) wf[0][j][e] = h2{f[2 * e], f[2 * e + 1]};
            }
        }
        // At most one global request per slot, spread over the K step: a burst of requests backs up
        // the address unit and the wave - which issues in order - stops feeding MFMAs.
        //   second MFMA step  : scales and zero points (for chunk c+2, or for the next run of four steps)
        //   MFMA step T_STAGE : activations of chunk c+1 (requested a step ago) to LDS, re-request for c+2
        //   last MFMA step    : weights for chunk c+2 (their registers are free after the last unpack).
        // The last MFMA step reads no fragments of its own K step, which is why the 4-bit staging fits there.
        auto slot_requests = [&](int t, int i) {
            static_assert(C::MF >= 4, "second and last MFMA step are distinct");
            if constexpr (META4) {
                if (t == 1 && ph == 0) issue_meta4(i / 2, i & 1, c + C::SPR, m_next);
            } else {
                if (t == 1) issue_meta(i / 2, i & 1, c + 2, ws);
            }
            if (t == C::T_STAGE && i < C::XL) {
                stage_unit(i, nxt);
                issue_x_unit(i, c + 2);
            }
            if (t == C::MF - 1 && (C::WL == 2 || !(i & 1))) issue_w_load(i / 2, C::WL == 2 ? (i & 1) : 0, c + 2, ws);
            asm volatile("" ::: "memory");
        };
        auto next_consts = [&](int j) {
            if constexpr (META4) set_consts(gn[j], j, wsn, ph < C::SPR - 1 ? m_cur : m_next, ph < C::SPR - 1 ? ph + 1 : 0);
            else set_consts(gn[j], j, wsn, m_cur, 0);
        };
#pragma unroll
        for (int t = 0; t < C::MF; t++) {
            const int cu = t & 1, nx = cu ^ 1;
            const bool last = t == C::MF - 1, early = last && C::EARLY_W;
#pragma unroll
            for (int i = 0; i < MT; i++) {
                if constexpr (BITS == 4) {
                    // An MFMA occupies the matrix pipe for 16 cycles but the issue port for 4: two or three
                    // VALU operations fit behind each one.  Slot i prepares half a weight fragment of
                    // the next MFMA step (tile i/2, words' low or high byte pair) in four such pieces.
                    const int jn = i / 2;
                    if (early && !(i & 1)) {
                        __builtin_amdgcn_sched_barrier(0);
                        next_consts(jn);
                    }
                    const GroupConst<4>& g4 = early ? gn[jn][0] : gc[jn][(last ? t : t + 1) / C::WPG];
                    const uint32_t word = early ? wsn.w[jn][0][0] : ws.w[jn][0][last ? t : t + 1];
                    const h2 k16 = splat((_Float16)0.0625f);
                    uint32_t wsrc = 0;
                    h2 pa = {0, 0}, pb = {0, 0};
#pragma unroll
                    for (int j = 0; j < NT; j++) {
                        __builtin_amdgcn_sched_barrier(0);
                        mfma_acc(acc[i][j], pack_h8(wf[cu][j]), xf[cu][i]);
                        __builtin_amdgcn_sched_barrier(0);
                        if (!last || early) {
                            if (j == 0) {
                                if (!last) xf[nx][i] = *reinterpret_cast<const h8*>(xp + i * 16 * C::PITCH + 8 * (t + 1));
                                wsrc = (i & 1) ? word >> 8 : word;
                                pa = as_h2(and_or(wsrc, 0x000F000Fu, kMagic));
                            } else if (j == 1) {
                                pb = as_h2(and_or(wsrc, 0x00F000F0u, kMagic));
                                pa = pa + g4.z0;
                            } else if (j == 2) {
                                pb = __builtin_elementwise_fma(pb, k16, g4.z1);
                                pa = pa * g4.s;
                            } else {
                                pb = pb * g4.s;
                                wf[nx][jn][2 * (i & 1)] = pa;
                                wf[nx][jn][2 * (i & 1) + 1] = pb;
                            }
                        }
                        if (j == NT - 1) slot_requests(t, i);
                    }
                } else {
                    __builtin_amdgcn_sched_barrier(0);
                    // weights as the A operand: the result fragment holds 4 consecutive n per lane
#pragma unroll
                    for (int j = 0; j < NT; j++) mfma_acc(acc[i][j], pack_h8(wf[cu][j]), xf[cu][i]);
                    __builtin_amdgcn_sched_barrier(0);
                    if (!last) xf[nx][i] = *reinterpret_cast<const h8*>(xp + i * 16 * C::PITCH + 8 * (t + 1));
                    if (!(i & 1)) {
                        if (early) next_consts(i / 2);
                    } else if (!last || early) {
                        const h8 f = early ? unpack(wsn, i / 2, 0, gn[i / 2]) : unpack(ws, i / 2, t + 1, gc[i / 2]);
#pragma unroll
                        for (int e = 0; e < 4; e++) wf[nx][i / 2][e] = h2{f[2 * e], f[2 * e + 1]};
                    }
                    slot_requests(t, i);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
    };

    // ---- One K step of the 256-row tile --------------------------------------------------------------------------
    // A wave issues in order, and what it can put between two MFMAs without holding up the matrix pipe is about one
    // VALU instruction plus one other (measured: 16 cycles per MFMA with one, 19 with two, 20 with three; LDS, scalar
    // and wait instructions cost 1-2 each).  So the side work of an MFMA step is cut into single instructions and dealt
    // out one per gap, by position: gap g = 4 i + j follows the MFMA of m-tile i and n-tile j; region r = g / 16 and
    // k = g % 16 name the 16 gaps of four slots.
    //   unpack      : n-tile r's fragment for the next MFMA step, 16 instructions at 4 bits and 12 at 8, in the first
    //                 three gaps of the region's slots (placement below); the last MFMA step prepares the first
    //                 fragment of the next K step from the other set;
    //   activations : the next chunk's 256 x 128 tile goes memory -> LDS by buffer loads with LDS destination, 16 per
    //                 wave (4 rows of 256 bytes each), one per slot of the first MFMA step so that they have three more
    //                 to land; no registers, no permute, and nothing the matrix pipe waits for;
    //   fragments   : slot i's last gap reads the activation fragment of slot i + 8 into the ring;
    //   requests    : scales / zero points in the second MFMA step, weights in the last, group constants of the next
    //                 step in the last but one.
    // LDS row r of a buffer holds the chunk's 16-byte slot q of x row r at slot q ^ (r & 7): a lane group of 16 rows
    // reading one slot then spreads over all banks (rows are 256 bytes apart: unswizzled they would share 4 banks).
    // The fragment reads are written as assembly: the compiler orders every LDS read it knows of behind all pending
    // loads with LDS destination, and would so wait for the next chunk before reading this one.  It does not track
    // assembly results either, so the waits are here too: fragment reads complete in order and nothing else uses LDS
    // in the loop, so before slot S of a K step (S = 16 t + i) at most 7 - max(0, S - 56) younger reads are in flight.
    // Request addresses are one VGPR per thread plus a scalar: the chunk part of an offset is uniform, and past the
    // slice it is replaced by an offset beyond every buffer, so that the hardware's range check returns zeros.
    // Requires K % CHUNK_K == 0 (the launcher's condition for this variant): no request straddles the end of a row.
    h2 up[NT][4];
    uint32_t uw[NT], pq[NT][2];
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    // activation loads: a wave brings in BM / 4 rows, 4 per instruction: unit u = rows RW wave + 4 u + (lane >> 4), lane & 15 = LDS slot
    constexpr int RW = BM / WAVES;
    uint32_t xd_base[2];
#pragma unroll
    for (int par = 0; par < 2; par++) {
        const int rr = 4 * par + (lane >> 4);
        xd_base[par] = (uint32_t)((m0 + RW * wave + rr) * a.ldx) * 2 + (((lane & 15) ^ (rr & 7)) * 16);
    }
    auto x_dma16 = [&](int u, int cc, char* buf) {
        uint32_t so = cc < c_end ? (uint32_t)((u >> 1) * 8 * a.ldx) * 2 + (uint32_t)cc * C::CHUNK_K * 2 : kOob;
        asm("" : "+s"(so));                                   // one scalar sum, one VALU add
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (__attribute__((address_space(3))) void*)(buf + (RW * wave_u + 4 * u) * 256), 16,
                                                 xd_base[u & 1] + so, 0, 0, 0);
    };
    auto w_req16 = [&](int j, int l, int cc, WSet& ws) {
        const uint32_t so = cc < c_end ? (uint32_t)cc * C::CHUNK_BYTES + l * 16 : kOob;
        if constexpr (C::LB == 8) {
            const u2 v = __builtin_amdgcn_raw_buffer_load_b64(rw, w_off[j] + so, 0, 0);
            ws.w[j][l][0] = v[0];
            ws.w[j][l][1] = v[1];
        } else {
            ws.w[j][l] = __builtin_amdgcn_raw_buffer_load_b128(rw, w_off[j] + so, 0, 0);
        }
    };
    // fragment (m-tile i, MFMA step t) of the lane: slot 4 kq + t of row 16 i + nl, swizzled
    uint32_t fa[4];
#pragma unroll
    for (int t = 0; t < 4; t++) fa[t] = (uint32_t)(nl * 256 + (((4 * kq + t) ^ (nl & 7)) * 16));
    auto step16 = [&](int c, const char* cur, char* nxt, WSet& ws, const WSet& wsn, auto& gc, auto& gn, const int ph, const bool tail) {
        static_assert(!NAT || (C::NG == 1 && C::MF == 4 && C::CHUNK_K == 128 && C::XRING == 8), "layout of the natural-order schedule");
        __builtin_amdgcn_sched_barrier(0);
        const uint32_t cur_a = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) char*)cur;
        auto frag_read = [&](auto tc, auto ic) {
            constexpr int t = decltype(tc)::value, i = decltype(ic)::value;
            lds_read_b128<i * 16 * 256>(xf[0][(MT * t + i) % C::XRING], cur_a + fa[t]);
        };
        static_for<0, C::XRING>([&](auto sc) {                 // the first XRING slots of the step: slot S = MT t + i
            constexpr int S0 = decltype(sc)::value;
            frag_read(std::integral_constant<int, S0 / MT>{}, std::integral_constant<int, S0 % MT>{});
        });
        const h2 k16 = h2{(_Float16)1.0f, (_Float16)0.0625f};
        const h2 k2a = h2{(_Float16)1.0f, (_Float16)0.25f}, k2b = h2{(_Float16)0.0625f, (_Float16)0.015625f};
        static_for<0, C::MF>([&](auto tc) {
            constexpr int t = decltype(tc)::value, cu = t & 1, nx = cu ^ 1;
            constexpr bool early = t == C::MF - 1;
            const WSet& src = early ? wsn : ws;
            constexpr int tt = early ? 0 : t + 1;
            static_for<0, 4 * MT>([&](auto gcnt) {
                // RG gaps (SLOTS slots) per region: 16 (4) with 256-row tiles, 8 (2) with 128-row tiles
                constexpr int RG = 4 * MT / NT, SLOTS = RG / 4;
                constexpr int g = decltype(gcnt)::value, i = g / NT, j = g % NT, r = g / RG, k = g % RG;
                constexpr int S = MT * t + i, SLAST = MT * C::MF - 1 - C::XRING;          // SLAST: the last slot that issues a fragment read
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (j == 0) __builtin_amdgcn_s_waitcnt(0xC07F | ((C::XRING - 1 - (S > SLAST + 1 ? S - SLAST - 1 : 0)) << 8));
                mfma_acc(acc[i][j], pack_h8(wf[cu][j]), xf[0][(MT * t + i) % C::XRING]);
                __builtin_amdgcn_sched_barrier(0);
                // ---- unpack of n-tile r: instruction v of its sequence ----
                const auto& gr = early ? gn[r][0] : gc[r][0];
                auto unpack_op = [&](auto vc) {
                    constexpr int v = decltype(vc)::value;
                    if constexpr (BITS == 4) {
                        const uint32_t word = src.w[r][0][tt];
                        if constexpr (v == 0) pq[r][0] = __builtin_amdgcn_perm(word, word, 0x01000100u);
                        if constexpr (v == 1) pq[r][1] = __builtin_amdgcn_perm(word, word, 0x03020302u);
                        if constexpr (v == 2) up[r][0] = as_h2(and_or(pq[r][0], 0x00F0000Fu, kMagic));
                        if constexpr (v == 3) uw[r] = pq[r][0] >> 8;
                        if constexpr (v == 4) up[r][1] = as_h2(and_or(uw[r], 0x00F0000Fu, kMagic));
                        if constexpr (v == 5) up[r][2] = as_h2(and_or(pq[r][1], 0x00F0000Fu, kMagic));
                        if constexpr (v == 6) uw[r] = pq[r][1] >> 8;
                        if constexpr (v == 7) up[r][3] = as_h2(and_or(uw[r], 0x00F0000Fu, kMagic));
                        if constexpr (v >= 8 && v < 12) up[r][v - 8] = __builtin_elementwise_fma(up[r][v - 8], k16, gr.zz);
                        if constexpr (v >= 12) wf[nx][r][v - 12] = up[r][v - 12] * gr.s;
                    } else if constexpr (BITS == 2) {
                        // half-word tt of the lane's 8 bytes
                        const uint32_t word = src.w[r][0][tt / 2];
                        if constexpr (v == 0) pq[r][0] = tt % 2 ? __builtin_amdgcn_perm(word, word, 0x03020302u) : __builtin_amdgcn_perm(word, word, 0x01000100u);
                        if constexpr (v == 1) uw[r] = pq[r][0] >> 8;
                        if constexpr (v == 2) up[r][0] = as_h2(and_or(pq[r][0], 0x000C0003u, kMagic));
                        if constexpr (v == 3) up[r][1] = as_h2(and_or(pq[r][0], 0x00C00030u, kMagic));
                        if constexpr (v == 4) up[r][2] = as_h2(and_or(uw[r], 0x000C0003u, kMagic));
                        if constexpr (v == 5) up[r][3] = as_h2(and_or(uw[r], 0x00C00030u, kMagic));
                        if constexpr (v >= 6 && v < 10) up[r][v - 6] = __builtin_elementwise_fma(up[r][v - 6], (v & 1) ? k2b : k2a, (v & 1) ? gr.zz2 : gr.zz);
                        if constexpr (v >= 10 && v < 14) wf[nx][r][v - 10] = up[r][v - 10] * gr.s;
                    } else {
                        // 8 bits: the two words of MFMA step tt are words 2 (tt % 2), + 1 of lane load tt / 2
                        const uint32_t w0 = src.w[r][tt / C::SPL][2 * (tt % C::SPL)], w1 = src.w[r][tt / C::SPL][2 * (tt % C::SPL) + 1];
                        if constexpr (v == 0) up[r][0] = as_h2(__builtin_amdgcn_perm(0x64646464u, w0, 0x04010400u));
                        if constexpr (v == 1) up[r][1] = as_h2(__builtin_amdgcn_perm(0x64646464u, w0, 0x04030402u));
                        if constexpr (v == 2) up[r][2] = as_h2(__builtin_amdgcn_perm(0x64646464u, w1, 0x04010400u));
                        if constexpr (v == 3) up[r][3] = as_h2(__builtin_amdgcn_perm(0x64646464u, w1, 0x04030402u));
                        if constexpr (v >= 4 && v < 8) up[r][v - 4] = up[r][v - 4] + gr.zz;
                        if constexpr (v >= 8 && v < 12) wf[nx][r][v - 8] = up[r][v - 8] * gr.s;
                    }
                };
                // A gap holds VALU work or the slot's fragment read, not both (measured: one VALU instruction in each of
                // a slot's four gaps plus the read costs 8.4 ns per MFMA, the read in a gap of its own 7.0 = the bare
                // MFMA rate; a second VALU instruction in a gap costs 3 cycles).  So the last gap of a slot belongs to the
                // read; 8 bits puts its 12 instructions one into each other gap, 4 bits its 16 two into the first gap
                // of each slot and one into the next two.
                // With 128-row tiles a region has two slots for the same instructions: twice as many per gap (8 bits: two in
                // each of the first three gaps; 4 and 2 bits: three, three and two, the read's gap still free).
                constexpr int sl = k / 4;                                  // slot of the region
                constexpr int OPS = BITS == 8 ? 12 : 16, PER_SLOT = OPS / SLOTS;          // (2 bits: 14 of the 16 do something)
                // instructions of a slot in its gaps 0, 1, 2: PER_SLOT = 3 -> 1 1 1, 4 -> 2 1 1, 6 -> 2 2 2, 8 -> 3 3 2
                // (64-row tiles, one slot per region: 12 -> 4 4 4, 16 -> 6 5 5)
                constexpr int n0 = PER_SLOT == 3 ? 1 : PER_SLOT == 8 ? 3 : PER_SLOT == 12 ? 4 : PER_SLOT == 16 ? 6 : 2,
                              n1 = PER_SLOT <= 4 ? 1 : PER_SLOT == 8 ? 3 : PER_SLOT == 12 ? 4 : PER_SLOT == 16 ? 5 : 2;
                constexpr int first = sl * PER_SLOT + (j == 0 ? 0 : j == 1 ? n0 : n0 + n1);
                constexpr int count = j == 0 ? n0 : j == 1 ? n1 : j == 2 ? PER_SLOT - n0 - n1 : 0;
                static_for<0, count>([&](auto oc) { unpack_op(std::integral_constant<int, first + decltype(oc)::value>{}); });
                // ---- the next chunk's activations: unit i of the wave in slot i of the first MFMA step ----
                if constexpr (t == 0 && j == 1) x_dma16(i, c + 1, nxt);
                // ---- fragment ring ----
                if constexpr (j == NT - 1) {
                    constexpr int i2 = (i + C::XRING) % MT, t2 = t + (i + C::XRING) / MT;
                    if constexpr (t2 < C::MF) frag_read(std::integral_constant<int, t2>{}, std::integral_constant<int, i2>{});
                }
                // ---- requests and constants (second gap of a slot) ----
                // two requests per region: slots 2 and 3 of four (second gap), or gaps 1 and 2 of the second slot of two
                constexpr bool meta_here = SLOTS == 4 ? (j == 1 && sl >= 2) : (sl == SLOTS - 1 && (j == 1 || j == 2));
                if constexpr (t == 1 && meta_here) {
                    constexpr int which = SLOTS == 4 ? sl - 2 : j - 1;
                    if constexpr (META4) {
                        if (ph == 0) issue_meta4(r, which, c + C::SPR, m_next);
                    } else {
                        issue_meta(r, which, c + 2, ws);
                    }
                }
                if constexpr (t == C::MF - 2 && k == RG - 2) {
                    if constexpr (META4) set_consts(gn[r], r, wsn, ph < C::SPR - 1 ? m_cur : m_next, ph < C::SPR - 1 ? ph + 1 : 0);
                    else set_consts(gn[r], r, wsn, m_cur, 0);
                }
                if constexpr (SLOTS == 4) {
                    if constexpr (t == C::MF - 1 && j == 1 && sl >= 4 - C::WL) w_req16(r, sl - (4 - C::WL), c + 2, ws);
                } else {                                                   // two slots: gaps 1 (and 2 at 8 bits) of the second
                    if constexpr (t == C::MF - 1 && sl == SLOTS - 1 && j >= 1 && j <= C::WL) w_req16(r, j - 1, c + 2, ws);
                }
                asm volatile("" ::: "memory");
            });
        });
        __builtin_amdgcn_sched_barrier(0);
        // this wave's rows of the next chunk are in LDS once only the requests made after them are still in flight:
        // the weights of the last MFMA step and, in a step that made them, the scales and zero points.  That count
        // holds inside the K loop, where every request feeds a later iteration; in the steps after the loop the
        // compiler drops the requests nothing reads any more, so those steps wait for everything.
        if (tail) wait_loads<0>();
        else if ((META4 && ph != 0)) wait_loads<NT * C::WL>();
        else wait_loads<NT * C::WL + 2 * NT>();
        lds_barrier();
    };
    auto step = [&](int c, _Float16* cur, _Float16* nxt, WSet& ws, const WSet& wsn, GC (&gc)[NT][C::NG], GC (&gn)[NT][C::NG],
                    const int ph, const bool tail = false) {
        if constexpr (NAT) step16(c, reinterpret_cast<const char*>(cur), reinterpret_cast<char*>(nxt), ws, wsn, gc, gn, ph, tail);
        else step8(c, cur, nxt, ws, wsn, gc, gn, ph);
    };

    _Float16* buf0 = reinterpret_cast<_Float16*>(smem);
    _Float16* buf1 = reinterpret_cast<_Float16*>(smem + C::STAGE_BYTES);
    if constexpr (NAT) {
        // Prologue of the 256-row tile: chunk c_begin's activations to the first buffer; scales and zero points and
        // the weights of the first two chunks in the order a steady-state step finds them outstanding.
        if constexpr (META4) {
#pragma unroll
            for (int j = 0; j < NT; j++) {
                issue_meta4(j, 0, c_begin, m_cur);
                issue_meta4(j, 1, c_begin, m_cur);
            }
        }
#pragma unroll
        for (int u = 0; u < MT; u++) x_dma16(u, c_begin, smem);
#pragma unroll
        for (int b = 0; b < 2; b++) {
            WSet& ws = b ? set1 : set0;
            if constexpr (!META4) {
#pragma unroll
                for (int j = 0; j < NT; j++) {
                    issue_meta(j, 0, c_begin + b, ws);
                    issue_meta(j, 1, c_begin + b, ws);
                }
            }
#pragma unroll
            for (int j = 0; j < NT; j++)
#pragma unroll
                for (int l = 0; l < C::WL; l++) w_req16(j, l, c_begin + b, ws);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
        }
    } else {
    // Prologue: the same two request batches, in the same order, that a steady-state step finds
    // outstanding - the compiler merges the wait counts of the loop entry with those of the back edge, and
    // any difference in order makes the steady state wait for requests it has only just issued.
    auto issue_batch = [&](int c, WSet& ws) {
#pragma unroll
        for (int i = 0; i < C::XL; i++) {
            issue_x_unit(i, c);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < NT; j++) {
            if constexpr (META4) break;
            issue_meta(j, 0, c, ws);
            issue_meta(j, 1, c, ws);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < NT; j++)
#pragma unroll
            for (int l = 0; l < C::WL; l++) {
                issue_w_load(j, l, c, ws);
                asm volatile("" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
            }
    };
    if constexpr (META4) {
#pragma unroll
        for (int j = 0; j < NT; j++) {
            issue_meta4(j, 0, c_begin, m_cur);
            issue_meta4(j, 1, c_begin, m_cur);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    issue_batch(c_begin, set0);
#pragma unroll
    for (int i = 0; i < C::XL; i++) stage_unit(i, buf0);
    __builtin_amdgcn_sched_barrier(0);
    // second batch in the order of a steady-state step
    if constexpr (C::T_STAGE == 0) {
        issue_batch(c_begin + 1, set1);
    } else {
    if constexpr (!META4) {
#pragma unroll
        for (int j = 0; j < NT; j++) {
            issue_meta(j, 0, c_begin + 1, set1);
            issue_meta(j, 1, c_begin + 1, set1);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int i = 0; i < MT; i++) {
        if (i < C::XL) issue_x_unit(i, c_begin + 1);
        if (C::WL == 2 || !(i & 1)) issue_w_load(i / 2, C::WL == 2 ? (i & 1) : 0, c_begin + 1, set1);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    }
    }
    }
    GC gc0[NT][C::NG], gc1[NT][C::NG];
#pragma unroll
    for (int j = 0; j < NT; j++) {
        set_consts(gc0[j], j, set0, m_cur, 0);
        const h8 f = unpack(set0, j, 0, gc0[j]);
#pragma unroll
        for (int e = 0; e < 4; e++) wf[0][j][e] = h2{f[2 * e], f[2 * e + 1]};
    }
    if constexpr (NAT) {
        wait_loads<NT * C::WL + (META4 ? 0 : 2 * NT)>();       // all but the second chunk's requests: the first buffer is written
        lds_barrier();
    } else {
        __syncthreads();
    }
    if constexpr (META4 && C::SPR == 2) {
        for (int c = c_begin; c < c_end; c += 2) {   // runs of two steps = one request; an odd count runs one step on zeros
            step(c, buf0, buf1, set0, set1, gc0, gc1, 0);
            step(c + 1, buf1, buf0, set1, set0, gc1, gc0, 1);
#pragma unroll
            for (int j = 0; j < NT; j++) { m_cur[j][0] = m_next[j][0]; m_cur[j][1] = m_next[j][1]; }
        }
    } else if constexpr (META4) {
        int c = c_begin;
        for (; c + 2 < c_end; c += 4) {          // runs of four steps; the last may run one step on zeros
            step(c, buf0, buf1, set0, set1, gc0, gc1, 0);
            step(c + 1, buf1, buf0, set1, set0, gc1, gc0, 1);
            step(c + 2, buf0, buf1, set0, set1, gc0, gc1, 2);
            step(c + 3, buf1, buf0, set1, set0, gc1, gc0, 3);
#pragma unroll
            for (int j = 0; j < NT; j++) { m_cur[j][0] = m_next[j][0]; m_cur[j][1] = m_next[j][1]; }
        }
        if (c < c_end) {                         // one or two steps left
            step(c, buf0, buf1, set0, set1, gc0, gc1, 0, true);
            step(c + 1, buf1, buf0, set1, set0, gc1, gc0, 1, true);
        }
    } else {
        for (int c = c_begin; c < c_end; c += 2) {   // an odd chunk count runs one extra step on zeros
            step(c, buf0, buf1, set0, set1, gc0, gc1, 0);
            step(c + 1, buf1, buf0, set1, set0, gc1, gc0, 0);
        }
    }
#ifdef BW_TUNE
    if (a.clk && tid == 0 && id < 256) {
        a.clk[2 * id] = clock64() - clk_c0;
        a.clk[2 * id + 1] = wall_clock64() - clk_r0;
    }
#endif
    // acc[i][j][r] = y[m0 + 16 i + nl][n0 + 16 j + 4 kq + r]
    if (partial) {
        // float32 partial tile to this workgroup's block of the workspace (tile-shaped; rows past M are never
        // read back, so they are not written either)
        float* blk = a.ws + (size_t)run * (BM * BN) + wave * (NT * 16) + 4 * kq;
#pragma unroll
        for (int i = 0; i < MT; i++) {
            if (m0 + 16 * i + nl >= a.M) continue;
#pragma unroll
            for (int j = 0; j < NT; j++) *reinterpret_cast<f4*>(blk + (16 * i + nl) * BN + 16 * j) = acc[i][j];
        }
        return;
    }
    // A lane's 8 bytes per MFMA tile make a wave's store 16 pieces of 32 bytes in 16 different rows: a quarter of every
    // cache line it touches.  Where the wave's 64 columns are all inside N and y allows 16-byte stores, the wave's
    // BM x 64 block goes through its own quarter of LDS instead (free after the last K step; 128-byte rows, the 16-byte
    // slots of a row XOR-swizzled by the row number) and leaves as whole 128-byte rows, 8 per store instruction.
    if (n0 + NT * 16 <= a.N && a.ldy % 8 == 0 && (((uintptr_t)a.y) & 15) == 0) {
        __builtin_amdgcn_s_waitcnt(0xC07F);                     // the assembly fragment reads of the last step (256-row tiles)
        char* ob = smem + wave * (BM * 128);
#pragma unroll
        for (int j = 0; j < NT; j++) {
            const int n = n0 + 16 * j + 4 * kq;
            float bv[4] = {0.f, 0.f, 0.f, 0.f};
            if (a.bias) {
#pragma unroll
                for (int r = 0; r < 4; r++) bv[r] = (float)a.bias[n + r];
            }
            const int ch = 4 * j + kq;                           // 8-byte piece of the 128-byte row
#pragma unroll
            for (int i = 0; i < MT; i++) {
                const int row = 16 * i + nl;
                const _Float16 v0 = (_Float16)(acc[i][j][0] + bv[0]), v1 = (_Float16)(acc[i][j][1] + bv[1]),
                               v2 = (_Float16)(acc[i][j][2] + bv[2]), v3 = (_Float16)(acc[i][j][3] + bv[3]);
                *reinterpret_cast<u2*>(ob + row * 128 + (((ch >> 1) ^ (row & 7)) * 16) + (ch & 1) * 8) = u2{as_u32(h2{v0, v1}), as_u32(h2{v2, v3})};
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int q = 0; q < BM / 8; q++) {
            const int row = 8 * q + (lane >> 3), unit = lane & 7;
            const u4 v = *reinterpret_cast<const u4*>(ob + row * 128 + ((unit ^ (row & 7)) * 16));
            if (m0 + row < a.M) *reinterpret_cast<u4*>(a.y + (int64_t)(m0 + row) * a.ldy + n0 + unit * 8) = v;
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < NT; j++) {
        const int n = n0 + 16 * j + 4 * kq;
        if (n >= a.N) continue;
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (a.bias) {
#pragma unroll
            for (int r = 0; r < 4; r++) bv[r] = n + r < a.N ? (float)a.bias[n + r] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < MT; i++) {
            const int m = m0 + 16 * i + nl;
            if (m >= a.M) continue;
            _Float16* dst = a.y + (int64_t)m * a.ldy + n;
            const _Float16 v0 = (_Float16)(acc[i][j][0] + bv[0]), v1 = (_Float16)(acc[i][j][1] + bv[1]),
                           v2 = (_Float16)(acc[i][j][2] + bv[2]), v3 = (_Float16)(acc[i][j][3] + bv[3]);
            if (n + 3 < a.N && (((uintptr_t)dst) & 7) == 0) {
                *reinterpret_cast<u2*>(dst) = u2{as_u32(h2{v0, v1}), as_u32(h2{v2, v3})};
            } else {
                dst[0] = v0;
                if (n + 1 < a.N) dst[1] = v1;
                if (n + 2 < a.N) dst[2] = v2;
                if (n + 3 < a.N) dst[3] = v3;
            }
        }
    }
}

// Adds up the partial tiles of the split workgroups: block (x, y) handles 1024 outputs of split tile y,
// a thread four consecutive n.  y[m][n] = fp16( sum_z partial_z[m][n] + bias[n] ).
__global__ __launch_bounds__(256) void qgemm_reduce_kernel(const GemmArgs a) {
    const int tile = a.full_tiles + (int)blockIdx.y;
    const int quad = (int)(blockIdx.x * blockDim.x + threadIdx.x);          // < bm * BN / 4
    const int ml = quad / (BN / 4), nl4 = (quad % (BN / 4)) * 4;
    int tm, tn;
    tile_coords(tile, a, tm, tn);
    const int m = tm * a.bm + ml, n = tn * BN + nl4;
    if (m >= a.M || n >= a.N) return;
    const size_t blk = (size_t)a.bm * BN;
    const float* src = a.ws + (size_t)blockIdx.y * a.splits * blk + ml * BN + nl4;
    f4 v = {0.f, 0.f, 0.f, 0.f};
    for (int z = 0; z < a.splits; z++) {
        const f4 t = *reinterpret_cast<const f4*>(src + (size_t)z * blk);
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] += t[i];
    }
    _Float16* dst = a.y + (int64_t)m * a.ldy + n;
    _Float16 o[4];
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = (_Float16)(v[i] + ((a.bias && n + i < a.N) ? (float)a.bias[n + i] : 0.f));
    if (n + 3 < a.N && (((uintptr_t)dst) & 7) == 0) {
        *reinterpret_cast<u2*>(dst) = u2{as_u32(h2{o[0], o[1]}), as_u32(h2{o[2], o[3]})};
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (n + i < a.N) dst[i] = o[i];
    }
}

// One workgroup fits per CU, so a grid runs in rounds of `cus` workgroups.  Two cases cut K:
//   * a grid of at most half a round (small M * N, long K): every tile is split so that one round is filled;
//   * a last round that is at most half full: its tiles are split so that it takes a fraction of a tile's time.
// Never below 4 chunks per slice.  Without a workspace nothing is split.
struct GemmPlan {
    int tiles_n, tiles, full_tiles, splits, chunks_per_split;
    size_t ws_bytes;
};

inline int gemm_chunks(int64_t K, int bits, bool nat) {   // K steps of a whole row: GemmCfg::CHUNK_BYTES each
    const int64_t chunk = bits == 8 ? 128 : (bits == 2 && nat) ? 32 : 64;
    return (int)((K * bits / 8 + chunk - 1) / chunk);
}

inline GemmPlan gemm_plan(int64_t M, int64_t N, int nchunks, bool have_workspace, int bm = 128) {
    GemmPlan p;
    p.tiles_n = (int)((N + BN - 1) / BN);
    p.tiles = p.tiles_n * (int)((M + bm - 1) / bm);
    p.full_tiles = p.tiles;
    p.splits = 1;
    p.chunks_per_split = nchunks;
    p.ws_bytes = 0;
    if (!have_workspace) return p;
    const int cus = bw_device_cus();
    const int rest = p.tiles <= cus / 2 ? p.tiles : p.tiles % cus;          // tiles of the (only or last) short round
    if (rest == 0 || rest > cus / 2) return p;
    int s = cus / rest;
    if (s > nchunks / 4) s = nchunks / 4;
    if (s > 16) s = 16;
    if (s < 2) return p;
    int cps = (nchunks + s - 1) / s;
    cps += cps & 1;                                                          // even: the K loop runs two steps per pass
    s = (nchunks + cps - 1) / cps;
    if (s < 2) return p;
    p.full_tiles = p.tiles - rest;
    p.splits = s;
    p.chunks_per_split = cps;
    p.ws_bytes = (size_t)rest * s * bm * BN * sizeof(float);
    return p;
}

template <int BITS, int GROUP, int MT, bool NAT>
int launch_gemm(GemmArgs a, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    using C = GemmCfg<BITS, GROUP, MT, NAT>;
    constexpr int BM = C::BM;
    static_assert(C::CHUNK_BYTES == (BITS == 8 ? 128 : (BITS == 2 && NAT) ? 32 : 64), "gemm_chunks() counts K steps of this size");
    const size_t lds = 2 * (size_t)C::STAGE_BYTES;
    void (*kern)(const GemmArgs) = qgemm_kernel<BITS, GROUP, false, MT, NAT>;
    static uint64_t big_lds_devices[2] = {0, 0};           // per kernel
    int which = 0;
    if constexpr (C::CAN_META4 || C::NG == 2) {
        // an even number of K steps (so that the loop never pads with a step that would read past the row's scales)
        // and rows of scales on 4-byte boundaries
        if (a.groups % (C::CAN_META4 ? 2 * C::GPS : 2) == 0 && bw_aligned(a.scale, 4) && bw_aligned(a.zp, 4)) {
            kern = qgemm_kernel<BITS, GROUP, true, MT, NAT>;
            which = 1;
        }
    }
    if (lds > 64 * 1024 && !bw_allow_big_lds(reinterpret_cast<const void*>(kern), big_lds_devices[which])) return BW_ELAUNCH;
    const GemmPlan p = gemm_plan(a.M, a.N, a.nchunks, workspace != nullptr, BM);
    if (p.ws_bytes > workspace_bytes) return BW_EWORKSPACE;
    a.ws = (float*)workspace;
    a.bm = BM;
    a.tiles_n = p.tiles_n;
    a.tiles_m = p.tiles / p.tiles_n;
    a.panel = a.tiles_m < 4 ? a.tiles_m : 4;
    a.xcd_tiles = p.full_tiles & ~7;
#ifdef BW_TUNE
    if (const char* e = getenv("BW_GEMM_PANEL")) {
        const int v = atoi(e);
        if (v <= 0) { a.panel = 1; a.xcd_tiles = 0; }
        else a.panel = a.tiles_m < v ? a.tiles_m : v;
    }
#endif
    a.full_tiles = p.full_tiles;
    a.splits = p.splits;
    a.chunks_per_split = p.chunks_per_split;
    const int split_tiles = p.tiles - p.full_tiles;
    hipLaunchKernelGGL(kern, dim3((unsigned)(p.full_tiles + split_tiles * p.splits)), dim3(WAVES * 64), lds, stream, a);
    if (hipGetLastError() != hipSuccess) return BW_ELAUNCH;
    if (split_tiles) {
        hipLaunchKernelGGL(qgemm_reduce_kernel, dim3(BM * BN / 4 / 256, (unsigned)split_tiles), dim3(256), 0, stream, a);
        if (hipGetLastError() != hipSuccess) return BW_ELAUNCH;
    }
    return BW_OK;
}

}  // namespace
