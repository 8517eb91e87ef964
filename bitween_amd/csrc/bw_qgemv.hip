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
#include <type_traits>

#include <string>

namespace {

// Name of the decode kernel this thread launched last (bw_qgemv_last_kernel): lets a benchmark label its numbers
// with the kernel that actually ran.  The string is built once per kernel instantiation; a launch only stores a pointer.
thread_local const char* g_last_kernel = "";
inline const char* kernel_name(const char* base, std::initializer_list<int> params) {
    std::string s = std::string(base) + "<";
    bool first = true;
    for (int v : params) { s += (first ? "" : ", ") + std::to_string(v); first = false; }
    return (new std::string(s + ">"))->c_str();           // lives as long as the library
}
#define BW_NOTE_KERNEL(base, ...) do { static const char* const nm = kernel_name(base, {__VA_ARGS__}); g_last_kernel = nm; } while (0)

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
    static constexpr int MAX_WAVES = 16;
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
    int x_bf16;                              // x holds bfloat16: every value is rounded to float16 as it is staged
    int ntiles, nsteps;                      // qgemv_tiles_kernel / qgemv_rounds_kernel: 16-row tiles of N; tiles or rounds per workgroup
    int meta_lds_off;                        // qgemv_tiles_kernel: where the scale blocks start in LDS
};

// two bfloat16 -> two float16, round to nearest even (what torch's .to(float16) does)
BW_DEV uint32_t bf16x2_to_f16x2(uint32_t w) {
    const float lo = __builtin_bit_cast(float, w << 16), hi = __builtin_bit_cast(float, w & 0xFFFF0000u);
    return as_u32(h2{(_Float16)lo, (_Float16)hi});
}

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
                if (a.x_bf16) {
#pragma unroll
                    for (int j = 0; j < 4 * UW; j++) in[j] = bf16x2_to_f16x2(in[j]);
                }
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

BW_DEV float half_of(uint32_t word, int hi) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(hi ? word >> 16 : word));
}

// ---- M <= 16 (from the row count tiles_min_rows names per format), K <= 4096: every request of a workgroup in flight at once ----
//
// qgemv_kernel re-reads and re-stages its slice of x in every round of every 16-row workgroup, and a wave only
// has one round of weights requested at a time: with 4 to 16 activation rows the x traffic (from L2) is several
// times the weight traffic (from HBM) and the rounds serialise on memory latency.  Here K fits one round: wave w
// of up to 16 owns chunks [w KBW, +KBW) of every row, stages its slice of x once, and then runs the workgroup's
// NT tiles of 16 rows (tiles b, b + grid, b + 2 grid, ...) against it.  The grid is sized so that every
// workgroup is resident at once: x is read once per workgroup, not per tile.  Each tile has its own accumulators;
// the partial sums of the waves meet in LDS once, at the end (in the space of the x tiles, which are dead by then).
// Scales and zero points of a tile's 16 rows are one contiguous block of each array: the workgroup fetches it with
// 4-byte requests that cover whole cache lines (a lane fetching its own two bytes costs a cache-line lookup per
// row and request: sixteen times the lookups of the weights themselves) and passes it on through LDS as (scale,
// zero point) pairs.
// The registers that requests land in are not touched until the code that uses them, so every wait sits where
// the data is needed; nothing is requested under a branch (a request under a branch costs a full wait).
// What bounds it: a CU keeps a limited number of cache lines requested at once, and a line of x from L2 holds
// its place for a few hundred cycles, a line of weights from HBM for over a thousand: the x lines of 16
// activation rows (128 KB per CU at K = 4096) add about 2 us to what the weights alone need.
template <int BITS, int GROUP, int MT, int NT>
__global__ __launch_bounds__(1024) void qgemv_tiles_kernel(const GemvArgs a) {
    using C = GemvCfg<BITS, GROUP, MT>;
    constexpr int KBW = BITS == 4 ? 2 : (BITS == 8 ? 4 : 1);     // chunks per wave: 256 values of K
    constexpr int BK = KBW * C::CHUNK_K, PITCH = BK + 8, UPR = BK / C::UNIT, XL = (MT * UPR + 63) / 64;
    constexpr int X_BYTES = MT * PITCH * 2, UW = C::UNIT / 8;
    constexpr int kOutPerTile = 16 * MT;
    constexpr uint32_t kOob = 0x80000000u;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const int nl = lane & 15, kq = lane >> 4;
    const int groups = a.groups, GP = groups | 1;         // odd row pitch: the 16 rows hit different banks
    // LDS: [x tile of wave 0] ... [x tile of wave n-1][(scale, zero point) pairs: NT blocks of 16 x GP][counter];
    // at the end the partial sums (NT x waves blocks of MT x 16 floats) take the place of the x tiles
    _Float16* xs = reinterpret_cast<_Float16*>(smem + wave * X_BYTES);
    float* red = reinterpret_cast<float*>(smem);
    uint32_t* meta = reinterpret_cast<uint32_t*>(smem + a.meta_lds_off);
    const __amdgpu_buffer_rsrc_t rw = make_rsrc(a.qweight, a.w_bytes), rx = make_rsrc(a.x, a.x_bytes),
                                 rs = make_rsrc(a.scale, a.meta_bytes), rz = make_rsrc(a.zp, a.meta_bytes),
                                 rb = make_rsrc(a.bias, a.bias ? (uint32_t)a.N * 2 : 0u);   // no bias: every read returns zero
    auto tile_of = [&](int t) { return (int)blockIdx.x + t * (int)gridDim.x; };
    auto barrier = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    };

    // "scales are in LDS" counter: the waves that bring them in count up, the others look before their first tile.
    // A workgroup barrier there instead would hold every wave until the slowest one has staged its x.
    uint32_t* ready = meta + NT * 16 * GP;
    if (tid == 0) *ready = 0u;
    barrier();

    // ---- requests, small things first (they return in order): scales / zero points of every tile (entries 2 tid,
    // 2 tid + 1 of each 16 x groups block: K <= 256 * waves, so one 4-byte request per thread covers a block), the
    // bias of the outputs this thread will store, x, and the weights of the first two tiles; the later tiles'
    // weights are requested as the tiles before them are worked on (a wave that requests everything first sits in
    // the request queue until most of it has come back, with its x waiting to be staged)
    uint32_t ms[NT], mz[NT], bias2[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        uint32_t off = (uint32_t)tile_of(t) * 16 * groups * 2 + tid * 4;
        asm volatile("" : "+v"(off));                         // a value of its own: the select below stays a select
        off = (tile_of(t) < a.ntiles && tid < 8 * groups) ? off : kOob;
        ms[t] = __builtin_amdgcn_raw_buffer_load_b32(rs, off, 0, 0);
        mz[t] = __builtin_amdgcn_raw_buffer_load_b32(rz, off, 0, 0);
    }
    // output o = tid + j * threads of the workgroup's NT * 16 * MT: tile o / (16 MT), row (o / 16) % MT, column o % 16
#pragma unroll
    for (int j = 0; j < NT; j++) {
        const int o = tid + j * (int)blockDim.x, tile = tile_of(o / kOutPerTile);
        uint32_t off = ((uint32_t)tile * 16 + (o & 15)) * 2 & ~3u;
        asm volatile("" : "+v"(off));
        bias2[j] = __builtin_amdgcn_raw_buffer_load_b32(rb, (o < NT * kOutPerTile && tile < a.ntiles) ? off : kOob, 0, 0);
    }
    // Every workgroup reads the same x: each starts at a different row, so that the CUs of an XCD are not all
    // asking the same L2 channel at the same time.
    const int xrot = (int)(blockIdx.x % XL);
    u4 xr[XL * UW];
#pragma unroll
    for (int j = 0; j < XL; j++) {
        const int jr = j + xrot < XL ? j + xrot : j + xrot - XL;
        const int u = lane + 64 * jr, m = u / UPR, k = wave * BK + (u - m * UPR) * C::UNIT;
        uint32_t off = (uint32_t)(m * a.ldx + k) * 2;
        asm volatile("" : "+v"(off));
        off = (m < a.M && k < a.K) ? off : kOob;
#pragma unroll
        for (int q = 0; q < UW; q++) xr[j * UW + q] = __builtin_amdgcn_raw_buffer_load_b128(rx, off + q * 16, 0, 0);
    }
    asm volatile("" ::: "memory");
    u4 wr[NT][KBW];
    auto issue_w = [&](int t) {
        const uint32_t n = (uint32_t)tile_of(t) * 16 + nl;
#pragma unroll
        for (int b = 0; b < KBW; b++) {
            const int c = wave * KBW + b;
            uint32_t off = n * a.row_bytes + c * 64 + kq * 16;
            asm volatile("" : "+v"(off));
            off = (tile_of(t) < a.ntiles && c < a.nchunks) ? off : kOob;
            wr[t][b] = __builtin_amdgcn_raw_buffer_load_b128(rw, off, 0, 0);
        }
        asm volatile("" ::: "memory");
    };
    issue_w(0);
    if constexpr (NT > 1) issue_w(1);

    // ---- scales / zero points -> LDS as pairs, by the waves whose threads hold entries
    const int meta_waves = (8 * groups + 63) / 64;
    if (wave < meta_waves) {                                  // wave-uniform
#pragma unroll
        for (int t = 0; t < NT; t++) {
            uint32_t sv = ms[t], zv = mz[t];
            asm volatile("" : "+v"(sv), "+v"(zv));            // the wait for them belongs here
            const int e = 2 * tid;                            // first of the two entries: row e / groups, column e % groups
            if (e < 16 * groups) {
                const int r = e / groups, c = e - r * groups; // groups is even: both entries lie in row r
                uint32_t* dst = meta + t * 16 * GP + r * GP + c;
                dst[0] = __builtin_amdgcn_perm(zv, sv, 0x05040100u);
                dst[1] = __builtin_amdgcn_perm(zv, sv, 0x07060302u);
            }
        }
        if (lane == 0) __hip_atomic_fetch_add(ready, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    // ---- x -> this wave's LDS tile, permuted to the unpack order
#pragma unroll
    for (int j = 0; j < XL; j++) {
        const int jr = j + xrot < XL ? j + xrot : j + xrot - XL;
        const int u = lane + 64 * jr, m = u / UPR, ku = u - m * UPR;
        if (m < MT) {
            uint32_t in[4 * UW], o[4 * UW];
#pragma unroll
            for (int q = 0; q < UW; q++) { in[4 * q] = xr[j * UW + q][0]; in[4 * q + 1] = xr[j * UW + q][1]; in[4 * q + 2] = xr[j * UW + q][2]; in[4 * q + 3] = xr[j * UW + q][3]; }
            if (a.x_bf16) {
#pragma unroll
                for (int q = 0; q < 4 * UW; q++) in[q] = bf16x2_to_f16x2(in[q]);
            }
            permute_unit<BITS>(in, o);
            u4* dst = reinterpret_cast<u4*>(xs + m * PITCH + ku * C::UNIT);
#pragma unroll
            for (int q = 0; q < UW; q++) dst[q] = u4{o[4 * q], o[4 * q + 1], o[4 * q + 2], o[4 * q + 3]};
        }
    }
    __builtin_amdgcn_wave_barrier();
    while (__hip_atomic_load(ready, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < (uint32_t)meta_waves) __builtin_amdgcn_s_sleep(1);

    // ---- the tiles, as their weights arrive
    f4 acc[NT][2];
    const int arow = nl < MT ? nl : MT - 1;              // MFMA rows >= MT repeat a valid row; never stored
#pragma unroll
    for (int t = 0; t < NT; t++) {
        if (t + 2 < NT) issue_w(t + 2);
        acc[t][0] = acc[t][1] = f4{0.f, 0.f, 0.f, 0.f};
        const uint32_t* mrow = meta + t * 16 * GP + nl * GP;
#pragma unroll
        for (int b = 0; b < KBW; b++) {
            u4 wv = wr[t][b];
            asm volatile("" : "+v"(wv));                      // use the registers here and not before
            // (a chunk may reach past the end of K: those lanes take the row's last groups, their x is zero)
            const int gb = min(((wave * KBW + b) * C::CHUNK_K + kq * C::VPL) / GROUP, groups - C::NG);
            GroupConst<BITS> gc[C::NG];
#pragma unroll
            for (int g = 0; g < C::NG; g++) {
                const uint32_t sz = mrow[gb + g];
                gc[g].set(__builtin_bit_cast(_Float16, (uint16_t)sz), __builtin_bit_cast(_Float16, (uint16_t)(sz >> 16)));
            }
            h2 wp[C::VPL / 2];
            dequant_lane16<BITS, C::NG, !C::POST>(wv, gc, wp);
            const _Float16* xp = xs + arow * PITCH + b * C::CHUNK_K + kq * C::VPL;
            if constexpr (C::POST) {
                f4 part = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < C::MF; s++)
                    part = __builtin_amdgcn_mfma_f32_16x16x32_f16(*reinterpret_cast<const h8*>(xp + 8 * s), pack_h8(wp + 4 * s), part, 0, 0, 0);
                const float sf = (float)gc[0].s[0];
#pragma unroll
                for (int q = 0; q < 4; q++) acc[t][b & 1][q] = __builtin_fmaf(sf, part[q], acc[t][b & 1][q]);
            } else {
#pragma unroll
                for (int s = 0; s < C::MF; s++)
                    acc[t][s & 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(*reinterpret_cast<const h8*>(xp + 8 * s), pack_h8(wp + 4 * s), acc[t][s & 1], 0, 0, 0);
            }
        }
    }

    // ---- partial sums of the waves -> y, all tiles at once: red[(t * waves + w) * MT * 16 + (m / 4) * 64 + n * 4 + m % 4]
    barrier();                                                // every wave is through with the x tiles
    if (4 * kq < MT) {
#pragma unroll
        for (int t = 0; t < NT; t++) {
            f4 v;
#pragma unroll
            for (int r = 0; r < 4; r++) v[r] = acc[t][0][r] + acc[t][1][r];
            *reinterpret_cast<f4*>(red + ((t * nwaves + wave) * MT + 4 * kq) * 16 + nl * 4) = v;
        }
    }
    barrier();
#pragma unroll
    for (int j = 0; j < NT; j++) {                            // the launch makes the workgroup at least 16 MT threads
        const int o = tid + j * (int)blockDim.x, t = o / kOutPerTile, m = (o >> 4) % MT, n = tile_of(t) * 16 + (o & 15);
        uint32_t b2 = bias2[j];
        asm volatile("" : "+v"(b2));
        if (o < NT * kOutPerTile) {
            float v = 0.f;
            for (int w = 0; w < nwaves; w++) v += red[((t * nwaves + w) * MT + (m & ~3)) * 16 + (o & 15) * 4 + (m & 3)];
            v += half_of(b2, o & 1);
            if (m < a.M && n < a.N) a.y[(int64_t)m * a.ldy + n] = (_Float16)v;
        }
    }
}

// ---- M <= 16 (same table), long K: one 16-row tile per workgroup, rounds of K -----------------------------------
//
// Wave w of up to 16 owns chunks [(r waves + w) KBW, +KBW) of round r.  The weights of DEPTH rounds are requested
// ahead in registers (all rounds, for the usual shapes; else a ring that is refilled as it drains); x is restaged
// per round into the wave's own LDS tile.  The tile's whole block of scales and zero points comes in once, at
// the start, as in qgemv_tiles_kernel.
template <int BITS, int GROUP, int MT, int DEPTH, bool LOOP>
__global__ __launch_bounds__(1024) void qgemv_rounds_kernel(const GemvArgs a) {
    using C = GemvCfg<BITS, GROUP, MT>;
    constexpr int KBW = BITS == 4 ? 2 : (BITS == 8 ? 4 : 1);     // chunks per wave and round: 256 values of K
    constexpr int BK = KBW * C::CHUNK_K, PITCH = BK + 8, UPR = BK / C::UNIT, XL = (MT * UPR + 63) / 64;
    constexpr int X_BYTES = MT * PITCH * 2, UW = C::UNIT / 8;
    constexpr int ME = 4;                                 // 4-byte requests (two entries) per thread for the scale block
    constexpr uint32_t kOob = 0x80000000u;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const int nl = lane & 15, kq = lane >> 4;
    const int groups = a.groups, GP = groups | 1;         // odd row pitch: the 16 rows hit different banks
    const int tile = (int)blockIdx.x, nsteps = a.nsteps;
    // LDS: [x tile of wave 0] ... [x tile of wave n-1][partial sums, one MT x 16 block per wave][(scale, zero point)]
    _Float16* xs = reinterpret_cast<_Float16*>(smem + wave * X_BYTES);
    float* red = reinterpret_cast<float*>(smem + nwaves * X_BYTES);
    uint32_t* meta = reinterpret_cast<uint32_t*>(smem + nwaves * (X_BYTES + MT * 64));
    const __amdgpu_buffer_rsrc_t rw = make_rsrc(a.qweight, a.w_bytes), rx = make_rsrc(a.x, a.x_bytes),
                                 rs = make_rsrc(a.scale, a.meta_bytes), rz = make_rsrc(a.zp, a.meta_bytes),
                                 rb = make_rsrc(a.bias, a.bias ? (uint32_t)a.N * 2 : 0u);   // no bias: every read returns zero
    // the next round's x is requested before this round's arithmetic where the registers allow (16 rows of x in
    // flight plus three rounds of weights do not fit 128 registers), else right behind it
    constexpr bool XPRE = MT < 16;

    u4 xr[XL * UW];
    u4 wr[DEPTH][KBW];
    uint32_t ms[ME], mz[ME];
    auto issue_x = [&](int i) {
        const int k0 = (i * nwaves + wave) * BK;
#pragma unroll
        for (int j = 0; j < XL; j++) {
            const int u = lane + 64 * j, m = u / UPR, k = k0 + (u - m * UPR) * C::UNIT;
            uint32_t off = (uint32_t)(m * a.ldx + k) * 2;
            asm volatile("" : "+v"(off));                     // a value of its own: the select below stays a select
            off = (i < nsteps && m < a.M && k < a.K) ? off : kOob;
#pragma unroll
            for (int q = 0; q < UW; q++) xr[j * UW + q] = __builtin_amdgcn_raw_buffer_load_b128(rx, off + q * 16, 0, 0);
        }
        asm volatile("" ::: "memory");
    };
    auto issue_w = [&](int d, int i) {
        const int c0 = (i * nwaves + wave) * KBW;
        const uint32_t n = (uint32_t)tile * 16 + nl;
#pragma unroll
        for (int b = 0; b < KBW; b++) {
            uint32_t off = n * a.row_bytes + (c0 + b) * 64 + kq * 16;
            asm volatile("" : "+v"(off));
            off = (i < nsteps && c0 + b < a.nchunks) ? off : kOob;
            wr[d][b] = __builtin_amdgcn_raw_buffer_load_b128(rw, off, 0, 0);
        }
        asm volatile("" ::: "memory");
    };
    auto stage_x = [&]() {
#pragma unroll
        for (int j = 0; j < XL; j++) {
            const int u = lane + 64 * j, m = u / UPR, ku = u - m * UPR;
            if (m < MT) {
                uint32_t in[4 * UW], o[4 * UW];
#pragma unroll
                for (int q = 0; q < UW; q++) { in[4 * q] = xr[j * UW + q][0]; in[4 * q + 1] = xr[j * UW + q][1]; in[4 * q + 2] = xr[j * UW + q][2]; in[4 * q + 3] = xr[j * UW + q][3]; }
                if (a.x_bf16) {
#pragma unroll
                    for (int q = 0; q < 4 * UW; q++) in[q] = bf16x2_to_f16x2(in[q]);
                }
                permute_unit<BITS>(in, o);
                u4* dst = reinterpret_cast<u4*>(xs + m * PITCH + ku * C::UNIT);
#pragma unroll
                for (int q = 0; q < UW; q++) dst[q] = u4{o[4 * q], o[4 * q + 1], o[4 * q + 2], o[4 * q + 3]};
            }
        }
    };
    auto barrier = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    };

    // ---- requests, small things first (they return in order): the tile's scales and zero points (entries 2 e,
    // 2 e + 1 of its 16 x groups block for e = tid, tid + threads, ...), its bias, x of round 0, the weights
    const uint32_t mbase = (uint32_t)tile * 16 * groups * 2;
#pragma unroll
    for (int j = 0; j < ME; j++) {
        const int e = tid + j * (int)blockDim.x;
        uint32_t off = mbase + e * 4;
        asm volatile("" : "+v"(off));
        off = e < 8 * groups ? off : kOob;
        ms[j] = __builtin_amdgcn_raw_buffer_load_b32(rs, off, 0, 0);
        mz[j] = __builtin_amdgcn_raw_buffer_load_b32(rz, off, 0, 0);
    }
    uint32_t bias2 = __builtin_amdgcn_raw_buffer_load_b32(rb, ((uint32_t)tile * 16 + nl) * 2 & ~3u, 0, 0);
    issue_x(0);
#pragma unroll
    for (int d = 0; d < DEPTH; d++) issue_w(d, d);
    // scales / zero points -> LDS as pairs
#pragma unroll
    for (int j = 0; j < ME; j++) {
        const int e = 2 * (tid + j * (int)blockDim.x);        // first of the two entries: row e / groups, column e % groups
        uint32_t sv = ms[j], zv = mz[j];
        asm volatile("" : "+v"(sv), "+v"(zv));                // the wait for them belongs here
        if (e < 16 * groups) {
            const int r = e / groups, c = e - r * groups;     // groups is even: both entries lie in row r
            meta[r * GP + c] = __builtin_amdgcn_perm(zv, sv, 0x05040100u);
            meta[r * GP + c + 1] = __builtin_amdgcn_perm(zv, sv, 0x07060302u);
        }
    }
    barrier();

    f4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    const int arow = nl < MT ? nl : MT - 1;              // MFMA rows >= MT repeat a valid row; never stored
    const uint32_t* mrow = meta + nl * GP;
    // one round from ring slot d; false = past the last round
    auto run_step = [&](int d, int i) -> bool {
        if (i >= nsteps) return false;                        // uniform over the workgroup
        if (i > 0) __builtin_amdgcn_wave_barrier();           // the reads of the round before are done
        stage_x();
        __builtin_amdgcn_wave_barrier();
        if constexpr (XPRE) issue_x(i + 1);                   // past the last round: range-checked to nothing
        const int c0 = (i * nwaves + wave) * KBW;
#pragma unroll
        for (int b = 0; b < KBW; b++) {
            u4 wv = wr[d][b];
            asm volatile("" : "+v"(wv));                      // use the round's registers here and not before
            // (a chunk may reach past the end of K: those lanes take the row's last groups, their x is zero)
            const int gb = min(((c0 + b) * C::CHUNK_K + kq * C::VPL) / GROUP, groups - C::NG);
            GroupConst<BITS> gc[C::NG];
#pragma unroll
            for (int g = 0; g < C::NG; g++) {
                const uint32_t sz = mrow[gb + g];
                gc[g].set(__builtin_bit_cast(_Float16, (uint16_t)sz), __builtin_bit_cast(_Float16, (uint16_t)(sz >> 16)));
            }
            h2 wp[C::VPL / 2];
            dequant_lane16<BITS, C::NG, !C::POST>(wv, gc, wp);
            const _Float16* xp = xs + arow * PITCH + b * C::CHUNK_K + kq * C::VPL;
            if constexpr (C::POST) {
                f4 part = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < C::MF; s++)
                    part = __builtin_amdgcn_mfma_f32_16x16x32_f16(*reinterpret_cast<const h8*>(xp + 8 * s), pack_h8(wp + 4 * s), part, 0, 0, 0);
                const float sf = (float)gc[0].s[0];
#pragma unroll
                for (int q = 0; q < 4; q++) acc[b & 1][q] = __builtin_fmaf(sf, part[q], acc[b & 1][q]);
            } else {
#pragma unroll
                for (int s = 0; s < C::MF; s++)
                    acc[s & 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(*reinterpret_cast<const h8*>(xp + 8 * s), pack_h8(wp + 4 * s), acc[s & 1], 0, 0, 0);
            }
        }
        if constexpr (!XPRE) {
            __builtin_amdgcn_wave_barrier();                  // the round's reads of the x tile are done
            issue_x(i + 1);
        }
        if constexpr (LOOP) issue_w(d, i + DEPTH);            // refill the slot
        return true;
    };
    if constexpr (LOOP) {
        for (int i0 = 0; i0 < nsteps; i0 += DEPTH) {
            bool more = true;
#pragma unroll
            for (int d = 0; d < DEPTH; d++) more = more && run_step(d, i0 + d);
            if (!more) break;
        }
    } else {
        // at most DEPTH rounds: straight code, every wait count exact, nothing requested that is not used
        bool more = true;
#pragma unroll
        for (int d = 0; d < DEPTH; d++) more = more && run_step(d, d);
    }

    // partial sums of the waves -> y
    if (4 * kq < MT) {
#pragma unroll
        for (int r = 0; r < 4; r++)
            if (4 * kq + r < MT) red[(wave * MT + 4 * kq + r) * 16 + nl] = acc[0][r] + acc[1][r];
    }
    asm volatile("" : "+v"(bias2));
    barrier();
    if (tid < 16 * MT) {                                      // the launch makes the workgroup at least this large
        const int m = tid >> 4, n = tile * 16 + nl;
        if (m < a.M && n < a.N) {
            float v = 0.f;
            for (int w = 0; w < nwaves; w++) v += red[(w * MT + m) * 16 + nl];
            v += half_of(bias2, nl & 1);
            a.y[(int64_t)m * a.ldy + n] = (_Float16)v;
        }
    }
}

// ---- packed weights, memory -> LDS -> MFMA operand layout ---------------------------------------------------------
//
// The B operand of v_mfma_f32_16x16x32_f16 wants lane l to hold row (l & 15), 16-byte piece (l >> 4) of a chunk: loaded
// that way straight from memory, neighbouring lanes touch 16 different rows and every 128-byte line of weights is
// asked for by eight separate quarter-line requests.  Measured on MI355X (weights only, graph replay): 3.5 / 6.0 us
// for the 8.4 / 22.5 MB of a Llama-7B projection that way, 2.8 / 4.8 us when eight neighbouring lanes ask for one
// whole line and the loads carry the non-temporal hint (a weight byte is read once; the hint alone, without whole
// lines, gains nothing).  So the weights take the coalesced route: a load instruction covers eight rows x 128 bytes
// (two chunks), lands in LDS without passing through registers (16 bytes per lane at lane * 16), and the lane that
// feeds the matrix core reads its 16 bytes back from there.  The piece a lane loads is XOR-swizzled with its row
// (lane (a, s) of an instruction loads piece s ^ a of row a), so that the sixteen rows a read instruction touches
// fall into different LDS banks; the second instruction of a pair (rows 8-15) sits 128 bytes further for the same reason.
struct WeightTile {
    static constexpr int kHalf = 1024 + 128;              // rows 0-7 | rows 8-15 of a pair of chunks
    static constexpr int kPair = 2 * kHalf;               // LDS bytes per pair of chunks (16 rows x 128 bytes + padding)
    static constexpr int kAuxNt = 2;                      // cache-policy bits of the buffer load: non-temporal

    // the 16 bytes lane (n = lane & 15, j = lane >> 4) feeds the matrix core with for chunk b of the batch
    static BW_DEV u4 fetch(const char* tile, int b, int lane) {
        const int n = lane & 15, j = lane >> 4, a = n & 7, p = (b & 1) * 4 + j;
        return *reinterpret_cast<const u4*>(tile + (b >> 1) * kPair + (n >> 3) * kHalf + (a * 8 + (p ^ a)) * 16);
    }
};

// ---- 4-bit, up to four MFMA rows (M x groups per chunk): integer operands, scale and zero point taken out of the inner loop ----
//
// A masked packed word is already a float16: bits 0-3 of a half are the subnormal q * 2^-24, bits 4-7 the
// subnormal q * 2^-20, and the matrix core keeps subnormal inputs exactly.  So a word unpacks with one shift
// and four ANDs, the products x * q are exact, and per group
//     sum_k x_k (q_k - z) = 2^24 * (E + O / 16) - z * S,     S = sum_k x_k,
// with E and O the accumulators of the even and the odd nibbles.  S comes from the lanes that stage x (a
// cross-lane reduction per group and row), so the inner loop holds no per-weight arithmetic at all; that
// staging cost grows with M, which is why wider activation tiles stay on the kernel above.
//
// A chunk is 128 weights of each row.  With groups of 64 or 32 it spans 2 or 4 groups, but an MFMA adds up
// all of a chunk's k.  The MFMA rows an M <= 2 activation tile leaves idle separate them: row m * NGC + g of
// the staged tile holds x[m] with everything outside group g of the chunk zeroed, so output row m * NGC + g is
// the partial sum of group g alone and gets that group's scale and zero point.
// Results agree with the per-weight float16 dequantisation to float32 rounding: a one-hot x still returns
// the reference's W16 column bit for bit.

// sum over aligned runs of LANES (4, 8 or 16) lanes; every lane of a run ends up with the run's total
template <int LANES>
BW_DEV float lanes_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    if constexpr (LANES >= 8)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));   // row_half_mirror
    if constexpr (LANES >= 16)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));   // row_mirror
    return v;
}

// the buffer [p + skip, p + bytes): empty when `skip` lies past the end.  All operands are wave-uniform, so this is
// scalar arithmetic; it lets the per-wave and per-round part of an address live in the descriptor (range-checked)
// instead of in a per-lane add.
BW_DEV __amdgpu_buffer_rsrc_t make_rsrc_at(const void* p, uint32_t bytes, uint32_t skip) {
    // (readfirstlane: the saturating subtraction is a vector instruction even for uniform operands, and a descriptor
    // the compiler cannot see to be uniform costs a loop around every load)
    const uint32_t left = __builtin_amdgcn_readfirstlane(skip < bytes ? bytes - skip : 0u);
    return make_rsrc(static_cast<const char*>(p) + skip, left);
}

template <int GROUP, int MT, int KB>
__global__ __launch_bounds__(1024) void qgemv_w4_kernel(const GemvArgs a) {
    constexpr int NGC = 128 / GROUP;                      // groups per chunk
    constexpr int ROWS = MT * NGC;                        // MFMA rows in use: (m, group of the chunk)
    static_assert(ROWS <= 4, "the outputs must fit the four rows the lanes with kq == 0 hold");
    static_assert(KB % 2 == 0, "weights are requested in pairs of chunks");
    constexpr int GL = GROUP / 8;                         // staging lanes per group (8 halves each)
    constexpr int P = KB / 2;                             // pairs of chunks per wave and round
    constexpr int UPR = KB * 16;                          // 8-half units per activation row and round
    constexpr int XL = (MT * UPR + 63) / 64;              // unit loads per lane and round
    constexpr int ROW_BYTES = KB * 256 + 16, X_BYTES = ROWS * ROW_BYTES;
    constexpr int KBG = KB * NGC, MP = KBG | 1;           // groups a wave covers per round; odd row pitch of its (scale, zp) block
    constexpr int ML = (KBG + 3) / 4;                     // 2-byte requests per lane, array and round
    constexpr int META_BYTES = (16 * MP * 4 + 15) & ~15;
    constexpr int WAVE_BYTES = X_BYTES + META_BYTES + P * WeightTile::kPair;
    constexpr uint32_t kOob = 0x80000000u;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, nwaves = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nl = lane & 15, kq = lane >> 4;
    const uint32_t n0 = blockIdx.x * 16;
    // LDS, everything a wave touches before the final sum is its own (no workgroup barrier until then):
    // [wave 0: x tile | (scale, zero point) pairs of its groups, 16 rows x MP | weight batch] ... [partial sums]
    char* xs = smem + wave * WAVE_BYTES;
    uint32_t* meta = reinterpret_cast<uint32_t*>(xs + X_BYTES);
    char* wt = xs + X_BYTES + META_BYTES;
    float* red = reinterpret_cast<float*>(smem + nwaves * WAVE_BYTES);

    // the bias of the outputs the first MT waves will store, requested before anything else
    uint32_t bias_v = 0;
    if (wave < MT && a.bias)
        bias_v = __builtin_amdgcn_raw_buffer_load_b16(make_rsrc(a.bias, (uint32_t)a.N * 2), (n0 + nl) * 2, 0, 0);

    // ---- per-lane parts of the addresses (the per-wave and per-round parts go into the descriptors)
    // scales / zero points: lane (row lane / 4, column lane % 4 + 4 t) - four neighbouring lanes ask for 8 adjacent bytes
    const uint32_t m_off = ((uint32_t)(lane >> 2) * a.groups + (lane & 3)) * 2;
    uint32_t* m_dst = meta + (lane >> 2) * MP + (lane & 3);
    // x: unit u = lane + 64 i of the round: activation row u / UPR, unit ku = u % UPR
    uint32_t x_off[XL], x_dst[XL];
#pragma unroll
    for (int i = 0; i < XL; i++) {
        const int u = lane + 64 * i, m = u / UPR, ku = u % UPR;
        x_off[i] = (MT == 1 || m < a.M) ? (uint32_t)(m * a.ldx + ku * 8) * 2 : kOob;
        x_dst[i] = m * NGC * ROW_BYTES + (ku >> 2) * 64 + (ku & 3) * 8;
    }
    // weights: lane (row lane / 8 (+ 8 for the second instruction of a pair), piece (lane % 8) ^ row)
    uint32_t w_off[2];
    {
        const int r = lane >> 3, p = (lane & 7) ^ r;
        w_off[0] = (uint32_t)r * a.row_bytes + (p >> 2) * 64 + (p & 3) * 16;
        w_off[1] = w_off[0] + 8u * a.row_bytes;
    }

    float acc[MT];
#pragma unroll
    for (int r = 0; r < MT; r++) acc[r] = 0.f;
    const char* xrow = xs + (nl < ROWS ? nl : ROWS - 1) * ROW_BYTES + kq * 64;
    const uint32_t* mrow = meta + nl * MP;
    const int my_group = ((lane & 15) * 8) / GROUP;       // group of the chunk this lane's staged unit lies in
    constexpr uint32_t kEven = 0x000F000Fu, kOdd = 0x00F000F0u;
    int c0 = wave * KB;
    while (true) {
        // ---- requests, small things first (loads return in order): scales / zero points, x, then the weights
        const uint32_t g0 = (uint32_t)c0 * NGC;           // first group of the round
        const __amdgpu_buffer_rsrc_t rs = make_rsrc_at(a.scale, a.meta_bytes, (n0 * a.groups + g0) * 2),
                                     rz = make_rsrc_at(a.zp, a.meta_bytes, (n0 * a.groups + g0) * 2),
                                     rx = make_rsrc_at(a.x, a.x_bytes, (uint32_t)c0 * 256),
                                     rw = make_rsrc_at(a.qweight, a.w_bytes, n0 * (uint32_t)a.row_bytes + (uint32_t)c0 * 64);
        const int glim = min(KBG, a.groups - (int)g0);    // groups of the round that exist (the others read as zero)
        uint32_t ms[ML], mz[ML];
#pragma unroll
        for (int t = 0; t < ML; t++) {
            const uint32_t off = (lane & 3) + 4 * t < glim ? m_off : kOob;
            ms[t] = __builtin_amdgcn_raw_buffer_load_b16(rs, off + 8 * t, 0, 0);
            mz[t] = __builtin_amdgcn_raw_buffer_load_b16(rz, off + 8 * t, 0, 0);
        }
        u4 xr[XL];
#pragma unroll
        for (int i = 0; i < XL; i++) {
            uint32_t xo = x_off[i];
            if constexpr (MT > 1) {                           // one row: the end of x is the end of the buffer
                const int ku = (lane + 64 * i) % UPR;
                xo = c0 * 128 + ku * 8 < a.K ? xo : kOob;
            }
            xr[i] = __builtin_amdgcn_raw_buffer_load_b128(rx, xo, 0, 0);
        }
        asm volatile("" ::: "memory");
        static_for<0, KB>([&](auto ic) {
            constexpr int q = decltype(ic)::value / 2, i = decltype(ic)::value % 2;
            // (the instruction's immediate offset moves the LDS destination as well as the memory address: taken off again here)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (__attribute__((address_space(3))) void*)(wt + q * (WeightTile::kPair - 128) + i * WeightTile::kHalf),
                                                     16, w_off[i], 0, q * 128, WeightTile::kAuxNt);
        });
        asm volatile("" ::: "memory");

        // ---- scales / zero points -> this wave's block, as (scale | zero point << 16)
#pragma unroll
        for (int t = 0; t < ML; t++)
            if (4 * t + 3 < KBG || (lane & 3) + 4 * t < KBG) m_dst[4 * t] = ms[t] | (mz[t] << 16);
        // ---- the round's activations: even-k quartets (x0,x4,x2,x6) and odd-k quartets (x1,x5,x3,x7) of every 8
        // values, in the order the masks below emit the nibbles, into the row of their group (zeros into the rows
        // of the chunk's other groups); and -2^-24 * sum(x) per group
        float nsum[XL];
#pragma unroll
        for (int i = 0; i < XL; i++) {
            u4 v = xr[i];
            if (a.x_bf16) {
#pragma unroll
                for (int j = 0; j < 4; j++) v[j] = bf16x2_to_f16x2(v[j]);
            }
            u2 ev, od;
            ev[0] = __builtin_amdgcn_perm(v[2], v[0], 0x05040100u);
            ev[1] = __builtin_amdgcn_perm(v[3], v[1], 0x05040100u);
            od[0] = __builtin_amdgcn_perm(v[2], v[0], 0x07060302u);
            od[1] = __builtin_amdgcn_perm(v[3], v[1], 0x07060302u);
            if (MT * UPR >= 64 * (i + 1) || lane + 64 * i < MT * UPR) {
#pragma unroll
                for (int g = 0; g < NGC; g++) {
                    const bool mine = NGC == 1 || g == my_group;
                    char* dst = xs + x_dst[i] + g * ROW_BYTES;
                    *reinterpret_cast<u2*>(dst) = mine ? ev : u2{0u, 0u};
                    *reinterpret_cast<u2*>(dst + 32) = mine ? od : u2{0u, 0u};
                }
            }
            float t = 0.f;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const h2 p = __builtin_bit_cast(h2, (uint32_t)v[j]);
                t -= (float)p[0];
                t -= (float)p[1];
            }
            nsum[i] = lanes_sum<GL>(t) * 0x1p-24f;
        }
        __builtin_amdgcn_wave_barrier();
        asm volatile("" ::: "memory");
        static_for<0, KB>([&](auto bc) {
            constexpr int b = decltype(bc)::value;
            if constexpr ((b & 1) == 0) {                     // the pair's two load instructions have landed in LDS
                wait_loads<KB - 2 - b>();
                __builtin_amdgcn_wave_barrier();
                asm volatile("" ::: "memory");                // the reads below stay below
            }
            const u4 w = WeightTile::fetch(wt, b, lane);
            u4 e0, e1, o0, o1;                            // B operands: even / odd nibbles of words 0,1 and 2,3
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const uint32_t wa = w[j], sa = wa >> 8, wb = w[2 + j], sb = wb >> 8;
                e0[2 * j] = wa & kEven; e0[2 * j + 1] = sa & kEven;
                o0[2 * j] = wa & kOdd;  o0[2 * j + 1] = sa & kOdd;
                e1[2 * j] = wb & kEven; e1[2 * j + 1] = sb & kEven;
                o1[2 * j] = wb & kOdd;  o1[2 * j + 1] = sb & kOdd;
            }
            const h8* xp = reinterpret_cast<const h8*>(xrow + b * 256);
            f4 pe = {0.f, 0.f, 0.f, 0.f}, po = {0.f, 0.f, 0.f, 0.f};
            pe = __builtin_amdgcn_mfma_f32_16x16x32_f16(xp[0], __builtin_bit_cast(h8, e0), pe, 0, 0, 0);
            po = __builtin_amdgcn_mfma_f32_16x16x32_f16(xp[2], __builtin_bit_cast(h8, o0), po, 0, 0, 0);
            pe = __builtin_amdgcn_mfma_f32_16x16x32_f16(xp[1], __builtin_bit_cast(h8, e1), pe, 0, 0, 0);
            po = __builtin_amdgcn_mfma_f32_16x16x32_f16(xp[3], __builtin_bit_cast(h8, o1), po, 0, 0, 0);
#pragma unroll
            for (int g = 0; g < NGC; g++) {
                const uint32_t sz = mrow[b * NGC + g];
                const float sf = half_of(sz, 0), zf = half_of(sz, 1);
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    // the sum of (row m, chunk b, group g) sits in the lanes that staged it: unit m * UPR + 16 b + g * GL
                    const int u = m * UPR + 16 * b + g * GL, r = m * NGC + g;
                    const float ns = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, nsum[u / 64]), u % 64));
                    const float t = __builtin_fmaf(po[r], 0.0625f, pe[r]);
                    acc[m] = __builtin_fmaf(sf, __builtin_fmaf(zf, ns, t), acc[m]);
                }
            }
        });
        c0 += nwaves * KB;
        if (c0 >= a.nchunks) break;                       // wave-uniform
        __builtin_amdgcn_s_waitcnt(0xC07F);               // lgkmcnt(0): everything has been read out of LDS, the next round may land
        __builtin_amdgcn_wave_barrier();
        asm volatile("" ::: "memory");
    }

    // acc[m] = 2^-24 * partial y[m][n = nl] in the lanes with kq == 0
    if (kq == 0) {
#pragma unroll
        for (int r = 0; r < MT; r++) red[(wave * MT + r) * 16 + nl] = acc[r];
    }
    lds_barrier();
    // wave m adds up row m: its four 16-lane quarters each take every fourth partial sum (all reads requested at
    // once), then fold
    if (wave < MT) {
        const int m = wave;
        float part[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (kq + 4 * i < nwaves) part[i] = red[((kq + 4 * i) * MT + m) * 16 + nl];
        float v = (part[0] + part[1]) + (part[2] + part[3]);
        v += __shfl_xor(v, 16);
        v += __shfl_xor(v, 32);
        const uint32_t n = n0 + nl;
        asm volatile("" : "+v"(bias_v));                      // the wait for the bias belongs here, not behind its request
        if (kq == 0 && m < a.M && n < (uint32_t)a.N) {
            v = __builtin_fmaf(v, 0x1p24f, half_of(bias_v, 0));
            a.y[(int64_t)m * a.ldy + n] = (_Float16)v;
        }
    }
}

// LDS a workgroup of qgemv_w4_kernel<GROUP, MT, KB> needs with `nwaves` waves
template <int GROUP, int MT, int KB>
constexpr size_t w4_lds_bytes(int nwaves) {
    constexpr int NGC = 128 / GROUP, MP = (KB * NGC) | 1;
    constexpr int WAVE_BYTES = MT * NGC * (KB * 256 + 16) + ((16 * MP * 4 + 15) & ~15) + (KB / 2) * WeightTile::kPair;
    return (size_t)nwaves * (WAVE_BYTES + MT * 64);
}

template <int GROUP, int MT, int KB>
int launch_w4_kb(const GemvArgs& a, hipStream_t stream) {
    int nwaves = (a.nchunks + KB - 1) / KB;
    if (nwaves > 16) nwaves = 16;
    while (nwaves > 1 && w4_lds_bytes<GROUP, MT, KB>(nwaves) > (size_t)160 * 1024) nwaves--;
    const size_t lds = w4_lds_bytes<GROUP, MT, KB>(nwaves);
    if (lds > (size_t)160 * 1024 || nwaves < MT) return BW_EUNSUPPORTED;
    auto kern = qgemv_w4_kernel<GROUP, MT, KB>;
    BW_NOTE_KERNEL("qgemv_w4_kernel", GROUP, MT, KB);
    static uint64_t big_lds_devices = 0;                   // per instantiation
    if (lds > 64 * 1024 && !bw_allow_big_lds(reinterpret_cast<const void*>(kern), big_lds_devices)) return BW_ELAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)((a.N + 15) / 16)), dim3(nwaves * 64), lds, stream, a);
    return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
}

// BW_EUNSUPPORTED = nothing fits LDS; the caller falls back
template <int GROUP, int MT>
int launch_w4(const GemvArgs& a, hipStream_t stream) {
    // Chunks a wave requests per round (pairs, each landing in LDS), from timing the Llama-7B shapes on MI355X at
    // M = 1 (us: 4096 x 4096 / 4096 -> 11008 / 11008 -> 4096): 2 chunks 4.00 / 7.02 / 6.20, 4 chunks 3.98 / 6.22 / 6.45,
    // 8 chunks 4.24 / 6.45 / 6.95 - rows that fit one round of up to 16 waves take 4, longer rows many short rounds
#ifdef BW_TUNE   // measurement builds only (-DBW_TUNE, never the library build.py makes): kernel choices from the environment, for A/B runs
    if (const char* e = getenv("BW_W4_KB")) {
        switch (atoi(e)) {
            case 2: return launch_w4_kb<GROUP, MT, 2>(a, stream);
            case 4: return launch_w4_kb<GROUP, MT, 4>(a, stream);
            case 8: return launch_w4_kb<GROUP, MT, 8>(a, stream);
        }
    }
#endif
    if (a.nchunks <= 64) return launch_w4_kb<GROUP, MT, 4>(a, stream);
    return launch_w4_kb<GROUP, MT, 2>(a, stream);
}

// ---- 8-bit, up to four MFMA rows: the same integer-operand scheme ----------------------------------------------
//
// A byte in bits 0-7 of a half is the subnormal q * 2^-24, so a packed word becomes two operand dwords with two byte
// permutes (bytes 0, 1 and bytes 2, 3, each byte zero-extended to a half): in natural k order, with a single
// accumulator class - sum x q = 2^24 P - and x staged as it lies in memory, no permutation.  A chunk is 64 weights
// of a row (two MFMAs); with groups of 128 two chunks accumulate into one group sum, with groups of 32 the two groups
// of a chunk take the MFMA rows (m, group) as in the 4-bit kernel.  Weights arrive as in qgemv_w4_kernel (whole
// cache lines, non-temporal, through LDS); everything before the final sum is private to a wave.
template <int GROUP, int MT, int KB>
__global__ __launch_bounds__(1024) void qgemv_w8_kernel(const GemvArgs a) {
    constexpr int GPC = GROUP >= 64 ? 1 : 64 / GROUP;     // groups per chunk
    constexpr int CPG = GROUP >= 64 ? GROUP / 64 : 1;     // chunks per group
    constexpr int ROWS = MT * GPC;                        // MFMA rows in use: (m, group of the chunk)
    static_assert(ROWS <= 4, "the outputs must fit the four rows the lanes with kq == 0 hold");
    static_assert(KB % 2 == 0, "weights are requested in pairs of chunks");
    constexpr int GL = GROUP / 8;                         // staging lanes per group (8 halves each)
    constexpr int P = KB / 2;                             // pairs of chunks per wave and round
    constexpr int UPR = KB * 8;                           // 8-half units per activation row and round
    constexpr int XL = (MT * UPR + 63) / 64;              // unit loads per lane and round
    constexpr int ROW_BYTES = KB * 128 + 16, X_BYTES = ROWS * ROW_BYTES;
    constexpr int KBG = KB * 64 / GROUP, MP = KBG | 1;    // groups a wave covers per round; odd row pitch of its (scale, zp) block
    constexpr int ML = (KBG + 3) / 4;                     // 2-byte requests per lane, array and round
    constexpr int META_BYTES = (16 * MP * 4 + 15) & ~15;
    constexpr int WAVE_BYTES = X_BYTES + META_BYTES + P * WeightTile::kPair;
    constexpr uint32_t kOob = 0x80000000u;
    static_assert(UPR % GL == 0, "a group's staging lanes must not straddle activation rows");
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, nwaves = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nl = lane & 15, kq = lane >> 4;
    const uint32_t n0 = blockIdx.x * 16;
    // LDS: [wave 0: x tile | (scale, zero point) pairs of its groups, 16 rows x MP | weight batch] ... [partial sums]
    char* xs = smem + wave * WAVE_BYTES;
    uint32_t* meta = reinterpret_cast<uint32_t*>(xs + X_BYTES);
    char* wt = xs + X_BYTES + META_BYTES;
    float* red = reinterpret_cast<float*>(smem + nwaves * WAVE_BYTES);

    // the bias of the outputs the first MT waves will store, requested before anything else
    uint32_t bias_v = 0;
    if (wave < MT && a.bias)
        bias_v = __builtin_amdgcn_raw_buffer_load_b16(make_rsrc(a.bias, (uint32_t)a.N * 2), (n0 + nl) * 2, 0, 0);

    // ---- per-lane parts of the addresses (the per-wave and per-round parts go into the descriptors)
    const uint32_t m_off = ((uint32_t)(lane >> 2) * a.groups + (lane & 3)) * 2;
    uint32_t* m_dst = meta + (lane >> 2) * MP + (lane & 3);
    // x: unit u = lane + 64 i of the round: activation row u / UPR, unit ku = u % UPR, kept in memory order
    uint32_t x_off[XL], x_dst[XL];
#pragma unroll
    for (int i = 0; i < XL; i++) {
        const int u = lane + 64 * i, m = u / UPR, ku = u % UPR;
        x_off[i] = (MT == 1 || m < a.M) ? (uint32_t)(m * a.ldx + ku * 8) * 2 : kOob;
        x_dst[i] = m * GPC * ROW_BYTES + ku * 16;
    }
    uint32_t w_off[2];
    {
        const int r = lane >> 3, p = (lane & 7) ^ r;
        w_off[0] = (uint32_t)r * a.row_bytes + (p >> 2) * 64 + (p & 3) * 16;
        w_off[1] = w_off[0] + 8u * a.row_bytes;
    }

    float acc[MT];
#pragma unroll
    for (int r = 0; r < MT; r++) acc[r] = 0.f;
    const char* xrow = xs + (nl < ROWS ? nl : ROWS - 1) * ROW_BYTES + kq * 32;
    const uint32_t* mrow = meta + nl * MP;
    int c0 = wave * KB;
    while (true) {
        // ---- requests, small things first (loads return in order): scales / zero points, x, then the weights
        const uint32_t g0 = (uint32_t)c0 * 64 / GROUP;    // first group of the round
        const __amdgpu_buffer_rsrc_t rs = make_rsrc_at(a.scale, a.meta_bytes, (n0 * a.groups + g0) * 2),
                                     rz = make_rsrc_at(a.zp, a.meta_bytes, (n0 * a.groups + g0) * 2),
                                     rx = make_rsrc_at(a.x, a.x_bytes, (uint32_t)c0 * 128),
                                     rw = make_rsrc_at(a.qweight, a.w_bytes, n0 * (uint32_t)a.row_bytes + (uint32_t)c0 * 64);
        const int glim = min(KBG, a.groups - (int)g0);    // groups of the round that exist (the others read as zero)
        uint32_t ms[ML], mz[ML];
#pragma unroll
        for (int t = 0; t < ML; t++) {
            const uint32_t off = (lane & 3) + 4 * t < glim ? m_off : kOob;
            ms[t] = __builtin_amdgcn_raw_buffer_load_b16(rs, off + 8 * t, 0, 0);
            mz[t] = __builtin_amdgcn_raw_buffer_load_b16(rz, off + 8 * t, 0, 0);
        }
        u4 xr[XL];
#pragma unroll
        for (int i = 0; i < XL; i++) {
            uint32_t xo = x_off[i];
            if constexpr (MT > 1) {                           // one row: the end of x is the end of the buffer
                const int ku = (lane + 64 * i) % UPR;
                xo = c0 * 64 + ku * 8 < a.K ? xo : kOob;
            }
            xr[i] = __builtin_amdgcn_raw_buffer_load_b128(rx, xo, 0, 0);
        }
        asm volatile("" ::: "memory");
        static_for<0, KB>([&](auto ic) {
            constexpr int q = decltype(ic)::value / 2, i = decltype(ic)::value % 2;
            // (the instruction's immediate offset moves the LDS destination as well as the memory address: taken off again here)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (__attribute__((address_space(3))) void*)(wt + q * (WeightTile::kPair - 128) + i * WeightTile::kHalf),
                                                     16, w_off[i], 0, q * 128, WeightTile::kAuxNt);
        });
        asm volatile("" ::: "memory");

        // ---- scales / zero points -> this wave's block, as (scale | zero point << 16)
#pragma unroll
        for (int t = 0; t < ML; t++)
            if (4 * t + 3 < KBG || (lane & 3) + 4 * t < KBG) m_dst[4 * t] = ms[t] | (mz[t] << 16);
        // ---- the round's activations, as they lie in memory (into the row of their group where a chunk holds two
        // groups, zeros into the other's row); and -2^-24 * sum(x) per group
        float nsum[XL];
#pragma unroll
        for (int i = 0; i < XL; i++) {
            u4 v = xr[i];
            if (a.x_bf16) {
#pragma unroll
                for (int j = 0; j < 4; j++) v[j] = bf16x2_to_f16x2(v[j]);
            }
            if (MT * UPR >= 64 * (i + 1) || lane + 64 * i < MT * UPR) {
                const int my_group = (((lane + 64 * i) % UPR) * 8 % 64) / (GROUP >= 64 ? 64 : GROUP);   // group of its chunk this unit lies in
#pragma unroll
                for (int g = 0; g < GPC; g++) {
                    const bool mine = GPC == 1 || g == my_group;
                    *reinterpret_cast<u4*>(xs + x_dst[i] + g * ROW_BYTES) = mine ? v : u4{0u, 0u, 0u, 0u};
                }
            }
            float t = 0.f;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const h2 p = __builtin_bit_cast(h2, (uint32_t)v[j]);
                t -= (float)p[0];
                t -= (float)p[1];
            }
            nsum[i] = lanes_sum<GL>(t) * 0x1p-24f;
        }
        __builtin_amdgcn_wave_barrier();
        asm volatile("" ::: "memory");
        f4 p = {0.f, 0.f, 0.f, 0.f};
        static_for<0, KB>([&](auto bc) {
            constexpr int b = decltype(bc)::value;
            if constexpr ((b & 1) == 0) {                     // the pair's two load instructions have landed in LDS
                wait_loads<KB - 2 - b>();
                __builtin_amdgcn_wave_barrier();
                asm volatile("" ::: "memory");                // the reads below stay below
            }
            const u4 w = WeightTile::fetch(wt, b, lane);
            u4 b0, b1;                                    // B operands: the bytes of words 0, 1 and of words 2, 3 as halves
#pragma unroll
            for (int j = 0; j < 2; j++) {
                b0[2 * j] = __builtin_amdgcn_perm(0u, w[j], 0x0C010C00u);
                b0[2 * j + 1] = __builtin_amdgcn_perm(0u, w[j], 0x0C030C02u);
                b1[2 * j] = __builtin_amdgcn_perm(0u, w[2 + j], 0x0C010C00u);
                b1[2 * j + 1] = __builtin_amdgcn_perm(0u, w[2 + j], 0x0C030C02u);
            }
            const h8* xp = reinterpret_cast<const h8*>(xrow + b * 128);
            if constexpr (b % CPG == 0) p = f4{0.f, 0.f, 0.f, 0.f};
            p = __builtin_amdgcn_mfma_f32_16x16x32_f16(xp[0], __builtin_bit_cast(h8, b0), p, 0, 0, 0);
            p = __builtin_amdgcn_mfma_f32_16x16x32_f16(xp[1], __builtin_bit_cast(h8, b1), p, 0, 0, 0);
            if constexpr (b % CPG == CPG - 1) {
#pragma unroll
                for (int g = 0; g < GPC; g++) {
                    constexpr int gbase = (b / CPG) * GPC;    // first group of the round this chunk closes
                    const uint32_t sz = mrow[gbase + g];
                    const float sf = half_of(sz, 0), zf = half_of(sz, 1);
#pragma unroll
                    for (int m = 0; m < MT; m++) {
                        // the sum of (row m, group) sits in the lanes that staged it: unit m * UPR + (gbase + g) * GL
                        const int u = m * UPR + (gbase + g) * GL, r = m * GPC + g;
                        const float ns = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, nsum[u / 64]), u % 64));
                        acc[m] = __builtin_fmaf(sf, __builtin_fmaf(zf, ns, p[r]), acc[m]);
                    }
                }
            }
        });
        c0 += nwaves * KB;
        if (c0 >= a.nchunks) break;                       // wave-uniform
        __builtin_amdgcn_s_waitcnt(0xC07F);               // lgkmcnt(0): everything has been read out of LDS, the next round may land
        __builtin_amdgcn_wave_barrier();
        asm volatile("" ::: "memory");
    }

    // acc[m] = 2^-24 * partial y[m][n = nl] in the lanes with kq == 0
    if (kq == 0) {
#pragma unroll
        for (int r = 0; r < MT; r++) red[(wave * MT + r) * 16 + nl] = acc[r];
    }
    lds_barrier();
    if (wave < MT) {
        const int m = wave;
        float part[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (kq + 4 * i < nwaves) part[i] = red[((kq + 4 * i) * MT + m) * 16 + nl];
        float v = (part[0] + part[1]) + (part[2] + part[3]);
        v += __shfl_xor(v, 16);
        v += __shfl_xor(v, 32);
        const uint32_t n = n0 + nl;
        asm volatile("" : "+v"(bias_v));                      // the wait for the bias belongs here, not behind its request
        if (kq == 0 && m < a.M && n < (uint32_t)a.N) {
            v = __builtin_fmaf(v, 0x1p24f, half_of(bias_v, 0));
            a.y[(int64_t)m * a.ldy + n] = (_Float16)v;
        }
    }
}

template <int GROUP, int MT, int KB>
constexpr size_t w8_lds_bytes(int nwaves) {
    constexpr int GPC = GROUP >= 64 ? 1 : 64 / GROUP, MP = (KB * 64 / GROUP) | 1;
    constexpr int WAVE_BYTES = MT * GPC * (KB * 128 + 16) + ((16 * MP * 4 + 15) & ~15) + (KB / 2) * WeightTile::kPair;
    return (size_t)nwaves * (WAVE_BYTES + MT * 64);
}

template <int GROUP, int MT, int KB>
int launch_w8_kb(const GemvArgs& a, hipStream_t stream) {
    int nwaves = (a.nchunks + KB - 1) / KB;
    if (nwaves > 16) nwaves = 16;
    while (nwaves > 1 && w8_lds_bytes<GROUP, MT, KB>(nwaves) > (size_t)160 * 1024) nwaves--;
    const size_t lds = w8_lds_bytes<GROUP, MT, KB>(nwaves);
    if (lds > (size_t)160 * 1024 || nwaves < MT) return BW_EUNSUPPORTED;
    auto kern = qgemv_w8_kernel<GROUP, MT, KB>;
    BW_NOTE_KERNEL("qgemv_w8_kernel", GROUP, MT, KB);
    static uint64_t big_lds_devices = 0;                   // per instantiation
    if (lds > 64 * 1024 && !bw_allow_big_lds(reinterpret_cast<const void*>(kern), big_lds_devices)) return BW_ELAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)((a.N + 15) / 16)), dim3(nwaves * 64), lds, stream, a);
    return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
}

template <int GROUP, int MT>
int launch_w8(const GemvArgs& a, hipStream_t stream) {
#ifdef BW_TUNE
    if (const char* e = getenv("BW_W8_KB")) {
        switch (atoi(e)) {
            case 2: return launch_w8_kb<GROUP, MT, 2>(a, stream);
            case 4: return launch_w8_kb<GROUP, MT, 4>(a, stream);
            case 8: return launch_w8_kb<GROUP, MT, 8>(a, stream);
        }
    }
#endif
    // Chunks a wave requests per round: the largest batch whose workgroups still all fit the chip at once (a grid of
    // 688 tiles wants three workgroups per compute unit, and the weight batches are what fills LDS).  Measured, M = 1,
    // groups of 128 (us: 4096 x 4096 / 4096 -> 11008 / 11008 -> 4096): 2 chunks 5.59 / 10.40 / 11.81, 4 chunks
    // 5.59 / 12.45 / 11.42, 8 chunks 5.36 / 11.90 / 11.39.
    const int cus = bw_device_cus(), tiles = (a.N + 15) / 16;
    const size_t per_wg = (size_t)160 * 1024 / (size_t)(tiles <= cus ? 1 : (tiles + cus - 1) / cus > 4 ? 4 : (tiles + cus - 1) / cus);
    auto waves = [&](int kb) { const int w = (a.nchunks + kb - 1) / kb; return w > 16 ? 16 : w; };
    if (w8_lds_bytes<GROUP, MT, 8>(waves(8)) <= per_wg) return launch_w8_kb<GROUP, MT, 8>(a, stream);
    if (w8_lds_bytes<GROUP, MT, 4>(waves(4)) <= per_wg) return launch_w8_kb<GROUP, MT, 4>(a, stream);
    return launch_w8_kb<GROUP, MT, 2>(a, stream);
}

// ---- 2-bit, M <= 2: the same integer-operand scheme ---------------------------------------------------------
//
// A masked 2-bit field at bits 2c..2c+1 (c = 0..3) of a half is the subnormal q * 4^c * 2^-24; the fields at bits
// 8-15 are brought down by one shift.  A word of 16 weights unpacks with 1 shift + 8 ANDs into four operand
// classes; class c accumulates in its own register quad and  sum x q = 2^24 (P0 + P1/4 + P2/16 + P3/64).
// A chunk is 256 weights of a row: 2, 4 or 8 groups.  Row m * NGC + g of the MFMA tile carries group g of
// activation row m: a lane reads its A operand from the staged x only where its 32-value slice lies in that
// group and from a row of zeros elsewhere, so output row m * NGC + g is the group's partial sum.
template <int LANES>
BW_DEV float lanes_sum_small(float v) {                  // aligned runs of 2, 4 or 8 lanes
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    if constexpr (LANES >= 4)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    if constexpr (LANES >= 8)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
    return v;
}

template <int GROUP, int MT, int KB>
__global__ __launch_bounds__(1024) void qgemv_w2_kernel(const GemvArgs a) {
    constexpr int NGC = 256 / GROUP;                      // groups per chunk
    constexpr int ROWS = MT * NGC;                        // MFMA rows in use: (m, group of the chunk)
    static_assert(ROWS <= 16, "one MFMA tile of rows");
    constexpr int SPG = GROUP / 32;                       // 32-value slices (half a lane load) per group
    constexpr int UPR = KB * 16;                          // 16-value units per activation row and round
    constexpr int XL = (MT * UPR + 63) / 64;              // unit loads per lane and round
    constexpr int ROW_BYTES = KB * 512 + 16;
    constexpr int X_BYTES = (MT + 1) * ROW_BYTES;         // the staged rows and one row of zeros
    constexpr int NS_BYTES = MT * KB * NGC * 4;
    constexpr int WAVE_BYTES = (X_BYTES + NS_BYTES + 15) & ~15;
    constexpr uint32_t kOob = 0x80000000u;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const int nl = lane & 15, kq = lane >> 4;
    const int n0 = blockIdx.x * 16;
    // LDS: [(scale, zero point) pairs, 16 rows x GP][wave 0: x rows, zero row, group sums] ... [partial sums]
    const int gcols = (a.groups + 31) & ~31, GP = gcols + 1;
    uint32_t* meta = reinterpret_cast<uint32_t*>(smem);
    char* after_meta = smem + ((16 * GP * 4 + 15) & ~15);
    char* xs = after_meta + wave * WAVE_BYTES;
    float* nsb = reinterpret_cast<float*>(xs + X_BYTES);
    float* red = reinterpret_cast<float*>(after_meta + nwaves * WAVE_BYTES);
    const __amdgpu_buffer_rsrc_t rw = make_rsrc(a.qweight, a.w_bytes), rx = make_rsrc(a.x, a.x_bytes),
                                 rs = make_rsrc(a.scale, a.meta_bytes), rz = make_rsrc(a.zp, a.meta_bytes);

    constexpr int ME = GROUP == 32 ? 4 : (GROUP == 64 ? 2 : 1);
    const uint32_t meta_base = (uint32_t)n0 * a.groups * 2;
    const int meta_entries = 16 * gcols;
    auto meta_off = [&](int e) {
        const int r = (e >> 5) & 15, c = (e & 31) + 32 * (e >> 9);
        return c < a.groups ? meta_base + (r * a.groups + c) * 2 : kOob;
    };
    auto meta_slot = [&](int e) { return ((e >> 5) & 15) * GP + (e & 31) + 32 * (e >> 9); };
    uint32_t ms[ME], mz[ME];
#pragma unroll
    for (int j = 0; j < ME; j++) {
        ms[j] = mz[j] = 0;
        if ((wave + j * nwaves) * 64 < meta_entries) {          // wave-uniform
            const uint32_t off = meta_off(tid + j * (int)blockDim.x);
            ms[j] = __builtin_amdgcn_raw_buffer_load_b16(rs, off, 0, 0);
            mz[j] = __builtin_amdgcn_raw_buffer_load_b16(rz, off, 0, 0);
        }
    }

    const uint32_t w_lane = (uint32_t)(n0 + nl) * a.row_bytes + kq * 16;
    // unit u = lane + 64 i of the round: activation row u / UPR, chunk b, 16-value unit w of the chunk; unit w is
    // word j = w % 4 of the 64-value slice kq_x = w / 4.  Class c of the unit goes to operand (p = j / 2, c) of
    // the lanes with kq == kq_x, second half if j is odd.
    uint32_t x_off[XL], x_dst[XL], ns_dst[XL];
#pragma unroll
    for (int i = 0; i < XL; i++) {
        const int u = lane + 64 * i, m = u / UPR, rest = u % UPR, b = rest >> 4, w = rest & 15;
        x_off[i] = m < a.M ? (uint32_t)(m * a.ldx + b * 256 + w * 16) * 2 : kOob;
        x_dst[i] = m * ROW_BYTES + b * 512 + ((w >> 1) & 1) * 256 + (w >> 2) * 16 + (w & 1) * 8;
        ns_dst[i] = (m * KB + b) * NGC + (w * 16) / GROUP;
    }
    u4 xr[XL][2], wr[KB];
    auto issue = [&](int c0) {
#pragma unroll
        for (int i = 0; i < XL; i++) {
            const int rest = (lane + 64 * i) % UPR;
            const uint32_t xo = (x_off[i] != kOob && c0 * 256 + rest * 16 < a.K) ? x_off[i] + c0 * 512 : kOob;
            xr[i][0] = __builtin_amdgcn_raw_buffer_load_b128(rx, xo, 0, 0);
            xr[i][1] = __builtin_amdgcn_raw_buffer_load_b128(rx, xo == kOob ? kOob : xo + 16, 0, 0);
        }
        asm volatile("" ::: "memory");
        const uint32_t off = c0 * 64 < a.row_bytes ? w_lane + c0 * 64 : kOob;
#pragma unroll
        for (int b = 0; b < KB; b++) wr[b] = __builtin_amdgcn_raw_buffer_load_b128(rw, off + b * 64, 0, 0);
        asm volatile("" ::: "memory");
    };
    int c0 = wave * KB;
    issue(c0);

#pragma unroll
    for (int j = 0; j < ME; j++) {
        const int e = tid + j * (int)blockDim.x;
        if (e < meta_entries) meta[meta_slot(e)] = ms[j] | (mz[j] << 16);
    }
    for (int e = tid + ME * (int)blockDim.x; e < meta_entries; e += blockDim.x) {
        const uint32_t off = meta_off(e);
        const uint32_t s2 = __builtin_amdgcn_raw_buffer_load_b16(rs, off, 0, 0);
        const uint32_t z2 = __builtin_amdgcn_raw_buffer_load_b16(rz, off, 0, 0);
        meta[meta_slot(e)] = s2 | (z2 << 16);
    }
    // the row of zeros behind the staged rows
    for (int o = lane * 4; o < ROW_BYTES; o += 256) *reinterpret_cast<uint32_t*>(xs + MT * ROW_BYTES + o) = 0u;
    __syncthreads();

    // this lane's MFMA row: activation row and group of the chunk; its two 32-value slices (p = 0, 1) are live
    // where they lie in that group
    const int row_m = nl / NGC < MT ? nl / NGC : MT - 1, row_g = nl % NGC;
    const char* xbase[2];
#pragma unroll
    for (int p = 0; p < 2; p++) {
        const bool live = nl < ROWS && (2 * kq + p) / SPG == row_g;
        xbase[p] = xs + (live ? row_m : MT) * ROW_BYTES + p * 256 + kq * 16;
    }
    // the four output rows this lane holds: rows 4 kq + r
    int out_m[4], out_g[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int row = 4 * kq + r;
        out_m[r] = row / NGC < MT ? row / NGC : MT - 1;
        out_g[r] = row % NGC;
    }
    f4 acc = {0.f, 0.f, 0.f, 0.f};
    const uint32_t* mrow = meta + nl * GP;
    while (true) {
        // stage the round's activations: per 16 values the pairs (x_f, x_f+8), f = 0..7, which is the order in which
        // the masks below emit the fields of a word; class c takes pairs c and c + 4.  And -2^-24 sum(x) per group.
#pragma unroll
        for (int i = 0; i < XL; i++) {
            uint32_t in[8], o[8];
#pragma unroll
            for (int j = 0; j < 4; j++) { in[j] = xr[i][0][j]; in[4 + j] = xr[i][1][j]; }
            if (a.x_bf16) {
#pragma unroll
                for (int j = 0; j < 8; j++) in[j] = bf16x2_to_f16x2(in[j]);
            }
            permute_unit<2>(in, o);
            const bool mine = MT * UPR >= 64 * (i + 1) || lane + 64 * i < MT * UPR;
            if (mine) {
#pragma unroll
                for (int c = 0; c < 4; c++) *reinterpret_cast<u2*>(xs + x_dst[i] + c * 64) = u2{o[c], o[c + 4]};
            }
            float t = 0.f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const h2 pr = __builtin_bit_cast(h2, in[j]);
                t -= (float)pr[0];
                t -= (float)pr[1];
            }
            t = lanes_sum_small<GROUP / 16>(t) * 0x1p-24f;
            if (mine && (lane & (GROUP / 16 - 1)) == 0) nsb[ns_dst[i]] = t;
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int b = 0; b < KB; b++) {
            const u4 w = wr[b];
            f4 pc[4];
#pragma unroll
            for (int c = 0; c < 4; c++) pc[c] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int p = 0; p < 2; p++) {
                const uint32_t wa = w[2 * p], sa = wa >> 8, wb = w[2 * p + 1], sb = wb >> 8;
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const uint32_t mask = 0x00030003u << (2 * c);
                    const u4 bop = {wa & mask, sa & mask, wb & mask, sb & mask};
                    const h8 xa = *reinterpret_cast<const h8*>(xbase[p] + b * 512 + c * 64);
                    pc[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa, __builtin_bit_cast(h8, bop), pc[c], 0, 0, 0);
                }
            }
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const uint32_t sz = mrow[min((c0 + b) * NGC + out_g[r], gcols - 1)];   // chunks past K: zero weights and x
                const float sf = half_of(sz, 0), zf = half_of(sz, 1);
                const float ns = nsb[(out_m[r] * KB + b) * NGC + out_g[r]];
                float t = __builtin_fmaf(pc[3][r], 0.25f, pc[2][r]);
                t = __builtin_fmaf(t, 0.25f, pc[1][r]);
                t = __builtin_fmaf(t, 0.25f, pc[0][r]);
                acc[r] = __builtin_fmaf(sf, __builtin_fmaf(zf, ns, t), acc[r]);
            }
        }
        c0 += nwaves * KB;
        if (c0 >= a.nchunks) break;                       // wave-uniform
        __builtin_amdgcn_wave_barrier();
        issue(c0);
    }

    // acc[r] = 2^-24 * partial of row 4 kq + r = (m, g); add the groups of each m, one value per (m, n) and wave
    if constexpr (NGC >= 4) {
        float v = (acc[0] + acc[1]) + (acc[2] + acc[3]);
        if constexpr (NGC == 8) v += __shfl_xor(v, 16);
        const int m = (4 * kq) / NGC;
        if (m < MT && (NGC == 4 || (kq & 1) == 0)) red[(wave * MT + m) * 16 + nl] = v;
    } else {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int m = 2 * kq + h;
            if (m < MT) red[(wave * MT + m) * 16 + nl] = acc[2 * h] + acc[2 * h + 1];
        }
    }
    __syncthreads();
    for (int m = wave; m < MT; m += nwaves) {
        float v = 0.f;
        for (int w = kq; w < nwaves; w += 4) v += red[(w * MT + m) * 16 + nl];
        v += __shfl_xor(v, 16);
        v += __shfl_xor(v, 32);
        const int n = n0 + nl;
        if (kq == 0 && m < a.M && n < a.N) {
            v *= 0x1p24f;
            if (a.bias) v += (float)a.bias[n];
            a.y[(int64_t)m * a.ldy + n] = (_Float16)v;
        }
    }
}

template <int GROUP, int MT, int KB>
int launch_w2_kb(const GemvArgs& a, hipStream_t stream) {
    constexpr int NGC = 256 / GROUP;
    constexpr int WAVE_BYTES = ((MT + 1) * (KB * 512 + 16) + MT * KB * NGC * 4 + 15) & ~15;
    const int gcols = (a.groups + 31) & ~31;
    const size_t fixed = (size_t)((16 * (gcols + 1) * 4 + 15) & ~15);
    int nwaves = (a.nchunks + KB - 1) / KB;
    if (nwaves > 16) nwaves = 16;
    while (nwaves > 1 && fixed + (size_t)nwaves * (WAVE_BYTES + MT * 64) > (size_t)150 * 1024) nwaves--;
    const size_t lds = fixed + (size_t)nwaves * (WAVE_BYTES + MT * 64);
    if (lds > (size_t)150 * 1024) return BW_EUNSUPPORTED;
    auto kern = qgemv_w2_kernel<GROUP, MT, KB>;
    BW_NOTE_KERNEL("qgemv_w2_kernel", GROUP, MT, KB);
    static uint64_t big_lds_devices = 0;                   // per instantiation
    if (lds > 64 * 1024 && !bw_allow_big_lds(reinterpret_cast<const void*>(kern), big_lds_devices)) return BW_ELAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)((a.N + 15) / 16)), dim3(nwaves * 64), lds, stream, a);
    return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
}

template <int GROUP, int MT>
int launch_w2(const GemvArgs& a, hipStream_t stream) {
    // chunks a wave has in flight per round: rows are short at 2 bits (K = 4096 is 16 chunks), so 2, and 1 where
    // groups of 32 make the scale block as large as half the weights
    if (GROUP == 32 && a.nchunks <= 16) return launch_w2_kb<GROUP, MT, 1>(a, stream);
    return launch_w2_kb<GROUP, MT, 2>(a, stream);
}

constexpr int kLdsBudget = 150 * 1024;

template <int BITS, int GROUP, int MT, int NT>
int launch_tiles_nt(const GemvArgs& a, int grid, int nwaves, size_t lds, hipStream_t stream) {
    auto kern = qgemv_tiles_kernel<BITS, GROUP, MT, NT>;
    BW_NOTE_KERNEL("qgemv_tiles_kernel", BITS, GROUP, MT, NT);
    static uint64_t big_lds_devices = 0;                   // per instantiation
    if (lds > 64 * 1024 && !bw_allow_big_lds(reinterpret_cast<const void*>(kern), big_lds_devices)) return BW_ELAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(nwaves * 64), lds, stream, a);
    return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
}

template <int BITS, int GROUP, int MT, int DEPTH, bool LOOP>
int launch_rounds_depth(const GemvArgs& a, int grid, int nwaves, size_t lds, hipStream_t stream) {
    auto kern = qgemv_rounds_kernel<BITS, GROUP, MT, DEPTH, LOOP>;
    BW_NOTE_KERNEL("qgemv_rounds_kernel", BITS, GROUP, MT, DEPTH, (int)LOOP);
    static uint64_t big_lds_devices = 0;                   // per instantiation
    if (lds > 64 * 1024 && !bw_allow_big_lds(reinterpret_cast<const void*>(kern), big_lds_devices)) return BW_ELAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(nwaves * 64), lds, stream, a);
    return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
}

// 3 <= M <= 16 through qgemv_tiles_kernel (K fits one round of a workgroup) or qgemv_rounds_kernel.
// BW_EUNSUPPORTED = this layout is not taken (scale arrays that 4-byte requests cannot address, a scale block that
// does not fit LDS, short K, more rounds than the registers hold); the caller falls back to qgemv_kernel
template <int BITS, int GROUP, int MT>
int launch_tiles(GemvArgs a, hipStream_t stream) {
    using C = GemvCfg<BITS, GROUP, MT>;
    constexpr int KBW = BITS == 4 ? 2 : (BITS == 8 ? 4 : 1);
    constexpr int X_BYTES = MT * (KBW * C::CHUNK_K + 8) * 2;
    constexpr size_t kLds = 160 * 1024;
    // 4-byte requests for scales, zero points and bias: aligned arrays, an even number of entries per row
    if (!bw_aligned(a.scale, 4) || !bw_aligned(a.zp, 4) || a.groups % 2 || (a.bias && (!bw_aligned(a.bias, 4) || a.N % 2)))
        return BW_EUNSUPPORTED;
    const size_t meta_lds = (size_t)16 * (a.groups | 1) * 4;
    int nwaves = (a.nchunks + KBW - 1) / KBW;
    if (nwaves > 16) nwaves = 16;
    while (nwaves > 1 && (size_t)nwaves * (X_BYTES + MT * 64) + meta_lds > kLds) nwaves--;
    const int rounds = (a.nchunks + nwaves * KBW - 1) / (nwaves * KBW);
    if (nwaves * 64 < 16 * MT) return BW_EUNSUPPORTED;
    a.ntiles = (a.N + 15) / 16;
    if (rounds == 1) {
        // one 4-byte request per thread brings in a tile's scale block, and the waves wait on a counter for the
        // ceil(8 groups / 64) waves that hold those requests: both need 8 groups <= threads.  (K <= 256 per wave
        // and group >= 32 give exactly that today; a launch that breaks it must fall back, not hang.)
        if (8 * a.groups > nwaves * 64) return BW_EUNSUPPORTED;
        // every workgroup resident at once (a CU holds 16 waves of this kernel: up to 128 registers each), each
        // running up to NTMAX tiles - and no more tiles per workgroup than that takes: fewer, longer workgroups would
        // read x fewer times but leave CUs without a weight stream (4096 x 4096 at 16 rows: 6.05 us with one tile per
        // workgroup, 7.24 with two, 8.61 with three; 4096 -> 11008: 9.67 with three, 10.63 with four)
        constexpr int NTMAX = BITS == 8 ? (MT == 16 ? 2 : 3) : 4;
        const int slots = bw_device_cus() * (16 / nwaves);
        int nt = (a.ntiles + slots - 1) / slots;
        if (nt > NTMAX) nt = NTMAX;
#ifdef BW_TUNE
        if (const char* e = getenv("BW_GEMV_NT")) { const int v = atoi(e); if (v >= nt && v <= NTMAX) nt = v; }
#endif
        size_t xred;
        while (true) {
            xred = (size_t)nwaves * X_BYTES;                                     // x tiles, later the partial sums
            if (xred < (size_t)nt * nwaves * MT * 64) xred = (size_t)nt * nwaves * MT * 64;
            if (xred + nt * meta_lds + 16 <= kLds || nt == 1) break;
            nt--;
        }
        const size_t lds = xred + nt * meta_lds + 16;                            // + the "scales are in LDS" counter
        if (lds > kLds) return BW_EUNSUPPORTED;
        const int grid = (a.ntiles + nt - 1) / nt;
        // 8 bits (four 16-byte loads per lane and tile, so fewer tiles fit the registers): measured to pay only
        // with more than one tile per workgroup and every workgroup resident
        if (BITS == 8 && (nt < 2 || grid > slots)) return BW_EUNSUPPORTED;
        a.meta_lds_off = (int)xred;
        a.nsteps = nt;
        if (nt == 1) return launch_tiles_nt<BITS, GROUP, MT, 1>(a, grid, nwaves, lds, stream);
        if (nt == 2) return launch_tiles_nt<BITS, GROUP, MT, 2>(a, grid, nwaves, lds, stream);
        if constexpr (NTMAX >= 3)
            if (nt == 3) return launch_tiles_nt<BITS, GROUP, MT, 3>(a, grid, nwaves, lds, stream);
        if constexpr (NTMAX >= 4)
            if (nt == 4) return launch_tiles_nt<BITS, GROUP, MT, 4>(a, grid, nwaves, lds, stream);
        return BW_EUNSUPPORTED;
    }
    // rounds: the tile's whole scale block comes in with at most four 4-byte requests per thread
    const size_t lds = (size_t)nwaves * (X_BYTES + MT * 64) + meta_lds;
    if (lds > kLds || 8 * a.groups > 4 * nwaves * 64) return BW_EUNSUPPORTED;
    a.nsteps = rounds;
    // Rounds a workgroup keeps requested ahead: all of them while they fit the 128 registers a wave of a 16-wave
    // workgroup has (8-bit rounds are four 16-byte loads per lane), else a ring of two where that fits.
    constexpr int RMAX = (BITS == 8 && MT >= 8) ? 2 : 3;
    constexpr bool RRING = BITS != 8 && MT < 16;
    if (rounds == 2) return launch_rounds_depth<BITS, GROUP, MT, 2, false>(a, a.ntiles, nwaves, lds, stream);
    if constexpr (RMAX >= 3)
        if (rounds == 3) return launch_rounds_depth<BITS, GROUP, MT, 3, false>(a, a.ntiles, nwaves, lds, stream);
    if constexpr (RRING) return launch_rounds_depth<BITS, GROUP, MT, 2, true>(a, a.ntiles, nwaves, lds, stream);
    return BW_EUNSUPPORTED;
}

template <int BITS, int GROUP, int MT, int KB>
int launch_gemv_kb(const GemvArgs& a, hipStream_t stream) {
    using C = GemvCfg<BITS, GROUP, MT>;
    constexpr int BK = KB * C::CHUNK_K, X_BYTES = MT * (BK + 8) * 2;
    const size_t fixed = (size_t)((16 * (a.groups | 1) * 4 + 15) & ~15);
    int nwaves = (a.nchunks + KB - 1) / KB;
    // 16 activation rows: when the grid has more workgroups than the chip has CUs, 8-wave workgroups (two fit
    // a CU) balance better than 16-wave ones; a grid of at most one workgroup per CU wants all 16 waves
    const int max_waves = (MT > 8 && (a.N + 15) / 16 > 256) ? 8 : C::MAX_WAVES;
    if (nwaves > max_waves) nwaves = max_waves;
    while (nwaves > 1 && fixed + (size_t)nwaves * (X_BYTES + MT * 64) > (size_t)kLdsBudget) nwaves--;
    const size_t lds = fixed + (size_t)nwaves * (X_BYTES + MT * 64);
    if (lds > (size_t)kLdsBudget) return BW_EUNSUPPORTED;
    auto kern = qgemv_kernel<BITS, GROUP, MT, KB>;
    BW_NOTE_KERNEL("qgemv_kernel", BITS, GROUP, MT, KB);
    static uint64_t big_lds_devices = 0;                   // per instantiation
    if (lds > 64 * 1024 && !bw_allow_big_lds(reinterpret_cast<const void*>(kern), big_lds_devices)) return BW_ELAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)((a.N + 15) / 16)), dim3(nwaves * 64), lds, stream, a);
    return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
}

template <int BITS, int GROUP, int MT>
int launch_gemv_mt(const GemvArgs& a, hipStream_t stream) {
    using C = GemvCfg<BITS, GROUP, MT>;
    // Chunks per wave and round, from timing Llama-shaped layers on MI355X: short rows want many small
    // waves (more requests in flight early), wide activation tiles want small batches (LDS, registers);
    // never more than ~16 KB of staged activations per wave.
    constexpr int fit = 8192 / (MT * C::CHUNK_K);
    int kb;
    if (MT >= 8) kb = a.nchunks <= 32 ? 1 : 2;
    else kb = (a.nchunks <= 32 && a.N < 8192) ? 2 : 4;
    if (kb > fit) kb = fit >= 4 ? 4 : (fit >= 2 ? 2 : 1);
    if (MT > 8 && kb > 2) kb = 2;                         // 16-wave workgroups leave a wave 128 registers
    if constexpr (MT <= 8)
        if (kb >= 4) return launch_gemv_kb<BITS, GROUP, MT, 4>(a, stream);
    if (kb >= 2) return launch_gemv_kb<BITS, GROUP, MT, 2>(a, stream);
    return launch_gemv_kb<BITS, GROUP, MT, 1>(a, stream);
}

// Rows from which qgemv_tiles_kernel (K fits one round: at most 16 * KBW chunks) or qgemv_rounds_kernel beats
// the kernels below, from timing the Llama-shaped layers on MI355X (4096 x 4096, 4096 -> 11008, 11008 -> 4096) at
// M = 1, 2, 4, 8, 16; 99 = never.  The formats with a subnormal-operand kernel keep it for M <= 2 where that wins;
// long rows pay more per round for x than qgemv_kernel's smaller rounds do, so 4-bit at groups of 64 and 128 and
// 8-bit stay there.
template <int BITS, int GROUP>
int tiles_min_rows(int nchunks) {
    constexpr int KBW = BITS == 4 ? 2 : (BITS == 8 ? 4 : 1);
    const bool one_round = nchunks <= 16 * KBW;
    if (BITS == 8) return one_round ? 2 : 99;
    if (BITS == 4) return GROUP == 128 ? (one_round ? 3 : 99) : GROUP == 64 ? (one_round ? 2 : 99) : (one_round ? 1 : 2);
    return GROUP == 32 ? 1 : (one_round ? (GROUP == 64 ? 1 : 2) : 3);
}

template <int BITS, int GROUP>
int launch_gemv(const GemvArgs& a, hipStream_t stream) {
    constexpr int KBW = BITS == 4 ? 2 : (BITS == 8 ? 4 : 1);
    const bool one_round = a.nchunks <= 16 * KBW;         // K fits one round of qgemv_tiles_kernel
    const bool many_tiles = (a.N + 15) / 16 > bw_device_cus();
    // The subnormal-operand kernels first, where they win (timed on the Llama-7B shapes, MI355X).
    if constexpr (BITS == 8) {
        // rows of the MFMA tile in use = M * groups per chunk, at most 4: faster than the tile kernels on every shape
        constexpr int GPC = GROUP >= 64 ? 1 : 64 / GROUP;
#ifdef BW_TUNE
        if (!getenv("BW_W8_OFF"))
#endif
        if (a.M * GPC <= 4) {
            const int st = a.M == 1 ? launch_w8<GROUP, 1>(a, stream)
                         : a.M == 2 ? launch_w8<GROUP, 2>(a, stream)
                                    : launch_w8<GROUP, (GPC == 1 ? 4 : 2)>(a, stream);
            if (st != BW_EUNSUPPORTED) return st;
        }
    }
    if constexpr (BITS == 4) {
        // rows in use = M * groups per chunk, at most 4.  At 3 and 4 rows (groups of 128) the tile kernel is ahead
        // where a workgroup gets several tiles out of one staging of x (one round of K, more tiles than compute
        // units: 7.4 against 7.9 us on 4096 -> 11008), this one elsewhere (4.4 against 4.7 us on 4096 x 4096, 7.4
        // against 8.5 us on 11008 -> 4096).
        const bool first = a.M <= 2 || !(one_round && many_tiles);
#ifdef BW_TUNE
        if (!getenv("BW_W4_OFF"))
#endif
        if (a.M * (128 / GROUP) <= 4 && first) {
            const int st = a.M == 1 ? launch_w4<GROUP, 1>(a, stream)
                         : a.M == 2 ? launch_w4<GROUP, (GROUP >= 64 ? 2 : 1)>(a, stream)
                                    : launch_w4<GROUP, (GROUP == 128 ? 4 : 1)>(a, stream);
            if (st != BW_EUNSUPPORTED) return st;
        }
    }
#ifdef BW_TUNE
    if (!getenv("BW_TILES_OFF"))
#endif
    if (a.M >= tiles_min_rows<BITS, GROUP>(a.nchunks)) {
        const int st = a.M <= 4 ? launch_tiles<BITS, GROUP, 4>(a, stream)
                                : (a.M <= 8 ? launch_tiles<BITS, GROUP, 8>(a, stream) : launch_tiles<BITS, GROUP, 16>(a, stream));
        if (st != BW_EUNSUPPORTED) return st;
    }
    if constexpr (BITS == 2) {
        if (a.M <= 2) {
            const int st = a.M == 1 ? launch_w2<GROUP, 1>(a, stream) : launch_w2<GROUP, 2>(a, stream);
            if (st != BW_EUNSUPPORTED) return st;
        }
    }
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

extern "C" const char* bw_qgemv_last_kernel(void) { return g_last_kernel; }

extern "C" int bw_qgemv(const void* x, int act_dtype, int64_t M, int64_t K, int64_t ldx, const int32_t* qweight,
                        const void* scale16, const void* zp16, const void* bias, int64_t N, int bits, int group,
                        void* y, int64_t ldy, void* stream) {
    if (!x || !qweight || !scale16 || !zp16 || !y) return BW_EINVAL;
    if (!bw_shape_ok(N, K, bits, group) || M < 1 || M > 16 || ldx < K || ldy < N) return BW_EINVAL;
    if (act_dtype != BW_F16 && act_dtype != BW_BF16) return BW_EUNSUPPORTED;
    g_last_kernel = "";
    if (!bw_fast_shape(M, N, K, ldx, bits, group) || !bw_aligned(x, 16) || (ldx * 2) % 16 || !bw_aligned(qweight, 16))
        return bw_qgemm_generic(x, act_dtype, M, K, ldx, qweight, scale16, zp16, bias, N, bits, group, y, ldy, stream);
    GemvArgs a;
    a.x = x; a.qweight = qweight; a.scale = scale16; a.zp = zp16; a.bias = (const _Float16*)bias; a.y = (_Float16*)y;
    a.M = (int)M; a.N = (int)N; a.K = (int)K; a.ldx = (int)ldx; a.ldy = (int)ldy;
    a.groups = (int)(K / group);
    a.row_bytes = (int)(K * bits / 8);
    a.x_bf16 = act_dtype == BW_BF16;
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
