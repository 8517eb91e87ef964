// Prefill path: y[M][N] = x[M][K] @ W16[N][K]^T (+ bias) for any M, built for
// M >= 128 where the matrix cores are the bound.
//
// A workgroup of 4 waves owns a 128 (M) x 256 (N) output tile; each wave owns
// 128 x 64 of it (8 x 4 MFMA 16x16 tiles, 128 accumulator registers).  Per K
// step of one chunk (64 packed bytes per weight row):
//   * weights go global -> registers with one 128-bit load per lane per 16
//     rows, already in MFMA operand layout, and are unpacked in registers
//     to the float16 values the reference's dequantize kernel would store
//     (bitween/modules.py:55-58).  No wave unpacks a weight another wave of
//     the workgroup also unpacks; each weight is unpacked M/128 times overall.
//   * activations go global -> LDS once per workgroup, double buffered, and
//     every fragment read from LDS feeds 4 MFMAs.
// Two schedules of that loop.  Natural order (K a multiple of 128: step16 below):
// the activations go memory -> LDS without passing through registers (buffer
// loads with LDS destination), the weights are unpacked to natural k order, and
// the side work of an MFMA step is dealt out one instruction per MFMA.  Register
// staged (any other K: step8): the activations pass through registers and are
// permuted into the k order a cheaper unpack emits.
// Grids that fill the device run the natural-order schedule with 256 x 256
// tiles (a wave owns 256 x 64: all 256 accumulation registers): every weight
// is unpacked once for twice the rows.  Which tile height a call gets is
// gemm_tile_rows(); a short last round of tiles is cut along K (gemm_plan()),
// and the tiles are numbered so that the workgroups an XCD runs together share
// operand tiles in its L2 (GemmArgs::panel).
// Also holds the shape-generic fallback used when the fast layouts do not
// apply (odd K or group size): correct for everything the reference accepts.
#include "bw_qgemm_kernel.h"

#include <atomic>

bool bw_fast_shape(int64_t M, int64_t N, int64_t K, int64_t ldx, int bits, int group);

namespace {

// The natural-order schedule (activations memory -> LDS by buffer loads with LDS destination, step16) takes whole K
// steps of 128 values and offsets of rows past M that still fit 32 bits; other shapes run the register-staged kernel.
inline bool gemm_nat(int64_t M, int64_t K, int64_t ldx) {
#ifdef BW_TUNE   // measurement builds only (-DBW_TUNE, never the library build.py makes): kernel choices from the environment, for A/B runs
    if (const char* e = getenv("BW_GEMM_NAT")) if (atoi(e) == 0) return false;
#endif
    return K % 128 == 0 && (M + 256) * ldx * 2 < ((int64_t)1 << 32);
}

// Rows of a tile for this call.  Calls of at most 64 rows take 64-row tiles: half the MFMAs and half the activation
// traffic of a 128-row tile that would be at least half padding (17 ... 64 rows on the five Llama MLP / attention shapes at
// 4 bits: 0.84-0.95 of the 128-row time, same bits).  A 256-row tile unpacks every weight once for twice the rows and keeps the matrix pipe
// busier: a full round of 256-row tiles takes about 1.65 x the time of a full round of 128-row tiles for twice the
// work.  Which grid finishes first then depends on how each fills its rounds (one workgroup per CU): whole rounds,
// plus a last round that costs a full one when more than half full and about three quarters of one when its tiles are
// split along K (a workspace is on offer).  That model reproduces a sweep of both heights over K, N in {4096, 11008,
// 14336} and M = 512 ... 2048 (4 bits; e.g. 4096 -> 14336 at 2048 rows: 3.75 against 3.3 rounds, measured 207 against
// 184 us; 4096 x 4096 at 2048 rows: 1.0 against 1.24, measured 60 against 75 us); the 256-row grid is taken when it is
// ahead by 5 % or more.  Only with the natural-order schedule, and only while the split-K blocks of its plan fit the
// workspace on offer.
inline int gemm_tile_rows(int64_t M, int64_t N, int64_t K, int64_t ldx, int bits, bool have_workspace, size_t workspace_bytes) {
    if (!gemm_nat(M, K, ldx)) return 128;
    const int nchunks = gemm_chunks(K, bits, true);
#ifdef BW_TUNE
    if (const char* e = getenv("BW_GEMM_BM")) return atoi(e) == 256 ? 256 : atoi(e) == 64 ? 64 : 128;
#endif
    // (up to 128 rows as two 64-row tiles where N is at most 16 tiles wide: 4096 x 4096, 11008 -> 4096 and 14336 -> 4096 at
    // 80 ... 128 rows 0.88-0.95 of the 128-row time - half the partial-tile traffic of the K split -, but 1.06-1.11 at
    // N = 11008 and 14336, where every weight would be unpacked twice for nothing)
    if (M <= 64) return 64;
    if (M <= 128 && (N + BN - 1) / BN <= 16 && !(have_workspace && gemm_plan(M, N, nchunks, true, 64).ws_bytes > workspace_bytes)) return 64;
    const int64_t cus = bw_device_cus();
    auto rounds = [&](int64_t tiles) {
        const int64_t full = tiles / cus, rest = tiles % cus;
        const bool split = have_workspace && nchunks >= 8 && rest <= cus / 2;
        return (double)full + (rest == 0 ? 0.0 : split ? 0.75 : 1.0);
    };
    const int64_t tiles_n = (N + BN - 1) / BN;
    const double t128 = rounds(tiles_n * ((M + 127) / 128)), t256 = 1.65 * rounds(tiles_n * ((M + 255) / 256));
    if (t256 > 0.95 * t128) return 128;
    if (have_workspace && gemm_plan(M, N, nchunks, true, 256).ws_bytes > workspace_bytes) return 128;
    return 256;
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

// bfloat16 -> float16 of a row-major matrix, 8 values (16 bytes) per unit; a thread converts the units
// idx, idx + T, idx + 2T, idx + 3T (T = all threads) with every load issued before the first store.
__global__ __launch_bounds__(256) void cast_bf16_f16_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ y,
                                                            int64_t units, int upr, int64_t ldx, int64_t ldy) {
    const int64_t t0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (int64_t)gridDim.x * blockDim.x;
    u4 v[4];
    int64_t dst[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int64_t u = t0 + i * stride;
        dst[i] = -1;
        if (u < units) {
            const int64_t r = u / upr, c = (u - r * upr) * 8;
            v[i] = *reinterpret_cast<const u4*>(x + r * ldx + c);
            dst[i] = r * ldy + c;
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        if (dst[i] < 0) continue;
        u4 o;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float lo = __builtin_bit_cast(float, v[i][j] << 16), hi = __builtin_bit_cast(float, v[i][j] & 0xFFFF0000u);
            o[j] = as_u32(h2{(_Float16)lo, (_Float16)hi});
        }
        *reinterpret_cast<u4*>(y + dst[i]) = o;
    }
}

}  // namespace

extern "C" int bw_cast_bf16_f16(const void* x, int64_t rows, int64_t cols, int64_t ldx, void* y, int64_t ldy, void* stream) {
    if (!x || !y || rows < 1 || cols < 1 || ldx < cols || ldy < cols) return BW_EINVAL;
    if (cols % 8 || ldx % 8 || ldy % 8 || cols / 8 >= ((int64_t)1 << 31)) return BW_EUNSUPPORTED;
    if (!bw_aligned(x, 16) || !bw_aligned(y, 16)) return BW_EALIGN;
    const int64_t units = rows * (cols / 8), blocks = (units + 4 * 256 - 1) / (4 * 256);
    if (blocks >= ((int64_t)1 << 31)) return BW_EUNSUPPORTED;
    hipLaunchKernelGGL(cast_bf16_f16_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const uint16_t*)x,
                       (uint16_t*)y, units, (int)(cols / 8), ldx, ldy);
    return hipGetLastError() == hipSuccess ? BW_OK : BW_ELAUNCH;
}

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

#ifdef BW_TUNE
static unsigned long long* g_tune_clk = nullptr;
extern "C" void bw_tune_clock_buffer(void* p) { g_tune_clk = (unsigned long long*)p; }   // 4096 bytes of device memory, or null
#endif

extern "C" size_t bw_qgemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits, int group) {
    if (!bw_shape_ok(N, K, bits, group) || M < 1 || M >= ((int64_t)1 << 31) || !bw_fast_shape(M, N, K, K, bits, group)) return 0;
    // any of the plans may run (the call's own ldx and workspace decide): enough for each of them
    size_t need = gemm_plan(M, N, gemm_chunks(K, bits, false), true, 128).ws_bytes;
    if (gemm_nat(M, K, K)) {
        const size_t nat128 = gemm_plan(M, N, gemm_chunks(K, bits, true), true, 128).ws_bytes;
        if (nat128 > need) need = nat128;
        const int rows = gemm_tile_rows(M, N, K, K, bits, true, ~(size_t)0);
        if (rows != 128) {
            const size_t other = gemm_plan(M, N, gemm_chunks(K, bits, true), true, rows).ws_bytes;
            if (other > need) need = other;
        }
    }
    return need;
}

extern "C" int bw_qgemm_tile_rows(int64_t M, int64_t N, int64_t K, int bits, int group) {
    if (!bw_shape_ok(N, K, bits, group) || M < 1 || M >= ((int64_t)1 << 31) || !bw_fast_shape(M, N, K, K, bits, group)) return 0;
    return gemm_tile_rows(M, N, K, K, bits, true, ~(size_t)0);
}

extern "C" int bw_qgemm_ws(const void* x, int act_dtype, int64_t M, int64_t K, int64_t ldx, const int32_t* qweight,
                           const void* scale16, const void* zp16, const void* bias, int64_t N, int bits, int group,
                           void* y, int64_t ldy, void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !qweight || !scale16 || !zp16 || !y) return BW_EINVAL;
    if (!bw_shape_ok(N, K, bits, group) || M < 1 || M >= ((int64_t)1 << 31) || ldx < K || ldy < N) return BW_EINVAL;
    if (act_dtype != BW_F16) return BW_EUNSUPPORTED;
    if (!bw_fast_shape(M, N, K, ldx, bits, group) || !bw_aligned(x, 16) || (ldx * 2) % 16 || !bw_aligned(qweight, 16))
        return bw_qgemm_generic(x, act_dtype, M, K, ldx, qweight, scale16, zp16, bias, N, bits, group, y, ldy, stream);
    if (workspace && !bw_aligned(workspace, 16)) return BW_EALIGN;
    GemmArgs a;
    a.x = x; a.qweight = qweight; a.scale = (const _Float16*)scale16; a.zp = (const _Float16*)zp16;
    a.bias = (const _Float16*)bias; a.y = (_Float16*)y;
    a.M = (int)M; a.N = (int)N; a.K = (int)K; a.ldx = (int)ldx; a.ldy = (int)ldy;
    a.groups = (int)(K / group);
    a.row_bytes = (int)(K * bits / 8);
    const bool nat = gemm_nat(M, K, ldx);
    a.nchunks = gemm_chunks(K, bits, nat);
    a.x_bytes = (uint32_t)(((M - 1) * ldx + K) * 2);
    a.w_bytes = (uint32_t)(N * a.row_bytes);
    a.meta_bytes = (uint32_t)(N * a.groups * 2);
    a.ws = nullptr;
    a.tiles_n = a.full_tiles = 0;
    a.tiles_m = a.panel = 1;
    a.xcd_tiles = 0;
#ifdef BW_TUNE
    a.clk = g_tune_clk;
#endif
    a.splits = 1;
    a.chunks_per_split = a.nchunks;
    hipStream_t st = (hipStream_t)stream;
    const int rows = nat ? gemm_tile_rows(M, N, K, ldx, bits, workspace != nullptr, workspace_bytes) : 128;
    if (rows != 128) return bw_launch_gemm_rows(bits, group, rows, a, workspace, workspace_bytes, st);
#define BW_CASE(B, G)                                                                               \
    if (bits == B && group == G)                                                                     \
        return nat ? launch_gemm<B, G, 8, true>(a, workspace, workspace_bytes, st)                   \
                   : launch_gemm<B, G, 8, false>(a, workspace, workspace_bytes, st);
    BW_CASE(4, 128) BW_CASE(4, 64) BW_CASE(4, 32)
    BW_CASE(8, 128) BW_CASE(8, 64) BW_CASE(8, 32)
    BW_CASE(2, 128) BW_CASE(2, 64) BW_CASE(2, 32)
#undef BW_CASE
    return BW_EUNSUPPORTED;
}

// ---- the same without a caller's workspace: the split-K partial tiles go to a device array of the library ----
// For callers that cannot allocate (code under graph capture, serving loops, harnesses that forbid it).  The array
// is one per GPU, shared by every call on that GPU and kept for the life of the process.
constexpr size_t kScratchBytes = (size_t)32 << 20;       // 256 partial tiles of 128 x 256 floats: one full round
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];    // device address of `scratch` on each GPU, looked up once

extern "C" int bw_qgemm_static(const void* x, int act_dtype, int64_t M, int64_t K, int64_t ldx, const int32_t* qweight,
                               const void* scale16, const void* zp16, const void* bias, int64_t N, int bits, int group,
                               void* y, int64_t ldy, void* stream) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return BW_ELAUNCH;
    void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        // `scratch` names the array in host code only as a handle: its memory on the current device is at the
        // address this returns (each GPU holds its own copy at its own address)
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return BW_ELAUNCH;
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    if (bw_qgemm_workspace_bytes(M, N, K, bits, group) > kScratchBytes) return BW_EWORKSPACE;
    return bw_qgemm_ws(x, act_dtype, M, K, ldx, qweight, scale16, zp16, bias, N, bits, group, y, ldy, ptr, kScratchBytes, stream);
}

extern "C" int bw_qgemm(const void* x, int act_dtype, int64_t M, int64_t K, int64_t ldx, const int32_t* qweight,
                        const void* scale16, const void* zp16, const void* bias, int64_t N, int bits, int group,
                        void* y, int64_t ldy, void* stream) {
    return bw_qgemm_ws(x, act_dtype, M, K, ldx, qweight, scale16, zp16, bias, N, bits, group, y, ldy, nullptr, 0, stream);
}

// Rows up to which bw_qlinear stays on the decode kernel (16 rows per launch; the later launches find the weights
// in L2 / Infinity Cache) before it hands the call to the prefill kernel, whose 64-row tiles take 17 ... 64 rows.  Measured
// under graph replay over rotating layer copies (decode launches against one prefill launch, us):
//   4096 x 4096 at 4 bits (8 MiB of packed weights): 8.9 / 10.6 / 15.2 against 13.9 / 14.9 / 16.9 at 17 / 32 / 48 rows, 18.2
//   against 16.8 at 49 - three launches still win;
//   4096 x 4096 at 8 bits (16 MiB), 4096 x 11008 at 2 and 4 bits (11 / 21.5 MiB), 4096 x 14336 at 4 bits (28 MiB): two
//   launches win (12.7 / 15.2 / 16.6 / 19.0 against 15.8 / 18.9 / 19.0 / 19.4 at 32 rows), a third does not (16.0 ... 24.6
//   against 16.0 ... 19.5 at 33);
//   4096 x 11008 at 8 bits (43 MiB): even the second launch loses (22.3 against 19.7 at 17 rows).
extern "C" int bw_qlinear_decode_rows(int64_t N, int64_t K, int bits) {
    if (N < 1 || K < 1 || !bw_bits_ok(bits)) return 0;
    const int64_t bytes = N * (K * bits / 8);
    return bytes < ((int64_t)10 << 20) ? 48 : bytes < ((int64_t)40 << 20) ? 32 : 16;
}

extern "C" int bw_qlinear(const void* x, int act_dtype, int64_t M, int64_t K, int64_t ldx, const int32_t* qweight,
                          const void* scale16, const void* zp16, const void* bias, int64_t N, int bits, int group,
                          void* y, int64_t ldy, void* stream) {
    if (M >= 1 && M <= bw_qlinear_decode_rows(N, K, bits) && (act_dtype == BW_F16 || act_dtype == BW_BF16)) {
        for (int64_t m0 = 0; m0 < M; m0 += 16) {
            const int st = bw_qgemv((const _Float16*)x + m0 * ldx, act_dtype, M - m0 < 16 ? M - m0 : 16, K, ldx, qweight, scale16,
                                    zp16, bias, N, bits, group, (_Float16*)y + m0 * ldy, ldy, stream);
            if (st != BW_OK) return st;
        }
        return BW_OK;
    }
    return bw_qgemm(x, act_dtype, M, K, ldx, qweight, scale16, zp16, bias, N, bits, group, y, ldy, stream);
}
