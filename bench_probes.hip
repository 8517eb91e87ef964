// Board probes of bench.py (extras.board_probes): the three constants the kernel ceilings are derived from.  Not part
// of the quantized-linear library.
//   probe_launch_floor   device time per launch of an empty kernel when `launches` dependent launches are replayed
//                        from one HIP graph (what separates two kernels of a decode step)
//   probe_read_rate      a kernel that only reads `bytes` of device memory, by grid, block, loads in flight and cache hint: GB/s
//   probe_mfma_issue     v_mfma_f32_16x16x32_f16 back to back, one wave per SIMD, 32 independent accumulator tiles, with
//                        0..3 independent VALU instructions after every MFMA: ns per MFMA and wave (how many issue
//                        slots a single wave has per MFMA)
//   probe_mfma_clock     the shader clock inside that kernel: core-clock ticks over real-time ticks between the first and
//                        the last instruction of every workgroup (the part lowers its clock under load, so "ns per
//                        MFMA" alone does not separate issue limits from clock limits)
// Every entry point returns a negative value on a HIP error.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef unsigned int u4v __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));

__global__ void empty_kernel(int* p) {
    if (p && threadIdx.x == 0x7fffffff) p[0] = 1;
}

// grid-stride read of n 16-byte words with UNROLL loads in flight per lane; NT = the loads carry the non-temporal hint
template <int UNROLL, bool NT>
__global__ __launch_bounds__(1024) void read_kernel(const u4v* __restrict__ s, int* out, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t st = (size_t)gridDim.x * blockDim.x;
    unsigned acc = 0;
    for (; i + (UNROLL - 1) * st < n; i += UNROLL * st) {
        u4v v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) v[u] = NT ? __builtin_nontemporal_load(&s[i + u * st]) : s[i + u * st];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) acc ^= v[u].x ^ v[u].w;
    }
    for (; i < n; i += st) acc ^= s[i].x;
    if (acc == 0x12345u) out[0] = 1;                          // keeps the loads alive; practically never true
}

template <int VPM>
__global__ __launch_bounds__(256) void mfma_kernel(float* out, int iters, float seed, unsigned long long* clk) {
    constexpr int NACC = 32;
    const unsigned long long c0 = clock64(), r0 = wall_clock64();
    f4 acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; i++) acc[i] = f4{0.f, 0.f, 0.f, 0.f};
    h8 a, b;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        a[e] = (_Float16)(seed + threadIdx.x * 1e-3f + e);
        b[e] = (_Float16)(seed * 0.5f + e);
    }
    float v0 = seed, v1 = seed + 1.f, v2 = seed + 2.f;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < NACC; i++) {
            asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i]) : "v"(a), "v"(b));
            if (VPM >= 1) asm volatile("v_fma_f32 %0, %0, %1, %1" : "+v"(v0) : "v"(v1));
            if (VPM >= 2) asm volatile("v_fma_f32 %0, %0, %1, %1" : "+v"(v1) : "v"(v2));
            if (VPM >= 3) asm volatile("v_fma_f32 %0, %0, %1, %1" : "+v"(v2) : "v"(v0));
        }
    }
    float s = v0 + v1 + v2;
#pragma unroll
    for (int i = 0; i < NACC; i++) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    if (s == 12345.678f) out[0] = s;
    if (clk && threadIdx.x == 0) {
        clk[2 * blockIdx.x] = clock64() - c0;
        clk[2 * blockIdx.x + 1] = wall_clock64() - r0;
    }
}

void launch_mfma(int valu_per_mfma, int workgroups, float* out, int n, unsigned long long* clk) {
    if (valu_per_mfma == 0) hipLaunchKernelGGL(mfma_kernel<0>, dim3(workgroups), dim3(256), 0, 0, out, n, 1.0f, clk);
    else if (valu_per_mfma == 1) hipLaunchKernelGGL(mfma_kernel<1>, dim3(workgroups), dim3(256), 0, 0, out, n, 1.0f, clk);
    else if (valu_per_mfma == 2) hipLaunchKernelGGL(mfma_kernel<2>, dim3(workgroups), dim3(256), 0, 0, out, n, 1.0f, clk);
    else hipLaunchKernelGGL(mfma_kernel<3>, dim3(workgroups), dim3(256), 0, 0, out, n, 1.0f, clk);
}

struct Timer {
    hipEvent_t a = nullptr, b = nullptr;
    bool ok = false;
    Timer() { ok = hipEventCreate(&a) == hipSuccess && hipEventCreate(&b) == hipSuccess; }
    ~Timer() {
        if (a) (void)hipEventDestroy(a);
        if (b) (void)hipEventDestroy(b);
    }
};

}  // namespace

extern "C" double probe_launch_floor(int launches, int grid, int block, int replays) {
    if (launches < 1 || grid < 1 || block < 1 || block > 1024 || replays < 1) return -1.0;
    hipStream_t st;
    if (hipStreamCreate(&st) != hipSuccess) return -2.0;
    hipGraph_t g = nullptr;
    hipGraphExec_t ge = nullptr;
    Timer t;
    double us = -2.0;
    if (t.ok && hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal) == hipSuccess) {
        for (int i = 0; i < launches; i++) hipLaunchKernelGGL(empty_kernel, dim3(grid), dim3(block), 0, st, (int*)nullptr);
        if (hipStreamEndCapture(st, &g) == hipSuccess && hipGraphInstantiate(&ge, g, nullptr, nullptr, 0) == hipSuccess) {
            bool ok = true;
            for (int i = 0; i < 3 && ok; i++) ok = hipGraphLaunch(ge, st) == hipSuccess;
            ok = ok && hipStreamSynchronize(st) == hipSuccess && hipEventRecord(t.a, st) == hipSuccess;
            for (int i = 0; i < replays && ok; i++) ok = hipGraphLaunch(ge, st) == hipSuccess;
            ok = ok && hipEventRecord(t.b, st) == hipSuccess && hipStreamSynchronize(st) == hipSuccess;
            float ms = 0.f;
            if (ok && hipEventElapsedTime(&ms, t.a, t.b) == hipSuccess) us = (double)ms * 1e3 / ((double)replays * launches);
        }
    }
    if (ge) (void)hipGraphExecDestroy(ge);
    if (g) (void)hipGraphDestroy(g);
    (void)hipStreamDestroy(st);
    return us;
}

// `src`: `bytes` of device memory (16-byte aligned, a multiple of 16), `scratch`: 4 bytes of device memory.
// `unroll` 4 or 8 loads in flight per lane, `nontemporal` 0 / 1, `grid` workgroups of `block` threads.
extern "C" double probe_read_rate(const void* src, size_t bytes, void* scratch, int grid, int block, int unroll, int nontemporal, int runs) {
    if (!src || !scratch || bytes < 16 || bytes % 16 || grid < 1 || block < 64 || block > 1024 || block % 64 || runs < 1 ||
        (unroll != 4 && unroll != 8) || ((uintptr_t)src & 15))
        return -1.0;
    Timer t;
    if (!t.ok) return -2.0;
    auto launch = [&]() {
        const u4v* p = (const u4v*)src;
        int* o = (int*)scratch;
        const size_t n = bytes / 16;
        if (unroll == 4 && !nontemporal) hipLaunchKernelGGL((read_kernel<4, false>), dim3(grid), dim3(block), 0, 0, p, o, n);
        else if (unroll == 4) hipLaunchKernelGGL((read_kernel<4, true>), dim3(grid), dim3(block), 0, 0, p, o, n);
        else if (!nontemporal) hipLaunchKernelGGL((read_kernel<8, false>), dim3(grid), dim3(block), 0, 0, p, o, n);
        else hipLaunchKernelGGL((read_kernel<8, true>), dim3(grid), dim3(block), 0, 0, p, o, n);
    };
    launch();
    if (hipDeviceSynchronize() != hipSuccess || hipEventRecord(t.a, 0) != hipSuccess) return -2.0;
    for (int i = 0; i < runs; i++) launch();
    float ms = 0.f;
    if (hipEventRecord(t.b, 0) != hipSuccess || hipDeviceSynchronize() != hipSuccess || hipEventElapsedTime(&ms, t.a, t.b) != hipSuccess)
        return -2.0;
    return (double)bytes * runs / ((double)ms * 1e-3) / 1e9;
}

// ns per MFMA and wave with `valu_per_mfma` (0..3) independent VALU instructions after every MFMA; `scratch`: 4 bytes
extern "C" double probe_mfma_issue(int valu_per_mfma, int workgroups, void* scratch) {
    if (valu_per_mfma < 0 || valu_per_mfma > 3 || workgroups < 1 || !scratch) return -1.0;
    const int iters = 2000;
    Timer t;
    if (!t.ok) return -2.0;
    auto launch = [&](int n) {
        float* out = (float*)scratch;
        launch_mfma(valu_per_mfma, workgroups, out, n, nullptr);
    };
    launch(50);
    if (hipDeviceSynchronize() != hipSuccess || hipEventRecord(t.a, 0) != hipSuccess) return -2.0;
    launch(iters);
    float ms = 0.f;
    if (hipEventRecord(t.b, 0) != hipSuccess || hipDeviceSynchronize() != hipSuccess || hipEventElapsedTime(&ms, t.a, t.b) != hipSuccess)
        return -2.0;
    return (double)ms * 1e6 / ((double)iters * 32);
}

// Shader clock in GHz inside the same kernel (mean over the workgroups of the last of `launches` back-to-back
// launches).  `scratch`: 4 + 16 * workgroups bytes of device memory, 8-byte aligned.
extern "C" double probe_mfma_clock(int valu_per_mfma, int workgroups, int launches, void* scratch) {
    if (valu_per_mfma < 0 || valu_per_mfma > 3 || workgroups < 1 || workgroups > 4096 || launches < 1 || !scratch) return -1.0;
    int dev = 0, khz = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess || khz <= 0)
        return -2.0;
    unsigned long long* clk = (unsigned long long*)((char*)scratch + 8);
    for (int i = 0; i < launches; i++) launch_mfma(valu_per_mfma, workgroups, (float*)scratch, 2000, clk);
    static unsigned long long host[2 * 4096];
    if (hipDeviceSynchronize() != hipSuccess || hipMemcpy(host, clk, 16 * (size_t)workgroups, hipMemcpyDeviceToHost) != hipSuccess) return -2.0;
    double sum = 0.0;
    for (int w = 0; w < workgroups; w++) sum += (double)host[2 * w] / (double)host[2 * w + 1];
    return sum / workgroups * khz * 1e-6;
}
