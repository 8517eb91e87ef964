// Glue kernels of the end-to-end decoder benchmark (bench_decoder.py): what sits between the quantized linears of a
// Llama-shaped layer when ONE token is decoded.  Not part of the quantized-linear library and not in its ABI: the
// benchmark measures that library inside a whole decode step, and with one torch kernel per elementwise operation
// (about seventeen small launches per layer) the step spends three quarters of its time between the linears.
// All float16 in memory with float32 arithmetic:
//
//   glue_add_rmsnorm     x_out = x + delta (rounded to float16); h = x_out * rsqrt(mean(x_out^2) + eps) * gamma
//   glue_rope_kv         rotate q and k of the new token by the angle of its position; q -> q_out, k and v -> the
//                        KV cache row of that position
//   glue_attention       one query row against the cache, in two launches: per slice of the cache the scores, softmax
//                        numerators and weighted sum of v; then the slices of a head -> the attention output
//   glue_rope_attention  the three above in two launches: the attention workgroups rotate q themselves and the one
//                        whose slice holds the new position rotates k and writes k and v into the cache first
//   glue_silu_mul        silu(gate) * up
//
// The position is read from device memory by the kernels, so a captured step can be replayed while the position
// advances.  Every entry point returns 0, or -1 when an argument is outside what the kernels take (nothing is launched
// then).
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// One workgroup of 1024 threads, one row of H = 8 * units values (units <= 1024: a thread keeps its 8 values).
__global__ __launch_bounds__(1024) void add_rmsnorm_kernel(const _Float16* x_in, const _Float16* delta, const _Float16* gamma,
                                                           _Float16* x_out, _Float16* h_out, int H, float eps) {
    __shared__ float red[16];
    const int tid = threadIdx.x, units = H / 8;
    h8 x = {0, 0, 0, 0, 0, 0, 0, 0};
    float ss = 0.f;
    if (tid < units) {
        x = *reinterpret_cast<const h8*>(x_in + tid * 8);
        if (delta) x = x + *reinterpret_cast<const h8*>(delta + tid * 8);       // float16 add, as torch's x + y
        *reinterpret_cast<h8*>(x_out + tid * 8) = x;
#pragma unroll
        for (int e = 0; e < 8; e++) ss += (float)x[e] * (float)x[e];
    }
    ss = wave_sum(ss);
    if ((tid & 63) == 0) red[tid >> 6] = ss;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < 16; w++) tot += red[w];
    const float rinv = rsqrtf(tot / (float)H + eps);
    if (tid < units) {
        const h8 g = *reinterpret_cast<const h8*>(gamma + tid * 8);
        h8 o;
#pragma unroll
        for (int e = 0; e < 8; e++) o[e] = (_Float16)((float)x[e] * rinv * (float)g[e]);
        *reinterpret_cast<h8*>(h_out + tid * 8) = o;
    }
}

// item = which * (H / 2) + j: which 0 = q, 1 = k (pairs (i, i + D / 2) of head j / (D / 2)), 2 = v (values 2 j, 2 j + 1)
__global__ __launch_bounds__(256) void rope_kv_kernel(const _Float16* q, const _Float16* k, const _Float16* v, const _Float16* cos_t,
                                                      const _Float16* sin_t, const int64_t* pos_ptr, _Float16* q_out, _Float16* kcache,
                                                      _Float16* vcache, int heads, int D, int max_len) {
    const int half = D / 2, pairs = heads * half;
    const int item = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    const int64_t pos = *pos_ptr;
    if (item >= 3 * pairs || pos < 0 || pos >= max_len) return;
    const int which = item / pairs, j = item - which * pairs;
    if (which == 2) {
        const int head = (2 * j) / D, i = 2 * j - head * D;
        *reinterpret_cast<h2*>(vcache + ((int64_t)head * max_len + pos) * D + i) = *reinterpret_cast<const h2*>(v + 2 * j);
        return;
    }
    const int head = j / half, i = j - head * half;
    const _Float16* src = which == 0 ? q : k;
    const float x1 = (float)src[head * D + i], x2 = (float)src[head * D + i + half];
    const float c = (float)cos_t[pos * half + i], s = (float)sin_t[pos * half + i];
    const _Float16 o1 = (_Float16)(x1 * c - x2 * s), o2 = (_Float16)(x2 * c + x1 * s);
    _Float16* dst = which == 0 ? q_out + head * D : kcache + ((int64_t)head * max_len + pos) * D;
    dst[i] = o1;
    dst[i + half] = o2;
}

// grid (heads, splits), 256 threads; head dimension 128.  Slice s of the n = pos + 1 cached positions is
// [s * chunk, min(n, (s + 1) * chunk)) with chunk = ceil(n / splits) <= 256 (checked on the host against max_len).
// part[(head * splits + s) * 130]: 128 unnormalised output values, the slice's score maximum, its sum of numerators.
// ROPE: q is the unrotated query and k_new / v_new the new token's key and value; every workgroup rotates its head's
// query itself, and the one whose slice holds position pos rotates the key, writes key and value into the cache
// and reads them back like any other row (a workgroup sees its own writes after a barrier).
constexpr int kD = 128, kMaxChunk = 256;
template <bool ROPE>
__global__ __launch_bounds__(256) void attn_partial_kernel(const _Float16* q, const _Float16* k_new, const _Float16* v_new,
                                                           const _Float16* cos_t, const _Float16* sin_t, _Float16* kcache,
                                                           _Float16* vcache, const int64_t* pos_ptr, float* part, int max_len,
                                                           int splits, float scale) {
    __shared__ float qs[kD];
    __shared__ float sc[kMaxChunk];
    __shared__ float red[8];
    __shared__ float oacc[16][kD];
    const int tid = threadIdx.x, head = blockIdx.x, split = blockIdx.y;
    const int64_t pos = *pos_ptr;
    int64_t n = pos + 1;                                        // the new token's position is part of the cache
    if (n > max_len) n = max_len;
    if (n < 0) n = 0;
    const int chunk = (int)((n + splits - 1) / splits);
    const int p0 = split * chunk, p1 = (int)n < p0 + chunk ? (int)n : p0 + chunk, cnt = p1 > p0 ? p1 - p0 : 0;
    float* out = part + ((int64_t)head * splits + split) * (kD + 2);
    if (cnt == 0 || cnt > kMaxChunk) {                          // an empty slice (uniform over the workgroup)
        if (tid < kD) out[tid] = 0.f;
        if (tid == 0) { out[kD] = -INFINITY; out[kD + 1] = 0.f; }
        return;
    }
    if constexpr (ROPE) {
        constexpr int half = kD / 2;
        const bool owner = pos >= p0 && pos < p1;               // then 0 <= pos < max_len
        const int64_t pc = pos < 0 ? 0 : (pos < max_len ? pos : max_len - 1);
        if (tid < half || (owner && tid < 2 * half)) {
            const int i = tid & (half - 1);
            const _Float16* src = (tid < half ? q : k_new) + head * kD;
            const float x1 = (float)src[i], x2 = (float)src[i + half];
            const float c = (float)cos_t[pc * half + i], sn = (float)sin_t[pc * half + i];
            const _Float16 o1 = (_Float16)(x1 * c - x2 * sn), o2 = (_Float16)(x2 * c + x1 * sn);
            if (tid < half) {
                qs[i] = (float)o1;
                qs[i + half] = (float)o2;
            } else {
                _Float16* dst = kcache + ((int64_t)head * max_len + pos) * kD;
                dst[i] = o1;
                dst[i + half] = o2;
            }
        } else if (owner && tid < 3 * half) {
            const int i = 2 * (tid - 2 * half);
            *reinterpret_cast<h2*>(vcache + ((int64_t)head * max_len + pos) * kD + i) = *reinterpret_cast<const h2*>(v_new + head * kD + i);
        }
        __threadfence_block();
        __syncthreads();
    }
    // v of the first 64 positions of the slice: requested now, used after the softmax (16 lanes per position, 8 values
    // of the head dimension each, 16 positions per pass, four passes in registers)
    const int d8 = tid & 15, ps = tid >> 4;
    const _Float16* vbase = vcache + ((int64_t)head * max_len + p0) * kD + d8 * 8;
    h8 vv[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const int p = 16 * u + ps;
        vv[u] = *reinterpret_cast<const h8*>(vbase + (int64_t)(p < cnt ? p : 0) * kD);
    }
    if constexpr (!ROPE) {
        if (tid < kD) qs[tid] = (float)q[head * kD + tid];
        __syncthreads();
    }
    // scores: 4 lanes per position, 32 values of the head dimension each
    const int part4 = tid & 3;
    for (int pi = tid >> 2; pi < cnt; pi += 64) {
        const _Float16* kr = kcache + ((int64_t)head * max_len + p0 + pi) * kD + part4 * 32;
        float s = 0.f;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const h8 kv = *reinterpret_cast<const h8*>(kr + 8 * u);
#pragma unroll
            for (int e = 0; e < 8; e++) s += (float)kv[e] * qs[part4 * 32 + 8 * u + e];
        }
        s += __shfl_xor(s, 1, 64);
        s += __shfl_xor(s, 2, 64);
        if (part4 == 0) sc[pi] = s * scale;
    }
    __syncthreads();
    // maximum and sum of numerators over the slice (cnt <= 256 = one value per thread)
    const float mine = tid < cnt ? sc[tid] : -INFINITY;
    float m = wave_max(mine);
    if ((tid & 63) == 0) red[tid >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float e = tid < cnt ? __expf(mine - m) : 0.f;
    float l = wave_sum(e);
    if ((tid & 63) == 0) red[4 + (tid >> 6)] = l;
    if (tid < cnt) sc[tid] = e;
    __syncthreads();
    l = red[4] + red[5] + red[6] + red[7];
    // weighted sum of v
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int pb = 0; pb < cnt; pb += 64) {
        float w[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int p = pb + 16 * u + ps;
            w[u] = p < cnt ? sc[p] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int e = 0; e < 8; e++) acc[e] += w[u] * (float)vv[u][e];
        if (pb + 64 < cnt) {                                    // slices of more than 64 positions: the next four passes
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int p = pb + 64 + 16 * u + ps;
                vv[u] = *reinterpret_cast<const h8*>(vbase + (int64_t)(p < cnt ? p : 0) * kD);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 8; e++) oacc[ps][d8 * 8 + e] = acc[e];
    __syncthreads();
    if (tid < kD) {
        float o = 0.f;
#pragma unroll
        for (int g = 0; g < 16; g++) o += oacc[g][tid];
        out[tid] = o;
    }
    if (tid == 0) { out[kD] = m; out[kD + 1] = l; }
}

// grid heads, 128 threads; at most 16 slices (all of a head's slice records are requested before any is used)
constexpr int kMaxSplits = 16;
__global__ __launch_bounds__(128) void attn_combine_kernel(const float* part, _Float16* o, int splits) {
    const int tid = threadIdx.x, head = blockIdx.x;
    const float* p = part + (int64_t)head * splits * (kD + 2);
    float ms[kMaxSplits], ls[kMaxSplits], os[kMaxSplits];
#pragma unroll
    for (int s = 0; s < kMaxSplits; s++) {
        const int sr = s < splits ? s : 0;
        ms[s] = p[sr * (kD + 2) + kD];
        ls[s] = s < splits ? p[sr * (kD + 2) + kD + 1] : 0.f;
        os[s] = p[sr * (kD + 2) + tid];
    }
    float m = -INFINITY;
#pragma unroll
    for (int s = 0; s < kMaxSplits; s++) m = fmaxf(m, ls[s] > 0.f ? ms[s] : -INFINITY);
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int s = 0; s < kMaxSplits; s++) {
        const float w = ls[s] > 0.f ? __expf(ms[s] - m) : 0.f;
        num += w * os[s];
        den += w * ls[s];
    }
    o[head * kD + tid] = (_Float16)(den > 0.f ? num / den : 0.f);
}

// torch's silu(gate) * up on float16 tensors: each of the two operations rounds to float16
__global__ __launch_bounds__(256) void silu_mul_kernel(const _Float16* gate, const _Float16* up, _Float16* out, int n8) {
    const int u = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (u >= n8) return;
    const h8 g = *reinterpret_cast<const h8*>(gate + 8 * u), w = *reinterpret_cast<const h8*>(up + 8 * u);
    h8 o;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const float gf = (float)g[e];
        const _Float16 s = (_Float16)(gf / (1.f + __expf(-gf)));
        o[e] = (_Float16)((float)s * (float)w[e]);
    }
    *reinterpret_cast<h8*>(out + 8 * u) = o;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
inline int launched() { return hipGetLastError() == hipSuccess ? 0 : -2; }

}  // namespace

extern "C" int glue_add_rmsnorm(const void* x_in, const void* delta, const void* gamma, void* x_out, void* h_out, int H, float eps,
                                void* stream) {
    if (!x_in || !gamma || !x_out || !h_out || H < 8 || H % 8 || H > 8192) return -1;
    if (!aligned16(x_in) || !aligned16(gamma) || !aligned16(x_out) || !aligned16(h_out) || (delta && !aligned16(delta))) return -1;
    hipLaunchKernelGGL(add_rmsnorm_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, (const _Float16*)x_in, (const _Float16*)delta,
                       (const _Float16*)gamma, (_Float16*)x_out, (_Float16*)h_out, H, eps);
    return launched();
}

extern "C" int glue_rope_kv(const void* q, const void* k, const void* v, const void* cos_t, const void* sin_t, const void* pos,
                            void* q_out, void* kcache, void* vcache, int heads, int D, int max_len, void* stream) {
    if (!q || !k || !v || !cos_t || !sin_t || !pos || !q_out || !kcache || !vcache || heads < 1 || D < 2 || D % 2 || max_len < 1) return -1;
    if ((reinterpret_cast<uintptr_t>(v) & 3) || (reinterpret_cast<uintptr_t>(vcache) & 3)) return -1;
    const int items = 3 * heads * (D / 2);
    hipLaunchKernelGGL(rope_kv_kernel, dim3((items + 255) / 256), dim3(256), 0, (hipStream_t)stream, (const _Float16*)q, (const _Float16*)k,
                       (const _Float16*)v, (const _Float16*)cos_t, (const _Float16*)sin_t, (const int64_t*)pos, (_Float16*)q_out,
                       (_Float16*)kcache, (_Float16*)vcache, heads, D, max_len);
    return launched();
}

// part: heads * splits * 130 floats
extern "C" int glue_attention(const void* q, const void* kcache, const void* vcache, const void* pos, void* part, void* o, int heads,
                              int D, int max_len, int splits, float scale, void* stream) {
    if (!q || !kcache || !vcache || !pos || !part || !o || heads < 1 || D != kD || max_len < 1 || splits < 1 || splits > kMaxSplits) return -1;
    if ((max_len + splits - 1) / splits > kMaxChunk || !aligned16(kcache) || !aligned16(vcache)) return -1;
    hipLaunchKernelGGL(attn_partial_kernel<false>, dim3(heads, splits), dim3(256), 0, (hipStream_t)stream, (const _Float16*)q,
                       (const _Float16*)nullptr, (const _Float16*)nullptr, (const _Float16*)nullptr, (const _Float16*)nullptr,
                       (_Float16*)const_cast<void*>(kcache), (_Float16*)const_cast<void*>(vcache), (const int64_t*)pos, (float*)part,
                       max_len, splits, scale);
    if (hipGetLastError() != hipSuccess) return -2;
    hipLaunchKernelGGL(attn_combine_kernel, dim3(heads), dim3(kD), 0, (hipStream_t)stream, (const float*)part, (_Float16*)o, splits);
    return launched();
}

// glue_rope_kv and glue_attention in one: q, k, v are the new token's unrotated projections
extern "C" int glue_rope_attention(const void* q, const void* k, const void* v, const void* cos_t, const void* sin_t, const void* pos,
                                   void* kcache, void* vcache, void* part, void* o, int heads, int D, int max_len, int splits,
                                   float scale, void* stream) {
    if (!q || !k || !v || !cos_t || !sin_t || !pos || !kcache || !vcache || !part || !o) return -1;
    if (heads < 1 || D != kD || max_len < 1 || splits < 1 || splits > kMaxSplits || (max_len + splits - 1) / splits > kMaxChunk) return -1;
    if (!aligned16(kcache) || !aligned16(vcache) || (reinterpret_cast<uintptr_t>(v) & 3)) return -1;
    hipLaunchKernelGGL(attn_partial_kernel<true>, dim3(heads, splits), dim3(256), 0, (hipStream_t)stream, (const _Float16*)q,
                       (const _Float16*)k, (const _Float16*)v, (const _Float16*)cos_t, (const _Float16*)sin_t, (_Float16*)kcache,
                       (_Float16*)vcache, (const int64_t*)pos, (float*)part, max_len, splits, scale);
    if (hipGetLastError() != hipSuccess) return -2;
    hipLaunchKernelGGL(attn_combine_kernel, dim3(heads), dim3(kD), 0, (hipStream_t)stream, (const float*)part, (_Float16*)o, splits);
    return launched();
}

extern "C" int glue_silu_mul(const void* gate, const void* up, void* out, int n, void* stream) {
    if (!gate || !up || !out || n < 8 || n % 8 || !aligned16(gate) || !aligned16(up) || !aligned16(out)) return -1;
    hipLaunchKernelGGL(silu_mul_kernel, dim3((n / 8 + 255) / 256), dim3(256), 0, (hipStream_t)stream, (const _Float16*)gate,
                       (const _Float16*)up, (_Float16*)out, n / 8);
    return launched();
}
