// Shared device helpers for the gfx950 kernels of libbitween_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <type_traits>
#include <stdint.h>

#include "../../include/bitween_hip.h"

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned int u4 __attribute__((ext_vector_type(4)));
typedef unsigned int u2 __attribute__((ext_vector_type(2)));

#define BW_DEV __device__ __forceinline__

BW_DEV h2 as_h2(uint32_t u) { return __builtin_bit_cast(h2, u); }
BW_DEV uint32_t as_u32(h2 v) { return __builtin_bit_cast(uint32_t, v); }
BW_DEV h2 splat(_Float16 v) { return h2{v, v}; }

// ---- bfloat16 <-> float32 (round to nearest even; NaN kept quiet) -----------
BW_DEV float bf16_to_f32(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }
BW_DEV uint16_t f32_to_bf16(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

// ---- in-register dequantisation to float16 pairs -----------------------------
// All routines produce W16 = fp16(s * (q - z)) with ONE rounding, which is
// bit-for-bit what the reference's dequantize kernel stores
// (bitween/modules.py:55-58): q - z is formed exactly in float16 from the
// magic-number encoding 0x6400 | q = 1024 + q, then multiplied by s.
// Requires z to be an integer in [0, 2^bits).
//
// Per-group constants a lane keeps while it walks the words of that group.
template <int BITS> struct GroupConst;

template <> struct GroupConst<4> {
    h2 s, z0, z1;   // s, -(1024+z), -(64+z)
    BW_DEV void set(_Float16 sv, _Float16 zv) {
        s = splat(sv);
        z0 = splat((_Float16)(-1024.0f) - zv);
        z1 = splat((_Float16)(-64.0f) - zv);
    }
};
template <> struct GroupConst<8> {
    h2 s, z0;
    BW_DEV void set(_Float16 sv, _Float16 zv) {
        s = splat(sv);
        z0 = splat((_Float16)(-1024.0f) - zv);
    }
};
template <> struct GroupConst<2> {
    h2 s, z0, z1, z2, z3, z4;   // -(1024+z), -(256+z), -(64+z), -(16+z), -(4+z)
    BW_DEV void set(_Float16 sv, _Float16 zv) {
        s = splat(sv);
        z0 = splat((_Float16)(-1024.0f) - zv);
        z1 = splat((_Float16)(-256.0f) - zv);
        z2 = splat((_Float16)(-64.0f) - zv);
        z3 = splat((_Float16)(-16.0f) - zv);
        z4 = splat((_Float16)(-4.0f) - zv);
    }
};

constexpr uint32_t kMagic = 0x64006400u;   // two float16 1024.0

// (a & mask) | orv in one VALU op.  The VOP3 encoding of gfx950 takes no 32-bit literals, so for literal operands the
// compiler emits v_and + v_or; with the mask in an SGPR and the magic in a VGPR the fused v_and_or_b32 is
// encodable.  The two empty statements only hide the constants from folding (they emit nothing, and being
// non-volatile they are hoisted and shared like any other pure computation).  The instruction itself stays one the
// compiler knows: after an inline-assembly and-or it pads every consumer with a wait state, which the MFMA-bound
// loops notice.
BW_DEV uint32_t and_or(uint32_t a, uint32_t mask, uint32_t orv) {
    asm("" : "+s"(mask));
    asm("" : "+v"(orv));
    return (a & mask) | orv;
}

// SCALE = true: out = fp16(s * (q - z)) (the reference's W16).  SCALE = false: out = q - z exactly
// (the caller multiplies the group's partial dot product by s afterwards).

// One 4-bit word (nibbles n0..n7) -> 4 pairs in slot order (n0,n4)(n1,n5)(n2,n6)(n3,n7).
template <bool SCALE>
BW_DEV void dequant_word4(uint32_t w, const GroupConst<4>& c, h2 out[4]) {
    const h2 k16 = splat((_Float16)0.0625f);
    const uint32_t w8 = w >> 8;
    h2 a = as_h2(and_or(w, 0x000F000Fu, kMagic));     // 1024 + n
    h2 b = as_h2(and_or(w, 0x00F000F0u, kMagic));     // 1024 + 16 n
    h2 d = as_h2(and_or(w8, 0x000F000Fu, kMagic));
    h2 e = as_h2(and_or(w8, 0x00F000F0u, kMagic));
    out[0] = a + c.z0;
    out[1] = __builtin_elementwise_fma(b, k16, c.z1);
    out[2] = d + c.z0;
    out[3] = __builtin_elementwise_fma(e, k16, c.z1);
    if constexpr (SCALE) {
#pragma unroll
        for (int i = 0; i < 4; i++) out[i] = out[i] * c.s;
    }
}

// One 8-bit word (bytes b0..b3) -> 2 pairs in natural order (b0,b1)(b2,b3).
template <bool SCALE>
BW_DEV void dequant_word8(uint32_t w, const GroupConst<8>& c, h2 out[2]) {
    h2 a = as_h2(__builtin_amdgcn_perm(0x64646464u, w, 0x04010400u));
    h2 b = as_h2(__builtin_amdgcn_perm(0x64646464u, w, 0x04030402u));
    out[0] = a + c.z0;
    out[1] = b + c.z0;
    if constexpr (SCALE) { out[0] = out[0] * c.s; out[1] = out[1] * c.s; }
}

// One 2-bit word (crumbs c0..c15) -> 8 pairs (c_i, c_{i+8}), i = 0..7.
template <bool SCALE>
BW_DEV void dequant_word2(uint32_t w, const GroupConst<2>& c, h2 out[8]) {
    const uint32_t w10 = w >> 10;
    h2 t0 = as_h2(and_or(w, 0x00030003u, kMagic));     // 1024 + c
    h2 t1 = as_h2(and_or(w, 0x000C000Cu, kMagic));     // 1024 + 4c
    h2 t2 = as_h2(and_or(w, 0x00300030u, kMagic));     // 1024 + 16c
    h2 t3 = as_h2(and_or(w, 0x00C000C0u, kMagic));     // 1024 + 64c
    h2 t4 = as_h2(and_or(w, 0x03000300u, kMagic));     // 1024 + 256c
    h2 t5 = as_h2(and_or(w10, 0x00030003u, kMagic));
    h2 t6 = as_h2(and_or(w10, 0x000C000Cu, kMagic));
    h2 t7 = as_h2(and_or(w10, 0x00300030u, kMagic));
    const h2 k4 = splat((_Float16)0.25f), k16 = splat((_Float16)0.0625f), k64 = splat((_Float16)0.015625f),
             k256 = splat((_Float16)0.00390625f);
    out[0] = t0 + c.z0;
    out[1] = __builtin_elementwise_fma(t1, k4, c.z1);
    out[2] = __builtin_elementwise_fma(t2, k16, c.z2);
    out[3] = __builtin_elementwise_fma(t3, k64, c.z3);
    out[4] = __builtin_elementwise_fma(t4, k256, c.z4);
    out[5] = t5 + c.z0;
    out[6] = __builtin_elementwise_fma(t6, k4, c.z1);
    out[7] = __builtin_elementwise_fma(t7, k16, c.z2);
    if constexpr (SCALE) {
#pragma unroll
        for (int i = 0; i < 8; i++) out[i] = out[i] * c.s;
    }
}

// ---- the same in natural k order ----
// For kernels whose other operand cannot be permuted on its way (activations that go memory -> LDS without passing
// through registers; the transposing LDS read of the input-gradient kernel).  A 4-bit word w = bytes B0..B3, nibbles
// n0..n7: p = [B0 B1 B0 B1] and q = [B2 B3 B2 B3] (one byte permute each) hold n0 in bits 0-3 of their low half and
// n1 in bits 4-7 of their high half, p >> 8 likewise n2 and n3; masked into the mantissa of 1024.0 that is
// (1024 + n0, 1024 + 16 n1), and one packed FMA with (1, 1/16) and (-(1024 + z), -(64 + z)) leaves (n0 - z, n1 - z),
// both exact.  Times the scale: the float16 the reference's dequantize stores (bitween/modules.py:55-58).
// 2 bits: a 16-bit half-word h = bytes b0 b1 holds fields c0..c7; p = [b0 b1 b0 b1] and p >> 8 = [b1 b0 b1 0] carry c0 / c4
// in bits 0-1 and c2 / c6 in bits 4-5 of their low half, c1 / c5 in bits 2-3 and c3 / c7 in bits 6-7 of their high half:
// masks 0x000C0003 and 0x00C00030 give (1024 + c0, 1024 + 4 c1) and (1024 + 16 c2, 1024 + 64 c3); packed FMAs with
// (1, 1/4), (-(1024+z), -(256+z)) and (1/16, 1/64), (-(64+z), -(16+z)) leave the exact differences.
// SCALE as above: false leaves the exact q - z.
template <int BITS> struct GroupConstNat {
    h2 s, zz, zz2;
    BW_DEV void set(_Float16 sv, _Float16 zv) {
        s = splat(sv);
        if constexpr (BITS == 4) zz = h2{(_Float16)(-1024.0f) - zv, (_Float16)(-64.0f) - zv};
        else if constexpr (BITS == 2) {
            zz = h2{(_Float16)(-1024.0f) - zv, (_Float16)(-256.0f) - zv};
            zz2 = h2{(_Float16)(-64.0f) - zv, (_Float16)(-16.0f) - zv};
        } else zz = splat((_Float16)(-1024.0f) - zv);
    }
};

// half-word `half` (0 or 1) of a 2-bit word -> 4 pairs in natural order
template <bool SCALE = true>
BW_DEV void dequant_halfword2_nat(uint32_t w, int half, const GroupConstNat<2>& c, h2 out[4]) {
    const h2 ka = h2{(_Float16)1.0f, (_Float16)0.25f}, kb = h2{(_Float16)0.0625f, (_Float16)0.015625f};
    const uint32_t p = half ? __builtin_amdgcn_perm(w, w, 0x03020302u) : __builtin_amdgcn_perm(w, w, 0x01000100u), q = p >> 8;
    out[0] = __builtin_elementwise_fma(as_h2(and_or(p, 0x000C0003u, kMagic)), ka, c.zz);
    out[1] = __builtin_elementwise_fma(as_h2(and_or(p, 0x00C00030u, kMagic)), kb, c.zz2);
    out[2] = __builtin_elementwise_fma(as_h2(and_or(q, 0x000C0003u, kMagic)), ka, c.zz);
    out[3] = __builtin_elementwise_fma(as_h2(and_or(q, 0x00C00030u, kMagic)), kb, c.zz2);
    if constexpr (SCALE) {
#pragma unroll
        for (int e = 0; e < 4; e++) out[e] = out[e] * c.s;
    }
}

// one 4-bit word -> 4 pairs in natural order
template <bool SCALE = true>
BW_DEV void dequant_word4_nat(uint32_t w, const GroupConstNat<4>& c, h2 out[4]) {
    const h2 kk = h2{(_Float16)1.0f, (_Float16)0.0625f};
    const uint32_t p = __builtin_amdgcn_perm(w, w, 0x01000100u), q = __builtin_amdgcn_perm(w, w, 0x03020302u);
    const uint32_t src[4] = {p, p >> 8, q, q >> 8};
#pragma unroll
    for (int e = 0; e < 4; e++) {
        out[e] = __builtin_elementwise_fma(as_h2(and_or(src[e], 0x00F0000Fu, kMagic)), kk, c.zz);
        if constexpr (SCALE) out[e] = out[e] * c.s;
    }
}

// one 8-bit word -> 2 pairs (natural order as it is)
template <bool SCALE = true>
BW_DEV void dequant_word8_nat(uint32_t w, const GroupConstNat<8>& c, h2 out[2]) {
    out[0] = as_h2(__builtin_amdgcn_perm(0x64646464u, w, 0x04010400u)) + c.zz;
    out[1] = as_h2(__builtin_amdgcn_perm(0x64646464u, w, 0x04030402u)) + c.zz;
    if constexpr (SCALE) { out[0] = out[0] * c.s; out[1] = out[1] * c.s; }
}

// Position p of a block of VPI consecutive k holds original element perm(p):
// the order in which the routines above emit the values of one word.
template <int BITS> BW_DEV constexpr int slot_to_k(int p);
template <> BW_DEV constexpr int slot_to_k<8>(int p) { return p; }
template <> BW_DEV constexpr int slot_to_k<4>(int p) { return (p >> 1) + ((p & 1) << 2); }
template <> BW_DEV constexpr int slot_to_k<2>(int p) { return (p >> 1) + ((p & 1) << 3); }

// Dequantise the 16 bytes a lane loaded (4 words = 128/BITS values) into
// 128/BITS/2 float16 pairs, MFMA-operand ready: pairs [4t, 4t+4) feed MFMA t.
// NG = number of quantisation groups those 16 bytes span (1 or 2).
template <int BITS, int NG, bool SCALE = true>
BW_DEV void dequant_lane16(const u4& w, const GroupConst<BITS>* gc, h2* out) {
    if constexpr (BITS == 4) {
#pragma unroll
        for (int i = 0; i < 4; i++) dequant_word4<SCALE>(w[i], gc[NG == 1 ? 0 : i / (4 / NG)], out + 4 * i);
    } else if constexpr (BITS == 8) {
#pragma unroll
        for (int i = 0; i < 4; i++) dequant_word8<SCALE>(w[i], gc[NG == 1 ? 0 : i / (4 / NG)], out + 2 * i);
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) dequant_word2<SCALE>(w[i], gc[NG == 1 ? 0 : i / (4 / NG)], out + 8 * i);
    }
}

BW_DEV h8 pack_h8(const h2* p) {
    h8 r;
    r[0] = p[0][0]; r[1] = p[0][1]; r[2] = p[1][0]; r[3] = p[1][1];
    r[4] = p[2][0]; r[5] = p[2][1]; r[6] = p[3][0]; r[7] = p[3][1];
    return r;
}

// f(integral_constant<int, 0>{}), ..., f(integral_constant<int, N - 1>{}): a loop whose index is a constant expression
// in the body (immediate operands, if constexpr) and that is unrolled whatever its size.
template <int I, int N, class F>
BW_DEV void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// Workgroup barrier for LDS data that ordinary stores of this wave wrote: waits for the wave's own LDS operations and
// then for the other waves, without the memory fence of __syncthreads() - a fence would also wait for every weight
// request in flight, since those land in LDS too.
BW_DEV void lds_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xC07F);                   // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// wait until at most `n` of this wave's memory loads are outstanding (loads return in order)
template <int N>
BW_DEV void wait_loads() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0F70);   // expcnt and lgkmcnt left alone
}

// Host-side argument checks shared by the entry points.
static inline bool bw_bits_ok(int bits) { return bits == 2 || bits == 4 || bits == 8; }
static inline bool bw_shape_ok(int64_t N, int64_t K, int bits, int group) {
    return N > 0 && K > 0 && group > 0 && bw_bits_ok(bits) && K % group == 0 && K % (32 / bits) == 0 &&
           N < (int64_t)1 << 31 && K < (int64_t)1 << 31;
}
static inline bool bw_aligned(const void* p, size_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

// Compute units of the current device (256 on MI355X); asked once per device.
static inline int bw_device_cus() {
    static int cus[64] = {0};                                 // per device ordinal; a race writes the same value twice
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    int& slot = cus[dev & 63];
    if (slot > 0) return slot;
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    slot = n;
    return n;
}

// A kernel that wants more than 64 KiB of dynamic LDS has to be told so once per device.  `done` is the caller's
// static bit mask of devices already served for that kernel (a race sets the attribute twice, which is harmless).
static inline bool bw_allow_big_lds(const void* kernel, uint64_t& done) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return false;
    const uint64_t bit = 1ull << (dev & 63);
    if (done & bit) return true;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) return false;
    done |= bit;
    return true;
}
