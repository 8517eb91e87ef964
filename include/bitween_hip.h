/* bitween_hip.h - C ABI of libbitween_hip.so, the MI355X (gfx950) implementation
 * of Bitween's quantized-linear hot path.
 *
 * The reference (Andriykkk/Bitween) is pure Python; its operator boundary for
 * this path is the set of Python callables cited at each entry point below
 * (paths relative to the reference checkout).  The host package bitween_amd
 * keeps those callables' names and signatures and forwards to this ABI.
 *
 * Conventions for every entry point:
 *   - plain C: pointers, sizes, ints.  All data pointers are DEVICE pointers
 *     owned by the caller; nothing is allocated, freed or retained.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).
 *     Work is enqueued on it; no entry point synchronises.
 *   - returns BW_OK (0) or a negative bw_status; never throws.  Arguments are
 *     checked before anything is enqueued: BW_EINVAL, BW_EUNSUPPORTED, BW_EALIGN
 *     and BW_EWORKSPACE mean nothing was launched.  BW_ELAUNCH (the HIP runtime
 *     refused a launch) can come from the second launch of a call that makes
 *     two (bw_qlinear beyond 16 rows, split-K with its reduction): the output
 *     is then undefined.
 *   - weight layout is the reference's: W is [N][K] (N = out_features,
 *     K = in_features); qweight is int32 [N][K*bits/32], value k of a row in
 *     word k / (32/bits) at bit offset (k % (32/bits)) * bits
 *     (bitween/functional.py:31-43); scale and zero_point are [N][K/group].
 *   - bits is 2, 4 or 8; K % group == 0 and K % (32/bits) == 0.
 */
#ifndef BITWEEN_HIP_H
#define BITWEEN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum bw_dtype { BW_F16 = 0, BW_BF16 = 1, BW_F32 = 2, BW_I32 = 3, BW_F64 = 4 } bw_dtype;

/* Flag for the math_dtype argument of bw_quantize_pack / bw_quantize_pack_add (OR it in): form the scale as
 * (max - min) * fl32(1 / Qmax) instead of (max - min) / Qmax.  bitween/functional.py:25 divides a tensor by the
 * Python scalar Qmax: eager torch performs that as a true division on the CPU and, on a GPU, as a
 * multiplication by the float32 reciprocal, which rounds differently in the last bit of most float32 scales
 * (and so moves a few zero points and packed values per layer).  Without the flag: the CPU arithmetic. */
enum { BW_SCALE_RECIPROCAL = 0x100 };

typedef enum bw_status {
    BW_OK = 0,
    BW_EINVAL = -1,       /* bad bits / group / shape / null pointer            */
    BW_EUNSUPPORTED = -2, /* valid for the reference, not built here (see msg)  */
    BW_EALIGN = -3,       /* pointer or pitch not aligned as the kernel needs   */
    BW_ELAUNCH = -4,      /* the HIP runtime refused the launch                 */
    BW_EWORKSPACE = -5    /* workspace missing or too small                     */
} bw_status;

/* Library ABI version (bumped on any signature change). */
int bw_abi_version(void);

/* Static text for a bw_status. */
const char* bw_strerror(int status);

/* quantize_rtn(weight, bits, group_size) -> (q_packed, scale, zero_point)
 * replaces bitween/functional.py:3-45 and, through the output dtypes, the
 * buffer stores of QuantizedLinear.from_float (bitween/modules.py:189-213).
 *   w          [N][ldw] of w_dtype (BW_F16 | BW_BF16 | BW_F32), row pitch ldw elements
 *   math_dtype dtype the arithmetic is rounded to after every operation:
 *              BW_F32 = what from_float does (upcast first, modules.py:191);
 *              BW_F16 / BW_BF16 = eager torch ops on a half tensor;
 *              optionally | BW_SCALE_RECIPROCAL (eager torch on a GPU, see above).
 *   qweight    int32 [N][K*bits/32]
 *   scale      [N][K/group] of scale_dtype (BW_F32 | BW_F16 | BW_BF16); a 16-bit
 *              type applies the module's round-to-nearest-even store
 *   zp         [N][K/group] of zp_dtype (BW_I32 | BW_F16 | BW_BF16)
 * A float64 tensor (functional.py is dtype-agnostic): w_dtype = math_dtype = scale_dtype = BW_F64, zp_dtype BW_I32 -
 * float64 arithmetic throughout, a float64 scale, as the reference returns for such a tensor.
 * Bit-exact against the reference arithmetic for finite inputs. */
int bw_quantize_pack(const void* w, int w_dtype, int math_dtype, int64_t N, int64_t K, int64_t ldw,
                     int bits, int group, int32_t* qweight, void* scale, int scale_dtype,
                     void* zp, int zp_dtype, void* stream);

/* quantize_rtn(orig_weight + value, bits, group_size): the hand-off of a tuned layer,
 * WrapperLinear.to_quantized_linear (bitween/wrapper.py:222-232), without materialising the sum.
 *   delta  [N][ldd] of w_dtype, or NULL (then identical to bw_quantize_pack); the sum w + delta is rounded
 *          once to w_dtype, as the eager tensor add does, before the arithmetic above. */
int bw_quantize_pack_add(const void* w, const void* delta, int w_dtype, int math_dtype, int64_t N, int64_t K,
                         int64_t ldw, int64_t ldd, int bits, int group, int32_t* qweight,
                         void* scale, int scale_dtype, void* zp, int zp_dtype, void* stream);

/* dequantize_rtn(q_packed, scale, zero_point, group_size, bits) -> weight
 * replaces bitween/functional.py:47-71 (out_dtype BW_F32) and the per-forward
 * dequantize kernel bitween/modules.py:10-58 (out_dtype BW_F16: one rounding
 * of the float32 product).  BW_BF16 output is an extension.
 *   scale [N][K/group] of scale_dtype (BW_F32 | BW_F16), zp of zp_dtype
 *   (BW_I32 | BW_F16); w_out [N][ldo] of out_dtype.  A BW_F64 scale goes with a BW_F64 output (the float64
 *   product functional.py:70 promotes to).  Bit-exact. */
int bw_dequantize(const int32_t* qweight, const void* scale, int scale_dtype, const void* zp, int zp_dtype,
                  int64_t N, int64_t K, int bits, int group, void* w_out, int out_dtype, int64_t ldo,
                  void* stream);

/* Fused dequantize + matmul (+ bias):  y[M][N] = x[M][K] @ W16[N][K]^T + bias
 * replaces QuantizedLinearFunction.forward (bitween/modules.py:62-106) and
 * fills the slot of the absent bitween.kernels.cuda_loader.quantized_matmul_cuda
 * (main.py:401,433).  W16 = fp16(scale16 * (q - zp16)) exactly as the
 * reference dequantizes; products accumulate in float32; y is rounded once
 * (the reference rounds before and after the bias add; within its 1e-2
 * tolerance, main.py:471-477).
 *   x      [M][ldx] of act_dtype: BW_F16, or BW_BF16 for bw_qgemv and for bw_qlinear while it stays on the decode kernel - the
 *          kernel then rounds every value to float16 as it reads it, which is the reference's
 *          x.to(float16) (bitween/modules.py:74) without a separate pass; other entry points return
 *          BW_EUNSUPPORTED for BW_BF16.  y [M][ldy] is float16 in every case, as in the reference.
 *   scale16, zp16  float16 [N][K/group] (the module buffers); zp16 must hold
 *                  integers in [0, 2^bits), as every quantizer here produces
 *   bias   [N] float16 or NULL
 * bw_qgemv: decode path, 1 <= M <= 16, HBM-bound, no workspace.
 * bw_qgemm: prefill path, any M >= 1, MFMA-bound.
 * bw_qlinear: picks between them by M (what the Python forward calls): the decode kernel, 16 rows per
 *             launch, up to M = bw_qlinear_decode_rows(N, K, bits) (48; 32 for layers of 10 MiB of packed
 *             weights and more; 16 from 40 MiB on); the prefill kernel (without a workspace) beyond. */
int bw_qgemv(const void* x, int act_dtype, int64_t M, int64_t K, int64_t ldx,
             const int32_t* qweight, const void* scale16, const void* zp16, const void* bias,
             int64_t N, int bits, int group, void* y, int64_t ldy, void* stream);

int bw_qgemm(const void* x, int act_dtype, int64_t M, int64_t K, int64_t ldx,
             const int32_t* qweight, const void* scale16, const void* zp16, const void* bias,
             int64_t N, int bits, int group, void* y, int64_t ldy, void* stream);

/* Prefill with split-K.  When the (M, N) tile grid alone would leave most of the chip idle (small M*N,
 * long K) bw_qgemm_ws cuts K into slices that run in parallel and adds their float32 partial sums in a
 * second kernel; the partial sums live in a caller-provided device workspace of at least
 * bw_qgemm_workspace_bytes(...) bytes (16-byte aligned; 0 = this shape needs none).  With workspace ==
 * NULL it behaves exactly like bw_qgemm.  No counterpart in the reference (its forward is one library
 * GEMM, bitween/modules.py:97). */
size_t bw_qgemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits, int group);

/* Rows of the output tile the prefill kernel runs this shape with (x rows K apart, any workspace it asks for granted):
 * 128, or 256 once a grid of 256-row tiles fills most of the device; 0 = the shape-generic kernel.
 * A diagnostic for benchmarks and tests; no counterpart in the reference. */
int bw_qgemm_tile_rows(int64_t M, int64_t N, int64_t K, int bits, int group);

int bw_qgemm_ws(const void* x, int act_dtype, int64_t M, int64_t K, int64_t ldx,
                const int32_t* qweight, const void* scale16, const void* zp16, const void* bias,
                int64_t N, int bits, int group, void* y, int64_t ldy,
                void* workspace, size_t workspace_bytes, void* stream);

/* bw_qgemm_ws without a workspace argument and without any allocation: the split-K partial tiles go to a device
 * array that the library itself holds (32 MiB per GPU that the library runs on, kept until the process ends),
 * so results are those of bw_qgemm_ws, bit for bit.  No counterpart in the reference; it is for callers that
 * cannot allocate: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * The first call on a device looks up the array's address there (hipGetSymbolAddress); no call allocates,
 * frees or synchronises.  A shape whose 256-row plan needs more than the array runs with 128-row tiles; one whose
 * partial tiles still exceed it returns BW_EWORKSPACE (none does on a 256-CU device).  One call at a time per GPU:
 * every call on a GPU shares that GPU's array, so calls on one stream (ordered) are safe, and calls that overlap in
 * time on one GPU (two streams, two threads) race on it - serialise them or use bw_qgemm_ws with a workspace per
 * stream.  The entry point does not detect an overlap (it would need an event query per call). */
int bw_qgemm_static(const void* x, int act_dtype, int64_t M, int64_t K, int64_t ldx,
                    const int32_t* qweight, const void* scale16, const void* zp16, const void* bias,
                    int64_t N, int bits, int group, void* y, int64_t ldy, void* stream);

int bw_qlinear_decode_rows(int64_t N, int64_t K, int bits);

/* Diagnostic, no counterpart in the reference: the name (with template arguments) of the decode kernel that the
 * calling thread's last bw_qgemv / bw_qlinear launch ran ("" before the first one, or when the generic kernel ran).
 * For benchmarks that label a timing with the kernel it belongs to; the string lives as long as the library. */
const char* bw_qgemv_last_kernel(void);

int bw_qlinear(const void* x, int act_dtype, int64_t M, int64_t K, int64_t ldx,
               const int32_t* qweight, const void* scale16, const void* zp16, const void* bias,
               int64_t N, int bits, int group, void* y, int64_t ldy, void* stream);

/* x.to(float16) of a bfloat16 activation matrix ahead of the prefill kernel
 * replaces the cast in QuantizedLinearFunction.forward (bitween/modules.py:74) for bfloat16 x beyond the rows
 * that bw_qgemv / bw_qlinear convert in-kernel.  Round to nearest even, as the tensor cast.
 *   x [rows][ldx] bfloat16, y [rows][ldy] float16; cols, ldx, ldy multiples of 8 and 16-byte-aligned pointers,
 *   otherwise BW_EUNSUPPORTED / BW_EALIGN (the Python forward then uses the tensor cast). */
int bw_cast_bf16_f16(const void* x, int64_t rows, int64_t cols, int64_t ldx, void* y, int64_t ldy, void* stream);

/* Input gradient, fused with the dequantisation:  grad_x[M][K] = grad_y[M][N] @ W16[N][K]
 * replaces QuantizedLinearFunction.backward (bitween/modules.py:108-141), which unpacks the weights, forms
 * scale * (q - zp), casts it to grad_output's dtype and calls matmul; for float16 gradients that cast gives the
 * same W16 as the forward, for bfloat16 gradients it is the float32 product rounded once to bfloat16 (computed in the
 * kernel from the exact q - zp and the float16 scale).  Products accumulate in float32, grad_x is rounded once.
 *   grad_y [M][ldg], grad_x [M][ldx] of act_dtype (BW_F16 or BW_BF16)
 * Built for K % 128 == 0, N % 32 == 0, group 32 | 64 | 128, ldg % 8 == 0, ldx % 4 == 0; other shapes and dtypes
 * return BW_EUNSUPPORTED (the Python backward then dequantises with bw_dequantize and calls the library GEMM).
 * When M * K is small the reduction over N is cut into slices whose float32 partial sums go through a
 * caller-provided workspace of bw_qdgrad_workspace_bytes(...) bytes (16-byte aligned; 0 = none needed);
 * workspace == NULL runs unsliced.
 * Two kernels: one that owns 128 (256 beyond 512 rows) x 128 tiles of grad_x and walks N in steps of 32 rows, and - for
 * large problems with K % 256 == 0 and N % 64 == 0 - one with 256 x 256 tiles and steps of 64 rows;
 * bw_qdgrad_tile_rows tells which a shape gets (128, 256; 129, 257 = the 256 x 256 kernel with 128 (up to 512 rows of
 * grad_y) or 256 rows of m per tile; 0 = no fused path): a diagnostic,
 * and what the Python backward asks before it prefers this entry point over dequantise + GEMM beyond 512 rows. */
size_t bw_qdgrad_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits, int group);

int bw_qdgrad_tile_rows(int64_t M, int64_t N, int64_t K, int bits, int group);

int bw_qdgrad(const void* grad_y, int act_dtype, int64_t M, int64_t N, int64_t ldg,
              const int32_t* qweight, const void* scale16, const void* zp16,
              int64_t K, int bits, int group, void* grad_x, int64_t ldx,
              void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BITWEEN_HIP_H */
