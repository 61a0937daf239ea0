/*
 * CPU restatement of the reference's int4 MatMulNBits operator. TEST INFRASTRUCTURE ONLY:
 * tests, the smoke check and the benchmark's cpu_baseline leg call it as the checker; the
 * product library never links, loads or falls back to anything in this directory.
 *
 * Every function names the reference lines it follows (paths under /root/reference/crates).
 * What pins each function (golden vectors, the compiled reference MLAS, closed forms, brute
 * force) is listed in tests/test_oracle_pins.py next to the check itself.
 */
#ifndef MATMUL_NBITS_ORACLE_H
#define MATMUL_NBITS_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Rounding rule of the accuracy_level=4 activation quantizer. The reference holds two CPU rules:
 * MNB_ROUND_HALF_AWAY: onnx-runtime-ep-cpu/src/kernels/simd_quant.rs:131-143 (f32::round, clamp +-127)
 * MNB_ROUND_HALF_EVEN: mlas .../sqnbitgemm_kernel_avx512.cpp:384-405 (roundscale NEAREST, cvtps_epi32) */
enum { MNB_ROUND_HALF_EVEN = 0, MNB_ROUND_HALF_AWAY = 1 };

/* element dtypes, same numbers as onnx-runtime-ir/src/dtype.rs:9-37 */
enum { MNB_F32 = 1, MNB_U8 = 2, MNB_I32 = 6, MNB_F16 = 10, MNB_BF16 = 16 };

/* dtype.rs:201,228 (half crate semantics: IEEE round-to-nearest-even, NaN stays NaN) */
float    mnb_f16_to_f32(uint16_t h);
uint16_t mnb_f32_to_f16(float f);
float    mnb_bf16_to_f32(uint16_t h);
uint16_t mnb_f32_to_bf16(float f);
void     mnb_widen(const void* src, int dtype, size_t count, float* dst);
void     mnb_narrow(const float* src, size_t count, int dtype, void* dst);

/* matmul_nbits.rs:1307-1321: nibble `index` of a packed row, low nibble first; zero point of a block
 * (default 8 when zero_points is NULL). */
uint8_t mnb_unpack_nibble(const uint8_t* packed, size_t index);
uint8_t mnb_zero_point(const uint8_t* zp_row, size_t block);

/* matmul_nbits.rs:1360-1363, 3682-3697, 3502-3661: w[n,k] = (q - zp) * scale, one f32 multiply.
 * b: [N, kb, bs/2]; scales: f32 [N, kb]; zp: [N, ceil(kb/2)] or NULL; out: f32 [N, K]. */
void mnb_dequantize_nk(const uint8_t* b, const float* scales, const uint8_t* zp,
                       size_t n, size_t k, size_t block_size, float* out_nk);

/* The same definition at the other bit widths the CPU provider takes (NBitsLayout, matmul_nbits.rs:1276-1321; bits 2, 4, 8):
 * element i of a packed row sits in byte i / (8 / bits), at bit (i % (8 / bits)) * bits; zero points are packed the same
 * way, ceil(kb * bits / 8) bytes per column, default 1 << (bits - 1); a block is block_size * bits / 8 bytes. */
uint8_t mnb_unpack_bits(const uint8_t* packed, size_t index, int bits);
void mnb_dequantize_nk_bits(const uint8_t* b, const float* scales, const uint8_t* zp, size_t n, size_t k, size_t block_size, int bits,
                            float* out_nk);
/* With g_idx (matmul_nbits.rs:3636-3658): scale and zero point of element k come from group g_idx[k] instead of block
 * k / block_size; the packed weights stay where they are. g_idx NULL: the functions above. Returns -1 - index of the first
 * entry outside 0..kb (matmul_nbits.rs:3515-3521 raises there), 0 otherwise. */
long mnb_dequantize_nk_gidx(const uint8_t* b, const float* scales, const uint8_t* zp, const int32_t* g_idx, size_t n, size_t k, size_t block_size,
                            int bits, float* out_nk);
/* int4_f64_reference (matmul_nbits.rs:10890-10933) over that layout: f64 accumulation, bias added in f64. */
void mnb_matmul_f64_bits(const float* a, const uint8_t* b, const float* scales, const uint8_t* zp, const float* bias,
                         size_t m, size_t n, size_t k, size_t block_size, int bits, double* y);

/* matmul_nbits.rs:12205-12230 (test `reference`) and mlas-sys/src/lib.rs:2997-3015 (ref_gemm_nk):
 * y[m,n] = bias[n] + sum_k a[m,k] * w[n,k], f32, k ascending. */
void mnb_matmul_dequant_f32(const float* a, const float* w_nk, const float* bias,
                            size_t m, size_t n, size_t k, float* y);

/* matmul_nbits.rs:10890-10933 (int4_f64_reference): reads the packed layout literally, f64 accumulate.
 * y: f64 [M, N]. bias (f32, may be NULL) is added in f64. */
void mnb_matmul_f64(const float* a, const uint8_t* b, const float* scales, const uint8_t* zp,
                    const float* bias, size_t m, size_t n, size_t k, size_t block_size, double* y);

/* matmul_nbits.rs:7499-7566 (borrowed_int4_output_element):
 * per block dot_u = sum a*q (q unsigned), asum = sum a; y += (dot_u - asum*zp) * scale; bias seeds y. */
void mnb_matmul_blocksum_f32(const float* a, const uint8_t* b, const float* scales, const uint8_t* zp,
                             const float* bias, size_t m, size_t n, size_t k, size_t block_size, float* y);

/* Activation quantizer (accuracy_level=4), one row-block at a time.
 * simd_quant.rs:131-143 / sqnbitgemm_kernel_avx512.cpp:349-426:
 * max = max|a|; scale = max/127; inv = 127/max (0 when max == 0); code = round(a*inv).
 * qa: int8 [M, kb*bs] (tail of a partial last block zero), qscale: f32 [M, kb]. */
void mnb_quantize_a(const float* a, size_t m, size_t k, size_t block_size, int rounding,
                    int8_t* qa, float* qscale);

/* matmul_nbits.rs:3360-3412 + 9159-9177 and qnbitgemm.cpp:727-893, the accumulator both compute:
 * acc[m,n,b] = sum_{k in block b} qa[m,k] * (q[n,k] - zp[n,b]), int32.  acc: [M, N, kb]. */
void mnb_block_acc_i32(const int8_t* qa, const uint8_t* b, const uint8_t* zp,
                       size_t m, size_t n, size_t k, size_t block_size, int32_t* acc);

/* matmul_nbits.rs:9159-9177 (int8_row): y = sum_b (f32)acc_b * (sa_b * sb_b), f32, blocks ascending,
 * starting from 0; bias added afterwards in f32 (matmul_nbits.rs:2320-2326). */
void mnb_matmul_acc4_f32(const float* a, const uint8_t* b, const float* scales, const uint8_t* zp,
                         const float* bias, size_t m, size_t n, size_t k, size_t block_size,
                         int rounding, float* y);

/* The whole operator as Kernel::execute runs it (matmul_nbits.rs:1490-1600, 2320-2330):
 * widen A / scales / bias to f32, compute in f32 (accuracy_level 0: mnb_matmul_blocksum_f32,
 * 4: mnb_matmul_acc4_f32), add bias, narrow Y once. a_dtype/scale_dtype/y_dtype are MNB_* codes. */
int mnb_matmul_nbits(const void* a, int a_dtype, const uint8_t* b, const void* scales, int scale_dtype,
                     const uint8_t* zp, const void* bias, int bias_dtype, void* y, int y_dtype,
                     size_t m, size_t n, size_t k, size_t block_size, int accuracy_level, int rounding);

/* The epilogue of the CUDA provider's fused gate/up node (a "next" neighbour of the operator, not part of the CPU path):
 * onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:4207-4219 (silu, the form of its standalone op_silu):
 *   x >= 0: x / (1 + (float)exp((double)-x));  x < 0: (x * e) / (1 + e) with e = (float)exp((double)x); every step one
 *   correctly rounded f32 operation, the exponential evaluated in double and rounded to f32;
 * :4221-4233 (decomposed silu: Sigmoid and Mul as two 16-bit ops): sigmoid = 1/(1+exp(-x)) resp. e/(1+e) in f32, rounded
 *   to the 16-bit type, times x, rounded to the 16-bit type again;
 * :4375-4386: gate and up arrive rounded to the 16-bit type; y = round16(silu(gate) * up), the product one f32 multiply.
 * `dtype` is MNB_F16 or MNB_BF16 (the reference is fp16 only; bf16 follows the same steps with bf16 roundings).
 * Pinned by the mathematics only (the reference holds no vectors for this node): parity unpinned in the last bit of
 * (float)exp((double)x), which is taken to round alike under every double-precision libm. */
float mnb_swiglu_silu(float x);
float mnb_swiglu_silu_decomposed(float x, int dtype);
void  mnb_swiglu(const void* gate, const void* up, size_t count, int dtype, int decomposed, void* y);

/* The RMS-normalization prologue the CUDA provider folds into a following MatMulNBits
 * (onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:4125-4205, the same arithmetic in-kernel at :3747-3783): per row of K
 * 16-bit elements, 32 lanes each own the 4-element chunks lane, lane + 32, ...; four running sums of squares per lane (one per
 * element of a chunk; a * a + s as one fused multiply-add, the CUDA compiler's default contraction), combined as
 * (s0 + s1) + (s2 + s3), then the shuffle tree off = 16, 8, 4, 2, 1 (lane += lane + off); inv_std = 1 / sqrtf(ss / K + eps),
 * every step correctly rounded; out = round16((a * inv_std) * gamma). K % 128 == 0. gamma: 16-bit of `dtype` or f32.
 * Pinned by the mathematics only (closed forms, a double-precision restatement): the reference holds no vectors, and
 * whether its compiler contracts the sum of squares is an assumption - parity unpinned in that respect. */
void mnb_rmsnorm16(const void* a, const void* gamma, int gamma_dtype, size_t rows, size_t k, float epsilon, int dtype, void* out);

#ifdef __cplusplus
}
#endif
#endif
