/*
 * CPU restatement of the reference's int4 MatMulNBits operator. TEST INFRASTRUCTURE ONLY
 * (see matmul_nbits_oracle.h). Plain scalar C, compiled with -ffp-contract=off so that every
 * float operation below is one correctly rounded IEEE operation, as in the reference's scalar code.
 */
#include "matmul_nbits_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ---- dtype.rs:201,228 : f16 / bf16 <-> f32 ------------------------------------------------ */

static uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

float mnb_f16_to_f32(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0x1f) return bits_f32(sign | 0x7f800000u | (man << 13) | (man ? 0x00400000u : 0));
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        int e = -1;
        do { man <<= 1; ++e; } while ((man & 0x400u) == 0);
        return bits_f32(sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13));
    }
    return bits_f32(sign | ((exp + 127 - 15) << 23) | (man << 13));
}

uint16_t mnb_f32_to_f16(float f)
{
    const uint32_t x = f32_bits(f);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t exp = (x >> 23) & 0xffu;
    uint32_t man = x & 0x7fffffu;
    if (exp == 0xff) return (uint16_t)(sign | 0x7c00u | (man ? (0x200u | (man >> 13)) : 0));
    int e = (int)exp - 127 + 15;
    if (e >= 0x1f) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return sign;
        man |= 0x800000u;
        const int shift = 14 - e;
        uint32_t half = man >> shift;
        const uint32_t rem = man & ((1u << shift) - 1);
        const uint32_t mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1))) ++half;
        return (uint16_t)(sign | half);
    }
    uint32_t half = ((uint32_t)e << 10) | (man >> 13);
    const uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1))) ++half;
    return (uint16_t)(sign | half);
}

float mnb_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

uint16_t mnb_f32_to_bf16(float f)
{
    const uint32_t x = f32_bits(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u);
    const uint32_t round = 0x7fffu + ((x >> 16) & 1u);
    return (uint16_t)((x + round) >> 16);
}

void mnb_widen(const void* src, int dtype, size_t count, float* dst)
{
    if (dtype == MNB_F32) { memcpy(dst, src, count * 4); return; }
    const uint16_t* s = (const uint16_t*)src;
    for (size_t i = 0; i < count; ++i) dst[i] = dtype == MNB_F16 ? mnb_f16_to_f32(s[i]) : mnb_bf16_to_f32(s[i]);
}

void mnb_narrow(const float* src, size_t count, int dtype, void* dst)
{
    if (dtype == MNB_F32) { memcpy(dst, src, count * 4); return; }
    uint16_t* d = (uint16_t*)dst;
    for (size_t i = 0; i < count; ++i) d[i] = dtype == MNB_F16 ? mnb_f32_to_f16(src[i]) : mnb_f32_to_bf16(src[i]);
}

/* ---- matmul_nbits.rs:1307-1321 : layout ---------------------------------------------------- */

uint8_t mnb_unpack_nibble(const uint8_t* packed, size_t index)
{
    return (uint8_t)((packed[index / 2] >> (4 * (index % 2))) & 0x0f);
}

uint8_t mnb_zero_point(const uint8_t* zp_row, size_t block)
{
    return zp_row ? mnb_unpack_nibble(zp_row, block) : 8;
}

static size_t div_ceil(size_t a, size_t b) { return (a + b - 1) / b; }

/* ---- matmul_nbits.rs:1360-1363, 3682-3697 : dequantization --------------------------------- */

void mnb_dequantize_nk(const uint8_t* b, const float* scales, const uint8_t* zp,
                       size_t n, size_t k, size_t block_size, float* out_nk)
{
    const size_t kb = div_ceil(k, block_size), blob = block_size / 2, zp_row = div_ceil(kb, 2);
    for (size_t col = 0; col < n; ++col) {
        const uint8_t* row = b + col * kb * blob;
        const uint8_t* zrow = zp ? zp + col * zp_row : NULL;
        for (size_t depth = 0; depth < k; ++depth) {
            const size_t block = depth / block_size;
            const uint8_t q = mnb_unpack_nibble(row + block * blob, depth % block_size);
            const uint8_t z = mnb_zero_point(zrow, block);
            out_nk[col * k + depth] = ((float)q - (float)z) * scales[col * kb + block];
        }
    }
}

/* ---- matmul_nbits.rs:12205-12230, mlas-sys/src/lib.rs:2997-3015 ----------------------------- */

void mnb_matmul_dequant_f32(const float* a, const float* w_nk, const float* bias,
                            size_t m, size_t n, size_t k, float* y)
{
    for (size_t row = 0; row < m; ++row)
        for (size_t col = 0; col < n; ++col) {
            float acc = bias ? bias[col] : 0.0f;
            for (size_t depth = 0; depth < k; ++depth) acc += a[row * k + depth] * w_nk[col * k + depth];
            y[row * n + col] = acc;
        }
}

/* ---- matmul_nbits.rs:10890-10933 ------------------------------------------------------------ */

void mnb_matmul_f64(const float* a, const uint8_t* b, const float* scales, const uint8_t* zp,
                    const float* bias, size_t m, size_t n, size_t k, size_t block_size, double* y)
{
    const size_t kb = div_ceil(k, block_size), blob = block_size / 2, zp_row = div_ceil(kb, 2);
    for (size_t row = 0; row < m; ++row)
        for (size_t col = 0; col < n; ++col) {
            double acc = 0.0;
            for (size_t block = 0; block < kb; ++block) {
                const double scale = (double)scales[col * kb + block];
                const double z = (double)mnb_zero_point(zp ? zp + col * zp_row : NULL, block);
                const uint8_t* blk = b + (col * kb + block) * blob;
                for (size_t off = 0; off < block_size; ++off) {
                    const size_t depth = block * block_size + off;
                    if (depth >= k) break;
                    const double q = (double)mnb_unpack_nibble(blk, off);
                    acc += (q - z) * scale * (double)a[row * k + depth];
                }
            }
            y[row * n + col] = acc + (bias ? (double)bias[col] : 0.0);
        }
}

/* ---- matmul_nbits.rs:7499-7566 (scalar arm) -------------------------------------------------- */

void mnb_matmul_blocksum_f32(const float* a, const uint8_t* b, const float* scales, const uint8_t* zp,
                             const float* bias, size_t m, size_t n, size_t k, size_t block_size, float* y)
{
    const size_t kb = div_ceil(k, block_size), blob = block_size / 2, zp_row = div_ceil(kb, 2);
    float* asum = (float*)malloc(sizeof(float) * (kb ? kb : 1));
    for (size_t row = 0; row < m; ++row) {
        const float* arow = a + row * k;
        for (size_t block = 0; block < kb; ++block) {
            float s = 0.0f;
            for (size_t depth = block * block_size; depth < k && depth < (block + 1) * block_size; ++depth) s += arow[depth];
            asum[block] = s;
        }
        for (size_t col = 0; col < n; ++col) {
            float sum = bias ? bias[col] : 0.0f;
            for (size_t block = 0; block < kb; ++block) {
                const size_t start = block * block_size;
                const size_t valid = k > start ? (k - start < block_size ? k - start : block_size) : 0;
                const uint8_t* blk = b + (col * kb + block) * blob;
                const float z = (float)mnb_zero_point(zp ? zp + col * zp_row : NULL, block);
                float dot = 0.0f;
                for (size_t off = 0; off < valid; ++off) dot += arow[start + off] * (float)mnb_unpack_nibble(blk, off);
                sum += (dot - asum[block] * z) * scales[col * kb + block];
            }
            y[row * n + col] = sum;
        }
    }
    free(asum);
}

/* ---- simd_quant.rs:131-143 / sqnbitgemm_kernel_avx512.cpp:349-426 ---------------------------- */

void mnb_quantize_a(const float* a, size_t m, size_t k, size_t block_size, int rounding,
                    int8_t* qa, float* qscale)
{
    const size_t kb = div_ceil(k, block_size);
    for (size_t row = 0; row < m; ++row)
        for (size_t block = 0; block < kb; ++block) {
            const size_t start = block * block_size;
            const size_t valid = k - start < block_size ? k - start : block_size;
            const float* src = a + row * k + start;
            int8_t* dst = qa + (row * kb + block) * block_size;
            float max_abs = 0.0f;
            for (size_t i = 0; i < valid; ++i) { const float v = fabsf(src[i]); if (v > max_abs) max_abs = v; }
            const float scale = max_abs / 127.0f;
            const float inv = max_abs != 0.0f ? 127.0f / max_abs : 0.0f;
            qscale[row * kb + block] = scale;
            for (size_t i = 0; i < block_size; ++i) {
                if (i >= valid) { dst[i] = 0; continue; }
                const float scaled = src[i] * inv;
                float r = rounding == MNB_ROUND_HALF_AWAY ? roundf(scaled) : nearbyintf(scaled);
                if (r > 127.0f) r = 127.0f;
                if (r < -127.0f) r = -127.0f;
                dst[i] = (int8_t)r;
            }
        }
}

/* ---- matmul_nbits.rs:3360-3412 + 9159-9177 ; qnbitgemm.cpp:727-893 ---------------------------- */

void mnb_block_acc_i32(const int8_t* qa, const uint8_t* b, const uint8_t* zp,
                       size_t m, size_t n, size_t k, size_t block_size, int32_t* acc)
{
    const size_t kb = div_ceil(k, block_size), blob = block_size / 2, zp_row = div_ceil(kb, 2);
    for (size_t row = 0; row < m; ++row)
        for (size_t col = 0; col < n; ++col)
            for (size_t block = 0; block < kb; ++block) {
                const size_t start = block * block_size;
                const size_t valid = k - start < block_size ? k - start : block_size;
                const uint8_t* blk = b + (col * kb + block) * blob;
                const int32_t z = mnb_zero_point(zp ? zp + col * zp_row : NULL, block);
                const int8_t* q = qa + (row * kb + block) * block_size;
                int32_t s = 0;
                for (size_t off = 0; off < valid; ++off) s += (int32_t)q[off] * ((int32_t)mnb_unpack_nibble(blk, off) - z);
                acc[(row * n + col) * kb + block] = s;
            }
}

void mnb_matmul_acc4_f32(const float* a, const uint8_t* b, const float* scales, const uint8_t* zp,
                         const float* bias, size_t m, size_t n, size_t k, size_t block_size,
                         int rounding, float* y)
{
    const size_t kb = div_ceil(k, block_size), blob = block_size / 2, zp_row = div_ceil(kb, 2);
    int8_t* qa = (int8_t*)malloc(m * kb * block_size + 1);
    float* sa = (float*)malloc(sizeof(float) * (m * kb + 1));
    mnb_quantize_a(a, m, k, block_size, rounding, qa, sa);
    for (size_t row = 0; row < m; ++row)
        for (size_t col = 0; col < n; ++col) {
            float value = 0.0f;
            for (size_t block = 0; block < kb; ++block) {
                const size_t start = block * block_size;
                const size_t valid = k - start < block_size ? k - start : block_size;
                const uint8_t* blk = b + (col * kb + block) * blob;
                const int32_t z = mnb_zero_point(zp ? zp + col * zp_row : NULL, block);
                const int8_t* q = qa + (row * kb + block) * block_size;
                int32_t s = 0;
                for (size_t off = 0; off < valid; ++off) s += (int32_t)q[off] * ((int32_t)mnb_unpack_nibble(blk, off) - z);
                value += (float)s * (sa[row * kb + block] * scales[col * kb + block]);
            }
            if (bias) value += bias[col];
            y[row * n + col] = value;
        }
    free(qa);
    free(sa);
}

/* ---- matmul_nbits.rs:1490-1600, 2320-2330 ----------------------------------------------------- */

int mnb_matmul_nbits(const void* a, int a_dtype, const uint8_t* b, const void* scales, int scale_dtype,
                     const uint8_t* zp, const void* bias, int bias_dtype, void* y, int y_dtype,
                     size_t m, size_t n, size_t k, size_t block_size, int accuracy_level, int rounding)
{
    const size_t kb = div_ceil(k, block_size);
    float* af = (float*)malloc(sizeof(float) * (m * k + 1));
    float* sf = (float*)malloc(sizeof(float) * (n * kb + 1));
    float* bf = bias ? (float*)malloc(sizeof(float) * (n + 1)) : NULL;
    float* yf = (float*)malloc(sizeof(float) * (m * n + 1));
    if (!af || !sf || !yf || (bias && !bf)) { free(af); free(sf); free(bf); free(yf); return -1; }
    mnb_widen(a, a_dtype, m * k, af);
    mnb_widen(scales, scale_dtype, n * kb, sf);
    if (bias) mnb_widen(bias, bias_dtype, n, bf);
    if (accuracy_level == 4) mnb_matmul_acc4_f32(af, b, sf, zp, bf, m, n, k, block_size, rounding, yf);
    else mnb_matmul_blocksum_f32(af, b, sf, zp, bf, m, n, k, block_size, yf);
    mnb_narrow(yf, m * n, y_dtype, y);
    free(af); free(sf); free(bf); free(yf);
    return 0;
}


/* ---- gate/up SwiGLU epilogue (onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:4207-4233, 4375-4386) ---- */

float mnb_swiglu_silu(float x)
{
    if (x >= 0.0f) {
        const float denominator = 1.0f + (float)exp((double)-x);
        return x / denominator;
    }
    const float e = (float)exp((double)x);
    const float numerator = x * e;
    return numerator / (1.0f + e);
}

static float round16(float v, int dtype)
{
    return dtype == MNB_F16 ? mnb_f16_to_f32(mnb_f32_to_f16(v)) : mnb_bf16_to_f32(mnb_f32_to_bf16(v));
}

float mnb_swiglu_silu_decomposed(float x, int dtype)
{
    float sigmoid;
    if (x >= 0.0f) {
        sigmoid = 1.0f / (1.0f + (float)exp((double)-x));
    } else {
        const float e = (float)exp((double)x);
        sigmoid = e / (1.0f + e);
    }
    const float sigmoid_h = round16(sigmoid, dtype);
    return round16(x * sigmoid_h, dtype);
}

void mnb_swiglu(const void* gate, const void* up, size_t count, int dtype, int decomposed, void* y)
{
    const uint16_t* g = (const uint16_t*)gate;
    const uint16_t* u = (const uint16_t*)up;
    uint16_t* out = (uint16_t*)y;
    for (size_t i = 0; i < count; ++i) {
        const float gate_h = dtype == MNB_F16 ? mnb_f16_to_f32(g[i]) : mnb_bf16_to_f32(g[i]);
        const float up_h = dtype == MNB_F16 ? mnb_f16_to_f32(u[i]) : mnb_bf16_to_f32(u[i]);
        const float silu_h = decomposed ? mnb_swiglu_silu_decomposed(gate_h, dtype) : mnb_swiglu_silu(gate_h);
        const float prod = silu_h * up_h;
        out[i] = dtype == MNB_F16 ? mnb_f32_to_f16(prod) : mnb_f32_to_bf16(prod);
    }
}


/* ---- RMS-normalization prologue (onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:4125-4205) ---- */

void mnb_rmsnorm16(const void* a, const void* gamma, int gamma_dtype, size_t rows, size_t k, float epsilon, int dtype, void* out)
{
    const uint16_t* in = (const uint16_t*)a;
    uint16_t* dst = (uint16_t*)out;
    const size_t chunks_per_lane = k / (32 * 4);
    for (size_t row = 0; row < rows; ++row) {
        const uint16_t* x = in + row * k;
        float lane_sum[32];
        for (size_t lane = 0; lane < 32; ++lane) {
            float ss[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            for (size_t item = 0; item < chunks_per_lane; ++item) {
                const size_t chunk = lane + item * 32;
                for (int e = 0; e < 4; ++e) {
                    const float v = dtype == MNB_F16 ? mnb_f16_to_f32(x[chunk * 4 + e]) : mnb_bf16_to_f32(x[chunk * 4 + e]);
                    ss[e] = fmaf(v, v, ss[e]);
                }
            }
            lane_sum[lane] = (ss[0] + ss[1]) + (ss[2] + ss[3]);
        }
        for (size_t off = 16; off > 0; off >>= 1) {
            float next[32];
            for (size_t lane = 0; lane < 32; ++lane) next[lane] = lane_sum[lane] + (lane + off < 32 ? lane_sum[lane + off] : lane_sum[lane]);
            memcpy(lane_sum, next, sizeof(next));
        }
        const float inv_std = 1.0f / sqrtf(lane_sum[0] / (float)k + epsilon);
        for (size_t j = 0; j < k; ++j) {
            const float v = dtype == MNB_F16 ? mnb_f16_to_f32(x[j]) : mnb_bf16_to_f32(x[j]);
            float g;
            if (gamma_dtype == MNB_F32) g = ((const float*)gamma)[j];
            else g = gamma_dtype == MNB_F16 ? mnb_f16_to_f32(((const uint16_t*)gamma)[j]) : mnb_bf16_to_f32(((const uint16_t*)gamma)[j]);
            const float y = (v * inv_std) * g;
            dst[row * k + j] = dtype == MNB_F16 ? mnb_f32_to_f16(y) : mnb_f32_to_bf16(y);
        }
    }
}


/* ---- bits 2 / 4 / 8: NBitsLayout, matmul_nbits.rs:1276-1321, 1360-1363 ---------------------------- */

uint8_t mnb_unpack_bits(const uint8_t* packed, size_t index, int bits)
{
    const size_t per_byte = 8 / (size_t)bits;
    const uint8_t mask = bits == 8 ? 0xff : (uint8_t)((1u << bits) - 1);
    return (uint8_t)((packed[index / per_byte] >> ((index % per_byte) * (size_t)bits)) & mask);
}

void mnb_dequantize_nk_bits(const uint8_t* b, const float* scales, const uint8_t* zp, size_t n, size_t k, size_t block_size, int bits,
                            float* out_nk)
{
    const size_t kb = div_ceil(k, block_size), blob = block_size * (size_t)bits / 8, zp_row = div_ceil(kb * (size_t)bits, 8);
    for (size_t col = 0; col < n; ++col) {
        const uint8_t* row = b + col * kb * blob;
        for (size_t depth = 0; depth < k; ++depth) {
            const size_t block = depth / block_size;
            const uint8_t q = mnb_unpack_bits(row + block * blob, depth % block_size, bits);
            const uint8_t z = zp ? mnb_unpack_bits(zp + col * zp_row, block, bits) : (uint8_t)(1u << (bits - 1));
            out_nk[col * k + depth] = ((float)q - (float)z) * scales[col * kb + block];
        }
    }
}

void mnb_matmul_f64_bits(const float* a, const uint8_t* b, const float* scales, const uint8_t* zp, const float* bias,
                         size_t m, size_t n, size_t k, size_t block_size, int bits, double* y)
{
    const size_t kb = div_ceil(k, block_size), blob = block_size * (size_t)bits / 8, zp_row = div_ceil(kb * (size_t)bits, 8);
    for (size_t row = 0; row < m; ++row)
        for (size_t col = 0; col < n; ++col) {
            double acc = 0.0;
            for (size_t block = 0; block < kb; ++block) {
                const double scale = (double)scales[col * kb + block];
                const double z = zp ? (double)mnb_unpack_bits(zp + col * zp_row, block, bits) : (double)(1u << (bits - 1));
                const uint8_t* blk = b + (col * kb + block) * blob;
                for (size_t off = 0; off < block_size; ++off) {
                    const size_t depth = block * block_size + off;
                    if (depth >= k) break;
                    acc += ((double)mnb_unpack_bits(blk, off, bits) - z) * scale * (double)a[row * k + depth];
                }
            }
            y[row * n + col] = acc + (bias ? (double)bias[col] : 0.0);
        }
}


/* ---- g_idx: matmul_nbits.rs:3515-3521, 3636-3658 --------------------------------------------------- */

long mnb_dequantize_nk_gidx(const uint8_t* b, const float* scales, const uint8_t* zp, const int32_t* g_idx, size_t n, size_t k, size_t block_size,
                            int bits, float* out_nk)
{
    const size_t kb = div_ceil(k, block_size), blob = block_size * (size_t)bits / 8, zp_row = div_ceil(kb * (size_t)bits, 8);
    if (g_idx)
        for (size_t depth = 0; depth < k; ++depth)
            if (g_idx[depth] < 0 || (size_t)g_idx[depth] >= kb) return -1 - (long)depth;
    for (size_t col = 0; col < n; ++col) {
        const uint8_t* row = b + col * kb * blob;
        for (size_t depth = 0; depth < k; ++depth) {
            const size_t block = depth / block_size;
            const size_t group = g_idx ? (size_t)g_idx[depth] : block;
            const uint8_t q = mnb_unpack_bits(row + block * blob, depth % block_size, bits);
            const uint8_t z = zp ? mnb_unpack_bits(zp + col * zp_row, group, bits) : (uint8_t)(1u << (bits - 1));
            out_nk[col * k + depth] = ((float)q - (float)z) * scales[col * kb + group];
        }
    }
    return 0;
}
