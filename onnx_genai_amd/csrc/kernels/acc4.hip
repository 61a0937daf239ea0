// accuracy_level = 4: activations quantized per K-block to symmetric int8, integer block dot
// products, one f32 scale-and-add per block.
//
//   scale = max|a| / 127, inv = 127 / max|a| (0 for an all-zero block), code = round(a * inv)
//   acc[m,n,b] = sum_{k in b} code[m,k] * (q[n,k] - zp[n,b])                       (int32, exact)
//   y[m,n]     = sum_b f32(acc[m,n,b]) * (scale_a[m,b] * scale_b[n,b]) + bias[n]   (f32)
//
// Two rounding rules exist in the reference's CPU code and both are implemented: ties to even (its
// MLAS kernels) and ties away from zero with a clamp to +-127 (its native Rust kernels).
#include "common.hiph"

namespace mnb {

// One wave per (row, block). Division and multiply are single correctly rounded f32 operations.
__global__ __launch_bounds__(256) void quantize_a_kernel(
    const void* __restrict__ a, int a_dtype, int64_t m, int64_t k, int bs, int64_t kb, int rounding, int interleave,
    int8_t* __restrict__ qa, float* __restrict__ qscale, int32_t* __restrict__ qsum, float* __restrict__ aq, float* __restrict__ aux16, float* __restrict__ sa_t)
{
    const int lane = threadIdx.x & 63;
    const int64_t item = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (item >= m * kb) return;
    const int64_t row = item / kb, blk = item - row * kb;
    const int64_t k0 = blk * bs;
    const int64_t valid = (k - k0 < bs) ? (k - k0) : bs;
    // Block sizes up to 256 keep a lane's (at most four) elements in registers between the two passes.
    constexpr int kHeld = 4;
    float held[kHeld];
    float vmax = 0.0f;
#pragma unroll
    for (int j = 0; j < kHeld; ++j) {
        const int i = lane + 64 * j;
        held[j] = i < valid ? load_as_f32(a, a_dtype, row * k + k0 + i) : 0.0f;
        vmax = fmaxf(vmax, fabsf(held[j]));
    }
    for (int i = lane + 64 * kHeld; i < valid; i += 64) vmax = fmaxf(vmax, fabsf(load_as_f32(a, a_dtype, row * k + k0 + i)));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) vmax = fmaxf(vmax, __shfl_xor(vmax, off, 64));
    const float scale = __fdiv_rn(vmax, 127.0f);
    const float inv = vmax != 0.0f ? __fdiv_rn(127.0f, vmax) : 0.0f;
    int sum = 0;
    auto emit = [&](int i, float value) {
        int code = 0;
        if (i < valid) {
            const float scaled = __fmul_rn(value, inv);
            float r = rounding == 1 ? roundf(scaled) : rintf(scaled);
            r = fminf(fmaxf(r, -127.0f), 127.0f);
            code = static_cast<int>(r);
        }
        // inside every run of 8: as is (0), elements 0,2,4,6,1,3,5,7 (1), or 0,4,1,5,2,6,3,7 (2)
        const int e = i & 7;
        const int pos = (i & ~7) | (interleave == 1 ? (((e & 1) << 2) | (e >> 1)) : interleave == 2 ? (((e & 3) << 1) | (e >> 2)) : e);
        qa[(row * kb + blk) * bs + pos] = static_cast<int8_t>(code);
        sum += code;
    };
#pragma unroll
    for (int j = 0; j < kHeld; ++j) {
        const int i = lane + 64 * j;
        if (i < bs) emit(i, held[j]);
    }
    for (int i = lane + 64 * kHeld; i < bs; i += 64) emit(i, i < valid ? load_as_f32(a, a_dtype, row * k + k0 + i) : 0.0f);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (lane == 0) {
        if (qscale) qscale[row * kb + blk] = scale;
        if (qsum) qsum[row * kb + blk] = sum;
        if (aq) {
            aq[(row * kb + blk) * 2] = scale;
            aq[(row * kb + blk) * 2 + 1] = static_cast<float>(sum);   // |sum| <= 127 * bs: exact
        }
        if (sa_t) sa_t[blk * m + row] = scale;
        if (aux16 && row < 16) {
            aux16[(blk * 16 + row) * 2] = scale;
            aux16[(blk * 16 + row) * 2 + 1] = static_cast<float>(sum);
        }
    }
}

// Parity probe: one thread per (m, n, block), straight integer loop.
__global__ __launch_bounds__(256) void block_acc_i32_kernel(
    const int8_t* __restrict__ qa, const uint8_t* __restrict__ b, const uint8_t* __restrict__ zp,
    int64_t m, int64_t n, int64_t k, int bs, int64_t kb, int32_t* __restrict__ acc)
{
    const int64_t total = m * n * kb;
    for (int64_t idx = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; idx < total; idx += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int64_t blk = idx % kb;
        const int64_t col = (idx / kb) % n;
        const int64_t row = idx / (kb * n);
        const int z = zero_point_of(zp ? zp + col * ((kb + 1) >> 1) : nullptr, blk);
        const uint8_t* wb = b + (col * kb + blk) * (bs / 2);
        const int8_t* q = qa + (row * kb + blk) * bs;
        const int64_t valid = (k - blk * bs < bs) ? (k - blk * bs) : bs;
        int s = 0;
        for (int i = 0; i < valid; ++i) s += static_cast<int>(q[i]) * (static_cast<int>((wb[i >> 1] >> ((i & 1) * 4)) & 0xf) - z);
        acc[idx] = s;
    }
}

// One wave per output column; a lane takes one packed dword (8 weights) at a time, dots it against the
// 8 matching activation codes with v_dot4_i32_i8, and the bs/8 lanes of a block add up with shuffles.
// Codes are in the interleaved order and (scale, code sum) pairs in `aq`, as the workspace holds them.
template <int ROWS>
__global__ __launch_bounds__(256) void acc4_gemv_kernel(RocmMatMulNBitsArgs p, const int8_t* __restrict__ qa, const float* __restrict__ aq,
                                                        int bs_log2, int64_t kb, int64_t row0)
{
    const int lane = threadIdx.x & 63;
    const int64_t col = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (col >= p.n) return;
    const int bs = 1 << bs_log2;
    const int lanes_per_block = bs >> 3;                       // 2 .. 32 lanes share a block
    const int64_t row_dwords = (kb << bs_log2) >> 3;
    const uint32_t* brow = reinterpret_cast<const uint32_t*>(p.b) + col * row_dwords;
    const uint8_t* zrow = p.zp ? p.zp + col * ((kb + 1) >> 1) : nullptr;
    const int rows = static_cast<int>(p.m - row0 < ROWS ? p.m - row0 : ROWS);
    const int64_t padded_k = kb << bs_log2;

    float acc[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) acc[r] = 0.0f;

    const int64_t steps = (row_dwords + 63) / 64;
    for (int64_t it = 0; it < steps; ++it) {
        const int64_t d = it * 64 + lane;
        const bool ok = d < row_dwords;
        const int64_t blk = ok ? ((d << 3) >> bs_log2) : 0;
        const uint32_t w = ok ? brow[d] : 0u;
        const int lo = static_cast<int>(w & 0x0f0f0f0fu);          // elements 0,2,4,6
        const int hi = static_cast<int>((w >> 4) & 0x0f0f0f0fu);   // elements 1,3,5,7
        const int z = zero_point_of(zrow, blk);
        const float sb = ok ? load_as_f32(p.scales, p.scale_dtype, col * kb + blk) : 0.0f;
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            int dot = 0;
            if (ok && r < rows) {
                const uint2 c = *reinterpret_cast<const uint2*>(qa + (row0 + r) * padded_k + (d << 3));   // interleaved: evens, odds
                dot = __builtin_amdgcn_sdot4(static_cast<int>(c.x), lo, 0, false);
                dot = __builtin_amdgcn_sdot4(static_cast<int>(c.y), hi, dot, false);
            }
            for (int off = 1; off < lanes_per_block; off <<= 1) dot += __shfl_xor(dot, off, 64);
            if (ok && r < rows && (lane & (lanes_per_block - 1)) == 0) {
                const float2 pair = *reinterpret_cast<const float2*>(aq + ((row0 + r) * kb + blk) * 2);
                const int block_acc = dot - z * static_cast<int>(pair.y);
                acc[r] += static_cast<float>(block_acc) * __fmul_rn(pair.x, sb);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const float total = wave_sum(acc[r]);
        if (lane == 0 && r < rows) {
            store_from_f32(p.y, p.y_dtype, (row0 + r) * p.n + col, with_bias(total, p.bias, p.bias_dtype, row0 + r, p.n, col, p.y_dtype));
        }
    }
}

// The same quantizer for f16 / bf16 rows with K a multiple of 8 and block size 32, 64 or 128: a lane owns eight consecutive
// elements (one 16-byte load, one 8-byte store of codes - the orders above only permute inside such a run), the BS / 8
// lanes of a block find its maximum and code sum with shuffles. Every arithmetic step is the one above (a maximum and an
// integer sum do not depend on the order), so the codes, scales and sums are the same bits; what changes is the traffic:
// one wave per block of 64 elements moved 2 bytes per lane per load and a byte per store (M = 4096, K = 28672: 622 us,
// 0.57 TB/s).
template <int BS>
__global__ __launch_bounds__(256) void quantize_a16_kernel(
    const uint16_t* __restrict__ a, int bf16, int64_t m, int64_t k, int64_t kb, int rounding, int interleave,
    int8_t* __restrict__ qa, float* __restrict__ qscale, int32_t* __restrict__ qsum, float* __restrict__ aq, float* __restrict__ aux16, float* __restrict__ sa_t)
{
    constexpr int L = BS / 8;                                    // lanes per block
    const int64_t row_pieces = kb * L;                           // 16-byte pieces of a padded row
    const int64_t piece = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const bool inside = piece < m * row_pieces;                  // (lanes past the end still take part in the shuffles)
    const int64_t row = inside ? piece / row_pieces : 0;
    const int64_t in_row = inside ? piece - row * row_pieces : 0;
    const int64_t blk = in_row / L;
    const int64_t k0 = in_row * 8;
    uint4 raw = make_uint4(0u, 0u, 0u, 0u);
    if (inside && k0 < k) raw = *reinterpret_cast<const uint4*>(a + row * k + k0);      // K % 8 = 0: a piece is all inside or all outside
    const uint32_t d[4] = {raw.x, raw.y, raw.z, raw.w};
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = bf16 ? __uint_as_float(d[i] << 16) : f16_bits_to_f32(static_cast<uint16_t>(d[i]));
        v[2 * i + 1] = bf16 ? __uint_as_float(d[i] & 0xffff0000u) : f16_bits_to_f32(static_cast<uint16_t>(d[i] >> 16));
    }
    float vmax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) vmax = fmaxf(vmax, fabsf(v[i]));
#pragma unroll
    for (int off = L / 2; off > 0; off >>= 1) vmax = fmaxf(vmax, __shfl_xor(vmax, off, 64));
    const float scale = __fdiv_rn(vmax, 127.0f);
    const float inv = vmax != 0.0f ? __fdiv_rn(127.0f, vmax) : 0.0f;
    int sum = 0;
    uint32_t lo = 0, hi = 0;                                      // the run's eight code bytes, in storage order
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float scaled = __fmul_rn(v[e], inv);
        float r = rounding == 1 ? roundf(scaled) : rintf(scaled);
        r = fminf(fmaxf(r, -127.0f), 127.0f);
        const int code = static_cast<int>(r);
        sum += code;
        // inside every run of 8: as is (0), elements 0,2,4,6,1,3,5,7 (1), or 0,4,1,5,2,6,3,7 (2)
        const int pos = interleave == 1 ? (((e & 1) << 2) | (e >> 1)) : interleave == 2 ? (((e & 3) << 1) | (e >> 2)) : e;
        const uint32_t byte = static_cast<uint32_t>(code) & 0xffu;
        if (pos < 4) lo |= byte << (8 * pos);
        else hi |= byte << (8 * (pos - 4));
    }
#pragma unroll
    for (int off = L / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (!inside) return;
    *reinterpret_cast<uint2*>(qa + row * kb * BS + k0) = make_uint2(lo, hi);
    if (in_row % L == 0) {
        if (qscale) qscale[row * kb + blk] = scale;
        if (qsum) qsum[row * kb + blk] = sum;
        if (aq) *reinterpret_cast<float2*>(aq + (row * kb + blk) * 2) = make_float2(scale, static_cast<float>(sum));   // |sum| <= 127 * bs: exact
        if (sa_t) sa_t[blk * m + row] = scale;
        if (aux16 && row < 16) *reinterpret_cast<float2*>(aux16 + (blk * 16 + row) * 2) = make_float2(scale, static_cast<float>(sum));
    }
}

}  // namespace mnb

static int launch_quantize(const void* a, int a_dtype, int64_t m, int64_t k, int block_size, int rounding, int interleave,
                           int8_t* qa, float* qscale, int32_t* qsum, float* aq, float* aux16, float* sa_t, rocm_stream_t stream)
{
    if (m <= 0 || k <= 0) return 0;
    const int64_t kb = (k + block_size - 1) / block_size;
    const int64_t items = m * kb;
    const bool half = a_dtype == ROCM_DT_F16 || a_dtype == ROCM_DT_BF16;
    if (half && k % 8 == 0 && (block_size == 32 || block_size == 64 || block_size == 128) && (reinterpret_cast<uintptr_t>(a) & 15) == 0 &&
        (reinterpret_cast<uintptr_t>(qa) & 7) == 0 && (!aq || (reinterpret_cast<uintptr_t>(aq) & 7) == 0) && (!aux16 || (reinterpret_cast<uintptr_t>(aux16) & 7) == 0)) {
        const int64_t pieces = items * (block_size / 8);
        const dim3 grid(static_cast<unsigned>((pieces + 255) / 256));
        const int bf16 = a_dtype == ROCM_DT_BF16;
        const uint16_t* a16 = static_cast<const uint16_t*>(a);
        hipStream_t s = static_cast<hipStream_t>(stream);
        if (block_size == 32) hipLaunchKernelGGL(mnb::quantize_a16_kernel<32>, grid, dim3(256), 0, s, a16, bf16, m, k, kb, rounding, interleave, qa, qscale, qsum, aq, aux16, sa_t);
        else if (block_size == 64) hipLaunchKernelGGL(mnb::quantize_a16_kernel<64>, grid, dim3(256), 0, s, a16, bf16, m, k, kb, rounding, interleave, qa, qscale, qsum, aq, aux16, sa_t);
        else hipLaunchKernelGGL(mnb::quantize_a16_kernel<128>, grid, dim3(256), 0, s, a16, bf16, m, k, kb, rounding, interleave, qa, qscale, qsum, aq, aux16, sa_t);
        return static_cast<int>(hipGetLastError());
    }
    hipLaunchKernelGGL(mnb::quantize_a_kernel, dim3(static_cast<unsigned>((items + 3) / 4)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       a, a_dtype, m, k, block_size, kb, rounding, interleave, qa, qscale, qsum, aq, aux16, sa_t);
    return static_cast<int>(hipGetLastError());
}

extern "C" int rocm_launch_quantize_a(const void* a, int a_dtype, int64_t m, int64_t k, int block_size, int rounding,
                                      int8_t* qa, float* qscale, int32_t* qsum, rocm_stream_t stream)
{
    return launch_quantize(a, a_dtype, m, k, block_size, rounding, 0, qa, qscale, qsum, nullptr, nullptr, nullptr, stream);
}

extern "C" int rocm_launch_quantize_a_workspace(const void* a, int a_dtype, int64_t m, int64_t k, int block_size, int rounding,
                                                const RocmAcc4Workspace* ws, rocm_stream_t stream)
{
    return launch_quantize(a, a_dtype, m, k, block_size, rounding, ws->code_order, ws->qa, nullptr, nullptr, ws->aq, m <= 16 ? ws->aux : nullptr, m > 16 ? ws->aux : nullptr, stream);
}

extern "C" int rocm_launch_block_acc_i32(const int8_t* qa, const uint8_t* b, const uint8_t* zp, int64_t m, int64_t n, int64_t k,
                                         int block_size, int32_t* acc, rocm_stream_t stream)
{
    if (m <= 0 || n <= 0 || k <= 0) return 0;
    const int64_t kb = (k + block_size - 1) / block_size;
    int64_t blocks = (m * n * kb + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(mnb::block_acc_i32_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       qa, b, zp, m, n, k, block_size, kb, acc);
    return static_cast<int>(hipGetLastError());
}

extern "C" int rocm_launch_acc4_gemv(const RocmMatMulNBitsArgs* args, const RocmAcc4Workspace* ws, rocm_stream_t stream)
{
    if (args->m <= 0 || args->n <= 0) return 0;
    const int bs_log2 = __builtin_ctz(static_cast<unsigned>(args->block_size));
    const int64_t kb = (args->k + args->block_size - 1) / args->block_size;
    const dim3 grid(static_cast<unsigned>((args->n + 3) / 4));
    constexpr int kRows = 4;
    for (int64_t row0 = 0; row0 < args->m; row0 += kRows) {
        if (args->m - row0 == 1)
            hipLaunchKernelGGL(mnb::acc4_gemv_kernel<1>, grid, dim3(256), 0, static_cast<hipStream_t>(stream), *args, ws->qa, ws->aq, bs_log2, kb, row0);
        else
            hipLaunchKernelGGL(mnb::acc4_gemv_kernel<kRows>, grid, dim3(256), 0, static_cast<hipStream_t>(stream), *args, ws->qa, ws->aq, bs_log2, kb, row0);
    }
    return static_cast<int>(hipGetLastError());
}
