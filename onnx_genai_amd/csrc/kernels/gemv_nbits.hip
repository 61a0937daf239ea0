// MatMulNBits at the bit widths other than 4 that the CPU provider takes (2 and 8; NBitsLayout,
// onnx-runtime-ep-cpu/src/kernels/matmul_nbits.rs:1276-1321): element i of a packed row sits in byte i / (8 / bits) at
// bit (i % (8 / bits)) * bits, zero points are packed the same way (default 1 << (bits - 1)), w = (q - zp) * scale with one
// f32 multiply. These widths get plain kernels: dequantization (f32 for the parity probe, 16 bits for the tall route's
// dense copy) and f32 GEMVs with one wave per output column - one that loads a dword per lane and takes any shape, and
// for up to four f16 / bf16 rows one per width that moves 16 bytes per load; the tuned kernels are 4-bit.
#include "common.hiph"

namespace mnb {

template <int BITS>
__device__ __forceinline__ uint32_t field(uint32_t word, int i)
{
    return (word >> (i * BITS)) & ((1u << BITS) - 1u);
}

// Zero point of block `blk` of one column; `zrow` null: the default.
template <int BITS>
__device__ __forceinline__ float zero_point_bits(const uint8_t* zrow, int64_t blk)
{
    if (zrow == nullptr) return static_cast<float>(1u << (BITS - 1));
    constexpr int kPerByte = 8 / BITS;
    return static_cast<float>((zrow[blk / kPerByte] >> ((blk % kPerByte) * BITS)) & ((1u << BITS) - 1u));
}

// One thread per packed dword (32 / BITS consecutive k of one column; a dword never straddles a block: block >= 16).
// OUT: 0 = f32, 1 = f16, 2 = bf16.
// `g`: per-element group indices (act-order), or null.
template <int BITS, int OUT>
__global__ __launch_bounds__(256) void dequant_nbits_kernel(const uint8_t* __restrict__ b, const void* __restrict__ scales, int scale_dtype,
                                                            const uint8_t* __restrict__ zp, const int32_t* __restrict__ g, int64_t n, int64_t k, int bs_log2,
                                                            int64_t kb, void* __restrict__ out)
{
    constexpr int W = 32 / BITS;                                         // weights per dword
    const int64_t row_dwords = ((kb << bs_log2) * BITS) >> 5;
    const int64_t zp_row = (kb * BITS + 7) >> 3;
    const int64_t total = n * row_dwords;
    for (int64_t idx = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; idx < total; idx += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int64_t col = idx / row_dwords;
        const int64_t k0 = (idx - col * row_dwords) * W;
        if (k0 >= k) continue;
        const int64_t blk = k0 >> bs_log2;
        const uint32_t w = reinterpret_cast<const uint32_t*>(b)[idx];
        const uint8_t* zrow = zp ? zp + col * zp_row : nullptr;
        float s = load_as_f32(scales, scale_dtype, col * kb + blk);
        float z = zero_point_bits<BITS>(zrow, blk);
#pragma unroll
        for (int i = 0; i < W; ++i) {
            if (k0 + i >= k) break;
            if (g) {
                const int64_t group = g[k0 + i];
                s = load_as_f32(scales, scale_dtype, col * kb + group);
                z = zero_point_bits<BITS>(zrow, group);
            }
            const float v = as_f32(__fmul_rn(static_cast<float>(field<BITS>(w, i)) - z, s));
            const int64_t at = col * k + k0 + i;
            if constexpr (OUT == 0) static_cast<float*>(out)[at] = v;
            else static_cast<uint16_t*>(out)[at] = OUT == 1 ? f32_to_f16_bits(v) : f32_to_bf16_bits(v);
        }
    }
}

constexpr int kNbitsRows = 8;

// One wave per output column, a dword of weights per lane and step, up to eight activation rows per pass. f32 math.
template <int BITS, int ROWS>
__global__ __launch_bounds__(256) void gemv_nbits_kernel(RocmMatMulNBitsArgs p, int bs_log2, int64_t kb, int64_t row0)
{
    constexpr int W = 32 / BITS;
    const int lane = threadIdx.x & 63;
    const int64_t col = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (col >= p.n) return;
    const int64_t row_dwords = ((kb << bs_log2) * BITS) >> 5;
    const uint32_t* brow = reinterpret_cast<const uint32_t*>(p.b) + col * row_dwords;
    const uint8_t* zrow = p.zp ? p.zp + col * ((kb * BITS + 7) >> 3) : nullptr;
    const int rows = static_cast<int>(p.m - row0 < ROWS ? p.m - row0 : ROWS);

    float acc[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) acc[r] = 0.0f;
    for (int64_t d = lane; d < row_dwords; d += 64) {
        const int64_t k0 = d * W;
        if (k0 >= p.k) break;
        const int64_t blk = k0 >> bs_log2;
        const uint32_t w = brow[d];
        float s = load_as_f32(p.scales, p.scale_dtype, col * kb + blk);
        float z = zero_point_bits<BITS>(zrow, blk);
#pragma unroll
        for (int i = 0; i < W; ++i) {
            if (k0 + i < p.k) {
                if (p.g_idx) {
                    const int64_t group = p.g_idx[k0 + i];
                    s = load_as_f32(p.scales, p.scale_dtype, col * kb + group);
                    z = zero_point_bits<BITS>(zrow, group);
                }
                const float wv = __fmul_rn(static_cast<float>(field<BITS>(w, i)) - z, s);
#pragma unroll
                for (int r = 0; r < ROWS; ++r)
                    if (r < rows) acc[r] = fmaf(load_as_f32(p.a, p.a_dtype, (row0 + r) * p.k + k0 + i), wv, acc[r]);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const float total = wave_sum(acc[r]);
        if (lane == 0 && r < rows) store_from_f32(p.y, p.y_dtype, (row0 + r) * p.n + col, with_bias(total, p.bias, p.bias_dtype, row0 + r, p.n, col, p.y_dtype));
    }
}

// 8 bits, f16 / bf16 activations, up to four rows, K % 16 == 0: one wave per output column, 16 weights (one 16-byte load)
// and 16 activations per row (two 16-byte loads, served by the caches: every wave reads the same rows) per lane and step,
// all loads of two steps issued before the arithmetic. f32 math; a 16-weight run never straddles a block (block >= 16).
template <bool BF16, int ROWS>
__global__ __launch_bounds__(256) void gemv_q8_kernel(RocmMatMulNBitsArgs p, int bs_log2, int64_t kb)
{
    const int lane = threadIdx.x & 63;
    const int64_t col = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (col >= p.n) return;
    const int64_t row_bytes = kb << bs_log2;
    const uint4* brow = reinterpret_cast<const uint4*>(p.b + col * row_bytes);
    const uint8_t* zrow = p.zp ? p.zp + col * kb : nullptr;
    const uint16_t* a = static_cast<const uint16_t*>(p.a);
    const int64_t runs = p.k >> 4;                         // 16-weight runs in K
    float acc[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) acc[r] = 0.0f;
    auto widen = [](uint32_t pair, int hi) { const uint16_t h = static_cast<uint16_t>(hi ? pair >> 16 : pair); return BF16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h); };
    for (int64_t run0 = lane; run0 < runs; run0 += 128) {
        uint4 w[2], av[2][ROWS][2];
        bool live[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int64_t run = run0 + 64 * u;
            live[u] = run < runs;
            const int64_t at = live[u] ? run : run0;
            w[u] = brow[at];
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                const uint4* arow = reinterpret_cast<const uint4*>(a + (r < p.m ? r : 0) * p.k) + at * 2;
                av[u][r][0] = arow[0];
                av[u][r][1] = arow[1];
            }
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            if (!live[u]) continue;
            const int64_t blk = ((run0 + 64 * u) << 4) >> bs_log2;
            const float s = load_as_f32(p.scales, p.scale_dtype, col * kb + blk);
            const float z = zrow ? static_cast<float>(zrow[blk]) : 128.0f;
            const uint32_t wd[4] = {w[u].x, w[u].y, w[u].z, w[u].w};
#pragma unroll
            for (int d = 0; d < 4; ++d) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float wv = __fmul_rn(static_cast<float>((wd[d] >> (8 * i)) & 0xffu) - z, s);
                    const int e = d * 4 + i;                                   // element of the run
#pragma unroll
                    for (int r = 0; r < ROWS; ++r) {
                        const uint4& piece = av[u][r][e >> 3];
                        const uint32_t pr[4] = {piece.x, piece.y, piece.z, piece.w};
                        acc[r] = fmaf(widen(pr[(e & 7) >> 1], e & 1), wv, acc[r]);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const float total = wave_sum(acc[r]);
        if (lane == 0 && r < p.m) store_from_f32(p.y, p.y_dtype, r * p.n + col, with_bias(total, p.bias, p.bias_dtype, r, p.n, col, p.y_dtype));
    }
}

// 2 bits, f16 / bf16 activations, up to four rows, K % 64 == 0: one wave per output column, 64 weights (one 16-byte load)
// and 64 activations per row (eight 16-byte loads, served by the caches: every wave reads the same rows) per lane and
// step, every load of the step issued before the arithmetic. f32 math in the plain kernel's order of operations per
// element ((q - zp) * scale rounded, then one FMA); a dword of 16 weights never straddles a block (block >= 16).
template <bool BF16, int ROWS>
__global__ __launch_bounds__(256) void gemv_q2_kernel(RocmMatMulNBitsArgs p, int bs_log2, int64_t kb)
{
    const int lane = threadIdx.x & 63;
    const int64_t col = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (col >= p.n) return;
    const int64_t row_bytes = (kb << bs_log2) >> 2;
    const uint4* brow = reinterpret_cast<const uint4*>(p.b + col * row_bytes);
    const uint8_t* zrow = p.zp ? p.zp + col * ((kb * 2 + 7) >> 3) : nullptr;
    const uint16_t* a = static_cast<const uint16_t*>(p.a);
    const int64_t runs = p.k >> 6;                         // 64-weight runs in K
    float acc[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) acc[r] = 0.0f;
    auto widen = [](uint32_t pair, int hi) { const uint16_t h = static_cast<uint16_t>(hi ? pair >> 16 : pair); return BF16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h); };
    for (int64_t run = lane; run < runs; run += 64) {
        const uint4 w = brow[run];
        uint4 av[ROWS][8];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const uint4* arow = reinterpret_cast<const uint4*>(a + (r < p.m ? r : 0) * p.k) + run * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) av[r][i] = arow[i];
        }
        const uint32_t wd[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const int64_t blk = ((run << 6) + d * 16) >> bs_log2;
            const float s = load_as_f32(p.scales, p.scale_dtype, col * kb + blk);
            const float z = zero_point_bits<2>(zrow, blk);
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float wv = __fmul_rn(static_cast<float>((wd[d] >> (2 * i)) & 3u) - z, s);
                const int e = d * 16 + i;                                  // element of the run
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    const uint4& piece = av[r][e >> 3];
                    const uint32_t pr[4] = {piece.x, piece.y, piece.z, piece.w};
                    acc[r] = fmaf(widen(pr[(e & 7) >> 1], e & 1), wv, acc[r]);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const float total = wave_sum(acc[r]);
        if (lane == 0 && r < p.m) store_from_f32(p.y, p.y_dtype, r * p.n + col, with_bias(total, p.bias, p.bias_dtype, r, p.n, col, p.y_dtype));
    }
}

template <int BITS>
static int launch_dequant(const uint8_t* b, const void* scales, int scale_dtype, const uint8_t* zp, const int32_t* g, int64_t n, int64_t k, int block_size,
                          int out_dtype, void* out, hipStream_t s)
{
    const int bs_log2 = __builtin_ctz(static_cast<unsigned>(block_size));
    const int64_t kb = (k + block_size - 1) / block_size;
    const int64_t total = n * ((kb * block_size * BITS) / 32);
    int64_t blocks = (total + 255) / 256;
    if (blocks > 262144) blocks = 262144;
    const dim3 grid(static_cast<unsigned>(blocks));
    if (out_dtype == ROCM_DT_F32) hipLaunchKernelGGL((dequant_nbits_kernel<BITS, 0>), grid, dim3(256), 0, s, b, scales, scale_dtype, zp, g, n, k, bs_log2, kb, out);
    else if (out_dtype == ROCM_DT_F16) hipLaunchKernelGGL((dequant_nbits_kernel<BITS, 1>), grid, dim3(256), 0, s, b, scales, scale_dtype, zp, g, n, k, bs_log2, kb, out);
    else hipLaunchKernelGGL((dequant_nbits_kernel<BITS, 2>), grid, dim3(256), 0, s, b, scales, scale_dtype, zp, g, n, k, bs_log2, kb, out);
    return static_cast<int>(hipGetLastError());
}

template <int BITS>
static int launch_gemv(const RocmMatMulNBitsArgs* args, hipStream_t s)
{
    const int bs_log2 = __builtin_ctz(static_cast<unsigned>(args->block_size));
    const int64_t kb = (args->k + args->block_size - 1) / args->block_size;
    const dim3 grid(static_cast<unsigned>((args->n + 3) / 4));
    for (int64_t row0 = 0; row0 < args->m; row0 += kNbitsRows) {
        if (args->m - row0 == 1) hipLaunchKernelGGL((gemv_nbits_kernel<BITS, 1>), grid, dim3(256), 0, s, *args, bs_log2, kb, row0);
        else hipLaunchKernelGGL((gemv_nbits_kernel<BITS, kNbitsRows>), grid, dim3(256), 0, s, *args, bs_log2, kb, row0);
    }
    return static_cast<int>(hipGetLastError());
}

// The smallest index whose group lies outside 0..kb, through an atomic minimum (count when every group is in range).
__global__ __launch_bounds__(256) void g_idx_check_kernel(const int32_t* __restrict__ g, int64_t count, int64_t kb, unsigned long long* first_bad)
{
    for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < count; i += static_cast<int64_t>(gridDim.x) * blockDim.x)
        if (g[i] < 0 || g[i] >= kb) atomicMin(first_bad, static_cast<unsigned long long>(i));
}

}  // namespace mnb

extern "C" int rocm_g_idx_first_bad(const int32_t* g_idx, int64_t count, int64_t kb, int64_t* first_bad, rocm_stream_t stream)
{
    *first_bad = -1;
    if (count <= 0) return 0;
    unsigned long long* dev = nullptr;
    hipError_t e = static_cast<hipError_t>(rocm_ffi_malloc(reinterpret_cast<void**>(&dev), sizeof(unsigned long long)));      // (counted with the library's other allocations)
    if (e != hipSuccess) return static_cast<int>(e);
    unsigned long long host = static_cast<unsigned long long>(count);
    hipStream_t s = static_cast<hipStream_t>(stream);
    e = hipMemcpyAsync(dev, &host, sizeof(host), hipMemcpyHostToDevice, s);
    if (e == hipSuccess) {
        int64_t blocks = (count + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(mnb::g_idx_check_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, g_idx, count, kb, dev);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpyAsync(&host, dev, sizeof(host), hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    (void)rocm_ffi_free(dev);
    if (e == hipSuccess && host < static_cast<unsigned long long>(count)) *first_bad = static_cast<int64_t>(host);
    return static_cast<int>(e);
}

extern "C" int rocm_launch_dequant_gidx(const uint8_t* b, const void* scales, int scale_dtype, const uint8_t* zp, const int32_t* g_idx, int64_t n, int64_t k,
                                        int block_size, int bits, int out_dtype, void* out_nk, rocm_stream_t stream)
{
    if (n <= 0 || k <= 0) return 0;
    if (out_dtype != ROCM_DT_F32 && out_dtype != ROCM_DT_F16 && out_dtype != ROCM_DT_BF16) return static_cast<int>(hipErrorInvalidValue);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (bits == 2) return mnb::launch_dequant<2>(b, scales, scale_dtype, zp, g_idx, n, k, block_size, out_dtype, out_nk, s);
    if (bits == 4) return mnb::launch_dequant<4>(b, scales, scale_dtype, zp, g_idx, n, k, block_size, out_dtype, out_nk, s);
    if (bits == 8) return mnb::launch_dequant<8>(b, scales, scale_dtype, zp, g_idx, n, k, block_size, out_dtype, out_nk, s);
    return static_cast<int>(hipErrorInvalidValue);
}

extern "C" int rocm_launch_dequant_nbits(const uint8_t* b, const void* scales, int scale_dtype, const uint8_t* zp, int64_t n, int64_t k, int block_size,
                                         int bits, int out_dtype, void* out_nk, rocm_stream_t stream)
{
    if (n <= 0 || k <= 0) return 0;
    if (out_dtype != ROCM_DT_F32 && out_dtype != ROCM_DT_F16 && out_dtype != ROCM_DT_BF16) return static_cast<int>(hipErrorInvalidValue);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (bits == 2) return mnb::launch_dequant<2>(b, scales, scale_dtype, zp, nullptr, n, k, block_size, out_dtype, out_nk, s);
    if (bits == 8) return mnb::launch_dequant<8>(b, scales, scale_dtype, zp, nullptr, n, k, block_size, out_dtype, out_nk, s);
    return static_cast<int>(hipErrorInvalidValue);
}

extern "C" int rocm_launch_gemv_nbits(const RocmMatMulNBitsArgs* args, int bits, rocm_stream_t stream)
{
    if (args->m <= 0 || args->n <= 0) return 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool half_in = args->a_dtype == ROCM_DT_F16 || args->a_dtype == ROCM_DT_BF16;
    if (bits == 8 && !args->g_idx && half_in && args->m <= 4 && args->k % 16 == 0 && (reinterpret_cast<uintptr_t>(args->a) & 15) == 0 &&
        (reinterpret_cast<uintptr_t>(args->b) & 15) == 0) {
        const int bs_log2 = __builtin_ctz(static_cast<unsigned>(args->block_size));
        const int64_t kb = (args->k + args->block_size - 1) / args->block_size;
        const dim3 grid(static_cast<unsigned>((args->n + 3) / 4));
        const bool bf16 = args->a_dtype == ROCM_DT_BF16;
        if (args->m == 1) {
            if (bf16) hipLaunchKernelGGL((mnb::gemv_q8_kernel<true, 1>), grid, dim3(256), 0, s, *args, bs_log2, kb);
            else hipLaunchKernelGGL((mnb::gemv_q8_kernel<false, 1>), grid, dim3(256), 0, s, *args, bs_log2, kb);
        } else {
            if (bf16) hipLaunchKernelGGL((mnb::gemv_q8_kernel<true, 4>), grid, dim3(256), 0, s, *args, bs_log2, kb);
            else hipLaunchKernelGGL((mnb::gemv_q8_kernel<false, 4>), grid, dim3(256), 0, s, *args, bs_log2, kb);
        }
        return static_cast<int>(hipGetLastError());
    }
    if (bits == 2 && !args->g_idx && half_in && args->m <= 4 && args->k % 64 == 0 && (reinterpret_cast<uintptr_t>(args->a) & 15) == 0 &&
        (reinterpret_cast<uintptr_t>(args->b) & 15) == 0) {
        const int bs_log2 = __builtin_ctz(static_cast<unsigned>(args->block_size));
        const int64_t kb = (args->k + args->block_size - 1) / args->block_size;
        if ((((kb << bs_log2) >> 2) & 15) == 0) {              // every column's row of weights starts on 16 bytes
            const dim3 grid(static_cast<unsigned>((args->n + 3) / 4));
            const bool bf16 = args->a_dtype == ROCM_DT_BF16;
            if (args->m == 1) {
                if (bf16) hipLaunchKernelGGL((mnb::gemv_q2_kernel<true, 1>), grid, dim3(256), 0, s, *args, bs_log2, kb);
                else hipLaunchKernelGGL((mnb::gemv_q2_kernel<false, 1>), grid, dim3(256), 0, s, *args, bs_log2, kb);
            } else {
                if (bf16) hipLaunchKernelGGL((mnb::gemv_q2_kernel<true, 4>), grid, dim3(256), 0, s, *args, bs_log2, kb);
                else hipLaunchKernelGGL((mnb::gemv_q2_kernel<false, 4>), grid, dim3(256), 0, s, *args, bs_log2, kb);
            }
            return static_cast<int>(hipGetLastError());
        }
    }
    if (bits == 2) return mnb::launch_gemv<2>(args, s);
    if (bits == 4) return mnb::launch_gemv<4>(args, s);            // 4 bits come here with g_idx only
    if (bits == 8) return mnb::launch_gemv<8>(args, s);
    return static_cast<int>(hipErrorInvalidValue);
}
