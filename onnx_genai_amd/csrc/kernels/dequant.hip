// Dequantization of packed 4-bit MatMulNBits weights to f32: w[n,k] = (q - zp) * scale.
// One exact int->f32 subtract and one f32 multiply per element, so the result is bit-identical
// to the reference's definition (onnx-runtime-ep-cpu/src/kernels/matmul_nbits.rs:1360-1363).
#include "common.hiph"

namespace mnb {

// Each thread expands one packed dword (8 consecutive k of one column) into two float4 stores.
__global__ __launch_bounds__(256) void dequant_f32_kernel(
    const uint8_t* __restrict__ b, const void* __restrict__ scales, int scale_dtype,
    const uint8_t* __restrict__ zp, int64_t n, int64_t k, int bs_log2, int64_t kb, float* __restrict__ out)
{
    const int64_t row_dwords = (kb << bs_log2) >> 3;           // packed dwords per column
    const int64_t zp_row = (kb + 1) >> 1;
    const int64_t total = n * row_dwords;
    for (int64_t idx = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; idx < total;
         idx += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int64_t col = idx / row_dwords;
        const int64_t d = idx - col * row_dwords;
        const int64_t k0 = d << 3;
        if (k0 >= k) continue;
        const int64_t blk = k0 >> bs_log2;
        const uint32_t w = reinterpret_cast<const uint32_t*>(b)[idx];
        const float s = load_as_f32(scales, scale_dtype, col * kb + blk);
        const float z = static_cast<float>(zero_point_of(zp ? zp + col * zp_row : nullptr, blk));
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = __fmul_rn(static_cast<float>((w >> (4 * i)) & 0xf) - z, s);
        float* dst = out + col * k + k0;
        if (k0 + 8 <= k && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
            reinterpret_cast<float4*>(dst)[0] = make_float4(v[0], v[1], v[2], v[3]);
            reinterpret_cast<float4*>(dst)[1] = make_float4(v[4], v[5], v[6], v[7]);
        } else {
            for (int i = 0; i < 8 && k0 + i < k; ++i) dst[i] = v[i];
        }
    }
}

}  // namespace mnb

extern "C" int rocm_launch_dequant_f32(const uint8_t* b, const void* scales, int scale_dtype, const uint8_t* zp,
                                       int64_t n, int64_t k, int block_size, float* out_nk, rocm_stream_t stream)
{
    if (n <= 0 || k <= 0) return 0;
    const int bs_log2 = __builtin_ctz(static_cast<unsigned>(block_size));
    const int64_t kb = (k + block_size - 1) / block_size;
    const int64_t total = n * ((kb * block_size) / 8);
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(mnb::dequant_f32_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), b, scales, scale_dtype, zp, n, k, bs_log2, kb, out_nk);
    return static_cast<int>(hipGetLastError());
}
