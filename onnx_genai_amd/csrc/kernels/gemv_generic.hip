// MatMulNBits for any dtype mix, any K and any power-of-two block size >= 16: f32 math throughout.
// One wave owns one output column and walks its packed row a dword (8 weights) per lane at a time;
// up to 8 activation rows share each dequantized weight. This is the fp32-activation path and the
// catch-all for shapes the MFMA kernels do not take.
#include "common.hiph"

namespace mnb {

constexpr int kGenericRows = 8;

template <int ROWS>
__global__ __launch_bounds__(256) void gemv_generic_kernel(RocmMatMulNBitsArgs p, int bs_log2, int64_t kb, int64_t row0)
{
    const int lane = threadIdx.x & 63;
    const int64_t col = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (col >= p.n) return;
    const int64_t row_dwords = (kb << bs_log2) >> 3;
    const uint32_t* brow = reinterpret_cast<const uint32_t*>(p.b) + col * row_dwords;
    const uint8_t* zrow = p.zp ? p.zp + col * ((kb + 1) >> 1) : nullptr;
    const int rows = static_cast<int>(p.m - row0 < ROWS ? p.m - row0 : ROWS);

    float acc[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) acc[r] = 0.0f;

    for (int64_t d = lane; d < row_dwords; d += 64) {
        const int64_t k0 = d << 3;
        if (k0 >= p.k) break;
        const int64_t blk = k0 >> bs_log2;
        const uint32_t w = brow[d];
        const float s = load_as_f32(p.scales, p.scale_dtype, col * kb + blk);
        const float z = static_cast<float>(zero_point_of(zrow, blk));
        float wv[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) wv[i] = (k0 + i < p.k) ? __fmul_rn(static_cast<float>((w >> (4 * i)) & 0xf) - z, s) : 0.0f;
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            if (r < rows) {
                const int64_t abase = (row0 + r) * p.k + k0;
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (k0 + i < p.k) acc[r] = fmaf(load_as_f32(p.a, p.a_dtype, abase + i), wv[i], acc[r]);
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

}  // namespace mnb

extern "C" int rocm_launch_gemv_generic(const RocmMatMulNBitsArgs* args, rocm_stream_t stream)
{
    if (args->m <= 0 || args->n <= 0) return 0;
    const int bs_log2 = __builtin_ctz(static_cast<unsigned>(args->block_size));
    const int64_t kb = (args->k + args->block_size - 1) / args->block_size;
    const dim3 grid(static_cast<unsigned>((args->n + 3) / 4));
    for (int64_t row0 = 0; row0 < args->m; row0 += mnb::kGenericRows) {
        if (args->m - row0 == 1)
            hipLaunchKernelGGL(mnb::gemv_generic_kernel<1>, grid, dim3(256), 0, static_cast<hipStream_t>(stream), *args, bs_log2, kb, row0);
        else
            hipLaunchKernelGGL(mnb::gemv_generic_kernel<mnb::kGenericRows>, grid, dim3(256), 0, static_cast<hipStream_t>(stream), *args, bs_log2, kb, row0);
    }
    return static_cast<int>(hipGetLastError());
}
