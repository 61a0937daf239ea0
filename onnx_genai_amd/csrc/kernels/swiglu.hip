// Epilogue of the fused gate/up projection: y = round16(silu(gate) * up) over two 16-bit [M, N] matrices, the arithmetic
// of the CUDA provider's paired kernel (onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:4207-4233, 4375-4386): both
// projections arrive rounded to the 16-bit type (as the separate nodes would store them), silu is evaluated in f32 with
// the exponential taken in double and rounded to f32, and the product is rounded once. `decomposed` reproduces a graph
// that spelled silu as Sigmoid and Mul: the sigmoid and x * sigmoid are each rounded to the 16-bit type.
#include "swiglu.hiph"

namespace mnb {

template <bool BF16>
__global__ __launch_bounds__(256) void swiglu_kernel(const uint16_t* __restrict__ gate, const uint16_t* __restrict__ up, int64_t count, int decomposed,
                                                     uint16_t* __restrict__ y)
{
    for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < count; i += static_cast<int64_t>(gridDim.x) * blockDim.x)
        y[i] = swiglu16<BF16>(gate[i], up[i], decomposed != 0);
}

// RMS-normalization prologue (onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:4125-4205): out = round16((a * inv_std) *
// gamma) per row, inv_std = 1 / sqrt(mean(a^2) + eps). The sum of squares follows the reference's order exactly - 32
// lanes, each with four running sums over its 4-element chunks, (s0 + s1) + (s2 + s3), then the shuffle tree over 32
// lanes - so half a wavefront plays one 32-lane warp. A workgroup of four waves normalizes two rows: its first wave
// sums the squares of both (sixteen loads in flight at a time), all four then scale four elements per lane and step.
template <bool BF16>
__global__ __launch_bounds__(256) void rmsnorm16_kernel(const uint16_t* __restrict__ a, const void* __restrict__ gamma, int gamma_dtype, int64_t rows,
                                                        int64_t k, float epsilon, uint16_t* __restrict__ out)
{
    __shared__ float inv_shared[2];
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * 2;
    auto widen = [](uint32_t bits16) { return BF16 ? bf16_bits_to_f32(static_cast<uint16_t>(bits16)) : f16_bits_to_f32(static_cast<uint16_t>(bits16)); };
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x & 31;
        const int64_t row = row0 + (threadIdx.x >> 5);
        const bool live = row < rows;
        const uint2* x = reinterpret_cast<const uint2*>(a + (live ? row : row0) * k);
        const int items = static_cast<int>(k / 128);
        float ss0 = 0.f, ss1 = 0.f, ss2 = 0.f, ss3 = 0.f;
        constexpr int kBatch = 16;
        for (int first = 0; first < items; first += kBatch) {
            uint2 raw[kBatch];
#pragma unroll
            for (int i = 0; i < kBatch; ++i) raw[i] = first + i < items ? x[lane + (first + i) * 32] : make_uint2(0u, 0u);      // fma(0, 0, s) = s
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                const float v0 = widen(raw[i].x & 0xffffu), v1 = widen(raw[i].x >> 16), v2 = widen(raw[i].y & 0xffffu), v3 = widen(raw[i].y >> 16);
                ss0 = __fmaf_rn(v0, v0, ss0);
                ss1 = __fmaf_rn(v1, v1, ss1);
                ss2 = __fmaf_rn(v2, v2, ss2);
                ss3 = __fmaf_rn(v3, v3, ss3);
            }
        }
        float ss = __fadd_rn(__fadd_rn(ss0, ss1), __fadd_rn(ss2, ss3));
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) ss = __fadd_rn(ss, __shfl_down(ss, off, 32));
        // sqrtf, not __fsqrt_rn: the latter is the hardware's approximate square root here; sqrtf and the division are
        // correctly rounded (the compiler's default for f32 divide and sqrt)
        const float inv_std = __fdiv_rn(1.0f, sqrtf(__fadd_rn(__fdiv_rn(ss, static_cast<float>(k)), epsilon)));
        if (lane == 0) inv_shared[threadIdx.x >> 5] = inv_std;
    }
    __syncthreads();
    const int chunks = static_cast<int>(k / 4);
    for (int r = 0; r < 2; ++r) {
        const int64_t row = row0 + r;
        if (row >= rows) break;
        const float inv_std = inv_shared[r];
        const uint2* x = reinterpret_cast<const uint2*>(a + row * k);
        uint2* y = reinterpret_cast<uint2*>(out + row * k);
        for (int chunk = threadIdx.x; chunk < chunks; chunk += 256) {
            const uint2 raw = x[chunk];
            float g[4];
            if (gamma_dtype == ROCM_DT_F32) {
                const float4 gv = static_cast<const float4*>(gamma)[chunk];
                g[0] = gv.x, g[1] = gv.y, g[2] = gv.z, g[3] = gv.w;
            } else {
                const uint2 gv = static_cast<const uint2*>(gamma)[chunk];
                const bool gbf = gamma_dtype == ROCM_DT_BF16;
                auto gw = [gbf](uint32_t bits16) { return gbf ? bf16_bits_to_f32(static_cast<uint16_t>(bits16)) : f16_bits_to_f32(static_cast<uint16_t>(bits16)); };
                g[0] = gw(gv.x & 0xffffu), g[1] = gw(gv.x >> 16), g[2] = gw(gv.y & 0xffffu), g[3] = gw(gv.y >> 16);
            }
            const float v[4] = {widen(raw.x & 0xffffu), widen(raw.x >> 16), widen(raw.y & 0xffffu), widen(raw.y >> 16)};
            uint32_t o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float scaled = as_f32(__fmul_rn(__fmul_rn(v[e], inv_std), g[e]));
                o[e] = BF16 ? f32_to_bf16_bits(scaled) : f32_to_f16_bits(scaled);
            }
            y[chunk] = make_uint2(o[0] | (o[1] << 16), o[2] | (o[3] << 16));
        }
    }
}

}  // namespace mnb

extern "C" int rocm_launch_rmsnorm16(const void* a, const void* gamma, int gamma_dtype, int64_t rows, int64_t k, float epsilon, int dtype, void* out,
                                     rocm_stream_t stream)
{
    if (rows <= 0 || k <= 0) return 0;
    if ((dtype != ROCM_DT_F16 && dtype != ROCM_DT_BF16) || k % 128 != 0) return static_cast<int>(hipErrorInvalidValue);
    // rows move four elements at a time: 8-byte pieces of a and out, 16- or 8-byte pieces of gamma
    const uintptr_t gamma_mask = gamma_dtype == ROCM_DT_F32 ? 15 : 7;
    if (((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(out)) & 7) != 0 || (reinterpret_cast<uintptr_t>(gamma) & gamma_mask) != 0)
        return static_cast<int>(hipErrorInvalidValue);
    const unsigned blocks = static_cast<unsigned>((rows + 1) / 2);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == ROCM_DT_BF16)
        hipLaunchKernelGGL(mnb::rmsnorm16_kernel<true>, dim3(blocks), dim3(256), 0, s, static_cast<const uint16_t*>(a), gamma, gamma_dtype, rows, k, epsilon,
                           static_cast<uint16_t*>(out));
    else
        hipLaunchKernelGGL(mnb::rmsnorm16_kernel<false>, dim3(blocks), dim3(256), 0, s, static_cast<const uint16_t*>(a), gamma, gamma_dtype, rows, k, epsilon,
                           static_cast<uint16_t*>(out));
    return static_cast<int>(hipGetLastError());
}

extern "C" int rocm_launch_swiglu(const void* gate, const void* up, int64_t count, int dtype, int decomposed, void* y, rocm_stream_t stream)
{
    if (count <= 0) return 0;
    if (dtype != ROCM_DT_F16 && dtype != ROCM_DT_BF16) return static_cast<int>(hipErrorInvalidValue);
    int64_t blocks = (count + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    const uint16_t* g = static_cast<const uint16_t*>(gate);
    const uint16_t* u = static_cast<const uint16_t*>(up);
    uint16_t* out = static_cast<uint16_t*>(y);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == ROCM_DT_BF16) hipLaunchKernelGGL(mnb::swiglu_kernel<true>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, g, u, count, decomposed, out);
    else hipLaunchKernelGGL(mnb::swiglu_kernel<false>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, g, u, count, decomposed, out);
    return static_cast<int>(hipGetLastError());
}
