// Epilogue of the fused gate/up projection: y = round16(silu(gate) * up) over two 16-bit [M, N] matrices, the arithmetic
// of the CUDA provider's paired kernel (onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:4207-4233, 4375-4386): both
// projections arrive rounded to the 16-bit type (as the separate nodes would store them), silu is evaluated in f32 with
// the exponential taken in double and rounded to f32, and the product is rounded once. `decomposed` reproduces a graph
// that spelled silu as Sigmoid and Mul: the sigmoid and x * sigmoid are each rounded to the 16-bit type.
#include "common.hiph"

namespace mnb {

__device__ __forceinline__ float silu_f32(float x)
{
    if (x >= 0.0f) return __fdiv_rn(x, __fadd_rn(1.0f, static_cast<float>(exp(static_cast<double>(-x)))));
    const float e = static_cast<float>(exp(static_cast<double>(x)));
    return __fdiv_rn(__fmul_rn(x, e), __fadd_rn(1.0f, e));
}

template <bool BF16>
__device__ __forceinline__ float round16(float v)
{
    return BF16 ? bf16_bits_to_f32(f32_to_bf16_bits(v)) : f16_bits_to_f32(f32_to_f16_bits(v));
}

template <bool BF16>
__device__ __forceinline__ float silu_decomposed_f32(float x)
{
    float sigmoid;
    if (x >= 0.0f) {
        sigmoid = __fdiv_rn(1.0f, __fadd_rn(1.0f, static_cast<float>(exp(static_cast<double>(-x)))));
    } else {
        const float e = static_cast<float>(exp(static_cast<double>(x)));
        sigmoid = __fdiv_rn(e, __fadd_rn(1.0f, e));
    }
    return round16<BF16>(as_f32(__fmul_rn(x, round16<BF16>(as_f32(sigmoid)))));
}

// 16-bit gate and up values (already rounded) -> the 16-bit result.
template <bool BF16>
__device__ __forceinline__ uint16_t swiglu16(uint16_t gate, uint16_t up, bool decomposed)
{
    const float g = BF16 ? bf16_bits_to_f32(gate) : f16_bits_to_f32(gate);
    const float u = BF16 ? bf16_bits_to_f32(up) : f16_bits_to_f32(up);
    const float s = decomposed ? silu_decomposed_f32<BF16>(g) : silu_f32(g);
    const float prod = as_f32(__fmul_rn(s, u));
    return BF16 ? f32_to_bf16_bits(prod) : f32_to_f16_bits(prod);
}

template <bool BF16>
__global__ __launch_bounds__(256) void swiglu_kernel(const uint16_t* __restrict__ gate, const uint16_t* __restrict__ up, int64_t count, int decomposed,
                                                     uint16_t* __restrict__ y)
{
    for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < count; i += static_cast<int64_t>(gridDim.x) * blockDim.x)
        y[i] = swiglu16<BF16>(gate[i], up[i], decomposed != 0);
}

}  // namespace mnb

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
