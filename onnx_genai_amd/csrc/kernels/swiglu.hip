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
