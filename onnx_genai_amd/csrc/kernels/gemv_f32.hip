// Decode path of MatMulNBits for f32 activations (M <= 4, block size >= 32): f32 FMA on the vector ALUs,
// nothing rounded below f32 - the arithmetic of the reference's fp32 route (matmul_nbits.rs:7499-7566):
// per run of 32 weights of one block  dot_u = sum a*q  with q the unsigned nibble,  asum = sum a,
// y += (dot_u - zp*asum) * scale.
//
// A workgroup of eight waves owns 32 output columns: every 16-lane group of a wave streams one column
// over the whole of K in 16-byte pieces (32 weights per lane per step, 512 k per step, requested one window
// ahead), so there is no split-K and no reduction across waves. The activation rows of the current K window sit in LDS together
// with their sums over runs of 32 elements; a lane reads its 32 activations as eight 16-byte LDS loads
// which the four lane groups of a wave share (one broadcast read each); the window is stored chunk-major so
// that those loads are free of bank conflicts.
#include "mfma_common.hiph"

namespace mnb {

struct GemvF32Params {
    const float* a;
    const uint8_t* b;
    const void* scales;
    const uint8_t* zp;
    const void* bias;
    void* y;
    int64_t m, n, k, kb;
    int64_t row_bytes, zp_row;
    int bs_log2;
    int scale_dtype, bias_dtype, y_dtype;
};

constexpr int kF32Window = 2048;            // k per LDS window of activations (four steps: 64 bytes of weights per lane in flight)
constexpr int kF32Waves = 8;

// ROWS: activation rows (1, 2 or 4; M <= ROWS). ST: float, or uint16_t for f16 / bf16 scales.
template <int ROWS, typename ST>
__global__ __launch_bounds__(kF32Waves * 64) void gemv_f32_kernel(GemvF32Params p)
{
    // [ROWS][kF32Window] activations, then [ROWS][kF32Window / 32] sums of runs of 32
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    float* lds_a = reinterpret_cast<float*>(smem);
    float* lds_sum = lds_a + ROWS * kF32Window;

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int sub = lane & 15;                 // lane inside its column's group
    const int64_t col = static_cast<int64_t>(blockIdx.x) * (4 * kF32Waves) + wave * 4 + (lane >> 4);
    const bool live = col < p.n;
    const int64_t padded_k = p.kb << p.bs_log2;

    const __amdgpu_buffer_rsrc_t srd_b = make_srd(p.b + static_cast<int64_t>(blockIdx.x) * (4 * kF32Waves) * p.row_bytes,
                                                  static_cast<uint64_t>((p.n - static_cast<int64_t>(blockIdx.x) * (4 * kF32Waves)) * p.row_bytes));
    const uint32_t b_off = static_cast<uint32_t>((wave * 4 + (lane >> 4)) * p.row_bytes) + static_cast<uint32_t>(sub * 16);   // beyond N: out of range, zeros
    // scales and packed zero points of the workgroup's columns, range-checked the same way; without zero points the
    // zero-sized range returns 0 and the mask / default pair turns that into 8
    const int64_t col0 = static_cast<int64_t>(blockIdx.x) * (4 * kF32Waves);
    const __amdgpu_buffer_rsrc_t srd_s = make_srd(static_cast<const ST*>(p.scales) + col0 * p.kb, static_cast<uint64_t>((p.n - col0) * p.kb) * sizeof(ST));
    const __amdgpu_buffer_rsrc_t srd_z = make_srd(p.zp ? p.zp + col0 * p.zp_row : nullptr, p.zp ? static_cast<uint64_t>((p.n - col0) * p.zp_row) : 0);
    const uint32_t s_off = static_cast<uint32_t>((wave * 4 + (lane >> 4)) * p.kb) * static_cast<uint32_t>(sizeof(ST));
    const uint32_t z_off = static_cast<uint32_t>((wave * 4 + (lane >> 4)) * p.zp_row);
    const uint32_t zp_mask = p.zp ? 0xfu : 0u, zp_default = p.zp ? 0u : 8u;
    const bool scale_bf16 = p.scale_dtype == ROCM_DT_BF16;

    float acc[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) acc[r] = 0.f;

    // The pieces of a window are requested a whole window ahead: piece s of the next window as soon as
    // piece s of this one has been taken out of its registers, so each lane keeps a window of weights in flight.
    constexpr int kSteps = kF32Window / 512;
    u32x4_t piece[kSteps];
    uint32_t scale_raw[kSteps], zp_raw[kSteps];
    auto request = [&](int64_t w0, int s) {
        const int64_t span = padded_k - w0;                    // <= 0 past the end: every lane out of range, nothing fetched
        const uint32_t oor = s * 512 + sub * 32 < span ? 0u : kOutOfRange;   // or-ed in: any offset with these bits is out of range
        const uint32_t blk = static_cast<uint32_t>((w0 + s * 512 + sub * 32) >> p.bs_log2);   // block size >= 32: a piece lies in one block
        piece[s] = __builtin_amdgcn_raw_buffer_load_b128(srd_b, static_cast<int>(b_off | oor), static_cast<int>((w0 + s * 512) >> 1), 0);
        scale_raw[s] = ScaleIo<ST>::load(srd_s, (s_off + blk * static_cast<uint32_t>(sizeof(ST))) | oor, 0);      // a column beyond N is out of range by itself
        zp_raw[s] = __builtin_amdgcn_raw_buffer_load_b8(srd_z, static_cast<int>((z_off + (blk >> 1)) | oor), 0, 0);
    };
#pragma unroll
    for (int s = 0; s < kSteps; ++s) request(0, s);

    for (int64_t w0 = 0; w0 < padded_k; w0 += kF32Window) {
        // ---- fill the window: 4 floats per thread per pass; the sum of a run of 32 by a shuffle over its 8 threads ----
        __syncthreads();
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
#pragma unroll
            for (int i0 = 0; i0 < kF32Window / 4; i0 += kF32Waves * 64) {
                const int i = i0 + t;
                const int64_t k0 = w0 + i * 4;
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (r < p.m && k0 < p.k) v = *reinterpret_cast<const float4*>(p.a + r * p.k + k0);   // K % 4 == 0: whole or nothing
                // 16-byte chunk c of the run of lane `sub` in step `st` sits at [st][c][sub]: the 16 lanes of a column
                // group then read 256 consecutive bytes (in natural order they would sit 128 bytes apart, a 4-way bank conflict)
                *reinterpret_cast<float4*>(lds_a + r * kF32Window + ((((i >> 7) * 8 + (i & 7)) * 16 + ((i >> 3) & 15)) << 2)) = v;
                float s = (v.x + v.y) + (v.z + v.w);
                s += __shfl_xor(s, 1, 64);
                s += __shfl_xor(s, 2, 64);
                s += __shfl_xor(s, 4, 64);
                if ((i & 7) == 0) lds_sum[r * (kF32Window / 32) + (i >> 3)] = s;
            }
        }
        __syncthreads();

        // ---- stream this window of the wave's four columns: steps of 512 k ----
        const int64_t span = padded_k - w0;
#pragma unroll
        for (int step = 0; step < kSteps; ++step) {
            const u32x4_t raw = piece[step];
            const uint32_t sraw = scale_raw[step], zraw = zp_raw[step];
            request(w0 + kF32Window, step);
            const int kw = step * 512 + sub * 32;              // first k of this lane's piece, inside the window
            if (kw >= span) continue;                          // past the end of K (whole steps or the tail of a ragged one)
            const uint32_t wd[4] = {raw.x, raw.y, raw.z, raw.w};
            float dot[ROWS];
#pragma unroll
            for (int r = 0; r < ROWS; ++r) dot[r] = 0.f;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                uint32_t lo = wd[d] & 0x0f0f0f0fu, hi = (wd[d] >> 4) & 0x0f0f0f0fu;         // elements 0,2,4,6 / 1,3,5,7, one per byte
                asm volatile("" : "+v"(lo), "+v"(hi));                                      // keep the bytes whole: one byte-to-float convert each
                float q[8];
                q[0] = static_cast<float>(lo & 0xffu);
                q[2] = static_cast<float>((lo >> 8) & 0xffu);
                q[4] = static_cast<float>((lo >> 16) & 0xffu);
                q[6] = static_cast<float>(lo >> 24);
                q[1] = static_cast<float>(hi & 0xffu);
                q[3] = static_cast<float>((hi >> 8) & 0xffu);
                q[5] = static_cast<float>((hi >> 16) & 0xffu);
                q[7] = static_cast<float>(hi >> 24);
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    const float4 a0 = *reinterpret_cast<const float4*>(lds_a + r * kF32Window + (((step * 8 + d * 2) * 16 + sub) << 2));
                    const float4 a1 = *reinterpret_cast<const float4*>(lds_a + r * kF32Window + (((step * 8 + d * 2 + 1) * 16 + sub) << 2));
                    float s = dot[r];
                    s = fmaf(a0.x, q[0], s);
                    s = fmaf(a0.y, q[1], s);
                    s = fmaf(a0.z, q[2], s);
                    s = fmaf(a0.w, q[3], s);
                    s = fmaf(a1.x, q[4], s);
                    s = fmaf(a1.y, q[5], s);
                    s = fmaf(a1.z, q[6], s);
                    s = fmaf(a1.w, q[7], s);
                    dot[r] = s;
                }
            }
            {
                const uint32_t blk = static_cast<uint32_t>((w0 + kw) >> p.bs_log2);
                const float sc = ScaleIo<ST>::to_f32(sraw, scale_bf16);                       // 0 for a column beyond N
                const float z = static_cast<float>((((zraw >> ((blk & 1u) * 4u)) & 0xfu) & zp_mask) | zp_default);
#pragma unroll
                for (int r = 0; r < ROWS; ++r) acc[r] = fmaf(fmaf(-z, lds_sum[r * (kF32Window / 32) + (kw >> 5)], dot[r]), sc, acc[r]);
            }
        }
    }

    // ---- the 16 lanes of a column add up; lane 0 of the group stores ----
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        float v = acc[r];
        v += __shfl_xor(v, 1, 64);
        v += __shfl_xor(v, 2, 64);
        v += __shfl_xor(v, 4, 64);
        v += __shfl_xor(v, 8, 64);
        if (sub == 0 && live && r < p.m) {
            v = with_bias(v, p.bias, p.bias_dtype, r, p.n, col, p.y_dtype);
            store_from_f32(p.y, p.y_dtype, r * p.n + col, v);
        }
    }
}

template <int ROWS, typename ST>
static int launch_gemv_f32(const GemvF32Params& p, hipStream_t stream)
{
    const unsigned grid = static_cast<unsigned>((p.n + 4 * kF32Waves - 1) / (4 * kF32Waves));
    const size_t lds = static_cast<size_t>(ROWS) * (kF32Window + kF32Window / 32) * sizeof(float);
    auto kernel = gemv_f32_kernel<ROWS, ST>;
    if (lds > 65536) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
        if (e != hipSuccess) return static_cast<int>(e);
    }
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kF32Waves * 64), lds, stream, p);
    return static_cast<int>(hipGetLastError());
}

}  // namespace mnb

extern "C" int rocm_gemv_f32_eligible(const RocmMatMulNBitsArgs* a)
{
    if (a->a_dtype != ROCM_DT_F32 || a->m < 1 || a->m > 4 || a->n < 1 || a->block_size < 32 || a->k % 4 != 0) return 0;
    const int64_t kb = (a->k + a->block_size - 1) / a->block_size;
    if (kb * a->block_size / 2 * 32 >= 0x7fffffff) return 0;                 // 32-bit offsets inside a workgroup's 32 columns
    return (reinterpret_cast<uintptr_t>(a->a) & 15) == 0 && (reinterpret_cast<uintptr_t>(a->b) & 15) == 0;
}

extern "C" int rocm_launch_gemv_f32(const RocmMatMulNBitsArgs* a, rocm_stream_t stream)
{
    if (!rocm_gemv_f32_eligible(a)) return -1;
    mnb::GemvF32Params p;
    p.a = static_cast<const float*>(a->a);
    p.b = a->b;
    p.scales = a->scales;
    p.zp = a->zp;
    p.bias = a->bias;
    p.y = a->y;
    p.m = a->m;
    p.n = a->n;
    p.k = a->k;
    p.kb = (a->k + a->block_size - 1) / a->block_size;
    p.row_bytes = p.kb * a->block_size / 2;
    p.zp_row = (p.kb + 1) / 2;
    p.bs_log2 = __builtin_ctz(static_cast<unsigned>(a->block_size));
    p.scale_dtype = a->scale_dtype;
    p.bias_dtype = a->bias_dtype;
    p.y_dtype = a->y_dtype;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (a->scale_dtype == ROCM_DT_F32) {
        if (a->m <= 1) return mnb::launch_gemv_f32<1, float>(p, s);
        if (a->m <= 2) return mnb::launch_gemv_f32<2, float>(p, s);
        return mnb::launch_gemv_f32<4, float>(p, s);
    }
    if (a->m <= 1) return mnb::launch_gemv_f32<1, uint16_t>(p, s);
    if (a->m <= 2) return mnb::launch_gemv_f32<2, uint16_t>(p, s);
    return mnb::launch_gemv_f32<4, uint16_t>(p, s);
}
