// Dense route for tall prefill calls: the packed weights are expanded once into a 16-bit [N, K] matrix in HBM and the
// product is a plain library GEMM (hipBLASLt, f32 accumulation). The expansion costs one pass over N*K regardless of
// M, so it pays once M is large; a constant weight can keep its dense copy, after which the call is the GEMM alone.
// Same idea as the reference's CUDA provider, which materializes fp16 weights and calls cuBLASLt for M >= 8
// (onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:6176-6222).
//
// Each dense element is (q - zp) * scale computed in f32 and rounded once to the 16-bit type (nearest even): the value
// the tiled kernel in prefill_mfma.hip feeds its matrix cores.
#include "common.hiph"

#include <hipblaslt/hipblaslt.h>

#include <dlfcn.h>

#include <map>
#include <mutex>
#include <tuple>
#include <type_traits>

namespace mnb {

// The library is an opt-in route (dense_gemm_min_rows, dense_weights = resident): it is opened when a provider first asks
// for it and is no link-time dependency of this library. The header only supplies the types.
struct BlasLt {
    decltype(&hipblasLtCreate) Create = nullptr;
    decltype(&hipblasLtDestroy) Destroy = nullptr;
    decltype(&hipblasLtMatmulDescCreate) MatmulDescCreate = nullptr;
    decltype(&hipblasLtMatmulDescDestroy) MatmulDescDestroy = nullptr;
    decltype(&hipblasLtMatmulDescSetAttribute) MatmulDescSetAttribute = nullptr;
    decltype(&hipblasLtMatrixLayoutCreate) MatrixLayoutCreate = nullptr;
    decltype(&hipblasLtMatrixLayoutDestroy) MatrixLayoutDestroy = nullptr;
    decltype(&hipblasLtMatmulPreferenceCreate) MatmulPreferenceCreate = nullptr;
    decltype(&hipblasLtMatmulPreferenceDestroy) MatmulPreferenceDestroy = nullptr;
    decltype(&hipblasLtMatmulPreferenceSetAttribute) MatmulPreferenceSetAttribute = nullptr;
    decltype(&hipblasLtMatmulAlgoGetHeuristic) MatmulAlgoGetHeuristic = nullptr;
    decltype(&hipblasLtMatmul) Matmul = nullptr;
    bool ok = false;
};

static const BlasLt& blaslt()
{
    static const BlasLt table = [] {
        BlasLt t;
        void* lib = dlopen("libhipblaslt.so", RTLD_NOW | RTLD_LOCAL);
        if (!lib) lib = dlopen("/opt/rocm/lib/libhipblaslt.so", RTLD_NOW | RTLD_LOCAL);
        if (!lib) return t;
        bool all = true;
        auto get = [&](auto& fn, const char* name) {
            fn = reinterpret_cast<std::remove_reference_t<decltype(fn)>>(dlsym(lib, name));
            all = all && fn != nullptr;
        };
        get(t.Create, "hipblasLtCreate");
        get(t.Destroy, "hipblasLtDestroy");
        get(t.MatmulDescCreate, "hipblasLtMatmulDescCreate");
        get(t.MatmulDescDestroy, "hipblasLtMatmulDescDestroy");
        get(t.MatmulDescSetAttribute, "hipblasLtMatmulDescSetAttribute");
        get(t.MatrixLayoutCreate, "hipblasLtMatrixLayoutCreate");
        get(t.MatrixLayoutDestroy, "hipblasLtMatrixLayoutDestroy");
        get(t.MatmulPreferenceCreate, "hipblasLtMatmulPreferenceCreate");
        get(t.MatmulPreferenceDestroy, "hipblasLtMatmulPreferenceDestroy");
        get(t.MatmulPreferenceSetAttribute, "hipblasLtMatmulPreferenceSetAttribute");
        get(t.MatmulAlgoGetHeuristic, "hipblasLtMatmulAlgoGetHeuristic");
        get(t.Matmul, "hipblasLtMatmul");
        t.ok = all;
        return t;
    }();
    return table;
}

// Each thread expands one packed dword (8 consecutive k of one column) into one 16-byte store. K % 8 == 0.
template <bool BF16>
__global__ __launch_bounds__(256) void dequant_16_kernel(
    const uint8_t* __restrict__ b, const void* __restrict__ scales, int scale_dtype,
    const uint8_t* __restrict__ zp, int64_t n, int64_t k, int bs_log2, int64_t kb, uint16_t* __restrict__ out)
{
    const int64_t row_dwords = (kb << bs_log2) >> 3;           // packed dwords per column, padding of the last block included
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
        uint32_t pair[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // as_f32: the f32 product is a value of its own (f32 scales: a fused product-and-convert would round once)
            const float lo = as_f32(__fmul_rn(static_cast<float>((w >> (8 * i)) & 0xf) - z, s));
            const float hi = as_f32(__fmul_rn(static_cast<float>((w >> (8 * i + 4)) & 0xf) - z, s));
            const uint32_t l16 = BF16 ? f32_to_bf16_bits(lo) : f32_to_f16_bits(lo);
            const uint32_t h16 = BF16 ? f32_to_bf16_bits(hi) : f32_to_f16_bits(hi);
            pair[i] = l16 | (h16 << 16);
        }
        *reinterpret_cast<uint4*>(out + col * k + k0) = make_uint4(pair[0], pair[1], pair[2], pair[3]);
    }
}

struct GemmPlan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t lay_w = nullptr, lay_a = nullptr, lay_y = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;
    bool usable = false;
};

}  // namespace mnb

struct RocmDenseGemm {
    hipblasLtHandle_t handle = nullptr;
    void* workspace = nullptr;
    size_t workspace_bytes = 0;
    std::mutex mu;
    // (m, n, k, 16-bit type, bias type or -1) -> plan
    std::map<std::tuple<int64_t, int64_t, int64_t, int, int>, mnb::GemmPlan> plans;
};

namespace mnb {

constexpr size_t kGemmWorkspace = 64u << 20;

static hipDataType hip_type(int dtype) { return dtype == ROCM_DT_BF16 ? HIP_R_16BF : dtype == ROCM_DT_F16 ? HIP_R_16F : HIP_R_32F; }

static void destroy_plan(GemmPlan& p)
{
    if (p.lay_w) mnb::blaslt().MatrixLayoutDestroy(p.lay_w);
    if (p.lay_a) mnb::blaslt().MatrixLayoutDestroy(p.lay_a);
    if (p.lay_y) mnb::blaslt().MatrixLayoutDestroy(p.lay_y);
    if (p.desc) mnb::blaslt().MatmulDescDestroy(p.desc);
    p = GemmPlan();
}

// Row-major Y[M,N] = A[M,K] * W[N,K]^T is, in the library's column-major terms, D(N x M) = W'(K x N)^T * A'(K x M).
static GemmPlan make_plan(RocmDenseGemm& g, int64_t m, int64_t n, int64_t k, int dtype, int bias_dtype)
{
    GemmPlan p;
    const hipDataType t = hip_type(dtype);
    bool ok = mnb::blaslt().MatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS;
    const hipblasOperation_t op_t = HIPBLAS_OP_T, op_n = HIPBLAS_OP_N;
    ok = ok && mnb::blaslt().MatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_t, sizeof(op_t)) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && mnb::blaslt().MatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof(op_n)) == HIPBLAS_STATUS_SUCCESS;
    if (ok && bias_dtype >= 0) {
        const hipblasLtEpilogue_t epi = HIPBLASLT_EPILOGUE_BIAS;
        const int32_t bt = static_cast<int32_t>(hip_type(bias_dtype));
        ok = mnb::blaslt().MatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epi, sizeof(epi)) == HIPBLAS_STATUS_SUCCESS &&
             mnb::blaslt().MatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bt, sizeof(bt)) == HIPBLAS_STATUS_SUCCESS;
    }
    ok = ok && mnb::blaslt().MatrixLayoutCreate(&p.lay_w, t, static_cast<uint64_t>(k), static_cast<uint64_t>(n), k) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && mnb::blaslt().MatrixLayoutCreate(&p.lay_a, t, static_cast<uint64_t>(k), static_cast<uint64_t>(m), k) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && mnb::blaslt().MatrixLayoutCreate(&p.lay_y, t, static_cast<uint64_t>(n), static_cast<uint64_t>(m), n) == HIPBLAS_STATUS_SUCCESS;
    hipblasLtMatmulPreference_t pref = nullptr;
    ok = ok && mnb::blaslt().MatmulPreferenceCreate(&pref) == HIPBLAS_STATUS_SUCCESS;
    if (ok) {
        const uint64_t cap = g.workspace_bytes;
        hipblasLtMatmulHeuristicResult_t found[1];
        int count = 0;
        ok = mnb::blaslt().MatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &cap, sizeof(cap)) == HIPBLAS_STATUS_SUCCESS &&
             mnb::blaslt().MatmulAlgoGetHeuristic(g.handle, p.desc, p.lay_w, p.lay_a, p.lay_y, p.lay_y, pref, 1, found, &count) == HIPBLAS_STATUS_SUCCESS &&
             count > 0 && found[0].state == HIPBLAS_STATUS_SUCCESS && found[0].workspaceSize <= g.workspace_bytes;
        if (ok) {
            p.algo = found[0].algo;
            p.workspace = found[0].workspaceSize;
        }
    }
    if (pref) mnb::blaslt().MatmulPreferenceDestroy(pref);
    if (!ok) {
        destroy_plan(p);
        return p;
    }
    p.usable = true;
    return p;
}

}  // namespace mnb

extern "C" int rocm_launch_dequant_16(const uint8_t* b, const void* scales, int scale_dtype, const uint8_t* zp,
                                      int64_t n, int64_t k, int block_size, int out_dtype, void* out_nk, rocm_stream_t stream)
{
    if (n <= 0 || k <= 0) return 0;
    if ((k & 7) != 0 || (out_dtype != ROCM_DT_F16 && out_dtype != ROCM_DT_BF16)) return static_cast<int>(hipErrorInvalidValue);
    const int bs_log2 = __builtin_ctz(static_cast<unsigned>(block_size));
    const int64_t kb = (k + block_size - 1) / block_size;
    const int64_t total = n * ((kb * block_size) / 8);
    int64_t blocks = (total + 255) / 256;
    if (blocks > 262144) blocks = 262144;
    uint16_t* out = static_cast<uint16_t*>(out_nk);
    if (out_dtype == ROCM_DT_BF16)
        hipLaunchKernelGGL(mnb::dequant_16_kernel<true>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream), b, scales,
                           scale_dtype, zp, n, k, bs_log2, kb, out);
    else
        hipLaunchKernelGGL(mnb::dequant_16_kernel<false>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream), b, scales,
                           scale_dtype, zp, n, k, bs_log2, kb, out);
    return static_cast<int>(hipGetLastError());
}

extern "C" int rocm_dense_gemm_create(RocmDenseGemm** out)
{
    *out = nullptr;
    RocmDenseGemm* g = new (std::nothrow) RocmDenseGemm();
    if (!g) return static_cast<int>(hipErrorOutOfMemory);
    if (!mnb::blaslt().ok) {                       // the library is not on this machine: the caller keeps the tiled kernel
        delete g;
        return static_cast<int>(hipErrorSharedObjectInitFailed);
    }
    if (mnb::blaslt().Create(&g->handle) != HIPBLAS_STATUS_SUCCESS) {
        delete g;
        return static_cast<int>(hipErrorNotInitialized);
    }
    const hipError_t e = static_cast<hipError_t>(rocm_ffi_malloc(&g->workspace, mnb::kGemmWorkspace));                 // (counted with the library's other allocations)
    if (e != hipSuccess) {
        mnb::blaslt().Destroy(g->handle);
        delete g;
        return static_cast<int>(e);
    }
    g->workspace_bytes = mnb::kGemmWorkspace;
    *out = g;
    return 0;
}

extern "C" void rocm_dense_gemm_destroy(RocmDenseGemm* g)
{
    if (!g) return;
    for (auto& kv : g->plans) mnb::destroy_plan(kv.second);
    if (g->workspace) (void)rocm_ffi_free(g->workspace);
    if (g->handle) mnb::blaslt().Destroy(g->handle);
    delete g;
}

// 1 when a library kernel is on hand for the shape. A shape is looked up once; `may_plan` = 0 (a graph capture is
// open) only consults what earlier calls found.
extern "C" int rocm_dense_gemm_ready(RocmDenseGemm* g, int64_t m, int64_t n, int64_t k, int dtype, int bias_dtype, int may_plan)
{
    if (!g || (dtype != ROCM_DT_F16 && dtype != ROCM_DT_BF16)) return 0;
    if (bias_dtype >= 0 && bias_dtype != ROCM_DT_F32 && bias_dtype != dtype) return 0;   // bias in the output's type or in f32
    std::lock_guard<std::mutex> lock(g->mu);
    const auto key = std::make_tuple(m, n, k, dtype, bias_dtype);
    auto it = g->plans.find(key);
    if (it == g->plans.end()) {
        if (!may_plan) return 0;
        it = g->plans.emplace(key, mnb::make_plan(*g, m, n, k, dtype, bias_dtype)).first;
    }
    return it->second.usable ? 1 : 0;
}

// Y[M,N] = A[M,K] * W[N,K]^T (+ bias[N]), all 16-bit of one type, f32 accumulation, one rounding at the end.
// Returns 0, a HIP error code, or 10000 + the library's status.
extern "C" int rocm_dense_gemm_run(RocmDenseGemm* g, const void* w_nk, const void* a, void* y, const void* bias, int bias_dtype,
                                   int64_t m, int64_t n, int64_t k, int dtype, rocm_stream_t stream)
{
    if (!g) return static_cast<int>(hipErrorInvalidValue);
    std::lock_guard<std::mutex> lock(g->mu);
    auto it = g->plans.find(std::make_tuple(m, n, k, dtype, bias ? bias_dtype : -1));
    if (it == g->plans.end() || !it->second.usable) return static_cast<int>(hipErrorInvalidValue);
    mnb::GemmPlan& p = it->second;
    if (bias && mnb::blaslt().MatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias)) != HIPBLAS_STATUS_SUCCESS)
        return 10000 + static_cast<int>(HIPBLAS_STATUS_INVALID_VALUE);
    const float one = 1.f, zero = 0.f;
    const hipblasStatus_t st = mnb::blaslt().Matmul(g->handle, p.desc, &one, w_nk, p.lay_w, a, p.lay_a, &zero, y, p.lay_y, y, p.lay_y, &p.algo,
                                               g->workspace, g->workspace_bytes, static_cast<hipStream_t>(stream));
    return st == HIPBLAS_STATUS_SUCCESS ? 0 : 10000 + static_cast<int>(st);
}
