// Accessor compiled INTO oracle/_ref/libmlas_ref.so next to the reference's own MLAS objects.
// It exposes two things the reference's plain-C shim (crates/mlas-sys/vendor/shim.cpp) keeps
// internal, so a parity test can look at them:
//   * the per-block int8 activation codes, scales and scaled block sums that
//     InitializeWorkspace_CompInt8 (core/mlas/lib/qnbitgemm.cpp:1105-1235) produces through the
//     dispatch entry QuantizeARowComputeBlkSum_CompInt8 (core/mlas/lib/qnbitgemm.h:672-680);
//   * which SQNBit dispatch table the host CPU selected (platform.cpp).
// Test infrastructure only; nothing in the product library links this file.

#include "mlasi.h"
#include "qnbitgemm.h"

extern "C" {

// Returns 0 on success, -1 when the selected dispatch has no separate-scale int8 row quantizer.
// qa: [m, kb*blk_len] int8, qscale: [m, kb] f32, blksum: [m, kb] f32 (scale * sum of codes).
int mlas_ref_quantize_a_rows(
    size_t m, size_t k, size_t blk_len, const float* a, size_t lda,
    int8_t* qa, float* qscale, float* blksum)
{
    const auto* dispatch = GetMlasPlatform().QNBitGemmDispatch;
    if (dispatch == nullptr || dispatch->QuantizeARowComputeBlkSum_CompInt8 == nullptr) {
        return -1;
    }
    const size_t kb = (k + blk_len - 1) / blk_len;
    for (size_t r = 0; r < m; ++r) {
        dispatch->QuantizeARowComputeBlkSum_CompInt8(
            blk_len, a + r * lda, k,
            reinterpret_cast<std::byte*>(qa + r * kb * blk_len),
            qscale + r * kb, blksum + r * kb);
    }
    return 0;
}

// 0 = none, 2 = AVX2, 3 = AVX2+VNNI, 512 = AVX-512 core, 513 = AVX-512 VNNI
int mlas_ref_qnbit_dispatch_id()
{
    const auto* d = GetMlasPlatform().QNBitGemmDispatch;
    if (d == nullptr) return 0;
    if (d == &MlasSQNBitGemmDispatchAvx512vnni) return 513;
    if (d == &MlasSQNBitGemmDispatchAvx512) return 512;
    if (d == &MlasSQNBitGemmDispatchAvx2vnni) return 3;
    if (d == &MlasSQNBitGemmDispatchAvx2) return 2;
    return 1;
}

}  // extern "C"
