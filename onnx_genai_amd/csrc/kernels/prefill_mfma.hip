// Prefill path placeholder: filled in by the LDS-staged dequant + MFMA GEMM.
#include "common.hiph"
extern "C" int rocm_prefill_mfma_eligible(const RocmMatMulNBitsArgs*) { return 0; }
extern "C" int rocm_launch_prefill_mfma(const RocmMatMulNBitsArgs*, rocm_stream_t) { return -1; }
