/*
 * The only doorway from the execution provider's host code to HIP: device memory, one stream,
 * events, and one launcher per hand-written gfx950 kernel. Plain C types only. Every function
 * returns 0 on success or the hipError_t value; rocm_ffi_error_string() names it.
 */
#ifndef NXRT_ROCM_HIP_FFI_H
#define NXRT_ROCM_HIP_FFI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* rocm_stream_t;
typedef void* rocm_event_t;

/* element dtypes on the wire (onnx-runtime-ir DataType discriminants) */
enum { ROCM_DT_F32 = 1, ROCM_DT_U8 = 2, ROCM_DT_I32 = 6, ROCM_DT_F16 = 10, ROCM_DT_BF16 = 16 };
/* Or-ed into a bias dtype: the bias is a folded standalone Add. The accumulator is rounded to the output's 16-bit type
 * first and the bias added with a second rounding, round(round(acc) + bias), which is what MatMulNBits followed by Add
 * produces (onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:1189-1212). Without it: round(acc + bias). */
enum { ROCM_BIAS_POST_ROUND = 0x100 };
/* Or-ed into a bias dtype: the bias slot carries a per-token residual [M, N] (row stride N) instead of a broadcast [N] - what
 * the CUDA provider's folded residual epilogue passes (kernels/matmul_nbits.rs:7891-7897). */
enum { ROCM_BIAS_PER_ROW = 0x200 };

const char* rocm_ffi_error_string(int err);
int rocm_ffi_device_count(int* count);
int rocm_ffi_set_device(int device);
int rocm_ffi_device_info(int device, char* arch, size_t arch_len, int* compute_units, size_t* total_mem);
/* Compute units of the current device (asked once per device and kept); 256, the MI355X's count, when it cannot be asked.
 * The launchers size grids and wave counts to it. */
int rocm_ffi_compute_units(void);
int rocm_ffi_malloc(void** ptr, size_t bytes);
int rocm_ffi_free(void* ptr);
/* How many times rocm_ffi_malloc has been called in this process. Every device allocation of the library goes through it, the
 * library GEMM route's workspace and the g_idx range check's flag included. */
uint64_t rocm_ffi_malloc_calls(void);
/* Device address and size of the library's static scratch array on `device` (a __device__ array of the code object, 256-byte
 * aligned, one per GPU, never freed). The first call for a device makes that device current and resolves the address; later
 * calls only read it back. Shared by every caller on that GPU and never cleared: contents are whatever the last user left.
 * The first call also creates the event that chains the array's users (below). */
int rocm_ffi_static_scratch(int device, void** ptr, size_t* bytes);
/* Bracket the launches of one user of that array. `begin` takes the device's host lock and, if the previous user enqueued
 * on another stream, makes `stream` wait (on the GPU, hipStreamWaitEvent) for the event that user recorded; `end` records
 * the event on `stream` and drops the lock: users on different streams of one GPU run one after the other, in the order
 * of their `begin`. Neither allocates device memory. Not for a stream under capture (events from outside a capture cannot
 * be waited for inside one): a caller skips both there. A failed `begin` holds no lock. */
int rocm_ffi_static_scratch_begin(int device, rocm_stream_t stream);
int rocm_ffi_static_scratch_end(int device, rocm_stream_t stream);
int rocm_ffi_memcpy_h2d(void* dst, const void* src, size_t bytes, rocm_stream_t stream);
int rocm_ffi_memcpy_d2h(void* dst, const void* src, size_t bytes, rocm_stream_t stream);
/* Reads `bytes` (a multiple of 16 is read) of device memory and keeps nothing: the time of the plainest kernel that pulls
 * that many bytes, for benchmarks to hold other kernels against. `sink`: 4 writable bytes, or NULL. */
int rocm_ffi_read_probe(const void* src, size_t bytes, void* sink, rocm_stream_t stream);
/* Bytes per clock one CU's LDS moves when `waves` waves (1..16) of one workgroup per CU each repeat eight 16-byte accesses
 * per lane `iters` times. mode 0: ds_read_b128; 1: ds_write_b128; 2: global memory straight into LDS; 3: even waves read, odd
 * waves write (the figure is the sum of both). Synchronous, allocates its own small buffers: a diagnostic, not a kernel path. */
int rocm_ffi_lds_probe(int mode, int waves, int iters, double* bytes_per_clock);
int rocm_ffi_memcpy_d2d(void* dst, const void* src, size_t bytes, rocm_stream_t stream);
int rocm_ffi_stream_create(rocm_stream_t* stream);
int rocm_ffi_stream_destroy(rocm_stream_t stream);
int rocm_ffi_stream_sync(rocm_stream_t stream);
int rocm_ffi_event_create(rocm_event_t* event);
int rocm_ffi_event_destroy(rocm_event_t event);
int rocm_ffi_event_record(rocm_event_t event, rocm_stream_t stream);
int rocm_ffi_event_sync(rocm_event_t event);
int rocm_ffi_event_elapsed_ms(rocm_event_t start, rocm_event_t stop, float* ms);
int rocm_ffi_fill_u32(void* dst, uint32_t value, size_t count, rocm_stream_t stream);

/* Stream capture into an executable HIP graph, and its replay on a stream. */
typedef void* rocm_graph_exec_t;
int rocm_ffi_capture_begin(rocm_stream_t stream);
int rocm_ffi_capture_end(rocm_stream_t stream, rocm_graph_exec_t* exec, size_t* num_nodes);
int rocm_ffi_graph_launch(rocm_graph_exec_t exec, rocm_stream_t stream);
int rocm_ffi_graph_destroy(rocm_graph_exec_t exec);

/* Operands of one MatMulNBits call, all device pointers, all contiguous. */
typedef struct RocmMatMulNBitsArgs {
  const void* a;        /* [M, K] a_dtype */
  const uint8_t* b;     /* [N, kb, bs/2] */
  const void* scales;   /* [N, kb] scale_dtype */
  const uint8_t* zp;    /* [N, ceil(kb/2)] or NULL (zero point 8) */
  const void* bias;     /* [N] bias_dtype or NULL; bias_dtype may carry ROCM_BIAS_POST_ROUND */
  void* y;              /* [M, N] y_dtype */
  int a_dtype, scale_dtype, bias_dtype, y_dtype;
  int64_t m, n, k;
  int block_size;
  const int32_t* g_idx;  /* [K] group of every element (act-order), or NULL: group = k / block_size. Only the plain kernels read it. */
  int32_t* acc_probe;    /* accuracy_level 4, int8 matrix-core kernels only: int32 [M, N, kb], or NULL. When set, the kernel also
                            stores every block accumulator sum_k code * (q - zp) it flushes - the integer its f32 result is built
                            from - so that a test can compare the production kernels' integers bit for bit. */
  const void* gamma;     /* RMS-normalization prologue inside the kernel: the weight [K], or NULL. Only rocm_launch_decode_packed and
                            rocm_launch_decode_packed_pair read it, and only where rocm_decode_packed_fuses_norm() holds: the
                            activations are then replaced by round16((a * inv_std) * gamma), inv_std = 1 / sqrt(mean(a^2) + eps). */
  int gamma_dtype;       /* ROCM_DT_F32 or a_dtype */
  float norm_epsilon;
} RocmMatMulNBitsArgs;

/* w[n,k] = (q - zp) * scale as f32 [N, K]. */
int rocm_launch_dequant_f32(const uint8_t* b, const void* scales, int scale_dtype, const uint8_t* zp,
                            int64_t n, int64_t k, int block_size, float* out_nk, rocm_stream_t stream);

/* w[n,k] = (q - zp) * scale, computed in f32 and rounded once (nearest even) to out_dtype (f16 or bf16), [N, K].
 * K % 8 == 0 and out_nk 16-byte aligned. */
int rocm_launch_dequant_16(const uint8_t* b, const void* scales, int scale_dtype, const uint8_t* zp,
                           int64_t n, int64_t k, int block_size, int out_dtype, void* out_nk, rocm_stream_t stream);

/* The library GEMM (hipBLASLt) behind the dense prefill route: Y[M,N] = A[M,K] * W[N,K]^T (+ bias[N]); A, W, Y of one
 * 16-bit type, f32 accumulation. create / destroy allocate and free (never inside a graph capture); ready looks a shape
 * up once (may_plan = 0 only consults earlier lookups) and returns 1 when a kernel is on hand; run enqueues it and
 * returns 0, a HIP error code, or 10000 + the library's status. */
typedef struct RocmDenseGemm RocmDenseGemm;
int rocm_dense_gemm_create(RocmDenseGemm** out);
void rocm_dense_gemm_destroy(RocmDenseGemm* g);
int rocm_dense_gemm_ready(RocmDenseGemm* g, int64_t m, int64_t n, int64_t k, int dtype, int bias_dtype, int may_plan);
int rocm_dense_gemm_run(RocmDenseGemm* g, const void* w_nk, const void* a, void* y, const void* bias, int bias_dtype,
                        int64_t m, int64_t n, int64_t k, int dtype, rocm_stream_t stream);

/* y = round16(silu(gate) * up) over `count` 16-bit elements (f16 or bf16): the epilogue of the fused gate/up node
 * (onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:4207-4233, 4375-4386). decomposed = 1: silu spelled as Sigmoid and Mul. */
int rocm_launch_swiglu(const void* gate, const void* up, int64_t count, int dtype, int decomposed, void* y, rocm_stream_t stream);

/* out = round16((a * inv_std) * gamma) per row of K 16-bit elements (K % 128 == 0), inv_std = 1 / sqrt(mean(a^2) + eps),
 * summed in the reference's order (onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:4125-4205). gamma: f32 or 16-bit. */
int rocm_launch_rmsnorm16(const void* a, const void* gamma, int gamma_dtype, int64_t rows, int64_t k, float epsilon, int dtype, void* out,
                          rocm_stream_t stream);

/* bits = 2 or 8 (element i of a packed row in byte i / (8 / bits) at bit (i % (8 / bits)) * bits; zero points packed alike,
 * default 1 << (bits - 1)): w[n,k] = (q - zp) * scale as f32, f16 or bf16 [N, K] (one f32 multiply, then one rounding), and
 * the f32 GEMV with one wave per output column (args as for 4 bits, b / zp in the wider or narrower layout). */
int rocm_launch_dequant_nbits(const uint8_t* b, const void* scales, int scale_dtype, const uint8_t* zp, int64_t n, int64_t k, int block_size,
                              int bits, int out_dtype, void* out_nk, rocm_stream_t stream);
int rocm_launch_gemv_nbits(const RocmMatMulNBitsArgs* args, int bits, rocm_stream_t stream);
/* The same with g_idx (bits 2, 4 or 8): scale and zero point of element k come from group g_idx[k]. */
int rocm_launch_dequant_gidx(const uint8_t* b, const void* scales, int scale_dtype, const uint8_t* zp, const int32_t* g_idx, int64_t n, int64_t k,
                             int block_size, int bits, int out_dtype, void* out_nk, rocm_stream_t stream);
/* First index whose group lies outside 0..kb, or -1: synchronizes the stream and allocates (never inside a graph capture). */
int rocm_g_idx_first_bad(const int32_t* g_idx, int64_t count, int64_t kb, int64_t* first_bad, rocm_stream_t stream);

/* Any dtype mix, any K, any block size: f32 math, one wave per output column. */
int rocm_launch_gemv_generic(const RocmMatMulNBitsArgs* args, rocm_stream_t stream);
/* f32 activations, M <= 4, block size >= 32, K % 4 == 0, A and B 16-byte aligned: f32 FMA streaming kernel */
int rocm_gemv_f32_eligible(const RocmMatMulNBitsArgs* args);
int rocm_launch_gemv_f32(const RocmMatMulNBitsArgs* args, rocm_stream_t stream);

/* Decode (M <= 16), f16/bf16 activations: split-K MFMA GEMV. Returns -1 when the shape is not eligible.
 * waves/col_groups = 0 lets the launcher choose. */
int rocm_decode_mfma_eligible(const RocmMatMulNBitsArgs* args);
int rocm_launch_decode_mfma(const RocmMatMulNBitsArgs* args, int waves, int col_groups, rocm_stream_t stream);

/* Decode over constant weights repacked for streaming (M <= 4). `packed` holds rocm_decode_packed_bytes() bytes and is
 * filled once by rocm_launch_pack_decode from args->b / scales / zp; rocm_launch_decode_packed then reads only it. */
int rocm_decode_packed_eligible(const RocmMatMulNBitsArgs* args);
uint64_t rocm_decode_packed_bytes(const RocmMatMulNBitsArgs* args);
int rocm_launch_pack_decode(const RocmMatMulNBitsArgs* args, void* packed, rocm_stream_t stream);
int rocm_launch_decode_packed(const RocmMatMulNBitsArgs* args, const void* packed, int waves, rocm_stream_t stream);
/* What rocm_launch_decode_packed would launch for `args` on a chip of `compute_units` CUs, without launching anything (only the
 * shape, dtypes, block size and gamma of `args` are read). pair_member: 0 = a plain call, 1 = one projection of a gate/up pair
 * launched alone, 2 = the paired launch. -1: the shape does not take this route. */
typedef struct RocmDecodePackedPlan {
  int shared_activations;   /* 1: the kernel that shares one LDS copy of the activations; 0: the split-K kernel */
  int rows_build;           /* rows the build stages: 1, 4, 8 or 16 (shared activations: 16, 32 or 64) */
  int waves;                /* per workgroup (split-K kernel: per projection) */
  int groups_per_wave;      /* tile groups of 512 k a wave walks */
  int register_sets;        /* sets of load registers in flight: 1 or 2 (shared activations: 1 + weights ahead + windows two ahead) */
  int activation_sums;      /* 1: offset and zero point leave through the block activation sums; 0: through a second MFMA */
  int64_t workgroups;
} RocmDecodePackedPlan;
int rocm_decode_packed_plan(const RocmMatMulNBitsArgs* args, int waves, int pair_member, int compute_units, RocmDecodePackedPlan* out);
/* 1 when the launch above (and the paired one below) applies args->gamma inside the kernel: up to 4 rows, K % 128 == 0, gamma f32 or
 * of the activations' type and 16-byte aligned, and a shape the split-K kernel takes (not the shared-activation one). */
int rocm_decode_packed_fuses_norm(const RocmMatMulNBitsArgs* args);
/* Waves per SIMD that the launcher assumes for the one-register-set build serving `m` rows (1, 2-4, 5-8, 9-16) when it sizes
 * a launch to the chip; a test holds it against the registers the build reported. */
int rocm_decode_packed_waves_per_simd(int block_size, int m, int f32_scales, int bf16);
/* The fused gate/up node at up to four rows: one launch over both projections' repacked copies; Y (the activations'
 * 16-bit type) = round16(silu(round16(gate)) * round16(up)), each projection summed exactly as its own launch would.
 * args names the shared operands (a, y, m, n, k, block_size, dtypes; b / scales / zp only for the eligibility checks).
 * rocm_decode_packed_pair_fits: 1 when both projections' waves fit one workgroup; otherwise run them separately.
 * rocm_launch_decode_packed_pair_member: one projection of such a pair on its own, with the pair's split of K. */
int rocm_launch_decode_packed_pair_member(const RocmMatMulNBitsArgs* args, const void* packed, int waves, rocm_stream_t stream);
int rocm_decode_packed_pair_fits(const RocmMatMulNBitsArgs* args, int waves);
int rocm_launch_decode_packed_pair(const RocmMatMulNBitsArgs* args, const void* packed_gate, const void* packed_up, int decomposed, int waves,
                                   rocm_stream_t stream);

/* Prefill (M > 16), f16/bf16 activations: B tiles dequantized into LDS, 32x32x16 MFMA.
 * tile_choice: 0 = by shape, 1 = 128 x 128, 2 = 256 x 128, 3 = 256 x 256, 4 = 128 x 64 tiles of Y per workgroup. */
int rocm_prefill_mfma_eligible(const RocmMatMulNBitsArgs* args);
/* Small grids with long K are cut into slices of K whose f32 partial sums land in `scratch` ([slices][M][N]) and are added up
 * by a second kernel; rocm_prefill_mfma_scratch_bytes says how much the preferred plan wants (0 = no slicing). With less
 * scratch the launcher uses fewer slices, with none it does not slice. */
uint64_t rocm_prefill_mfma_scratch_bytes(const RocmMatMulNBitsArgs* args, int tile_choice);
/* The plan rocm_launch_prefill_mfma would follow with `scratch_bytes` of scratch: the tile and the slices of K (no GPU work;
 * only the shape, dtype and pointer alignment of `args` are read). -1: shape not eligible. */
int rocm_prefill_mfma_plan(const RocmMatMulNBitsArgs* args, int tile_choice, uint64_t scratch_bytes, int* tile_rows, int* tile_cols, int* slices);
/* Y = sum over `slices` of partial[slice][M][N] (f32), in slice order, + bias. */
int rocm_launch_slice_reduce(const float* partial, int slices, int64_t m, int64_t n, const void* bias, int bias_dtype, void* y, int y_dtype,
                             rocm_stream_t stream);
int rocm_launch_prefill_mfma(const RocmMatMulNBitsArgs* args, int tile_choice, void* scratch, uint64_t scratch_bytes, rocm_stream_t stream);
/* The same tiled kernel over weights that a launch of their own has expanded to a dense [N, K] matrix of the activations' 16-bit
 * type (w16_nk, 16-byte aligned; K % 64 == 0): the tall route of bits = 2 / 8 and of weights with g_idx, whose packed forms the
 * tile loader does not read. args->b / scales / zp are not read; tiles of 128 columns at most. */
int rocm_prefill_dense16_eligible(const RocmMatMulNBitsArgs* args);
int rocm_launch_prefill_dense16(const RocmMatMulNBitsArgs* args, const void* w16_nk, int tile_choice, void* scratch, uint64_t scratch_bytes, rocm_stream_t stream);

/* accuracy_level 4. rounding: 0 = ties to even (MLAS rule), 1 = ties away (native Rust rule).
 * qa: int8 [M, kb*bs]; qscale: f32 [M, kb]; qsum: int32 [M, kb] (sum of codes per block). */
int rocm_launch_quantize_a(const void* a, int a_dtype, int64_t m, int64_t k, int block_size, int rounding,
                           int8_t* qa, float* qscale, int32_t* qsum, rocm_stream_t stream);
/* acc[m,n,b] = sum_k qa[m,k] * (q[n,k] - zp[n,b]), int32 [M, N, kb]. */
int rocm_launch_block_acc_i32(const int8_t* qa, const uint8_t* b, const uint8_t* zp,
                              int64_t m, int64_t n, int64_t k, int block_size, int32_t* acc, rocm_stream_t stream);
/* Workspace of one accuracy_level 4 call (device memory, each part 256-byte aligned):
 * qa: int8 [M, kb*bs], inside every run of 8 in the order `code_order` names (1: elements 0,2,4,6,1,3,5,7 - what the
 * kernels over the caller's weight layout want; 2: 0,4,1,5,2,6,3,7 - what the repacked stream wants);
 * aq: f32 [M, kb, 2] = (scale, sum of codes);
 * aux: for M <= 16, f32 [kb, 16, 2], the same pairs block-major; for M > 16, f32 [kb, M], the scales block-major. */
typedef struct RocmAcc4Workspace {
  int8_t* qa;
  float* aq;
  float* aux;
  int code_order;
  float* partial;          /* M > 16: room for the f32 partial sums of K slices (rocm_acc4_mfma_scratch_bytes), or NULL */
  uint64_t partial_bytes;
} RocmAcc4Workspace;
int rocm_launch_quantize_a_workspace(const void* a, int a_dtype, int64_t m, int64_t k, int block_size, int rounding,
                                     const RocmAcc4Workspace* ws, rocm_stream_t stream);
/* y = sum_b f32(acc_b) * (sa_b * sb_b) + bias, from a filled workspace. Any block size, any M (4 rows per launch). */
int rocm_launch_acc4_gemv(const RocmMatMulNBitsArgs* args, const RocmAcc4Workspace* ws, rocm_stream_t stream);
/* The same on the int8 matrix cores: M <= 16 with block size 32/64/128 (split-K; waves = 0 lets the launcher choose),
 * M > 16 with any block size >= 32 (tiled). */
int rocm_acc4_mfma_eligible(const RocmMatMulNBitsArgs* args);
/* Bytes of partial sums the tiled kernel wants when it cuts K into slices (small grids); 0 when it does not. With less
 * it uses fewer slices or none. */
uint64_t rocm_acc4_mfma_scratch_bytes(const RocmMatMulNBitsArgs* args);
int rocm_launch_acc4_mfma(const RocmMatMulNBitsArgs* args, const RocmAcc4Workspace* ws, int waves, rocm_stream_t stream);
/* One row over the repacked copy of constant weights (the copy rocm_launch_pack_decode makes); code_order 2. */
int rocm_acc4_packed_eligible(const RocmMatMulNBitsArgs* args);
/* `ws` = NULL: the kernel quantizes the row itself (rocm_acc4_packed_fuses_quantizer() must hold: f16 / bf16 row,
 * K % 8 == 0, 16-byte aligned) with the given rounding rule; otherwise codes and pairs come from the workspace. */
int rocm_acc4_packed_fuses_quantizer(const RocmMatMulNBitsArgs* args);
int rocm_launch_acc4_packed(const RocmMatMulNBitsArgs* args, const void* packed, const RocmAcc4Workspace* ws, int rounding, int waves, rocm_stream_t stream);
/* The split of K that launch takes on a chip of `compute_units` CUs (no GPU work): waves per workgroup, tile groups of 512 k per
 * wave, register sets (1 or 2). -1: the shape does not take this route. */
int rocm_acc4_packed_plan(const RocmMatMulNBitsArgs* args, int waves, int compute_units, int* waves_out, int* groups_per_wave, int* register_sets);

#ifdef __cplusplus
}
#endif
#endif
