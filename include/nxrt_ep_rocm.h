/*
 * libnxrt_ep_rocm.so — MI355X (gfx950) execution provider for com.microsoft::MatMulNBits, bits=4.
 *
 * Three groups of C entry points:
 *   1. the nxrt plugin exports (nxrt_abi.h) and the nxmem allocator exports (nxmem_abi.h);
 *   2. a C mirror of the reference's ExecutionProvider / KernelFactory / Kernel traits for this one
 *      operator, because NxrtKernelVtable.execute (vtable.rs:108-122) carries raw pointers only —
 *      no shapes, dtypes or attributes — and the reference's own nxrt wrapper still leaves
 *      get_capability / compile / get_allocator unwired (vtable.rs:355-398);
 *   3. entry points for the pieces the parity contract names one by one (dequantized weights,
 *      activation codes, int32 block accumulators) and for timing on the provider's stream.
 *
 * Every pointer named "device" is device memory obtained from nxrt_rocm_ep_allocate (or any HIP
 * allocation on the provider's GPU). Nothing here takes or returns a torch / C++ type. All calls on
 * one provider are issued on that provider's single HIP stream, in call order; host-visible results
 * require nxrt_rocm_ep_sync or a copy_to_host (which synchronises).
 */
#ifndef NXRT_EP_ROCM_H
#define NXRT_EP_ROCM_H

#include "nxmem_abi.h"
#include "nxrt_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct NxrtRocmEp NxrtRocmEp;                     /* one provider = one GPU + one stream */
typedef struct NxrtRocmMatMulNBits NxrtRocmMatMulNBits;   /* one kernel = one MatMulNBits node */

/* ---- ExecutionProvider (crates/onnx-runtime-ep-api/src/provider.rs:708-1600) ------------------ */

/* initialize(&EpConfig) — provider.rs:93 (string map). keys/values: n_config NUL-terminated pairs.
 * Known keys: "acc4_rounding" = "mlas" (ties to even, default) | "native" (ties away) | "auto" (native below
 *             "acc4_native_below" rows, else mlas: the CPU provider's route, matmul_nbits.rs:640-660);
 *             "prepack" = "1" (default: constant weights are copied once into the decode kernels' streaming order) | "0";
 *             "dense_gemm_min_rows" = rows from which a 16-bit call expands the weights to a dense [N, K] matrix and runs
 *             the library GEMM (hipBLASLt) instead of this provider's own tiled kernel: opt-in, default "0" = never (256 once
 *             "dense_weights" = "resident" is chosen; the CUDA provider's dequantize + cuBLASLt route,
 *             onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:6176-6222);
 *             "dense_gemm_max_mb" = largest dense copy of one weight (default 1024, as matmul_nbits.rs:6212);
 *             "dense_weights" = "transient" (default: one buffer per provider, refilled by every such call) |
 *             "resident" (a constant weight keeps its dense copy: 2 bytes per weight of HBM for a call that is the
 *             GEMM alone);
 *             "rmsnorm_in_kernel_max_cols" = widest launch (columns; both projections of a gate/up node together) whose
 *             decode kernel applies an RMS-normalization prologue itself at up to four rows; wider nodes and "0" normalize
 *             in a launch of their own (default 8192: every workgroup repeats the row's normalization, which pays only
 *             while there are few of them);
 *             "decode_waves", "decode_col_groups", "prefill_tile" = launch overrides (tests, tuning).
 * The same settings are read from NXRT_ROCM_RMSNORM_IN_KERNEL_MAX_COLS, NXRT_ROCM_ACC4_ROUNDING, NXRT_SQNBIT_DECODE_MIN, NXRT_ROCM_PREPACK,
 * NXRT_ROCM_DENSE_GEMM_MIN_ROWS, NXRT_ROCM_DENSE_GEMM_MAX_MB, NXRT_ROCM_DENSE_WEIGHTS, NXRT_ROCM_DECODE_WAVES,
 * NXRT_ROCM_DECODE_COL_GROUPS, NXRT_ROCM_PREFILL_TILE when the map does not give them. */
NxrtStatus nxrt_rocm_ep_create(uint32_t device_ordinal, const char* const* config_keys,
                               const char* const* config_values, uint32_t n_config, NxrtRocmEp** out_ep);
/* shutdown + drop. Frees the stream and every buffer the provider still owns. Kernels and allocator vtables made from the
 * provider each hold a reference to it: the host may release them and the provider in any order, and the provider's
 * resources go with the last of them. */
void nxrt_rocm_ep_release(NxrtRocmEp* ep);
/* name() / device_type() / device_id() / memory_vendor_id() — provider.rs:708-731. */
const char* nxrt_rocm_ep_name(const NxrtRocmEp* ep);                   /* "RocmExecutionProvider" */
uint32_t nxrt_rocm_ep_device_type(const NxrtRocmEp* ep);               /* NXRT_DEVICE_ROCM */
uint32_t nxrt_rocm_ep_device_id(const NxrtRocmEp* ep);
uint32_t nxrt_rocm_ep_memory_vendor_id(const NxrtRocmEp* ep);          /* 0x1002 */
/* Architecture string ("gfx950..."), compute units, bytes of device memory. */
NxrtStatus nxrt_rocm_ep_device_info(const NxrtRocmEp* ep, char* arch, size_t arch_len, uint32_t* compute_units, uint64_t* total_memory);
/* allocate(size, align) / deallocate — provider.rs (DeviceBuffer); align <= 256 is always met. */
NxrtStatus nxrt_rocm_ep_allocate(NxrtRocmEp* ep, size_t size, size_t align, void** out_device);
NxrtStatus nxrt_rocm_ep_deallocate(NxrtRocmEp* ep, void* device);
/* copy_from_host / copy_to_host (provider.rs:1434,1502), copy (device to device), sync. */
NxrtStatus nxrt_rocm_ep_copy_from_host(NxrtRocmEp* ep, void* dst_device, const void* src_host, size_t bytes);
NxrtStatus nxrt_rocm_ep_copy_to_host(NxrtRocmEp* ep, void* dst_host, const void* src_device, size_t bytes);
NxrtStatus nxrt_rocm_ep_copy(NxrtRocmEp* ep, void* dst_device, const void* src_device, size_t bytes);
NxrtStatus nxrt_rocm_ep_sync(NxrtRocmEp* ep);
/* A benchmark's yardstick, not part of the reference's interface: enqueues a kernel that reads `bytes` of device memory (16-byte
 * loads, four in flight per lane, one workgroup per 16 KiB) and keeps nothing. Its time is the least any kernel can spend
 * pulling that many bytes from HBM; bench.py --read-floor reports it beside the decode kernels' times. */
NxrtStatus nxrt_rocm_ep_read_probe(NxrtRocmEp* ep, const void* src_device, size_t bytes);
/* Diagnostic for benchmarks (no counterpart in the reference): bytes per clock one CU's LDS moves with `waves` waves (1..16)
 * of a workgroup repeating 16-byte accesses. mode 0: reads; 1: writes; 2: global memory straight into LDS; 3: half the waves
 * read while the others write. Synchronous; allocates and frees its own small buffers. */
NxrtStatus nxrt_rocm_ep_lds_probe(NxrtRocmEp* ep, uint32_t mode, uint32_t waves, uint32_t iters, double* bytes_per_clock);
/* The nxrt EP vtable whose ctx is this provider (what NxrtEpFactoryVtable.create_ep hands out);
 * the inverse recovers the provider from a vtable obtained through the plugin exports. */
NxrtRocmEp* nxrt_rocm_ep_from_vtable(const NxrtEpVtable* vtable);

/* ---- KernelFactory + Kernel (registry.rs:39-45, kernel.rs:548-706) ----------------------------- */

/* Node attributes of MatMulNBits. `present` has bit i set when attribute i was on the node:
 * 0=K 1=N 2=bits 3=block_size 4=accuracy_level 5=weight_prepacked
 * (onnx-runtime-ep-cpu/src/kernels/matmul_nbits.rs:1410-1481; bits 2, 4 (default) or 8 as there - 4 is the tuned path, and the
 * only one with accuracy_level = 4; weight_prepacked must be 0), and 6=folded_bias: the marker an optimizer pass sets
 * when it folds a standalone Add into the bias input (the CUDA provider's `_cuda_matmul_nbits_folded_bias`,
 * onnx-runtime-ep-cuda/src/optimizer.rs:35, kernels/matmul_nbits.rs:1189-1212). With folded_bias = 1 and a 16-bit
 * output the result is round(round(acc) + bias), bit for bit what the two nodes gave; otherwise round(acc + bias).
 * 7=gate_up_swiglu, 8=decomposed_silu: the CUDA provider's fused gate/up node (`_cuda_gate_up_swiglu`, `_cuda_decomposed_silu`,
 * onnx-runtime-ep-cuda/src/optimizer.rs:14, 36-46; kernels/matmul_nbits.rs:9017-9130). With gate_up_swiglu = 1 the inputs are
 * [x, W_gate, scales_gate, W_up, scales_up, (gamma: must be absent), (zp_gate, zp_up: both or neither)], x and Y Float16 or
 * BFloat16, and Y = round16(silu(round16(x W_gate^T)) * round16(x W_up^T)) - bit for bit what the two projections followed by
 * the 16-bit silu-and-multiply give (kernels/matmul_nbits.rs:4207-4233, 4375-4386). workspace_requirement then sizes the
 * two 16-bit [M, N] intermediates.
 * 9=rmsnorm_prologue, 10=rmsnorm_epsilon (default 1e-5): the CUDA provider's `_cuda_matmul_nbits_rmsnorm_prologue` / `_epsilon`
 * (optimizer.rs:48-60). The activations (Float16 or BFloat16, K % 128 == 0) are RMS-normalized before the product,
 * x' = round16((x / sqrt(mean(x^2) + epsilon)) * gamma), with gamma [K] (Float32 or the activations' dtype) at input 6, or
 * input 5 of the fused gate/up node - the arithmetic and summation order of kernels/matmul_nbits.rs:4125-4205.
 * struct_size tells which fields the caller's struct has: fields past its end are read as 0. */
typedef struct NxrtRocmMatMulNBitsAttrs {
  uint32_t struct_size;
  uint32_t present;
  int64_t K, N, bits, block_size, accuracy_level, weight_prepacked;
  int64_t folded_bias;
  int64_t gate_up_swiglu, decomposed_silu;
  int64_t rmsnorm_prologue;
  double rmsnorm_epsilon;
} NxrtRocmMatMulNBitsAttrs;

/* C layout of TensorView / TensorMut (crates/onnx-runtime-ep-api/src/tensor.rs:132-143, 241).
 * data == NULL marks an absent optional input (tensor.rs:173-192). strides are in elements;
 * NULL means contiguous row-major. */
typedef struct NxrtRocmTensorView {
  void* data;
  uint32_t dtype;        /* NXRT_DT_* */
  uint32_t ndim;
  const uint64_t* shape;
  const int64_t* strides;
  uint64_t byte_offset;
  uint32_t device_type;  /* NXRT_DEVICE_* */
  uint32_t device_index;
} NxrtRocmTensorView;

/* kernel.rs:508-524 */
typedef struct NxrtRocmWorkspaceRequirement {
  uint64_t bytes;
  uint64_t alignment;
} NxrtRocmWorkspaceRequirement;

/* supports_op(node, opset, shapes, dtypes, layouts) -> KernelMatch (kernel.rs:118-130).
 * Returns 1 when the provider takes the node; otherwise 0 with an actionable reason. */
int nxrt_rocm_ep_supports_matmul_nbits(const NxrtRocmEp* ep, const NxrtRocmMatMulNBitsAttrs* attrs,
                                       const NxrtTensorDesc* inputs, uint32_t n_inputs, char* reason, size_t reason_len);

/* get_kernel -> KernelFactory::create (matmul_nbits.rs:1410-1481): attribute checks, same messages. */
NxrtStatus nxrt_rocm_matmul_nbits_create(NxrtRocmEp* ep, const NxrtRocmMatMulNBitsAttrs* attrs,
                                         const NxrtTensorDesc* input_shapes, uint32_t n_inputs,
                                         NxrtRocmMatMulNBits** out_kernel);
/* Kernel::set_constant_inputs (kernel.rs:548-, matmul_nbits.rs:1483-1488). */
void nxrt_rocm_matmul_nbits_set_constant_inputs(NxrtRocmMatMulNBits* kernel, const uint8_t* is_constant, uint32_t n);
/* Kernel::workspace_requirement: scratch for these input shapes (accuracy_level 4 activation codes). */
NxrtStatus nxrt_rocm_matmul_nbits_workspace_requirement(const NxrtRocmMatMulNBits* kernel, const NxrtTensorDesc* inputs,
                                                        uint32_t n_inputs, NxrtRocmWorkspaceRequirement* out);
/* Kernel::execute / execute_with_workspace (matmul_nbits.rs:1490-1600, 2320-2330).
 * inputs: A, B, scales, [zero_points], [g_idx], [bias]; outputs: Y. workspace may be NULL: the
 * kernel then keeps its own scratch, grown on demand (an allocation inside the call). B is [N, kb, block_size * bits / 8],
 * zero_points [N, ceil(kb * bits / 8)]; g_idx (Int32 [K] or [kb * block_size], accuracy_level 0 only) is range-checked on first
 * use (matmul_nbits.rs:3515-3521). bias has N elements in any shape ([N], [1, N], [1, 1, N]: broadcast over the rows), or
 * rows * N elements: a per-token residual folded into the bias slot, row stride N
 * (onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:7728-7735, 7891-7897). A required tensor with a NULL data pointer is
 * refused with a status, never launched. Fused nodes (gate_up_swiglu, rmsnorm_prologue) take their own input lists, see the attributes. */
NxrtStatus nxrt_rocm_matmul_nbits_execute(NxrtRocmMatMulNBits* kernel, const NxrtRocmTensorView* inputs, uint32_t n_inputs,
                                          NxrtRocmTensorView* outputs, uint32_t n_outputs,
                                          void* workspace_device, uint64_t workspace_bytes);
/* execute for callers that cannot allocate: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc. It has no counterpart in the reference. Same inputs, outputs, validation and results as
 * nxrt_rocm_matmul_nbits_execute on a plain MatMulNBits node (fused gate/up and RMS-normalization nodes are refused), but the
 * call allocates and frees nothing and calls no library routine that might: whatever scratch its kernels need (activation
 * codes and scales of accuracy_level 4; partial sums of a tall call that cuts K into slices) lives in a static device array
 * of NXRT_ROCM_STATIC_SCRATCH_BYTES that is part of the library's code object - one copy per GPU, held until the process
 * ends, its address resolved once when the provider is created. Consequences:
 *   - a call whose scratch does not fit is refused with INVALID_ARGUMENT and the sizes (accuracy_level 4 needs about
 *     rows * K * (1 + 12 / block_size) bytes: at K = 8192, block 64, up to ~860 rows); optional scratch (K slices) shrinks to fit;
 *   - nothing is set up on the fly: constant weights that have no repacked copy yet are streamed in the caller's layout, the
 *     library GEMM route is not taken, a g_idx tensor must have been range-checked by an earlier execute;
 *   - every call on one GPU shares that GPU's array, which keeps the last call's contents (the kernels overwrite all they
 *     read). Calls through one provider are ordered by its stream. Calls through different providers on the same GPU are
 *     chained on the GPU: each call records an event behind its launches, and a call on another stream waits for it
 *     (hipStreamWaitEvent) before its own - they run one after the other, in the order in which the host made them. The
 *     exception is a call made while its provider has a graph capture open: it neither waits nor records (an event from
 *     outside a capture cannot be waited for inside one), so graphs recorded through several providers of one GPU must not
 *     be replayed at the same time; the host orders them. */
#define NXRT_ROCM_STATIC_SCRATCH_BYTES (8u << 20)
NxrtStatus nxrt_rocm_matmul_nbits_execute_static(NxrtRocmMatMulNBits* kernel, const NxrtRocmTensorView* inputs, uint32_t n_inputs,
                                                 NxrtRocmTensorView* outputs, uint32_t n_outputs);
/* Kernel::estimated_flops (matmul_nbits.rs:2338): 2*M*N*K, 0 when M is not known from the shapes. */
uint64_t nxrt_rocm_matmul_nbits_estimated_flops(const NxrtRocmMatMulNBits* kernel);
/* record_kernel_variant (kernel.rs:361): which kernel served the last execute. */
const char* nxrt_rocm_matmul_nbits_last_variant(const NxrtRocmMatMulNBits* kernel);
/* record_kernel_metrics (onnx-runtime-ep-api/src/kernel.rs:243-267, called at matmul_nbits.rs:1588-1597): what the last plain
 * execute moved and computed by the reference's count - bytes = the bytes of every present input tensor + the output's;
 * flops = 2*M*N*K, + M*N with a bias. Zero before the first call. */
void nxrt_rocm_matmul_nbits_last_metrics(const NxrtRocmMatMulNBits* kernel, uint64_t* flops, uint64_t* bytes);
void nxrt_rocm_matmul_nbits_release(NxrtRocmMatMulNBits* kernel);
/* The same kernel behind the nxrt kernel vtable (raw pointers only: the shapes are those given at
 * create time, M taken from input_shapes[0]). The host calls release(ctx) once. */
NxrtStatus nxrt_rocm_matmul_nbits_as_vtable(NxrtRocmMatMulNBits* kernel, NxrtKernelVtable** out_vtable);

/* ---- pieces of the operator the parity contract checks one by one ------------------------------ */

/* w[n,k] = (q - zp) * scale as f32 [N, K] (matmul_nbits.rs:1360-1363, 3502-3661; the CUDA sibling's
 * matmul_nbits_dequant_f32, ep-cuda matmul_nbits.rs:414-455). scales dtype: f32 / f16 / bf16. */
NxrtStatus nxrt_rocm_matmul_nbits_dequantize(NxrtRocmEp* ep, const void* b_device, const void* scales_device, uint32_t scale_dtype,
                                             const void* zero_points_device, uint64_t n, uint64_t k, uint32_t block_size,
                                             float* out_nk_device);
/* The same at bits = 2, 4 or 8 (NBitsLayout, matmul_nbits.rs:1276-1321): b is [N, kb, block_size * bits / 8], zero points
 * [N, ceil(kb * bits / 8)], default zero point 1 << (bits - 1). */
NxrtStatus nxrt_rocm_matmul_nbits_dequantize_bits(NxrtRocmEp* ep, const void* b_device, const void* scales_device, uint32_t scale_dtype,
                                                  const void* zero_points_device, uint64_t n, uint64_t k, uint32_t block_size, uint32_t bits,
                                                  float* out_nk_device);
/* accuracy_level=4 activation quantizer (simd_quant.rs:131-143 / sqnbitgemm_kernel_avx512.cpp:349-426).
 * rounding: 0 = ties to even (MLAS), 1 = ties away from zero (native). qa: int8 [M, kb*bs];
 * qscale: f32 [M, kb]. */
NxrtStatus nxrt_rocm_matmul_nbits_quantize_a(NxrtRocmEp* ep, const void* a_device, uint32_t a_dtype, uint64_t m, uint64_t k,
                                             uint32_t block_size, uint32_t rounding, int8_t* qa_device, float* qscale_device);
/* acc[m,n,b] = sum_{k in block b} qa[m,k] * (q[n,k] - zp[n,b]), int32 [M, N, kb]
 * (matmul_nbits.rs:3360-3412 + 9159-9177; qnbitgemm.cpp:727-893). */
NxrtStatus nxrt_rocm_matmul_nbits_block_acc(NxrtRocmEp* ep, const int8_t* qa_device, const void* b_device,
                                            const void* zero_points_device, uint64_t m, uint64_t n, uint64_t k,
                                            uint32_t block_size, int32_t* acc_device);

/* The same integers as the production kernels hold them: with a probe buffer set (int32 [M, N, kb] device memory, NULL
 * clears it), every later accuracy_level=4 execute of this kernel that runs on the int8 matrix cores also stores each
 * block accumulator at the moment it is scaled into the f32 result (matmul_nbits.rs:9159-9177: `acc` of `int8_row`).
 * The launch is the same kernel with the store compiled in; a call the dot-product catch-all would serve is refused. */
NxrtStatus nxrt_rocm_matmul_nbits_set_block_acc_probe(NxrtRocmMatMulNBits* kernel, int32_t* acc_device, uint64_t capacity_elements);
/* Device buffers the kernel object has replaced (outgrown scratch, a repacked or dense copy of weights that changed) and
 * keeps until it is released, because a HIP graph recorded earlier may still replay through them. */
uint64_t nxrt_rocm_matmul_nbits_retired_buffers(const NxrtRocmMatMulNBits* kernel);

/* ---- timing on the provider's stream (HIP events) ---------------------------------------------- */

typedef struct NxrtRocmEvent NxrtRocmEvent;
NxrtStatus nxrt_rocm_ep_event_create(NxrtRocmEp* ep, NxrtRocmEvent** out_event);
NxrtStatus nxrt_rocm_ep_event_record(NxrtRocmEp* ep, NxrtRocmEvent* event);
NxrtStatus nxrt_rocm_ep_event_elapsed_ms(NxrtRocmEp* ep, NxrtRocmEvent* start, NxrtRocmEvent* stop, float* out_ms);
void nxrt_rocm_ep_event_destroy(NxrtRocmEp* ep, NxrtRocmEvent* event);

/* ---- graph capture (Kernel::capture_support in kernel.rs; the CUDA sibling's capture-safe decode path,
 * ep-cuda matmul_nbits.rs:11136-11162) ---------------------------------------------------------
 * Between begin and end, execute calls on this provider are recorded instead of run. Only calls that
 * allocate nothing may be recorded: accuracy_level 0 always, accuracy_level 4 with a caller workspace.
 * A recorded graph replays the same launches on the same device pointers. */
typedef struct NxrtRocmGraph NxrtRocmGraph;
NxrtStatus nxrt_rocm_ep_capture_begin(NxrtRocmEp* ep);
NxrtStatus nxrt_rocm_ep_capture_end(NxrtRocmEp* ep, NxrtRocmGraph** out_graph, uint64_t* out_num_nodes);
NxrtStatus nxrt_rocm_ep_graph_replay(NxrtRocmEp* ep, NxrtRocmGraph* graph);
void nxrt_rocm_ep_graph_release(NxrtRocmEp* ep, NxrtRocmGraph* graph);

/* Counters a harness reads to prove the provider, not a fallback, did the work
 * (the role of nxrt_ep_compiled_node_count in ep-cuda-plugin/src/lib.rs:345-372). */
uint64_t nxrt_rocm_ep_kernel_launch_count(const NxrtRocmEp* ep);
uint64_t nxrt_rocm_live_provider_count(void);
/* Device allocations (hipMalloc calls) the library has made in this process so far. */
uint64_t nxrt_rocm_device_allocation_count(void);

#ifdef __cplusplus
}
#endif
#endif /* NXRT_EP_ROCM_H */
