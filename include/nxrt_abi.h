/*
 * nxrt execution-provider plugin ABI, version 1.0, as a C header.
 *
 * The reference defines this ABI in Rust (#[repr(C)]) only; this header states the same wire
 * layout for a C/C++ plugin. Reference definitions:
 *   status      crates/onnx-runtime-ep-nxrt-abi/src/status.rs:29-48,105-119
 *   negotiation crates/onnx-runtime-ep-nxrt-abi/src/version.rs:32-137
 *   vtables     crates/onnx-runtime-ep-nxrt-abi/src/vtable.rs:55-242
 *   exports     crates/onnx-runtime-ep-nxrt-abi/src/lib.rs:54-94
 *
 * Ownership: the host owns every vtable pointer it is handed and calls that vtable's
 * release(ctx) exactly once; it never frees the vtable memory itself. Pointers passed INTO a
 * callback (dims, op-type strings) are borrowed for the duration of the call. Errors travel as
 * NxrtStatus values, returned by value; nothing unwinds across the boundary.
 */
#ifndef NXRT_ABI_H
#define NXRT_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NXRT_ABI_VERSION_MAJOR 1u
#define NXRT_ABI_VERSION_MINOR 0u

/* status.rs:29-48 */
enum {
  NXRT_OK = 0,
  NXRT_VERSION_MISMATCH = 1,
  NXRT_UNSUPPORTED_CAPABILITY = 2,
  NXRT_INVALID_ARGUMENT = 3,
  NXRT_INTERNAL_ERROR = 4,
  NXRT_NOT_IMPLEMENTED = 5,
  NXRT_DEVICE_ERROR = 6,
  NXRT_OUT_OF_MEMORY = 7
};

#define NXRT_STATUS_MESSAGE_MAX 255u

/* status.rs:105-119 — 264 bytes, no pointers, nothing to free */
typedef struct NxrtStatus {
  uint32_t code;
  uint32_t message_len;                          /* bytes of UTF-8 in message, <= 255 */
  uint8_t message[NXRT_STATUS_MESSAGE_MAX + 1u]; /* NUL-terminated */
} NxrtStatus;

/* version.rs:40-78 */
typedef struct NxrtVersionRange {
  uint32_t major_min, major_max, minor_max;
} NxrtVersionRange;

typedef struct NxrtNegotiateRequest {
  uint32_t struct_size;
  NxrtVersionRange host_range;
} NxrtNegotiateRequest;

typedef struct NxrtNegotiateResponse {
  uint32_t struct_size;
  uint32_t agreed_major, agreed_minor;
  NxrtVersionRange plugin_range;
  uint64_t capability_flags;
} NxrtNegotiateResponse;

/* version.rs:100-108 */
#define NXRT_CAP_DEVICE_ENUMERATION (1ull << 0)
#define NXRT_CAP_ALLOCATOR (1ull << 1)
#define NXRT_CAP_STREAM_SYNC (1ull << 2)
#define NXRT_CAP_EP_CONTEXT (1ull << 3)
#define NXRT_CAP_KNOWN_MASK (NXRT_CAP_DEVICE_ENUMERATION | NXRT_CAP_ALLOCATOR | NXRT_CAP_STREAM_SYNC | NXRT_CAP_EP_CONTEXT)

/* vtable.rs:32-45 — device types on the wire */
enum { NXRT_DEVICE_CPU = 0, NXRT_DEVICE_CUDA = 1, NXRT_DEVICE_ROCM = 2 };

/* onnx-runtime-ir/src/dtype.rs:9-37 — element types on the wire */
enum { NXRT_DT_FLOAT32 = 1, NXRT_DT_UINT8 = 2, NXRT_DT_INT8 = 3, NXRT_DT_INT32 = 6, NXRT_DT_FLOAT16 = 10, NXRT_DT_BFLOAT16 = 16 };

/* vtable.rs:55-66 */
typedef struct NxrtTensorDesc {
  uint32_t ndim;
  uint32_t pad_;
  const int64_t* dims; /* borrowed, ndim entries; -1 = dynamic */
  uint32_t dtype;
  uint32_t pad2_;
} NxrtTensorDesc;

/* vtable.rs:70-76 */
typedef struct NxrtNodeCapability {
  uint32_t node_index;
  uint32_t cost;
} NxrtNodeCapability;

/* vtable.rs:80-104 */
typedef struct NxrtAllocatorVtable {
  uint32_t struct_size;
  uint32_t pad_;
  void* (*alloc)(void* ctx, size_t size, size_t align);
  void (*free)(void* ctx, void* ptr);
  NxrtStatus (*copy_from_host)(void* ctx, void* dst, const uint8_t* src, size_t size);
  NxrtStatus (*copy_to_host)(void* ctx, uint8_t* dst, const void* src, size_t size);
  NxrtStatus (*sync)(void* ctx);
  void (*release)(void* ctx);
  void* ctx;
} NxrtAllocatorVtable;

/* vtable.rs:108-122 */
typedef struct NxrtKernelVtable {
  uint32_t struct_size;
  uint32_t pad_;
  NxrtStatus (*execute)(void* ctx, const void* const* inputs, uint32_t num_inputs, void** outputs, uint32_t num_outputs);
  void (*release)(void* ctx);
  void* ctx;
} NxrtKernelVtable;

/* vtable.rs:126-168 */
typedef struct NxrtEpVtable {
  uint32_t struct_size;
  uint32_t device_type;
  uint32_t device_id;
  uint32_t pad_;
  const uint8_t* name; /* NUL-terminated, lives as long as the EP */
  NxrtStatus (*get_capability)(void* ctx, const uint8_t* const* op_types, const NxrtTensorDesc* const* input_descs,
                               const uint32_t* num_inputs_per_node, uint32_t num_nodes, NxrtNodeCapability* out_claims,
                               uint32_t max_claims, uint32_t* out_num_claims);
  NxrtStatus (*compile)(void* ctx, const uint32_t* node_indices, uint32_t num_nodes, NxrtKernelVtable** out_kernel);
  NxrtStatus (*get_allocator)(void* ctx, NxrtAllocatorVtable** out_allocator);
  void (*release)(void* ctx);
  void* ctx;
} NxrtEpVtable;

/* vtable.rs:172-188 */
typedef struct NxrtEpFactoryVtable {
  uint32_t struct_size;
  uint32_t num_devices;
  const uint8_t* name;
  NxrtStatus (*create_ep)(void* ctx, uint32_t device_ordinal, NxrtEpVtable** out_ep);
  void (*release)(void* ctx);
  void* ctx;
} NxrtEpFactoryVtable;

/* lib.rs:73-94 — the two symbols every nxrt plugin exports */
NxrtStatus NxrtNegotiate(const NxrtNegotiateRequest* request, NxrtNegotiateResponse* response_out);
NxrtStatus NxrtCreateEpFactories(NxrtEpFactoryVtable** out_factories, size_t max_factories, size_t* out_num);

#ifdef __cplusplus
}
#endif
#endif /* NXRT_ABI_H */
