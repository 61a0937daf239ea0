/*
 * nxmem allocator-plugin ABI (major 1, minor 1), the subset of declarations an allocator plugin
 * needs, restated for this provider. The wire layout is the one published in the reference's
 * crates/onnx-runtime-memory-abi/include/nxmem_memory_abi.h (sizes at :174-465, exports at
 * :698-718); the static assertions below pin every struct size to the figure annotated there.
 *
 * Rules a plugin must keep (same header, :72-86 and the optional-slot notes at :581-610):
 * fill struct_size on everything written; refuse an allocation whose mechanism or device is not
 * the plugin's own; optional vtable slots that are not offered are NULL, never stubs; count live
 * objects and report them from NxmemQueryUnloadReadiness; never block across a host callback.
 */
#ifndef NXMEM_ABI_H
#define NXMEM_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#define NXMEM_SIZE_CHECK(T, n) static_assert(sizeof(T) == (n), #T " layout")
#else
#define NXMEM_SIZE_CHECK(T, n) _Static_assert(sizeof(T) == (n), #T " layout")
#endif

#define NXMEM_ABI_VERSION_MAJOR 1u
#define NXMEM_ABI_VERSION_MINOR 1u
#define NXMEM_ABI_VERSION_MINOR_BASELINE 0u

#define NXMEM_CAP_ALLOCATOR (1ull << 0)
#define NXMEM_CAP_VIRTUAL_BACKING (1ull << 1)
#define NXMEM_CAP_SHARED_MAPPING (1ull << 2)
#define NXMEM_CAP_DEFERRED_RELEASE (1ull << 3)
#define NXMEM_CAP_STRUCTURED_RELEASE (1ull << 4)

enum {
  NXMEM_STATUS_OK = 0,
  NXMEM_STATUS_VERSION_MISMATCH = 1,
  NXMEM_STATUS_SHORT_STRUCT = 2,
  NXMEM_STATUS_UNSUPPORTED_CAPABILITY = 3,
  NXMEM_STATUS_INVALID_ARGUMENT = 4,
  NXMEM_STATUS_INTERNAL_ERROR = 5,
  NXMEM_STATUS_NOT_IMPLEMENTED = 6,
  NXMEM_STATUS_DEVICE_ERROR = 7,
  NXMEM_STATUS_OUT_OF_MEMORY = 8,
  NXMEM_STATUS_WRONG_DEVICE = 9,
  NXMEM_STATUS_WRONG_MECHANISM = 10,
  NXMEM_STATUS_UNKNOWN_ALLOCATION = 11,
  NXMEM_STATUS_RELEASE_QUARANTINED = 12,
  NXMEM_STATUS_CALLBACK_FAILED = 13,
  NXMEM_STATUS_BUSY = 14
};

#define NXMEM_STATUS_MESSAGE_MAX 255u

typedef struct NxmemStatus {
  uint32_t code;
  uint32_t message_len;
  uint8_t message[NXMEM_STATUS_MESSAGE_MAX + 1u];
} NxmemStatus;
NXMEM_SIZE_CHECK(NxmemStatus, 264);

enum { NXMEM_TIER_DEVICE = 0, NXMEM_TIER_HOST = 1, NXMEM_TIER_DISK = 2 };

typedef struct NxmemDeviceId {
  uint32_t tier;
  uint32_t index;
} NxmemDeviceId;
NXMEM_SIZE_CHECK(NxmemDeviceId, 8);

/* An allocation is named by the host-assigned allocation_id, not by its address. */
typedef struct NxmemAllocation {
  uint32_t struct_size;
  uint32_t reserved;
  uint64_t mechanism_id;
  uint64_t allocation_id;
  NxmemDeviceId device;
  uint8_t* ptr;
  uint64_t bytes;
  uint64_t align;
} NxmemAllocation;
NXMEM_SIZE_CHECK(NxmemAllocation, 56);

typedef struct NxmemByteRange {
  uint64_t offset;
  uint64_t bytes;
} NxmemByteRange;
NXMEM_SIZE_CHECK(NxmemByteRange, 16);

typedef struct NxmemAllocRequest {
  uint32_t struct_size;
  uint32_t reserved;
  uint64_t mechanism_id;
  uint64_t allocation_id;
  NxmemDeviceId device;
  uint64_t bytes;
  uint64_t align;
  const NxmemByteRange* committed_ranges;
  uint64_t committed_range_count;
} NxmemAllocRequest;
NXMEM_SIZE_CHECK(NxmemAllocRequest, 64);

typedef struct NxmemAllocResult {
  uint32_t struct_size;
  uint32_t reserved;
  uint8_t* ptr;
  uint64_t owned_bytes;
  uint64_t mapped_bytes;
} NxmemAllocResult;
NXMEM_SIZE_CHECK(NxmemAllocResult, 32);

typedef struct NxmemReleaseOutcome {
  uint32_t struct_size;
  uint32_t state;
  uint64_t allocation_bytes;
  uint64_t unmapped_bytes;
  uint64_t residual_owned_bytes;
  NxmemStatus failure;
} NxmemReleaseOutcome;
NXMEM_SIZE_CHECK(NxmemReleaseOutcome, 296);

typedef struct NxmemReleaseCompletion {
  uint32_t struct_size;
  uint32_t reserved;
  uint64_t ticket;
  uint64_t mechanism_id;
  uint64_t allocation_id;
  NxmemReleaseOutcome outcome;
} NxmemReleaseCompletion;
NXMEM_SIZE_CHECK(NxmemReleaseCompletion, 328);

typedef struct NxmemReclaimRequest {
  uint32_t struct_size;
  uint32_t reserved;
  uint64_t mechanism_id;
  NxmemDeviceId device;
  uint64_t bytes;
} NxmemReclaimRequest;
NXMEM_SIZE_CHECK(NxmemReclaimRequest, 32);

typedef struct NxmemUnloadReport {
  uint32_t struct_size;
  uint32_t reserved;
  uint64_t live_allocators;
  uint64_t live_allocations;
  uint64_t live_views;
  uint64_t live_capabilities;
  uint64_t queued_releases;
} NxmemUnloadReport;
NXMEM_SIZE_CHECK(NxmemUnloadReport, 48);

typedef struct NxmemHostCallbacks {
  uint32_t struct_size;
  uint32_t abi_minor;
  void* host_ctx;
  NxmemStatus (*request_reclaim)(void* host_ctx, const NxmemReclaimRequest* request, uint64_t* reclaimed_out);
  NxmemStatus (*release_completed)(void* host_ctx, const NxmemReleaseCompletion* completion);
} NxmemHostCallbacks;
NXMEM_SIZE_CHECK(NxmemHostCallbacks, 32);

typedef struct NxmemOpenRequest {
  uint32_t struct_size;
  uint32_t abi_minor;
  NxmemDeviceId device;
  uint64_t required_capability_flags;
  const NxmemHostCallbacks* callbacks;
} NxmemOpenRequest;
NXMEM_SIZE_CHECK(NxmemOpenRequest, 32);

/* Optional capability tables this provider does not offer; only their pointers appear below. */
struct NxmemVirtualBackingVtable;
struct NxmemSharedMappingVtable;

typedef struct NxmemAllocatorVtable {
  uint32_t struct_size;
  uint32_t abi_minor;
  uint64_t mechanism_id;
  NxmemDeviceId device;
  uint64_t capability_flags;
  const uint8_t* name;
  void* ctx;
  NxmemStatus (*allocate)(void* ctx, const NxmemAllocRequest* request, NxmemAllocResult* result_out);
  NxmemStatus (*deallocate)(void* ctx, const NxmemAllocation* allocation, uint64_t* unmapped_bytes_out);
  void (*retain)(void* ctx);
  void (*release)(void* ctx);
  const struct NxmemVirtualBackingVtable* virtual_backing;
  const struct NxmemSharedMappingVtable* shared_mapping;
  NxmemStatus (*enqueue_release)(void* ctx, const NxmemAllocation* allocation, uint64_t* ticket_out);
  NxmemStatus (*drain_releases)(void* ctx, uint64_t max, uint64_t* retired_out);
  NxmemStatus (*pending_release_count)(void* ctx, uint64_t* count_out);
  NxmemStatus (*release_allocation)(void* ctx, const NxmemAllocation* allocation, NxmemReleaseOutcome* outcome_out);
} NxmemAllocatorVtable;
NXMEM_SIZE_CHECK(NxmemAllocatorVtable, 128);

typedef struct NxmemAllocatorFactoryVtable {
  uint32_t struct_size;
  uint32_t abi_minor;
  const uint8_t* name;
  NxmemDeviceId device;
  uint64_t capability_flags;
  void* ctx;
  NxmemStatus (*open_allocator)(void* ctx, const NxmemOpenRequest* request, const NxmemAllocatorVtable** allocator_out);
  void (*release)(void* ctx);
} NxmemAllocatorFactoryVtable;
NXMEM_SIZE_CHECK(NxmemAllocatorFactoryVtable, 56);

typedef struct NxmemVersionRange {
  uint32_t major_min, major_max, minor_min, minor_max;
} NxmemVersionRange;

typedef struct NxmemNegotiateRequest {
  uint32_t struct_size;
  uint32_t reserved;
  NxmemVersionRange host_range;
  uint64_t host_capability_flags;
} NxmemNegotiateRequest;
NXMEM_SIZE_CHECK(NxmemNegotiateRequest, 32);

typedef struct NxmemNegotiateResponse {
  uint32_t struct_size;
  uint32_t agreed_major;
  uint32_t agreed_minor;
  uint32_t reserved;
  NxmemVersionRange plugin_range;
  uint64_t capability_flags;
} NxmemNegotiateResponse;
NXMEM_SIZE_CHECK(NxmemNegotiateResponse, 40);

/* nxmem_memory_abi.h:698-718 — all three are required exports. */
NxmemStatus NxmemNegotiate(const NxmemNegotiateRequest* request, NxmemNegotiateResponse* response_out);
NxmemStatus NxmemCreateAllocatorFactories(const NxmemAllocatorFactoryVtable** out_factories, uint64_t max_factories, uint64_t* out_count);
NxmemStatus NxmemQueryUnloadReadiness(NxmemUnloadReport* report_out);

#ifdef __cplusplus
}
#endif
#endif /* NXMEM_ABI_H */
