// The two symbols an nxrt plugin exports, and the factory / EP / allocator vtables behind them
// (crates/onnx-runtime-ep-nxrt-abi/src/lib.rs:73-94, version.rs:110-137, vtable.rs:190-398).
#include <cstring>
#include <string>

#include "provider.h"

using namespace nxrt_rocm;

namespace {

const char kEpName[] = "RocmExecutionProvider";

struct Factory {
    NxrtEpFactoryVtable vtable;
};

struct AllocatorHandle {
    NxrtAllocatorVtable vtable;
    NxrtRocmEp* ep;
};

// ---- allocator vtable (vtable.rs:80-104) ----
void* alloc_cb(void* ctx, size_t size, size_t align)
{
    auto* h = static_cast<AllocatorHandle*>(ctx);
    void* p = nullptr;
    if (!h || nxrt_rocm_ep_allocate(h->ep, size, align ? align : 1, &p).code != NXRT_OK) return nullptr;
    return p;
}
void free_cb(void* ctx, void* ptr)
{
    auto* h = static_cast<AllocatorHandle*>(ctx);
    if (h) nxrt_rocm_ep_deallocate(h->ep, ptr);
}
NxrtStatus copy_from_host_cb(void* ctx, void* dst, const uint8_t* src, size_t size)
{
    auto* h = static_cast<AllocatorHandle*>(ctx);
    if (!h) return make_status(NXRT_INVALID_ARGUMENT, "allocator: null ctx");
    return nxrt_rocm_ep_copy_from_host(h->ep, dst, src, size);
}
NxrtStatus copy_to_host_cb(void* ctx, uint8_t* dst, const void* src, size_t size)
{
    auto* h = static_cast<AllocatorHandle*>(ctx);
    if (!h) return make_status(NXRT_INVALID_ARGUMENT, "allocator: null ctx");
    return nxrt_rocm_ep_copy_to_host(h->ep, dst, src, size);
}
NxrtStatus sync_cb(void* ctx)
{
    auto* h = static_cast<AllocatorHandle*>(ctx);
    if (!h) return make_status(NXRT_INVALID_ARGUMENT, "allocator: null ctx");
    return nxrt_rocm_ep_sync(h->ep);
}
void allocator_release_cb(void* ctx)
{
    auto* h = static_cast<AllocatorHandle*>(ctx);
    if (!h) return;
    nxrt_rocm_ep_release(h->ep);                // the handle's reference: the provider outlives every allocator it handed out
    delete h;
}

// ---- EP vtable (vtable.rs:126-168) ----
NxrtStatus get_capability_cb(void* ctx, const uint8_t* const* op_types, const NxrtTensorDesc* const* input_descs, const uint32_t* num_inputs_per_node,
                             uint32_t num_nodes, NxrtNodeCapability* out_claims, uint32_t max_claims, uint32_t* out_num_claims)
{
    return fenced([&]() -> NxrtStatus {
        if (!out_num_claims) return make_status(NXRT_INVALID_ARGUMENT, "get_capability: null out_num_claims");
        *out_num_claims = 0;
        if (!ctx || (num_nodes && !op_types)) return make_status(NXRT_INVALID_ARGUMENT, "get_capability: null pointer");
        uint32_t claimed = 0;
        for (uint32_t i = 0; i < num_nodes; ++i) {
            if (!op_types[i] || std::strcmp(reinterpret_cast<const char*>(op_types[i]), "MatMulNBits") != 0) continue;
            // Claimed on arity and dtypes alone: this slot carries no attributes, so bits, block_size, weight_prepacked and
            // accuracy_level (which decides whether a g_idx input is taken) are checked when the kernel is created, and a
            // node can still be declined there with the reason.
            if (input_descs && num_inputs_per_node && input_descs[i]) {
                const uint32_t n = num_inputs_per_node[i];
                const NxrtTensorDesc* d = input_descs[i];
                if (n < 3 || n > 6) continue;
                const auto is_float = [](uint32_t dt) { return dt == NXRT_DT_FLOAT32 || dt == NXRT_DT_FLOAT16 || dt == NXRT_DT_BFLOAT16; };
                if (!is_float(d[0].dtype) || d[1].dtype != NXRT_DT_UINT8 || !is_float(d[2].dtype)) continue;
                if (n > 4 && d[4].dtype != 0 && d[4].dtype != NXRT_DT_INT32) continue;   // g_idx, when present, is int32
            }
            if (claimed < max_claims && out_claims) {
                out_claims[claimed].node_index = i;
                out_claims[claimed].cost = 1;
                ++claimed;
            }
        }
        *out_num_claims = claimed;
        return ok();
    });
}

NxrtStatus compile_cb(void*, const uint32_t*, uint32_t, NxrtKernelVtable** out_kernel)
{
    if (out_kernel) *out_kernel = nullptr;
    return make_status(NXRT_NOT_IMPLEMENTED,
                       "compile: this ABI slot carries node indices only, no attributes or shapes. Create the kernel with "
                       "nxrt_rocm_matmul_nbits_create and take its vtable with nxrt_rocm_matmul_nbits_as_vtable");
}

NxrtStatus get_allocator_cb(void* ctx, NxrtAllocatorVtable** out_allocator)
{
    return fenced([&]() -> NxrtStatus {
        if (!out_allocator) return make_status(NXRT_INVALID_ARGUMENT, "get_allocator: null out pointer");
        *out_allocator = nullptr;
        if (!ctx) return make_status(NXRT_INVALID_ARGUMENT, "get_allocator: null ctx");
        auto* h = new AllocatorHandle();
        std::memset(&h->vtable, 0, sizeof(h->vtable));
        h->ep = static_cast<NxrtRocmEp*>(ctx);
        h->ep->retain();
        h->vtable.struct_size = sizeof(NxrtAllocatorVtable);
        h->vtable.alloc = alloc_cb;
        h->vtable.free = free_cb;
        h->vtable.copy_from_host = copy_from_host_cb;
        h->vtable.copy_to_host = copy_to_host_cb;
        h->vtable.sync = sync_cb;
        h->vtable.release = allocator_release_cb;
        h->vtable.ctx = h;
        *out_allocator = &h->vtable;
        return ok();
    });
}

void ep_release_cb(void* ctx) { nxrt_rocm_ep_release(static_cast<NxrtRocmEp*>(ctx)); }

// ---- factory vtable (vtable.rs:172-188) ----
NxrtStatus create_ep_cb(void* ctx, uint32_t device_ordinal, NxrtEpVtable** out_ep)
{
    return fenced([&]() -> NxrtStatus {
        if (!ctx || !out_ep) return make_status(NXRT_INVALID_ARGUMENT, "factory_create_ep: null pointer");
        *out_ep = nullptr;
        NxrtRocmEp* ep = nullptr;
        NxrtStatus st = nxrt_rocm_ep_create(device_ordinal, nullptr, nullptr, 0, &ep);
        if (st.code != NXRT_OK) return st;
        *out_ep = &ep->vtable;
        return ok();
    });
}

void factory_release_cb(void* ctx) { delete static_cast<Factory*>(ctx); }

}  // namespace

namespace nxrt_rocm {
void init_ep_vtable(NxrtRocmEp* ep)
{
    std::memset(&ep->vtable, 0, sizeof(ep->vtable));
    ep->vtable.struct_size = sizeof(NxrtEpVtable);
    ep->vtable.device_type = NXRT_DEVICE_ROCM;
    ep->vtable.device_id = ep->device;
    ep->vtable.name = reinterpret_cast<const uint8_t*>(ep->name.c_str());
    ep->vtable.get_capability = get_capability_cb;
    ep->vtable.compile = compile_cb;
    ep->vtable.get_allocator = get_allocator_cb;
    ep->vtable.release = ep_release_cb;
    ep->vtable.ctx = ep;
}
}  // namespace nxrt_rocm

extern "C" {

NxrtRocmEp* nxrt_rocm_ep_from_vtable(const NxrtEpVtable* vtable)
{
    if (!vtable || vtable->release != ep_release_cb) return nullptr;
    return static_cast<NxrtRocmEp*>(vtable->ctx);
}

// version.rs:110-137
NxrtStatus NxrtNegotiate(const NxrtNegotiateRequest* request, NxrtNegotiateResponse* response_out)
{
    return fenced([&]() -> NxrtStatus {
        if (!request || !response_out) return make_status(NXRT_INVALID_ARGUMENT, "NxrtNegotiate: null request or response pointer");
        response_out->struct_size = sizeof(NxrtNegotiateResponse);
        response_out->plugin_range.major_min = NXRT_ABI_VERSION_MAJOR;
        response_out->plugin_range.major_max = NXRT_ABI_VERSION_MAJOR;
        response_out->plugin_range.minor_max = NXRT_ABI_VERSION_MINOR;
        const uint32_t major = NXRT_ABI_VERSION_MAJOR;
        if (major < request->host_range.major_min || major > request->host_range.major_max)
            return make_status(NXRT_VERSION_MISMATCH, "NxrtNegotiate: plugin major version " + std::to_string(major) + " outside host range [" +
                                                          std::to_string(request->host_range.major_min) + ", " + std::to_string(request->host_range.major_max) + "]");
        const uint32_t minor = NXRT_ABI_VERSION_MINOR < request->host_range.minor_max ? NXRT_ABI_VERSION_MINOR : request->host_range.minor_max;
        response_out->agreed_major = major;
        response_out->agreed_minor = minor;
        response_out->capability_flags = NXRT_CAP_DEVICE_ENUMERATION | NXRT_CAP_ALLOCATOR | NXRT_CAP_STREAM_SYNC;
        return ok();
    });
}

// vtable.rs:200-258
NxrtStatus NxrtCreateEpFactories(NxrtEpFactoryVtable** out_factories, size_t max_factories, size_t* out_num)
{
    return fenced([&]() -> NxrtStatus {
        if (max_factories == 0 || !out_factories || !out_num) {
            if (out_num) *out_num = 0;
            return make_status(NXRT_INVALID_ARGUMENT, "NxrtCreateEpFactories: null pointer or zero max_factories");
        }
        int count = 0;
        if (rocm_ffi_device_count(&count) != 0 || count < 0) count = 0;
        auto* f = new Factory();
        std::memset(&f->vtable, 0, sizeof(f->vtable));
        f->vtable.struct_size = sizeof(NxrtEpFactoryVtable);
        f->vtable.num_devices = static_cast<uint32_t>(count);
        f->vtable.name = reinterpret_cast<const uint8_t*>(kEpName);
        f->vtable.create_ep = create_ep_cb;
        f->vtable.release = factory_release_cb;
        f->vtable.ctx = f;
        out_factories[0] = &f->vtable;
        *out_num = 1;
        return ok();
    });
}

}  // extern "C"
