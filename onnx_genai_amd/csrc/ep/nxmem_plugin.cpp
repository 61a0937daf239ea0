// nxmem allocator plugin: one mechanism, "rocm-hip", plain hipMalloc/hipFree device memory per GPU.
// Required exports and slot rules: crates/onnx-runtime-memory-abi/include/nxmem_memory_abi.h:72-86,
// 556-610, 698-718. Optional capability tables (virtual backing, shared mapping, deferred release,
// structured release) are not offered: their slots are NULL and asking for them is refused.
#include <atomic>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>

#include "status.h"

using namespace nxrt_rocm;

namespace {

constexpr uint64_t kMechanismId = 0x726f636d68697031ull;   // "rocmhip1"
constexpr int kMaxDevices = 16;
const char kMechanismName[] = "rocm-hip";

std::atomic<uint64_t> g_live_allocators{0};
std::atomic<uint64_t> g_live_allocations{0};

struct DeviceAllocator {
    NxmemAllocatorVtable vtable;
    uint32_t device = 0;
    std::mutex mu;
    std::unordered_map<uint64_t, uint8_t*> by_id;   // allocations are named by the host's id
};

struct DeviceFactory {
    NxmemAllocatorFactoryVtable vtable;
    DeviceAllocator allocator;
};

DeviceFactory g_factories[kMaxDevices];
std::once_flag g_once;
int g_device_count = 0;

NxmemStatus mem_ok() { return make_mem_status(NXMEM_STATUS_OK); }

NxmemStatus allocate_cb(void* ctx, const NxmemAllocRequest* request, NxmemAllocResult* result_out)
{
    try {
        auto* a = static_cast<DeviceAllocator*>(ctx);
        if (!a || !request || !result_out) return make_mem_status(NXMEM_STATUS_INVALID_ARGUMENT, "rocm-hip: null pointer in allocate");
        if (request->struct_size < sizeof(NxmemAllocRequest)) return make_mem_status(NXMEM_STATUS_SHORT_STRUCT, "rocm-hip: allocate request is too short");
        if (request->mechanism_id != kMechanismId) return make_mem_status(NXMEM_STATUS_WRONG_MECHANISM, "rocm-hip: allocate called on another mechanism");
        if (request->device.tier != NXMEM_TIER_DEVICE || request->device.index != a->device)
            return make_mem_status(NXMEM_STATUS_WRONG_DEVICE, "rocm-hip: allocate called for another device");
        if (request->align > 256 || (request->align & (request->align - 1)) != 0)
            return make_mem_status(NXMEM_STATUS_INVALID_ARGUMENT, "rocm-hip: alignment must be a power of two <= 256");
        int err = rocm_ffi_set_device(static_cast<int>(a->device));
        void* p = nullptr;
        const uint64_t bytes = request->bytes ? request->bytes : 256;
        if (err == 0) err = rocm_ffi_malloc(&p, bytes);
        if (err != 0) return make_mem_status(err == 2 ? NXMEM_STATUS_OUT_OF_MEMORY : NXMEM_STATUS_DEVICE_ERROR, std::string("rocm-hip: hipMalloc: ") + rocm_ffi_error_string(err));
        {
            std::lock_guard<std::mutex> lock(a->mu);
            a->by_id[request->allocation_id] = static_cast<uint8_t*>(p);
        }
        std::memset(result_out, 0, sizeof(*result_out));
        result_out->struct_size = sizeof(*result_out);
        result_out->ptr = static_cast<uint8_t*>(p);
        result_out->owned_bytes = bytes;      // eager mechanism: everything owned is also mapped
        result_out->mapped_bytes = bytes;
        g_live_allocations.fetch_add(1);
        return mem_ok();
    } catch (...) {
        return make_mem_status(NXMEM_STATUS_INTERNAL_ERROR, "rocm-hip: exception in allocate (fail-closed)");
    }
}

NxmemStatus deallocate_cb(void* ctx, const NxmemAllocation* allocation, uint64_t* unmapped_bytes_out)
{
    try {
        auto* a = static_cast<DeviceAllocator*>(ctx);
        if (!a || !unmapped_bytes_out) return make_mem_status(NXMEM_STATUS_INVALID_ARGUMENT, "rocm-hip: null pointer in deallocate");
        if (!allocation) return make_mem_status(NXMEM_STATUS_INVALID_ARGUMENT, "rocm-hip: null allocation");
        if (allocation->mechanism_id != kMechanismId) return make_mem_status(NXMEM_STATUS_WRONG_MECHANISM, "rocm-hip: that allocation belongs to another mechanism");
        if (allocation->device.tier != NXMEM_TIER_DEVICE || allocation->device.index != a->device)
            return make_mem_status(NXMEM_STATUS_WRONG_DEVICE, "rocm-hip: that allocation belongs to another device");
        uint8_t* p = nullptr;
        {
            std::lock_guard<std::mutex> lock(a->mu);
            auto it = a->by_id.find(allocation->allocation_id);
            if (it == a->by_id.end() || it->second != allocation->ptr)
                return make_mem_status(NXMEM_STATUS_UNKNOWN_ALLOCATION, "rocm-hip: no live allocation with that id and address");
            p = it->second;
            a->by_id.erase(it);
        }
        int err = rocm_ffi_set_device(static_cast<int>(a->device));
        if (err == 0) err = rocm_ffi_free(p);
        if (err != 0) return make_mem_status(NXMEM_STATUS_DEVICE_ERROR, std::string("rocm-hip: hipFree: ") + rocm_ffi_error_string(err));
        *unmapped_bytes_out = allocation->bytes;
        g_live_allocations.fetch_sub(1);
        return mem_ok();
    } catch (...) {
        return make_mem_status(NXMEM_STATUS_INTERNAL_ERROR, "rocm-hip: exception in deallocate (fail-closed)");
    }
}

void retain_cb(void*) { g_live_allocators.fetch_add(1); }
void release_cb(void*)
{
    uint64_t cur = g_live_allocators.load();
    while (cur > 0 && !g_live_allocators.compare_exchange_weak(cur, cur - 1)) {}
}

NxmemStatus open_allocator_cb(void* ctx, const NxmemOpenRequest* request, const NxmemAllocatorVtable** allocator_out)
{
    auto* f = static_cast<DeviceFactory*>(ctx);
    if (!f || !request || !allocator_out) return make_mem_status(NXMEM_STATUS_INVALID_ARGUMENT, "rocm-hip: null pointer in open_allocator");
    if (request->struct_size < sizeof(NxmemOpenRequest)) return make_mem_status(NXMEM_STATUS_SHORT_STRUCT, "rocm-hip: open request is too short");
    if ((request->required_capability_flags & ~static_cast<uint64_t>(NXMEM_CAP_ALLOCATOR)) != 0)
        return make_mem_status(NXMEM_STATUS_UNSUPPORTED_CAPABILITY, "rocm-hip: this mechanism offers plain allocation only");
    if (request->device.tier != NXMEM_TIER_DEVICE || request->device.index != f->allocator.device)
        return make_mem_status(NXMEM_STATUS_WRONG_DEVICE, "rocm-hip: this factory serves another device");
    g_live_allocators.fetch_add(1);
    *allocator_out = &f->allocator.vtable;
    return mem_ok();
}

void factory_release_cb(void*) {}

void init_factories()
{
    int count = 0;
    if (rocm_ffi_device_count(&count) != 0 || count < 0) count = 0;
    if (count > kMaxDevices) count = kMaxDevices;
    g_device_count = count;
    for (int d = 0; d < count; ++d) {
        DeviceFactory& f = g_factories[d];
        std::memset(&f.vtable, 0, sizeof(f.vtable));
        std::memset(&f.allocator.vtable, 0, sizeof(f.allocator.vtable));
        f.allocator.device = static_cast<uint32_t>(d);
        NxmemAllocatorVtable& a = f.allocator.vtable;
        a.struct_size = sizeof(NxmemAllocatorVtable);
        a.abi_minor = NXMEM_ABI_VERSION_MINOR_BASELINE;
        a.mechanism_id = kMechanismId;
        a.device.tier = NXMEM_TIER_DEVICE;
        a.device.index = static_cast<uint32_t>(d);
        a.capability_flags = NXMEM_CAP_ALLOCATOR;
        a.name = reinterpret_cast<const uint8_t*>(kMechanismName);
        a.ctx = &f.allocator;
        a.allocate = allocate_cb;
        a.deallocate = deallocate_cb;
        a.retain = retain_cb;
        a.release = release_cb;
        f.vtable.struct_size = sizeof(NxmemAllocatorFactoryVtable);
        f.vtable.abi_minor = NXMEM_ABI_VERSION_MINOR_BASELINE;
        f.vtable.name = reinterpret_cast<const uint8_t*>(kMechanismName);
        f.vtable.device = a.device;
        f.vtable.capability_flags = NXMEM_CAP_ALLOCATOR;
        f.vtable.ctx = &f;
        f.vtable.open_allocator = open_allocator_cb;
        f.vtable.release = factory_release_cb;
    }
}

}  // namespace

extern "C" {

NxmemStatus NxmemNegotiate(const NxmemNegotiateRequest* request, NxmemNegotiateResponse* response_out)
{
    if (!request || !response_out) return make_mem_status(NXMEM_STATUS_INVALID_ARGUMENT, "rocm-hip: null pointer in negotiate");
    if (request->struct_size < sizeof(NxmemNegotiateRequest)) return make_mem_status(NXMEM_STATUS_SHORT_STRUCT, "rocm-hip: the host's negotiate request is too short");
    if (request->host_range.major_min > NXMEM_ABI_VERSION_MAJOR || request->host_range.major_max < NXMEM_ABI_VERSION_MAJOR)
        return make_mem_status(NXMEM_STATUS_VERSION_MISMATCH, "rocm-hip: this plugin implements nxmem major 1");
    if (request->host_range.minor_min > NXMEM_ABI_VERSION_MINOR_BASELINE)
        return make_mem_status(NXMEM_STATUS_VERSION_MISMATCH, "rocm-hip: this plugin implements the nxmem baseline minor only");
    std::memset(response_out, 0, sizeof(*response_out));
    response_out->struct_size = sizeof(*response_out);
    response_out->agreed_major = NXMEM_ABI_VERSION_MAJOR;
    response_out->agreed_minor = NXMEM_ABI_VERSION_MINOR_BASELINE;
    response_out->plugin_range.major_min = NXMEM_ABI_VERSION_MAJOR;
    response_out->plugin_range.major_max = NXMEM_ABI_VERSION_MAJOR;
    response_out->plugin_range.minor_min = NXMEM_ABI_VERSION_MINOR_BASELINE;
    response_out->plugin_range.minor_max = NXMEM_ABI_VERSION_MINOR_BASELINE;
    response_out->capability_flags = request->host_capability_flags & static_cast<uint64_t>(NXMEM_CAP_ALLOCATOR);
    if (response_out->capability_flags == 0) return make_mem_status(NXMEM_STATUS_UNSUPPORTED_CAPABILITY, "rocm-hip: the host did not offer plain allocation");
    return mem_ok();
}

NxmemStatus NxmemCreateAllocatorFactories(const NxmemAllocatorFactoryVtable** out_factories, uint64_t max_factories, uint64_t* out_count)
{
    if (!out_factories || !out_count) return make_mem_status(NXMEM_STATUS_INVALID_ARGUMENT, "rocm-hip: null pointer in create_allocator_factories");
    if (max_factories < 1) return make_mem_status(NXMEM_STATUS_INVALID_ARGUMENT, "rocm-hip: no room for even one factory");
    std::call_once(g_once, init_factories);
    uint64_t n = 0;
    for (int d = 0; d < g_device_count && n < max_factories; ++d) out_factories[n++] = &g_factories[d].vtable;
    *out_count = n;
    return mem_ok();
}

NxmemStatus NxmemQueryUnloadReadiness(NxmemUnloadReport* report_out)
{
    if (!report_out) return make_mem_status(NXMEM_STATUS_INVALID_ARGUMENT, "rocm-hip: null report pointer");
    std::memset(report_out, 0, sizeof(*report_out));
    report_out->struct_size = sizeof(*report_out);
    report_out->live_allocators = g_live_allocators.load();
    report_out->live_allocations = g_live_allocations.load();
    return mem_ok();
}

}  // extern "C"
