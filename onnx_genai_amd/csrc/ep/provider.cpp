// ExecutionProvider side of the C ABI: lifecycle, device memory, copies, events.
// Mirrors crates/onnx-runtime-ep-api/src/provider.rs:708-1600 for one ROCm device.
#include "provider.h"

#include <cstdlib>

namespace nxrt_rocm {
std::atomic<uint64_t> g_live_providers{0};
}

using namespace nxrt_rocm;

NxrtRocmEp::NxrtRocmEp() { g_live_providers.fetch_add(1); }

NxrtRocmEp::~NxrtRocmEp()
{
    if (rocm_ffi_set_device(static_cast<int>(device)) == 0) {
        if (stream) rocm_ffi_stream_sync(stream);
        for (auto& kv : live) rocm_ffi_free(kv.first);
        if (dense_scratch) rocm_ffi_free(dense_scratch);
        for (void* old : dense_retired) rocm_ffi_free(old);
        if (dense) rocm_dense_gemm_destroy(dense);
        if (stream) rocm_ffi_stream_destroy(stream);
    }
    g_live_providers.fetch_sub(1);
}

NxrtStatus NxrtRocmEp::bind() const { return hip_status(rocm_ffi_set_device(static_cast<int>(device)), "hipSetDevice"); }

// The dense route (expand the weights to 16 bits, then the library GEMM) is opt-in: by default every call runs on this
// provider's own kernels. `dense_gemm_min_rows` > 0 turns it on from that many rows; `dense_weights = resident` turns it
// on from kDenseGemmMinRowsResident rows unless `dense_gemm_min_rows` says otherwise. Measured at 8B / 7B MLP shapes
// against the tiled kernel: refilling the dense buffer on every call pays from about a thousand rows; a resident copy
// (no expansion per call) from a few hundred.
constexpr int kDenseGemmMinRowsResident = 256;

static int parse_int(const std::string& v, int fallback)
{
    char* end = nullptr;
    const long x = std::strtol(v.c_str(), &end, 10);
    return (end && *end == 0 && !v.empty()) ? static_cast<int>(x) : fallback;
}

extern "C" {

NxrtStatus nxrt_rocm_ep_create(uint32_t device_ordinal, const char* const* keys, const char* const* values, uint32_t n_config, NxrtRocmEp** out_ep)
{
    return fenced([&]() -> NxrtStatus {
        if (!out_ep) return make_status(NXRT_INVALID_ARGUMENT, "nxrt_rocm_ep_create: null out_ep");
        *out_ep = nullptr;
        int count = 0;
        int err = rocm_ffi_device_count(&count);
        if (err != 0 || count <= 0)
            return make_status(NXRT_DEVICE_ERROR, "RocmExecutionProvider: no HIP device is visible. Why: hipGetDeviceCount found none. "
                                                  "How to fix: run on a host with an AMD GPU and the ROCm driver loaded");
        if (device_ordinal >= static_cast<uint32_t>(count))
            return make_status(NXRT_INVALID_ARGUMENT, "RocmExecutionProvider: device ordinal " + std::to_string(device_ordinal) + " out of range (" + std::to_string(count) + " visible)");
        auto* ep = new NxrtRocmEp();
        ep->device = device_ordinal;
        for (uint32_t i = 0; i < n_config; ++i)
            if (keys && values && keys[i] && values[i]) ep->config[keys[i]] = values[i];
        if (const char* env = std::getenv("NXRT_ROCM_ACC4_ROUNDING")) ep->config.emplace("acc4_rounding", env);
        if (const char* env = std::getenv("NXRT_ROCM_DECODE_WAVES")) ep->config.emplace("decode_waves", env);
        if (const char* env = std::getenv("NXRT_ROCM_DECODE_COL_GROUPS")) ep->config.emplace("decode_col_groups", env);
        if (const char* env = std::getenv("NXRT_ROCM_PREPACK")) ep->config.emplace("prepack", env);
        if (const char* env = std::getenv("NXRT_ROCM_PREFILL_TILE")) ep->config.emplace("prefill_tile", env);
        if (const char* env = std::getenv("NXRT_ROCM_DENSE_GEMM_MIN_ROWS")) ep->config.emplace("dense_gemm_min_rows", env);
        if (const char* env = std::getenv("NXRT_ROCM_DENSE_GEMM_MAX_MB")) ep->config.emplace("dense_gemm_max_mb", env);
        if (const char* env = std::getenv("NXRT_ROCM_DENSE_WEIGHTS")) ep->config.emplace("dense_weights", env);
        auto it = ep->config.find("acc4_rounding");
        if (it != ep->config.end()) {
            if (it->second == "native") ep->acc4_rounding = 1;
            else if (it->second == "mlas") ep->acc4_rounding = 0;
            else if (it->second == "auto") ep->acc4_rounding = 2;
            else {
                delete ep;
                return make_status(NXRT_INVALID_ARGUMENT, "RocmExecutionProvider: acc4_rounding must be 'mlas', 'native' or 'auto'");
            }
        }
        // 'auto' follows the CPU provider's route (matmul_nbits.rs:640-660): fewer rows than the crossover take the native
        // rule, the rest the MLAS rule. The crossover is host-dependent there (twice the decode threads), so it is a
        // setting here, read from the same environment variable when the config does not give it.
        if (const char* env = std::getenv("NXRT_SQNBIT_DECODE_MIN")) ep->config.emplace("acc4_native_below", env);
        if ((it = ep->config.find("acc4_native_below")) != ep->config.end()) ep->acc4_native_below = parse_int(it->second, 0);
        if ((it = ep->config.find("decode_waves")) != ep->config.end()) ep->decode_waves = parse_int(it->second, 0);
        if ((it = ep->config.find("decode_col_groups")) != ep->config.end()) ep->decode_col_groups = parse_int(it->second, 0);
        if ((it = ep->config.find("prepack")) != ep->config.end()) ep->prepack = parse_int(it->second, 1);
        if ((it = ep->config.find("prefill_tile")) != ep->config.end()) ep->prefill_tile = parse_int(it->second, 0);
        if (const char* env = std::getenv("NXRT_ROCM_RMSNORM_IN_KERNEL_MAX_COLS")) ep->config.emplace("rmsnorm_in_kernel_max_cols", env);
        if ((it = ep->config.find("rmsnorm_in_kernel_max_cols")) != ep->config.end()) ep->rmsnorm_in_kernel_max_cols = parse_int(it->second, 8192);
        if ((it = ep->config.find("dense_gemm_max_mb")) != ep->config.end()) ep->dense_gemm_max_bytes = static_cast<uint64_t>(parse_int(it->second, 1024)) << 20;
        if ((it = ep->config.find("dense_weights")) != ep->config.end()) {
            if (it->second == "resident") ep->dense_resident = 1;
            else if (it->second == "transient") ep->dense_resident = 0;
            else {
                delete ep;
                return make_status(NXRT_INVALID_ARGUMENT, "RocmExecutionProvider: dense_weights must be 'transient' or 'resident'");
            }
        }
        ep->dense_gemm_min_rows = ep->dense_resident ? kDenseGemmMinRowsResident : 0;
        if ((it = ep->config.find("dense_gemm_min_rows")) != ep->config.end()) ep->dense_gemm_min_rows = parse_int(it->second, ep->dense_gemm_min_rows);
        NxrtStatus st = ep->bind();
        if (st.code == NXRT_OK) st = hip_status(rocm_ffi_stream_create(&ep->stream), "hipStreamCreate");
        if (st.code == NXRT_OK) st = hip_status(rocm_ffi_static_scratch(static_cast<int>(ep->device), &ep->static_scratch, &ep->static_scratch_bytes), "hipGetSymbolAddress(static scratch)");
        if (st.code != NXRT_OK) {
            delete ep;
            return st;
        }
        init_ep_vtable(ep);
        *out_ep = ep;
        return ok();
    });
}

void nxrt_rocm_ep_release(NxrtRocmEp* ep)
{
    if (!ep || ep->refs.fetch_sub(1) != 1) return;      // kernels and allocator handles still hold it
    try {
        delete ep;
    } catch (...) {
    }
}

const char* nxrt_rocm_ep_name(const NxrtRocmEp* ep) { return ep ? ep->name.c_str() : ""; }
uint32_t nxrt_rocm_ep_device_type(const NxrtRocmEp*) { return NXRT_DEVICE_ROCM; }
uint32_t nxrt_rocm_ep_device_id(const NxrtRocmEp* ep) { return ep ? ep->device : 0; }
uint32_t nxrt_rocm_ep_memory_vendor_id(const NxrtRocmEp*) { return 0x1002u; }

NxrtStatus nxrt_rocm_ep_device_info(const NxrtRocmEp* ep, char* arch, size_t arch_len, uint32_t* compute_units, uint64_t* total_memory)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep) return make_status(NXRT_INVALID_ARGUMENT, "null provider");
        int cus = 0;
        size_t mem = 0;
        const int err = rocm_ffi_device_info(static_cast<int>(ep->device), arch, arch_len, &cus, &mem);
        if (compute_units) *compute_units = static_cast<uint32_t>(cus);
        if (total_memory) *total_memory = mem;
        return hip_status(err, "hipGetDeviceProperties");
    });
}

NxrtStatus nxrt_rocm_ep_allocate(NxrtRocmEp* ep, size_t size, size_t align, void** out_device)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep || !out_device) return make_status(NXRT_INVALID_ARGUMENT, "nxrt_rocm_ep_allocate: null pointer");
        *out_device = nullptr;
        if (align > 256 || (align & (align - 1)) != 0)
            return make_status(NXRT_INVALID_ARGUMENT, "nxrt_rocm_ep_allocate: alignment must be a power of two <= 256, got " + std::to_string(align));
        NxrtStatus st = ep->bind();
        if (st.code != NXRT_OK) return st;
        void* p = nullptr;
        const int err = rocm_ffi_malloc(&p, size ? size : 1);
        if (err != 0) return hip_status(err, "hipMalloc");
        std::lock_guard<std::mutex> lock(ep->mu);
        ep->live[p] = size;
        *out_device = p;
        return ok();
    });
}

NxrtStatus nxrt_rocm_ep_deallocate(NxrtRocmEp* ep, void* device)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep) return make_status(NXRT_INVALID_ARGUMENT, "nxrt_rocm_ep_deallocate: null provider");
        if (!device) return ok();
        {
            std::lock_guard<std::mutex> lock(ep->mu);
            auto it = ep->live.find(device);
            if (it == ep->live.end()) return make_status(NXRT_INVALID_ARGUMENT, "nxrt_rocm_ep_deallocate: pointer was not allocated by this provider");
            ep->live.erase(it);
        }
        NxrtStatus st = ep->bind();
        if (st.code != NXRT_OK) return st;
        rocm_ffi_stream_sync(ep->stream);   // work queued on the stream may still read the buffer
        return hip_status(rocm_ffi_free(device), "hipFree");
    });
}

NxrtStatus nxrt_rocm_ep_copy_from_host(NxrtRocmEp* ep, void* dst, const void* src, size_t bytes)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep || (bytes && (!dst || !src))) return make_status(NXRT_INVALID_ARGUMENT, "copy_from_host: null pointer");
        if (!bytes) return ok();
        NxrtStatus st = ep->bind();
        if (st.code != NXRT_OK) return st;
        return hip_status(rocm_ffi_memcpy_h2d(dst, src, bytes, ep->stream), "hipMemcpy host to device");
    });
}

NxrtStatus nxrt_rocm_ep_copy_to_host(NxrtRocmEp* ep, void* dst, const void* src, size_t bytes)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep || (bytes && (!dst || !src))) return make_status(NXRT_INVALID_ARGUMENT, "copy_to_host: null pointer");
        if (!bytes) return ok();
        NxrtStatus st = ep->bind();
        if (st.code != NXRT_OK) return st;
        return hip_status(rocm_ffi_memcpy_d2h(dst, src, bytes, ep->stream), "hipMemcpy device to host");
    });
}

NxrtStatus nxrt_rocm_ep_copy(NxrtRocmEp* ep, void* dst, const void* src, size_t bytes)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep || (bytes && (!dst || !src))) return make_status(NXRT_INVALID_ARGUMENT, "copy: null pointer");
        if (!bytes) return ok();
        NxrtStatus st = ep->bind();
        if (st.code != NXRT_OK) return st;
        return hip_status(rocm_ffi_memcpy_d2d(dst, src, bytes, ep->stream), "hipMemcpy device to device");
    });
}

NxrtStatus nxrt_rocm_ep_read_probe(NxrtRocmEp* ep, const void* src, size_t bytes)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep || (bytes && !src)) return make_status(NXRT_INVALID_ARGUMENT, "read_probe: null pointer");
        NxrtStatus st = ep->bind();
        if (st.code != NXRT_OK) return st;
        return hip_status(rocm_ffi_read_probe(src, bytes, nullptr, ep->stream), "read probe launch");
    });
}

NxrtStatus nxrt_rocm_ep_lds_probe(NxrtRocmEp* ep, uint32_t mode, uint32_t waves, uint32_t iters, double* bytes_per_clock)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep || !bytes_per_clock) return make_status(NXRT_INVALID_ARGUMENT, "lds_probe: null pointer");
        NxrtStatus st = ep->bind();
        if (st.code != NXRT_OK) return st;
        return hip_status(rocm_ffi_lds_probe(static_cast<int>(mode), static_cast<int>(waves), static_cast<int>(iters), bytes_per_clock), "LDS probe");
    });
}

NxrtStatus nxrt_rocm_ep_sync(NxrtRocmEp* ep)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep) return make_status(NXRT_INVALID_ARGUMENT, "sync: null provider");
        NxrtStatus st = ep->bind();
        if (st.code != NXRT_OK) return st;
        return hip_status(rocm_ffi_stream_sync(ep->stream), "hipStreamSynchronize");
    });
}

NxrtStatus nxrt_rocm_ep_event_create(NxrtRocmEp* ep, NxrtRocmEvent** out_event)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep || !out_event) return make_status(NXRT_INVALID_ARGUMENT, "event_create: null pointer");
        NxrtStatus st = ep->bind();
        if (st.code != NXRT_OK) return st;
        auto* e = new NxrtRocmEvent();
        const int err = rocm_ffi_event_create(&e->ev);
        if (err != 0) {
            delete e;
            return hip_status(err, "hipEventCreate");
        }
        *out_event = e;
        return ok();
    });
}

NxrtStatus nxrt_rocm_ep_event_record(NxrtRocmEp* ep, NxrtRocmEvent* event)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep || !event) return make_status(NXRT_INVALID_ARGUMENT, "event_record: null pointer");
        return hip_status(rocm_ffi_event_record(event->ev, ep->stream), "hipEventRecord");
    });
}

NxrtStatus nxrt_rocm_ep_event_elapsed_ms(NxrtRocmEp* ep, NxrtRocmEvent* start, NxrtRocmEvent* stop, float* out_ms)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep || !start || !stop || !out_ms) return make_status(NXRT_INVALID_ARGUMENT, "event_elapsed_ms: null pointer");
        int err = rocm_ffi_event_sync(stop->ev);
        if (err == 0) err = rocm_ffi_event_elapsed_ms(start->ev, stop->ev, out_ms);
        return hip_status(err, "hipEventElapsedTime");
    });
}

void nxrt_rocm_ep_event_destroy(NxrtRocmEp*, NxrtRocmEvent* event)
{
    if (!event) return;
    rocm_ffi_event_destroy(event->ev);
    delete event;
}

NxrtStatus nxrt_rocm_ep_capture_begin(NxrtRocmEp* ep)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep) return make_status(NXRT_INVALID_ARGUMENT, "capture_begin: null provider");
        NxrtStatus st = ep->bind();
        if (st.code != NXRT_OK) return st;
        if (ep->capturing) return make_status(NXRT_INVALID_ARGUMENT, "capture_begin: a capture is already open on this provider");
        st = hip_status(rocm_ffi_capture_begin(ep->stream), "hipStreamBeginCapture");
        if (st.code == NXRT_OK) {
            ep->capturing = true;
            ep->captures.fetch_add(1);
        }
        return st;
    });
}

NxrtStatus nxrt_rocm_ep_capture_end(NxrtRocmEp* ep, NxrtRocmGraph** out_graph, uint64_t* out_num_nodes)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep || !out_graph) return make_status(NXRT_INVALID_ARGUMENT, "capture_end: null pointer");
        *out_graph = nullptr;
        if (!ep->capturing) return make_status(NXRT_INVALID_ARGUMENT, "capture_end: no capture is open on this provider");
        ep->capturing = false;
        rocm_graph_exec_t exec = nullptr;
        size_t nodes = 0;
        const int err = rocm_ffi_capture_end(ep->stream, &exec, &nodes);
        if (err != 0) return hip_status(err, "hipStreamEndCapture");
        auto* g = new NxrtRocmGraph();
        g->exec = exec;
        if (out_num_nodes) *out_num_nodes = nodes;
        *out_graph = g;
        return ok();
    });
}

NxrtStatus nxrt_rocm_ep_graph_replay(NxrtRocmEp* ep, NxrtRocmGraph* graph)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep || !graph) return make_status(NXRT_INVALID_ARGUMENT, "graph_replay: null pointer");
        return hip_status(rocm_ffi_graph_launch(graph->exec, ep->stream), "hipGraphLaunch");
    });
}

void nxrt_rocm_ep_graph_release(NxrtRocmEp* ep, NxrtRocmGraph* graph)
{
    if (!graph) return;
    if (ep && ep->bind().code == NXRT_OK) rocm_ffi_stream_sync(ep->stream);
    rocm_ffi_graph_destroy(graph->exec);
    delete graph;
}

uint64_t nxrt_rocm_ep_kernel_launch_count(const NxrtRocmEp* ep) { return ep ? ep->launches.load() : 0; }
uint64_t nxrt_rocm_live_provider_count(void) { return g_live_providers.load(); }
uint64_t nxrt_rocm_device_allocation_count(void) { return rocm_ffi_malloc_calls(); }

}  // extern "C"
