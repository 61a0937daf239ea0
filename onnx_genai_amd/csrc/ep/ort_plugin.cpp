// The ORT plugin execution-provider export: CreateEpFactories / ReleaseEpFactory and the OrtEpFactory / OrtEp /
// OrtNodeComputeInfo / OrtAllocator / OrtDataTransferImpl callbacks behind them, so that upstream ONNX Runtime can load
// this library as an EP and hand it com.microsoft::MatMulNBits nodes
// (crates/onnx-runtime-ep-plugin/src/lib.rs:113-188 for the two entry points, factory.rs:131-158 and ep.rs:250-270 for
// the tables, crates/onnx-runtime-ep-cpu/src/kernels/mod.rs:197-209 for the per-slot dtype rule of a claim).
//
// The plugin claims every MatMulNBits node the provider's own supports_op accepts, each as a one-node fusion
// (EpGraphSupportInfo_AddNodesToFuse), compiles it to an OrtNodeComputeInfo that owns one nxrt kernel object, and runs it
// through nxrt_rocm_matmul_nbits_execute on tensors ORT allocated with this plugin's device allocator. The provider
// (one per GPU ordinal, shared by every EP, allocator and kernel of a factory) is created on first use, so listing
// devices, creating an EP and answering GetCapability touch no GPU.
//
// Every callback catches what its body throws and answers with an OrtStatus (or the callback's neutral value): nothing
// unwinds into the host.
#include <atomic>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#if defined(NXRT_ORT_REAL_HEADERS)
#include <onnxruntime_c_api.h>
#include <onnxruntime_ep_c_api.h>
#else
#include "../../../include/ort_plugin_ep_subset.h"
#endif
#include "../../../include/nxrt_ep_rocm.h"
#include "../../../include/nxrt_ort_plugin.h"

namespace {

constexpr uint32_t kAmdVendorId = 0x1002;
const char kDefaultName[] = "RocmExecutionProvider";
const char kVendor[] = "nxrt";
const char kVersion[] = "0.1.0";

struct Host {
    const OrtApi* api = nullptr;
    const OrtEpApi* ep_api = nullptr;
    OrtStatus* status(OrtErrorCode code, const std::string& message) const { return api->CreateStatus(code, message.c_str()); }
};

OrtErrorCode ort_code(uint32_t nxrt_code)
{
    switch (nxrt_code) {
        case NXRT_INVALID_ARGUMENT: return ORT_INVALID_ARGUMENT;
        case NXRT_NOT_IMPLEMENTED:
        case NXRT_UNSUPPORTED_CAPABILITY: return ORT_NOT_IMPLEMENTED;
        default: return ORT_EP_FAIL;
    }
}

OrtStatus* from_nxrt(const Host& host, const NxrtStatus& st)
{
    if (st.code == NXRT_OK) return nullptr;
    return host.status(ort_code(st.code), std::string(reinterpret_cast<const char*>(st.message), st.message_len));
}

// A host call whose failure this plugin treats as "not there" (an absent attribute): the status is released.
bool succeeded(const Host& host, OrtStatus* st)
{
    if (!st) return true;
    host.api->ReleaseStatus(st);
    return false;
}

template <class F>
OrtStatus* guarded(const Host& host, const char* where, F&& body)
{
    try {
        return body();
    } catch (const std::bad_alloc&) {
        return host.status(ORT_EP_FAIL, std::string(where) + ": out of host memory");
    } catch (const std::exception& e) {
        return host.status(ORT_EP_FAIL, std::string(where) + ": " + e.what());
    } catch (...) {
        return host.status(ORT_EP_FAIL, std::string(where) + ": unknown exception");
    }
}

struct RocmOrtFactory {
    OrtEpFactory vtable;             // first: the host's OrtEpFactory* is this object
    Host host;
    std::string name;
    std::mutex mu;
    std::vector<const OrtHardwareDevice*> claimed;        // index = GPU ordinal
    std::vector<OrtMemoryInfo*> memory_infos;             // one per claimed device, owned
    std::map<uint32_t, NxrtRocmEp*> providers;            // created on first use, one per ordinal
    std::atomic<int> live_eps{0}, live_allocators{0}, live_transfers{0};

    // The provider of a GPU ordinal; made on first use (the first call that needs the GPU).
    OrtStatus* provider(uint32_t ordinal, NxrtRocmEp** out)
    {
        std::lock_guard<std::mutex> lock(mu);
        auto it = providers.find(ordinal);
        if (it == providers.end()) {
            NxrtRocmEp* ep = nullptr;
            const NxrtStatus st = nxrt_rocm_ep_create(ordinal, nullptr, nullptr, 0, &ep);
            if (st.code != NXRT_OK) return from_nxrt(host, st);
            it = providers.emplace(ordinal, ep).first;
        }
        *out = it->second;
        return nullptr;
    }
};

struct RocmOrtEp {
    OrtEp vtable;
    RocmOrtFactory* factory;
    uint32_t ordinal;
    std::atomic<int> live_compute_infos{0};
};

struct RocmNodeCompute {
    OrtNodeComputeInfo vtable;
    RocmOrtEp* ep;
    NxrtRocmMatMulNBitsAttrs attrs;
    std::vector<uint8_t> constant_inputs;
};

struct RocmNodeState {
    NxrtRocmEp* provider;
    NxrtRocmMatMulNBits* kernel;
};

struct RocmOrtAllocator {
    OrtAllocator vtable;
    RocmOrtFactory* factory;
    const OrtMemoryInfo* info;
    uint32_t ordinal;
};

struct RocmDataTransfer {
    OrtDataTransferImpl vtable;
    RocmOrtFactory* factory;
};

// ---------------------------------------------------------------------------------------------
// Node inspection shared by GetCapability and Compile
// ---------------------------------------------------------------------------------------------
enum AttrBit { kK = 0, kN = 1, kBits = 2, kBlockSize = 3, kAccuracy = 4, kPrepacked = 5 };

bool read_int_attr(const Host& host, const OrtNode* node, const char* name, int64_t* out)
{
    const OrtOpAttr* attr = nullptr;
    if (!succeeded(host, host.api->Node_GetAttributeByName(node, name, &attr)) || !attr) return false;
    size_t used = 0;
    return succeeded(host, host.api->ReadOpAttr(attr, ORT_OP_ATTR_INT, out, sizeof(*out), &used));
}

NxrtRocmMatMulNBitsAttrs read_attrs(const Host& host, const OrtNode* node)
{
    NxrtRocmMatMulNBitsAttrs a;
    std::memset(&a, 0, sizeof(a));
    a.struct_size = sizeof(a);
    const struct { const char* name; int64_t* field; int bit; } wanted[] = {
        {"K", &a.K, kK}, {"N", &a.N, kN}, {"bits", &a.bits, kBits}, {"block_size", &a.block_size, kBlockSize},
        {"accuracy_level", &a.accuracy_level, kAccuracy}, {"weight_prepacked", &a.weight_prepacked, kPrepacked}};
    for (const auto& w : wanted)
        if (read_int_attr(host, node, w.name, w.field)) a.present |= 1u << w.bit;
    return a;
}

bool is_matmul_nbits(const Host& host, const OrtNode* node)
{
    const char* op = nullptr;
    const char* domain = nullptr;
    if (!succeeded(host, host.api->Node_GetOperatorType(node, &op)) || !op || std::strcmp(op, "MatMulNBits") != 0) return false;
    if (!succeeded(host, host.api->Node_GetDomain(node, &domain)) || !domain) return false;
    return std::strcmp(domain, "com.microsoft") == 0;
}

// Element type and dimensions of every input slot; an absent optional input has dtype 0.
struct NodeInputs {
    std::vector<const OrtValueInfo*> infos;
    std::vector<std::vector<int64_t>> dims;
    std::vector<NxrtTensorDesc> descs;
};

bool read_inputs(const Host& host, const OrtNode* node, NodeInputs& out)
{
    size_t n = 0;
    if (!succeeded(host, host.api->Node_GetNumInputs(node, &n))) return false;
    out.infos.assign(n, nullptr);
    if (n && !succeeded(host, host.api->Node_GetInputs(node, out.infos.data(), n))) return false;
    out.dims.assign(n, {});
    out.descs.assign(n, NxrtTensorDesc{});
    for (size_t i = 0; i < n; ++i) {
        NxrtTensorDesc& d = out.descs[i];
        std::memset(&d, 0, sizeof(d));
        if (!out.infos[i]) continue;
        const OrtTypeInfo* type_info = nullptr;
        const OrtTensorTypeAndShapeInfo* tensor = nullptr;
        if (!succeeded(host, host.api->GetValueInfoTypeInfo(out.infos[i], &type_info)) || !type_info) return false;
        if (!succeeded(host, host.api->CastTypeInfoToTensorInfo(type_info, &tensor)) || !tensor) return false;      // not a tensor
        ONNXTensorElementDataType et = ONNX_TENSOR_ELEMENT_DATA_TYPE_UNDEFINED;
        if (!succeeded(host, host.api->GetTensorElementType(tensor, &et))) return false;
        d.dtype = static_cast<uint32_t>(et);          // the nxrt dtype codes are the ONNX element type codes
        size_t nd = 0;
        if (succeeded(host, host.api->GetDimensionsCount(tensor, &nd)) && nd) {
            out.dims[i].assign(nd, -1);
            if (!succeeded(host, host.api->GetDimensions(tensor, out.dims[i].data(), nd))) out.dims[i].clear();
        }
        d.ndim = static_cast<uint32_t>(out.dims[i].size());
        d.dims = out.dims[i].data();
    }
    return true;
}

// kernels/mod.rs:197-209: every present slot is held to its own dtype set, not to the union over all slots
// (A, B, scales, zero_points, g_idx, bias).
bool slot_dtypes_ok(const NodeInputs& in)
{
    auto float_compute = [](uint32_t dt) { return dt == NXRT_DT_FLOAT32 || dt == NXRT_DT_FLOAT16 || dt == NXRT_DT_BFLOAT16; };
    for (size_t i = 0; i < in.descs.size() && i < 6; ++i) {
        const uint32_t dt = in.descs[i].dtype;
        if (dt == 0) {
            if (i < 3) return false;                  // A, B and scales are required
            continue;
        }
        const bool ok = (i == 0 || i == 2 || i == 5) ? float_compute(dt) : (i == 4 ? dt == NXRT_DT_INT32 : dt == NXRT_DT_UINT8);
        if (!ok) return false;
    }
    return in.descs.size() >= 3 && in.descs.size() <= 6;
}

// ---------------------------------------------------------------------------------------------
// OrtNodeComputeInfo
// ---------------------------------------------------------------------------------------------
OrtStatus* ORT_API_CALL compute_create_state(OrtNodeComputeInfo* this_ptr, OrtNodeComputeContext*, void** compute_state)
{
    auto* nc = reinterpret_cast<RocmNodeCompute*>(this_ptr);
    const Host& host = nc->ep->factory->host;
    return guarded(host, "CreateState", [&]() -> OrtStatus* {
        if (!compute_state) return host.status(ORT_INVALID_ARGUMENT, "CreateState: null compute_state");
        *compute_state = nullptr;
        NxrtRocmEp* provider = nullptr;
        if (OrtStatus* st = nc->ep->factory->provider(nc->ep->ordinal, &provider)) return st;
        NxrtRocmMatMulNBits* kernel = nullptr;
        const NxrtStatus st = nxrt_rocm_matmul_nbits_create(provider, &nc->attrs, nullptr, 0, &kernel);
        if (st.code != NXRT_OK) return from_nxrt(host, st);
        nxrt_rocm_matmul_nbits_set_constant_inputs(kernel, nc->constant_inputs.data(), static_cast<uint32_t>(nc->constant_inputs.size()));
        *compute_state = new RocmNodeState{provider, kernel};
        return nullptr;
    });
}

OrtStatus* ORT_API_CALL compute_compute(OrtNodeComputeInfo* this_ptr, void* compute_state, OrtKernelContext* ctx)
{
    auto* nc = reinterpret_cast<RocmNodeCompute*>(this_ptr);
    const Host& host = nc->ep->factory->host;
    return guarded(host, "Compute", [&]() -> OrtStatus* {
        auto* state = static_cast<RocmNodeState*>(compute_state);
        if (!state || !ctx) return host.status(ORT_INVALID_ARGUMENT, "Compute: null state or kernel context");
        size_t n = 0;
        if (OrtStatus* st = host.api->KernelContext_GetInputCount(ctx, &n)) return st;
        if (n < 3 || n > 6) return host.status(ORT_INVALID_ARGUMENT, "MatMulNBits: expected 3..=6 inputs, got " + std::to_string(n));
        std::vector<NxrtRocmTensorView> views(n);
        std::vector<std::vector<uint64_t>> shapes(n);
        const uint32_t device = nxrt_rocm_ep_device_id(state->provider);
        for (size_t i = 0; i < n; ++i) {
            NxrtRocmTensorView& v = views[i];
            std::memset(&v, 0, sizeof(v));
            const OrtValue* value = nullptr;
            if (OrtStatus* st = host.api->KernelContext_GetInput(ctx, i, &value)) return st;
            if (!value) continue;                                  // an absent optional input: data stays NULL
            OrtTensorTypeAndShapeInfo* info = nullptr;
            if (OrtStatus* st = host.api->GetTensorTypeAndShape(value, &info)) return st;
            ONNXTensorElementDataType et = ONNX_TENSOR_ELEMENT_DATA_TYPE_UNDEFINED;
            size_t nd = 0;
            OrtStatus* st = host.api->GetTensorElementType(info, &et);
            if (!st) st = host.api->GetDimensionsCount(info, &nd);
            std::vector<int64_t> dims(nd);
            if (!st && nd) st = host.api->GetDimensions(info, dims.data(), nd);
            host.api->ReleaseTensorTypeAndShapeInfo(info);
            if (st) return st;
            shapes[i].assign(dims.begin(), dims.end());
            const void* data = nullptr;
            if (OrtStatus* e = host.api->GetTensorData(value, &data)) return e;
            // the tensors must be where this provider's kernels can read them
            if (host.ep_api->Value_GetMemoryDevice) {
                const OrtMemoryDevice* md = host.ep_api->Value_GetMemoryDevice(value);
                if (md && (host.ep_api->MemoryDevice_GetDeviceType(md) != OrtMemoryInfoDeviceType_GPU || host.ep_api->MemoryDevice_GetVendorId(md) != kAmdVendorId))
                    return host.status(ORT_INVALID_ARGUMENT, "MatMulNBits: input " + std::to_string(i) + " is not in ROCm device memory (the session must allocate "
                                                             "this node's tensors with the ROCm execution provider's allocator)");
                if (md && host.ep_api->MemoryDevice_GetDeviceId && host.ep_api->MemoryDevice_GetDeviceId(md) != device)
                    return host.status(ORT_INVALID_ARGUMENT, "MatMulNBits: input " + std::to_string(i) + " lives on GPU " +
                                                             std::to_string(host.ep_api->MemoryDevice_GetDeviceId(md)) + ", this execution provider runs on GPU " +
                                                             std::to_string(device));
            }
            v.data = const_cast<void*>(data);
            v.dtype = static_cast<uint32_t>(et);
            v.ndim = static_cast<uint32_t>(nd);
            v.shape = shapes[i].data();
            v.device_type = NXRT_DEVICE_ROCM;
            v.device_index = device;
        }
        if (!views[0].data || views[0].ndim == 0) return host.status(ORT_INVALID_ARGUMENT, "MatMulNBits: A must be a tensor of rank >= 1");
        // Y = A.shape[:-1] + [N], of A's element type
        std::vector<int64_t> y_dims(shapes[0].begin(), shapes[0].end());
        y_dims.back() = nc->attrs.N;
        OrtValue* y = nullptr;
        if (OrtStatus* st = host.api->KernelContext_GetOutput(ctx, 0, y_dims.data(), y_dims.size(), &y)) return st;
        if (!y) return host.status(ORT_EP_FAIL, "MatMulNBits: the host returned no output tensor");
        void* y_data = nullptr;
        if (OrtStatus* st = host.api->GetTensorMutableData(y, &y_data)) return st;
        std::vector<uint64_t> y_shape(y_dims.begin(), y_dims.end());
        NxrtRocmTensorView out;
        std::memset(&out, 0, sizeof(out));
        out.data = y_data;
        out.dtype = views[0].dtype;
        out.ndim = static_cast<uint32_t>(y_shape.size());
        out.shape = y_shape.data();
        out.device_type = NXRT_DEVICE_ROCM;
        out.device_index = device;
        const NxrtStatus st = nxrt_rocm_matmul_nbits_execute(state->kernel, views.data(), static_cast<uint32_t>(n), &out, 1, nullptr, 0);
        if (st.code != NXRT_OK) return from_nxrt(host, st);
        // this EP announces no streams of its own (IsStreamAware = false): the result is complete when Compute returns
        return from_nxrt(host, nxrt_rocm_ep_sync(state->provider));
    });
}

void ORT_API_CALL compute_release_state(OrtNodeComputeInfo*, void* compute_state)
{
    auto* state = static_cast<RocmNodeState*>(compute_state);
    if (!state) return;
    nxrt_rocm_matmul_nbits_release(state->kernel);
    delete state;
}

// ---------------------------------------------------------------------------------------------
// OrtEp
// ---------------------------------------------------------------------------------------------
const char* ORT_API_CALL ep_get_name(const OrtEp* this_ptr)
{
    return this_ptr ? reinterpret_cast<const RocmOrtEp*>(this_ptr)->factory->name.c_str() : kDefaultName;
}

OrtStatus* ORT_API_CALL ep_get_capability(OrtEp* this_ptr, const OrtGraph* graph, OrtEpGraphSupportInfo* support)
{
    auto* ep = reinterpret_cast<RocmOrtEp*>(this_ptr);
    const Host& host = ep->factory->host;
    return guarded(host, "GetCapability", [&]() -> OrtStatus* {
        if (!graph || !support) return host.status(ORT_INVALID_ARGUMENT, "GetCapability: null argument");
        size_t count = 0;
        if (OrtStatus* st = host.api->Graph_GetNumNodes(graph, &count)) return st;
        std::vector<const OrtNode*> nodes(count, nullptr);
        if (count)
            if (OrtStatus* st = host.api->Graph_GetNodes(graph, nodes.data(), count)) return st;
        for (const OrtNode* node : nodes) {
            if (!node || !is_matmul_nbits(host, node)) continue;
            NodeInputs in;
            if (!read_inputs(host, node, in) || !slot_dtypes_ok(in)) continue;
            const NxrtRocmMatMulNBitsAttrs attrs = read_attrs(host, node);
            char reason[256];
            if (!nxrt_rocm_ep_supports_matmul_nbits(nullptr, &attrs, in.descs.data(), static_cast<uint32_t>(in.descs.size()), reason, sizeof(reason))) continue;
            if (OrtStatus* st = host.ep_api->EpGraphSupportInfo_AddNodesToFuse(support, &node, 1, nullptr)) return st;
        }
        return nullptr;
    });
}

OrtStatus* ORT_API_CALL ep_compile(OrtEp* this_ptr, const OrtGraph** graphs, const OrtNode** fused_nodes, size_t count, OrtNodeComputeInfo** node_compute_infos,
                                   OrtNode** /*ep_context_nodes*/)
{
    auto* ep = reinterpret_cast<RocmOrtEp*>(this_ptr);
    const Host& host = ep->factory->host;
    return guarded(host, "Compile", [&]() -> OrtStatus* {
        if (count && (!graphs || !fused_nodes || !node_compute_infos)) return host.status(ORT_INVALID_ARGUMENT, "Compile: null argument");
        std::vector<std::unique_ptr<RocmNodeCompute>> made;
        for (size_t i = 0; i < count; ++i) {
            size_t n_nodes = 0;
            if (OrtStatus* st = host.api->Graph_GetNumNodes(graphs[i], &n_nodes)) return st;
            if (n_nodes != 1) return host.status(ORT_EP_FAIL, "Compile: this EP claims single MatMulNBits nodes; fused graph " + std::to_string(i) + " has " +
                                                                  std::to_string(n_nodes) + " nodes");
            const OrtNode* node = nullptr;
            if (OrtStatus* st = host.api->Graph_GetNodes(graphs[i], &node, 1)) return st;
            if (!node || !is_matmul_nbits(host, node)) return host.status(ORT_EP_FAIL, "Compile: fused graph " + std::to_string(i) + " is not a com.microsoft::MatMulNBits node");
            NodeInputs in;
            if (!read_inputs(host, node, in)) return host.status(ORT_EP_FAIL, "Compile: cannot read the inputs of fused graph " + std::to_string(i));
            auto nc = std::make_unique<RocmNodeCompute>();
            std::memset(&nc->vtable, 0, sizeof(nc->vtable));
            nc->vtable.ort_version_supported = ORT_API_VERSION;
            nc->vtable.CreateState = compute_create_state;
            nc->vtable.Compute = compute_compute;
            nc->vtable.ReleaseState = compute_release_state;
            nc->ep = ep;
            nc->attrs = read_attrs(host, node);
            // factory checks (K, N, bits, block_size ...) with the provider's own messages, before any state exists
            char reason[256];
            if (!nxrt_rocm_ep_supports_matmul_nbits(nullptr, &nc->attrs, in.descs.data(), static_cast<uint32_t>(in.descs.size()), reason, sizeof(reason)))
                return host.status(ORT_INVALID_ARGUMENT, reason);
            nc->constant_inputs.assign(in.infos.size(), 0);
            for (size_t s = 0; s < in.infos.size(); ++s) {
                bool constant = false;
                if (in.infos[s] && host.api->ValueInfo_IsConstantInitializer && succeeded(host, host.api->ValueInfo_IsConstantInitializer(in.infos[s], &constant)))
                    nc->constant_inputs[s] = constant ? 1 : 0;
            }
            made.push_back(std::move(nc));
        }
        for (size_t i = 0; i < count; ++i) {
            node_compute_infos[i] = &made[i]->vtable;
            made[i].release();
            ep->live_compute_infos.fetch_add(1);
        }
        return nullptr;
    });
}

void ORT_API_CALL ep_release_node_compute_infos(OrtEp* this_ptr, OrtNodeComputeInfo** infos, size_t count)
{
    auto* ep = reinterpret_cast<RocmOrtEp*>(this_ptr);
    if (!infos) return;
    for (size_t i = 0; i < count; ++i) {
        if (!infos[i]) continue;
        delete reinterpret_cast<RocmNodeCompute*>(infos[i]);
        infos[i] = nullptr;
        if (ep) ep->live_compute_infos.fetch_sub(1);
    }
}

// ---------------------------------------------------------------------------------------------
// OrtAllocator (device memory of one GPU) and OrtDataTransferImpl (host <-> device, device -> device)
// ---------------------------------------------------------------------------------------------
void* ORT_API_CALL allocator_alloc(OrtAllocator* this_, size_t size)
{
    auto* a = reinterpret_cast<RocmOrtAllocator*>(this_);
    try {
        NxrtRocmEp* provider = nullptr;
        if (OrtStatus* st = a->factory->provider(a->ordinal, &provider)) {
            a->factory->host.api->ReleaseStatus(st);
            return nullptr;
        }
        void* p = nullptr;
        return nxrt_rocm_ep_allocate(provider, size ? size : 1, 256, &p).code == NXRT_OK ? p : nullptr;
    } catch (...) {
        return nullptr;
    }
}

void ORT_API_CALL allocator_free(OrtAllocator* this_, void* p)
{
    auto* a = reinterpret_cast<RocmOrtAllocator*>(this_);
    if (!p) return;
    try {
        NxrtRocmEp* provider = nullptr;
        if (OrtStatus* st = a->factory->provider(a->ordinal, &provider)) {
            a->factory->host.api->ReleaseStatus(st);
            return;
        }
        (void)nxrt_rocm_ep_deallocate(provider, p);
    } catch (...) {
    }
}

const OrtMemoryInfo* ORT_API_CALL allocator_info(const OrtAllocator* this_) { return reinterpret_cast<const RocmOrtAllocator*>(this_)->info; }
void* ORT_API_CALL allocator_reserve(OrtAllocator* this_, size_t size) { return allocator_alloc(this_, size); }

void ORT_API_CALL transfer_release(OrtDataTransferImpl* this_ptr)
{
    auto* t = reinterpret_cast<RocmDataTransfer*>(this_ptr);
    if (!t) return;
    t->factory->live_transfers.fetch_sub(1);
    delete t;
}

bool is_rocm(const Host& host, const OrtMemoryDevice* d)
{
    return d && host.ep_api->MemoryDevice_GetDeviceType(d) == OrtMemoryInfoDeviceType_GPU && host.ep_api->MemoryDevice_GetVendorId(d) == kAmdVendorId;
}
bool is_host(const Host& host, const OrtMemoryDevice* d) { return d && host.ep_api->MemoryDevice_GetDeviceType(d) == OrtMemoryInfoDeviceType_CPU; }

bool ORT_API_CALL transfer_can_copy(const OrtDataTransferImpl* this_ptr, const OrtMemoryDevice* src, const OrtMemoryDevice* dst)
{
    const Host& host = reinterpret_cast<const RocmDataTransfer*>(this_ptr)->factory->host;
    try {
        return (is_rocm(host, src) && (is_rocm(host, dst) || is_host(host, dst))) || (is_host(host, src) && is_rocm(host, dst));
    } catch (...) {
        return false;
    }
}

OrtStatus* ORT_API_CALL transfer_copy_tensors(OrtDataTransferImpl* this_ptr, const OrtValue** src, OrtValue** dst, OrtSyncStream** /*streams*/, size_t count)
{
    auto* t = reinterpret_cast<RocmDataTransfer*>(this_ptr);
    const Host& host = t->factory->host;
    return guarded(host, "CopyTensors", [&]() -> OrtStatus* {
        for (size_t i = 0; i < count; ++i) {
            const OrtMemoryDevice* sd = host.ep_api->Value_GetMemoryDevice(src[i]);
            const OrtMemoryDevice* dd = host.ep_api->Value_GetMemoryDevice(dst[i]);
            size_t bytes = 0, dst_bytes = 0;
            if (OrtStatus* st = host.api->GetTensorSizeInBytes(src[i], &bytes)) return st;
            if (OrtStatus* st = host.api->GetTensorSizeInBytes(dst[i], &dst_bytes)) return st;
            if (dst_bytes < bytes) return host.status(ORT_INVALID_ARGUMENT, "CopyTensors: destination " + std::to_string(i) + " is smaller than its source");
            const void* from = nullptr;
            void* to = nullptr;
            if (OrtStatus* st = host.api->GetTensorData(src[i], &from)) return st;
            if (OrtStatus* st = host.api->GetTensorMutableData(dst[i], &to)) return st;
            const bool src_dev = is_rocm(host, sd), dst_dev = is_rocm(host, dd);
            if (!src_dev && !dst_dev) return host.status(ORT_INVALID_ARGUMENT, "CopyTensors: neither side of copy " + std::to_string(i) + " is ROCm device memory");
            NxrtRocmEp* provider = nullptr;
            if (OrtStatus* st = t->factory->provider(host.ep_api->MemoryDevice_GetDeviceId(src_dev ? sd : dd), &provider)) return st;
            if (bytes == 0) continue;
            const NxrtStatus st = src_dev && dst_dev ? nxrt_rocm_ep_copy(provider, to, from, bytes)
                                  : dst_dev          ? nxrt_rocm_ep_copy_from_host(provider, to, from, bytes)
                                                     : nxrt_rocm_ep_copy_to_host(provider, to, from, bytes);
            if (st.code != NXRT_OK) return from_nxrt(host, st);
            if (src_dev && dst_dev)
                if (OrtStatus* e = from_nxrt(host, nxrt_rocm_ep_sync(provider))) return e;       // the host assumes a finished copy
        }
        return nullptr;
    });
}

// ---------------------------------------------------------------------------------------------
// OrtEpFactory
// ---------------------------------------------------------------------------------------------
RocmOrtFactory* self(OrtEpFactory* f) { return reinterpret_cast<RocmOrtFactory*>(f); }
const RocmOrtFactory* self(const OrtEpFactory* f) { return reinterpret_cast<const RocmOrtFactory*>(f); }

const char* ORT_API_CALL factory_get_name(const OrtEpFactory* f) { return f ? self(f)->name.c_str() : kDefaultName; }
const char* ORT_API_CALL factory_get_vendor(const OrtEpFactory*) { return kVendor; }
uint32_t ORT_API_CALL factory_get_vendor_id(const OrtEpFactory*) { return kAmdVendorId; }
const char* ORT_API_CALL factory_get_version(const OrtEpFactory*) { return kVersion; }
bool ORT_API_CALL factory_is_stream_aware(const OrtEpFactory*) { return false; }

// Every AMD GPU the host lists becomes an OrtEpDevice with this plugin's device-memory info attached; the n-th such
// device is GPU ordinal n (the order HIP enumerates them in is the order of the PCI bus, as the host's list is).
OrtStatus* ORT_API_CALL factory_get_supported_devices(OrtEpFactory* f, const OrtHardwareDevice* const* devices, size_t num_devices, OrtEpDevice** ep_devices,
                                                      size_t max_ep_devices, size_t* num_ep_devices)
{
    RocmOrtFactory* fac = self(f);
    const Host& host = fac->host;
    return guarded(host, "GetSupportedDevices", [&]() -> OrtStatus* {
        if (!num_ep_devices || (num_devices && !devices) || (max_ep_devices && !ep_devices)) return host.status(ORT_INVALID_ARGUMENT, "GetSupportedDevices: null argument");
        *num_ep_devices = 0;
        std::lock_guard<std::mutex> lock(fac->mu);
        for (size_t i = 0; i < num_devices && *num_ep_devices < max_ep_devices; ++i) {
            const OrtHardwareDevice* hw = devices[i];
            if (!hw || host.api->HardwareDevice_Type(hw) != OrtHardwareDeviceType_GPU || host.api->HardwareDevice_VendorId(hw) != kAmdVendorId) continue;
            size_t ordinal = 0;
            while (ordinal < fac->claimed.size() && fac->claimed[ordinal] != hw) ++ordinal;
            if (ordinal == fac->claimed.size()) {
                OrtMemoryInfo* info = nullptr;
                if (OrtStatus* st = host.api->CreateMemoryInfo_V2(kDefaultName, OrtMemoryInfoDeviceType_GPU, kAmdVendorId, static_cast<int32_t>(ordinal),
                                                                  OrtDeviceMemoryType_DEFAULT, 256, OrtDeviceAllocator, &info))
                    return st;
                fac->claimed.push_back(hw);
                fac->memory_infos.push_back(info);
            }
            OrtEpDevice* ep_device = nullptr;
            if (OrtStatus* st = host.ep_api->CreateEpDevice(f, hw, nullptr, nullptr, &ep_device)) return st;
            if (OrtStatus* st = host.ep_api->EpDevice_AddAllocatorInfo(ep_device, fac->memory_infos[ordinal])) {
                host.ep_api->ReleaseEpDevice(ep_device);
                return st;
            }
            ep_devices[(*num_ep_devices)++] = ep_device;
        }
        return nullptr;
    });
}

OrtStatus* ORT_API_CALL factory_create_ep(OrtEpFactory* f, const OrtHardwareDevice* const* devices, const OrtKeyValuePairs* const*, size_t num_devices,
                                          const OrtSessionOptions*, const OrtLogger*, OrtEp** out)
{
    RocmOrtFactory* fac = self(f);
    const Host& host = fac->host;
    return guarded(host, "CreateEp", [&]() -> OrtStatus* {
        if (!out) return host.status(ORT_INVALID_ARGUMENT, "CreateEp: null output pointer");
        *out = nullptr;
        if (num_devices != 1 || !devices || !devices[0])
            return host.status(ORT_INVALID_ARGUMENT, "CreateEp: the ROCm execution provider runs on exactly one GPU per EP instance, got " + std::to_string(num_devices) + " devices");
        uint32_t ordinal = 0;
        {
            std::lock_guard<std::mutex> lock(fac->mu);
            size_t at = 0;
            while (at < fac->claimed.size() && fac->claimed[at] != devices[0]) ++at;
            if (at == fac->claimed.size()) return host.status(ORT_INVALID_ARGUMENT, "CreateEp: the device was not offered by this factory's GetSupportedDevices");
            ordinal = static_cast<uint32_t>(at);
        }
        auto* ep = new RocmOrtEp();
        std::memset(&ep->vtable, 0, sizeof(ep->vtable));
        ep->vtable.ort_version_supported = ORT_API_VERSION;
        ep->vtable.GetName = ep_get_name;
        ep->vtable.GetCapability = ep_get_capability;
        ep->vtable.Compile = ep_compile;
        ep->vtable.ReleaseNodeComputeInfos = ep_release_node_compute_infos;
        ep->factory = fac;
        ep->ordinal = ordinal;
        fac->live_eps.fetch_add(1);
        *out = &ep->vtable;
        return nullptr;
    });
}

void ORT_API_CALL factory_release_ep(OrtEpFactory* f, OrtEp* ep)
{
    if (!ep) return;
    self(f)->live_eps.fetch_sub(1);
    delete reinterpret_cast<RocmOrtEp*>(ep);
}

OrtStatus* ORT_API_CALL factory_validate_compiled(OrtEpFactory*, const OrtHardwareDevice* const*, size_t, const char*, OrtCompiledModelCompatibility* out)
{
    if (out) *out = OrtCompiledModelCompatibility_EP_NOT_APPLICABLE;      // this EP writes no compiled-model (EPContext) nodes
    return nullptr;
}

OrtStatus* ORT_API_CALL factory_create_allocator(OrtEpFactory* f, const OrtMemoryInfo* memory_info, const OrtKeyValuePairs*, OrtAllocator** out)
{
    RocmOrtFactory* fac = self(f);
    const Host& host = fac->host;
    return guarded(host, "CreateAllocator", [&]() -> OrtStatus* {
        if (!out) return host.status(ORT_INVALID_ARGUMENT, "CreateAllocator: null output pointer");
        *out = nullptr;
        size_t ordinal = 0;
        {
            std::lock_guard<std::mutex> lock(fac->mu);
            while (ordinal < fac->memory_infos.size() && fac->memory_infos[ordinal] != memory_info) ++ordinal;
            if (ordinal == fac->memory_infos.size()) return host.status(ORT_INVALID_ARGUMENT, "CreateAllocator: the memory info is not one this factory registered");
        }
        auto* a = new RocmOrtAllocator();
        std::memset(&a->vtable, 0, sizeof(a->vtable));
        a->vtable.version = ORT_API_VERSION;
        a->vtable.Alloc = allocator_alloc;
        a->vtable.Free = allocator_free;
        a->vtable.Info = allocator_info;
        a->vtable.Reserve = allocator_reserve;
        a->factory = fac;
        a->info = memory_info;
        a->ordinal = static_cast<uint32_t>(ordinal);
        fac->live_allocators.fetch_add(1);
        *out = &a->vtable;
        return nullptr;
    });
}

void ORT_API_CALL factory_release_allocator(OrtEpFactory* f, OrtAllocator* allocator)
{
    if (!allocator) return;
    self(f)->live_allocators.fetch_sub(1);
    delete reinterpret_cast<RocmOrtAllocator*>(allocator);
}

OrtStatus* ORT_API_CALL factory_create_data_transfer(OrtEpFactory* f, OrtDataTransferImpl** out)
{
    RocmOrtFactory* fac = self(f);
    const Host& host = fac->host;
    return guarded(host, "CreateDataTransfer", [&]() -> OrtStatus* {
        if (!out) return host.status(ORT_INVALID_ARGUMENT, "CreateDataTransfer: null output pointer");
        auto* t = new RocmDataTransfer();
        std::memset(&t->vtable, 0, sizeof(t->vtable));
        t->vtable.ort_version_supported = ORT_API_VERSION;
        t->vtable.Release = transfer_release;
        t->vtable.CanCopy = transfer_can_copy;
        t->vtable.CopyTensors = transfer_copy_tensors;
        t->factory = fac;
        fac->live_transfers.fetch_add(1);
        *out = &t->vtable;
        return nullptr;
    });
}

OrtStatus* ORT_API_CALL factory_create_sync_stream(OrtEpFactory* f, const OrtMemoryDevice*, const OrtKeyValuePairs*, OrtSyncStreamImpl** out)
{
    if (out) *out = nullptr;
    return self(f)->host.status(ORT_NOT_IMPLEMENTED, "CreateSyncStreamForDevice: the ROCm execution provider is not stream-aware (IsStreamAware answers false)");
}

}  // namespace

extern "C" {

OrtStatus* CreateEpFactories(const char* registration_name, const OrtApiBase* api_base, const OrtLogger* /*default_logger*/, OrtEpFactory** factories,
                             size_t max_factories, size_t* num_factories)
{
    if (num_factories) *num_factories = 0;
    if (!api_base || !api_base->GetApi) return nullptr;        // no host API: there is nothing to build a status with
#if !defined(NXRT_ORT_REAL_HEADERS)
    // Built against the subset header: OrtApi / OrtEpApi members sit at that header's offsets, not at onnxruntime's. Only a
    // host that announces the same layout is called through them; any other gets no factory and no call into its tables.
    const char* host_version = api_base->GetVersionString ? api_base->GetVersionString() : nullptr;
    if (!host_version || !std::strstr(host_version, ORT_SUBSET_LAYOUT_MARKER)) return nullptr;
#endif
    const OrtApi* api = api_base->GetApi(ORT_API_VERSION);
    if (!api) return nullptr;                                   // the host is older than the API this plugin was built for
    Host host;
    host.api = api;
    host.ep_api = api->GetEpApi ? api->GetEpApi() : nullptr;
    return guarded(host, "CreateEpFactories", [&]() -> OrtStatus* {
        if (!host.ep_api) return host.status(ORT_NOT_IMPLEMENTED, "CreateEpFactories: the host offers no plugin-EP API (GetEpApi)");
        if (!factories || !num_factories || max_factories < 1)
            return host.status(ORT_INVALID_ARGUMENT, "CreateEpFactories: null output pointer or room for no factory");
        auto* fac = new RocmOrtFactory();
        std::memset(&fac->vtable, 0, sizeof(fac->vtable));
        fac->vtable.ort_version_supported = ORT_API_VERSION;
        fac->vtable.GetName = factory_get_name;
        fac->vtable.GetVendor = factory_get_vendor;
        fac->vtable.GetSupportedDevices = factory_get_supported_devices;
        fac->vtable.CreateEp = factory_create_ep;
        fac->vtable.ReleaseEp = factory_release_ep;
        fac->vtable.GetVendorId = factory_get_vendor_id;
        fac->vtable.GetVersion = factory_get_version;
        fac->vtable.ValidateCompiledModelCompatibilityInfo = factory_validate_compiled;
        fac->vtable.CreateAllocator = factory_create_allocator;
        fac->vtable.ReleaseAllocator = factory_release_allocator;
        fac->vtable.CreateDataTransfer = factory_create_data_transfer;
        fac->vtable.IsStreamAware = factory_is_stream_aware;
        fac->vtable.CreateSyncStreamForDevice = factory_create_sync_stream;
        fac->host = host;
        fac->name = (registration_name && registration_name[0]) ? registration_name : kDefaultName;
        for (size_t i = 0; i < max_factories; ++i) factories[i] = nullptr;
        factories[0] = &fac->vtable;
        *num_factories = 1;
        return nullptr;
    });
}

OrtStatus* ReleaseEpFactory(OrtEpFactory* factory)
{
    if (!factory) return nullptr;
    RocmOrtFactory* fac = self(factory);
    const Host host = fac->host;
    return guarded(host, "ReleaseEpFactory", [&]() -> OrtStatus* {
        // The host releases EPs, allocators and data transfers before their factory; one that did not gets the factory
        // kept alive (leaked) rather than a dangling pointer behind a live table.
        if (fac->live_eps.load() != 0 || fac->live_allocators.load() != 0 || fac->live_transfers.load() != 0)
            return host.status(ORT_FAIL, "ReleaseEpFactory: " + std::to_string(fac->live_eps.load()) + " EPs, " + std::to_string(fac->live_allocators.load()) +
                                             " allocators and " + std::to_string(fac->live_transfers.load()) + " data transfers of this factory are still alive; "
                                             "release them first (the factory stays valid)");
        for (OrtMemoryInfo* info : fac->memory_infos) host.api->ReleaseMemoryInfo(info);
        for (auto& kv : fac->providers) nxrt_rocm_ep_release(kv.second);      // kernels still alive hold their own reference
        delete fac;
        return nullptr;
    });
}

}  // extern "C"
