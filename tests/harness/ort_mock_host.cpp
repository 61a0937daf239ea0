// A stand-in for ONNX Runtime's side of the plugin execution-provider API: it loads the library the way ORT's
// RegisterExecutionProviderLibrary does (dlopen, CreateEpFactories / ReleaseEpFactory by name), serves the host functions
// the plugin calls from tables of its own, and walks the lifecycle a session goes through - list devices, create an EP,
// GetCapability over a small graph, Compile, create allocator and data transfer, release everything in the host's order
// and in a wrong one - checking every answer. Without arguments nothing here touches a GPU. With --gpu it also runs one
// compiled node: device tensors from the plugin's allocator, filled through its data transfer, Compute through a mock
// kernel context, the result compared with a double-precision product computed here.
//
// Usage: ort_mock_host <library> [--gpu]
#include <dlfcn.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "ort_plugin_ep_subset.h"

// ---- the host's objects (opaque to the plugin) ----
struct OrtStatus { OrtErrorCode code; std::string message; };
struct OrtHardwareDevice { OrtHardwareDeviceType type; uint32_t vendor, device_id; };
struct OrtMemoryInfo { std::string name; OrtMemoryInfoDeviceType type; uint32_t vendor; int32_t id; };
struct OrtMemoryDevice { OrtMemoryInfoDeviceType type; uint32_t vendor, id; };
struct OrtEpDevice { OrtEpFactory* factory; const OrtHardwareDevice* hw; std::vector<const OrtMemoryInfo*> infos; };
struct OrtTensorTypeAndShapeInfo { ONNXTensorElementDataType type; std::vector<int64_t> dims; };
struct OrtTypeInfo { bool is_tensor; OrtTensorTypeAndShapeInfo tensor; };
struct OrtValueInfo { OrtTypeInfo type; bool constant; };
struct OrtOpAttr { std::string name; int64_t value; };
struct OrtNode { std::string op, domain; std::vector<OrtOpAttr> attrs; std::vector<const OrtValueInfo*> inputs; };
struct OrtGraph { std::vector<const OrtNode*> nodes; };
struct OrtEpGraphSupportInfo { std::vector<std::vector<const OrtNode*>> fused; };
struct OrtValue { OrtTensorTypeAndShapeInfo info; void* data; OrtMemoryDevice device; size_t bytes; };
struct OrtKernelContext { std::vector<const OrtValue*> inputs; OrtValue* output; OrtAllocator* allocator; size_t output_elem_bytes; };

static int g_live_status = 0, g_live_meminfo = 0, g_live_epdev = 0, g_live_shape = 0, g_failures = 0;

#define CHECK(cond)                                                                     \
    do {                                                                                \
        if (!(cond)) {                                                                  \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);               \
            ++g_failures;                                                               \
        }                                                                               \
    } while (0)

static OrtStatus* make_status(OrtErrorCode code, const char* msg)
{
    ++g_live_status;
    return new OrtStatus{code, msg ? msg : ""};
}
static void release_status(OrtStatus* s)
{
    if (s) {
        --g_live_status;
        delete s;
    }
}
// consumes the status; true when it is an error of `code` whose message contains `needle`
static bool is_error(OrtStatus* s, OrtErrorCode code, const char* needle)
{
    const bool ok = s && s->code == code && s->message.find(needle) != std::string::npos;
    if (s && !ok) std::printf("  status %d: %s\n", static_cast<int>(s->code), s->message.c_str());
    release_status(s);
    return ok;
}
static bool is_ok(OrtStatus* s)
{
    if (s) std::printf("  unexpected status %d: %s\n", static_cast<int>(s->code), s->message.c_str());
    const bool ok = s == nullptr;
    release_status(s);
    return ok;
}

// ---- OrtApi ----
static OrtStatus* api_CastTypeInfoToTensorInfo(const OrtTypeInfo* t, const OrtTensorTypeAndShapeInfo** out)
{
    *out = t->is_tensor ? &t->tensor : nullptr;
    return nullptr;
}
static OrtStatus* api_CreateMemoryInfo_V2(const char* name, OrtMemoryInfoDeviceType type, uint32_t vendor, int32_t id, OrtDeviceMemoryType, size_t, OrtAllocatorType,
                                          OrtMemoryInfo** out)
{
    ++g_live_meminfo;
    *out = new OrtMemoryInfo{name, type, vendor, id};
    return nullptr;
}
static OrtStatus* api_GetDimensions(const OrtTensorTypeAndShapeInfo* info, int64_t* dims, size_t n)
{
    if (n < info->dims.size()) return make_status(ORT_INVALID_ARGUMENT, "dims buffer too small");
    for (size_t i = 0; i < info->dims.size(); ++i) dims[i] = info->dims[i];
    return nullptr;
}
static OrtStatus* api_GetDimensionsCount(const OrtTensorTypeAndShapeInfo* info, size_t* out) { *out = info->dims.size(); return nullptr; }
static OrtStatus* api_GetTensorData(const OrtValue* v, const void** out) { *out = v->data; return nullptr; }
static OrtStatus* api_GetTensorElementType(const OrtTensorTypeAndShapeInfo* info, ONNXTensorElementDataType* out) { *out = info->type; return nullptr; }
static OrtStatus* api_GetTensorMutableData(OrtValue* v, void** out) { *out = v->data; return nullptr; }
static OrtStatus* api_GetTensorSizeInBytes(const OrtValue* v, size_t* out) { *out = v->bytes; return nullptr; }
static OrtStatus* api_GetTensorTypeAndShape(const OrtValue* v, OrtTensorTypeAndShapeInfo** out)
{
    ++g_live_shape;
    *out = new OrtTensorTypeAndShapeInfo(v->info);
    return nullptr;
}
static OrtStatus* api_GetValueInfoTypeInfo(const OrtValueInfo* vi, const OrtTypeInfo** out) { *out = &vi->type; return nullptr; }
static OrtStatus* api_Graph_GetNodes(const OrtGraph* g, const OrtNode** nodes, size_t n)
{
    if (n < g->nodes.size()) return make_status(ORT_INVALID_ARGUMENT, "nodes buffer too small");
    for (size_t i = 0; i < g->nodes.size(); ++i) nodes[i] = g->nodes[i];
    return nullptr;
}
static OrtStatus* api_Graph_GetNumNodes(const OrtGraph* g, size_t* out) { *out = g->nodes.size(); return nullptr; }
static uint32_t api_HardwareDevice_DeviceId(const OrtHardwareDevice* d) { return d->device_id; }
static OrtHardwareDeviceType api_HardwareDevice_Type(const OrtHardwareDevice* d) { return d->type; }
static uint32_t api_HardwareDevice_VendorId(const OrtHardwareDevice* d) { return d->vendor; }
static OrtStatus* api_KernelContext_GetInput(const OrtKernelContext* c, size_t i, const OrtValue** out)
{
    *out = i < c->inputs.size() ? c->inputs[i] : nullptr;
    return nullptr;
}
static OrtStatus* api_KernelContext_GetInputCount(const OrtKernelContext* c, size_t* out) { *out = c->inputs.size(); return nullptr; }
static OrtStatus* api_KernelContext_GetOutput(OrtKernelContext* c, size_t index, const int64_t* dims, size_t nd, OrtValue** out)
{
    if (index != 0) return make_status(ORT_INVALID_ARGUMENT, "one output");
    size_t elems = 1;
    for (size_t i = 0; i < nd; ++i) elems *= static_cast<size_t>(dims[i]);
    OrtValue* v = c->output;
    v->info.dims.assign(dims, dims + nd);
    v->bytes = elems * c->output_elem_bytes;
    v->data = c->allocator->Alloc(c->allocator, v->bytes);
    if (!v->data) return make_status(ORT_FAIL, "output allocation failed");
    *out = v;
    return nullptr;
}
static OrtStatus* api_Node_GetAttributeByName(const OrtNode* n, const char* name, const OrtOpAttr** out)
{
    *out = nullptr;
    for (const OrtOpAttr& a : n->attrs)
        if (a.name == name) {
            *out = &a;
            return nullptr;
        }
    return make_status(ORT_FAIL, "attribute not found");       // as the real host: an error status for an absent attribute
}
static OrtStatus* api_Node_GetDomain(const OrtNode* n, const char** out) { *out = n->domain.c_str(); return nullptr; }
static OrtStatus* api_Node_GetInputs(const OrtNode* n, const OrtValueInfo** inputs, size_t count)
{
    if (count < n->inputs.size()) return make_status(ORT_INVALID_ARGUMENT, "inputs buffer too small");
    for (size_t i = 0; i < n->inputs.size(); ++i) inputs[i] = n->inputs[i];
    return nullptr;
}
static OrtStatus* api_Node_GetNumInputs(const OrtNode* n, size_t* out) { *out = n->inputs.size(); return nullptr; }
static OrtStatus* api_Node_GetOperatorType(const OrtNode* n, const char** out) { *out = n->op.c_str(); return nullptr; }
static OrtStatus* api_ReadOpAttr(const OrtOpAttr* a, OrtOpAttrType type, void* data, size_t len, size_t* out)
{
    if (type != ORT_OP_ATTR_INT || len < sizeof(int64_t)) return make_status(ORT_INVALID_ARGUMENT, "int attributes only");
    std::memcpy(data, &a->value, sizeof(int64_t));
    *out = sizeof(int64_t);
    return nullptr;
}
static void api_ReleaseMemoryInfo(OrtMemoryInfo* m)
{
    if (m) {
        --g_live_meminfo;
        delete m;
    }
}
static void api_ReleaseTensorTypeAndShapeInfo(OrtTensorTypeAndShapeInfo* i)
{
    if (i) {
        --g_live_shape;
        delete i;
    }
}
static OrtStatus* api_ValueInfo_IsConstantInitializer(const OrtValueInfo* vi, bool* out) { *out = vi->constant; return nullptr; }

// ---- OrtEpApi ----
static OrtStatus* ep_CreateEpDevice(OrtEpFactory* f, const OrtHardwareDevice* hw, const OrtKeyValuePairs*, const OrtKeyValuePairs*, OrtEpDevice** out)
{
    ++g_live_epdev;
    *out = new OrtEpDevice{f, hw, {}};
    return nullptr;
}
static OrtStatus* ep_EpDevice_AddAllocatorInfo(OrtEpDevice* d, const OrtMemoryInfo* info) { d->infos.push_back(info); return nullptr; }
static OrtStatus* ep_AddNodesToFuse(OrtEpGraphSupportInfo* s, const OrtNode* const* nodes, size_t n, const OrtNodeFusionOptions*)
{
    s->fused.emplace_back(nodes, nodes + n);
    return nullptr;
}
static uint32_t ep_MemoryDevice_GetDeviceId(const OrtMemoryDevice* d) { return d->id; }
static OrtMemoryInfoDeviceType ep_MemoryDevice_GetDeviceType(const OrtMemoryDevice* d) { return d->type; }
static uint32_t ep_MemoryDevice_GetVendorId(const OrtMemoryDevice* d) { return d->vendor; }
static void ep_ReleaseEpDevice(OrtEpDevice* d)
{
    if (d) {
        --g_live_epdev;
        delete d;
    }
}
static const OrtMemoryDevice* ep_Value_GetMemoryDevice(const OrtValue* v) { return &v->device; }

static OrtEpApi g_ep_api;
static OrtApi g_api;
static const OrtEpApi* api_GetEpApi() { return &g_ep_api; }
static const OrtApi* base_GetApi(uint32_t version) { return version <= ORT_API_VERSION ? &g_api : nullptr; }
static const char* base_GetVersionString() { return "1.23.0-mock " ORT_SUBSET_LAYOUT_MARKER; }
// What a real onnxruntime answers: no marker. Its tables must never be touched by a subset build.
static int g_foreign_get_api_calls = 0;
static const OrtApi* foreign_GetApi(uint32_t) { ++g_foreign_get_api_calls; return nullptr; }
static const char* foreign_GetVersionString() { return "1.23.0"; }

static void fill_tables()
{
    g_api.CastTypeInfoToTensorInfo = api_CastTypeInfoToTensorInfo;
    g_api.CreateMemoryInfo_V2 = api_CreateMemoryInfo_V2;
    g_api.CreateStatus = make_status;
    g_api.GetDimensions = api_GetDimensions;
    g_api.GetDimensionsCount = api_GetDimensionsCount;
    g_api.GetEpApi = api_GetEpApi;
    g_api.GetTensorData = api_GetTensorData;
    g_api.GetTensorElementType = api_GetTensorElementType;
    g_api.GetTensorMutableData = api_GetTensorMutableData;
    g_api.GetTensorSizeInBytes = api_GetTensorSizeInBytes;
    g_api.GetTensorTypeAndShape = api_GetTensorTypeAndShape;
    g_api.GetValueInfoTypeInfo = api_GetValueInfoTypeInfo;
    g_api.Graph_GetNodes = api_Graph_GetNodes;
    g_api.Graph_GetNumNodes = api_Graph_GetNumNodes;
    g_api.HardwareDevice_DeviceId = api_HardwareDevice_DeviceId;
    g_api.HardwareDevice_Type = api_HardwareDevice_Type;
    g_api.HardwareDevice_VendorId = api_HardwareDevice_VendorId;
    g_api.KernelContext_GetInput = api_KernelContext_GetInput;
    g_api.KernelContext_GetInputCount = api_KernelContext_GetInputCount;
    g_api.KernelContext_GetOutput = api_KernelContext_GetOutput;
    g_api.Node_GetAttributeByName = api_Node_GetAttributeByName;
    g_api.Node_GetDomain = api_Node_GetDomain;
    g_api.Node_GetInputs = api_Node_GetInputs;
    g_api.Node_GetNumInputs = api_Node_GetNumInputs;
    g_api.Node_GetOperatorType = api_Node_GetOperatorType;
    g_api.ReadOpAttr = api_ReadOpAttr;
    g_api.ReleaseMemoryInfo = api_ReleaseMemoryInfo;
    g_api.ReleaseStatus = release_status;
    g_api.ReleaseTensorTypeAndShapeInfo = api_ReleaseTensorTypeAndShapeInfo;
    g_api.ValueInfo_IsConstantInitializer = api_ValueInfo_IsConstantInitializer;
    g_ep_api.CreateEpDevice = ep_CreateEpDevice;
    g_ep_api.EpDevice_AddAllocatorInfo = ep_EpDevice_AddAllocatorInfo;
    g_ep_api.EpGraphSupportInfo_AddNodesToFuse = ep_AddNodesToFuse;
    g_ep_api.MemoryDevice_GetDeviceId = ep_MemoryDevice_GetDeviceId;
    g_ep_api.MemoryDevice_GetDeviceType = ep_MemoryDevice_GetDeviceType;
    g_ep_api.MemoryDevice_GetVendorId = ep_MemoryDevice_GetVendorId;
    g_ep_api.ReleaseEpDevice = ep_ReleaseEpDevice;
    g_ep_api.Value_GetMemoryDevice = ep_Value_GetMemoryDevice;
}

// ---- a small graph ----
static OrtValueInfo tensor_info(ONNXTensorElementDataType type, std::vector<int64_t> dims, bool constant)
{
    return OrtValueInfo{OrtTypeInfo{true, OrtTensorTypeAndShapeInfo{type, std::move(dims)}}, constant};
}

typedef OrtStatus* (*CreateFn)(const char*, const OrtApiBase*, const OrtLogger*, OrtEpFactory**, size_t, size_t*);
typedef OrtStatus* (*ReleaseFn)(OrtEpFactory*);

int main(int argc, char** argv)
{
    if (argc < 2) {
        std::printf("usage: %s <library> [--gpu]\n", argv[0]);
        return 2;
    }
    const bool gpu = argc > 2 && std::strcmp(argv[2], "--gpu") == 0;
    void* lib = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
    if (!lib) {
        std::printf("dlopen: %s\n", dlerror());
        return 2;
    }
    auto create = reinterpret_cast<CreateFn>(dlsym(lib, "CreateEpFactories"));
    auto release = reinterpret_cast<ReleaseFn>(dlsym(lib, "ReleaseEpFactory"));
    if (!create || !release) {
        std::printf("the library does not export CreateEpFactories / ReleaseEpFactory\n");
        return 2;
    }
    fill_tables();
    const OrtApiBase base{base_GetApi, base_GetVersionString};

    // ---- entry-point argument checks ----
    OrtEpFactory* factories[2] = {reinterpret_cast<OrtEpFactory*>(1), reinterpret_cast<OrtEpFactory*>(1)};
    size_t n = 7;
    CHECK(create("x", nullptr, nullptr, factories, 2, &n) == nullptr && n == 0);                       // no host API: no status to make
    n = 7;
    CHECK(is_error(create("x", &base, nullptr, factories, 0, &n), ORT_INVALID_ARGUMENT, "room for no factory") && n == 0);
    CHECK(is_error(create("x", &base, nullptr, nullptr, 2, &n), ORT_INVALID_ARGUMENT, "null output"));
    CHECK(release(nullptr) == nullptr);
    // a host that does not announce the subset layout (a real onnxruntime): no factory, and not one call into its tables
    const OrtApiBase real_host{foreign_GetApi, foreign_GetVersionString};
    n = 7;
    factories[0] = reinterpret_cast<OrtEpFactory*>(1);
    CHECK(create("x", &real_host, nullptr, factories, 2, &n) == nullptr && n == 0 && g_foreign_get_api_calls == 0);
    CHECK(factories[0] == reinterpret_cast<OrtEpFactory*>(1));

    // ---- a factory under the default name and one under the registration name ----
    CHECK(is_ok(create(nullptr, &base, nullptr, factories, 2, &n)) && n == 1 && factories[1] == nullptr);
    OrtEpFactory* named = factories[0];
    CHECK(std::strcmp(named->GetName(named), "RocmExecutionProvider") == 0);
    CHECK(is_ok(release(named)));
    CHECK(is_ok(create("my_rocm", &base, nullptr, factories, 1, &n)) && n == 1);
    OrtEpFactory* f = factories[0];
    CHECK(f->ort_version_supported == ORT_API_VERSION);
    CHECK(std::strcmp(f->GetName(f), "my_rocm") == 0 && std::strcmp(f->GetVendor(f), "nxrt") == 0 && f->GetVendorId(f) == 0x1002);
    CHECK(std::strlen(f->GetVersion(f)) > 0 && !f->IsStreamAware(f));
    OrtSyncStreamImpl* stream = reinterpret_cast<OrtSyncStreamImpl*>(1);
    CHECK(is_error(f->CreateSyncStreamForDevice(f, nullptr, nullptr, &stream), ORT_NOT_IMPLEMENTED, "not stream-aware") && stream == nullptr);
    OrtCompiledModelCompatibility compat = OrtCompiledModelCompatibility_EP_UNSUPPORTED;
    CHECK(is_ok(f->ValidateCompiledModelCompatibilityInfo(f, nullptr, 0, "anything", &compat)) && compat == OrtCompiledModelCompatibility_EP_NOT_APPLICABLE);

    // ---- devices: only the AMD GPUs, in the host's order ----
    const OrtHardwareDevice cpu{OrtHardwareDeviceType_CPU, 0x8086, 1}, nvidia{OrtHardwareDeviceType_GPU, 0x10de, 2}, amd_a{OrtHardwareDeviceType_GPU, 0x1002, 0x75a3},
        amd_b{OrtHardwareDeviceType_GPU, 0x1002, 0x75a3}, amd_npu{OrtHardwareDeviceType_NPU, 0x1002, 9};
    const OrtHardwareDevice* hw[] = {&cpu, &nvidia, &amd_a, &amd_npu, &amd_b};
    OrtEpDevice* ep_devices[4] = {};
    size_t n_dev = 9;
    CHECK(is_ok(f->GetSupportedDevices(f, hw, 5, ep_devices, 1, &n_dev)) && n_dev == 1 && ep_devices[0]->hw == &amd_a);
    ep_ReleaseEpDevice(ep_devices[0]);
    CHECK(is_ok(f->GetSupportedDevices(f, hw, 5, ep_devices, 4, &n_dev)) && n_dev == 2);
    CHECK(ep_devices[0]->hw == &amd_a && ep_devices[1]->hw == &amd_b && ep_devices[0]->factory == f);
    CHECK(ep_devices[0]->infos.size() == 1 && ep_devices[0]->infos[0]->id == 0 && ep_devices[1]->infos[0]->id == 1);
    CHECK(ep_devices[1]->infos[0]->type == OrtMemoryInfoDeviceType_GPU && ep_devices[1]->infos[0]->vendor == 0x1002);
    CHECK(g_live_meminfo == 2);                                                                       // asked twice, registered once per GPU
    CHECK(is_error(f->GetSupportedDevices(f, hw, 5, ep_devices, 4, nullptr), ORT_INVALID_ARGUMENT, "null argument"));

    // ---- EP creation ----
    OrtEp* ep = reinterpret_cast<OrtEp*>(1);
    const OrtHardwareDevice* one[] = {&amd_b};
    const OrtHardwareDevice* two[] = {&amd_a, &amd_b};
    const OrtHardwareDevice* foreign[] = {&nvidia};
    CHECK(is_error(f->CreateEp(f, two, nullptr, 2, nullptr, nullptr, &ep), ORT_INVALID_ARGUMENT, "exactly one GPU") && ep == nullptr);
    CHECK(is_error(f->CreateEp(f, foreign, nullptr, 1, nullptr, nullptr, &ep), ORT_INVALID_ARGUMENT, "not offered"));
    CHECK(is_ok(f->CreateEp(f, one, nullptr, 1, nullptr, nullptr, &ep)) && ep != nullptr);
    CHECK(ep->ort_version_supported == ORT_API_VERSION && std::strcmp(ep->GetName(ep), "my_rocm") == 0);

    // ---- GetCapability ----
    const int64_t K = 256, N = 64, BS = 32, KB = K / BS;
    const OrtValueInfo a16 = tensor_info(ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT16, {-1, K}, false), a32 = tensor_info(ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT, {-1, K}, false);
    const OrtValueInfo b8 = tensor_info(ONNX_TENSOR_ELEMENT_DATA_TYPE_UINT8, {N, KB, BS / 2}, true);
    const OrtValueInfo s16 = tensor_info(ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT16, {N, KB}, true), s32 = tensor_info(ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT, {N, KB}, true);
    const OrtValueInfo zp8 = tensor_info(ONNX_TENSOR_ELEMENT_DATA_TYPE_UINT8, {N, KB / 2}, true), zp16 = tensor_info(ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT16, {N, KB}, true);
    const OrtValueInfo g32 = tensor_info(ONNX_TENSOR_ELEMENT_DATA_TYPE_INT32, {K}, true), g64 = tensor_info(ONNX_TENSOR_ELEMENT_DATA_TYPE_INT64, {K}, true);
    const OrtValueInfo bias32 = tensor_info(ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT, {N}, true);
    const OrtValueInfo not_a_tensor{OrtTypeInfo{false, {}}, false};
    auto attrs = [&](int64_t bits, std::vector<OrtOpAttr> more = {}) {
        std::vector<OrtOpAttr> a{{"K", K}, {"N", N}, {"bits", bits}, {"block_size", BS}};
        a.insert(a.end(), more.begin(), more.end());
        return a;
    };
    const OrtNode plain16{"MatMulNBits", "com.microsoft", attrs(4), {&a16, &b8, &s16, &zp8}};
    const OrtNode relu{"Relu", "", {}, {&a16}};
    const OrtNode float_zero_points{"MatMulNBits", "com.microsoft", attrs(4), {&a16, &b8, &s16, &zp16}};
    const OrtNode three_bits{"MatMulNBits", "com.microsoft", attrs(3), {&a16, &b8, &s16}};
    const OrtNode other_domain{"MatMulNBits", "", attrs(4), {&a16, &b8, &s16}};
    const OrtNode full32{"MatMulNBits", "com.microsoft", attrs(4), {&a32, &b8, &s32, nullptr, &g32, &bias32}};
    const OrtNode prepacked{"MatMulNBits", "com.microsoft", attrs(4, {{"weight_prepacked", 1}}), {&a16, &b8, &s16}};
    const OrtNode acc4_g_idx{"MatMulNBits", "com.microsoft", attrs(4, {{"accuracy_level", 4}}), {&a32, &b8, &s32, nullptr, &g32}};
    const OrtNode wide_g_idx{"MatMulNBits", "com.microsoft", attrs(4), {&a32, &b8, &s32, nullptr, &g64}};
    const OrtNode sequence_input{"MatMulNBits", "com.microsoft", attrs(4), {&not_a_tensor, &b8, &s16}};
    const OrtNode no_scales{"MatMulNBits", "com.microsoft", attrs(4), {&a16, &b8}};
    const OrtNode acc4{"MatMulNBits", "com.microsoft", attrs(4, {{"accuracy_level", 4}}), {&a16, &b8, &s16, &zp8}};
    const OrtGraph graph{{&plain16, &relu, &float_zero_points, &three_bits, &other_domain, &full32, &prepacked, &acc4_g_idx, &wide_g_idx, &sequence_input, &no_scales, &acc4}};
    OrtEpGraphSupportInfo support;
    CHECK(is_ok(ep->GetCapability(ep, &graph, &support)));
    CHECK(support.fused.size() == 3);
    if (support.fused.size() == 3) {
        CHECK(support.fused[0].size() == 1 && support.fused[0][0] == &plain16);
        CHECK(support.fused[1].size() == 1 && support.fused[1][0] == &full32);
        CHECK(support.fused[2].size() == 1 && support.fused[2][0] == &acc4);
    }
    CHECK(is_error(ep->GetCapability(ep, nullptr, &support), ORT_INVALID_ARGUMENT, "null argument"));
    const OrtGraph empty{{}};
    OrtEpGraphSupportInfo none;
    CHECK(is_ok(ep->GetCapability(ep, &empty, &none)) && none.fused.empty());

    // ---- Compile ----
    const OrtGraph g_plain{{&plain16}}, g_full{{&full32}}, g_two{{&plain16, &full32}}, g_relu{{&relu}}, g_bits{{&three_bits}};
    const OrtGraph* graphs[] = {&g_plain, &g_full};
    const OrtNode* fused_nodes[] = {&plain16, &full32};
    OrtNodeComputeInfo* infos[2] = {};
    CHECK(is_ok(ep->Compile(ep, graphs, fused_nodes, 2, infos, nullptr)) && infos[0] && infos[1] && infos[0] != infos[1]);
    CHECK(infos[0]->ort_version_supported == ORT_API_VERSION && infos[0]->CreateState && infos[0]->Compute && infos[0]->ReleaseState);
    OrtNodeComputeInfo* rejected[1] = {};
    const OrtGraph* bad_graph[] = {&g_two};
    CHECK(is_error(ep->Compile(ep, bad_graph, fused_nodes, 1, rejected, nullptr), ORT_EP_FAIL, "has 2 nodes") && rejected[0] == nullptr);
    bad_graph[0] = &g_relu;
    CHECK(is_error(ep->Compile(ep, bad_graph, fused_nodes, 1, rejected, nullptr), ORT_EP_FAIL, "not a com.microsoft::MatMulNBits"));
    bad_graph[0] = &g_bits;
    CHECK(is_error(ep->Compile(ep, bad_graph, fused_nodes, 1, rejected, nullptr), ORT_INVALID_ARGUMENT, "bits") && rejected[0] == nullptr);

    // ---- allocator and data transfer ----
    OrtAllocator* allocator = nullptr;
    const OrtMemoryInfo foreign_info{"Cuda", OrtMemoryInfoDeviceType_GPU, 0x10de, 0};
    CHECK(is_error(f->CreateAllocator(f, &foreign_info, nullptr, &allocator), ORT_INVALID_ARGUMENT, "not one this factory registered") && allocator == nullptr);
    CHECK(is_ok(f->CreateAllocator(f, ep_devices[1]->infos[0], nullptr, &allocator)) && allocator);
    CHECK(allocator->Info(allocator) == ep_devices[1]->infos[0] && allocator->Alloc && allocator->Free && allocator->Reserve);
    OrtDataTransferImpl* transfer = nullptr;
    CHECK(is_ok(f->CreateDataTransfer(f, &transfer)) && transfer);
    const OrtMemoryDevice host_mem{OrtMemoryInfoDeviceType_CPU, 0, 0}, rocm_mem{OrtMemoryInfoDeviceType_GPU, 0x1002, 0}, cuda_mem{OrtMemoryInfoDeviceType_GPU, 0x10de, 0};
    CHECK(transfer->CanCopy(transfer, &host_mem, &rocm_mem) && transfer->CanCopy(transfer, &rocm_mem, &host_mem) && transfer->CanCopy(transfer, &rocm_mem, &rocm_mem));
    CHECK(!transfer->CanCopy(transfer, &host_mem, &host_mem) && !transfer->CanCopy(transfer, &cuda_mem, &host_mem) && !transfer->CanCopy(transfer, &rocm_mem, &cuda_mem));

    // ---- one compiled node on the GPU ----
    if (gpu) {
        // GPU ordinal 0 carries the work: a second EP on the first AMD device, its allocator, the full32 node without g_idx
        const OrtHardwareDevice* first[] = {&amd_a};
        OrtEp* ep0 = nullptr;
        OrtAllocator* alloc0 = nullptr;
        CHECK(is_ok(f->CreateEp(f, first, nullptr, 1, nullptr, nullptr, &ep0)));
        CHECK(is_ok(f->CreateAllocator(f, ep_devices[0]->infos[0], nullptr, &alloc0)));
        const OrtNode node{"MatMulNBits", "com.microsoft", attrs(4), {&a32, &b8, &s32, &zp8, nullptr, &bias32}};
        const OrtGraph g_node{{&node}};
        const OrtGraph* gs[] = {&g_node};
        const OrtNode* fn[] = {&node};
        OrtNodeComputeInfo* info[1] = {};
        CHECK(is_ok(ep0->Compile(ep0, gs, fn, 1, info, nullptr)));
        void* state = nullptr;
        CHECK(is_ok(info[0]->CreateState(info[0], nullptr, &state)) && state);
        const int64_t M = 3;
        std::vector<float> a(M * K), scales(N * KB), bias(N);
        std::vector<uint8_t> b(N * KB * BS / 2), zp(N * KB / 2);
        uint32_t seed = 12345;
        auto next = [&]() { seed = seed * 1664525u + 1013904223u; return seed >> 8; };
        for (float& v : a) v = static_cast<float>(next() % 2001) / 1000.0f - 1.0f;
        for (float& v : scales) v = 0.002f + static_cast<float>(next() % 800) / 100000.0f;
        for (float& v : bias) v = static_cast<float>(next() % 2001) / 1000.0f - 1.0f;
        for (uint8_t& v : b) v = static_cast<uint8_t>(next());
        for (uint8_t& v : zp) v = static_cast<uint8_t>(next());
        auto device_tensor = [&](ONNXTensorElementDataType type, std::vector<int64_t> dims, const void* src, size_t bytes) {
            auto* v = new OrtValue{OrtTensorTypeAndShapeInfo{type, std::move(dims)}, alloc0->Alloc(alloc0, bytes), rocm_mem, bytes};
            CHECK(v->data != nullptr);
            OrtValue from{v->info, const_cast<void*>(src), host_mem, bytes};
            const OrtValue* srcs[] = {&from};
            OrtValue* dsts[] = {v};
            CHECK(is_ok(transfer->CopyTensors(transfer, srcs, dsts, nullptr, 1)));
            return v;
        };
        OrtValue* va = device_tensor(ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT, {M, K}, a.data(), a.size() * 4);
        OrtValue* vb = device_tensor(ONNX_TENSOR_ELEMENT_DATA_TYPE_UINT8, {N, KB, BS / 2}, b.data(), b.size());
        OrtValue* vs = device_tensor(ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT, {N, KB}, scales.data(), scales.size() * 4);
        OrtValue* vz = device_tensor(ONNX_TENSOR_ELEMENT_DATA_TYPE_UINT8, {N, KB / 2}, zp.data(), zp.size());
        OrtValue* vbias = device_tensor(ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT, {N}, bias.data(), bias.size() * 4);
        OrtValue y{OrtTensorTypeAndShapeInfo{ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT, {}}, nullptr, rocm_mem, 0};
        OrtKernelContext ctx{{va, vb, vs, vz, nullptr, vbias}, &y, alloc0, 4};
        CHECK(is_ok(info[0]->Compute(info[0], state, &ctx)));
        CHECK(y.info.dims.size() == 2 && y.info.dims[0] == M && y.info.dims[1] == N && y.bytes == static_cast<size_t>(M * N * 4));
        std::vector<float> got(M * N, 0.f);
        OrtValue to{y.info, got.data(), host_mem, y.bytes};
        const OrtValue* srcs[] = {&y};
        OrtValue* dsts[] = {&to};
        CHECK(is_ok(transfer->CopyTensors(transfer, srcs, dsts, nullptr, 1)));
        double num = 0, den = 0;
        for (int64_t m = 0; m < M; ++m)
            for (int64_t col = 0; col < N; ++col) {
                double want = bias[col];
                for (int64_t k = 0; k < K; ++k) {
                    const int64_t blk = k / BS;
                    const int q = (b[(col * KB + blk) * (BS / 2) + (k % BS) / 2] >> ((k & 1) * 4)) & 15;      // low nibble first
                    const int z = (zp[col * (KB / 2) + blk / 2] >> ((blk & 1) * 4)) & 15;
                    want += static_cast<double>(a[m * K + k]) * static_cast<double>(static_cast<float>(q - z) * scales[col * KB + blk]);
                }
                num += (got[m * N + col] - want) * (got[m * N + col] - want);
                den += want * want;
            }
        const double rel = std::sqrt(num / den);
        std::printf("compute through the ORT tables: rel-L2 %.3g against the double-precision product\n", rel);
        CHECK(rel <= 1e-5);
        // a tensor in host memory is refused, not read
        OrtValue host_a{va->info, a.data(), host_mem, va->bytes};
        OrtKernelContext bad{{&host_a, vb, vs, vz, nullptr, vbias}, &y, alloc0, 4};
        CHECK(is_error(info[0]->Compute(info[0], state, &bad), ORT_INVALID_ARGUMENT, "not in ROCm device memory"));
        // nor is one that another AMD GPU holds
        const OrtMemoryDevice other_gpu{OrtMemoryInfoDeviceType_GPU, 0x1002, 5};
        OrtValue far_a{va->info, va->data, other_gpu, va->bytes};
        OrtKernelContext far{{&far_a, vb, vs, vz, nullptr, vbias}, &y, alloc0, 4};
        CHECK(is_error(info[0]->Compute(info[0], state, &far), ORT_INVALID_ARGUMENT, "lives on GPU 5"));
        alloc0->Free(alloc0, y.data);
        for (OrtValue* v : {va, vb, vs, vz, vbias}) {
            alloc0->Free(alloc0, v->data);
            delete v;
        }
        info[0]->ReleaseState(info[0], state);
        ep0->ReleaseNodeComputeInfos(ep0, info, 1);
        CHECK(info[0] == nullptr);
        f->ReleaseAllocator(f, alloc0);
        f->ReleaseEp(f, ep0);
    }

    // ---- release: the factory refuses to go while its objects live, then goes last ----
    CHECK(is_error(release(f), ORT_FAIL, "still alive"));
    CHECK(std::strcmp(f->GetName(f), "my_rocm") == 0);                      // still valid
    ep->ReleaseNodeComputeInfos(ep, infos, 2);
    CHECK(infos[0] == nullptr && infos[1] == nullptr);
    f->ReleaseEp(f, ep);
    f->ReleaseAllocator(f, allocator);
    CHECK(is_error(release(f), ORT_FAIL, "1 data transfers"));
    transfer->Release(transfer);
    ep_ReleaseEpDevice(ep_devices[0]);
    ep_ReleaseEpDevice(ep_devices[1]);
    CHECK(is_ok(release(f)));
    CHECK(g_live_status == 0 && g_live_meminfo == 0 && g_live_epdev == 0 && g_live_shape == 0);
    if (g_live_status || g_live_meminfo || g_live_epdev || g_live_shape)
        std::printf("  live: %d statuses, %d memory infos, %d ep devices, %d shape infos\n", g_live_status, g_live_meminfo, g_live_epdev, g_live_shape);

    dlclose(lib);
    if (g_failures) {
        std::printf("%d checks failed\n", g_failures);
        return 1;
    }
    std::printf("ort plugin lifecycle ok%s\n", gpu ? " (with compute)" : "");
    return 0;
}
