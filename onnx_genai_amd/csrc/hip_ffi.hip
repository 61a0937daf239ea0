// HIP runtime half of hip_ffi.h: device memory, the stream, events. No kernels live here.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstring>
#include <mutex>

#include "hip_ffi.h"
#include "../../include/nxrt_ep_rocm.h"      // NXRT_ROCM_STATIC_SCRATCH_BYTES: the size the public header promises is the size of the array

namespace {
// Scratch for the entry point that may not allocate (rocm_ffi_static_scratch): one array per GPU, part of the code object,
// alive from the moment the library is loaded on a device until the process ends. Host code never uses this name as an
// address - it is a host-side stand-in; the device address is asked for once per device (hipGetSymbolAddress) and kept.
constexpr size_t kStaticScratchBytes = NXRT_ROCM_STATIC_SCRATCH_BYTES;
__device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxScratchDevices = 64;
void* g_scratch_ptr[kMaxScratchDevices] = {};
std::mutex g_scratch_mu;
// Users of one GPU's scratch array are chained on the GPU: each records this event when its launches are enqueued, and a
// user on another stream waits for it first.
hipEvent_t g_scratch_event[kMaxScratchDevices] = {};
hipStream_t g_scratch_last_stream[kMaxScratchDevices] = {};
bool g_scratch_event_recorded[kMaxScratchDevices] = {};
std::mutex g_scratch_use_mu[kMaxScratchDevices];
std::atomic<uint64_t> g_device_allocations{0};

__global__ void fill_u32_kernel(uint32_t* dst, uint32_t value, size_t count)
{
    for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < count; i += static_cast<size_t>(gridDim.x) * blockDim.x) dst[i] = value;
}
// Plain device-to-device copy, 16 bytes per lane per step; also the yardstick that hardware byte counters are scaled by.
__global__ __launch_bounds__(256) void copy_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n16, uint8_t* dst_tail, const uint8_t* src_tail, size_t tail)
{
    for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < n16; i += static_cast<size_t>(gridDim.x) * blockDim.x) dst[i] = src[i];
    if (blockIdx.x == 0 && threadIdx.x < tail) dst_tail[threadIdx.x] = src_tail[threadIdx.x];
}
// Plain read of a buffer, one workgroup of 256 lanes per 16 KiB, four 16-byte loads in flight per lane, nothing written
// unless the xor of everything read is a value it never is: the shortest time any kernel can take to pull these bytes
// from HBM - the yardstick the decode kernels' times are held against.
__global__ __launch_bounds__(256) void read_probe_kernel(const uint4* __restrict__ src, size_t n16, uint32_t* sink)
{
    const size_t base = static_cast<size_t>(blockIdx.x) * 1024 + threadIdx.x;
    uint4 v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = base + i * 256 < n16 ? src[base + i * 256] : make_uint4(0, 0, 0, 0);
    uint32_t x = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) x ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
    if (x == 0x9e3779b9u && sink) *sink = x;
}

// What one CU's LDS moves per clock, by kind of access: every workgroup (one per CU, `waves` waves) repeats eight 16-byte
// accesses per lane and waits for them, `iters` times; lane 0 of each wave notes the cycles it took. MODE 0: ds_read_b128;
// 1: ds_write_b128; 2: global memory straight into LDS (buffer_load_dwordx4 ... lds, from a small buffer that stays in
// cache); 3: even waves read while odd waves write. The tiled kernels' step is sized against these figures.
typedef __attribute__((ext_vector_type(4))) uint32_t lds_u32x4_t;
template <int MODE>
__global__ __launch_bounds__(1024) void lds_probe_kernel(unsigned long long* cycles, const uint32_t* src, int iters)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char probe_smem[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    for (int i = threadIdx.x; i < 16384; i += blockDim.x) reinterpret_cast<uint32_t*>(probe_smem)[i] = i;
    __syncthreads();
    lds_u32x4_t srd;
    const uint64_t base = reinterpret_cast<uint64_t>(src);
    srd.x = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(base));
    srd.y = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(base >> 32));
    srd.z = 1u << 20;
    srd.w = 0x00020000u;
    const uint32_t off = lane * 16;
    lds_u32x4_t acc = {1, 2, 3, 4};
    const int role = MODE == 3 ? (wave & 1) : MODE;
    const unsigned long long t0 = __builtin_readcyclecounter();
    for (int it = 0; it < iters; ++it) {
        if (role == 0) {
            lds_u32x4_t v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t a = (off + ((j + wave) & 7) * 4096 + ((it & 1) << 10)) & 0xfff0;
                asm volatile("ds_read_b128 %0, %1" : "=v"(v[j]) : "v"(a));
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                asm volatile("" ::"v"(v[j]));
                acc.x ^= v[j].x;
            }
        } else if (role == 1) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t a = (off + ((j + wave) & 7) * 4096 + ((it & 1) << 10)) & 0xfff0;
                asm volatile("ds_write_b128 %0, %1" ::"v"(a), "v"(acc));
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t lds = __builtin_amdgcn_readfirstlane((((j + wave) & 7) * 4096 + ((it & 1) << 10)) & 0xffff);
                const uint32_t soff = (j * 1024 + wave * 8192 + blockIdx.x * 131072) & 0xfffff;
                asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" ::"s"(lds), "v"(off), "s"(srd), "s"(soff) : "memory");
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
    }
    const unsigned long long t1 = __builtin_readcyclecounter();
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345) cycles[1000] = 1;
    if (lane == 0) cycles[blockIdx.x * 16 + wave] = t1 - t0;
}
}  // namespace

extern "C" {

int rocm_ffi_lds_probe(int mode, int waves, int iters, double* bytes_per_clock)
{
    if (mode < 0 || mode > 3 || waves < 1 || waves > 16 || iters < 1 || !bytes_per_clock) return static_cast<int>(hipErrorInvalidValue);
    constexpr int kBlocks = 256;
    unsigned long long* dev = nullptr;
    uint32_t* src = nullptr;
    hipError_t e = static_cast<hipError_t>(rocm_ffi_malloc(reinterpret_cast<void**>(&dev), (kBlocks * 16 + 1024) * sizeof(unsigned long long)));
    if (e == hipSuccess) e = static_cast<hipError_t>(rocm_ffi_malloc(reinterpret_cast<void**>(&src), 1u << 21));
    if (e == hipSuccess) e = hipMemset(src, 1, 1u << 21);
    if (e == hipSuccess) {
        const dim3 grid(kBlocks), block(static_cast<unsigned>(waves * 64));
        if (mode == 0) hipLaunchKernelGGL(lds_probe_kernel<0>, grid, block, 65536, nullptr, dev, src, iters);
        else if (mode == 1) hipLaunchKernelGGL(lds_probe_kernel<1>, grid, block, 65536, nullptr, dev, src, iters);
        else if (mode == 2) hipLaunchKernelGGL(lds_probe_kernel<2>, grid, block, 65536, nullptr, dev, src, iters);
        else hipLaunchKernelGGL(lds_probe_kernel<3>, grid, block, 65536, nullptr, dev, src, iters);
        e = hipGetLastError();
    }
    unsigned long long host[16] = {};
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e == hipSuccess) e = hipMemcpy(host, dev, sizeof(host), hipMemcpyDeviceToHost);
    if (dev) (void)rocm_ffi_free(dev);
    if (src) (void)rocm_ffi_free(src);
    if (e != hipSuccess) return static_cast<int>(e);
    unsigned long long longest = 1;
    for (int w = 0; w < waves; ++w) longest = host[w] > longest ? host[w] : longest;
    *bytes_per_clock = static_cast<double>(waves) * iters * 8.0 * 64.0 * 16.0 / static_cast<double>(longest);
    return 0;
}

int rocm_ffi_read_probe(const void* src, size_t bytes, void* sink, rocm_stream_t stream)
{
    const size_t n16 = bytes / 16;
    if (n16 == 0) return 0;
    const size_t blocks = (n16 + 1023) / 1024;
    if (blocks > 0x7fffffffu) return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(read_probe_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<const uint4*>(src), n16,
                       static_cast<uint32_t*>(sink));
    return static_cast<int>(hipGetLastError());
}

const char* rocm_ffi_error_string(int err) { return err < 0 ? "shape not eligible for this kernel" : hipGetErrorString(static_cast<hipError_t>(err)); }
int rocm_ffi_device_count(int* count) { return static_cast<int>(hipGetDeviceCount(count)); }
int rocm_ffi_set_device(int device) { return static_cast<int>(hipSetDevice(device)); }

int rocm_ffi_device_info(int device, char* arch, size_t arch_len, int* compute_units, size_t* total_mem)
{
    hipDeviceProp_t prop;
    const hipError_t e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return static_cast<int>(e);
    if (arch && arch_len) {
        std::strncpy(arch, prop.gcnArchName, arch_len - 1);
        arch[arch_len - 1] = 0;
    }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (total_mem) *total_mem = prop.totalGlobalMem;
    return 0;
}

int rocm_ffi_compute_units(void)
{
    static std::atomic<int> cached[64];
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 256;
    int cus = cached[device].load(std::memory_order_relaxed);
    if (cus > 0) return cus;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0) return 256;
    cached[device].store(cus, std::memory_order_relaxed);
    return cus;
}

int rocm_ffi_malloc(void** ptr, size_t bytes)
{
    g_device_allocations.fetch_add(1);
    return static_cast<int>(hipMalloc(ptr, bytes));
}
uint64_t rocm_ffi_malloc_calls(void) { return g_device_allocations.load(); }

int rocm_ffi_static_scratch(int device, void** ptr, size_t* bytes)
{
    if (!ptr || !bytes || device < 0 || device >= kMaxScratchDevices) return static_cast<int>(hipErrorInvalidValue);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[device]) {
        // every GPU holds its own copy of the array at its own address: ask with that GPU current
        hipError_t e = hipSetDevice(device);
        void* p = nullptr;
        if (e == hipSuccess) e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return static_cast<int>(e);
        if (!p) return static_cast<int>(hipErrorInvalidSymbol);
        hipEvent_t ev = nullptr;
        e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
        if (e != hipSuccess) return static_cast<int>(e);
        g_scratch_event[device] = ev;
        g_scratch_ptr[device] = p;
    }
    *ptr = g_scratch_ptr[device];
    *bytes = kStaticScratchBytes;
    return 0;
}

int rocm_ffi_static_scratch_begin(int device, rocm_stream_t stream)
{
    if (device < 0 || device >= kMaxScratchDevices || !g_scratch_event[device]) return static_cast<int>(hipErrorInvalidValue);
    g_scratch_use_mu[device].lock();
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (g_scratch_event_recorded[device] && g_scratch_last_stream[device] != s) {
        const hipError_t e = hipStreamWaitEvent(s, g_scratch_event[device], 0);
        if (e != hipSuccess) {
            g_scratch_use_mu[device].unlock();
            return static_cast<int>(e);
        }
    }
    return 0;
}

int rocm_ffi_static_scratch_end(int device, rocm_stream_t stream)
{
    if (device < 0 || device >= kMaxScratchDevices || !g_scratch_event[device]) return static_cast<int>(hipErrorInvalidValue);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const hipError_t e = hipEventRecord(g_scratch_event[device], s);
    if (e == hipSuccess) {
        g_scratch_event_recorded[device] = true;
        g_scratch_last_stream[device] = s;
    }
    g_scratch_use_mu[device].unlock();
    return static_cast<int>(e);
}
int rocm_ffi_free(void* ptr) { return static_cast<int>(hipFree(ptr)); }

int rocm_ffi_memcpy_h2d(void* dst, const void* src, size_t bytes, rocm_stream_t stream)
{
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream));
    if (e == hipSuccess) e = hipStreamSynchronize(static_cast<hipStream_t>(stream));
    return static_cast<int>(e);
}

int rocm_ffi_memcpy_d2h(void* dst, const void* src, size_t bytes, rocm_stream_t stream)
{
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream));
    if (e == hipSuccess) e = hipStreamSynchronize(static_cast<hipStream_t>(stream));
    return static_cast<int>(e);
}

int rocm_ffi_memcpy_d2d(void* dst, const void* src, size_t bytes, rocm_stream_t stream)
{
    if (bytes == 0) return 0;
    if (((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15) != 0)
        return static_cast<int>(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)));
    const size_t n16 = bytes / 16, tail = bytes % 16;
    size_t blocks = (n16 + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(copy_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<uint4*>(dst),
                       static_cast<const uint4*>(src), n16, static_cast<uint8_t*>(dst) + n16 * 16, static_cast<const uint8_t*>(src) + n16 * 16, tail);
    return static_cast<int>(hipGetLastError());
}

int rocm_ffi_stream_create(rocm_stream_t* stream)
{
    hipStream_t s = nullptr;
    const hipError_t e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);   // default priority
    *stream = s;
    return static_cast<int>(e);
}

int rocm_ffi_stream_destroy(rocm_stream_t stream) { return static_cast<int>(hipStreamDestroy(static_cast<hipStream_t>(stream))); }
int rocm_ffi_stream_sync(rocm_stream_t stream) { return static_cast<int>(hipStreamSynchronize(static_cast<hipStream_t>(stream))); }

int rocm_ffi_event_create(rocm_event_t* event)
{
    hipEvent_t e = nullptr;
    const hipError_t r = hipEventCreate(&e);
    *event = e;
    return static_cast<int>(r);
}

int rocm_ffi_event_destroy(rocm_event_t event) { return static_cast<int>(hipEventDestroy(static_cast<hipEvent_t>(event))); }
int rocm_ffi_event_record(rocm_event_t event, rocm_stream_t stream) { return static_cast<int>(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream))); }
int rocm_ffi_event_sync(rocm_event_t event) { return static_cast<int>(hipEventSynchronize(static_cast<hipEvent_t>(event))); }
int rocm_ffi_event_elapsed_ms(rocm_event_t start, rocm_event_t stop, float* ms) { return static_cast<int>(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop))); }

int rocm_ffi_fill_u32(void* dst, uint32_t value, size_t count, rocm_stream_t stream)
{
    if (count == 0) return 0;
    size_t blocks = (count + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(fill_u32_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<uint32_t*>(dst), value, count);
    return static_cast<int>(hipGetLastError());
}

int rocm_ffi_capture_begin(rocm_stream_t stream)
{
    return static_cast<int>(hipStreamBeginCapture(static_cast<hipStream_t>(stream), hipStreamCaptureModeThreadLocal));
}

int rocm_ffi_capture_end(rocm_stream_t stream, rocm_graph_exec_t* exec, size_t* num_nodes)
{
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(static_cast<hipStream_t>(stream), &graph);
    if (e != hipSuccess) return static_cast<int>(e);
    if (num_nodes) {
        size_t n = 0;
        (void)hipGraphGetNodes(graph, nullptr, &n);
        *num_nodes = n;
    }
    hipGraphExec_t ge = nullptr;
    e = hipGraphInstantiate(&ge, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    *exec = ge;
    return static_cast<int>(e);
}

int rocm_ffi_graph_launch(rocm_graph_exec_t exec, rocm_stream_t stream)
{
    return static_cast<int>(hipGraphLaunch(static_cast<hipGraphExec_t>(exec), static_cast<hipStream_t>(stream)));
}

int rocm_ffi_graph_destroy(rocm_graph_exec_t exec) { return static_cast<int>(hipGraphExecDestroy(static_cast<hipGraphExec_t>(exec))); }

}  // extern "C"
