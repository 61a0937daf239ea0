// The execution provider object: one GPU, one HIP stream, the buffers it handed out.
#pragma once

#include <atomic>
#include <cstdint>
#include <map>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "status.h"

struct NxrtRocmEp {
    uint32_t device = 0;
    rocm_stream_t stream = nullptr;
    std::string name = "RocmExecutionProvider";
    std::map<std::string, std::string> config;   // EpConfig: a string map
    int acc4_rounding = 0;                        // 0 = ties to even (MLAS), 1 = ties away (native), 2 = by row count
    int acc4_native_below = 0;                    // with 2: calls with fewer rows than this round the native way
    int decode_waves = 0;                         // 0 = chosen per shape
    int decode_col_groups = 0;
    int prefill_tile = 0;                         // 0 = chosen per shape; 1..3 force a tile (tests, tuning)
    int prepack = 1;                              // repack constant weights for the decode kernel on first use
    int rmsnorm_in_kernel_max_cols = 8192;        // widest node (columns the launch covers) whose decode kernel applies an RMS-norm prologue itself; 0 = never
    int dense_gemm_min_rows = 0;                  // calls with at least this many rows expand the weights and run the library GEMM; 0 = never
    uint64_t dense_gemm_max_bytes = 1ull << 30;   // largest dense copy of one weight that route makes
    int dense_resident = 0;                       // 1: a constant weight keeps its dense copy (made once); 0: one shared buffer, refilled per call
    RocmDenseGemm* dense = nullptr;               // library handle + its workspace, made on first use
    void* dense_scratch = nullptr;                // the shared buffer of dense_resident = 0
    size_t dense_scratch_bytes = 0;
    std::vector<void*> dense_retired;             // outgrown shared buffers, kept for graphs recorded while they were current
    std::mutex dense_mu;                          // expansion and GEMM of one call are enqueued back to back under it
    std::mutex mu;
    std::unordered_map<void*, size_t> live;       // allocations handed out and not yet returned
    std::atomic<uint64_t> launches{0};
    void* static_scratch = nullptr;               // this GPU's static scratch array (device address), resolved when the provider is created
    size_t static_scratch_bytes = 0;
    bool capturing = false;                       // a stream capture is open: nothing may allocate or synchronise
    std::atomic<uint64_t> captures{0};            // stream captures opened on this provider so far: while 0, no HIP graph can name a buffer of its kernels
    // The host may release the provider, its kernels and its allocators in any order (each vtable is released exactly
    // once, independently): every kernel object and allocator handle holds one reference, the creator holds the first,
    // and the provider dies with the last.
    std::atomic<uint32_t> refs{1};
    void retain() { refs.fetch_add(1); }
    NxrtEpVtable vtable;                          // ctx points back at this object

    NxrtRocmEp();
    ~NxrtRocmEp();
    NxrtStatus bind() const;                      // make this provider's GPU current on the calling thread
};

struct NxrtRocmGraph {
    rocm_graph_exec_t exec = nullptr;
};

struct NxrtRocmEvent {
    rocm_event_t ev = nullptr;
};

namespace nxrt_rocm {
extern std::atomic<uint64_t> g_live_providers;
void init_ep_vtable(NxrtRocmEp* ep);
}  // namespace nxrt_rocm
