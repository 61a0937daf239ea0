// The execution provider object: one GPU, one HIP stream, the buffers it handed out.
#pragma once

#include <atomic>
#include <cstdint>
#include <map>
#include <mutex>
#include <string>
#include <unordered_map>

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
    std::mutex mu;
    std::unordered_map<void*, size_t> live;       // allocations handed out and not yet returned
    std::atomic<uint64_t> launches{0};
    bool capturing = false;                       // a stream capture is open: nothing may allocate or synchronise
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
