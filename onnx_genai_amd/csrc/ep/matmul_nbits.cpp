// KernelFactory + Kernel for com.microsoft::MatMulNBits on the ROCm provider.
// Attribute parsing, input validation and their messages follow the reference's CPU kernel
// (crates/onnx-runtime-ep-cpu/src/kernels/matmul_nbits.rs:1410-1600, helpers at :10254-10378);
// the contiguity rule follows its CUDA sibling (crates/onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:7089-7106).
#include <cstddef>
#include <mutex>
#include <string>
#include <vector>

#include "provider.h"

using namespace nxrt_rocm;

namespace {

enum AttrBit { kAttrK = 0, kAttrN = 1, kAttrBits = 2, kAttrBlockSize = 3, kAttrAccuracy = 4, kAttrPrepacked = 5, kAttrFoldedBias = 6, kAttrGateUpSwiglu = 7, kAttrDecomposedSilu = 8, kAttrRmsnormPrologue = 9, kAttrRmsnormEpsilon = 10 };

std::string err(const std::string& message) { return "MatMulNBits: " + message; }   // matmul_nbits.rs:10376

const char* dtype_name(uint32_t dt)
{
    switch (dt) {
        case 0: return "Undefined";
        case 1: return "Float32";
        case 2: return "Uint8";
        case 3: return "Int8";
        case 4: return "Uint16";
        case 5: return "Int16";
        case 6: return "Int32";
        case 7: return "Int64";
        case 8: return "String";
        case 9: return "Bool";
        case 10: return "Float16";
        case 11: return "Float64";
        case 12: return "Uint32";
        case 13: return "Uint64";
        case 16: return "BFloat16";
        default: return "Unknown";
    }
}

std::string shape_str(const uint64_t* shape, uint32_t ndim)
{
    std::string s = "[";
    for (uint32_t i = 0; i < ndim; ++i) {
        if (i) s += ", ";
        s += std::to_string(shape[i]);
    }
    return s + "]";
}

std::string shape_str(const std::vector<uint64_t>& v) { return shape_str(v.data(), static_cast<uint32_t>(v.size())); }

bool is_float_compute(uint32_t dt) { return dt == NXRT_DT_FLOAT32 || dt == NXRT_DT_FLOAT16 || dt == NXRT_DT_BFLOAT16; }

bool shape_is(const NxrtRocmTensorView& v, const std::vector<uint64_t>& want)
{
    if (v.ndim != want.size()) return false;
    for (uint32_t i = 0; i < v.ndim; ++i)
        if (v.shape[i] != want[i]) return false;
    return true;
}

bool is_contiguous(const NxrtRocmTensorView& v)
{
    if (!v.strides) return true;
    int64_t expect = 1;
    for (int i = static_cast<int>(v.ndim) - 1; i >= 0; --i) {
        if (v.shape[i] != 1 && v.strides[i] != expect) return false;
        expect *= static_cast<int64_t>(v.shape[i]);
    }
    return true;
}

struct Check {
    std::string message;
    bool failed = false;
    void fail(const std::string& m)
    {
        if (!failed) {
            failed = true;
            message = err(m);
        }
    }
};

// matmul_nbits.rs:10258-10277 + 1410-1445
void check_attrs(const NxrtRocmMatMulNBitsAttrs& a, Check& c)
{
    auto required_positive = [&](int bit, const char* name, int64_t value) {
        if (!(a.present & (1u << bit))) return c.fail(std::string("missing required integer attribute '") + name + "'");
        if (value <= 0) c.fail(std::string("attribute '") + name + "' must be positive, got " + std::to_string(value));
    };
    required_positive(kAttrK, "K", a.K);
    if (c.failed) return;
    required_positive(kAttrN, "N", a.N);
    if (c.failed) return;
    const int64_t bits = (a.present & (1u << kAttrBits)) ? a.bits : 4;
    if (bits != 2 && bits != 4 && bits != 8) {                     // the widths the CPU provider takes (matmul_nbits.rs:1424-1431)
        c.failed = true;
        c.message = "MatMulNBits ROCm supports bits in {2, 4, 8}, got bits=" + std::to_string(bits) +
                    ". Why: only these packed layouts have gfx950 kernels. How to fix: export bits=4 (the tuned path), 2 or 8, "
                    "or select the CPU execution provider for this node";
        return;
    }
    const int64_t accuracy = (a.present & (1u << kAttrAccuracy)) ? a.accuracy_level : 0;
    if (bits != 4 && accuracy == 4) {
        c.failed = true;
        c.message = "MatMulNBits ROCm: accuracy_level=4 is implemented for bits=4 only, got bits=" + std::to_string(bits) +
                    ". How to fix: use accuracy_level=0 with this bit width, or run this node on the CPU execution provider";
        return;
    }
    const int64_t prepacked = (a.present & (1u << kAttrPrepacked)) ? a.weight_prepacked : 0;
    if (prepacked != 0 && prepacked != 1)
        return c.fail("weight_prepacked must be 0 (standard ONNX layout) or 1 (MLAS SQNBit packed layout), got " + std::to_string(prepacked));
    if (prepacked == 1)
        return c.fail("weight_prepacked=1 holds the MLAS SQNBit CPU layout; the ROCm execution provider takes the standard ONNX layout (weight_prepacked=0)");
    required_positive(kAttrBlockSize, "block_size", a.block_size);
    if (c.failed) return;
    if (a.block_size < 16 || (a.block_size & (a.block_size - 1)) != 0)
        c.fail("block_size must be a power of two and at least 16, got " + std::to_string(a.block_size));
}

}  // namespace

struct NxrtRocmMatMulNBits {
    NxrtRocmEp* ep = nullptr;
    int64_t k = 0, n = 0, block_size = 0, accuracy_level = 0;
    int64_t bits = 4;                    // 2 and 8 run on the plain kernels (and the dense route), 4 on everything
    int64_t rows_hint = -1;              // M when the create-time shape of A was static
    bool bias_post_round = false;        // the bias is a folded Add: round(round(acc) + bias) on 16-bit outputs
    // The fused gate/up node: two ordinary kernels (each with its own repacked copy, scratch and variant) whose 16-bit
    // results meet in the silu(gate) * up epilogue.
    bool gate_up_swiglu = false, decomposed_silu = false;
    NxrtRocmMatMulNBits* gate = nullptr;
    NxrtRocmMatMulNBits* up = nullptr;
    bool pair_member = false;            // this kernel is one projection of a fused gate/up node
    const void* g_idx_checked = nullptr; // the g_idx tensor whose groups were found in range
    int32_t* acc_probe = nullptr;        // accuracy_level 4: where the int8 matrix-core kernels also store their block accumulators (tests)
    uint64_t acc_probe_elems = 0;
    // RMS-normalization prologue: the activations are normalized into `norm` first (gamma at input 6, or 5 of the fused node)
    bool rmsnorm_prologue = false;
    float rmsnorm_epsilon = 1e-5f;
    void* norm = nullptr;
    size_t norm_bytes = 0;
    std::mutex norm_mu;                  // held across a normalized call: `norm` feeds the kernels enqueued under it
    bool constant_inputs[6] = {false, false, false, false, false, false};
    std::string variant = "none";
    uint64_t last_flops = 0, last_bytes = 0;   // of the last plain MatMulNBits call: what the CPU provider's record_kernel_metrics notes (matmul_nbits.rs:1588-1597)
    void* scratch = nullptr;             // kernel-owned workspace, grown on demand
    size_t scratch_bytes = 0;
    std::vector<void*> retired;          // outgrown workspaces: kept until the kernel dies, since a HIP graph recorded earlier may still name them
    void* packed = nullptr;              // constant B / scales / zero points in the decode kernel's streaming order
    const void* packed_from[3] = {nullptr, nullptr, nullptr};   // the tensors `packed` was made from
    int packed_scale_dtype = 0;
    void* dense = nullptr;               // constant weights expanded to the activations' 16-bit type, [N, K] (dense_weights = resident)
    const void* dense_from[3] = {nullptr, nullptr, nullptr};
    int dense_dtype = 0, dense_scale_dtype = 0;
    std::mutex mu;                       // one execute at a time per kernel object: scratch, repacked copy and variant are per-object state
    bool no_alloc = false;               // the call in progress (under `mu`) may not allocate or free device memory
    NxrtKernelVtable vtable;
    uint32_t vt_a_dtype = 0, vt_scale_dtype = 0, vt_y_dtype = 0;

    explicit NxrtRocmMatMulNBits(NxrtRocmEp* provider) : ep(provider) { ep->retain(); }     // the kernel keeps its provider alive
    NxrtRocmMatMulNBits(const NxrtRocmMatMulNBits&) = delete;
    NxrtRocmMatMulNBits& operator=(const NxrtRocmMatMulNBits&) = delete;

    ~NxrtRocmMatMulNBits()
    {
        delete gate;
        delete up;
        if ((scratch || packed || dense || norm || !retired.empty()) && ep->bind().code == NXRT_OK) {
            rocm_ffi_stream_sync(ep->stream);
            if (norm) rocm_ffi_free(norm);
            for (void* old : retired) rocm_ffi_free(old);
            if (scratch) rocm_ffi_free(scratch);
            if (packed) rocm_ffi_free(packed);
            if (dense) rocm_ffi_free(dense);
        }
        nxrt_rocm_ep_release(ep);
    }
};

namespace {

// True while nothing may allocate, free or synchronise: a graph capture is open, or the call came in through the entry point
// that allocates nothing.
bool frozen(const NxrtRocmMatMulNBits& kn) { return kn.ep->capturing || kn.no_alloc; }

// Scratch of accuracy_level=4 for M rows: int8 codes, (scale, code sum) pairs, and a block-major copy of the
// pairs (M <= 16) or of the scales (M > 16) for the matrix-core kernels.
// Last comes room for the f32 partial sums of a tiled call that cuts K into slices (small grids only).
struct Acc4Layout { uint64_t codes, pairs, aux, partial, total; };
Acc4Layout acc4_layout(const NxrtRocmMatMulNBits& kn, uint64_t m)
{
    const uint64_t kb = (kn.k + kn.block_size - 1) / kn.block_size;
    Acc4Layout l;
    l.codes = (m * kb * kn.block_size + 255) / 256 * 256;
    l.pairs = (m * kb * 8 + 255) / 256 * 256;
    l.aux = (kb * (m > 32 ? m : 32) * 4 + 255) / 256 * 256;
    RocmMatMulNBitsArgs probe;
    std::memset(&probe, 0, sizeof(probe));
    probe.m = static_cast<int64_t>(m);
    probe.n = kn.n;
    probe.k = kn.k;
    probe.block_size = static_cast<int>(kn.block_size);
    l.partial = (rocm_acc4_mfma_scratch_bytes(&probe) + 255) / 256 * 256;
    l.total = l.codes + l.pairs + l.aux + l.partial;
    return l;
}
uint64_t acc4_workspace_bytes(const NxrtRocmMatMulNBits& kn, uint64_t m) { return acc4_layout(kn, m).total; }

// Replaces an owned device buffer by a larger one. The old buffer is not freed but retired: a HIP graph recorded while
// it was current would otherwise write through a dangling pointer on its next replay. Returns the HIP error code.
int grow_buffer(void*& buf, size_t& bytes, uint64_t need, std::vector<void*>& retired)
{
    void* fresh = nullptr;
    const int e = rocm_ffi_malloc(&fresh, need);
    if (e != 0) return e;
    if (buf) retired.push_back(buf);
    buf = fresh;
    bytes = static_cast<size_t>(need);
    return 0;
}

// A copy of the weights (repacked or dense) that a call with other weights has replaced. Once the provider has recorded a
// HIP graph, a graph may still replay through the copy, so it is kept until the kernel dies. Before that, nothing can name
// it after the stream has drained, and it is freed: a host that alternates a node between weight sets without recording
// graphs holds one copy, not one per switch. (Never called while frozen.)
void drop_weight_copy(NxrtRocmMatMulNBits& kn, void* old)
{
    if (kn.ep->captures.load() != 0) {
        kn.retired.push_back(old);
        return;
    }
    rocm_ffi_stream_sync(kn.ep->stream);
    rocm_ffi_free(old);
}

// True when the call can run on the repacked copy of constant weights; makes that copy on first use (never while a
// graph capture is open: a capture may neither allocate nor should it record the one-time repack). `rc` receives a
// HIP error of the repack.
bool use_packed(NxrtRocmMatMulNBits& kn, const RocmMatMulNBitsArgs& args, int& rc)
{
    rc = 0;
    if (!kn.ep->prepack || !kn.constant_inputs[1] || !kn.constant_inputs[2] || (args.zp && !kn.constant_inputs[3])) return false;
    if (!(kn.accuracy_level == 4 ? rocm_acc4_packed_eligible(&args) : rocm_decode_packed_eligible(&args))) return false;
    const bool current = kn.packed && kn.packed_from[0] == args.b && kn.packed_from[1] == args.scales && kn.packed_from[2] == args.zp &&
                         kn.packed_scale_dtype == args.scale_dtype;
    if (current) return true;
    if (frozen(kn)) return false;
    if (kn.packed) {
        drop_weight_copy(kn, kn.packed);
        kn.packed = nullptr;
    }
    if (rocm_ffi_malloc(&kn.packed, rocm_decode_packed_bytes(&args)) != 0) {
        kn.packed = nullptr;
        return false;                       // no memory for a second copy: stream the caller's tensors instead
    }
    rc = rocm_launch_pack_decode(&args, kn.packed, kn.ep->stream);
    if (rc != 0) {                          // a copy that was not made must not pass for current on the next call
        rocm_ffi_free(kn.packed);
        kn.packed = nullptr;
        return false;
    }
    kn.packed_from[0] = args.b;
    kn.packed_from[1] = args.scales;
    kn.packed_from[2] = args.zp;
    kn.packed_scale_dtype = args.scale_dtype;
    return true;
}

// Tall 16-bit calls over a dense [N, K] copy of the weights in the activations' type, expanded by a launch of its own. Two users:
//  * the opt-in library route (dense_gemm_min_rows > 0): the product is the library GEMM, as in the CUDA provider for M >= 8
//    (onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:6176-6222);
//  * by default, calls from five rows whose weights the tile loader does not read - bits = 2 / 8 and weights with g_idx
//    (matmul_nbits.rs:2035, 3636-3658): the product is this provider's own tiled kernel over the dense copy, instead of a
//    one-wave-per-column GEMV that reads all M rows of A per column.
// Returns false with nothing launched when the route does not apply or is not ready (then the caller's next route takes the
// call): too few rows, another dtype mix, a dense copy beyond the configured size, no library kernel for the shape, or a first
// use while a graph capture is open (nothing may allocate then).
bool dense_route(NxrtRocmMatMulNBits& kn, const RocmMatMulNBitsArgs& args, int& rc)
{
    rc = 0;
    NxrtRocmEp& ep = *kn.ep;
    if (kn.no_alloc) return false;              // the library GEMM and its buffers are out of bounds for a call that may not allocate
    // other bit widths have no tiled kernel to fall back on, only the plain GEMV: the route pays from a few dozen rows
    const bool plain_only = kn.bits != 4 || args.g_idx != nullptr;
    const int64_t min_rows = !plain_only ? ep.dense_gemm_min_rows : (ep.dense_gemm_min_rows < 32 ? ep.dense_gemm_min_rows : 32);
    bool library = ep.dense_gemm_min_rows > 0 && args.m >= min_rows;
    if ((args.a_dtype != ROCM_DT_F16 && args.a_dtype != ROCM_DT_BF16) || (args.k & 7) != 0) return false;
    if ((reinterpret_cast<uintptr_t>(args.a) & 15) != 0 || (reinterpret_cast<uintptr_t>(args.b) & 3) != 0) return false;
    const uint64_t need = static_cast<uint64_t>(args.n) * static_cast<uint64_t>(args.k) * 2;
    if (need > ep.dense_gemm_max_bytes) return false;
    // what the library cannot take: another output type, an unaligned Y, a bias its epilogue does not add before the one rounding
    if (args.y_dtype != args.a_dtype || (reinterpret_cast<uintptr_t>(args.y) & 15) != 0 ||
        (args.bias && (args.bias_dtype & (ROCM_BIAS_POST_ROUND | ROCM_BIAS_PER_ROW))))
        library = false;
    const bool own = plain_only && rocm_prefill_dense16_eligible(&args);      // (five rows or more, K a multiple of 64)
    if (!library && !own) return false;
    const int bias_dtype = args.bias ? args.bias_dtype : -1;

    std::lock_guard<std::mutex> lock(ep.dense_mu);
    if (library) {
        if (!ep.dense && (ep.capturing || rocm_dense_gemm_create(&ep.dense) != 0)) {
            ep.dense = nullptr;
            library = false;
        }
        if (library && !rocm_dense_gemm_ready(ep.dense, args.m, args.n, args.k, args.a_dtype, bias_dtype, ep.capturing ? 0 : 1)) library = false;
        if (!library && !own) return false;      // no library kernel for the shape: the tiled kernel over the dense copy where it applies
    }

    const bool constant = kn.constant_inputs[1] && kn.constant_inputs[2] && (!args.zp || kn.constant_inputs[3]) && !args.g_idx;
    auto expand = [&](void* dst) {
        if (args.g_idx)
            return rocm_launch_dequant_gidx(args.b, args.scales, args.scale_dtype, args.zp, args.g_idx, args.n, args.k, args.block_size, static_cast<int>(kn.bits),
                                            args.a_dtype, dst, ep.stream);
        if (kn.bits == 4) return rocm_launch_dequant_16(args.b, args.scales, args.scale_dtype, args.zp, args.n, args.k, args.block_size, args.a_dtype, dst, ep.stream);
        return rocm_launch_dequant_nbits(args.b, args.scales, args.scale_dtype, args.zp, args.n, args.k, args.block_size, static_cast<int>(kn.bits), args.a_dtype,
                                         dst, ep.stream);
    };
    const void* w16 = nullptr;
    if (ep.dense_resident && constant) {
        const bool current = kn.dense && kn.dense_from[0] == args.b && kn.dense_from[1] == args.scales && kn.dense_from[2] == args.zp &&
                             kn.dense_dtype == args.a_dtype && kn.dense_scale_dtype == args.scale_dtype;
        if (!current) {
            if (ep.capturing) return false;
            if (kn.dense) {
                drop_weight_copy(kn, kn.dense);
                kn.dense = nullptr;
            }
            if (rocm_ffi_malloc(&kn.dense, need) != 0) {
                kn.dense = nullptr;
                return false;                   // no memory for a dense copy: the tiled kernel reads the packed weights
            }
            rc = expand(kn.dense);
            kn.dense_from[0] = args.b;
            kn.dense_from[1] = args.scales;
            kn.dense_from[2] = args.zp;
            kn.dense_dtype = args.a_dtype;
            kn.dense_scale_dtype = args.scale_dtype;
        }
        w16 = kn.dense;
        kn.variant = library ? "dense_resident_blaslt" : "dense_resident_tiled";
    } else {
        if (ep.dense_scratch_bytes < need) {
            if (ep.capturing) return false;
            if (grow_buffer(ep.dense_scratch, ep.dense_scratch_bytes, need, ep.dense_retired) != 0) return false;
        }
        rc = expand(ep.dense_scratch);
        w16 = ep.dense_scratch;
        kn.variant = library ? "dense_transient_blaslt" : "dense_transient_tiled";
    }
    if (rc != 0) return true;
    if (library) rc = rocm_dense_gemm_run(ep.dense, w16, args.a, args.y, args.bias, args.bias_dtype, args.m, args.n, args.k, args.a_dtype, ep.stream);
    else rc = rocm_launch_prefill_dense16(&args, w16, ep.prefill_tile, nullptr, 0, ep.stream);       // (no slices of K: they would want scratch of their own)
    return true;
}

// The bias of a pass that starts at row `row0`: a per-token residual moves with the rows, a broadcast bias stays.
const void* rows_of_bias(const RocmMatMulNBitsArgs& args, int64_t row0)
{
    if (!args.bias || !(args.bias_dtype & ROCM_BIAS_PER_ROW)) return args.bias;
    const size_t elem = (args.bias_dtype & 0xff) == ROCM_DT_F32 ? 4 : 2;
    return static_cast<const uint8_t*>(args.bias) + static_cast<size_t>(row0) * static_cast<size_t>(args.n) * elem;
}

// 17..32 rows as two blocks of at most 16 through the decode kernels. The tiled kernel needs a few hundred rows to
// pay for itself; below that a call costs what streaming the weights costs, and two streams can be cheaper than one
// under-filled tiled launch. Measured against the tiled kernel (which slices K for small grids), bf16:
//   block 128, 3584 -> 3584 / 4096 -> 4096 / 18944 -> 3584 / 14336 -> 4096: blocks win at 17, 24 and 32 rows
//     (11.9-13.1 against 14.5-15.8 us; 12.3-13.8 against 16.2-16.7; 28-36 against 38-39; 25-31 against 34-35);
//   block 128, 4096 -> 14336: 26.7 against 30.0 us at 17 rows, 31.5 against 30.3 at 24, 35.9 against 31.1 at 32;
//   block 64, 4096 -> 14336: the tiled kernel wins throughout (33-47 against 30-31.5 us);
//   block 32, 896 -> 4864 / 4864 -> 896 / 2048 -> 8192: the tiled kernel wins or ties (10.5-18.8 against 11.0-15.9 us).
// So: blocks over the repacked copy whenever it applies (one pass per block at full stream rate); otherwise blocks only
// at block size 128, and there up to 8192 columns or up to 20 rows (a second block of at most four rows is the cheap one;
// at 24 rows the two routes tie or the tiled kernel leads). Returns false (nothing launched) when the decode
// kernels do not take the shape or the tiled kernel is the better route.
bool decode_in_row_blocks(NxrtRocmMatMulNBits& kn, const RocmMatMulNBitsArgs& args, int& rc)
{
    rc = 0;
    RocmMatMulNBitsArgs probe = args;
    probe.m = 16;
    if (!rocm_decode_mfma_eligible(&probe)) return false;
    int probe_rc = 0;       // stays 0: a repack that fails leaves no copy behind and use_packed then answers false
    // (block size 32 below 16384 columns: two repacked passes of 16 rows take 41 us where the tiled kernel takes 32 -
    // asked first, so that no repacked copy is made for a call the tiled kernel then takes)
    const bool packed_blocks = !(args.block_size == 32 && args.n < 16384) && use_packed(kn, probe, probe_rc);
    if (!packed_blocks && rocm_prefill_mfma_eligible(&args) &&
        !(args.block_size >= 128 && (args.n <= 8192 || args.m <= 20)))
        return false;
    const size_t a_elem = 2;                                            // eligibility means f16 / bf16 activations
    const size_t y_elem = args.y_dtype == ROCM_DT_F32 ? 4 : 2;
    bool all_packed = true;
    for (int64_t row0 = 0; row0 < args.m && rc == 0; row0 += 16) {
        RocmMatMulNBitsArgs part = args;
        part.m = args.m - row0 < 16 ? args.m - row0 : 16;
        part.a = static_cast<const uint8_t*>(args.a) + static_cast<size_t>(row0) * static_cast<size_t>(args.k) * a_elem;
        part.y = static_cast<uint8_t*>(args.y) + static_cast<size_t>(row0) * static_cast<size_t>(args.n) * y_elem;
        part.bias = rows_of_bias(args, row0);
        int pack_rc = 0;
        if (use_packed(kn, part, pack_rc)) {
            rc = pack_rc != 0 ? pack_rc : rocm_launch_decode_packed(&part, kn.packed, kn.ep->decode_waves, kn.ep->stream);
        } else {
            all_packed = false;
            rc = rocm_launch_decode_mfma(&part, kn.ep->decode_waves, kn.ep->decode_col_groups, kn.ep->stream);
        }
    }
    kn.variant = all_packed ? "decode_mfma_packed" : "decode_mfma_splitk";
    return true;
}

// f32 activations: passes of up to four rows through the f32 streaming kernel. Returns false (nothing launched) when
// that kernel does not take the shape.
bool f32_in_row_blocks(NxrtRocmMatMulNBits& kn, const RocmMatMulNBitsArgs& args, int& rc)
{
    rc = 0;
    RocmMatMulNBitsArgs probe = args;
    probe.m = 1;
    if (!rocm_gemv_f32_eligible(&probe)) return false;
    const size_t y_elem = args.y_dtype == ROCM_DT_F32 ? 4 : 2;
    for (int64_t row0 = 0; row0 < args.m && rc == 0; row0 += 4) {
        RocmMatMulNBitsArgs part = args;
        part.m = args.m - row0 < 4 ? args.m - row0 : 4;
        part.a = static_cast<const uint8_t*>(args.a) + static_cast<size_t>(row0) * static_cast<size_t>(args.k) * 4;
        part.y = static_cast<uint8_t*>(args.y) + static_cast<size_t>(row0) * static_cast<size_t>(args.n) * y_elem;
        part.bias = rows_of_bias(args, row0);
        rc = rocm_launch_gemv_f32(&part, kn.ep->stream);
    }
    kn.variant = "gemv_f32_valu";
    return true;
}

// The RMS-normalization prologue of a node on its way through the dispatch: the decode kernels over the repacked stream
// apply it themselves (up to four rows); every other route first normalizes the rows into `owner`'s buffer with a
// launch of its own.
struct NormPrologue {
    const void* gamma;
    int gamma_dtype;
    float epsilon;
    NxrtRocmMatMulNBits* owner;     // the node that carries the prologue: its buffer holds the normalized rows
    bool fused = false;             // out: the kernel applied it
};

// a -> round16((a * inv_std) * gamma), [rows, K] of a 16-bit type, into owner.norm; `a` is replaced by the buffer.
NxrtStatus normalize_rows(const NormPrologue& np, const void*& a, int a_dtype, uint64_t rows, uint64_t k)
{
    NxrtRocmMatMulNBits& owner = *np.owner;
    const uint64_t need = rows * k * 2;
    if (owner.norm_bytes < need) {
        if (frozen(owner))
            return make_status(NXRT_INVALID_ARGUMENT, err("rmsnorm_prologue fusion under graph capture needs one eager call of this height first (the "
                                                          "normalized activations live in a buffer the kernel may not allocate while a capture is open)"));
        const int e = grow_buffer(owner.norm, owner.norm_bytes, need, owner.retired);
        if (e != 0) return hip_status(e, "MatMulNBits: workspace hipMalloc");
    }
    if ((reinterpret_cast<uintptr_t>(a) & 7) != 0 || (reinterpret_cast<uintptr_t>(np.gamma) & 15) != 0)
        return make_status(NXRT_INVALID_ARGUMENT, err("rmsnorm_prologue fusion needs A at an 8-byte and gamma at a 16-byte boundary (data pointer plus byte offset)"));
    const int rc = rocm_launch_rmsnorm16(a, np.gamma, np.gamma_dtype, static_cast<int64_t>(rows), static_cast<int64_t>(k), np.epsilon, a_dtype, owner.norm, owner.ep->stream);
    if (rc != 0) return hip_status(rc, "MatMulNBits: kernel launch");
    owner.ep->launches.fetch_add(1);
    a = owner.norm;
    return ok();
}

NxrtStatus execute_impl(NxrtRocmMatMulNBits& kn, const NxrtRocmTensorView* in, uint32_t n_in, NxrtRocmTensorView* out, uint32_t n_out,
                        void* workspace, uint64_t workspace_bytes, bool no_alloc = false, NormPrologue* norm = nullptr)
{
    std::lock_guard<std::mutex> lock(kn.mu);
    struct Mode {
        NxrtRocmMatMulNBits& k;
        Mode(NxrtRocmMatMulNBits& kernel, bool on) : k(kernel) { k.no_alloc = on; }
        ~Mode() { k.no_alloc = false; }
    } mode(kn, no_alloc);
    // kernels/mod.rs:1898-1919 (check_arity)
    if (n_in < 3 || n_in > 6) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits: expected 3..=6 inputs, got " + std::to_string(n_in));
    if (n_out < 1) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits: expected at least 1 output(s), got " + std::to_string(n_out));
    if (!in || !out) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits: null tensor view array");

    Check c;
    auto require_float = [&](const char* name, uint32_t dt) {
        if (!is_float_compute(dt)) c.fail(std::string(name) + " must have dtype Float32, Float16, or BFloat16, got " + dtype_name(dt));
    };
    auto require_dtype = [&](const char* name, uint32_t got, uint32_t want) {
        if (got != want) c.fail(std::string(name) + " must have dtype " + dtype_name(want) + ", got " + dtype_name(got));
    };
    auto optional = [&](uint32_t i) -> const NxrtRocmTensorView* { return (i < n_in && in[i].data != nullptr) ? &in[i] : nullptr; };
    auto flat_or_matrix = [&](const char* name, const NxrtRocmTensorView& v, uint64_t rows, uint64_t cols) {
        if (!shape_is(v, {rows * cols}) && !shape_is(v, {rows, cols}))
            c.fail(std::string(name) + " must have shape [" + std::to_string(rows * cols) + "] or [" + std::to_string(rows) + ", " + std::to_string(cols) +
                   "], got " + shape_str(v.shape, v.ndim));
    };

    const NxrtRocmTensorView& A = in[0];
    const NxrtRocmTensorView& B = in[1];
    const NxrtRocmTensorView& S = in[2];
    NxrtRocmTensorView& Y = out[0];
    require_float("A", A.dtype);
    require_dtype("B", B.dtype, NXRT_DT_UINT8);
    require_float("scales", S.dtype);
    require_float("Y", Y.dtype);
    if (c.failed) return make_status(NXRT_INVALID_ARGUMENT, c.message);

    const uint64_t K = static_cast<uint64_t>(kn.k), N = static_cast<uint64_t>(kn.n), BS = static_cast<uint64_t>(kn.block_size);
    if (A.ndim == 0 || A.shape[A.ndim - 1] != K)
        return make_status(NXRT_INVALID_ARGUMENT, err("A must have rank >= 1 and last dimension K=" + std::to_string(K) + ", got " + shape_str(A.shape, A.ndim)));
    std::vector<uint64_t> y_shape(A.shape, A.shape + A.ndim - 1);
    y_shape.push_back(N);
    if (!shape_is(Y, y_shape))
        return make_status(NXRT_INVALID_ARGUMENT, err("Y must have shape " + shape_str(y_shape) + ", got " + shape_str(Y.shape, Y.ndim)));

    const uint64_t kb = (K + BS - 1) / BS;
    const uint64_t bits = static_cast<uint64_t>(kn.bits);
    const uint64_t blob = BS * bits / 8;
    flat_or_matrix("scales", S, N, kb);
    const NxrtRocmTensorView* ZP = optional(3);
    if (ZP && !c.failed) {
        require_dtype("zero_points", ZP->dtype, NXRT_DT_UINT8);
        if (!c.failed) flat_or_matrix("zero_points", *ZP, N, (kb * bits + 7) / 8);
    }
    const NxrtRocmTensorView* G = optional(4);
    if (G && !c.failed) {
        require_dtype("g_idx", G->dtype, NXRT_DT_INT32);
        if (!c.failed && !shape_is(*G, {K}) && !shape_is(*G, {kb * BS}))
            c.fail("g_idx must have shape [" + std::to_string(K) + "] or [" + std::to_string(kb * BS) + "], got " + shape_str(G->shape, G->ndim));
        if (!c.failed && kn.accuracy_level == 4)
            c.fail("accuracy_level=4 does not take g_idx on the ROCm execution provider. Why: its int8 kernels scale whole contiguous K blocks. "
                   "How to fix: export the weight without act-order, use accuracy_level=0, or run this node on the CPU execution provider");
    }
    if (!c.failed && !shape_is(B, {N, kb, blob}))
        c.fail("B must have shape " + shape_str({N, kb, blob}) + ", got " + shape_str(B.shape, B.ndim));
    const NxrtRocmTensorView* BIAS = optional(5);
    // A folded residual epilogue passes a per-token residual in the bias slot: Y's shape (or M * N elements flat), indexed
    // with row stride N (onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:7891-7897). A genuine bias is [N].
    bool bias_per_row = false;
    if (BIAS && !c.failed) {
        require_float("bias", BIAS->dtype);
        if (!c.failed && !shape_is(*BIAS, {N})) {
            // By element count, as the CUDA sibling does (matmul_nbits.rs:7728-7735): N elements in any shape ([1, N],
            // [1, 1, N] - the residual of a one-row decode step) broadcast with stride 0, rows * N elements are per-token.
            uint64_t rows = 1, numel = 1;
            for (uint32_t i = 0; i + 1 < A.ndim; ++i) rows *= A.shape[i];
            for (uint32_t i = 0; i < BIAS->ndim; ++i) numel *= BIAS->shape[i];
            bias_per_row = numel == rows * N && rows * N != N;
            if (!bias_per_row && numel != N)
                c.fail("bias must have " + std::to_string(N) + " elements (broadcast [N]) or " + std::to_string(rows * N) + " elements (a per-token residual of Y's shape " +
                       shape_str(y_shape) + "), got " + shape_str(BIAS->shape, BIAS->ndim));
        }
    }
    if (c.failed) return make_status(NXRT_INVALID_ARGUMENT, c.message);

    struct Named { const char* name; const NxrtRocmTensorView* v; };
    const Named all[] = {{"A", &A}, {"B", &B}, {"scales", &S}, {"zero_points", ZP}, {"g_idx", G}, {"bias", BIAS}, {"Y", &Y}};
    for (const Named& t : all) {
        if (!t.v) continue;
        if (!is_contiguous(*t.v)) return make_status(NXRT_INVALID_ARGUMENT, err(std::string(t.name) + " must be contiguous on the ROCm execution provider"));
        if (t.v->device_type != NXRT_DEVICE_ROCM || t.v->device_index != kn.ep->device)
            return make_status(NXRT_INVALID_ARGUMENT, err(std::string(t.name) + " must live on ROCm device " + std::to_string(kn.ep->device) +
                                                          " (allocate it with this provider and copy the data in)"));
    }

    uint64_t M = 1;
    for (uint32_t i = 0; i + 1 < A.ndim; ++i) M *= A.shape[i];
    {
        // record_kernel_metrics (onnx-runtime-ep-api/src/kernel.rs:243-267): bytes = every present input's bytes + the output's;
        // flops = 2 M N K, + M N with a bias (matmul_nbits.rs:1588-1597)
        uint64_t bytes = 0;
        for (const Named& t : all) {
            if (!t.v) continue;
            uint64_t elems = 1;
            for (uint32_t i = 0; i < t.v->ndim; ++i) elems *= t.v->shape[i];
            const uint32_t dt = t.v->dtype;
            bytes += elems * (dt == NXRT_DT_FLOAT32 || dt == NXRT_DT_INT32 ? 4u : dt == NXRT_DT_UINT8 ? 1u : 2u);
        }
        kn.last_bytes = bytes;
        kn.last_flops = 2ull * M * static_cast<uint64_t>(kn.n) * static_cast<uint64_t>(kn.k) + (BIAS ? M * static_cast<uint64_t>(kn.n) : 0ull);
    }
    if (M == 0) return ok();
    // A required tensor without memory behind it would reach a kernel as address 0: a GPU memory fault instead of a status.
    for (const Named& t : {Named{"A", &A}, Named{"B", &B}, Named{"scales", &S}, Named{"Y", &Y}})
        if (t.v->data == nullptr) return make_status(NXRT_INVALID_ARGUMENT, err(std::string(t.name) + " has a null data pointer"));

    NxrtStatus st = kn.ep->bind();
    if (st.code != NXRT_OK) return st;

    auto at = [](const NxrtRocmTensorView& v) { return static_cast<void*>(static_cast<uint8_t*>(v.data) + v.byte_offset); };
    RocmMatMulNBitsArgs args;
    args.a = at(A);
    args.b = static_cast<const uint8_t*>(at(B));
    args.scales = at(S);
    args.zp = ZP ? static_cast<const uint8_t*>(at(*ZP)) : nullptr;
    args.bias = BIAS ? at(*BIAS) : nullptr;
    args.y = at(Y);
    args.a_dtype = static_cast<int>(A.dtype);
    args.scale_dtype = static_cast<int>(S.dtype);
    args.bias_dtype = BIAS ? static_cast<int>(BIAS->dtype) : ROCM_DT_F32;
    if (BIAS && kn.bias_post_round) args.bias_dtype |= ROCM_BIAS_POST_ROUND;
    if (BIAS && bias_per_row) args.bias_dtype |= ROCM_BIAS_PER_ROW;
    args.y_dtype = static_cast<int>(Y.dtype);
    args.m = static_cast<int64_t>(M);
    args.n = kn.n;
    args.k = kn.k;
    args.block_size = static_cast<int>(kn.block_size);
    args.g_idx = G ? static_cast<const int32_t*>(at(*G)) : nullptr;
    args.acc_probe = nullptr;
    args.gamma = nullptr;
    args.gamma_dtype = 0;
    args.norm_epsilon = 0.f;
    if (kn.acc_probe) {
        if (kn.accuracy_level != 4) return make_status(NXRT_INVALID_ARGUMENT, err("the block-accumulator probe needs accuracy_level=4"));
        if (M * N * kb > kn.acc_probe_elems)
            return make_status(NXRT_INVALID_ARGUMENT, err("the block-accumulator probe buffer holds " + std::to_string(kn.acc_probe_elems) + " int32 values, this call needs " +
                                                          std::to_string(M * N * kb)));
        args.acc_probe = kn.acc_probe;
    }

    rocm_stream_t stream = kn.ep->stream;
    int rc = 0;
    if (norm) {
        // up to four rows over the repacked stream: the decode kernel normalizes the rows itself; otherwise a launch of its own
        RocmMatMulNBitsArgs fused = args;
        fused.gamma = norm->gamma;
        fused.gamma_dtype = norm->gamma_dtype;
        fused.norm_epsilon = norm->epsilon;
        int pack_rc = 0;
        if (kn.bits == 4 && !G && kn.accuracy_level != 4 && !kn.pair_member && kn.n <= kn.ep->rmsnorm_in_kernel_max_cols && rocm_decode_packed_fuses_norm(&fused) &&
            use_packed(kn, args, pack_rc) && pack_rc == 0) {
            args = fused;
            norm->fused = true;
        } else {
            const NxrtStatus ns = normalize_rows(*norm, args.a, args.a_dtype, M, K);
            if (ns.code != NXRT_OK) return ns;
        }
    }
    if (G && kn.g_idx_checked != args.g_idx) {
        // matmul_nbits.rs:3515-3521: every group must lie in 0..kb. Checked once per tensor (a device pass and a read-back).
        if (frozen(kn))
            return make_status(NXRT_INVALID_ARGUMENT, err("g_idx has not been range-checked yet and this call may not allocate or synchronise (a graph capture is open, or it came "
                                                          "through execute_static); run this node once through execute first"));
        int64_t bad = -1;
        const int e = rocm_g_idx_first_bad(args.g_idx, static_cast<int64_t>(K), static_cast<int64_t>(kb), &bad, stream);
        if (e != 0) return hip_status(e, "MatMulNBits: g_idx check");
        if (bad >= 0) return make_status(NXRT_INVALID_ARGUMENT, err("g_idx[" + std::to_string(bad) + "] is outside 0.." + std::to_string(kb)));
        kn.g_idx_checked = args.g_idx;
    }
    if (kn.bits != 4 || G) {
        // 2 and 8 bits, and act-order weights of any width: 16-bit calls from five rows expand the weights and run the tiled
        // kernel over the dense copy (or, opt-in, the library GEMM), everything else the plain f32 GEMV
        if (!dense_route(kn, args, rc)) {
            rc = rocm_launch_gemv_nbits(&args, static_cast<int>(kn.bits), stream);
            kn.variant = "gemv_nbits_f32";
        }
        kn.ep->launches.fetch_add(1);
        return hip_status(rc, "MatMulNBits: kernel launch");
    }
    if (kn.accuracy_level == 4) {
        const int rounding = kn.ep->acc4_rounding == 2 ? (static_cast<int64_t>(M) < static_cast<int64_t>(kn.ep->acc4_native_below) ? 1 : 0) : kn.ep->acc4_rounding;   // matmul_nbits.rs:640-660
        int pack_rc = 0;
        const bool packed = M <= 16 && use_packed(kn, args, pack_rc);       // up to 16 rows read the repacked stream
        if (packed && rocm_acc4_packed_fuses_quantizer(&args)) {
            // one f16 / bf16 row over the repacked stream: the kernel quantizes the row itself, no workspace and no second launch
            rc = pack_rc != 0 ? pack_rc : rocm_launch_acc4_packed(&args, kn.packed, nullptr, rounding, kn.ep->decode_waves, stream);
            kn.variant = "acc4_mfma_i8_packed";
            kn.ep->launches.fetch_add(1);
            return hip_status(rc, "MatMulNBits: kernel launch");
        }
        const Acc4Layout lay = acc4_layout(kn, M);
        const uint64_t need = lay.total, mandatory = lay.codes + lay.pairs + lay.aux;
        uint8_t* ws = static_cast<uint8_t*>(workspace);
        uint64_t partial_bytes = lay.partial;
        if (kn.no_alloc) {
            // the static scratch: codes, pairs and their block-major copy must fit; partial sums of K slices get what is left
            // (with less room the tiled kernel cuts K into fewer slices, or none)
            if (!ws || workspace_bytes < mandatory)
                return make_status(NXRT_INVALID_ARGUMENT, err("accuracy_level=4 at " + std::to_string(M) + " rows needs " + std::to_string(mandatory) + " bytes of scratch and the static scratch of "
                                                              "execute_static holds " + std::to_string(workspace_bytes) + "; call execute with a workspace of workspace_requirement() bytes instead"));
            if (partial_bytes > workspace_bytes - mandatory) partial_bytes = (workspace_bytes - mandatory) / 256 * 256;
        } else if (!ws || workspace_bytes < need) {
            if (kn.scratch_bytes < need) {
                if (kn.ep->capturing)
                    return make_status(NXRT_INVALID_ARGUMENT, err("accuracy_level=4 under graph capture needs a caller workspace of " + std::to_string(need) +
                                                                  " bytes (see workspace_requirement); the kernel may not allocate while a capture is open"));
                const int e = grow_buffer(kn.scratch, kn.scratch_bytes, need, kn.retired);
                if (e != 0) return hip_status(e, "MatMulNBits: workspace hipMalloc");
            }
            ws = static_cast<uint8_t*>(kn.scratch);
        }
        RocmAcc4Workspace w4;
        w4.qa = reinterpret_cast<int8_t*>(ws);
        w4.aq = reinterpret_cast<float*>(ws + lay.codes);
        w4.aux = reinterpret_cast<float*>(ws + lay.codes + lay.pairs);
        w4.code_order = packed ? 2 : 1;
        w4.partial = partial_bytes ? reinterpret_cast<float*>(ws + lay.codes + lay.pairs + lay.aux) : nullptr;
        w4.partial_bytes = partial_bytes;
        rc = rocm_launch_quantize_a_workspace(args.a, args.a_dtype, args.m, args.k, args.block_size, rounding, &w4, stream);
        if (rc == 0 && pack_rc != 0) rc = pack_rc;
        if (rc == 0) {
            if (packed) {
                rc = rocm_launch_acc4_packed(&args, kn.packed, &w4, rounding, kn.ep->decode_waves, stream);
                kn.variant = "acc4_mfma_i8_packed";
            } else if (rocm_acc4_mfma_eligible(&args)) {
                rc = rocm_launch_acc4_mfma(&args, &w4, kn.ep->decode_waves, stream);
                kn.variant = "acc4_mfma_i8";
            } else {
                if (args.acc_probe) return make_status(NXRT_INVALID_ARGUMENT, err("the block-accumulator probe covers the int8 matrix-core kernels only; this shape runs on the dot-product kernel"));
                rc = rocm_launch_acc4_gemv(&args, &w4, stream);
                kn.variant = "acc4_gemv_dot4";
            }
        }
    } else if (M <= 64 && use_packed(kn, args, rc)) {
        if (rc == 0) rc = (kn.pair_member && M <= 16) ? rocm_launch_decode_packed_pair_member(&args, kn.packed, kn.ep->decode_waves, stream)
                                                      : rocm_launch_decode_packed(&args, kn.packed, kn.ep->decode_waves, stream);
        kn.variant = "decode_mfma_packed";
    } else if (M <= 16 && rocm_decode_mfma_eligible(&args)) {
        rc = rocm_launch_decode_mfma(&args, kn.ep->decode_waves, kn.ep->decode_col_groups, stream);
        kn.variant = "decode_mfma_splitk";
    } else if (M <= 32 && decode_in_row_blocks(kn, args, rc)) {
        // done: a few passes of the streaming kernels beat one pass of the tiled kernel at these heights
    } else if (dense_route(kn, args, rc)) {
        // done: weights expanded to 16 bits, then the library GEMM
    } else if (M > 16 && rocm_prefill_mfma_eligible(&args)) {
        // Small grids slice K and want scratch for the partial sums: the caller's workspace if it is large enough, else
        // the kernel's own (grown outside a capture only; with too little the launcher slices less or not at all).
        const uint64_t need = rocm_prefill_mfma_scratch_bytes(&args, kn.ep->prefill_tile);
        void* scratch = workspace;
        uint64_t scratch_bytes = workspace ? workspace_bytes : 0;
        if (need > scratch_bytes) {
            if (kn.scratch_bytes < need && !frozen(kn)) (void)grow_buffer(kn.scratch, kn.scratch_bytes, need, kn.retired);   // on failure: slice less
            if (kn.scratch_bytes > scratch_bytes) {
                scratch = kn.scratch;
                scratch_bytes = kn.scratch_bytes;
            }
        }
        rc = rocm_launch_prefill_mfma(&args, kn.ep->prefill_tile, scratch, scratch_bytes, stream);
        kn.variant = "prefill_mfma_lds";
    } else if (M <= 64 && f32_in_row_blocks(kn, args, rc)) {
        // done: f32 activations stay in f32 arithmetic end to end
    } else {
        rc = rocm_launch_gemv_generic(&args, stream);
        kn.variant = "gemv_generic_f32";
    }
    kn.ep->launches.fetch_add(1);
    return hip_status(rc, "MatMulNBits: kernel launch");
}

// The fused gate/up node of the CUDA provider (onnx-runtime-ep-cuda/src/optimizer.rs:36-46, kernels/matmul_nbits.rs:9017-9130):
// inputs [x, W_gate, scales_gate, W_up, scales_up, (gamma), (zp_gate, zp_up)], output silu(gate) * up with both projections
// rounded to the 16-bit type first. Here both projections run through the ordinary dispatch into scratch, then the epilogue.
NxrtStatus execute_swiglu(NxrtRocmMatMulNBits& kn, const NxrtRocmTensorView* in, uint32_t n_in, NxrtRocmTensorView* out, uint32_t n_out,
                          void* workspace, uint64_t workspace_bytes, NormPrologue* norm = nullptr)
{
    std::lock_guard<std::mutex> lock(kn.mu);
    if (n_in < 5 || n_in > 8 || n_out != 1)
        return make_status(NXRT_INVALID_ARGUMENT, err("gate/up SwiGLU fusion expects 5 to 8 inputs [x, W_gate, scales_gate, W_up, scales_up, (gamma), "
                                                      "(zp_gate, zp_up)] and 1 output, got " + std::to_string(n_in) + " inputs and " + std::to_string(n_out) + " outputs"));
    if (!in || !out) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits: null tensor view array");
    auto optional = [&](uint32_t i) -> const NxrtRocmTensorView* { return (i < n_in && in[i].data != nullptr) ? &in[i] : nullptr; };
    if (optional(5))
        return make_status(NXRT_INVALID_ARGUMENT, err("gate/up SwiGLU fusion received a normalization weight at input 5 but no RMS-norm prologue marker. "
                                                      "How to fix: set rmsnorm_prologue = 1 on the node, or leave input 5 absent"));
    const NxrtRocmTensorView* zp_gate = optional(6);
    const NxrtRocmTensorView* zp_up = optional(7);
    if ((zp_gate != nullptr) != (zp_up != nullptr))
        return make_status(NXRT_INVALID_ARGUMENT, err("gate/up SwiGLU fusion requires zero points for both projections or neither"));
    const NxrtRocmTensorView& A = in[0];
    NxrtRocmTensorView& Y = out[0];
    if (A.dtype != NXRT_DT_FLOAT16 && A.dtype != NXRT_DT_BFLOAT16)
        return make_status(NXRT_INVALID_ARGUMENT, err(std::string("gate/up SwiGLU fusion needs Float16 or BFloat16 activations, got ") + dtype_name(A.dtype)));
    if (Y.dtype != A.dtype)
        return make_status(NXRT_INVALID_ARGUMENT, err(std::string("Y must have dtype ") + dtype_name(A.dtype) + ", got " + dtype_name(Y.dtype)));
    const uint64_t K = static_cast<uint64_t>(kn.k), N = static_cast<uint64_t>(kn.n);
    if (A.ndim == 0 || A.shape[A.ndim - 1] != K)
        return make_status(NXRT_INVALID_ARGUMENT, err("A must have rank >= 1 and last dimension K=" + std::to_string(K) + ", got " + shape_str(A.shape, A.ndim)));
    std::vector<uint64_t> y_shape(A.shape, A.shape + A.ndim - 1);
    y_shape.push_back(N);
    if (!shape_is(Y, y_shape)) return make_status(NXRT_INVALID_ARGUMENT, err("Y must have shape " + shape_str(y_shape) + ", got " + shape_str(Y.shape, Y.ndim)));
    if (!is_contiguous(Y)) return make_status(NXRT_INVALID_ARGUMENT, err("Y must be contiguous on the ROCm execution provider"));
    if (Y.device_type != NXRT_DEVICE_ROCM || Y.device_index != kn.ep->device)
        return make_status(NXRT_INVALID_ARGUMENT, err("Y must live on ROCm device " + std::to_string(kn.ep->device) + " (allocate it with this provider and copy the data in)"));
    uint64_t M = 1;
    for (uint32_t i = 0; i + 1 < A.ndim; ++i) M *= A.shape[i];
    if (M == 0) return ok();
    {
        const char* names[5] = {"x", "W_gate", "scales_gate", "W_up", "scales_up"};
        for (uint32_t i = 0; i < 5; ++i)
            if (in[i].data == nullptr) return make_status(NXRT_INVALID_ARGUMENT, err(std::string(names[i]) + " has a null data pointer"));
        if (Y.data == nullptr) return make_status(NXRT_INVALID_ARGUMENT, err("Y has a null data pointer"));
    }
    NxrtStatus st = kn.ep->bind();
    if (st.code != NXRT_OK) return st;

    // Up to four rows over constant weights (up to sixteen where the projections are wide enough for the shared-activation
    // kernel): one launch over both repacked copies. The copies are made (and every weight tensor validated) by the
    // projections' own first call below, so this path serves the calls after the first with the same weight tensors; it
    // sums each projection exactly as that first call did.
    // (accuracy_level 4 stays on its own int8 kernels for every call: the paired launch is the float path)
    const void* normalized = nullptr;                    // the rows after a normalization launch of their own, once made
    if (M <= 16 && kn.accuracy_level != 4 && kn.gate->packed && kn.up->packed) {
        auto current = [&](const NxrtRocmMatMulNBits& child, const NxrtRocmTensorView& w, const NxrtRocmTensorView& s, const NxrtRocmTensorView* zp) {
            auto at = [](const NxrtRocmTensorView& v) { return static_cast<const void*>(static_cast<const uint8_t*>(v.data) + v.byte_offset); };
            return child.packed_from[0] == at(w) && child.packed_from[1] == at(s) && child.packed_from[2] == (zp ? at(*zp) : nullptr) &&
                   child.packed_scale_dtype == static_cast<int>(s.dtype);
        };
        if (current(*kn.gate, in[1], in[2], zp_gate) && current(*kn.up, in[3], in[4], zp_up) && is_contiguous(A) &&
            A.device_type == NXRT_DEVICE_ROCM && A.device_index == kn.ep->device) {
            RocmMatMulNBitsArgs args;
            std::memset(&args, 0, sizeof(args));
            args.a = static_cast<uint8_t*>(A.data) + A.byte_offset;
            args.b = static_cast<const uint8_t*>(kn.gate->packed_from[0]);
            args.scales = kn.gate->packed_from[1];
            args.zp = static_cast<const uint8_t*>(kn.gate->packed_from[2]);
            args.y = static_cast<uint8_t*>(Y.data) + Y.byte_offset;
            args.a_dtype = args.y_dtype = static_cast<int>(A.dtype);
            args.scale_dtype = kn.gate->packed_scale_dtype;
            args.bias_dtype = ROCM_DT_F32;
            args.m = static_cast<int64_t>(M);
            args.n = kn.n;
            args.k = kn.k;
            args.block_size = static_cast<int>(kn.block_size);
            // (a prologue rides along where the pair is narrow enough for the in-kernel form to pay; a wider pair normalizes first)
            const bool norm_inside = norm && M <= 4 && 2 * kn.n <= kn.ep->rmsnorm_in_kernel_max_cols;
            if (norm_inside) {
                args.gamma = norm->gamma;
                args.gamma_dtype = norm->gamma_dtype;
                args.norm_epsilon = norm->epsilon;
            } else if (norm) {
                normalized = args.a;
                const NxrtStatus ns = normalize_rows(*norm, normalized, args.a_dtype, M, K);
                if (ns.code != NXRT_OK) return ns;
                args.a = normalized;                     // whatever runs below sees these rows
            }
            if (rocm_decode_packed_eligible(&args) && (!norm_inside || rocm_decode_packed_fuses_norm(&args)) && rocm_decode_packed_pair_fits(&args, kn.ep->decode_waves)) {
                if (norm_inside) norm->fused = true;
                const int rc = rocm_launch_decode_packed_pair(&args, kn.gate->packed, kn.up->packed, kn.decomposed_silu ? 1 : 0, kn.ep->decode_waves, kn.ep->stream);
                kn.ep->launches.fetch_add(1);
                kn.variant = "gate_up_swiglu_packed";
                return hip_status(rc, "MatMulNBits: kernel launch");
            }
        }
    }

    // two 16-bit [M, N] matrices: the caller's workspace if it is large enough, else the kernel's own
    const uint64_t each = (M * N * 2 + 255) / 256 * 256;
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    if (!ws || workspace_bytes < 2 * each) {
        if (kn.scratch_bytes < 2 * each) {
            if (kn.ep->capturing)
                return make_status(NXRT_INVALID_ARGUMENT, err("gate/up SwiGLU fusion under graph capture needs a caller workspace of " + std::to_string(2 * each) +
                                                              " bytes (see workspace_requirement), or one eager call of this height first"));
            const int e = grow_buffer(kn.scratch, kn.scratch_bytes, 2 * each, kn.retired);
            if (e != 0) return hip_status(e, "MatMulNBits: workspace hipMalloc");
        }
        ws = static_cast<uint8_t*>(kn.scratch);
    }
    // the children see normalized rows: one launch for both projections
    NxrtRocmTensorView a_view = A;
    if (norm) {
        if (!normalized) {
            if (!is_contiguous(A) || A.device_type != NXRT_DEVICE_ROCM || A.device_index != kn.ep->device)
                return make_status(NXRT_INVALID_ARGUMENT, err("A must be contiguous and live on ROCm device " + std::to_string(kn.ep->device)));
            normalized = static_cast<const uint8_t*>(A.data) + A.byte_offset;
            const NxrtStatus ns = normalize_rows(*norm, normalized, static_cast<int>(A.dtype), M, K);
            if (ns.code != NXRT_OK) return ns;
        }
        a_view.data = const_cast<void*>(normalized);
        a_view.byte_offset = 0;
        a_view.strides = nullptr;
    }
    auto run = [&](NxrtRocmMatMulNBits& child, const NxrtRocmTensorView& w, const NxrtRocmTensorView& s, const NxrtRocmTensorView* zp, void* dst) {
        NxrtRocmTensorView cin[4];
        cin[0] = a_view;
        cin[1] = w;
        cin[2] = s;
        if (zp) cin[3] = *zp;
        NxrtRocmTensorView cy = Y;
        cy.data = dst;
        cy.byte_offset = 0;
        cy.strides = nullptr;
        return execute_impl(child, cin, zp ? 4u : 3u, &cy, 1, nullptr, 0);
    };
    st = run(*kn.gate, in[1], in[2], zp_gate, ws);
    if (st.code != NXRT_OK) return st;
    st = run(*kn.up, in[3], in[4], zp_up, ws + each);
    if (st.code != NXRT_OK) return st;
    void* y = static_cast<uint8_t*>(Y.data) + Y.byte_offset;
    const int rc = rocm_launch_swiglu(ws, ws + each, static_cast<int64_t>(M * N), static_cast<int>(A.dtype), kn.decomposed_silu ? 1 : 0, y, kn.ep->stream);
    kn.ep->launches.fetch_add(1);
    kn.variant = "gate_up_swiglu[" + kn.gate->variant + "]";
    return hip_status(rc, "MatMulNBits: kernel launch");
}

// A node with the RMS-normalization prologue (the CUDA provider's `_cuda_matmul_nbits_rmsnorm_prologue`,
// onnx-runtime-ep-cuda/src/optimizer.rs:48-60; kernels/matmul_nbits.rs:7739-7745, 9042-9050): gamma [K] rides at input 6
// (input 5 of the fused gate/up node). Up to four rows over the repacked stream are normalized inside the decode kernel
// (kernels/matmul_nbits.rs:3747-3783 does the same in its GEMV); on every other route the activations are normalized into a
// buffer of the kernel's own, then the node runs on them as it would without the prologue.
NxrtStatus execute_normalized(NxrtRocmMatMulNBits& kn, const NxrtRocmTensorView* in, uint32_t n_in, NxrtRocmTensorView* out, uint32_t n_out,
                              void* workspace, uint64_t workspace_bytes)
{
    std::lock_guard<std::mutex> lock(kn.norm_mu);
    const uint32_t slot = kn.gate_up_swiglu ? 5u : 6u;
    if (!in || n_in <= slot || in[slot].data == nullptr)
        return make_status(NXRT_INVALID_ARGUMENT, err("rmsnorm_prologue fusion requires the normalization weight at input " + std::to_string(slot)));
    if (n_in > (kn.gate_up_swiglu ? 8u : 7u)) return make_status(NXRT_INVALID_ARGUMENT, err("too many inputs for a node with the RMS-normalization prologue, got " + std::to_string(n_in)));
    const NxrtRocmTensorView& A = in[0];
    const NxrtRocmTensorView& G = in[slot];
    const uint64_t K = static_cast<uint64_t>(kn.k);
    if (A.dtype != NXRT_DT_FLOAT16 && A.dtype != NXRT_DT_BFLOAT16)
        return make_status(NXRT_INVALID_ARGUMENT, err(std::string("rmsnorm_prologue fusion needs Float16 or BFloat16 activations, got ") + dtype_name(A.dtype)));
    if (G.dtype != NXRT_DT_FLOAT32 && G.dtype != A.dtype)
        return make_status(NXRT_INVALID_ARGUMENT, err(std::string("gamma must have dtype Float32 or the activations' dtype, got ") + dtype_name(G.dtype)));
    if (!shape_is(G, {K})) return make_status(NXRT_INVALID_ARGUMENT, err("gamma must have shape [" + std::to_string(K) + "], got " + shape_str(G.shape, G.ndim)));
    if (A.ndim == 0 || A.shape[A.ndim - 1] != K)
        return make_status(NXRT_INVALID_ARGUMENT, err("A must have rank >= 1 and last dimension K=" + std::to_string(K) + ", got " + shape_str(A.shape, A.ndim)));
    if (K % 128 != 0)
        return make_status(NXRT_INVALID_ARGUMENT, err("rmsnorm_prologue fusion needs K to be a multiple of 128 (the reduction runs in 4-element chunks over 32 lanes), got K=" + std::to_string(K)));
    for (const NxrtRocmTensorView* t : {&A, &G}) {
        if (!is_contiguous(*t)) return make_status(NXRT_INVALID_ARGUMENT, err(std::string(t == &A ? "A" : "gamma") + " must be contiguous on the ROCm execution provider"));
        if (t->device_type != NXRT_DEVICE_ROCM || t->device_index != kn.ep->device)
            return make_status(NXRT_INVALID_ARGUMENT, err(std::string(t == &A ? "A" : "gamma") + " must live on ROCm device " + std::to_string(kn.ep->device)));
    }
    std::vector<NxrtRocmTensorView> views(in, in + n_in);
    views[slot].data = nullptr;                                  // the node proper sees no gamma
    uint32_t n_views = n_in;
    if (!kn.gate_up_swiglu) n_views = n_in < 6 ? n_in : 6;
    NormPrologue np;
    np.gamma = static_cast<const uint8_t*>(G.data) + G.byte_offset;
    np.gamma_dtype = static_cast<int>(G.dtype);
    np.epsilon = kn.rmsnorm_epsilon;
    np.owner = &kn;
    NxrtStatus st = kn.gate_up_swiglu ? execute_swiglu(kn, views.data(), n_views, out, n_out, workspace, workspace_bytes, &np)
                                      : execute_impl(kn, views.data(), n_views, out, n_out, workspace, workspace_bytes, false, &np);
    // "rmsnorm[...]": the kernel normalized the rows itself; "rmsnorm+...": a launch of its own did
    if (st.code == NXRT_OK) kn.variant = np.fused ? "rmsnorm[" + kn.variant + "]" : "rmsnorm+" + kn.variant;
    return st;
}

NxrtStatus vtable_execute(void* ctx, const void* const* inputs, uint32_t n_in, void** outputs, uint32_t n_out)
{
    return fenced([&]() -> NxrtStatus {
        auto* kn = static_cast<NxrtRocmMatMulNBits*>(ctx);
        if (!kn || !inputs || !outputs) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits: null pointer in kernel vtable execute");
        if (kn->gate_up_swiglu || kn->rmsnorm_prologue)
            return make_status(NXRT_INVALID_ARGUMENT, err("fused nodes (gate/up, RMS-normalization prologue) are not served through the raw kernel vtable; call nxrt_rocm_matmul_nbits_execute"));
        if (kn->rows_hint < 0)
            return make_status(NXRT_INVALID_ARGUMENT, err("the kernel vtable carries no shapes; create the kernel with a static shape for A"));
        const uint64_t K = kn->k, N = kn->n, BS = kn->block_size, kb = (K + BS - 1) / BS;
        const uint64_t a_shape[2] = {static_cast<uint64_t>(kn->rows_hint), K}, b_shape[3] = {N, kb, BS * static_cast<uint64_t>(kn->bits) / 8},
                       s_shape[2] = {N, kb}, z_shape[2] = {N, (kb * static_cast<uint64_t>(kn->bits) + 7) / 8}, bias_shape[1] = {N}, y_shape[2] = {static_cast<uint64_t>(kn->rows_hint), N};
        NxrtRocmTensorView in[6];
        std::memset(in, 0, sizeof(in));
        auto set = [&](NxrtRocmTensorView& v, const void* p, uint32_t dt, uint32_t nd, const uint64_t* sh) {
            v.data = const_cast<void*>(p);
            v.dtype = dt;
            v.ndim = nd;
            v.shape = sh;
            v.device_type = NXRT_DEVICE_ROCM;
            v.device_index = kn->ep->device;
        };
        set(in[0], n_in > 0 ? inputs[0] : nullptr, kn->vt_a_dtype, 2, a_shape);
        set(in[1], n_in > 1 ? inputs[1] : nullptr, NXRT_DT_UINT8, 3, b_shape);
        set(in[2], n_in > 2 ? inputs[2] : nullptr, kn->vt_scale_dtype, 2, s_shape);
        set(in[3], n_in > 3 ? inputs[3] : nullptr, NXRT_DT_UINT8, 2, z_shape);
        set(in[4], n_in > 4 ? inputs[4] : nullptr, NXRT_DT_INT32, 0, nullptr);
        set(in[5], n_in > 5 ? inputs[5] : nullptr, kn->vt_a_dtype, 1, bias_shape);
        NxrtRocmTensorView y;
        std::memset(&y, 0, sizeof(y));
        set(y, n_out > 0 ? outputs[0] : nullptr, kn->vt_y_dtype, 2, y_shape);
        return execute_impl(*kn, in, n_in, &y, n_out, nullptr, 0);
    });
}

void vtable_release(void* ctx)
{
    try {
        delete static_cast<NxrtRocmMatMulNBits*>(ctx);
    } catch (...) {
    }
}

}  // namespace

extern "C" {

int nxrt_rocm_ep_supports_matmul_nbits(const NxrtRocmEp* ep, const NxrtRocmMatMulNBitsAttrs* attrs, const NxrtTensorDesc* inputs, uint32_t n_inputs,
                                       char* reason, size_t reason_len)
{
    auto decline = [&](const std::string& why) {
        if (reason && reason_len) {
            std::strncpy(reason, why.c_str(), reason_len - 1);
            reason[reason_len - 1] = 0;
        }
        return 0;
    };
    if (reason && reason_len) reason[0] = 0;
    if (!attrs) return decline("MatMulNBits: null attributes");
    Check c;
    check_attrs(*attrs, c);
    if (c.failed) return decline(c.message);
    if (inputs) {
        const bool swiglu = attrs->struct_size >= offsetof(NxrtRocmMatMulNBitsAttrs, gate_up_swiglu) + sizeof(int64_t) &&
                            (attrs->present & (1u << kAttrGateUpSwiglu)) && attrs->gate_up_swiglu == 1;
        const bool rmsnorm = attrs->struct_size >= offsetof(NxrtRocmMatMulNBitsAttrs, rmsnorm_prologue) + sizeof(int64_t) &&
                             (attrs->present & (1u << kAttrRmsnormPrologue)) && attrs->rmsnorm_prologue == 1;
        if (rmsnorm) {
            if (attrs->K % 128 != 0) return decline(err("rmsnorm_prologue fusion needs K to be a multiple of 128, got K=" + std::to_string(attrs->K)));
            if (inputs[0].dtype != NXRT_DT_FLOAT16 && inputs[0].dtype != NXRT_DT_BFLOAT16)
                return decline(err(std::string("rmsnorm_prologue fusion needs Float16 or BFloat16 activations, got ") + dtype_name(inputs[0].dtype)));
            if (!swiglu) return n_inputs == 7 ? 1 : decline(err("rmsnorm_prologue fusion requires the normalization weight at input 6"));
            return (n_inputs >= 6 && n_inputs <= 8 && inputs[5].dtype != 0) ? 1 : decline(err("rmsnorm_prologue fusion requires the normalization weight at input 5"));
        }
        if (swiglu) {
            if (n_inputs < 5 || n_inputs > 8) return decline(err("gate/up SwiGLU fusion expects 5 to 8 inputs, got " + std::to_string(n_inputs)));
            if (inputs[0].dtype != NXRT_DT_FLOAT16 && inputs[0].dtype != NXRT_DT_BFLOAT16)
                return decline(err(std::string("gate/up SwiGLU fusion needs Float16 or BFloat16 activations, got ") + dtype_name(inputs[0].dtype)));
            if (n_inputs > 5 && inputs[5].dtype != 0) return decline(err("gate/up SwiGLU fusion received a normalization weight at input 5 but no RMS-norm prologue marker"));
            return 1;
        }
        if (n_inputs < 3 || n_inputs > 6) return decline("MatMulNBits: expected 3..=6 inputs, got " + std::to_string(n_inputs));
        if (!is_float_compute(inputs[0].dtype)) return decline(err(std::string("A must have dtype Float32, Float16, or BFloat16, got ") + dtype_name(inputs[0].dtype)));
        if (inputs[1].dtype != NXRT_DT_UINT8) return decline(err(std::string("B must have dtype Uint8, got ") + dtype_name(inputs[1].dtype)));
        if (!is_float_compute(inputs[2].dtype)) return decline(err(std::string("scales must have dtype Float32, Float16, or BFloat16, got ") + dtype_name(inputs[2].dtype)));
        const int64_t accuracy = (attrs->present & (1u << kAttrAccuracy)) ? attrs->accuracy_level : 0;
        if (n_inputs > 4 && inputs[4].dtype != 0 && accuracy == 4)
            return decline(err("accuracy_level=4 does not take g_idx on the ROCm execution provider. Why: its int8 kernels scale whole contiguous K blocks. "
                               "How to fix: export the weight without act-order, use accuracy_level=0, or run this node on the CPU execution provider"));
    }
    return 1;
}

NxrtStatus nxrt_rocm_matmul_nbits_create(NxrtRocmEp* ep, const NxrtRocmMatMulNBitsAttrs* attrs, const NxrtTensorDesc* input_shapes, uint32_t n_inputs,
                                         NxrtRocmMatMulNBits** out_kernel)
{
    return fenced([&]() -> NxrtStatus {
        if (!out_kernel) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits: null out_kernel");
        *out_kernel = nullptr;
        if (!attrs) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits: null attributes");
        Check c;
        check_attrs(*attrs, c);
        if (c.failed) return make_status(NXRT_INVALID_ARGUMENT, c.message);
        if (!ep) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits: null provider");
        auto* kn = new NxrtRocmMatMulNBits(ep);
        kn->k = attrs->K;
        kn->n = attrs->N;
        kn->block_size = attrs->block_size;
        kn->accuracy_level = (attrs->present & (1u << kAttrAccuracy)) ? attrs->accuracy_level : 0;
        kn->bits = (attrs->present & (1u << kAttrBits)) ? attrs->bits : 4;
        const bool has_folded_bias = attrs->struct_size >= offsetof(NxrtRocmMatMulNBitsAttrs, folded_bias) + sizeof(int64_t);
        kn->bias_post_round = has_folded_bias && (attrs->present & (1u << kAttrFoldedBias)) && attrs->folded_bias == 1;
        // flops::leading_rows: product of A's leading dims when all are static
        if (input_shapes && n_inputs >= 1 && input_shapes[0].ndim >= 1 && input_shapes[0].dims) {
            int64_t rows = 1;
            for (uint32_t i = 0; i + 1 < input_shapes[0].ndim; ++i) {
                const int64_t d = input_shapes[0].dims[i];
                if (d < 0) { rows = -1; break; }
                rows *= d;
            }
            kn->rows_hint = rows;
            kn->vt_a_dtype = input_shapes[0].dtype;
            kn->vt_y_dtype = input_shapes[0].dtype;
            kn->vt_scale_dtype = n_inputs >= 3 ? input_shapes[2].dtype : input_shapes[0].dtype;
        }
        const bool has_swiglu = attrs->struct_size >= offsetof(NxrtRocmMatMulNBitsAttrs, decomposed_silu) + sizeof(int64_t);
        kn->gate_up_swiglu = has_swiglu && (attrs->present & (1u << kAttrGateUpSwiglu)) && attrs->gate_up_swiglu == 1;
        kn->decomposed_silu = has_swiglu && (attrs->present & (1u << kAttrDecomposedSilu)) && attrs->decomposed_silu == 1;
        const bool has_rmsnorm = attrs->struct_size >= offsetof(NxrtRocmMatMulNBitsAttrs, rmsnorm_epsilon) + sizeof(double);
        kn->rmsnorm_prologue = has_rmsnorm && (attrs->present & (1u << kAttrRmsnormPrologue)) && attrs->rmsnorm_prologue == 1;
        if (has_rmsnorm && (attrs->present & (1u << kAttrRmsnormEpsilon))) kn->rmsnorm_epsilon = static_cast<float>(attrs->rmsnorm_epsilon);
        if (kn->gate_up_swiglu) {
            for (NxrtRocmMatMulNBits** child : {&kn->gate, &kn->up}) {
                auto* c2 = new NxrtRocmMatMulNBits(ep);
                c2->k = kn->k;
                c2->n = kn->n;
                c2->block_size = kn->block_size;
                c2->accuracy_level = kn->accuracy_level;
                c2->bits = kn->bits;
                c2->rows_hint = kn->rows_hint;
                c2->pair_member = true;
                *child = c2;
            }
        }
        std::memset(&kn->vtable, 0, sizeof(kn->vtable));
        kn->vtable.struct_size = sizeof(NxrtKernelVtable);
        kn->vtable.execute = vtable_execute;
        kn->vtable.release = vtable_release;
        kn->vtable.ctx = kn;
        *out_kernel = kn;
        return ok();
    });
}

void nxrt_rocm_matmul_nbits_set_constant_inputs(NxrtRocmMatMulNBits* kernel, const uint8_t* is_constant, uint32_t n)
{
    if (!kernel) return;
    if (kernel->gate_up_swiglu) {
        // [x, W_gate, scales_gate, W_up, scales_up, gamma, zp_gate, zp_up] -> each projection's [x, B, scales, zero_points]
        auto flag = [&](uint32_t i) { return is_constant && i < n && is_constant[i] != 0; };
        const uint32_t gate_slots[4] = {0, 1, 2, 6}, up_slots[4] = {0, 3, 4, 7};
        for (uint32_t i = 0; i < 4; ++i) {
            kernel->gate->constant_inputs[i] = flag(gate_slots[i]);
            kernel->up->constant_inputs[i] = flag(up_slots[i]);
        }
        return;
    }
    for (uint32_t i = 0; i < 6; ++i) kernel->constant_inputs[i] = (is_constant && i < n) ? is_constant[i] != 0 : false;
}

NxrtStatus nxrt_rocm_matmul_nbits_workspace_requirement(const NxrtRocmMatMulNBits* kernel, const NxrtTensorDesc* inputs, uint32_t n_inputs,
                                                        NxrtRocmWorkspaceRequirement* out)
{
    return fenced([&]() -> NxrtStatus {
        if (!kernel || !out) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits: null pointer in workspace_requirement");
        out->bytes = 0;
        out->alignment = 1;
        if (!inputs || n_inputs < 1 || inputs[0].ndim < 1 || !inputs[0].dims) {
            if (kernel->accuracy_level != 4) return ok();        // no shape, no slicing plan: the kernel manages without
            return make_status(NXRT_INVALID_ARGUMENT, err("workspace_requirement needs the shape of A"));
        }
        uint64_t m = 1;
        for (uint32_t i = 0; i + 1 < inputs[0].ndim; ++i) {
            if (inputs[0].dims[i] < 0) {
                if (kernel->accuracy_level != 4) return ok();
                return make_status(NXRT_INVALID_ARGUMENT, err("workspace_requirement needs static leading dimensions of A"));
            }
            m *= static_cast<uint64_t>(inputs[0].dims[i]);
        }
        if (kernel->gate_up_swiglu) {
            out->bytes = 2 * ((m * static_cast<uint64_t>(kernel->n) * 2 + 255) / 256 * 256);     // both projections, 16 bits each
            out->alignment = 256;
            return ok();
        }
        if (kernel->accuracy_level == 4) {
            out->bytes = acc4_workspace_bytes(*kernel, m);
            out->alignment = 256;
            return ok();
        }
        // float path: partial sums of a K-sliced prefill call (optional - without it the kernel allocates its own
        // outside a capture, or does not slice)
        RocmMatMulNBitsArgs probe;
        std::memset(&probe, 0, sizeof(probe));
        probe.a = probe.b = nullptr;
        probe.a_dtype = probe.scale_dtype = static_cast<int>(inputs[0].dtype);
        if (n_inputs > 2) probe.scale_dtype = static_cast<int>(inputs[2].dtype);
        probe.m = static_cast<int64_t>(m);
        probe.n = kernel->n;
        probe.k = kernel->k;
        probe.block_size = static_cast<int>(kernel->block_size);
        out->bytes = m > 16 ? rocm_prefill_mfma_scratch_bytes(&probe, kernel->ep->prefill_tile) : 0;
        out->alignment = out->bytes ? 256 : 1;
        return ok();
    });
}

NxrtStatus nxrt_rocm_matmul_nbits_execute(NxrtRocmMatMulNBits* kernel, const NxrtRocmTensorView* inputs, uint32_t n_inputs, NxrtRocmTensorView* outputs,
                                          uint32_t n_outputs, void* workspace_device, uint64_t workspace_bytes)
{
    return fenced([&]() -> NxrtStatus {
        if (!kernel) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits: null kernel");
        if (kernel->rmsnorm_prologue) return execute_normalized(*kernel, inputs, n_inputs, outputs, n_outputs, workspace_device, workspace_bytes);
        if (kernel->gate_up_swiglu) return execute_swiglu(*kernel, inputs, n_inputs, outputs, n_outputs, workspace_device, workspace_bytes);
        return execute_impl(*kernel, inputs, n_inputs, outputs, n_outputs, workspace_device, workspace_bytes);
    });
}

NxrtStatus nxrt_rocm_matmul_nbits_execute_static(NxrtRocmMatMulNBits* kernel, const NxrtRocmTensorView* inputs, uint32_t n_inputs, NxrtRocmTensorView* outputs,
                                                 uint32_t n_outputs)
{
    return fenced([&]() -> NxrtStatus {
        if (!kernel) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits: null kernel");
        if (kernel->rmsnorm_prologue || kernel->gate_up_swiglu)
            return make_status(NXRT_INVALID_ARGUMENT, err("execute_static serves plain MatMulNBits nodes; fused nodes (gate/up, RMS-normalization prologue) keep intermediates of their own - "
                                                          "call execute with a workspace"));
        NxrtRocmEp* ep = kernel->ep;
        if (!ep->static_scratch) return make_status(NXRT_INTERNAL_ERROR, err("the static scratch of this GPU was not resolved when the provider was created"));
        // Every provider of a GPU shares the array: a call behind another provider's call (another stream) waits for it on
        // the GPU. Under an open capture neither the wait nor the record can be taken (an event from outside a capture
        // cannot be waited for inside one): graphs recorded through several providers of one GPU are the host's to order.
        if (ep->capturing) return execute_impl(*kernel, inputs, n_inputs, outputs, n_outputs, ep->static_scratch, ep->static_scratch_bytes, true);
        NxrtStatus st = ep->bind();
        if (st.code != NXRT_OK) return st;
        st = hip_status(rocm_ffi_static_scratch_begin(static_cast<int>(ep->device), ep->stream), "hipStreamWaitEvent(static scratch)");
        if (st.code != NXRT_OK) return st;
        NxrtStatus run;
        try {
            run = execute_impl(*kernel, inputs, n_inputs, outputs, n_outputs, ep->static_scratch, ep->static_scratch_bytes, true);
        } catch (...) {
            rocm_ffi_static_scratch_end(static_cast<int>(ep->device), ep->stream);
            throw;
        }
        st = hip_status(rocm_ffi_static_scratch_end(static_cast<int>(ep->device), ep->stream), "hipEventRecord(static scratch)");
        return run.code != NXRT_OK ? run : st;
    });
}

uint64_t nxrt_rocm_matmul_nbits_estimated_flops(const NxrtRocmMatMulNBits* kernel)
{
    if (!kernel || kernel->rows_hint < 0) return 0;
    return (kernel->gate_up_swiglu ? 4ull : 2ull) * static_cast<uint64_t>(kernel->rows_hint) * static_cast<uint64_t>(kernel->n) * static_cast<uint64_t>(kernel->k);
}

const char* nxrt_rocm_matmul_nbits_last_variant(const NxrtRocmMatMulNBits* kernel) { return kernel ? kernel->variant.c_str() : ""; }

void nxrt_rocm_matmul_nbits_last_metrics(const NxrtRocmMatMulNBits* kernel, uint64_t* flops, uint64_t* bytes)
{
    if (flops) *flops = kernel ? kernel->last_flops : 0;
    if (bytes) *bytes = kernel ? kernel->last_bytes : 0;
}

void nxrt_rocm_matmul_nbits_release(NxrtRocmMatMulNBits* kernel) { vtable_release(kernel); }

NxrtStatus nxrt_rocm_matmul_nbits_set_block_acc_probe(NxrtRocmMatMulNBits* kernel, int32_t* acc_device, uint64_t capacity_elements)
{
    if (!kernel) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits: null kernel");
    if (kernel->gate_up_swiglu) return make_status(NXRT_INVALID_ARGUMENT, err("the block-accumulator probe is not offered on the fused gate/up node"));
    std::lock_guard<std::mutex> lock(kernel->mu);
    kernel->acc_probe = acc_device;
    kernel->acc_probe_elems = acc_device ? capacity_elements : 0;
    return ok();
}

uint64_t nxrt_rocm_matmul_nbits_retired_buffers(const NxrtRocmMatMulNBits* kernel) { return kernel ? kernel->retired.size() : 0; }

NxrtStatus nxrt_rocm_matmul_nbits_as_vtable(NxrtRocmMatMulNBits* kernel, NxrtKernelVtable** out_vtable)
{
    if (!kernel || !out_vtable) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits: null pointer in as_vtable");
    *out_vtable = &kernel->vtable;
    return ok();
}

NxrtStatus nxrt_rocm_matmul_nbits_dequantize(NxrtRocmEp* ep, const void* b, const void* scales, uint32_t scale_dtype, const void* zp, uint64_t n, uint64_t k,
                                             uint32_t block_size, float* out_nk)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep || !b || !scales || !out_nk) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits dequantize: null pointer");
        if (!is_float_compute(scale_dtype)) return make_status(NXRT_INVALID_ARGUMENT, err(std::string("scales must have dtype Float32, Float16, or BFloat16, got ") + dtype_name(scale_dtype)));
        if (block_size < 16 || (block_size & (block_size - 1)) != 0) return make_status(NXRT_INVALID_ARGUMENT, err("block_size must be a power of two and at least 16, got " + std::to_string(block_size)));
        NxrtStatus st = ep->bind();
        if (st.code != NXRT_OK) return st;
        ep->launches.fetch_add(1);
        return hip_status(rocm_launch_dequant_f32(static_cast<const uint8_t*>(b), scales, static_cast<int>(scale_dtype), static_cast<const uint8_t*>(zp),
                                                  static_cast<int64_t>(n), static_cast<int64_t>(k), static_cast<int>(block_size), out_nk, ep->stream),
                          "MatMulNBits dequantize launch");
    });
}

NxrtStatus nxrt_rocm_matmul_nbits_dequantize_bits(NxrtRocmEp* ep, const void* b, const void* scales, uint32_t scale_dtype, const void* zp, uint64_t n,
                                                  uint64_t k, uint32_t block_size, uint32_t bits, float* out_nk)
{
    if (bits == 4) return nxrt_rocm_matmul_nbits_dequantize(ep, b, scales, scale_dtype, zp, n, k, block_size, out_nk);
    return fenced([&]() -> NxrtStatus {
        if (!ep || !b || !scales || !out_nk) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits dequantize: null pointer");
        if (bits != 2 && bits != 8) return make_status(NXRT_INVALID_ARGUMENT, err("bits must be 2, 4 or 8, got " + std::to_string(bits)));
        if (!is_float_compute(scale_dtype)) return make_status(NXRT_INVALID_ARGUMENT, err(std::string("scales must have dtype Float32, Float16, or BFloat16, got ") + dtype_name(scale_dtype)));
        if (block_size < 16 || (block_size & (block_size - 1)) != 0) return make_status(NXRT_INVALID_ARGUMENT, err("block_size must be a power of two and at least 16, got " + std::to_string(block_size)));
        NxrtStatus st = ep->bind();
        if (st.code != NXRT_OK) return st;
        ep->launches.fetch_add(1);
        return hip_status(rocm_launch_dequant_nbits(static_cast<const uint8_t*>(b), scales, static_cast<int>(scale_dtype), static_cast<const uint8_t*>(zp),
                                                    static_cast<int64_t>(n), static_cast<int64_t>(k), static_cast<int>(block_size), static_cast<int>(bits),
                                                    ROCM_DT_F32, out_nk, ep->stream),
                          "MatMulNBits dequantize launch");
    });
}

NxrtStatus nxrt_rocm_matmul_nbits_quantize_a(NxrtRocmEp* ep, const void* a, uint32_t a_dtype, uint64_t m, uint64_t k, uint32_t block_size, uint32_t rounding,
                                             int8_t* qa, float* qscale)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep || !a || !qa || !qscale) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits quantize_a: null pointer");
        if (!is_float_compute(a_dtype)) return make_status(NXRT_INVALID_ARGUMENT, err(std::string("A must have dtype Float32, Float16, or BFloat16, got ") + dtype_name(a_dtype)));
        if (rounding > 1) return make_status(NXRT_INVALID_ARGUMENT, err("rounding must be 0 (ties to even) or 1 (ties away from zero)"));
        if (block_size < 16 || (block_size & (block_size - 1)) != 0) return make_status(NXRT_INVALID_ARGUMENT, err("block_size must be a power of two and at least 16, got " + std::to_string(block_size)));
        NxrtStatus st = ep->bind();
        if (st.code != NXRT_OK) return st;
        ep->launches.fetch_add(1);
        return hip_status(rocm_launch_quantize_a(a, static_cast<int>(a_dtype), static_cast<int64_t>(m), static_cast<int64_t>(k), static_cast<int>(block_size),
                                                 static_cast<int>(rounding), qa, qscale, nullptr, ep->stream),
                          "MatMulNBits quantize_a launch");
    });
}

NxrtStatus nxrt_rocm_matmul_nbits_block_acc(NxrtRocmEp* ep, const int8_t* qa, const void* b, const void* zp, uint64_t m, uint64_t n, uint64_t k,
                                            uint32_t block_size, int32_t* acc)
{
    return fenced([&]() -> NxrtStatus {
        if (!ep || !qa || !b || !acc) return make_status(NXRT_INVALID_ARGUMENT, "MatMulNBits block_acc: null pointer");
        if (block_size < 16 || (block_size & (block_size - 1)) != 0) return make_status(NXRT_INVALID_ARGUMENT, err("block_size must be a power of two and at least 16, got " + std::to_string(block_size)));
        NxrtStatus st = ep->bind();
        if (st.code != NXRT_OK) return st;
        ep->launches.fetch_add(1);
        return hip_status(rocm_launch_block_acc_i32(qa, static_cast<const uint8_t*>(b), static_cast<const uint8_t*>(zp), static_cast<int64_t>(m),
                                                    static_cast<int64_t>(n), static_cast<int64_t>(k), static_cast<int>(block_size), acc, ep->stream),
                          "MatMulNBits block_acc launch");
    });
}

}  // extern "C"
