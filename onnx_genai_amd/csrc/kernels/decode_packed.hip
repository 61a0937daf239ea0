// Decode path of MatMulNBits over weights repacked for streaming (f16/bf16 activations; M <= 16 at every width, up to 64 rows when N is large).
//
// When B, scales and zero points are constant initializers, the kernel object repacks them once into
// the order in which the split-K MFMA kernel consumes them, so that every vector load of a wave is
// one contiguous kilobyte and everything a group of four 128-element tiles needs lies in one chunk:
//
//   chunk(column group cg of 16 columns, tile group tg of 4 tiles) =
//       4 x [lane 0..63] 16 bytes of weights      lane (c = lane % 16, g = lane / 16) of tile u at u*1024 + lane*16
//       16 x record(column c)                     scales of the group's blocks, then one zero-point byte per block
//
// Dword j of a lane's 16 bytes holds the eight weights k = tile*128 + j*32 + g*8 + e (e = 0..7) of column c:
// one MFMA therefore covers 32 consecutive k and never mixes two blocks, whatever the block size, and no
// cross-lane transpose is needed. Inside the dword, element e sits at bit 4*(e/2) + 16*(e%2), so that
// ((w >> 4i) & 0x000F000F) | magic is the pair (e = 2i, 2i+1) as two 16-bit floats - seven VALU
// instructions per eight weights. The arithmetic is that of the unpacked decode kernel: magic-number
// operands, a second MFMA with the constant -(magic + zp), one scale per block on the f32 accumulator.
//
// The copy costs one extra byte of device memory per byte of weights plus 2 to 6 % for the records; it is
// read instead of the caller's tensors, which are not touched again.
#include <type_traits>

#include "mfma_common.hiph"
#include "swiglu.hiph"

namespace mnb {

typedef __attribute__((ext_vector_type(8))) _Float16 half8p_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8p_t;
typedef __attribute__((ext_vector_type(4))) float float4p_t;
typedef __attribute__((ext_vector_type(2))) _Float16 half2p_t;

constexpr int kGroupTiles = 4;
constexpr int kChunkWeights = kGroupTiles * 1024;
constexpr int kRowPitchP = 272;   // bytes between activation rows in LDS: 256 + 16

__host__ __device__ constexpr int packed_record_bytes(int bs, int scale_bytes)
{
    const int nb = kGroupTiles * 128 / bs;
    return (nb * scale_bytes + nb + 15) / 16 * 16;
}

struct PackParams {
    const uint8_t* b;
    const void* scales;
    const uint8_t* zp;
    uint8_t* out;
    int64_t n, kb, row_bytes, zp_row;
    int bs_log2, scale_bytes;
    int groups;             // tile groups per column group
    int chunk_bytes, record;
};

// grid (tile group, column group), 256 threads: four dwords of weights per thread, then one record per thread < 16.
__global__ __launch_bounds__(256) void pack_decode_kernel(PackParams p)
{
    const int t = threadIdx.x;
    const int64_t tg = blockIdx.x, cg = blockIdx.y;
    uint8_t* chunk = p.out + (cg * p.groups + tg) * static_cast<int64_t>(p.chunk_bytes);
    const int64_t padded_k = p.kb << p.bs_log2;
    const uint32_t* b32 = reinterpret_cast<const uint32_t*>(p.b);
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int x = it * 256 + t;              // dword of the weight part: u*256 + lane*4 + j
        const int u = x >> 8, lane = (x >> 2) & 63, j = x & 3;
        const int64_t col = cg * 16 + (lane & 15);
        const int64_t k = (tg * kGroupTiles + u) * 128 + j * 32 + (lane >> 4) * 8;
        uint32_t out = 0;
        if (col < p.n && k < padded_k) {
            const uint32_t w = b32[(col * p.row_bytes + (k >> 1)) >> 2];   // eight weights, element e at bit 4e
            uint32_t lo = w & 0x0f0f0f0fu, hi = (w >> 4) & 0x0f0f0f0fu;    // even / odd elements, one per byte
            lo = (lo | (lo >> 4)) & 0x00ff00ffu;
            lo = (lo | (lo >> 8)) & 0x0000ffffu;                            // e0 | e2 << 4 | e4 << 8 | e6 << 12
            hi = (hi | (hi >> 4)) & 0x00ff00ffu;
            hi = (hi | (hi >> 8)) & 0x0000ffffu;
            out = lo | (hi << 16);
        }
        reinterpret_cast<uint32_t*>(chunk)[x] = out;
    }
    if (t < 16) {
        const int nb = (kGroupTiles * 128) >> p.bs_log2;
        uint8_t* rec = chunk + kChunkWeights + t * p.record;
        const int64_t col = cg * 16 + t;
        for (int i = 0; i < p.record; ++i) rec[i] = 0;
        for (int bi = 0; bi < nb; ++bi) {
            const int64_t blk = tg * nb + bi;
            const bool live = col < p.n && blk < p.kb;
            if (p.scale_bytes == 4) {
                reinterpret_cast<uint32_t*>(rec)[bi] = live ? static_cast<const uint32_t*>(p.scales)[col * p.kb + blk] : 0u;
            } else {
                reinterpret_cast<uint16_t*>(rec)[bi] = live ? static_cast<const uint16_t*>(p.scales)[col * p.kb + blk] : static_cast<uint16_t>(0);
            }
            rec[nb * p.scale_bytes + bi] = static_cast<uint8_t>(live ? zero_point_of(p.zp ? p.zp + col * p.zp_row : nullptr, blk) : 8);
        }
    }
}

struct PackedParams {
    const uint16_t* a;
    const uint8_t* packed;
    const uint8_t* packed_up;   // paired launch only: the up projection's repacked copy (`packed` is the gate's)
    int decomposed_silu;        // paired launch only
    const void* bias;
    void* y;
    int64_t m, n, k;
    int64_t cg_stride;      // bytes of one column group: groups * chunk_bytes
    int groups;             // tile groups
    int groups_per_wave;
    int chunk_bytes;
    int bias_dtype, y_dtype;
    uint32_t nibble_mask;   // 0x000F000F
    uint32_t magic;         // two 16-bit magic exponents; a kernel argument so that it stays in a scalar register
    const void* gamma;      // NORM kernels: the RMS-normalization weight [k], f32 or the activations' type
    int gamma_f32;
    float norm_epsilon;
};

template <bool BF16>
__device__ __forceinline__ float4p_t mfma16p(const uint4& act, const uint4& wgt, float4p_t acc)
{
    if constexpr (BF16) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8p_t, act), __builtin_bit_cast(bf16x8p_t, wgt), acc, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8p_t, act), __builtin_bit_cast(half8p_t, wgt), acc, 0, 0, 0);
}

template <int NR, int NA, int NG>
struct PackedGroup {
    uint4 w[kGroupTiles];
    uint4 r[NR];
    uint4 a[NA];
    uint4 gm[NG];     // NORM: the normalization weights of the activation pieces (two loads each: f32 weights are 32 bytes a piece)
};

// v + (v of the lane a DPP control selects): quad_perm [1,0,3,2] = 0xB1, [2,3,0,1] = 0x4E, row_half_mirror = 0x141,
// row_mirror = 0x140 - applied in that order they leave the sum over 4, 8, 16 lanes in every lane of the run.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v)
{
    return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

template <int CTRL>
__device__ __forceinline__ float dpp_max(float v)
{
    return fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false)));
}
template <int CTRL>
__device__ __forceinline__ int dpp_addi(int v)
{
    return v + __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false);
}

// Sum of the 8 activations of one 16-byte piece, in f32.
template <bool BF16>
__device__ __forceinline__ float sum_piece(const uint4& v)
{
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if constexpr (BF16) {
            s += __uint_as_float(d[i] << 16);
            s += __uint_as_float(d[i] & 0xffff0000u);
        } else {
            const half2p_t h = __builtin_bit_cast(half2p_t, d[i]);
            s += static_cast<float>(h.x);
            s += static_cast<float>(h.y);
        }
    }
    return s;
}

// Sum over the BS / 8 consecutive lanes that hold one block's pieces; every lane of the run receives it.
template <int BS>
__device__ __forceinline__ float block_sum(float s)
{
    s = dpp_add<0xB1>(s);
    s = dpp_add<0x4E>(s);
    if constexpr (BS >= 64) s = dpp_add<0x141>(s);
    if constexpr (BS >= 128) s = dpp_add<0x140>(s);
    return s;
}

// BF16: activation element type. BS: block size. MR: rows staged (1, 4 or 16; M <= MR). ST: storage type of the scales.
// SETS: register sets of one group each. 2: the next group's loads are in flight while this one is multiplied - for
// launches with few waves, where each wave must cover memory latency by itself. 1: no prefetch, 62 registers, eight
// waves per SIMD - for launches with thousands of waves, where the other resident waves cover it better (measured on
// 3584 -> 37888: 15.6 us against 17.0 us). With two sets the one-row, block-128, 16-bit-scale variant fits 96
// registers without spilling (a fifth wave per SIMD); the other variants keep the compiler's own choice.
// PAIR: the fused gate/up node. The first half of the workgroup's waves runs the gate projection's column group, the
// second half the up projection's - each half exactly as a launch of its own would (same split of K, same order of
// summation, so the same f32 totals) - and the epilogue writes round16(silu(round16(gate)) * round16(up)).
// NORM (up to 4 rows): the RMS-normalization prologue inside the kernel (the CUDA provider's form,
// onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:3747-3783). Every wave first sums the squares of the call's rows in
// the reference's order (32 lanes, four running sums over 4-element chunks, (s0 + s1) + (s2 + s3), a shuffle tree over
// 32 lanes: half a wavefront plays one warp, so a wave covers two rows per pass), then replaces each activation piece it
// loads by round16((a * inv_std) * gamma) before the piece is staged - the values a separate normalization launch
// would have written, bit for bit.
template <bool BF16, int BS, int MR, typename ST, int SETS, bool PAIR, bool NORM = false>
__global__ __launch_bounds__((BS == 128 && sizeof(ST) == 2 && (MR != 16 || BF16)) ? 1024 : 512)   // block 128, 16-bit scales, up to 4 rows: up to 16 waves split a long K
__attribute__((amdgpu_waves_per_eu((BS == 128 && MR == 1 && sizeof(ST) == 2 && !NORM) ? (SETS == 1 ? 8 : 5) : 1)))
void decode_packed_kernel(PackedParams p)
{
    static_assert(!NORM || MR <= 4, "the fused normalization covers up to four rows");
    constexpr int U = kGroupTiles;
    constexpr int NBT = 128 / BS;
    constexpr int NB = U * NBT;
    constexpr int R = packed_record_bytes(BS, static_cast<int>(sizeof(ST)));
    constexpr int NR = R / 16;
    constexpr int RQ = MR == 1 ? 1 : MR / 4;       // loads per tile: each covers four rows (row g + 4 i, piece c)
    constexpr int NA = MR == 1 ? 1 : U * RQ;
    constexpr int NGP = MR == 1 ? 1 : U;           // activation pieces with distinct elements per group (rows share them)
    constexpr int NG = NORM ? 2 * NGP : 1;
    constexpr int kStageBytes = MR == 1 ? 1024 : MR * kRowPitchP;
    constexpr float kMagicF = BF16 ? 128.0f : 1024.0f;
    constexpr uint32_t kMagicNeg = BF16 ? 0xC300C300u : 0xE400E400u;
    // How the magic offset and the zero point leave the accumulator. Launches of many short waves (one row, no
    // prefetch) are bound by what a wave computes per byte: there they leave through the block's activation sum,
    // y += scale * (acc - (magic + zp) * sum a), one FMA per block. Elsewhere a second MFMA per 32 elements against
    // -(magic + zp) does it: more matrix-core work, but nothing between a wave's loads and its first MFMA, which is
    // what the few-wave launches are sensitive to (measured: 3584 -> 37888 16.4 against 17.0 us and 3584 -> 152064 54.5
    // against 59 us with the sums; 18944 -> 3584 12.2 against 11.4 us, so not there).
    constexpr bool SUMS = MR == 1 && SETS == 1;
    // With one row staged every accumulator row is a copy of row 0: only component 0 is scaled and reduced.
    constexpr int kRowsKept = MR == 1 ? 1 : 4;
    constexpr int kBlockLanes = BS / 8;         // lanes whose 16-byte pieces make up one block
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = PAIR ? static_cast<int>(blockDim.x >> 7) : static_cast<int>(blockDim.x >> 6);      // per projection
    const bool second = PAIR && wave >= waves;                                                           // wave-uniform
    const int split = second ? wave - waves : wave;                                                      // this wave's share of K
    const int c = lane & 15;
    const int g = lane >> 4;
    const int64_t n_base = static_cast<int64_t>(blockIdx.x) * 16;

    const __amdgpu_buffer_rsrc_t srd_p = make_srd((second ? p.packed_up : p.packed) + static_cast<int64_t>(blockIdx.x) * p.cg_stride, static_cast<uint64_t>(p.cg_stride));
    const __amdgpu_buffer_rsrc_t srd_a = make_srd(p.a, static_cast<uint64_t>(p.m * p.k) * 2);
    const __amdgpu_buffer_rsrc_t srd_g = make_srd(NORM ? p.gamma : p.a, NORM ? static_cast<uint64_t>(p.k) * (p.gamma_f32 ? 4 : 2) : 0);

    const uint32_t w_off = static_cast<uint32_t>(lane * 16);
    const uint32_t r_off = static_cast<uint32_t>(kChunkWeights + c * R);
    // compact activation load. MR = 1: piece c of tile g of the group. MR = 4 / 16: row g (+ 4 i), piece c of one tile.
    const uint32_t a_off = MR == 1 ? static_cast<uint32_t>(g * 256 + c * 16) : static_cast<uint32_t>(g) * static_cast<uint32_t>(p.k) * 2u + static_cast<uint32_t>(c * 16);
    unsigned char* stage = smem + wave * (2 * kStageBytes);
    const uint32_t st_write = MR == 1 ? static_cast<uint32_t>(lane * 16) : static_cast<uint32_t>(g * kRowPitchP + c * 16);
    // operand of MFMA j: elements j*32 + g*8 .. +8 of the tile, of row c % MR
    const uint32_t st_read = (MR == 1 ? 0u : static_cast<uint32_t>((c & (MR - 1)) * kRowPitchP)) + static_cast<uint32_t>(g * 16);
    const uint32_t mask = __builtin_amdgcn_mov_dpp(p.nibble_mask, 0xE4, 0xf, 0xf, false), magic = p.magic;

    float4p_t y = {0.f, 0.f, 0.f, 0.f};
    float4p_t acc = {0.f, 0.f, 0.f, 0.f};

    const int g_begin = split * p.groups_per_wave;
    const int g_end = min(g_begin + p.groups_per_wave, p.groups);

    using Grp = PackedGroup<NR, NA, NG>;
    // No branch in here: a group past the wave's last one (the prefetch of the final iteration) gets every offset out of
    // range, which fetches nothing and returns zeros - weights 0, scale 0, activations 0: a group that adds nothing.
    // With a branch instead, the compiler waits for all loads in flight at the next use, the prefetch included.
    auto fetch_group = [&](Grp& grp, int gi) {
        const uint32_t oor = gi < g_end ? 0u : kOutOfRange;        // or-ed in: any offset with these bits is out of range
        const uint32_t soff = static_cast<uint32_t>(gi) * static_cast<uint32_t>(p.chunk_bytes);
        const int t0 = gi * U;
        // every offset first, then the loads back to back: vector arithmetic between two loads can land in a register
        // that an outstanding load still owns, and then waits for it
        uint32_t a_voff[NA];
#pragma unroll
        for (int x = 0; x < NA; ++x) {
            const int u = x / RQ, i = x % RQ;
            const int tile = MR == 1 ? t0 + g : t0 + u;
            const bool beyond = static_cast<int64_t>(tile) * 128 + c * 8 + 8 > p.k;        // K is a multiple of 8: a piece is all in or all out
            // rows past M lie past the end of the activations' range and read as zeros
            a_voff[x] = (beyond ? kOutOfRange : a_off + static_cast<uint32_t>(4 * i) * static_cast<uint32_t>(p.k) * 2u) | oor;
        }
        uint32_t g_voff[NG];
        if constexpr (NORM) {
#pragma unroll
            for (int x = 0; x < NGP; ++x) {
                const int tile = MR == 1 ? t0 + g : t0 + x;
                const bool beyond = static_cast<int64_t>(tile) * 128 + c * 8 + 8 > p.k;
                const uint32_t first = static_cast<uint32_t>(tile * 128 + c * 8) * (p.gamma_f32 ? 4u : 2u);
                g_voff[2 * x] = (beyond ? kOutOfRange : first) | oor;
                g_voff[2 * x + 1] = ((beyond || !p.gamma_f32) ? kOutOfRange : first + 16u) | oor;
            }
        }
        const uint32_t w_voff = w_off | oor, r_voff = r_off | oor;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < U; ++u) grp.w[u] = load16(srd_p, w_voff + static_cast<uint32_t>(u * 1024), soff);
#pragma unroll
        for (int i = 0; i < NR; ++i) grp.r[i] = load16(srd_p, r_voff + static_cast<uint32_t>(i * 16), soff);
#pragma unroll
        for (int x = 0; x < NA; ++x) grp.a[x] = load16(srd_a, a_voff[x], static_cast<uint32_t>(MR == 1 ? t0 : t0 + x / RQ) * 256u);
        if constexpr (NORM) {
#pragma unroll
            for (int x = 0; x < NG; ++x) grp.gm[x] = load16(srd_g, g_voff[x], 0u);
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    // ---- NORM: 1 / sqrt(mean(a^2) + eps) of this lane's row (row 0, or row g of up to four) ----
    // With one row the wave's first group is requested before, so that its trip to memory overlaps the sums (with four
    // rows the compiler would keep the group in scratch memory across the passes).
    constexpr bool kEarly = NORM && MR == 1;
    Grp ga;
    if constexpr (kEarly || SETS == 2) fetch_group(ga, g_begin);
    float inv_std = 1.0f;
    if constexpr (NORM) {
        // One wave per pair of rows does the sums (every wave doing them would re-read the rows once per wave: at 3584 ->
        // 2 x 18944 three times the bytes of the weights) and leaves the results in LDS behind the staging buffers.
        float* inv_shared = reinterpret_cast<float*>(smem + (blockDim.x >> 6) * (2 * kStageBytes));
        const int all_waves = static_cast<int>(blockDim.x >> 6);
        const int l32 = lane & 31;
        const int items = static_cast<int>(p.k >> 7);
#pragma unroll
        for (int pass = 0; pass < (MR == 1 ? 1 : 2); ++pass) {
            if (wave != pass % all_waves) continue;              // (wave-uniform)
            const int row = 2 * pass + (lane >> 5);              // rows past M lie past the range and read as zeros
            const uint32_t base = static_cast<uint32_t>(row) * static_cast<uint32_t>(p.k) * 2u + static_cast<uint32_t>(l32 * 8);
            float inv = 1.0f;
            if (MR == 1 || 2 * pass < p.m) {                     // (wave-uniform) rows 2 and 3 only where the call has them
                float ss0 = 0.f, ss1 = 0.f, ss2 = 0.f, ss3 = 0.f;
                // sixteen loads in flight at a time: one after the other they would cost a trip to the cache each. A chunk past
                // the row reads as zeros, and fma(0, 0, s) = s.
                constexpr int kBatch = 16;
                for (int first = 0; first < items; first += kBatch) {
                    uint32_t d0[kBatch], d1[kBatch];
#pragma unroll
                    for (int i = 0; i < kBatch; ++i) {
                        const auto raw = __builtin_amdgcn_raw_buffer_load_b64(srd_a, static_cast<int>(first + i < items ? base : kOutOfRange), (first + i) * 256, 0);
                        d0[i] = raw[0];
                        d1[i] = raw[1];
                    }
#pragma unroll
                    for (int i = 0; i < kBatch; ++i) {
                        const float v0 = BF16 ? __uint_as_float(d0[i] << 16) : f16_bits_to_f32(static_cast<uint16_t>(d0[i]));
                        const float v1 = BF16 ? __uint_as_float(d0[i] & 0xffff0000u) : f16_bits_to_f32(static_cast<uint16_t>(d0[i] >> 16));
                        const float v2 = BF16 ? __uint_as_float(d1[i] << 16) : f16_bits_to_f32(static_cast<uint16_t>(d1[i]));
                        const float v3 = BF16 ? __uint_as_float(d1[i] & 0xffff0000u) : f16_bits_to_f32(static_cast<uint16_t>(d1[i] >> 16));
                        ss0 = __fmaf_rn(v0, v0, ss0);
                        ss1 = __fmaf_rn(v1, v1, ss1);
                        ss2 = __fmaf_rn(v2, v2, ss2);
                        ss3 = __fmaf_rn(v3, v3, ss3);
                    }
                }
                float ss = __fadd_rn(__fadd_rn(ss0, ss1), __fadd_rn(ss2, ss3));
#pragma unroll
                for (int off = 16; off > 0; off >>= 1) ss = __fadd_rn(ss, __shfl_down(ss, off, 32));
                // sqrtf and the divisions are correctly rounded (the compiler's default for f32)
                inv = __fdiv_rn(1.0f, sqrtf(__fadd_rn(__fdiv_rn(ss, static_cast<float>(p.k)), p.norm_epsilon)));
            }
            if (l32 == 0) inv_shared[row] = inv;
        }
        __syncthreads();
        inv_std = inv_shared[MR == 1 ? 0 : g];
    }
    // round16((a * inv_std) * gamma) of one 16-byte piece; g0 / g1: the piece's weights (16-bit: all eight in g0)
    auto normalized = [&](const uint4& a, const uint4& g0, const uint4& g1) -> uint4 {
        const uint32_t ad[4] = {a.x, a.y, a.z, a.w};
        const uint32_t gd[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
        uint32_t out[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float v0 = BF16 ? __uint_as_float(ad[i] << 16) : f16_bits_to_f32(static_cast<uint16_t>(ad[i]));
            const float v1 = BF16 ? __uint_as_float(ad[i] & 0xffff0000u) : f16_bits_to_f32(static_cast<uint16_t>(ad[i] >> 16));
            float w0, w1;
            if (p.gamma_f32) {
                w0 = __uint_as_float(gd[2 * i]);
                w1 = __uint_as_float(gd[2 * i + 1]);
            } else {
                w0 = BF16 ? __uint_as_float(gd[i] << 16) : f16_bits_to_f32(static_cast<uint16_t>(gd[i]));
                w1 = BF16 ? __uint_as_float(gd[i] & 0xffff0000u) : f16_bits_to_f32(static_cast<uint16_t>(gd[i] >> 16));
            }
            // (as_f32: the product is rounded to f32 before the 16-bit conversion sees it, never folded into one mixed-precision multiply)
            const float y0 = as_f32(__fmul_rn(__fmul_rn(v0, inv_std), w0)), y1 = as_f32(__fmul_rn(__fmul_rn(v1, inv_std), w1));
            const uint32_t lo = BF16 ? f32_to_bf16_bits(y0) : f32_to_f16_bits(y0);
            const uint32_t hi = BF16 ? f32_to_bf16_bits(y1) : f32_to_f16_bits(y1);
            out[i] = lo | (hi << 16);
        }
        return make_uint4(out[0], out[1], out[2], out[3]);
    };
    // `asum` (with SUMS): this lane's block sum of the group's tile lane / 16 (one load covers the group's four tiles).
    auto compute_tile = [&](const Grp& grp, int u, int parity, float asum) {
        unsigned char* st = stage + (MR == 1 ? parity : (u & 1)) * kStageBytes;
        if constexpr (MR != 1) {
#pragma unroll
            for (int i = 0; i < RQ; ++i) {
                if constexpr (NORM) *reinterpret_cast<uint4*>(st + st_write + i * 4 * kRowPitchP) = normalized(grp.a[u * RQ + i], grp.gm[2 * u], grp.gm[2 * u + 1]);
                else *reinterpret_cast<uint4*>(st + st_write + i * 4 * kRowPitchP) = grp.a[u * RQ + i];
            }
            lds_order();
        }
        uint4 av[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) av[j] = *reinterpret_cast<const uint4*>(st + st_read + (MR == 1 ? u * 256 : 0) + j * 64);
        const uint32_t wd[4] = {grp.w[u].x, grp.w[u].y, grp.w[u].z, grp.w[u].w};
        uint32_t rr[NR * 4];
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            rr[4 * i] = grp.r[i].x;
            rr[4 * i + 1] = grp.r[i].y;
            rr[4 * i + 2] = grp.r[i].z;
            rr[4 * i + 3] = grp.r[i].w;
        }
        // Every dword of the record counts as used here, also the padding at its end: a destination register of a load
        // that the compiler knows to be dead is handed out again at once, and writing it waits for the load in flight.
#pragma unroll
        for (int i = 0; i < NR * 4; ++i) asm volatile("" : : "v"(rr[i]));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int bi = u * NBT + (j * 32) / BS;                          // block of the group (compile-time)
            const int zbyte = NB * static_cast<int>(sizeof(ST)) + bi;
            const uint32_t w = wd[j];
            uint4 op;
            op.x = (w & mask) | magic;
            op.y = ((w >> 4) & mask) | magic;
            op.z = ((w >> 8) & mask) | magic;
            op.w = ((w >> 12) & mask) | magic;
            acc = mfma16p<BF16>(av[j], op, acc);
            const uint32_t z = (rr[zbyte / 4] >> ((zbyte % 4) * 8)) & 0xffu;
            if constexpr (!SUMS) {
                const uint32_t zpair = kMagicNeg | (z * 0x00010001u);
                acc = mfma16p<BF16>(av[j], make_uint4(zpair, zpair, zpair, zpair), acc);
            }
            if (((j + 1) * 32) % BS == 0 || j == 3) {
                float sf;
                if constexpr (sizeof(ST) == 4) {
                    sf = __uint_as_float(rr[bi]);
                } else {
                    const uint32_t raw = (rr[bi / 2] >> ((bi % 2) * 16)) & 0xffffu;
                    sf = BF16 ? __uint_as_float(raw << 16) : f16_bits_to_f32(static_cast<uint16_t>(raw));
                }
                if constexpr (SUMS) {
                    // the block's pieces sit in lanes first .. first + kBlockLanes - 1 of lane group u; any of them has the sum
                    const int first = u * 16 + ((j * 32) / BS) % NBT * kBlockLanes;
                    const float sa = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(asum), first));
                    const float off = kMagicF + static_cast<float>(z);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if (r < kRowsKept) y[r] = fmaf(sf, fmaf(-off, sa, acc[r]), y[r]);      // the product is not rounded on its own
                        acc[r] = 0.f;
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if (r < kRowsKept) y[r] = fmaf(sf, acc[r], y[r]);
                        acc[r] = 0.f;
                    }
                }
            }
        }
    };
    auto run_group = [&](const Grp& cur, Grp& next, int gi, int parity, bool prefetch) {
        // Nothing of this group moves up into the previous one: its activation piece is the newest load in flight
        // there, and staging it early would wait for every load, the prefetch included.
        __builtin_amdgcn_sched_barrier(0);
        if (prefetch) fetch_group(next, gi + 1);
        if constexpr (MR == 1) {
            if constexpr (NORM) *reinterpret_cast<uint4*>(stage + parity * kStageBytes + st_write) = normalized(cur.a[0], cur.gm[0], cur.gm[1]);
            else *reinterpret_cast<uint4*>(stage + parity * kStageBytes + st_write) = cur.a[0];
            lds_order();
        }
#pragma unroll
        for (int u = 0; u < U; ++u) compute_tile(cur, u, parity, 0.f);
    };

    if constexpr (SETS == 2) {
        Grp gb;
        int gi = g_begin;
        for (; gi + 1 < g_end; gi += 2) {                      // whole pairs, no branch inside: every wait counts loads exactly
            run_group(ga, gb, gi, 0, true);
            run_group(gb, ga, gi + 1, 1, true);                // past the end this prefetch fetches nothing
        }
        if (gi < g_end) run_group(ga, gb, gi, 0, false);       // an odd group out

    } else {
        auto multiply = [&]() {
            float asum = 0.f;
            if constexpr (MR == 1) {
                uint4 piece = ga.a[0];
                if constexpr (NORM) piece = normalized(ga.a[0], ga.gm[0], ga.gm[1]);
                *reinterpret_cast<uint4*>(stage + st_write) = piece;
                lds_order();
                if constexpr (SUMS) asum = block_sum<BS>(sum_piece<BF16>(piece));
            }
#pragma unroll
            for (int u = 0; u < U; ++u) compute_tile(ga, u, 0, asum);
        };
        int gi = g_begin;
        if constexpr (kEarly) {                                // the first group is already on its way
            if (gi < g_end) multiply();
            ++gi;
        }
        for (; gi < g_end; ++gi) {
            fetch_group(ga, gi);
            multiply();
        }
    }

    // ---- split-K reduction across the waves of this workgroup, in wave order ----
    __syncthreads();
    float* red = reinterpret_cast<float*>(smem);       // [waves][4][64]
#pragma unroll
    for (int r = 0; r < kRowsKept; ++r) red[(wave * 4 + r) * 64 + lane] = y[r];
    __syncthreads();
    for (int idx = threadIdx.x; idx < kRowsKept * 64; idx += blockDim.x) {
        const int r = idx >> 6;
        const int l = idx & 63;
        const int row = 4 * (l >> 4) + r;
        const int64_t col = n_base + (l & 15);
        if (row < p.m && col < p.n) {
            float total = 0.f;
            for (int w = 0; w < waves; ++w) total += red[(w * 4 + r) * 64 + l];
            if constexpr (PAIR) {
                float total_up = 0.f;
                for (int w = waves; w < 2 * waves; ++w) total_up += red[(w * 4 + r) * 64 + l];
                const uint16_t gate16 = BF16 ? f32_to_bf16_bits(total) : f32_to_f16_bits(total);
                const uint16_t up16 = BF16 ? f32_to_bf16_bits(total_up) : f32_to_f16_bits(total_up);
                static_cast<uint16_t*>(p.y)[static_cast<int64_t>(row) * p.n + col] = swiglu16<BF16>(gate16, up16, p.decomposed_silu != 0);
            } else {
                total = with_bias(total, p.bias, p.bias_dtype, row, p.n, col, p.y_dtype);
                store_from_f32(p.y, p.y_dtype, static_cast<int64_t>(row) * p.n + col, total);
            }
        }
    }
}

// `waves` = waves per projection; a paired launch has twice as many in a workgroup.
template <bool BF16, int BS, int MR, typename ST, int SETS>
static int launch_packed_cfg(const PackedParams& p, int waves, hipStream_t stream)
{
    const unsigned grid = static_cast<unsigned>((p.n + 15) / 16);
    const bool pair = p.packed_up != nullptr;
    const int all = pair ? 2 * waves : waves;
    const size_t stage = static_cast<size_t>(all) * 2 * (MR == 1 ? 1024 : MR * kRowPitchP);
    const size_t red = static_cast<size_t>(all) * 1024;
    const size_t lds = (stage > red ? stage : red) + (p.gamma ? 16 : 0);      // + the rows' 1 / rms of a launch with the normalization prologue
    if constexpr (MR == 1 || (MR == 4 && SETS == 1)) {       // (four rows with a second register set and the weights of the prologue would spill)
        if (p.gamma) {
            if (pair) hipLaunchKernelGGL((decode_packed_kernel<BF16, BS, MR, ST, SETS, true, true>), dim3(grid), dim3(all * 64), lds, stream, p);
            else hipLaunchKernelGGL((decode_packed_kernel<BF16, BS, MR, ST, SETS, false, true>), dim3(grid), dim3(all * 64), lds, stream, p);
            return static_cast<int>(hipGetLastError());
        }
    }
    if constexpr (MR >= 8) {
        // sixteen staged rows of sixteen waves outgrow the 64 KiB a kernel gets without asking
        if (lds > 65536) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(decode_packed_kernel<BF16, BS, MR, ST, SETS, false>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
            if (e != hipSuccess) return static_cast<int>(e);
        }
        hipLaunchKernelGGL((decode_packed_kernel<BF16, BS, MR, ST, SETS, false>), dim3(grid), dim3(all * 64), lds, stream, p);
    } else {
        if (pair) hipLaunchKernelGGL((decode_packed_kernel<BF16, BS, MR, ST, SETS, true>), dim3(grid), dim3(all * 64), lds, stream, p);
        else hipLaunchKernelGGL((decode_packed_kernel<BF16, BS, MR, ST, SETS, false>), dim3(grid), dim3(all * 64), lds, stream, p);
    }
    return static_cast<int>(hipGetLastError());
}

template <bool BF16, int BS, typename ST>
static int launch_packed_mr(const PackedParams& p, int waves, bool single_set, hipStream_t stream)
{
    if (p.m <= 1) return single_set ? launch_packed_cfg<BF16, BS, 1, ST, 1>(p, waves, stream) : launch_packed_cfg<BF16, BS, 1, ST, 2>(p, waves, stream);
    if (p.m <= 4) return (single_set || p.gamma) ? launch_packed_cfg<BF16, BS, 4, ST, 1>(p, waves, stream) : launch_packed_cfg<BF16, BS, 4, ST, 2>(p, waves, stream);
    // 5 .. 16 rows: one register set (64 registers of activations per group at 16 rows; a second set in flight measured
    // slower). Up to 8 rows a build that stages eight: half the activation bytes per wave and group.
    if (p.m <= 8) return launch_packed_cfg<BF16, BS, 8, ST, 1>(p, waves, stream);
    return launch_packed_cfg<BF16, BS, 16, ST, 1>(p, waves, stream);
}

template <bool BF16, typename ST>
static int launch_packed_bs(const PackedParams& p, int bs, int waves, bool single_set, hipStream_t stream)
{
    switch (bs) {
        case 32: return launch_packed_mr<BF16, 32, ST>(p, waves, single_set, stream);
        case 64: return launch_packed_mr<BF16, 64, ST>(p, waves, single_set, stream);
        default: return launch_packed_mr<BF16, 128, ST>(p, waves, single_set, stream);
    }
}

// ---------------------------------------------------------------------------------------------
// The same stream for 5 <= M <= 64 and many columns: activations shared through LDS.
// ---------------------------------------------------------------------------------------------
//
// With several rows the activations outweigh a column group's weights (16 rows x 128 k x 2 bytes against 16 columns
// x 64 bytes per tile), and a kernel in which every wave fetches its own copy is bound by L2, not HBM. Here a
// workgroup of eight waves owns eight column groups - one wave each, streaming the whole of K - and all eight read
// the activations from one LDS copy, filled window by window (double buffered: the next window travels global ->
// registers while the current one is multiplied, and moves registers -> LDS just before the barrier that ends the
// window). No split-K, so no reduction: a wave stores its 16 columns itself. Weights are not prefetched: the kernel is
// small enough for several workgroups per CU, and the other resident waves cover a wave's memory latency better than
// a second register set does. Up to 64 rows ride on one pass over the weights: RB blocks of 16 rows, each with its own
// accumulators, share every unpacked weight operand - up to that height the call still costs what streaming the
// weights costs, which the tiled kernel cannot offer below a few hundred rows.

constexpr int kWideWaves = 8;        // waves that fill the activation windows; a workgroup has 8 .. kWideWavesMax waves
constexpr int kWideWavesMax = 12;    // (a launch picks the count that spreads its column groups evenly over the CUs)

// RB: blocks of 16 rows (1, 2 or 4). A window is WT tiles of 128 k: a whole tile group for RB <= 2, half of one for
// RB = 4, so that two buffers of RB * 16 rows stay within 66 KB.
// SUMS: offset and zero point leave through the block activation sums (one FMA per accumulator and block) instead of a
// second MFMA per 32 elements. Fewer matrix-core cycles, but 95 registers instead of 80 at 16 rows: launches with
// several workgroups per CU run better with the sixth wave per SIMD (3584 -> 152064 at 16 rows: 59 against 64 us), the
// others with the sums (3584 -> 37888: 22.9 against 24.5 us).
// PF (with DEEP only): the next group's weights travel while the current one is multiplied (a second register set):
// for grids with fewer workgroups than CUs, where no other workgroup covers a wave's memory latency.
// DEEP: the activation windows travel two ahead instead of one (a second set of window registers; RB <= 2).
// PAIR (RB = 1): the fused gate/up node at 5 .. 16 rows. Waves 0 .. 3 own four column groups of the gate projection,
// waves 4 .. 7 the same four of the up projection - each wave exactly as in a launch of its projection alone (the whole
// of K, the same order of summation) - and the epilogue writes round16(silu(round16(gate)) * round16(up)).
// WMAX: the most waves a workgroup of this build may have (8, or 12 for the builds that balanced grids launch).
template <bool BF16, int BS, typename ST, int RB, bool SUMS, bool PF, bool DEEP, bool PAIR = false, int WMAX = kWideWaves>
__global__ __launch_bounds__(WMAX * 64)
__attribute__((amdgpu_waves_per_eu((BS == 128 && sizeof(ST) == 2 && RB == 1) ? (PF ? (SUMS ? 3 : 4) : SUMS ? (DEEP || WMAX > kWideWaves ? 4 : 5) : (DEEP ? 5 : 6)) : (WMAX > kWideWaves ? 3 : 1))))
void decode_wide_kernel(PackedParams p)
{
    static_assert(WMAX == kWideWaves || (WMAX == kWideWavesMax && RB == 1), "twelve waves: the one-block builds only");
    static_assert(DEEP || !PF, "weights ahead only together with deep windows");
    static_assert(!PAIR || RB == 1, "the paired form takes up to 16 rows");
    // column groups per workgroup (and projection): one per wave. The first eight waves also fill the windows.
    // (a build for eight waves knows both at compile time)
    const int tile_waves = WMAX == kWideWaves ? (PAIR ? kWideWaves / 2 : kWideWaves) : (PAIR ? static_cast<int>(blockDim.x >> 7) : static_cast<int>(blockDim.x >> 6));
    constexpr int U = kGroupTiles;
    constexpr int NBT = 128 / BS;
    constexpr int NB = U * NBT;
    constexpr int R = packed_record_bytes(BS, static_cast<int>(sizeof(ST)));
    constexpr int NR = R / 16;
    constexpr int WT = RB == 4 ? 2 : 4;                 // tiles per window
    constexpr int kWindowsPerGroup = U / WT;
    constexpr int kPitch = WT * 256 + 16;               // bytes per LDS row: consecutive rows start in different bank quads
    constexpr int kRows = RB * 16;
    constexpr int kBufBytes = kRows * kPitch;
    constexpr int kPieces = WT * 16;                    // 16-byte pieces per row of a window
    constexpr int NW = kRows * kPieces / 512;           // pieces per thread per window (2 or 4)
    constexpr float kMagicF = BF16 ? 128.0f : 1024.0f;
    constexpr uint32_t kMagicNeg = BF16 ? 0xC300C300u : 0xE400E400u;
    constexpr int kBlockLanes = BS / 8;                 // consecutive threads whose pieces make up one block of a row
    constexpr int kWinBlocks = WT * NBT;                // blocks per window
    constexpr int kSumBytes = kWinBlocks * kRows * 4;
    // [2][kRows][kPitch] activations, then [2][kWinBlocks][kRows] f32 sums of each row over each block of the window:
    // the magic offset and the zero point leave the accumulators through them, y += scale * (acc - (magic + zp) * sum a)
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    float* lds_sums = reinterpret_cast<float*>(smem + 2 * kBufBytes);

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int c = lane & 15;
    const int g = lane >> 4;
    const int64_t col_groups = (p.n + 15) / 16;
    const bool filler = WMAX == kWideWaves || wave < kWideWaves;      // (wave-uniform)
    const bool second = PAIR && wave >= tile_waves;       // (wave-uniform) the up projection's half
    const int64_t cgi = static_cast<int64_t>(blockIdx.x) * tile_waves + (second ? wave - tile_waves : wave);
    const bool active = cgi < col_groups;                 // a wave beyond the last column group still helps with the windows
    const int64_t n_base = cgi * 16;

    const __amdgpu_buffer_rsrc_t srd_p = make_srd((second ? p.packed_up : p.packed) + (active ? cgi : 0) * p.cg_stride, active ? static_cast<uint64_t>(p.cg_stride) : 0);
    const __amdgpu_buffer_rsrc_t srd_a = make_srd(p.a, static_cast<uint64_t>(p.m * p.k) * 2);

    const uint32_t w_off = static_cast<uint32_t>(lane * 16);
    const uint32_t r_off = static_cast<uint32_t>(kChunkWeights + c * R);
    // operand of MFMA j of tile x of the window, row block rb: row rb*16 + c, elements x*128 + j*32 + g*8 .. +8
    const uint32_t frag_off = static_cast<uint32_t>(c * kPitch + g * 16);
    const uint32_t mask = __builtin_amdgcn_mov_dpp(p.nibble_mask, 0xE4, 0xf, 0xf, false), magic = p.magic;

    float4p_t y[RB], acc[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        y[rb] = float4p_t{0.f, 0.f, 0.f, 0.f};
        acc[rb] = float4p_t{0.f, 0.f, 0.f, 0.f};
    }

    struct Grp {
        uint4 w[kGroupTiles];
        uint4 r[NR];
    };
    // a group past the last lies beyond the column group's range: the loads return zeros and touch no memory
    auto fetch_group = [&](Grp& grp, int gi) {
        const uint32_t soff = static_cast<uint32_t>(gi) * static_cast<uint32_t>(p.chunk_bytes);
#pragma unroll
        for (int u = 0; u < U; ++u) grp.w[u] = load16(srd_p, w_off + static_cast<uint32_t>(u * 1024), soff);
#pragma unroll
        for (int i = 0; i < NR; ++i) grp.r[i] = load16(srd_p, r_off + static_cast<uint32_t>(i * 16), soff);
    };
    // window fill: piece q = t + 512 i of the window's kRows * kPieces pieces -> (row q / kPieces, piece q % kPieces)
    uint4 wa[NW];
    uint4 wb[DEEP ? NW : 1];                               // DEEP: the second set of window registers
    auto load_window_into = [&](uint4* dst, int win) {
#pragma unroll
        for (int i = 0; i < NW; ++i) {
            const int q = t + 512 * i;
            const int row = q / kPieces, piece = q % kPieces;
            const int64_t k0 = static_cast<int64_t>(win) * (WT * 128) + piece * 8;
            uint32_t off = static_cast<uint32_t>(row) * static_cast<uint32_t>(p.k) * 2u + static_cast<uint32_t>(piece * 16);
            if (row >= p.m || k0 >= p.k || !filler) off = kOutOfRange;       // K is a multiple of 8: a piece is all inside or all outside
            dst[i] = load16(srd_a, off, static_cast<uint32_t>(win) * (WT * 256u));
        }
    };
    auto load_window = [&](int win) { load_window_into(wa, win); };
    auto store_window_from = [&](const uint4* src, int buf) {
        if (!filler) return;
#pragma unroll
        for (int i = 0; i < NW; ++i) {
            const int q = t + 512 * i;
            const int row = q / kPieces, piece = q % kPieces;
            *reinterpret_cast<uint4*>(smem + buf * kBufBytes + row * kPitch + piece * 16) = src[i];
            if constexpr (SUMS) {
                const float sum = block_sum<BS>(sum_piece<BF16>(src[i]));     // a block's pieces sit in consecutive lanes
                if (piece % kBlockLanes == 0) lds_sums[(buf * kWinBlocks + piece / kBlockLanes) * kRows + row] = sum;
            }
        }
    };
    auto store_window = [&](int buf) { store_window_from(wa, buf); };
    // tiles [first, first + WT) of the group against window buffer `buf`
    auto compute_window = [&](const Grp& grp, int buf, int first) {
        uint32_t rr[NR * 4];
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            rr[4 * i] = grp.r[i].x;
            rr[4 * i + 1] = grp.r[i].y;
            rr[4 * i + 2] = grp.r[i].z;
            rr[4 * i + 3] = grp.r[i].w;
        }
#pragma unroll
        for (int x = 0; x < WT; ++x) {
            const int u = first + x;                               // tile of the group (compile-time after unrolling)
            const unsigned char* fa = smem + buf * kBufBytes + frag_off + x * 256;
            const uint32_t wd[4] = {grp.w[u].x, grp.w[u].y, grp.w[u].z, grp.w[u].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int bi = u * NBT + (j * 32) / BS;
                const int zbyte = NB * static_cast<int>(sizeof(ST)) + bi;
                const uint32_t w = wd[j];
                uint4 op;
                op.x = (w & mask) | magic;
                op.y = ((w >> 4) & mask) | magic;
                op.z = ((w >> 8) & mask) | magic;
                op.w = ((w >> 12) & mask) | magic;
                const bool last = ((j + 1) * 32) % BS == 0 || j == 3;
                float sf = 0.f, off = 0.f;
                if (last) {
                    if constexpr (sizeof(ST) == 4) {
                        sf = __uint_as_float(rr[bi]);
                    } else {
                        const uint32_t raw = (rr[bi / 2] >> ((bi % 2) * 16)) & 0xffffu;
                        sf = BF16 ? __uint_as_float(raw << 16) : f16_bits_to_f32(static_cast<uint16_t>(raw));
                    }
                    if constexpr (SUMS) off = kMagicF + static_cast<float>((rr[zbyte / 4] >> ((zbyte % 4) * 8)) & 0xffu);
                }
                const uint32_t zpair = kMagicNeg | (((rr[zbyte / 4] >> ((zbyte % 4) * 8)) & 0xffu) * 0x00010001u);
                const uint4 zc = make_uint4(zpair, zpair, zpair, zpair);       // used without SUMS only
                const int wb = x * NBT + (j * 32) / BS;                // block of the window
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) {
                    const uint4 av = *reinterpret_cast<const uint4*>(fa + rb * 16 * kPitch + j * 64);
                    acc[rb] = mfma16p<BF16>(av, op, acc[rb]);
                    if constexpr (!SUMS) acc[rb] = mfma16p<BF16>(av, zc, acc[rb]);
                    if (last) {
                        float sav[4] = {0.f, 0.f, 0.f, 0.f};
                        if constexpr (SUMS) {
                            // this lane's accumulator rows are rows rb * 16 + 4 g + r of the window
                            const float4 sa = *reinterpret_cast<const float4*>(lds_sums + (buf * kWinBlocks + wb) * kRows + rb * 16 + 4 * g);
                            sav[0] = sa.x;
                            sav[1] = sa.y;
                            sav[2] = sa.z;
                            sav[3] = sa.w;
                        }
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            y[rb][r] = fmaf(sf, SUMS ? fmaf(-off, sav[r], acc[rb][r]) : acc[rb][r], y[rb][r]);
                            acc[rb][r] = 0.f;
                        }
                    }
                }
            }
        }
    };

    const int windows = p.groups * kWindowsPerGroup;
    Grp ga;
    if constexpr (DEEP) {
        // One window per group (RB <= 2). The next window's activations sit in one register set, the one after that is
        // in flight into the other: a pass no longer lasts at least one L2 round trip. No branch inside a pass (a branch
        // makes the compiler wait for every load in flight): a window or group past the end loads zeros, passes run in
        // pairs so that the register sets alternate at compile time, an odd one is peeled.
        static_assert(!DEEP || kWindowsPerGroup == 1, "deep windows: one window per group");
        Grp gb;
        load_window_into(wa, 0);
        load_window_into(wb, 1);
        if constexpr (PF) fetch_group(ga, 0);
        store_window_from(wa, 0);
        __syncthreads();
        // `ready` holds window gi + 1, `idle` receives window gi + 2
        auto pass = [&](Grp& cur, Grp& next, int gi, const uint4* ready, uint4* idle, bool prefetch) {
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (!PF) fetch_group(cur, gi);           // needed at once: issued first, so that the wait leaves the window in flight
            load_window_into(idle, gi + 2);
            if constexpr (PF) {
                if (prefetch) fetch_group(next, gi + 1);
            }
            __builtin_amdgcn_sched_barrier(0);
            compute_window(cur, gi & 1, 0);
            store_window_from(ready, (gi & 1) ^ 1);
            __syncthreads();
        };
        int gi = 0;
        for (; gi + 1 < p.groups; gi += 2) {
            pass(ga, gb, gi, wb, wa, true);
            pass(PF ? gb : ga, ga, gi + 1, wa, wb, true);
        }
        if (gi < p.groups) pass(ga, gb, gi, wb, wa, false);
    } else {
        load_window(0);
        store_window(0);
        __syncthreads();
        for (int gi = 0; gi < p.groups; ++gi) {
            fetch_group(ga, gi);
#pragma unroll
            for (int h = 0; h < kWindowsPerGroup; ++h) {
                const int win = gi * kWindowsPerGroup + h;
                const int buf = win & 1;
                if (win + 1 < windows) load_window(win + 1);
                compute_window(ga, buf, h * WT);
                if (win + 1 < windows) store_window(buf ^ 1);
                __syncthreads();
            }
        }
    }

    if constexpr (PAIR) {
        // every window has been read (the loop ends on a barrier): the up half leaves its totals where the windows were
        float* up_totals = reinterpret_cast<float*>(smem);            // [tile_waves][4][64]
        if (second) {
#pragma unroll
            for (int r = 0; r < 4; ++r) up_totals[((wave - tile_waves) * 4 + r) * 64 + lane] = y[0][r];
        }
        __syncthreads();
        const int64_t col = n_base + c;
        if (!second && active && col < p.n) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = 4 * g + r;
                if (row < p.m) {
                    const float up = up_totals[(wave * 4 + r) * 64 + lane];
                    const uint16_t gate16 = BF16 ? f32_to_bf16_bits(y[0][r]) : f32_to_f16_bits(y[0][r]);
                    const uint16_t up16 = BF16 ? f32_to_bf16_bits(up) : f32_to_f16_bits(up);
                    static_cast<uint16_t*>(p.y)[static_cast<int64_t>(row) * p.n + col] = swiglu16<BF16>(gate16, up16, p.decomposed_silu != 0);
                }
            }
        }
    } else
    if (active) {
        const int64_t col = n_base + c;
        if (col < p.n) {
            const bool per_row = (p.bias_dtype & ROCM_BIAS_PER_ROW) != 0;
            const BiasTerm bias = load_bias(p.bias, p.bias_dtype, 0, p.n, col);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int row = rb * 16 + 4 * g + r;
                    if (row < p.m) store_from_f32(p.y, p.y_dtype, static_cast<int64_t>(row) * p.n + col, add_bias(y[rb][r], per_row ? load_bias(p.bias, p.bias_dtype, row, p.n, col) : bias, p.y_dtype));
                }
            }
        }
    }
}

// What launch_wide_bs launches for a shape: the build (row blocks, sums or second MFMA, weights / windows ahead, the
// workgroup's most waves), the waves per workgroup and the grid. No GPU work: a CPU test holds the answers for the model
// shapes against a committed table, so that a change made for one shape cannot move another unnoticed.
struct WidePlan {
    int rb;            // blocks of 16 rows per wave: 1, 2 or 4
    bool sums, pf, deep;
    int wmax;          // kWideWaves or kWideWavesMax
    int waves;         // per workgroup
    unsigned grid;
    bool ok;           // false: no build for this call (the dispatch does not send it here)
};

static WidePlan plan_wide(int64_t m, int64_t n, int bs, bool st16, bool pair, int64_t cus)
{
    WidePlan w{};
    const int64_t col_groups = (n + 15) / 16;
    const int64_t all_groups = pair ? 2 * col_groups : col_groups;
    // A grid between one and one and a half workgroups of eight waves per CU (3584 -> 37888: 296 workgroups on 256 CUs)
    // leaves some CUs with two workgroups while the others run one, and the launch lasts as long as the doubly loaded ones.
    const bool in_between = all_groups > cus * kWideWaves && all_groups <= cus * kWideWavesMax;
    const int64_t alone = (col_groups + kWideWaves - 1) / kWideWaves;
    // How offset and zero point leave the accumulator (it shows in the last bits, so it is decided as for a launch of one
    // projection alone, and a pair follows its projections). Through the block activation sums, except:
    //  * grids of three or more workgroups per CU (3584 -> 152064 at 16 rows: 59 against 64 us);
    //  * block size 32: the sums build takes 185-196 registers there, one workgroup per CU, and a grid above one workgroup
    //    per CU runs in two rounds (3584 -> 37888 at 8 rows: 37.8 us; the second-MFMA build with the next group's
    //    weights in flight 26.2, 4096 -> 14336 21.6 -> 17.2, 4096 -> 28672 24.0 -> 20.2);
    //  * block size 64 where a launch of the projection gets a balanced grid (below): the sums build with weights ahead
    //    takes 218 registers, too many for more than eight waves a workgroup.
    w.sums = alone < 3 * cus && bs != 32 && !(bs == 64 && st16 && col_groups > cus * kWideWaves && col_groups <= cus * kWideWavesMax);
    // Waves (= column groups) per workgroup: eight, unless the grid is in between and a build for more waves exists - then
    // as many as spread the column groups over one workgroup per CU, up to twelve (3584 -> 37888 at block 128: ten waves,
    // 237 workgroups, 22.6 -> 18.0 us at 8 rows; at block 64 23.7 -> 21.2). Larger workgroups lose where the grid is several
    // times the CUs (3584 -> 152064 65 -> 80 us with ten). A paired launch holds half of its waves' column groups from each
    // projection. The builds for twelve waves: block 128 with the sums, block 64 without (16-bit scales).
    int ww = kWideWaves;
    if (m <= 16 && st16 && in_between && ((bs == 128 && w.sums) || (bs == 64 && !w.sums && !pair))) {
        ww = static_cast<int>((all_groups + cus - 1) / cus);
        if (pair && (ww & 1)) ++ww;
        if (ww > kWideWavesMax) ww = kWideWaves;
    }
    const int per_wg = pair ? ww / 2 : ww;
    w.waves = ww;
    w.grid = static_cast<unsigned>((col_groups + per_wg - 1) / per_wg);
    w.wmax = ww > kWideWaves ? kWideWavesMax : kWideWaves;
    w.rb = m <= 16 ? 1 : m <= 32 ? 2 : 4;
    w.ok = true;
    if (m <= 16) {
        // The build by grid size. Measured at 8 / 16 rows (3584 -> 152064, 3584 -> 37888, 4096 -> 16384): three or more
        // workgroups per CU run best with the windows two ahead (68 -> 64 us); fewer workgroups than CUs with weights and
        // windows both ahead (17.2 -> 14.5 us); in between neither helps the sums build (20.6 us either way; with both ahead
        // it spills at block size 32).
        if (ww > kWideWaves) {
            // a balanced grid has at most one workgroup per CU: the builds for few workgroups, compiled for twelve waves
            if (bs == 128 && st16) {
                w.pf = w.deep = w.grid < cus;
            } else if (bs == 64 && st16 && !pair) {
                w.pf = w.deep = true;              // (sums is false here)
            } else {
                w.ok = false;
            }
        } else if (!w.sums) {
            w.deep = true;
            w.pf = !(alone >= 3 * cus && bs != 32);
        } else if (bs != 32) {
            w.pf = w.deep = w.grid < cus;
        } else {
            w.ok = false;                          // (block size 32 never takes the sums)
        }
    } else {
        // More row blocks per wave only where they fit the register file: two from block size 64, four at 128. The
        // spilling forms ran several times slower than the routes that take those calls instead (3584 -> 37888: 153 us
        // at block 32 and 32 rows against 2 x 37 us in blocks of 16 rows; 258 us at block 64 and 64 rows against 83 us
        // in the tiled kernel). The paired form takes up to 16 rows.
        w.sums = true;
        w.pf = w.deep = false;
        if (pair || bs == 32 || (m > 32 && bs == 64)) w.ok = false;
    }
    return w;
}

template <bool BF16, typename ST>
static int launch_wide_bs(const PackedParams& p, int bs, int64_t cus, hipStream_t stream)
{
    const bool pair = p.packed_up != nullptr;
    const WidePlan w = plan_wide(p.m, p.n, bs, sizeof(ST) == 2, pair, cus);
    if (!w.ok) return -1;
    const dim3 grid(w.grid);
    auto go = [&](auto kernel, size_t lds) {
        if (lds > 65536) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
            if (e != hipSuccess) return static_cast<int>(e);
        }
        hipLaunchKernelGGL(kernel, grid, dim3(w.waves * 64), lds, stream, p);
        return static_cast<int>(hipGetLastError());
    };
    auto by_rows = [&](auto bs_tag) {
        constexpr int BS = decltype(bs_tag)::value;
        // two window buffers of rows x (tiles x 256 + 16) bytes, then two tables of (blocks per window) x rows f32 sums
        constexpr int NBT = 128 / BS;
        constexpr size_t lds16 = 2 * 16 * (4 * 256 + 16), sums16 = 2 * 4 * NBT * 16 * 4;
        auto upto16 = [&](auto pair_tag) {
            constexpr bool P = decltype(pair_tag)::value;
            if (w.wmax > kWideWaves) {
                if constexpr (BS == 128 && sizeof(ST) == 2) {
                    if (w.pf) return go(decode_wide_kernel<BF16, BS, ST, 1, true, true, true, P, kWideWavesMax>, lds16 + sums16);
                    return go(decode_wide_kernel<BF16, BS, ST, 1, true, false, false, P, kWideWavesMax>, lds16 + sums16);
                } else if constexpr (BS == 64 && sizeof(ST) == 2 && !P) {
                    return go(decode_wide_kernel<BF16, BS, ST, 1, false, true, true, false, kWideWavesMax>, lds16);
                } else {
                    return -1;
                }
            }
            if (!w.sums) {
                if (!w.pf) return go(decode_wide_kernel<BF16, BS, ST, 1, false, false, true, P>, lds16);
                return go(decode_wide_kernel<BF16, BS, ST, 1, false, true, true, P>, lds16);
            }
            if constexpr (BS != 32) {
                if (w.pf) return go(decode_wide_kernel<BF16, BS, ST, 1, true, true, true, P>, lds16 + sums16);
                return go(decode_wide_kernel<BF16, BS, ST, 1, true, false, false, P>, lds16 + sums16);
            } else {
                return -1;
            }
        };
        if (p.m <= 16) return pair ? upto16(std::true_type{}) : upto16(std::false_type{});
        if constexpr (BS == 32) return -1;
        else {
            if (p.m <= 32) return go(decode_wide_kernel<BF16, BS, ST, 2, true, false, false>, 2 * 32 * (4 * 256 + 16) + 2 * 4 * NBT * 32 * 4);
            if constexpr (BS == 64) return -1;
            else return go(decode_wide_kernel<BF16, BS, ST, 4, true, false, false>, 2 * 64 * (2 * 256 + 16) + 2 * 2 * NBT * 64 * 4);
        }
    };
    switch (bs) {
        case 32: return by_rows(std::integral_constant<int, 32>{});
        case 64: return by_rows(std::integral_constant<int, 64>{});
        default: return by_rows(std::integral_constant<int, 128>{});
    }
}

// ---------------------------------------------------------------------------------------------
// accuracy_level = 4, up to 16 rows, over the same repacked stream: v_mfma_i32_16x16x32_i8.
// ---------------------------------------------------------------------------------------------
//
// `w & 0x0f0f0f0f` and `(w >> 4) & 0x0f0f0f0f` turn a repacked dword into the eight weights as unsigned bytes in the
// order e0,e4,e1,e5 | e2,e6,e3,e7; the activation codes are stored in that same order inside every run of 8, so an
// operand costs three instructions and no byte shuffles. Arithmetic as in the unpacked int8 kernel: exact integer
// block sums, zero point through the code sums, one f32 scale-and-add per block.

typedef __attribute__((ext_vector_type(4))) int int4p_t;

struct Acc4PackedParams {
    const int8_t* qa;       // [m, padded_k] codes, packed order
    const float* aq;        // one row: [kb, 2] = scale_a, f32(sum of codes)
    const float* aux16;     // 2 .. 16 rows: [kb, 16, 2], the same pairs block-major
    int64_t m;
    const void* a;          // FUSE: the one row itself, f16 or bf16 [k]; every wave quantizes the groups it multiplies
    int64_t k;
    int rounding;           // FUSE: 0 = ties to even, 1 = ties away from zero
    const uint8_t* packed;
    const void* bias;
    void* y;
    int64_t n, kb;
    int64_t padded_k;
    int64_t cg_stride;
    int groups, groups_per_wave, chunk_bytes;
    int bias_dtype, y_dtype;
    int scales_bf16;
    int32_t* acc_probe;     // PROBE builds: int32 [M, N, kb] block accumulators, as flushed
};

constexpr int kCodePitchP = 144;   // bytes between the rows of one tile of codes in LDS: 128 + 16

template <int NR, int NA, int NX>
struct Acc4PackedGroup {
    uint4 w[kGroupTiles];
    uint4 r[NR];
    uint4 a[NA];  // one row: 16 codes of the group (lanes 0..31). 16 rows: per tile, row lane / 8 (+ 8), piece lane % 8
    uint4 x[NX];  // one row: .x/.y = (scale_a, code sum) of block `lane` of the group. 16 rows: 16 bytes of the group's aux16 rows
};

// FUSE: 0 = codes and (scale, sum) pairs come from the workspace a quantizer kernel filled; 1 / 2 = the row arrives as
// f16 / bf16 and each wave quantizes the 512 activations of a group itself, with the arithmetic of quantize_a_kernel
// (one correctly rounded divide each for scale and inverse, one multiply and one rounding per element) - a lane holds
// 8 consecutive activations, a block is BS / 8 consecutive lanes. That is redundant across workgroups but saves the
// separate launch, which at one row costs about as much as a fifth of this kernel.
// PROBE: every flushed block accumulator (the integer acc - zp * code_sum that is about to be scaled) is also stored to
// p.acc_probe; the same code otherwise, for tests that compare the integers themselves.
// MR: rows staged, 1, 4, 8 or 16 (M <= MR). Beyond one row the codes come from the workspace (FUSE = 0): per tile a wave
// loads the rows' 128 codes, stages them in LDS at a padded pitch and reads MFMA operand j of row lane % 16 from there;
// the activation-side (scale, sum) pairs of the group's blocks are staged once per group and read when a block ends.
// With 4 (8), call row r sits in matrix row 4 r (2 r) and the rows between stay zero, so that a lane finds its rows in
// component 0 (0 and 2) of its accumulator and a block's end scales one (two) values per lane instead of four.
// ST: float, uint16_t, or Bf16Scale for the several-row builds when the 16-bit scales are bf16 - there the scale type is
// known at compile time (a run-time choice between the two conversions made the compiler prepare both for all of a
// group's blocks up front: 220 registers instead of 94 at block size 32 and 16 rows, two waves per SIMD instead of five).
struct Bf16Scale {
    uint16_t bits;
};

template <int BS, typename ST, int SETS, int FUSE, bool PROBE, int MR = 1>
__global__ __launch_bounds__(512) void acc4_packed_kernel(Acc4PackedParams p)
{
    static_assert(MR == 1 || ((MR == 4 || MR == 8 || MR == 16) && (FUSE == 0 || MR == 4) && SETS == 1),
                  "several rows: one register set; codes from the workspace, or up to four rows quantized here");
    constexpr int U = kGroupTiles;
    constexpr int NBT = 128 / BS;
    constexpr int NB = U * NBT;
    constexpr int R = packed_record_bytes(BS, static_cast<int>(sizeof(ST)));
    constexpr int NR = R / 16;
    constexpr int NA = MR == 16 ? 2 * U : MR == 1 ? 1 : U;
    constexpr int SP = MR == 1 ? 1 : 16 / MR;                                     // matrix rows per call row
    constexpr int NX = MR == 1 ? 1 : (NB * 8 + 63) / 64;
    constexpr int kCodeStage = 16 * kCodePitchP;                                  // 16 rows: one tile of codes
    constexpr int kWaveBytes = MR == 1 ? SETS * 512 : 2 * kCodeStage + NB * 128;  // 16 rows: two tiles in turn + the group's pairs
    constexpr int kRowsKept = MR == 1 ? 1 : MR / 4;                               // call rows per lane: g * kRowsKept + r
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = blockDim.x >> 6;
    const int c = lane & 15;
    const int g = lane >> 4;
    const int64_t n_base = static_cast<int64_t>(blockIdx.x) * 16;
    const bool bf16_scales = std::is_same<ST, Bf16Scale>::value || (MR == 1 && p.scales_bf16 != 0);

    const __amdgpu_buffer_rsrc_t srd_p = make_srd(p.packed + static_cast<int64_t>(blockIdx.x) * p.cg_stride, static_cast<uint64_t>(p.cg_stride));
    const __amdgpu_buffer_rsrc_t srd_a = FUSE ? make_srd(p.a, static_cast<uint64_t>(p.m * p.k) * 2) : make_srd(p.qa, static_cast<uint64_t>(p.m * p.padded_k));
    const __amdgpu_buffer_rsrc_t srd_x = MR == 1 ? make_srd(p.aq, FUSE ? 0 : static_cast<uint64_t>(p.kb) * 8) : make_srd(p.aux16, static_cast<uint64_t>(p.kb) * 128);
    constexpr int kBlockLanes = BS / 8;

    const uint32_t w_off = static_cast<uint32_t>(lane * 16);
    const uint32_t r_off = static_cast<uint32_t>(kChunkWeights + c * R);
    unsigned char* stage = smem + wave * kWaveBytes;
    unsigned char* aux_stage = stage + 2 * kCodeStage;            // 16 rows only
    // operand of MFMA j of tile u: the 8 codes of elements u*128 + j*32 + g*8 .. +8. One row: only row 0 matters, every
    // lane of a lane group reads the same 8 bytes of the group's 512. 16 rows: row lane % 16 of the staged tile.
    const uint32_t st_read = MR == 1 ? static_cast<uint32_t>(g * 8) : static_cast<uint32_t>(c * kCodePitchP + g * 8);
    // several rows: a tile's codes arrive as row lane / 8 (+ 8), piece lane % 8, and go to matrix row SP * row
    const uint32_t a_off16 = static_cast<uint32_t>(lane >> 3) * static_cast<uint32_t>(p.padded_k) + static_cast<uint32_t>((lane & 7) * 16);
    const uint32_t st_write16 = static_cast<uint32_t>((lane >> 3) * SP * kCodePitchP + (lane & 7) * 16);
    if constexpr (MR == 4 || MR == 8) {
        for (int i = lane; i < 2 * kCodeStage / 16; i += 64) *reinterpret_cast<uint4*>(stage + i * 16) = make_uint4(0, 0, 0, 0);
        lds_order();
    }

    float y[kRowsKept];
#pragma unroll
    for (int r = 0; r < kRowsKept; ++r) y[r] = 0.f;
    int4p_t acc = {0, 0, 0, 0};

    const int g_begin = wave * p.groups_per_wave;
    const int g_end = min(g_begin + p.groups_per_wave, p.groups);

    using Grp = Acc4PackedGroup<NR, NA, NX>;
    // No branch in here (a branch would make the compiler wait for every load in flight, the prefetch included): a group
    // past the wave's last one gets every offset out of range, fetches nothing and reads as zeros - it adds nothing.
    auto fetch_group = [&](Grp& grp, int gi) {
        const uint32_t oor = gi < g_end ? 0u : kOutOfRange;        // or-ed in: any offset with these bits is out of range
        const uint32_t soff = static_cast<uint32_t>(gi) * static_cast<uint32_t>(p.chunk_bytes);
#pragma unroll
        for (int u = 0; u < U; ++u) grp.w[u] = load16(srd_p, (w_off + static_cast<uint32_t>(u * 1024)) | oor, soff);
#pragma unroll
        for (int i = 0; i < NR; ++i) grp.r[i] = load16(srd_p, (r_off + static_cast<uint32_t>(i * 16)) | oor, soff);
        if constexpr (MR != 1 && FUSE != 0) {
            // up to four rows quantized here: a[r] = 8 activations of row r (lane * 8 of the group's 512); a row past M lies past
            // the range and reads as zeros, a piece past K would be the next row's and is kept out
            const bool beyond = static_cast<int64_t>(gi) * 512 + lane * 8 >= p.k;
#pragma unroll
            for (int r = 0; r < NA; ++r) {
                const uint32_t off = beyond ? kOutOfRange : static_cast<uint32_t>(r) * static_cast<uint32_t>(p.k) * 2u + static_cast<uint32_t>(lane * 16);
                grp.a[r] = load16(srd_a, off | oor, static_cast<uint32_t>(gi) * 1024u);
            }
        } else if constexpr (MR != 1) {
#pragma unroll
            for (int x = 0; x < NA; ++x) {
                const int u = MR == 16 ? x / 2 : x, i = MR == 16 ? x % 2 : 0;
                // a piece past the end of its row would read the next row's codes (rows past M lie past the range and read as zeros)
                const bool beyond = static_cast<int64_t>(gi * U + u) * 128 + (lane & 7) * 16 >= p.padded_k || (MR == 4 && lane >= 32);
                const uint32_t off = beyond ? kOutOfRange : a_off16 + static_cast<uint32_t>(i * 8) * static_cast<uint32_t>(p.padded_k);
                grp.a[x] = load16(srd_a, off | oor, static_cast<uint32_t>(gi * U + u) * 128u);
            }
#pragma unroll
            for (int x = 0; x < NX; ++x)
                grp.x[x] = load16(srd_x, (lane + 64 * x < NB * 8 ? static_cast<uint32_t>((lane + 64 * x) * 16) : kOutOfRange) | oor, static_cast<uint32_t>(gi * NB) * 128u);
        } else if constexpr (FUSE) {
            grp.a[0] = load16(srd_a, static_cast<uint32_t>(lane * 16) | oor, static_cast<uint32_t>(gi) * 1024u);   // 8 activations; K % 8 == 0 and the range ends the row
        } else {
            grp.a[0] = load16(srd_a, (lane < 32 ? static_cast<uint32_t>(lane * 16) : kOutOfRange) | oor, static_cast<uint32_t>(gi) * 512u);   // the range ends the row at padded_k
            const auto v = __builtin_amdgcn_raw_buffer_load_b64(srd_x, static_cast<int>((lane < NB ? static_cast<uint32_t>(lane * 8) : kOutOfRange) | oor), static_cast<int>(gi * NB * 8), 0);
            grp.x[0].x = v[0];
            grp.x[0].y = v[1];
        }
    };
    auto compute_group = [&](const Grp& grp, int gi, int slot) {
        unsigned char* st = stage + slot * 512;
        float sa_lane = 0.f, qs_lane = 0.f;          // FUSE: scale and f32(code sum) of the block this lane's activations lie in
        uint2 fused_codes[MR != 1 && FUSE != 0 ? MR : 1];
        // FUSE: the quantizer's arithmetic on one 16-byte piece (8 activations); the block's lanes share maximum and code sum.
        // Returns the eight codes in the byte order the repacked weights unpack to, elements 0,4,1,5 | 2,6,3,7.
        auto quantize_piece = [&](const uint4& piece) -> uint2 {
            const uint32_t d[4] = {piece.x, piece.y, piece.z, piece.w};
            float v[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if constexpr (FUSE == 2) {
                    v[2 * i] = __uint_as_float(d[i] << 16);
                    v[2 * i + 1] = __uint_as_float(d[i] & 0xffff0000u);
                } else {
                    const half2p_t h = __builtin_bit_cast(half2p_t, d[i]);
                    v[2 * i] = static_cast<float>(h.x);
                    v[2 * i + 1] = static_cast<float>(h.y);
                }
            }
            float vmax = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) vmax = fmaxf(vmax, fabsf(v[i]));
            vmax = dpp_max<0xB1>(vmax);
            vmax = dpp_max<0x4E>(vmax);
            if constexpr (BS >= 64) vmax = dpp_max<0x141>(vmax);
            if constexpr (BS >= 128) vmax = dpp_max<0x140>(vmax);
            sa_lane = __fdiv_rn(vmax, 127.0f);
            const float inv = vmax != 0.0f ? __fdiv_rn(127.0f, vmax) : 0.0f;
            int q[8], sum = 0;
            auto round_all = [&](auto away) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float scaled = __fmul_rn(v[i], inv);
                    float r = decltype(away)::value ? roundf(scaled) : rintf(scaled);
                    r = fminf(fmaxf(r, -127.0f), 127.0f);
                    q[i] = static_cast<int>(r);
                    sum += q[i];
                }
            };
            if (p.rounding == 1) round_all(std::true_type{});      // wave-uniform: one branch per group, not one select per element
            else round_all(std::false_type{});
            sum = dpp_addi<0xB1>(sum);
            sum = dpp_addi<0x4E>(sum);
            if constexpr (BS >= 64) sum = dpp_addi<0x141>(sum);
            if constexpr (BS >= 128) sum = dpp_addi<0x140>(sum);
            qs_lane = static_cast<float>(sum);                     // |sum| <= 127 * BS: exact
            const uint32_t lo = (q[0] & 0xff) | ((q[4] & 0xff) << 8) | ((q[1] & 0xff) << 16) | (static_cast<uint32_t>(q[5]) << 24);
            const uint32_t hi = (q[2] & 0xff) | ((q[6] & 0xff) << 8) | ((q[3] & 0xff) << 16) | (static_cast<uint32_t>(q[7]) << 24);
            return make_uint2(lo, hi);
        };
        if constexpr (MR != 1 && FUSE != 0) {
            // every row's piece is quantized; the first lane of a block leaves the row's (scale, code sum) where a block's end
            // reads it: pair [block][row] of the group
#pragma unroll
            for (int r = 0; r < MR; ++r) {
                fused_codes[r] = quantize_piece(grp.a[r]);
                if (lane % kBlockLanes == 0) *reinterpret_cast<float2*>(aux_stage + (lane / kBlockLanes) * 128 + r * 8) = make_float2(sa_lane, qs_lane);
            }
        } else if constexpr (MR != 1) {
#pragma unroll
            for (int x = 0; x < NX; ++x)
                if (lane + 64 * x < NB * 8) *reinterpret_cast<uint4*>(aux_stage + (lane + 64 * x) * 16) = grp.x[x];
        } else if constexpr (FUSE) {
            *reinterpret_cast<uint2*>(st + lane * 8) = quantize_piece(grp.a[0]);
        } else {
            if (lane < 32) *reinterpret_cast<uint4*>(st + lane * 16) = grp.a[0];
        }
        lds_order();
        uint32_t rr[NR * 4];
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            rr[4 * i] = grp.r[i].x;
            rr[4 * i + 1] = grp.r[i].y;
            rr[4 * i + 2] = grp.r[i].z;
            rr[4 * i + 3] = grp.r[i].w;
        }
        // every dword of the record counts as used, also its padding: a load destination known to be dead is handed out
        // again at once, and writing it waits for the load in flight
#pragma unroll
        for (int i = 0; i < NR * 4; ++i) asm volatile("" : : "v"(rr[i]));
#pragma unroll
        for (int u = 0; u < U; ++u) {
            long av[4];
            if constexpr (MR != 1) {
                unsigned char* tile = stage + (u & 1) * kCodeStage;
                if constexpr (FUSE != 0) {
                    // the lanes that hold this tile's elements (lane / 16 = u) write each row's eight codes into its matrix row
                    if ((lane >> 4) == u) {
#pragma unroll
                        for (int r = 0; r < MR; ++r) *reinterpret_cast<uint2*>(tile + r * SP * kCodePitchP + (lane & 15) * 8) = fused_codes[r];
                    }
                } else if constexpr (MR != 16) {
                    if (MR == 8 || lane < 32) *reinterpret_cast<uint4*>(tile + st_write16) = grp.a[u];
                } else {
#pragma unroll
                    for (int i = 0; i < 2; ++i) *reinterpret_cast<uint4*>(tile + st_write16 + i * 8 * kCodePitchP) = grp.a[u * 2 + i];
                }
                lds_order();
#pragma unroll
                for (int j = 0; j < 4; ++j) av[j] = *reinterpret_cast<const long*>(tile + st_read + j * 32);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) av[j] = *reinterpret_cast<const long*>(st + st_read + u * 128 + j * 32);
            }
            const uint32_t wd[4] = {grp.w[u].x, grp.w[u].y, grp.w[u].z, grp.w[u].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool first = (j * 32) % BS == 0;
                const bool last = ((j + 1) * 32) % BS == 0 || j == 3;
                const uint64_t bw = static_cast<uint64_t>(wd[j] & 0x0f0f0f0fu) | (static_cast<uint64_t>((wd[j] >> 4) & 0x0f0f0f0fu) << 32);
                const int4p_t zero = {0, 0, 0, 0};
                acc = __builtin_amdgcn_mfma_i32_16x16x32_i8(av[j], static_cast<long>(bw), first ? zero : acc, 0, 0, 0);
                if (last) {
                    const int bi = u * NBT + (j * 32) / BS;
                    // (a block beyond K needs no guard: its repacked scale is 0 and its codes and sums are 0)
                    const int zbyte = NB * static_cast<int>(sizeof(ST)) + bi;
                    const float zf = static_cast<float>((rr[zbyte / 4] >> ((zbyte % 4) * 8)) & 0xffu);
                    float sb;
                    if constexpr (sizeof(ST) == 4) {
                        sb = __uint_as_float(rr[bi]);
                    } else {
                        const uint32_t raw = (rr[bi / 2] >> ((bi % 2) * 16)) & 0xffffu;
                        sb = bf16_scales ? __uint_as_float(raw << 16) : f16_bits_to_f32(static_cast<uint16_t>(raw));
                    }
                    if constexpr (MR != 1) {
                        // this lane's call rows g * kRowsKept + r sit in components SP * r of its accumulator
                        const float2* pairs = reinterpret_cast<const float2*>(aux_stage + bi * 128 + g * kRowsKept * 8);
#pragma unroll
                        for (int r = 0; r < kRowsKept; ++r) {
                            const float2 pr = pairs[r];                                           // (scale, sum of codes)
                            const float f = fmaf(-zf, pr.y, static_cast<float>(acc[SP * r]));      // both terms are integers below 2^24: exact
                            y[r] = fmaf(f, __fmul_rn(pr.x, sb), y[r]);
                            if constexpr (PROBE) {
                                const int64_t blk = static_cast<int64_t>(gi) * NB + bi;
                                const int64_t row = g * kRowsKept + r;
                                if (row < p.m && n_base + c < p.n && blk < p.kb) p.acc_probe[(row * p.n + n_base + c) * p.kb + blk] = static_cast<int>(f);
                            }
                        }
                    } else {
                        const int src = FUSE ? bi * kBlockLanes : bi;         // a lane of the block, or the lane that loaded its pair
                        const float sa = __int_as_float(__builtin_amdgcn_readlane(FUSE ? __float_as_int(sa_lane) : static_cast<int>(grp.x[0].x), src));
                        const float qs = __int_as_float(__builtin_amdgcn_readlane(FUSE ? __float_as_int(qs_lane) : static_cast<int>(grp.x[0].y), src));
                        const float f = fmaf(-zf, qs, static_cast<float>(acc[0]));   // both terms are integers below 2^24: exact
                        y[0] = fmaf(f, __fmul_rn(sa, sb), y[0]);
                        if constexpr (PROBE) {                                       // row 0 sits in lanes 0..15
                            const int64_t blk = static_cast<int64_t>(gi) * NB + bi;
                            if (lane < 16 && n_base + lane < p.n && blk < p.kb) p.acc_probe[(n_base + lane) * p.kb + blk] = static_cast<int>(f);
                        }
                    }
                }
            }
        }
    };

    if constexpr (SETS == 2) {
        Grp ga, gb;
        fetch_group(ga, g_begin);
        int gi = g_begin;
        for (; gi + 1 < g_end; gi += 2) {                      // whole pairs, no branch inside: every wait counts loads exactly
            __builtin_amdgcn_sched_barrier(0);                 // nothing of a group moves up into the one before it
            fetch_group(gb, gi + 1);
            __builtin_amdgcn_sched_barrier(0);
            compute_group(ga, gi, 0);
            __builtin_amdgcn_sched_barrier(0);
            fetch_group(ga, gi + 2);                           // past the end this fetches nothing
            __builtin_amdgcn_sched_barrier(0);
            compute_group(gb, gi + 1, 1);
        }
        if (gi < g_end) compute_group(ga, gi, 0);              // an odd group out

    } else {
        Grp ga;
        for (int gi = g_begin; gi < g_end; ++gi) {
            fetch_group(ga, gi);
            compute_group(ga, gi, 0);
        }
    }

    // ---- split-K reduction across the waves of this workgroup, in wave order ----
    __syncthreads();
    float* red = reinterpret_cast<float*>(smem);
    if constexpr (MR != 1) {                           // [waves][kRowsKept][64]: lane (c, g) holds rows g * kRowsKept + r of column c
#pragma unroll
        for (int r = 0; r < kRowsKept; ++r) red[(wave * kRowsKept + r) * 64 + lane] = y[r];
        __syncthreads();
        for (int idx = threadIdx.x; idx < kRowsKept * 64; idx += blockDim.x) {
            const int r = idx >> 6;
            const int l = idx & 63;
            const int row = (l >> 4) * kRowsKept + r;
            const int64_t col = n_base + (l & 15);
            if (row < p.m && col < p.n) {
                float total = 0.f;
                for (int w = 0; w < waves; ++w) total += red[(w * kRowsKept + r) * 64 + l];
                total = with_bias(total, p.bias, p.bias_dtype, row, p.n, col, p.y_dtype);
                store_from_f32(p.y, p.y_dtype, static_cast<int64_t>(row) * p.n + col, total);
            }
        }
    } else {                                           // [waves][16]: row 0 lives in lanes 0..15
        if (lane < 16) red[wave * 16 + lane] = y[0];
        __syncthreads();
        if (threadIdx.x < 16) {
            const int64_t col = n_base + threadIdx.x;
            if (col < p.n) {
                float total = 0.f;
                for (int w = 0; w < waves; ++w) total += red[w * 16 + threadIdx.x];
                total = with_bias(total, p.bias, p.bias_dtype, 0, p.n, col, p.y_dtype);       // one row
                store_from_f32(p.y, p.y_dtype, col, total);
            }
        }
    }
}

template <int BS, typename ST>
static int launch_acc4_packed(const Acc4PackedParams& p, int waves, bool single_set, int fuse, hipStream_t stream)
{
    const unsigned grid = static_cast<unsigned>((p.n + 15) / 16);
    if (p.m > 1) {
        if constexpr (std::is_same<ST, uint16_t>::value) {
            if (p.scales_bf16) return launch_acc4_packed<BS, Bf16Scale>(p, waves, single_set, fuse, stream);
        }
        // two tiles of codes in turn + the group's pairs per wave; the reduction reuses the space (1 KiB per wave)
        const size_t lds16 = static_cast<size_t>(waves) * (2 * 16 * kCodePitchP + kGroupTiles * (128 / BS) * 128);
        if (fuse != 0) {
            // up to four f16 / bf16 rows: the kernel quantizes them itself (no codes, no pairs, no launch before this one)
            if (p.m > 4 || p.acc_probe) return -1;
            if (fuse == 2) hipLaunchKernelGGL((acc4_packed_kernel<BS, ST, 1, 2, false, 4>), dim3(grid), dim3(waves * 64), lds16, stream, p);
            else hipLaunchKernelGGL((acc4_packed_kernel<BS, ST, 1, 1, false, 4>), dim3(grid), dim3(waves * 64), lds16, stream, p);
            return static_cast<int>(hipGetLastError());
        }
        if (p.m <= 4) {
            if (p.acc_probe) hipLaunchKernelGGL((acc4_packed_kernel<BS, ST, 1, 0, true, 4>), dim3(grid), dim3(waves * 64), lds16, stream, p);
            else hipLaunchKernelGGL((acc4_packed_kernel<BS, ST, 1, 0, false, 4>), dim3(grid), dim3(waves * 64), lds16, stream, p);
        } else if (p.m <= 8) {
            if (p.acc_probe) hipLaunchKernelGGL((acc4_packed_kernel<BS, ST, 1, 0, true, 8>), dim3(grid), dim3(waves * 64), lds16, stream, p);
            else hipLaunchKernelGGL((acc4_packed_kernel<BS, ST, 1, 0, false, 8>), dim3(grid), dim3(waves * 64), lds16, stream, p);
        } else if (p.acc_probe) hipLaunchKernelGGL((acc4_packed_kernel<BS, ST, 1, 0, true, 16>), dim3(grid), dim3(waves * 64), lds16, stream, p);
        else hipLaunchKernelGGL((acc4_packed_kernel<BS, ST, 1, 0, false, 16>), dim3(grid), dim3(waves * 64), lds16, stream, p);
        return static_cast<int>(hipGetLastError());
    }
    if constexpr (std::is_same<ST, Bf16Scale>::value) {
        return -1;                                         // (several rows only)
    } else {
    const size_t lds = static_cast<size_t>(waves) * 1024;
    auto go = [&](auto fuse) {
        constexpr int F = decltype(fuse)::value;
        if (p.acc_probe) {
            if (single_set) hipLaunchKernelGGL((acc4_packed_kernel<BS, ST, 1, F, true>), dim3(grid), dim3(waves * 64), lds, stream, p);
            else hipLaunchKernelGGL((acc4_packed_kernel<BS, ST, 2, F, true>), dim3(grid), dim3(waves * 64), lds, stream, p);
        } else if (single_set) hipLaunchKernelGGL((acc4_packed_kernel<BS, ST, 1, F, false>), dim3(grid), dim3(waves * 64), lds, stream, p);
        else hipLaunchKernelGGL((acc4_packed_kernel<BS, ST, 2, F, false>), dim3(grid), dim3(waves * 64), lds, stream, p);
    };
    if (fuse == 1) go(std::integral_constant<int, 1>{});
    else if (fuse == 2) go(std::integral_constant<int, 2>{});
    else go(std::integral_constant<int, 0>{});
    return static_cast<int>(hipGetLastError());
    }
}

static int packed_groups(const RocmMatMulNBitsArgs* a)
{
    const int64_t kb = (a->k + a->block_size - 1) / a->block_size;
    const int64_t tiles = (kb * a->block_size + 127) / 128;
    return static_cast<int>((tiles + kGroupTiles - 1) / kGroupTiles);
}

static int packed_chunk_bytes(const RocmMatMulNBitsArgs* a)
{
    return kChunkWeights + 16 * packed_record_bytes(a->block_size, a->scale_dtype == ROCM_DT_F32 ? 4 : 2);
}

}  // namespace mnb

// Rows 5..64 only run from the repacked copy in the shared-activation kernel, which wants many column groups.
// (16 rows at block size 32, 32 at 64, 64 at 128: more row blocks than that do not fit the register file)
// `pair`: the call is the fused gate/up launch or one of its two projections - both projections' columns count, since the
// paired launch streams both, and a projection launched on its own must add up the way the paired launch does.
// The shared-activation kernel's window below five rows: block 128 on 18432 .. 49151 columns, four rows of a plain call, two to
// four of a gate/up pair (whose columns count together).
static bool few_row_wide(const RocmMatMulNBitsArgs* a, bool pair)
{
    const int64_t cols = a->n * (pair ? 2 : 1);
    return a->m <= 4 && a->m >= (pair ? 2 : 4) && a->block_size == 128 && cols >= 18432 && cols < 49152;
}

static bool wide_shape(const RocmMatMulNBitsArgs* a, bool pair)
{
    const int64_t max_rows = a->block_size == 32 ? 16 : a->block_size == 64 ? 32 : 64;
    // Columns from which it beats the other kernels. 17 rows and more (against the tiled kernel and two passes of the
    // split-K kernel; bf16, 4096 -> 14336: 30.6 -> 24.4 us at 32 rows with block 128, 31.5 -> 25.7 with block 64; 33-64 rows
    // lose below 16384 columns: 32.9 -> 38.7 us). Up to 16 rows the 16-row split-K kernel over the same repacked stream is
    // the alternative, and with 4096 rows of K it stays ahead up to 16384 columns at block 128 (5 / 8 / 16 rows, 14336
    // columns: 12.0 / 12.1 / 13.8 against 13.2 / 13.3 / 14.2 us; 16384: 12.5 / 12.8 / 14.4 against 13.4 / 13.5 / 14.5; at 20480
    // it loses, 14.9-17.3 against 14.1-15.3) and up to 20480 at block 32 (14336: 13.2 / 13.2 / 14.7 against 17.1 / 17.2 / 17.7;
    // 20480: 16.9 / 17.2 / 18.6 against 17.8 / 17.9 / 18.4; at 28672 it loses, 22-25 against 20-21).
    // (block 64: 12.3 / 12.6 / 14.4 us at 14336 and 13.2 / 13.7 / 15.2 at 16384 against 15.4-16.0 in the shared-activation kernel)
    const int64_t min_cols = a->m > 32 ? 16384 : a->m > 16 ? 14336 : a->block_size == 32 ? 22528 : a->block_size == 64 ? 20480 : 18432;
    // Four rows of a plain call on 18432 .. 49151 columns at block 128 run here as well: level with the four-row split-K build
    // on a GPU that runs it well (3584 -> 37888 18.1 -> 17.6 us, 4096 -> 28672 16.0 -> 16.2, 3072 -> 32064 13.8 -> 13.5), and this kernel
    // moved far less from one GPU to the next (on two others the same three calls took 21-22.5 / 18.0-18.3 / 16.8-17.0 us there
    // against 18.8 / 16.5 / 14.9-15.4 at five rows here). More columns lose (4096 -> 128256: 56.4 -> 62.3), and so do three rows.
    // A gate/up pair counts both projections' columns, as below, and comes here from two rows: the paired four-row split-K
    // launch is further behind than the plain one (3584 -> 2 x 18944 at 2 / 3 / 4 rows: 20.2-21.2 / 20.5-21.1 / 20.9 -> 17.9 / 18.5 /
    // 18.9 us, the unfused call over 37888 columns 18.5 at four; 5120 -> 2 x 13824: 20.0 / 20.4-21.3 -> 18.6-18.9 / 19.0-19.7;
    // 4096 -> 2 x 14336 level).
    if (few_row_wide(a, pair)) return a->gamma == nullptr;
    return a->m >= 5 && a->m <= max_rows && a->n * (pair ? 2 : 1) >= min_cols;
}

extern "C" int rocm_decode_packed_eligible(const RocmMatMulNBitsArgs* a)
{
    RocmMatMulNBitsArgs base = *a;
    if (base.m > 16) base.m = 16;                         // the shared-activation kernel takes up to 64 rows
    if (!rocm_decode_mfma_eligible(&base)) return 0;
    if (a->m * a->k * 2 >= 0x7ffffff0) return 0;
    if (a->m > 16 && !wide_shape(a, false)) return 0;    // up to 16 rows the split-K kernel stages the rows per wave
    return static_cast<int64_t>(mnb::packed_groups(a)) * mnb::packed_chunk_bytes(a) < 0x7fffffff;
}

extern "C" uint64_t rocm_decode_packed_bytes(const RocmMatMulNBitsArgs* a)
{
    const uint64_t col_groups = static_cast<uint64_t>((a->n + 15) / 16);
    return col_groups * static_cast<uint64_t>(mnb::packed_groups(a)) * static_cast<uint64_t>(mnb::packed_chunk_bytes(a));
}

extern "C" int rocm_launch_pack_decode(const RocmMatMulNBitsArgs* a, void* packed, rocm_stream_t stream)
{
    mnb::PackParams p;
    p.b = a->b;
    p.scales = a->scales;
    p.zp = a->zp;
    p.out = static_cast<uint8_t*>(packed);
    p.n = a->n;
    p.kb = (a->k + a->block_size - 1) / a->block_size;
    p.row_bytes = p.kb * a->block_size / 2;
    p.zp_row = (p.kb + 1) / 2;
    p.bs_log2 = __builtin_ctz(static_cast<unsigned>(a->block_size));
    p.scale_bytes = a->scale_dtype == ROCM_DT_F32 ? 4 : 2;
    p.groups = mnb::packed_groups(a);
    p.chunk_bytes = mnb::packed_chunk_bytes(a);
    p.record = mnb::packed_record_bytes(a->block_size, p.scale_bytes);
    const dim3 grid(static_cast<unsigned>(p.groups), static_cast<unsigned>((a->n + 15) / 16));
    hipLaunchKernelGGL(mnb::pack_decode_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), p);
    return static_cast<int>(hipGetLastError());
}

// The launch of rocm_launch_decode_packed; with `packed_up` the paired gate/up launch. `probe_only`: nothing is launched,
// the return value says whether a paired launch with this split of K fits a workgroup (1) or not (0).
// `pair_member`: the launch is one projection of a gate/up pair (or the paired launch itself): the split of K is chosen
// for the pair's column groups together, so that the separate launches and the paired one add up in the same order.
extern "C" int rocm_decode_packed_fuses_norm(const RocmMatMulNBitsArgs* a)
{
    if (!a->gamma || a->m > 4 || a->k % 128 != 0 || !rocm_decode_packed_eligible(a)) return 0;      // (with gamma, up to four rows never take the shared-activation kernel)
    // Where up to four rows take the shared-activation kernel (alone, or as one projection of a pair), the rows are normalized
    // by a launch of their own: a pair's first call runs its projections over normalized rows, and the later single launch has
    // to add up in the same order.
    if (few_row_wide(a, false) || few_row_wide(a, true)) return 0;
    if (a->gamma_dtype != ROCM_DT_F32 && a->gamma_dtype != a->a_dtype) return 0;
    return (reinterpret_cast<uintptr_t>(a->gamma) & 15) == 0;
}

// Waves per SIMD of the one-set builds, from the registers the compiler reported for them (59-76 with one row, 71-102 with
// four, 84-112 with eight, 110-134 with sixteen); a test holds the table against the build's report.
static int waves_per_simd(const RocmMatMulNBitsArgs* a, bool f32_scales)
{
    // [f16 / bf16][rows: 1, 2-4, 5-8, 9-16][block 32, 64, 128][16-bit / f32 scales]
    static const unsigned char table[2][4][3][2] = {
        {{{5, 6}, {7, 7}, {8, 8}}, {{5, 4}, {5, 6}, {6, 6}}, {{4, 4}, {5, 5}, {5, 5}}, {{4, 3}, {4, 4}, {3, 4}}},
        {{{7, 6}, {8, 7}, {8, 8}}, {{5, 4}, {6, 6}, {7, 6}}, {{4, 4}, {5, 5}, {5, 5}}, {{4, 3}, {4, 4}, {4, 4}}},
    };
    const int rows = a->m <= 1 ? 0 : a->m <= 4 ? 1 : a->m <= 8 ? 2 : 3;
    const int block = a->block_size == 32 ? 0 : a->block_size == 64 ? 1 : 2;
    return table[a->a_dtype == ROCM_DT_BF16][rows][block][f32_scales];
}

extern "C" int rocm_decode_packed_waves_per_simd(int block_size, int m, int f32_scales, int bf16)
{
    RocmMatMulNBitsArgs a{};
    a.block_size = block_size;
    a.m = m;
    a.a_dtype = bf16 ? ROCM_DT_BF16 : ROCM_DT_F16;
    return waves_per_simd(&a, f32_scales != 0);
}

// the most waves a workgroup of decode_packed_kernel may have (see the kernel's launch bounds)
static int w_max_of(const RocmMatMulNBitsArgs* a, bool f32_scales)
{
    return (a->block_size == 128 && !f32_scales && (a->m <= 8 || a->a_dtype == ROCM_DT_BF16)) ? 16 : 8;
}

// What rocm_launch_decode_packed launches for a shape, without launching it: which kernel, which build of it, how many waves
// split K and over how many register sets. Everything below is arithmetic on the shape and the chip's CU count (the
// thresholds were measured on 256 CUs and are written as multiples of that count), so a CPU test can hold the answers for
// the model shapes against a committed table: a change made for one shape cannot move another unnoticed.
struct PackedPlan {
    bool wide;          // the shared-activation kernel (plan in `w`); otherwise the split-K kernel
    mnb::WidePlan w;
    int rows_build;     // split-K kernel: rows the build stages (1, 4, 8, 16)
    int waves;          // per projection and workgroup
    int groups_per_wave;
    bool single_set;
};

static PackedPlan plan_decode_packed(const RocmMatMulNBitsArgs* a, int waves, bool pair_member, bool paired_launch, int64_t cus)
{
    PackedPlan plan{};
    const bool f32_scales = a->scale_dtype == ROCM_DT_F32;
    if (wide_shape(a, pair_member)) {
        plan.wide = true;
        plan.w = mnb::plan_wide(a->m, a->n, a->block_size, !f32_scales, paired_launch, cus);
        plan.groups_per_wave = mnb::packed_groups(a);
        plan.waves = plan.w.waves;
        return plan;
    }
    const int groups = mnb::packed_groups(a);
    // Waves per workgroup (they split K in whole tile groups). Many column groups (thousands of waves even at four per
    // group): short waves of at most two tile groups. Few column groups: enough waves per group to reach about 8k in
    // flight. Then the adjustments below: register sets, and wave counts that fit the chip.
    const int64_t wgs = (a->n + 15) / 16 * ((pair_member && a->m <= 4) ? 2 : 1);      // (a pair shares a launch up to four rows here)
    int w = waves;
    const int w_max = w_max_of(a, f32_scales);
    // One row: one tile group per wave where the workgroup can hold that many waves, no prefetch, offset and zero point
    // through the activation sums. Every byte of the call is then requested as soon as its wave starts, and what a wave
    // computes between its loads and the reduction is the least any variant here does. Measured against the few-wave
    // prefetching build it replaced on the small shapes (bf16, block 128): 3584 -> 4608 5.06 -> 4.78 us, 3584 -> 3584
    // 4.17 -> 3.97, 18944 -> 3584 9.94 -> 9.41, 3584 -> 37888 15.81 -> 15.48.
    // (a gate/up pair keeps the few-wave split: with fourteen waves a workgroup the paired launch measured 17.8 us against 15.5)
    const bool one_row = a->m <= 1 && !pair_member;
    const bool large_grid = wgs * 4 >= 24 * cus;
    if (w <= 0) {
        if (one_row) {
            w = groups;
        } else if (large_grid) {
            w = (groups + 1) / 2;
        } else {
            const int want = static_cast<int>((32 * cus + wgs - 1) / wgs);
            w = want < groups ? want : groups;               // at least one group per wave
        }
        if (w < 1) w = 1;
    }
    // One register set or two (the second holds the next group's loads while the current one is multiplied, at the price
    // of waves per SIMD). Swept over 384 .. 1024 column groups x K = 3584 .. 8192 x 1 / 2 / 4 rows x block 32 / 128: one set is
    // ahead or level nearly everywhere, by up to 30 % from K = 5120 (block 128, 4 rows, 5120 -> 16384: 12.4 against 16.5 us;
    // block 32: 15.8 against 21.7). Two sets keep:
    //  * two to four rows on small grids, where the second set's first fetch, issued before anything else, is worth 1-3 %
    //    (block 128, 3584 -> 4608: 5.56 against 5.72 us; 18944 -> 3584 at block 32: 13.3 against 13.9) - below 256 column groups at
    //    block 32, else up to 512 (two workgroups per CU: 4096 -> 8192 6.4 against 6.5 us at two rows, but 4096 -> 9216 7.7 against
    //    7.3 and 3072 -> 9216 7.75 against 6.8), or below 320 when K is more than eight groups;
    //  * one row at block size 32 with more groups than a workgroup has waves, on small grids: sixteen scale steps per group
    //    leave enough arithmetic between a wave's loads that fetching ahead pays (18944 -> 3584 12.4 -> 11.8 us; with 1024
    //    column groups it loses, 5120 -> 16384: 17.3 against 12.2; at block 128 one set stays ahead, 9.5 against 9.9 us).
    bool single_set;
    if (one_row) single_set = !(a->block_size == 32 && groups > w_max && wgs <= cus);
    else if (a->block_size == 32) single_set = wgs >= cus;
    else single_set = wgs > 2 * cus || (wgs >= cus + cus / 4 && groups > 8);
    if (w > w_max) w = w_max;
    if (w > groups) w = groups;
    // Mid-size grids: a launch whose waves do not all fit the chip at once queues workgroups behind each other, and
    // workgroups of 6, 10 or 12 waves leave slots of a CU empty on top; fewer waves of more groups each run it faster
    // (16 rows, block 128: 3072 -> 16384 13.8 -> 12.2 us, 5120 -> 13824 21.0 -> 17.6, 6144 -> 16384 24.6 -> 21.1, 5120 -> 17920
    // 24.1 -> 21.7; 8 rows: 16.2 -> 13.9 on 5120 -> 13824; one row: 7168 -> 16384 16.2 -> 14.3; 4 rows at block 32: 3584 -> 16384
    // 12.5 -> 11.4). Workgroups of eight waves of one group each fill a CU's slots exactly and stay (K = 4096, 16 rows: 14336
    // columns 13.9 against 14.9 us with four waves, 11008 11.3 against 11.6), and so do the large grids, whose waves are
    // short enough for the queue not to show (one row, 3584 -> 37888: seven waves of one group, 15.5 against 15.8 us).
    // Which of the wave counts that fit: a workgroup's waves go round the four SIMDs, so k workgroups of w waves put
    // k * ceil(w / 4) of them on the first SIMD, and with three to five waves per SIMD a workgroup of 5, 6 or 10 waves keeps
    // a CU from filling up (16 rows, 5120 -> 13824: five waves 21.4 us, four 17.5, ten 21.0; 2 rows at block 32, 8192 -> 12288:
    // six waves 18.9 us, four 16.6). Builds of up to five waves per SIMD take the count that holds the most waves per CU that way.
    if (waves <= 0 && !(w == 8 && groups == 8)) {
        const int per_simd = waves_per_simd(a, f32_scales);
        const int64_t fit = cus * 4 * per_simd / wgs;
        const int64_t least = a->m <= 1 ? 6 : a->m <= 4 ? 4 : 1;
        // A count within that bound can still be too many once the waves' places on the SIMDs are counted (576 workgroups of six
        // waves at five waves per SIMD: two workgroups a CU, 3072 slots for 3456 waves). Then the count that holds the most is
        // taken as well, if it leaves a wave two tile groups at most (block 32, two / four rows: 3072 -> 9216 8.9 / 8.9 -> 8.3 / 8.7 us,
        // 3072 -> 12288 10.0 / 10.1 -> 8.5 / 9.0; block 128, five / eight rows: 3072 -> 12288 9.2 -> 8.1; with three groups a wave it
        // lost, 5120 -> 10240 at block 32: 10.1 -> 10.8).
        const bool crowded = per_simd <= 5 && w <= fit && wgs * w > cus * static_cast<int64_t>(per_simd / ((w + 3) / 4) * w);
        if (fit >= least && (w > fit || crowded)) {
            if (w > fit) w = static_cast<int>(fit);
            const int limit = w;
            if (per_simd <= 5) {                       // (with six or more waves per SIMD the plain count is as good or better: 4 rows at block 128, 6144 -> 16384: six waves 14.2 us, four 15.4)
                int best = -1;
                for (int g = 1; g <= groups; ++g) {
                    const int cand = (groups + g - 1) / g;
                    if (cand > limit || (crowded && g > 2)) continue;
                    const int held = per_simd / ((cand + 3) / 4) * cand;
                    if (held > best) {                 // (ties: the first found, which has the most waves)
                        best = held;
                        w = cand;
                    }
                    if (cand == 1) break;
                }
            }
        }
    }
    // A projection of a gate/up pair takes at most half a workgroup's waves where that leaves a wave five tile groups or fewer,
    // so that the pair runs as one launch and not as two and the epilogue (bf16, one / two / four rows: 3072 -> 2 x 8192 at block 32
    // 14.3 -> 9.1 us at one row; 5120 -> 2 x 13824 at block 32 25.5 / 30.9 / 32.6 -> 20.6 / 25.4 / 25.7, at block 64 24.1 / 26.5 / 28.0 ->
    // 18.8 / 21.7 / 22.8; 8192 -> 2 x 8192 at block 64 22.5 / 25.3 / 26.8 -> 17.7 / 18.6 / 19.9). The projection launched alone on a
    // pair's first call takes the same count, as everything here.
    if (pair_member && a->m <= 4 && waves <= 0 && 2 * w > w_max && (groups + w_max / 2 - 1) / (w_max / 2) <= 5) w = w_max / 2;
    const int gpw = (groups + w - 1) / w;
    w = (groups + gpw - 1) / gpw;
        plan.rows_build = a->m <= 1 ? 1 : a->m <= 4 ? 4 : a->m <= 8 ? 8 : 16;
    plan.waves = w;
    plan.groups_per_wave = gpw;
    plan.single_set = a->m > 4 || single_set || (a->m > 1 && a->gamma != nullptr);
    return plan;
}

extern "C" int rocm_decode_packed_plan(const RocmMatMulNBitsArgs* a, int waves, int pair_member, int compute_units, RocmDecodePackedPlan* out)
{
    if (!a || !out || compute_units <= 0 || !rocm_decode_packed_eligible(a)) return -1;
    const PackedPlan plan = plan_decode_packed(a, waves, pair_member != 0, pair_member == 2, compute_units);
    if (plan.wide && !plan.w.ok) return -1;
    const int64_t col_groups = (a->n + 15) / 16;
    out->shared_activations = plan.wide;
    out->rows_build = plan.wide ? plan.w.rb * 16 : plan.rows_build;
    out->waves = plan.waves;
    out->groups_per_wave = plan.groups_per_wave;
    out->register_sets = plan.wide ? ((plan.w.pf ? 1 : 0) + (plan.w.deep ? 1 : 0) + 1) : (plan.single_set ? 1 : 2);
    out->activation_sums = plan.wide ? plan.w.sums : (plan.rows_build == 1 && plan.single_set);
    out->workgroups = plan.wide ? static_cast<int64_t>(plan.w.grid) : col_groups;
    return 0;
}

static int launch_decode_packed(const RocmMatMulNBitsArgs* a, const void* packed, const void* packed_up, int decomposed, int waves, bool probe_only,
                                bool pair_member, rocm_stream_t stream)
{
    if (!rocm_decode_packed_eligible(a)) return probe_only ? 0 : -1;
    const int64_t cus = rocm_ffi_compute_units();
    const PackedPlan plan = plan_decode_packed(a, waves, pair_member, packed_up != nullptr, cus);
    mnb::PackedParams p;
    p.a = static_cast<const uint16_t*>(a->a);
    p.packed = static_cast<const uint8_t*>(packed);
    p.packed_up = static_cast<const uint8_t*>(packed_up);
    p.decomposed_silu = decomposed;
    p.bias = a->bias;
    p.y = a->y;
    p.m = a->m;
    p.n = a->n;
    p.k = a->k;
    p.groups = mnb::packed_groups(a);
    p.chunk_bytes = mnb::packed_chunk_bytes(a);
    p.cg_stride = static_cast<int64_t>(p.groups) * p.chunk_bytes;
    p.bias_dtype = a->bias_dtype;
    p.y_dtype = a->y_dtype;
    p.nibble_mask = 0x000F000Fu;
    const bool bf16 = a->a_dtype == ROCM_DT_BF16;
    p.magic = bf16 ? 0x43004300u : 0x64006400u;
    p.gamma = nullptr;
    p.gamma_f32 = 0;
    p.norm_epsilon = 0.f;
    if (a->gamma) {
        if (!rocm_decode_packed_fuses_norm(a)) return probe_only ? 0 : -1;
        p.gamma = a->gamma;
        p.gamma_f32 = a->gamma_dtype == ROCM_DT_F32;
        p.norm_epsilon = a->norm_epsilon;
    }

    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool f32_scales = a->scale_dtype == ROCM_DT_F32;
    if (plan.wide) {
        // the shared-activation kernel's paired form takes up to 16 rows (one block of rows per wave)
        if (probe_only) return a->m <= 16 ? 1 : 0;
        if (packed_up && a->m > 16) return -1;
        p.groups_per_wave = p.groups;
        if (bf16) return f32_scales ? mnb::launch_wide_bs<true, float>(p, a->block_size, cus, s) : mnb::launch_wide_bs<true, uint16_t>(p, a->block_size, cus, s);
        return f32_scales ? mnb::launch_wide_bs<false, float>(p, a->block_size, cus, s) : mnb::launch_wide_bs<false, uint16_t>(p, a->block_size, cus, s);
    }
    const int w = plan.waves;
    const int w_max = w_max_of(a, f32_scales);
    const bool single_set = plan.single_set;
    p.groups_per_wave = plan.groups_per_wave;
    // a paired launch keeps each projection's own split of K (so that it adds up in the same order) and needs twice the waves
    if (probe_only) return a->m <= 4 && 2 * w <= w_max ? 1 : 0;
    if (packed_up && (a->m > 4 || 2 * w > w_max)) return -1;

    if (bf16) return f32_scales ? mnb::launch_packed_bs<true, float>(p, a->block_size, w, single_set, s) : mnb::launch_packed_bs<true, uint16_t>(p, a->block_size, w, single_set, s);
    return f32_scales ? mnb::launch_packed_bs<false, float>(p, a->block_size, w, single_set, s) : mnb::launch_packed_bs<false, uint16_t>(p, a->block_size, w, single_set, s);
}

extern "C" int rocm_launch_decode_packed(const RocmMatMulNBitsArgs* a, const void* packed, int waves, rocm_stream_t stream)
{
    return launch_decode_packed(a, packed, nullptr, 0, waves, false, false, stream);
}

extern "C" int rocm_launch_decode_packed_pair_member(const RocmMatMulNBitsArgs* a, const void* packed, int waves, rocm_stream_t stream)
{
    return launch_decode_packed(a, packed, nullptr, 0, waves, false, true, stream);
}

extern "C" int rocm_decode_packed_pair_fits(const RocmMatMulNBitsArgs* a, int waves)
{
    return launch_decode_packed(a, nullptr, nullptr, 0, waves, true, true, nullptr);
}

extern "C" int rocm_launch_decode_packed_pair(const RocmMatMulNBitsArgs* a, const void* packed_gate, const void* packed_up, int decomposed, int waves,
                                              rocm_stream_t stream)
{
    if (!packed_gate || !packed_up || a->y_dtype != a->a_dtype) return -1;
    return launch_decode_packed(a, packed_gate, packed_up, decomposed, waves, false, true, stream);
}

extern "C" int rocm_acc4_packed_eligible(const RocmMatMulNBitsArgs* a)
{
    const bool bs_ok = a->block_size == 32 || a->block_size == 64 || a->block_size == 128;
    if (!(bs_ok && a->m >= 1 && a->m <= 16 && a->n >= 1)) return 0;
    if ((reinterpret_cast<uintptr_t>(a->b) & 15) != 0 || (reinterpret_cast<uintptr_t>(a->scales) & 3) != 0) return 0;
    const int64_t padded_k = (a->k + a->block_size - 1) / a->block_size * a->block_size;
    if (a->m * padded_k >= 0x7fffffff) return 0;                          // the codes are addressed with 32-bit offsets
    return static_cast<int64_t>(mnb::packed_groups(a)) * mnb::packed_chunk_bytes(a) < 0x7fffffff;
}

extern "C" int rocm_acc4_packed_fuses_quantizer(const RocmMatMulNBitsArgs* a)
{
    if (!(rocm_acc4_packed_eligible(a) && (a->a_dtype == ROCM_DT_F16 || a->a_dtype == ROCM_DT_BF16) && a->k % 8 == 0 && (reinterpret_cast<uintptr_t>(a->a) & 15) == 0))
        return 0;
    if (a->m == 1) return 1;
    // Two to four rows: every workgroup quantizes the rows again, which more than doubles what a wave computes per tile
    // group - worth it only where the call is short enough for the quantizer's own launch (about 3 us) to weigh more:
    // 3584 -> 3584 8.2 -> 6.3 us, 3584 -> 4608 8.9 -> 8.0; 4096 -> 14336 level; 18944 -> 3584 14.5 -> 16.6 and 3584 -> 37888 19.6 -> 22.4
    // the wrong way. (The builds that probe block accumulators read the workspace's codes.)
    const int64_t work = (a->n + 15) / 16 * mnb::packed_groups(a);            // column groups x tile groups
    return a->m <= 4 && !a->acc_probe && work <= 4096;
}

// Waves per workgroup, tile groups per wave and register sets of rocm_launch_acc4_packed for a shape on a chip of `cus` CUs
// (thresholds measured on 256 CUs, written as multiples of the count). No GPU work.
static void plan_acc4_packed(const RocmMatMulNBitsArgs* a, int waves, int64_t cus, int* waves_out, int* groups_per_wave, bool* one_set)
{
    const int groups = mnb::packed_groups(a);
    const int64_t wgs = (a->n + 15) / 16;
    int w = waves;
    bool single_set = wgs * 4 >= 24 * cus;
    if (w <= 0) {
        if (single_set) {
            w = (groups + 1) / 2;
        } else {
            const int want = static_cast<int>((32 * cus + wgs - 1) / wgs);
            w = want < groups ? want : groups;
        }
        if (w < 1) w = 1;
    } else {
        single_set = wgs * w >= 24 * cus;
    }
    if (w > 8) w = 8;
    if (w > groups) w = groups;
    const int gpw = (groups + w - 1) / w;
    w = (groups + gpw - 1) / gpw;
    // One register set (one-row launches; the builds for several rows have no other): with one group per wave a second set
    // has nothing to fetch ahead (4096 -> 14336: 14.3 -> 9.8 us at block 32, 9.7 -> 8.8 at 64, 9.2 -> 8.4 at 128); at block 32 the
    // two-set build holds three waves per SIMD against eight (5120 -> 13824 21.4 -> 11.6 us, 6144 -> 16384 23.8 -> 14.4,
    // 8192 -> 8192 14.1 -> 10.5); and from a few hundred column groups on the other block sizes are level or ahead with one
    // (13824 -> 5120 at block 128: 12.3 -> 11.2; 8192 -> 10240 at 64: 12.3 -> 11.5). Small K-heavy grids keep two (18944 -> 3584 at
    // block 128: 9.3 against 10.2 us).
    if (gpw == 1 || a->block_size == 32 || wgs > cus) single_set = true;

    *waves_out = w;
    *groups_per_wave = gpw;
    *one_set = single_set;
}

extern "C" int rocm_acc4_packed_plan(const RocmMatMulNBitsArgs* a, int waves, int compute_units, int* waves_out, int* groups_per_wave, int* register_sets)
{
    if (!a || compute_units <= 0 || !rocm_acc4_packed_eligible(a)) return -1;
    int w = 0, gpw = 0;
    bool one_set = false;
    plan_acc4_packed(a, waves, compute_units, &w, &gpw, &one_set);
    if (waves_out) *waves_out = w;
    if (groups_per_wave) *groups_per_wave = gpw;
    if (register_sets) *register_sets = (one_set || a->m > 1) ? 1 : 2;
    return 0;
}

extern "C" int rocm_launch_acc4_packed(const RocmMatMulNBitsArgs* a, const void* packed, const RocmAcc4Workspace* ws, int rounding, int waves, rocm_stream_t stream)
{
    if (!rocm_acc4_packed_eligible(a)) return -1;
    const int fuse = ws ? 0 : (a->a_dtype == ROCM_DT_BF16 ? 2 : 1);
    if (!ws && !rocm_acc4_packed_fuses_quantizer(a)) return -1;
    mnb::Acc4PackedParams p;
    p.qa = ws ? ws->qa : nullptr;
    p.aq = ws ? ws->aq : nullptr;
    p.aux16 = ws ? ws->aux : nullptr;
    p.m = a->m;
    p.a = a->a;
    p.k = a->k;
    p.rounding = rounding;
    p.packed = static_cast<const uint8_t*>(packed);
    p.bias = a->bias;
    p.y = a->y;
    p.n = a->n;
    p.kb = (a->k + a->block_size - 1) / a->block_size;
    p.padded_k = p.kb * a->block_size;
    p.groups = mnb::packed_groups(a);
    p.chunk_bytes = mnb::packed_chunk_bytes(a);
    p.cg_stride = static_cast<int64_t>(p.groups) * p.chunk_bytes;
    p.bias_dtype = a->bias_dtype;
    p.y_dtype = a->y_dtype;
    p.scales_bf16 = a->scale_dtype == ROCM_DT_BF16;
    p.acc_probe = a->acc_probe;

    int w = 0, gpw = 0;
    bool single_set = false;
    plan_acc4_packed(a, waves, rocm_ffi_compute_units(), &w, &gpw, &single_set);
    p.groups_per_wave = gpw;

    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool f32_scales = a->scale_dtype == ROCM_DT_F32;
    switch (a->block_size) {
        case 32: return f32_scales ? mnb::launch_acc4_packed<32, float>(p, w, single_set, fuse, s) : mnb::launch_acc4_packed<32, uint16_t>(p, w, single_set, fuse, s);
        case 64: return f32_scales ? mnb::launch_acc4_packed<64, float>(p, w, single_set, fuse, s) : mnb::launch_acc4_packed<64, uint16_t>(p, w, single_set, fuse, s);
        default: return f32_scales ? mnb::launch_acc4_packed<128, float>(p, w, single_set, fuse, s) : mnb::launch_acc4_packed<128, uint16_t>(p, w, single_set, fuse, s);
    }
}
