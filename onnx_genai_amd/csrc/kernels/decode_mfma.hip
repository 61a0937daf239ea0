// Decode path of MatMulNBits (M <= 16, f16/bf16 activations): a split-K GEMV on the matrix cores.
//
// Work split. A workgroup owns 16*CG output columns; its waves split K between them in runs of
// 128-element tiles and meet once at the end in LDS, in wave order, so the result is deterministic.
//
// Streaming. Lane (c = lane % 16, g = lane / 16) reads, per tile, one 16-byte piece of packed
// column c: 32 nibbles that never leave registers. Each of its four dwords becomes the eight
// 16-bit operands one v_mfma_f32_16x16x32 wants from that lane, by OR-ing the nibble under a
// constant exponent ("magic" value: 1024+q as f16, 128+q as bf16 - both exact). The activation
// rows are the other MFMA operand (rows beyond M read as zero). A second MFMA per dword, whose
// weight operand is the constant -(magic+zp), removes magic and zero point inside the f32
// accumulator, so the accumulator holds sum a*(q-zp) for the block and is scaled once per block:
//     y += scale[n, block] * acc.
// For block sizes below 128 the four lane groups first swap dwords (two v_permlane*_swap stages,
// a 4x4 transpose) so that one MFMA never mixes two blocks.
//
// Memory. All global loads are buffer loads with hardware range checking, so ragged edges
// (columns beyond N, rows beyond M, the end of K) cost no branches: they read zeros. A wave keeps
// two groups of tiles in registers: while the MFMAs consume one, the loads of the next are in
// flight. Activations travel with their tile in the most compact form (one 16-byte piece per lane
// per four rows) and are turned into MFMA operand order through a small wave-private LDS buffer,
// whose reads are counted separately from global loads and so never drain the prefetch queue.
#include "mfma_common.hiph"

namespace mnb {

typedef __attribute__((ext_vector_type(8))) _Float16 half8_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float float4_t;

struct DecodeParams {
    const uint16_t* a;
    const uint8_t* b;
    const void* scales;
    const uint8_t* zp;
    const void* bias;
    void* y;
    int64_t m, n, k, kb;
    int64_t row_bytes;      // packed bytes of one column: kb * BS / 2
    int64_t zp_row;         // ceil(kb / 2)
    int tiles;              // ceil(K / 128)
    int tiles_per_wave;     // multiple of the group size
    int bias_dtype, y_dtype;
    uint32_t nibble_mask;   // 0x000F000F
    uint32_t magic;         // two 16-bit magic exponents (see Magic<>::pos); passed in so that the compiler keeps it in a register
};

template <bool BF16> struct Magic;
template <> struct Magic<false> { static constexpr uint32_t pos = 0x64006400u, neg = 0xE400E400u; };
template <> struct Magic<true> { static constexpr uint32_t pos = 0x43004300u, neg = 0xC300C300u; };

constexpr int kRowPitch = 272;                   // bytes between activation rows in LDS: 256 + 16, so 16 rows hit 64 distinct banks

template <bool BF16>
__device__ __forceinline__ float4_t mfma16(const uint4& act, const uint4& wgt, float4_t acc)
{
    if constexpr (BF16) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, act), __builtin_bit_cast(bf16x8_t, wgt), acc, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, act), __builtin_bit_cast(half8_t, wgt), acc, 0, 0, 0);
    }
}

__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t bits)
{
    return (x & mask) | bits;   // v_and_or_b32: both constants arrive as kernel arguments, so neither is a literal
}

// Eight nibbles of `w` (k ascending from bit 0) -> four registers of two 16-bit floats (magic + q),
// element 2i in the low half and 2i+1 in the high half: the order activations lie in memory.
__device__ __forceinline__ uint4 unpack8(uint32_t w, uint32_t mask, uint32_t magic)
{
    const uint32_t w4 = w >> 4;
    uint4 r;
    r.x = and_or(__builtin_amdgcn_perm(w4, w, 0x0c040c00u), mask, magic);
    r.y = and_or(__builtin_amdgcn_perm(w4, w, 0x0c050c01u), mask, magic);
    r.z = and_or(__builtin_amdgcn_perm(w4, w, 0x0c060c02u), mask, magic);
    r.w = and_or(__builtin_amdgcn_perm(w4, w, 0x0c070c03u), mask, magic);
    return r;
}

// One group of U tiles held in registers: packed weights of CG column groups, the activations in compact
// form, scales and zero points. NA / NS count the activation / scale loads of a group (see the kernel).
template <int U, int CG, int NA, int NS, typename SRaw>
struct Group {
    uint4 w[U][CG];
    uint4 a[NA];
    SRaw s[NS][CG];             // as loaded; widened where used, so that nothing waits for the load before that
    unsigned char z[NS][CG];
};

// BF16: activation element type. BS: block size (32, 64, 128). CG: 16-column groups per workgroup.
// MR: rows staged (1, 4, 8 or 16; M <= MR). ST: storage type of the scales (uint16_t = the activations'
// 16-bit type, float = f32).
//
// Vector memory instructions, not bytes, are what this kernel runs out of first, so everything except the
// weights is fetched as rarely as possible: with one row (MR = 1) the activations of a whole group arrive in
// one 16-byte-per-lane load; with block size 128 the scale and zero point of tile t0 + g are loaded once per
// group by lane group g and handed to the other lanes with a lane shuffle.
template <bool BF16, int BS, int CG, int MR, typename ST>
__global__ __launch_bounds__(512) void decode_mfma_kernel(DecodeParams p)
{
    constexpr bool kTranspose = BS < 128;              // several blocks inside one 128-element tile
    constexpr int kBsLog2 = BS == 32 ? 5 : BS == 64 ? 6 : 7;
    constexpr int kBlocksPerTile = 128 / BS;
    constexpr int AR = (MR + 3) / 4;                    // 16-byte activation pieces per lane per tile (MR > 1)
    constexpr int U = (CG == 1 && MR <= 4) ? 4 : 2;     // tiles per prefetch group
    constexpr bool kGroupA = MR == 1;                   // one activation load per group
    constexpr int NA = kGroupA ? 1 : U * AR;
    constexpr bool kGroupS = !kTranspose;               // one scale / zero-point load per group
    constexpr int NS = kGroupS ? 1 : U;
    constexpr int kStageBytes = kGroupA ? 1024 : MR * kRowPitch;   // one staging buffer in LDS (a group / a tile)
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform by construction; say so, or every
    const int waves = blockDim.x >> 6;                                   // tile offset below is treated as divergent
    const int c = lane & 15;
    const int g = lane >> 4;
    const int64_t n_base = static_cast<int64_t>(blockIdx.x) * (16 * CG);
    const int64_t cols_left = p.n - n_base;
    const bool has_zp = p.zp != nullptr;

    const __amdgpu_buffer_rsrc_t srd_b = make_srd(p.b + n_base * p.row_bytes, static_cast<uint64_t>(cols_left * p.row_bytes));
    const __amdgpu_buffer_rsrc_t srd_s = make_srd(static_cast<const ST*>(p.scales) + n_base * p.kb, static_cast<uint64_t>(cols_left * p.kb) * sizeof(ST));
    const __amdgpu_buffer_rsrc_t srd_z = make_srd(has_zp ? p.zp + n_base * p.zp_row : p.b, has_zp ? static_cast<uint64_t>(cols_left * p.zp_row) : 0);
    const __amdgpu_buffer_rsrc_t srd_a = make_srd(p.a, static_cast<uint64_t>(p.m * p.k) * 2);

    // Per-lane byte offsets; the tile-dependent part is wave-uniform and travels in the scalar offset.
    uint32_t b_off[CG], s_off[CG], z_off[CG];
    // block (inside a tile, or inside a group when scales are loaded per group) whose scale this lane fetches
    const uint32_t lane_blk = kTranspose ? static_cast<uint32_t>((g * 32) >> kBsLog2) : static_cast<uint32_t>(g);
#pragma unroll
    for (int cg = 0; cg < CG; ++cg) {
        const uint32_t col = static_cast<uint32_t>(cg * 16 + c);
        b_off[cg] = col * static_cast<uint32_t>(p.row_bytes) + static_cast<uint32_t>(g * 16);
        s_off[cg] = (col * static_cast<uint32_t>(p.kb) + lane_blk) * static_cast<uint32_t>(sizeof(ST));
        z_off[cg] = col * static_cast<uint32_t>(p.zp_row) + (lane_blk >> 1);
    }
    // compact activation load. MR > 1: row g (+4i), piece c of one tile. MR = 1: piece c of tile g of the group.
    const uint32_t a_off = kGroupA ? static_cast<uint32_t>(g * 256 + c * 16)
                                   : static_cast<uint32_t>(g) * static_cast<uint32_t>(p.k) * 2u + static_cast<uint32_t>(c * 16);
    const uint32_t a_row_step = 4u * static_cast<uint32_t>(p.k) * 2u;
    // LDS: this wave's two staging buffers. MR > 1: written at (row g + 4i, piece c), read at (row c % MR, piece of
    // MFMA j). MR = 1: written at (tile g, piece c), every lane reads the piece of MFMA j of the tile at hand.
    unsigned char* stage = smem + wave * (2 * kStageBytes);
    const uint32_t st_write = kGroupA ? static_cast<uint32_t>(lane * 16) : static_cast<uint32_t>(g * kRowPitch + c * 16);
    const uint32_t st_read = (kGroupA ? 0u : static_cast<uint32_t>((c & (MR - 1)) * kRowPitch)) + static_cast<uint32_t>(kTranspose ? g * 16 : g * 64);
    // v_and_or_b32 may read one scalar operand only: keep the mask in a vector register (an identity DPP move
    // makes it one), the magic in a scalar register.
    const uint32_t mask = __builtin_amdgcn_mov_dpp(p.nibble_mask, 0xE4, 0xf, 0xf, false), magic = p.magic;

    float4_t y[CG];
    float4_t acc[CG];
#pragma unroll
    for (int cg = 0; cg < CG; ++cg) {
        y[cg] = float4_t{0.f, 0.f, 0.f, 0.f};
        acc[cg] = float4_t{0.f, 0.f, 0.f, 0.f};
    }

    const int t_begin = wave * p.tiles_per_wave;
    const int t_end = min(t_begin + p.tiles_per_wave, p.tiles);

    using Grp = Group<U, CG, NA, NS, typename ScaleIo<ST>::raw_t>;
    const uint32_t zp_mask = has_zp ? 0xfu : 0u, zp_default = has_zp ? 0u : 8u;     // branch-free "8 when absent"
    // No branch in here: a tile past the wave's range gets every offset out of range, which fetches nothing and returns
    // zeros - weights 0, scale 0, activations 0, a tile that adds nothing. With branches around the loads the compiler
    // waits for every load in flight at the next use, the prefetch included. All offsets first, then the loads back
    // to back.
    auto fetch_group = [&](Grp& grp, int t0) {
        uint32_t tile_oor[U];
#pragma unroll
        for (int u = 0; u < U; ++u) tile_oor[u] = t0 + u < t_end ? 0u : kOutOfRange;       // or-ed in: out of range
        uint32_t a_voff[NA];
        if constexpr (kGroupA) {
            const bool out = g >= U || t0 + g >= t_end || static_cast<int64_t>(t0 + g) * 128 + c * 8 + 8 > p.k;
            a_voff[0] = out ? kOutOfRange : a_off;
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const bool out = static_cast<int64_t>(t0 + u) * 128 + c * 8 + 8 > p.k || (MR < 4 && g >= MR);
#pragma unroll
                for (int i = 0; i < AR; ++i) a_voff[u * AR + i] = (out ? kOutOfRange : a_off + static_cast<uint32_t>(i) * a_row_step) | tile_oor[u];
            }
        }
        const uint32_t group_oor = (g < U && t0 + g < t_end) ? 0u : kOutOfRange;           // per-group scales: lane group g fetches tile t0 + g's
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int cg = 0; cg < CG; ++cg) grp.w[u][cg] = load16(srd_b, b_off[cg] | tile_oor[u], static_cast<uint32_t>(t0 + u) * 64u);
        if constexpr (kGroupA) {
            grp.a[0] = load16(srd_a, a_voff[0], static_cast<uint32_t>(t0) * 256u);
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int i = 0; i < AR; ++i) grp.a[u * AR + i] = load16(srd_a, a_voff[u * AR + i], static_cast<uint32_t>(t0 + u) * 256u);
        }
        if constexpr (kGroupS) {
            // lane group g fetches scale and zero point of tile t0 + g (t0 is even, so the nibble is g & 1)
#pragma unroll
            for (int cg = 0; cg < CG; ++cg) {
                grp.s[0][cg] = ScaleIo<ST>::load_raw(srd_s, s_off[cg] | group_oor, static_cast<uint32_t>(t0) * static_cast<uint32_t>(sizeof(ST)));
                grp.z[0][cg] = __builtin_amdgcn_raw_buffer_load_b8(srd_z, static_cast<int>(z_off[cg] | group_oor), static_cast<int>(t0 >> 1), 0);
            }
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t blk0 = static_cast<uint32_t>(t0 + u) * kBlocksPerTile;
#pragma unroll
                for (int cg = 0; cg < CG; ++cg) {
                    grp.s[u][cg] = ScaleIo<ST>::load_raw(srd_s, s_off[cg] | tile_oor[u], blk0 * static_cast<uint32_t>(sizeof(ST)));
                    grp.z[u][cg] = __builtin_amdgcn_raw_buffer_load_b8(srd_z, static_cast<int>(z_off[cg] | tile_oor[u]), static_cast<int>(blk0 >> 1), 0);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    auto compute_tile = [&](const Grp& grp, int u, int parity) {
        // activations: compact registers -> LDS -> MFMA operand order
        unsigned char* st = stage + (kGroupA ? parity : (u & 1)) * kStageBytes;
        if constexpr (!kGroupA) {
#pragma unroll
            for (int i = 0; i < AR; ++i)
                if (MR >= 4 || g < MR) *reinterpret_cast<uint4*>(st + st_write + i * 4 * kRowPitch) = grp.a[u * AR + i];
            lds_order();
        }
        uint4 av[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) av[j] = *reinterpret_cast<const uint4*>(st + st_read + (kGroupA ? u * 256 : 0) + (kTranspose ? j * 64 : j * 16));
#pragma unroll
        for (int cg = 0; cg < CG; ++cg) {
            uint4 w = grp.w[u][cg];
            if constexpr (kTranspose) transpose_groups(w);
            const uint32_t wd[4] = {w.x, w.y, w.z, w.w};
            // scale and zero-point nibble this lane fetched: of its own block (BS < 128) or of tile g (BS = 128)
            const uint32_t z_lane = (((static_cast<uint32_t>(grp.z[kGroupS ? 0 : u][cg]) >> ((lane_blk & 1u) * 4u)) & 0xfu) & zp_mask) | zp_default;
            const uint32_t s_lane = static_cast<uint32_t>(grp.s[kGroupS ? 0 : u][cg]);
            uint32_t z_tile = z_lane, s_tile = s_lane;
            if constexpr (kGroupS) {
                z_tile = __shfl(z_lane, c + 16 * u, kWave);
                s_tile = __shfl(s_lane, c + 16 * u, kWave);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                uint32_t z = z_tile, s = s_tile;
                if constexpr (kTranspose) {
                    const int src = c + 16 * (((j * 32) / BS) * (BS / 32));   // a lane whose piece lies in MFMA j's block
                    z = __shfl(z_lane, src, kWave);
                    s = __shfl(s_lane, src, kWave);
                }
                const uint32_t zpair = Magic<BF16>::neg | (z * 0x00010001u);
                const uint4 zc = make_uint4(zpair, zpair, zpair, zpair);
                acc[cg] = mfma16<BF16>(av[j], unpack8(wd[j], mask, magic), acc[cg]);
                acc[cg] = mfma16<BF16>(av[j], zc, acc[cg]);
                if (kTranspose ? (((j + 1) * 32) % BS == 0) : (j == 3)) {
                    const float sf = ScaleIo<ST>::to_f32(s, BF16);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        y[cg][r] = fmaf(sf, acc[cg][r], y[cg][r]);
                        acc[cg][r] = 0.f;
                    }
                }
            }
        }
    };
    auto run_group = [&](const Grp& cur, Grp& next, int t0, int parity, bool prefetch) {
        // nothing of this group moves up into the previous one (its loads are the newest in flight there)
        __builtin_amdgcn_sched_barrier(0);
        if (prefetch) fetch_group(next, t0 + U);
        if constexpr (kGroupA) {
            *reinterpret_cast<uint4*>(stage + parity * kStageBytes + st_write) = cur.a[0];
            lds_order();
        }
#pragma unroll
        for (int u = 0; u < U; ++u) compute_tile(cur, u, parity);        // a tile past the range is all zeros
    };

    Grp ga, gb;
    fetch_group(ga, t_begin);
    int t0 = t_begin;
    for (; t0 + U < t_end; t0 += 2 * U) {                  // whole pairs of groups, no branch inside: every wait counts loads exactly
        run_group(ga, gb, t0, 0, true);
        run_group(gb, ga, t0 + U, 1, true);                // past the end this prefetch fetches nothing
    }
    if (t0 < t_end) run_group(ga, gb, t0, 0, false);       // an odd group out

    // ---- split-K reduction across the waves of this workgroup, in wave order ----
    __syncthreads();                                   // every wave is done with its staging tiles
    float* red = reinterpret_cast<float*>(smem);       // [waves][CG][4][64]
#pragma unroll
    for (int cg = 0; cg < CG; ++cg)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[((wave * CG + cg) * 4 + r) * 64 + lane] = y[cg][r];
    __syncthreads();
    for (int idx = threadIdx.x; idx < CG * 256; idx += blockDim.x) {
        const int cg = idx >> 8;
        const int r = (idx >> 6) & 3;
        const int l = idx & 63;
        const int row = 4 * (l >> 4) + r;
        const int64_t col = n_base + cg * 16 + (l & 15);
        if (row < p.m && col < p.n) {
            float total = 0.f;
            for (int w = 0; w < waves; ++w) total += red[((w * CG + cg) * 4 + r) * 64 + l];
            total = with_bias(total, p.bias, p.bias_dtype, row, p.n, col, p.y_dtype);
            store_from_f32(p.y, p.y_dtype, static_cast<int64_t>(row) * p.n + col, total);
        }
    }
}

template <int CG, int MR> constexpr int group_tiles() { return (CG == 1 && MR <= 4) ? 4 : 2; }

template <bool BF16, int BS, int CG, int MR, typename ST>
static int launch_cfg(const DecodeParams& p, int waves, hipStream_t stream)
{
    const unsigned grid = static_cast<unsigned>((p.n + 16 * CG - 1) / (16 * CG));
    const size_t stage = static_cast<size_t>(waves) * 2 * (MR == 1 ? 1024 : MR * kRowPitch);
    const size_t red = static_cast<size_t>(waves) * CG * 256 * sizeof(float);
    hipLaunchKernelGGL((decode_mfma_kernel<BF16, BS, CG, MR, ST>), dim3(grid), dim3(waves * 64), stage > red ? stage : red, stream, p);
    return static_cast<int>(hipGetLastError());
}

template <bool BF16, int BS, int CG, typename ST>
static int launch_mr(const DecodeParams& p, int waves, hipStream_t stream)
{
    if (p.m <= 1) return launch_cfg<BF16, BS, CG, 1, ST>(p, waves, stream);
    if (p.m <= 4) return launch_cfg<BF16, BS, CG, 4, ST>(p, waves, stream);
    if (p.m <= 8) return launch_cfg<BF16, BS, CG, 8, ST>(p, waves, stream);
    return launch_cfg<BF16, BS, CG, 16, ST>(p, waves, stream);
}

template <bool BF16, typename ST>
static int launch_bs(const DecodeParams& p, int bs, int waves, int cg, hipStream_t stream)
{
    if (cg == 1) {
        switch (bs) {
            case 32: return launch_mr<BF16, 32, 1, ST>(p, waves, stream);
            case 64: return launch_mr<BF16, 64, 1, ST>(p, waves, stream);
            default: return launch_mr<BF16, 128, 1, ST>(p, waves, stream);
        }
    }
    switch (bs) {
        case 32: return launch_mr<BF16, 32, 2, ST>(p, waves, stream);
        case 64: return launch_mr<BF16, 64, 2, ST>(p, waves, stream);
        default: return launch_mr<BF16, 128, 2, ST>(p, waves, stream);
    }
}

}  // namespace mnb

extern "C" int rocm_decode_mfma_eligible(const RocmMatMulNBitsArgs* a)
{
    const bool half_in = a->a_dtype == ROCM_DT_F16 || a->a_dtype == ROCM_DT_BF16;
    const bool scale_ok = a->scale_dtype == a->a_dtype || a->scale_dtype == ROCM_DT_F32;
    const bool bs_ok = a->block_size == 32 || a->block_size == 64 || a->block_size == 128;
    if (!(half_in && scale_ok && bs_ok && a->m >= 1 && a->m <= 16 && a->n >= 1 && a->k % 8 == 0)) return 0;
    // 32-bit offsets inside one workgroup's 32-column window of B, and inside A
    const int64_t kb = (a->k + a->block_size - 1) / a->block_size;
    if (kb * a->block_size / 2 * 32 >= 0x7fffffff || a->m * a->k * 2 >= 0x7ffffff0) return 0;
    return (reinterpret_cast<uintptr_t>(a->a) & 15) == 0 && (reinterpret_cast<uintptr_t>(a->b) & 15) == 0 &&
           (reinterpret_cast<uintptr_t>(a->scales) & 3) == 0;
}

extern "C" int rocm_launch_decode_mfma(const RocmMatMulNBitsArgs* a, int waves, int col_groups, rocm_stream_t stream)
{
    if (!rocm_decode_mfma_eligible(a)) return -1;
    mnb::DecodeParams p;
    p.a = static_cast<const uint16_t*>(a->a);
    p.b = a->b;
    p.scales = a->scales;
    p.zp = a->zp;
    p.bias = a->bias;
    p.y = a->y;
    p.m = a->m;
    p.n = a->n;
    p.k = a->k;
    p.kb = (a->k + a->block_size - 1) / a->block_size;
    p.row_bytes = p.kb * a->block_size / 2;
    p.zp_row = (p.kb + 1) / 2;
    p.tiles = static_cast<int>((a->k + 127) / 128);
    p.bias_dtype = a->bias_dtype;
    p.y_dtype = a->y_dtype;
    p.nibble_mask = 0x000F000Fu;
    p.magic = a->a_dtype == ROCM_DT_BF16 ? mnb::Magic<true>::pos : mnb::Magic<false>::pos;

    int cg = col_groups;
    if (cg != 1 && cg != 2) {
        const int64_t groups = (a->n + 15) / 16;
        cg = (a->m > 8 && groups >= 2048) ? 2 : 1;
    }
    const int group_tiles = (cg == 1 && a->m <= 4) ? 4 : 2;   // U of the kernel: wave ranges are whole groups
    int w = waves;
    if (w <= 0) {
        const int64_t wgs = (a->n + 16 * cg - 1) / (16 * cg);
        const int want = static_cast<int>((8192 + wgs - 1) / wgs);   // waves per workgroup to reach ~8k waves
        int by_work = p.tiles / group_tiles;                          // at least one full group per wave
        if (by_work < 1) by_work = 1;
        w = want < by_work ? want : by_work;
        if (w < 1) w = 1;
    }
    if (w > 8) w = 8;
    const int mr = a->m <= 1 ? 1 : a->m <= 4 ? 4 : a->m <= 8 ? 8 : 16;
    const int lds_cap = 65536 / (2 * (mr == 1 ? 1024 : mr * mnb::kRowPitch));   // staging buffers must fit the default LDS window
    if (w > lds_cap) w = lds_cap;
    int tpw = (p.tiles + w - 1) / w;
    tpw = (tpw + group_tiles - 1) / group_tiles * group_tiles;
    w = (p.tiles + tpw - 1) / tpw;
    p.tiles_per_wave = tpw;

    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool bf16 = a->a_dtype == ROCM_DT_BF16;
    const bool f32_scales = a->scale_dtype == ROCM_DT_F32;
    if (bf16) return f32_scales ? mnb::launch_bs<true, float>(p, a->block_size, w, cg, s) : mnb::launch_bs<true, uint16_t>(p, a->block_size, w, cg, s);
    return f32_scales ? mnb::launch_bs<false, float>(p, a->block_size, w, cg, s) : mnb::launch_bs<false, uint16_t>(p, a->block_size, w, cg, s);
}
