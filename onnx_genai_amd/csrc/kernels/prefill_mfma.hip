// Prefill path of MatMulNBits (M > 16, f16/bf16 activations): Y[M,N] = A[M,K] . dequant(B)[N,K]^T on the matrix cores.
//
// A workgroup of eight waves owns a BM x 128 tile of Y and walks K in steps of 64. Per step it
//   * copies a BM x 64 tile of A from global memory to LDS (16 bytes per lane, rows padded to 144 bytes so that
//     the 32 lanes of an MFMA operand read hit different banks);
//   * reads 128 x 64 packed 4-bit weights (one 8-byte piece = 16 nibbles = one lane), dequantizes them in registers
//     and writes them to LDS as 16-bit floats. f16 with f16 scales: (0x6400|q) is 1024+q, a packed subtract of 1024+zp
//     is exact and one packed multiply by the scale rounds once - the tile is bit-identical to f16((q-zp)*scale).
//     Otherwise (bf16, or f32 scales): (q-zp)*scale in f32, rounded to nearest even;
//   * runs v_mfma_f32_32x32x16 on 4 x 2 waves, each owning a (BM/4) x 64 sub-tile, f32 accumulators. Two waves share
//     a SIMD, so one's LDS and global waits are covered by the other's MFMAs.
// LDS is double buffered: the global loads of step t+1 are in flight while the MFMAs of step t run, and one barrier
// per step separates the two buffers. Edges in M and N are handled by range-checked buffer loads and masked stores.
#include <hip/hip_fp16.h>

#include <type_traits>

#include <cmath>
#include "prefill_common.hiph"

namespace mnb {

// BF16: element type. BM x BN: tile of Y per workgroup (128 x 64, 128 x 128, 256 x 128 or 256 x 256). SF32: scales are stored
// as f32 (otherwise in the activations' 16-bit type). f16 activations with f16 scales dequantize in packed f16,
// everything else in f32.
// DENSE: B is not packed 4-bit weights but a [N, K] matrix of the activations' 16-bit type (weights of another width or with
// g_idx, expanded by a launch of their own): a lane copies its 16-byte pieces to LDS as they are; no scales, no zero points.
template <bool BF16, int BM, int BN, bool SF32, bool DENSE = false>
__global__ __launch_bounds__(512) void prefill_mfma_kernel(PrefillParams p)
{
    static_assert(!DENSE || (BN <= 128 && !SF32), "dense weights: four times the bytes per column, so only the narrower tiles have the registers");
    constexpr bool F32MATH = BF16 || SF32;
    constexpr int WM = BM / 4;             // wave sub-tile rows
    constexpr int WN = BN / 2;             // and columns
    constexpr int TM = WM / 32;            // 32x32 MFMA tiles per wave along M
    constexpr int TN = WN / 32;            // and along N
    constexpr int A_LOADS = BM / 64;       // 16-byte pieces of A per lane per step
    constexpr int B_DW = BN / 64;          // packed dwords of B per lane per step (1, 2 or 4); dense: 16-byte pieces
    constexpr int B_PIECES = 8 / B_DW;     // lanes that share one column's 32 (dense: 128) bytes of a step
    constexpr int B_REGS = DENSE ? 4 * B_DW : B_DW;
    constexpr uint32_t kBStep = DENSE ? 128u : 32u;            // bytes of one column per step
    const uint32_t nib_mask = __builtin_amdgcn_mov_dpp(p.nibble_mask, 0xE4, 0xf, 0xf, false);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char* lds_a = smem;                                   // [2][BM][kPitch]
    unsigned char* lds_b = smem + 2 * BM * kPitch;                 // [2][BN][kPitch]

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave >> 1, wn = wave & 1;      // 4 x 2 waves
    // Column blocks vary fastest: the workgroups running at one time share a few row blocks of A (each XCD's L2 then
    // holds them once) and sweep the small packed B.
    const int64_t m_base = static_cast<int64_t>(blockIdx.y) * BM;
    const int64_t n_base = static_cast<int64_t>(blockIdx.x) * BN;
    const int64_t rows_left = p.m - m_base, cols_left = p.n - n_base;

    const __amdgpu_buffer_rsrc_t srd_a = make_srd(p.a + m_base * p.k, static_cast<uint64_t>(rows_left * p.k) * 2);
    const __amdgpu_buffer_rsrc_t srd_b = make_srd(p.b + n_base * p.row_bytes, static_cast<uint64_t>(cols_left * p.row_bytes));
    constexpr uint32_t kScaleBytes = SF32 ? 4 : 2;
    const __amdgpu_buffer_rsrc_t srd_s = make_srd(static_cast<const unsigned char*>(p.scales) + n_base * p.kb * kScaleBytes,
                                                    static_cast<uint64_t>(cols_left * p.kb) * kScaleBytes);
    const bool has_zp = p.zp != nullptr;
    const uint32_t zp_mask = has_zp ? 0xfu : 0u, zp_default = has_zp ? 0u : 8u;   // branch-free "8 when absent"
    const __amdgpu_buffer_rsrc_t srd_z = make_srd(has_zp ? p.zp + n_base * p.zp_row : p.b, has_zp ? static_cast<uint64_t>(cols_left * p.zp_row) : 0);

    // A: lane -> (row t/8 + 64 i, piece t%8). B: lane -> (column t / B_PIECES, piece t % B_PIECES of the 64-element step).
    const uint32_t a_goff = static_cast<uint32_t>(t >> 3) * static_cast<uint32_t>(p.k) * 2u + static_cast<uint32_t>((t & 7) * 16);
    const uint32_t a_gstep = 64u * static_cast<uint32_t>(p.k) * 2u;
    const uint32_t a_loff = static_cast<uint32_t>((t >> 3) * kPitch + (t & 7) * 16);
    const int bcol = t / B_PIECES, bpiece = t % B_PIECES;
    const uint32_t b_goff = static_cast<uint32_t>(bcol) * static_cast<uint32_t>(p.row_bytes) + static_cast<uint32_t>(bpiece * B_DW * (DENSE ? 16 : 4));
    const uint32_t b_loff = static_cast<uint32_t>(bcol * kPitch + bpiece * B_DW * 16);
    const uint32_t s_goff = static_cast<uint32_t>(bcol) * static_cast<uint32_t>(p.kb) * kScaleBytes;
    const uint32_t z_goff = static_cast<uint32_t>(bcol) * static_cast<uint32_t>(p.zp_row);

    // MFMA operand reads: lane (r = lane % 32, kg = lane / 32) reads 8 consecutive k of row r.
    const uint32_t frag_off = static_cast<uint32_t>((lane & 31) * kPitch + (lane >> 5) * 16);

    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // K range of this workgroup: all of K, or one of grid.z slices whose f32 partial sums a second kernel adds up in
    // slice order (small grids: long K, few tiles of Y).
    const int kt_begin = static_cast<int>(blockIdx.z) * p.steps_per_split;
    const int steps = min(kt_begin + p.steps_per_split, static_cast<int>(p.k / kBK));
    // Global loads run D-1 steps ahead of the MFMAs, in D register sets; step x lives in set x % D from its load
    // (issued while step x-D+1 is being multiplied) to its dequantize-and-store into LDS (while step x-1 is).
    constexpr int D = BN == 256 ? 3 : 4;   // the 256 x 256 tile has no registers left for a fourth set
    struct Regs {
        uint4 a[A_LOADS];
        uint32_t b[B_REGS];
        uint32_t s;      // raw scale bits; converted when the step is dequantized, so that no load is waited for early
        uint32_t z;      // raw zero-point byte
        uint32_t zsh;    // shift of the nibble to take from it
    };
    Regs regs[D];

    auto load_global = [&](Regs& r, int kt) {
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) r.a[i] = load16(srd_a, a_goff + static_cast<uint32_t>(i) * a_gstep, static_cast<uint32_t>(kt) * 128u);
        if constexpr (DENSE) {
#pragma unroll
            for (int i = 0; i < B_DW; ++i) {
                const uint4 bw = load16(srd_b, b_goff + static_cast<uint32_t>(i) * 16u, static_cast<uint32_t>(kt) * kBStep);
                r.b[4 * i] = bw.x;
                r.b[4 * i + 1] = bw.y;
                r.b[4 * i + 2] = bw.z;
                r.b[4 * i + 3] = bw.w;
            }
            r.s = r.z = r.zsh = 0;
            return;
        }
        if constexpr (B_DW == 1) {
            r.b[0] = __builtin_amdgcn_raw_buffer_load_b32(srd_b, static_cast<int>(b_goff), static_cast<int>(kt * 32), 0);
        } else if constexpr (B_DW == 2) {
            const auto bw = __builtin_amdgcn_raw_buffer_load_b64(srd_b, static_cast<int>(b_goff), static_cast<int>(kt * 32), 0);
            r.b[0] = bw[0];
            r.b[1] = bw[1];
        } else {
            const uint4 bw = load16(srd_b, b_goff, static_cast<uint32_t>(kt) * 32u);
            r.b[0] = bw.x;
            r.b[1] = bw.y;
            r.b[2] = bw.z;
            r.b[3] = bw.w;
        }
        const uint32_t blk = static_cast<uint32_t>((kt * kBK + bpiece * B_DW * 8) >> p.bs_log2);
        if constexpr (SF32) r.s = __builtin_amdgcn_raw_buffer_load_b32(srd_s, static_cast<int>(s_goff + blk * 4u), 0, 0);
        else r.s = __builtin_amdgcn_raw_buffer_load_b16(srd_s, static_cast<int>(s_goff + blk * 2u), 0, 0);
        // loaded even without zero points (the empty range then returns 0): a branch here would split the loop body
        const uint32_t zraw = static_cast<uint32_t>(__builtin_amdgcn_raw_buffer_load_b8(srd_z, static_cast<int>(z_goff + (blk >> 1)), 0, 0));
        r.z = zraw;                 // no arithmetic on a loaded value here: it would wait for the load at once
        r.zsh = (blk & 1u) * 4u;
    };
    // Quarter `part` (0..3) of one step's trip from registers to LDS: A pieces part, part+4, ... and one packed dword of
    // B, dequantized (with two dwords per lane: in quarters 0 and 2). Four quarters make a step; they are issued between
    // the MFMA batches of the step before, so that their VALU and LDS-write work runs while the matrix cores are busy.
    auto store_part = [&](const Regs& r, int buf, int part) {
        unsigned char* la = lds_a + buf * (BM * kPitch) + a_loff;
#pragma unroll
        for (int i = part; i < A_LOADS; i += 4) *reinterpret_cast<uint4*>(la + i * 64 * kPitch) = r.a[i];
        if ((B_DW == 2 && (part & 1)) || (B_DW == 1 && part != 0)) return;
        const int dw = B_DW == 4 ? part : (part >> 1);
        unsigned char* lb = lds_b + buf * (BN * kPitch) + b_loff;
        if constexpr (DENSE) {
            *reinterpret_cast<uint4*>(lb + dw * 16) = make_uint4(r.b[4 * dw], r.b[4 * dw + 1], r.b[4 * dw + 2], r.b[4 * dw + 3]);
            return;
        }
        const uint32_t w = r.b[dw];
        const uint32_t zq = ((r.z >> r.zsh) & zp_mask) | zp_default;
        if constexpr (F32MATH) {
            const float sc = SF32 ? __uint_as_float(r.s) : (BF16 ? __uint_as_float(r.s << 16) : f16_bits_to_f32(static_cast<uint16_t>(r.s)));
            *reinterpret_cast<uint4*>(lb + dw * 16) = dequant_dword_f32<BF16>(w, (16u - zq) * 0x01010101u, sc, -16.0f * sc);
        } else {
            const uint32_t w4 = w >> 4;
            uint32_t pr[4];
            pr[0] = magic_pair(w, w4, 0x0c040c00u, nib_mask, p.magic);
            pr[1] = magic_pair(w, w4, 0x0c050c01u, nib_mask, p.magic);
            pr[2] = magic_pair(w, w4, 0x0c060c02u, nib_mask, p.magic);
            pr[3] = magic_pair(w, w4, 0x0c070c03u, nib_mask, p.magic);
            const uint32_t o2 = 0xE400E400u | (zq * 0x00010001u);   // -(1024 + zp) twice, exact in f16
            const uint32_t s2 = r.s * 0x00010001u;                  // the f16 scale twice
#pragma unroll
            for (int i = 0; i < 4; ++i) pr[i] = finish_f16(pr[i], __builtin_bit_cast(half2_t, o2), __builtin_bit_cast(half2_t, s2));
            *reinterpret_cast<uint4*>(lb + dw * 16) = make_uint4(pr[0], pr[1], pr[2], pr[3]);
        }
    };
    auto store_lds = [&](const Regs& r, int buf) {
#pragma unroll
        for (int part = 0; part < 4; ++part) store_part(r, buf, part);
    };
    // MFMAs of one 64-element step out of LDS buffer `buf`; the operand fragments of the next 16 elements are read
    // while these run, and (when asked) the following step moves from registers into the other buffer.
    auto compute = [&](int buf, const Regs& next, bool store_next) {
        const unsigned char* la = lds_a + buf * (BM * kPitch) + wm * (WM * kPitch) + frag_off;
        const unsigned char* lb = lds_b + buf * (BN * kPitch) + wn * (WN * kPitch) + frag_off;
        uint4 fa[2][TM], fb[2][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[0][i] = *reinterpret_cast<const uint4*>(la + i * 32 * kPitch);
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[0][j] = *reinterpret_cast<const uint4*>(lb + j * 32 * kPitch);
#pragma unroll
        for (int kk = 0; kk < kBK / 16; ++kk) {
            const int cur = kk & 1, nxt = cur ^ 1;
            if (kk + 1 < kBK / 16) {
#pragma unroll
                for (int i = 0; i < TM; ++i) fa[nxt][i] = *reinterpret_cast<const uint4*>(la + i * 32 * kPitch + (kk + 1) * 32);
#pragma unroll
                for (int j = 0; j < TN; ++j) fb[nxt][j] = *reinterpret_cast<const uint4*>(lb + j * 32 * kPitch + (kk + 1) * 32);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = mfma32<BF16>(fa[cur][i], fb[cur][j], acc[i][j]);
            if (store_next) store_part(next, buf ^ 1, kk);
        }
    };

    // Every load below is issued unconditionally (past the end of K it reads in-range garbage or range-checked zeros
    // that are never stored): with a fixed number of loads per step the compiler can wait for exactly the step it
    // needs and leave the newer ones in flight.
#pragma unroll
    for (int s0 = 0; s0 < D - 1; ++s0) load_global(regs[s0], kt_begin + s0);
    store_lds(regs[0], kt_begin & 1);
    __syncthreads();
    // Main loop: whole rounds of D steps with no branch inside, so that the wait before each step counts loads
    // exactly and the newer ones stay in flight (a branch would make the compiler drain them all). The last
    // round, which holds the final step, runs with the conditions.
    int kt0 = kt_begin;
    for (; kt0 + D < steps; kt0 += D) {
#pragma unroll
        for (int s0 = 0; s0 < D; ++s0) {
            load_global(regs[(s0 + D - 1) % D], kt0 + s0 + D - 1);
            compute((kt0 + s0) & 1, regs[(s0 + 1) % D], true);
            __syncthreads();
        }
    }
#pragma unroll
    for (int s0 = 0; s0 < D; ++s0) {
        const int kt = kt0 + s0;
        load_global(regs[(s0 + D - 1) % D], kt + D - 1);
        if (kt < steps) {
            compute(kt & 1, regs[(s0 + 1) % D], kt + 1 < steps);
            __syncthreads();
        }
    }

    store_tile<TM, TN>(p, acc, m_base, n_base, wm * WM, wn * WN, lane, wave, smem);
}

// Y = sum over slices of the partial sums, in slice order, plus bias; one thread per element.
__global__ __launch_bounds__(256) void prefill_reduce_kernel(const float* __restrict__ partial, int splits, int64_t m, int64_t n,
                                                             const void* __restrict__ bias, int bias_dtype, void* __restrict__ y, int y_dtype)
{
    const int64_t total = m * n;
    for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total; i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        float sum = 0.f;
        for (int z = 0; z < splits; ++z) sum += partial[z * total + i];
        store_from_f32(y, y_dtype, i, with_bias(sum, bias, bias_dtype, i / n, n, i % n, y_dtype));
    }
}

template <bool BF16, int BM, int BN, bool SF32, bool DENSE = false>
static int launch_prefill(const PrefillParams& p, int splits, hipStream_t stream)
{
    const dim3 grid(static_cast<unsigned>((p.n + BN - 1) / BN), static_cast<unsigned>((p.m + BM - 1) / BM), static_cast<unsigned>(splits));
    const size_t lds = 2 * static_cast<size_t>(BM + BN) * kPitch;
    auto kernel = prefill_mfma_kernel<BF16, BM, BN, SF32, DENSE>;
    if (lds > 65536) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
        if (e != hipSuccess) return static_cast<int>(e);
    }
    hipLaunchKernelGGL(kernel, grid, dim3(512), lds, stream, p);
    return static_cast<int>(hipGetLastError());
}

}  // namespace mnb

extern "C" int rocm_prefill_mfma_eligible(const RocmMatMulNBitsArgs* a)
{
    const bool half_in = a->a_dtype == ROCM_DT_F16 || a->a_dtype == ROCM_DT_BF16;
    const bool bs_ok = a->block_size >= 32;                            // a 16-byte piece must lie inside one block
    const bool scale_ok = a->scale_dtype == a->a_dtype || a->scale_dtype == ROCM_DT_F32;
    if (!(half_in && bs_ok && scale_ok && a->m > 16 && a->n >= 1 && a->k >= 64 && a->k % 64 == 0)) return 0;
    const int64_t kb = (a->k + a->block_size - 1) / a->block_size;
    if (kb * a->block_size / 2 * 128 >= 0x7fffffff || 256 * a->k * 2 >= 0x7fffffff) return 0;   // 32-bit offsets inside one tile
    return (reinterpret_cast<uintptr_t>(a->a) & 15) == 0 && (reinterpret_cast<uintptr_t>(a->b) & 15) == 0;
}

namespace {

struct PrefillPlan {
    int tile;        // 0: 128 x 128, 1: 256 x 128, 2: 256 x 256, 3: 128 x 64
    int splits;      // slices of K (1 = none)
    int steps_per_split;
};

// The largest tile that still gives every CU a workgroup: 256 x 256, then 256 x 128, 128 x 128. If 128 x 128 tiles leave
// CUs idle, K is cut into slices over grid.z (measured at M = 512: 18944 -> 3584 113 us against 134 us with 128 x 64
// tiles in slices; 14336 -> 4096 106 against 111 us); shapes too short for that take 128 x 64 tiles, sliced if they can be.
PrefillPlan plan_prefill(const RocmMatMulNBitsArgs* a, int tile_choice, uint64_t scratch_bytes)
{
    const int steps = static_cast<int>(a->k / 64);
    const int64_t cus = rocm_ffi_compute_units();      // (256 where no device can be asked: the plan of a host without a GPU is the MI355X's)
    const uint64_t per_split = static_cast<uint64_t>(a->m) * static_cast<uint64_t>(a->n) * 4;
    auto workgroups = [&](int tile) {
        const int bm = (tile == 1 || tile == 2) ? 256 : 128;
        const int bn = tile == 2 ? 256 : tile == 3 ? 64 : 128;
        return ((a->m + bm - 1) / bm) * ((a->n + bn - 1) / bn);
    };
    // slices of K that bring a short grid to about 1.5 workgroups per CU: at least 8 steps each, at most 16, and never
    // more than the scratch holds
    auto slices = [&](int tile) {
        const int64_t wgs = workgroups(tile);
        int want = static_cast<int>((cus + cus / 2 + wgs - 1) / wgs);
        if (want > steps / 8) want = steps / 8;
        if (want > 16) want = 16;
        while (want > 1 && static_cast<uint64_t>(want) * per_split > scratch_bytes) --want;
        return want < 1 ? 1 : want;
    };
    PrefillPlan plan;
    plan.splits = 1;
    if (tile_choice >= 1 && tile_choice <= 4) {
        plan.tile = tile_choice == 4 ? 3 : tile_choice - 1;
        plan.splits = slices(plan.tile);
    } else if (a->m >= 256 && workgroups(2) >= cus) {
        plan.tile = 2;
    } else if (a->m >= 256 && workgroups(1) >= cus) {
        plan.tile = 1;
    } else if (workgroups(0) >= cus) {
        plan.tile = 0;
    } else if (a->m >= 512 && workgroups(0) * slices(0) >= cus) {
        plan.tile = 0;                       // few tiles of Y but a long K: 128 x 128 tiles over slices of K (below 512 rows 128 x 64 is ahead)
        plan.splits = slices(0);
    } else {
        plan.tile = 3;
        plan.splits = slices(3);
    }
    // The plan above is the one to beat: a model of the launch looks at the other tiles, whole and over their slices of K,
    // and takes one that it puts 3 % or more ahead. Two things the rule above misses: a long K on a short grid runs
    // better in larger tiles over more slices (18944 -> 3584 at M = 1536: 336 tiles of 128 x 128, one per CU, two rounds,
    // 423 us; 256 x 128 tiles over three slices 300 us), and one round of larger tiles that leaves some CUs idle beats two
    // rounds of smaller ones (4096 -> 14336 at M = 1024: 224 tiles of 256 x 256 152 us, 448 of 256 x 128 177 us) - a workgroup
    // runs faster when fewer of them share the memory system. The model: workgroups go round by round over the CUs (256 where it was fitted); a round
    // costs (steps per slice) x (the tile's time per step: 2.52 / 1.42 / 0.78 us for 256 x 256 / 256 x 128 / 128 x 128 with every
    // CU busy, 0.45 for 128 x 64; two of the small tiles share a CU) x (0.4 + 0.6 x the fraction of CUs busy) + 8 us for the
    // ends of a workgroup, and the reduction adds its bytes at 4 TB/s. Fitted to 160 timings of 60 shapes (K = 3584 ..
    // 28672, M = 128 .. 4096; 9 % rms): among the plans timed per shape its choice is 0.5 % behind the best on average
    // and 15 % at worst; the rule above alone is 13 % and 41 %.
    if (tile_choice <= 0 && a->m >= 256) {
        const bool bf16 = a->a_dtype == ROCM_DT_BF16;
        auto modelled = [&](int tile, int splits) {
            static const double step_us[4] = {0.78, 1.42, 2.52, 0.45};
            const int occ = tile == 3 ? 2 : (tile == 0 && !bf16) ? 2 : 1;                 // workgroups per CU
            const int sps = (steps + splits - 1) / splits;
            const int sl = (steps + sps - 1) / sps;
            const int64_t total = workgroups(tile) * sl, cap = cus * occ;
            const int64_t full = total / cap, rem = total % cap;
            const double work = sps * step_us[tile];
            double t = full * (work * occ + 8.0);
            if (rem > cus) t += work * 2 * (0.4 + 0.6 * rem / (2.0 * cus)) + 8.0;                // (occ = 2: pairs share CUs)
            else if (rem > 0) t += work * (0.4 + 0.6 * rem / static_cast<double>(cus)) + 8.0;
            if (sl > 1) t += sl * static_cast<double>(a->m) * static_cast<double>(a->n) * 4.0 / 4e6 + 3.0;
            return t;
        };
        double best = modelled(plan.tile, plan.splits) * 0.97;
        const PrefillPlan base = plan;
        for (int tile = 0; tile <= 2; ++tile) {            // (128 x 64 only where the rule above chose it: few timings back its figure)
            for (int pass = 0; pass < 2; ++pass) {
                const int sl = pass == 0 ? 1 : slices(tile);
                if ((pass == 1 && sl == 1) || (tile == base.tile && sl == base.splits)) continue;
                const double t = modelled(tile, sl);
                if (t < best) {
                    best = t;
                    plan.tile = tile;
                    plan.splits = sl;
                }
            }
        }
    }
    plan.steps_per_split = (steps + plan.splits - 1) / plan.splits;
    plan.splits = (steps + plan.steps_per_split - 1) / plan.steps_per_split;
    return plan;
}

}  // namespace

extern "C" uint64_t rocm_prefill_mfma_scratch_bytes(const RocmMatMulNBitsArgs* a, int tile_choice)
{
    if (!rocm_prefill_mfma_eligible(a)) return 0;
    const PrefillPlan plan = plan_prefill(a, tile_choice, ~0ull);
    return plan.splits > 1 ? static_cast<uint64_t>(plan.splits) * static_cast<uint64_t>(a->m) * static_cast<uint64_t>(a->n) * 4 : 0;
}

extern "C" int rocm_prefill_mfma_plan(const RocmMatMulNBitsArgs* a, int tile_choice, uint64_t scratch_bytes, int* tile_rows, int* tile_cols, int* slices)
{
    if (!rocm_prefill_mfma_eligible(a)) return -1;
    const PrefillPlan plan = plan_prefill(a, tile_choice, scratch_bytes);
    if (tile_rows) *tile_rows = (plan.tile == 1 || plan.tile == 2) ? 256 : 128;
    if (tile_cols) *tile_cols = plan.tile == 2 ? 256 : plan.tile == 3 ? 64 : 128;
    if (slices) *slices = plan.splits;
    return 0;
}

// The launch of both entry points below. `dense`: a->b is a [N, K] matrix of the activations' 16-bit type instead of packed weights.
static int launch_tiled(const RocmMatMulNBitsArgs* a, bool dense, int tile_choice, void* scratch, uint64_t scratch_bytes, rocm_stream_t stream)
{
    mnb::PrefillParams p;
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
    p.row_bytes = dense ? a->k * 2 : p.kb * a->block_size / 2;
    p.zp_row = (p.kb + 1) / 2;
    p.bs_log2 = __builtin_ctz(static_cast<unsigned>(a->block_size));
    p.scale_dtype = a->scale_dtype;
    p.bias_dtype = a->bias_dtype;
    p.y_dtype = a->y_dtype;
    p.nibble_mask = 0x000F000Fu;
    p.magic = a->a_dtype == ROCM_DT_BF16 ? 0x43004300u : 0x64006400u;
    PrefillPlan plan = plan_prefill(a, tile_choice, scratch ? scratch_bytes : 0);
    if (dense && plan.tile == 2) plan.tile = 1;          // dense weights: no 256 x 256 build (four times the bytes per column in registers)
    p.steps_per_split = plan.steps_per_split;
    p.partial = plan.splits > 1 ? static_cast<float*>(scratch) : nullptr;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool bf16 = a->a_dtype == ROCM_DT_BF16;
    const bool sf32 = a->scale_dtype == ROCM_DT_F32;
    auto go = [&](auto bf, auto sf) {
        constexpr bool B = decltype(bf)::value, S = decltype(sf)::value;
        if (plan.tile == 2) return mnb::launch_prefill<B, 256, 256, S>(p, plan.splits, s);
        if (plan.tile == 1) return mnb::launch_prefill<B, 256, 128, S>(p, plan.splits, s);
        if (plan.tile == 3) return mnb::launch_prefill<B, 128, 64, S>(p, plan.splits, s);
        return mnb::launch_prefill<B, 128, 128, S>(p, plan.splits, s);
    };
    auto go_dense = [&](auto bf) {
        constexpr bool B = decltype(bf)::value;
        if (plan.tile == 1) return mnb::launch_prefill<B, 256, 128, false, true>(p, plan.splits, s);
        if (plan.tile == 3) return mnb::launch_prefill<B, 128, 64, false, true>(p, plan.splits, s);
        return mnb::launch_prefill<B, 128, 128, false, true>(p, plan.splits, s);
    };
    int rc;
    if (dense) rc = bf16 ? go_dense(std::true_type{}) : go_dense(std::false_type{});
    else if (bf16 && sf32) rc = go(std::true_type{}, std::true_type{});
    else if (bf16) rc = go(std::true_type{}, std::false_type{});
    else if (sf32) rc = go(std::false_type{}, std::true_type{});
    else rc = go(std::false_type{}, std::false_type{});
    if (rc != 0 || plan.splits == 1) return rc;
    return rocm_launch_slice_reduce(static_cast<const float*>(scratch), plan.splits, a->m, a->n, a->bias, a->bias_dtype, a->y, a->y_dtype, stream);
}

extern "C" int rocm_launch_prefill_mfma(const RocmMatMulNBitsArgs* a, int tile_choice, void* scratch, uint64_t scratch_bytes, rocm_stream_t stream)
{
    if (!rocm_prefill_mfma_eligible(a)) return -1;
    return launch_tiled(a, false, tile_choice, scratch, scratch_bytes, stream);
}

extern "C" int rocm_prefill_dense16_eligible(const RocmMatMulNBitsArgs* a)
{
    const bool half_in = a->a_dtype == ROCM_DT_F16 || a->a_dtype == ROCM_DT_BF16;
    // From five rows: what this route replaces is a GEMV of one wave per column that reads every row of A per column
    // (8 bits, 3584 -> 18944: 28 us at one row, 306 us at seven; 2 bits, 4096 -> 14336: 115 and 720 us), while expansion and
    // tiled kernel together cost the same at every height up to a few dozen rows (110-115 us and 166-170 us on those two).
    // Up to four rows the 8-bit GEMV with 16-byte loads is the better one.
    if (!(half_in && a->m >= 5 && a->n >= 1 && a->k >= 64 && a->k % 64 == 0)) return 0;
    if (256 * a->k * 2 >= 0x7fffffff) return 0;                                                  // 32-bit offsets inside one tile
    return (reinterpret_cast<uintptr_t>(a->a) & 15) == 0;
}

extern "C" int rocm_launch_prefill_dense16(const RocmMatMulNBitsArgs* a, const void* w16_nk, int tile_choice, void* scratch, uint64_t scratch_bytes, rocm_stream_t stream)
{
    if (!rocm_prefill_dense16_eligible(a) || (reinterpret_cast<uintptr_t>(w16_nk) & 15) != 0) return -1;
    RocmMatMulNBitsArgs d = *a;
    d.b = static_cast<const uint8_t*>(w16_nk);
    d.scales = nullptr;
    d.zp = nullptr;
    d.scale_dtype = a->a_dtype;
    d.block_size = 64;                      // (the planner only reads it through the eligibility of the packed form)
    return launch_tiled(&d, true, tile_choice, scratch, scratch_bytes, stream);
}

extern "C" int rocm_launch_slice_reduce(const float* partial, int slices, int64_t m, int64_t n, const void* bias, int bias_dtype, void* y, int y_dtype,
                                        rocm_stream_t stream)
{
    int64_t blocks = (m * n + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL(mnb::prefill_reduce_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream), partial, slices, m, n,
                       bias, bias_dtype, y, y_dtype);
    return static_cast<int>(hipGetLastError());
}
