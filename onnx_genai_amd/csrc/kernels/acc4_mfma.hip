// accuracy_level = 4 on the int8 matrix cores.
//
// The activations arrive already quantized (see quantize_a_kernel): int8 codes, one f32 scale and
// the sum of codes per (row, block). A 4-bit weight is used as the unsigned int8 0..15; the zero
// point leaves through the code sums:
//     acc[m,n,b] = sum_k code[m,k] * q[n,k]  -  zp[n,b] * sum_k code[m,k]          (exact integers)
//     y[m,n]     = sum_b f32(acc[m,n,b]) * (scale_a[m,b] * scale_b[n,b]) + bias[n]
// Both integer terms stay below 2^24 for every block size up to 256, so the subtraction is done in
// f32 without rounding.
//
// Codes are stored "even/odd interleaved" inside every run of 8: positions 0..3 hold elements
// 0,2,4,6 and positions 4..7 hold 1,3,5,7. That is the order in which `w & 0x0f0f0f0f` and
// `(w >> 4) & 0x0f0f0f0f` deliver the eight weights of one packed dword, so unpacking costs three
// instructions per dword and no byte shuffles.
#include "mfma_common.hiph"

namespace mnb {

typedef __attribute__((ext_vector_type(4))) int int4_t;
typedef __attribute__((ext_vector_type(16))) int int16_t_v;
typedef __attribute__((ext_vector_type(32))) float float32_v;

__device__ __forceinline__ long pack64(uint32_t lo, uint32_t hi)
{
    return static_cast<long>(static_cast<uint64_t>(lo) | (static_cast<uint64_t>(hi) << 32));
}

// ---------------------------------------------------------------------------------------------
// Decode (M <= 16): split-K over the waves of a workgroup, v_mfma_i32_16x16x32_i8.
// ---------------------------------------------------------------------------------------------

struct Acc4DecodeParams {
    const int8_t* qa;       // [M, padded_k] interleaved codes
    const float* aq;        // [M, kb, 2]: scale_a, f32(sum of codes)
    const float* aux16;     // [kb, 16, 2]: the same pairs, block-major, rows beyond M unspecified (M > 1 only)
    const uint8_t* b;
    const void* scales;
    const uint8_t* zp;
    const void* bias;
    void* y;
    int64_t m, n, kb;
    int64_t padded_k;       // kb * BS
    int64_t row_bytes;      // padded_k / 2
    int64_t zp_row;         // ceil(kb / 2)
    int tiles;              // ceil(padded_k / 128)
    int tiles_per_wave;     // multiple of the group size
    int bias_dtype, y_dtype;
    int scales_bf16;        // 16-bit scales are bf16 (else f16)
    int32_t* acc_probe;     // PROBE builds: int32 [M, N, kb] block accumulators, as flushed
};

constexpr int kCodePitch = 144;   // bytes between activation rows of one tile in LDS: 128 + 16

template <int U, int NA, int NS, int NZ>
struct Acc4Group {
    uint4 w[U];
    uint4 a[NA];
    uint32_t s[NS];
    uint32_t z[NZ];
    uint4 x;     // MR = 1: .x/.y = (scale_a, code sum) of block `lane` of the group; MR = 16: 16 bytes of the group's aux16 rows
};

// BS: block size (32, 64, 128). MR: rows staged (1 or 16; M <= MR). ST: storage type of the scales.
//
// Lane (c = lane % 16, g = lane / 16) streams column c in 16-byte pieces, as the float decode kernel does.
// A group is U tiles of 128 elements and NB = U * 128 / BS blocks. Per group a lane issues U weight loads,
// one load of codes (MR = 1) or two per tile (MR = 16), NS scale loads (lane group g fetches block 4i + g),
// NZ zero-point loads (lane group g fetches the byte of blocks 8i + 2g and 8i + 2g + 1) and one load of
// the activation-side pairs; scale and zero point reach the other lane groups by shuffle when a block ends.
// SETS: 2 = the next group's loads are in flight while this one is multiplied (few waves per launch); 1 = no prefetch,
// fewer registers, more waves per SIMD (launches with thousands of waves, where occupancy hides latency better).
// PROBE: every flushed block accumulator (the integer acc - zp * code_sum that is about to be scaled) is also stored to
// p.acc_probe; the same code otherwise, for tests that compare the integers themselves.
template <int BS, int MR, typename ST, int SETS, bool PROBE>
__global__ __launch_bounds__(512) void acc4_decode_kernel(Acc4DecodeParams p)
{
    constexpr bool kTranspose = BS < 128;
    constexpr int NBT = 128 / BS;                       // blocks per tile
    constexpr int U = MR == 1 ? 4 : 2;
    constexpr int NB = U * NBT;                         // blocks per group
    constexpr int NS = (NB + 3) / 4;
    constexpr int NZ = (NB + 7) / 8;
    constexpr int NA = MR == 1 ? 1 : 2 * U;
    constexpr int kCodeStage = MR == 1 ? 1024 : 16 * kCodePitch;   // one staging buffer of codes (a group / a tile)
    constexpr int kAuxStage = MR == 1 ? 0 : 1024;                  // one staging buffer of aux16 rows (a group)
    constexpr int kWaveBytes = 2 * kCodeStage + 2 * kAuxStage;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = blockDim.x >> 6;
    const int c = lane & 15;
    const int g = lane >> 4;
    const int64_t n_base = static_cast<int64_t>(blockIdx.x) * 16;
    const int64_t cols_left = p.n - n_base;
    const bool has_zp = p.zp != nullptr;
    const bool full_k = (p.padded_k & 127) == 0;
    const bool bf16_scales = p.scales_bf16 != 0;

    const __amdgpu_buffer_rsrc_t srd_b = make_srd(p.b + n_base * p.row_bytes, static_cast<uint64_t>(cols_left * p.row_bytes));
    const __amdgpu_buffer_rsrc_t srd_s = make_srd(static_cast<const ST*>(p.scales) + n_base * p.kb, static_cast<uint64_t>(cols_left * p.kb) * sizeof(ST));
    const __amdgpu_buffer_rsrc_t srd_z = make_srd(has_zp ? p.zp + n_base * p.zp_row : p.b, has_zp ? static_cast<uint64_t>(cols_left * p.zp_row) : 0);
    const __amdgpu_buffer_rsrc_t srd_a = make_srd(p.qa, static_cast<uint64_t>(p.m * p.padded_k));
    const __amdgpu_buffer_rsrc_t srd_x = MR == 1 ? make_srd(p.aq, static_cast<uint64_t>(p.kb) * 8) : make_srd(p.aux16, static_cast<uint64_t>(p.kb) * 128);

    const uint32_t b_off = static_cast<uint32_t>(c) * static_cast<uint32_t>(p.row_bytes) + static_cast<uint32_t>(g * 16);
    const uint32_t s_off = (static_cast<uint32_t>(c) * static_cast<uint32_t>(p.kb) + static_cast<uint32_t>(g)) * static_cast<uint32_t>(sizeof(ST));
    const uint32_t z_off = static_cast<uint32_t>(c) * static_cast<uint32_t>(p.zp_row) + static_cast<uint32_t>(g);
    // codes. MR = 1: piece `lane` (16 bytes) of the group's 512. MR = 16: row lane / 8 (+8), piece lane % 8 of a tile.
    const uint32_t a_off = MR == 1 ? static_cast<uint32_t>(lane * 16)
                                   : static_cast<uint32_t>(lane >> 3) * static_cast<uint32_t>(p.padded_k) + static_cast<uint32_t>((lane & 7) * 16);
    unsigned char* stage = smem + wave * kWaveBytes;
    unsigned char* aux_stage = stage + 2 * kCodeStage;
    const uint32_t st_write = MR == 1 ? static_cast<uint32_t>(lane * 16) : static_cast<uint32_t>((lane >> 3) * kCodePitch + (lane & 7) * 16);
    // operand of MFMA j: 8 codes at element j*32 + g*8 of the tile (transposed weights) or g*32 + j*8
    const uint32_t st_read = (MR == 1 ? 0u : static_cast<uint32_t>(c * kCodePitch)) + static_cast<uint32_t>(kTranspose ? g * 8 : g * 32);
    constexpr int kReadStep = kTranspose ? 32 : 8;

    float y[4] = {0.f, 0.f, 0.f, 0.f};
    int4_t acc = {0, 0, 0, 0};

    const int t_begin = wave * p.tiles_per_wave;
    const int t_end = min(t_begin + p.tiles_per_wave, p.tiles);

    using Grp = Acc4Group<U, NA, NS, NZ>;
    auto fetch_group = [&](Grp& grp, int t0) {
        if (t0 >= t_end) return;
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (t0 + u < t_end) grp.w[u] = load16(srd_b, b_off, static_cast<uint32_t>(t0 + u) * 64u);
        if constexpr (MR == 1) {
            // the range check of srd_a ends the row at padded_k; tiles beyond this wave's share are not read
            uint32_t off = a_off;
            if (lane >= U * 8 || t0 + (lane >> 3) >= t_end) off = kOutOfRange;
            grp.a[0] = load16(srd_a, off, static_cast<uint32_t>(t0) * 128u);
            const int blocks = (min(t0 + U, t_end) - t0) * NBT;
            const auto v = __builtin_amdgcn_raw_buffer_load_b64(srd_x, static_cast<int>(lane < blocks ? lane * 8 : kOutOfRange), static_cast<int>(t0 * NBT * 8), 0);
            grp.x.x = v[0];
            grp.x.y = v[1];
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (t0 + u < t_end) {
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
                        uint32_t off = a_off + static_cast<uint32_t>(i * 8) * static_cast<uint32_t>(p.padded_k);
                        if (!full_k && static_cast<int64_t>(t0 + u) * 128 + (lane & 7) * 16 >= p.padded_k) off = kOutOfRange;
                        grp.a[u * 2 + i] = load16(srd_a, off, static_cast<uint32_t>(t0 + u) * 128u);
                    }
                }
            }
            grp.x = load16(srd_x, lane < NB * 8 ? static_cast<uint32_t>(lane * 16) : kOutOfRange, static_cast<uint32_t>(t0 * NBT) * 128u);
        }
#pragma unroll
        for (int i = 0; i < NS; ++i)
            grp.s[i] = ScaleIo<ST>::load(srd_s, (4 * i + g < NB) ? s_off : kOutOfRange, static_cast<uint32_t>(t0 * NBT + 4 * i) * static_cast<uint32_t>(sizeof(ST)));
#pragma unroll
        for (int i = 0; i < NZ; ++i)
            grp.z[i] = has_zp ? static_cast<uint32_t>(__builtin_amdgcn_raw_buffer_load_b8(srd_z, static_cast<int>((8 * i + 2 * g < NB) ? z_off : kOutOfRange),
                                                                                            static_cast<int>((t0 * NBT) / 2 + 4 * i), 0))
                              : 0x88u;
    };

    // End of block `bi` of the group: y += f32(acc - zp * code_sum) * (scale_a * scale_b).
    auto flush = [&](const Grp& grp, int bi, int t0, int parity) {
        if (static_cast<int64_t>(t0) * NBT + bi >= p.kb) return;            // a block beyond K (wave-uniform)
        const uint32_t s_raw = __shfl(grp.s[bi / 4], c + 16 * (bi % 4), kWave);
        const uint32_t z_raw = __shfl(grp.z[bi / 8], c + 16 * ((bi / 2) % 4), kWave);
        const float sb = ScaleIo<ST>::to_f32(s_raw, bf16_scales);
        const float zf = static_cast<float>((z_raw >> ((bi & 1) * 4)) & 0xfu);
        if constexpr (MR == 1) {
            const float sa = __int_as_float(__builtin_amdgcn_readlane(static_cast<int>(grp.x.x), bi));
            const float qs = __int_as_float(__builtin_amdgcn_readlane(static_cast<int>(grp.x.y), bi));
            const float f = fmaf(-zf, qs, static_cast<float>(acc[0]));
            y[0] = fmaf(f, __fmul_rn(sa, sb), y[0]);
            if constexpr (PROBE) {                                          // row 0 sits in lanes 0..15
                if (g == 0 && n_base + c < p.n) p.acc_probe[(n_base + c) * p.kb + static_cast<int64_t>(t0) * NBT + bi] = static_cast<int>(f);
            }
        } else {
            const float4* rows = reinterpret_cast<const float4*>(aux_stage + parity * kAuxStage + bi * 128 + g * 32);
            const float4 r01 = rows[0], r23 = rows[1];
            const float sa[4] = {r01.x, r01.z, r23.x, r23.z};
            const float qs[4] = {r01.y, r01.w, r23.y, r23.w};
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float f = fmaf(-zf, qs[r], static_cast<float>(acc[r]));
                y[r] = fmaf(f, __fmul_rn(sa[r], sb), y[r]);
                if constexpr (PROBE) {
                    const int64_t row = 4 * g + r;
                    if (row < p.m && n_base + c < p.n) p.acc_probe[(row * p.n + n_base + c) * p.kb + static_cast<int64_t>(t0) * NBT + bi] = static_cast<int>(f);
                }
            }
        }
    };

    auto compute_tile = [&](const Grp& grp, int u, int t0, int parity) {
        unsigned char* st = stage + (MR == 1 ? parity : (u & 1)) * kCodeStage;
        if constexpr (MR != 1) {
#pragma unroll
            for (int i = 0; i < 2; ++i) *reinterpret_cast<uint4*>(st + st_write + i * 8 * kCodePitch) = grp.a[u * 2 + i];
            lds_order();
        }
        long av[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) av[j] = *reinterpret_cast<const long*>(st + st_read + (MR == 1 ? u * 128 : 0) + j * kReadStep);
        uint4 w = grp.w[u];
        if constexpr (kTranspose) transpose_groups(w);
        const uint32_t wd[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool first = kTranspose ? ((j * 32) % BS == 0) : (j == 0);
            const bool last = kTranspose ? (((j + 1) * 32) % BS == 0) : (j == 3);
            const long bw = pack64(wd[j] & 0x0f0f0f0fu, (wd[j] >> 4) & 0x0f0f0f0fu);
            const int4_t zero = {0, 0, 0, 0};
            acc = __builtin_amdgcn_mfma_i32_16x16x32_i8(av[j], bw, first ? zero : acc, 0, 0, 0);
            if (last) flush(grp, u * NBT + (kTranspose ? (j * 32) / BS : 0), t0, parity);
        }
    };
    auto run_group = [&](const Grp& cur, Grp& next, int t0, int parity) {
        fetch_group(next, t0 + U);
        if constexpr (MR == 1) {
            *reinterpret_cast<uint4*>(stage + parity * kCodeStage + st_write) = cur.a[0];
        } else {
            *reinterpret_cast<uint4*>(aux_stage + parity * kAuxStage + lane * 16) = cur.x;
        }
        lds_order();
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (t0 + u < t_end) compute_tile(cur, u, t0, parity);
    };

    if constexpr (SETS == 2) {
        Grp ga, gb;
        fetch_group(ga, t_begin);
        for (int t0 = t_begin; t0 < t_end; t0 += 2 * U) {
            run_group(ga, gb, t0, 0);
            if (t0 + U < t_end) run_group(gb, ga, t0 + U, 1);
        }
    } else {
        Grp ga;
        for (int t0 = t_begin; t0 < t_end; t0 += U) {
            fetch_group(ga, t0);
            if constexpr (MR == 1) {
                *reinterpret_cast<uint4*>(stage + st_write) = ga.a[0];
            } else {
                *reinterpret_cast<uint4*>(aux_stage + lane * 16) = ga.x;
            }
            lds_order();
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (t0 + u < t_end) compute_tile(ga, u, t0, 0);
        }
    }

    // ---- split-K reduction across the waves of this workgroup, in wave order ----
    __syncthreads();
    float* red = reinterpret_cast<float*>(smem);       // [waves][4][64]
#pragma unroll
    for (int r = 0; r < 4; ++r) red[(wave * 4 + r) * 64 + lane] = y[r];
    __syncthreads();
    for (int idx = threadIdx.x; idx < 256; idx += blockDim.x) {
        const int r = idx >> 6;
        const int l = idx & 63;
        const int row = 4 * (l >> 4) + r;
        const int64_t col = n_base + (l & 15);
        if (row < p.m && col < p.n) {
            float total = 0.f;
            for (int w = 0; w < waves; ++w) total += red[(w * 4 + r) * 64 + l];
            total = with_bias(total, p.bias, p.bias_dtype, row, p.n, col, p.y_dtype);
            store_from_f32(p.y, p.y_dtype, static_cast<int64_t>(row) * p.n + col, total);
        }
    }
}

template <int BS, int MR, typename ST, int SETS>
static int launch_acc4_decode(const Acc4DecodeParams& p, int waves, hipStream_t stream)
{
    const unsigned grid = static_cast<unsigned>((p.n + 15) / 16);
    const size_t stage = static_cast<size_t>(waves) * (MR == 1 ? 2048 : 2 * 16 * kCodePitch + 2048);
    const size_t red = static_cast<size_t>(waves) * 1024;
    if (p.acc_probe) hipLaunchKernelGGL((acc4_decode_kernel<BS, MR, ST, SETS, true>), dim3(grid), dim3(waves * 64), stage > red ? stage : red, stream, p);
    else hipLaunchKernelGGL((acc4_decode_kernel<BS, MR, ST, SETS, false>), dim3(grid), dim3(waves * 64), stage > red ? stage : red, stream, p);
    return static_cast<int>(hipGetLastError());
}

template <int BS, typename ST>
static int launch_acc4_decode_mr(const Acc4DecodeParams& p, int waves, bool single_set, hipStream_t stream)
{
    if (p.m <= 1) return single_set ? launch_acc4_decode<BS, 1, ST, 1>(p, waves, stream) : launch_acc4_decode<BS, 1, ST, 2>(p, waves, stream);
    return launch_acc4_decode<BS, 16, ST, 2>(p, waves, stream);
}

template <typename ST>
static int launch_acc4_decode_bs(const Acc4DecodeParams& p, int bs, int waves, bool single_set, hipStream_t stream)
{
    switch (bs) {
        case 32: return launch_acc4_decode_mr<32, ST>(p, waves, single_set, stream);
        case 64: return launch_acc4_decode_mr<64, ST>(p, waves, single_set, stream);
        default: return launch_acc4_decode_mr<128, ST>(p, waves, single_set, stream);
    }
}

// ---------------------------------------------------------------------------------------------
// Prefill (M > 16): 128 x 128 tiles of Y, K in steps of 64 codes, v_mfma_i32_32x32x32_i8.
// ---------------------------------------------------------------------------------------------
//
// Per step a workgroup of eight waves copies 128 x 64 activation codes to LDS and unpacks 128 x 64 weights into
// signed int8 (q - zp) beside them: with c = 0x80 - zp in every byte, (q + c) ^ 0x80 is q - zp in two's
// complement and no byte ever borrows from its neighbour. The zero point therefore costs two instructions per
// four weights here instead of one per accumulator. When a
// block ends, every int32 accumulator is converted, scaled by scale_a[row] * scale_b[column] and added to the
// f32 result: three VALU instructions per accumulator per block, which - not the matrix cores - bound this kernel.
// Activation scales come block-major ([kb, M]) so that a step's 128 of them are one contiguous run.

struct Acc4PrefillParams {
    const int8_t* qa;       // [M, padded_k] interleaved codes
    const float* sa_t;      // [kb, M] activation scales, block-major
    const uint8_t* b;
    const void* scales;
    const uint8_t* zp;
    const void* bias;
    void* y;
    int64_t m, n, kb;
    int64_t padded_k, row_bytes, zp_row;
    int bs_log2;
    int scales_bf16;
    int bias_dtype, y_dtype;
    int steps_per_slice;    // K steps per grid.z slice (a whole number of blocks); all steps when there is one slice
    float* partial;         // [slices, M, N] f32 partial sums when K is cut into slices, else NULL
    int32_t* acc_probe;     // PROBE builds: int32 [M, N, kb] block accumulators, as flushed
};

constexpr int kTile = 128;           // rows and columns of Y per workgroup
constexpr int kStep = 64;            // codes of K per step
constexpr int kPitch8 = 80;          // bytes per LDS row: 64 codes + 16 of padding (16 rows then cover all 64 banks)

// NBS: blocks per step - 2 (block size 32), 1 (block size 64) or 0 (block size >= 128: a block spans several steps).
// SF32: scales stored as f32 (else 16 bits, f16 or bf16 by a run-time flag).
// Eight waves, 4 (rows) x 2 (columns); each owns a 32 x 64 sub-tile: two MFMA tiles, 32 f32 results per lane. The
// small per-wave state leaves room for four waves per SIMD, which is what overlaps one wave's flush arithmetic
// with another's MFMAs.
// PROBE: every int32 tile that is flushed is also stored to p.acc_probe ([M, N, kb]); the same code otherwise.
template <int NBS, bool SF32, int D, bool PROBE>
__global__ __launch_bounds__(512) void acc4_prefill_kernel(Acc4PrefillParams p)
{
    constexpr int kSlots = NBS == 2 ? 2 : 1;                   // scale slots per step
    constexpr int kBufBytes = 2 * kTile * kPitch8 + 2 * kSlots * kTile * 4;
    constexpr int TN = 2;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int64_t m_base = static_cast<int64_t>(blockIdx.y) * kTile;
    const int64_t n_base = static_cast<int64_t>(blockIdx.x) * kTile;
    const int64_t rows_left = p.m - m_base, cols_left = p.n - n_base;
    const bool has_zp = p.zp != nullptr;
    const bool ragged_k = (p.padded_k & 63) != 0;
    constexpr uint32_t kScaleBytes = SF32 ? 4 : 2;

    const __amdgpu_buffer_rsrc_t srd_a = make_srd(p.qa + m_base * p.padded_k, static_cast<uint64_t>(rows_left * p.padded_k));
    const __amdgpu_buffer_rsrc_t srd_b = make_srd(p.b + n_base * p.row_bytes, static_cast<uint64_t>(cols_left * p.row_bytes));
    const __amdgpu_buffer_rsrc_t srd_s = make_srd(static_cast<const unsigned char*>(p.scales) + n_base * p.kb * kScaleBytes,
                                                  static_cast<uint64_t>(cols_left * p.kb) * kScaleBytes);
    const uint32_t zp_mask = has_zp ? 0xfu : 0u, zp_default = has_zp ? 0u : 8u;   // branch-free "8 when absent"
    const __amdgpu_buffer_rsrc_t srd_z = make_srd(has_zp ? p.zp + n_base * p.zp_row : p.b, has_zp ? static_cast<uint64_t>(cols_left * p.zp_row) : 0);
    const __amdgpu_buffer_rsrc_t srd_sa = make_srd(p.sa_t, static_cast<uint64_t>(p.kb * p.m) * 4);

    // codes: thread -> (row t/4, 16-byte piece t%4). weights: thread -> (column t/4, 8-byte quarter t%4 of the step).
    const int prow = t >> 2, quarter = t & 3;
    const uint32_t a_goff = static_cast<uint32_t>(prow) * static_cast<uint32_t>(p.padded_k) + static_cast<uint32_t>(quarter * 16);
    const uint32_t a_loff = static_cast<uint32_t>(prow * kPitch8 + quarter * 16);
    const uint32_t b_goff = static_cast<uint32_t>(prow) * static_cast<uint32_t>(p.row_bytes) + static_cast<uint32_t>(quarter * 8);
    const uint32_t b_loff = static_cast<uint32_t>(kTile * kPitch8 + prow * kPitch8 + quarter * 16);
    const uint32_t s_goff = static_cast<uint32_t>(prow) * static_cast<uint32_t>(p.kb) * kScaleBytes;
    const uint32_t z_goff = static_cast<uint32_t>(prow) * static_cast<uint32_t>(p.zp_row);
    // activation scales: thread -> (slot t/128, row t%128)
    const int sa_slot = t >> 7, sa_row = t & 127;
    const uint32_t sa_goff = (sa_slot < kSlots && m_base + sa_row < p.m) ? static_cast<uint32_t>(m_base + sa_row) * 4u : kOutOfRange;
    constexpr int kSaOff = 2 * kTile * kPitch8;                 // [kSlots][128] f32 activation scales of the step
    constexpr int kSbOff = kSaOff + kSlots * kTile * 4;         // [kSlots][128] f32 weight scales of the step

    // PROBE: this lane's first accumulator element, (row m_base + wm * 32 + 4 (lane / 32), column n_base + wn * 64 + lane % 32),
    // as a byte offset into the [M, N, kb] probe (the launcher refuses probes of 2^31 bytes or more)
    const int64_t probe_row = m_base + wm * 32 + (lane >> 5) * 4;
    const uint32_t probe_voff = PROBE ? static_cast<uint32_t>((probe_row * p.n + n_base + wn * 64 + (lane & 31)) * p.kb) * 4u : 0u;
    const __amdgpu_buffer_rsrc_t srd_probe = make_srd(PROBE ? p.acc_probe : nullptr, PROBE ? static_cast<uint64_t>(p.m * p.n * p.kb) * 4 : 0);

    // MFMA operand reads: lane (r = lane % 32, h = lane / 32) reads 16 consecutive codes of row r.
    const uint32_t frag_off = static_cast<uint32_t>((lane & 31) * kPitch8 + (lane >> 5) * 16);

    int16_t_v acc[NBS == 0 ? TN : 1];   // integer accumulators that outlive a step (block size >= 128 only)
    float y[TN][16];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) y[j][r] = 0.f;

    // K range of this workgroup: all of K, or one of grid.z slices whose f32 partial sums a second kernel adds in slice
    // order (small grids: few tiles of Y, long K). `kt` below counts steps from the slice's first.
    const int kt_base = static_cast<int>(blockIdx.z) * p.steps_per_slice;
    const int steps = min(static_cast<int>((p.padded_k + kStep - 1) / kStep) - kt_base, p.steps_per_slice);
    // Global loads run D-1 steps ahead of the MFMAs, in D register sets (D = 2 or 4; the launcher chooses). Two sets
    // keep the kernel within 128 registers, so that two workgroups share a CU: better on grids that fill the GPU twice
    // over (measured +2 to +8 %). A grid with at most one workgroup per CU gains nothing from that and runs its lone
    // workgroup 30 % faster with four sets in flight; so does block size 32, whose steps hold two flushes.
    struct Regs {
        uint4 a;
        uint2 b;
        uint32_t s, z, zsh, sa;
    };
    Regs regs[D];

    auto block_of = [&](int kt, int offset) -> uint32_t { return static_cast<uint32_t>((kt * kStep + offset) >> p.bs_log2); };
    auto load_global = [&](Regs& r, int kt_in_slice) {
        const int kt = kt_base + kt_in_slice;
        uint32_t off = a_goff;
        if (ragged_k && static_cast<int64_t>(kt) * kStep + quarter * 16 >= p.padded_k) off = kOutOfRange;   // else the next row's codes
        r.a = load16(srd_a, off, static_cast<uint32_t>(kt) * 64u);
        const auto w = __builtin_amdgcn_raw_buffer_load_b64(srd_b, static_cast<int>(b_goff), static_cast<int>(kt * 32), 0);
        r.b = make_uint2(w[0], w[1]);
        const uint32_t blk = block_of(kt, quarter * 16);
        if constexpr (SF32) r.s = __builtin_amdgcn_raw_buffer_load_b32(srd_s, static_cast<int>(s_goff + blk * 4u), 0, 0);
        else r.s = __builtin_amdgcn_raw_buffer_load_b16(srd_s, static_cast<int>(s_goff + blk * 2u), 0, 0);
        // loaded even without zero points (the empty range then returns 0): a branch here would split the loop body
        const uint32_t zraw = static_cast<uint32_t>(__builtin_amdgcn_raw_buffer_load_b8(srd_z, static_cast<int>(z_goff + (blk >> 1)), 0, 0));
        r.z = zraw;                 // no arithmetic on a loaded value here: it would wait for the load at once
        r.zsh = (blk & 1u) * 4u;
        // The block depends on the thread's slot, so it belongs in the vector offset (an out-of-range sa_goff stays out
        // of range: kb * m * 4 < 2^31): as a scalar offset the compiler loops over its distinct values. With one block
        // per step that loop is kept on purpose: it splits the step into two scheduling regions, and the schedule the
        // compiler finds for the whole step in one region needs 203 registers instead of 126 with two register sets
        // (one workgroup per CU instead of two, 20 % slower) and spills with four.
        const uint32_t sa_block = block_of(kt, sa_slot * 32) * static_cast<uint32_t>(p.m) * 4u;
        if constexpr (NBS == 1) r.sa = __builtin_amdgcn_raw_buffer_load_b32(srd_sa, static_cast<int>(sa_goff), static_cast<int>(sa_block), 0);
        else r.sa = __builtin_amdgcn_raw_buffer_load_b32(srd_sa, static_cast<int>(sa_goff + sa_block), 0, 0);
    };
    // Half `part` of a step's trip from registers into LDS buffer `buf`.
    auto store_part = [&](const Regs& r, int buf, int part) {
        unsigned char* base = smem + buf * kBufBytes;
        const uint32_t w = part == 0 ? r.b.x : r.b.y;
        const uint32_t zq = ((r.z >> r.zsh) & zp_mask) | zp_default;
        const uint32_t c4 = 0x80808080u - zq * 0x01010101u;
        const uint32_t lo = ((w & 0x0f0f0f0fu) + c4) ^ 0x80808080u;            // elements 0,2,4,6 of the dword, minus zp
        const uint32_t hi = (((w >> 4) & 0x0f0f0f0fu) + c4) ^ 0x80808080u;     // elements 1,3,5,7
        *reinterpret_cast<uint2*>(base + b_loff + part * 8) = make_uint2(lo, hi);
        if (part == 0) {
            *reinterpret_cast<uint4*>(base + a_loff) = r.a;
        } else {
            if ((quarter & 1) == 0 && (quarter >> 1) < kSlots) {
                const float sc = SF32 ? __uint_as_float(r.s) : (p.scales_bf16 ? __uint_as_float(r.s << 16) : f16_bits_to_f32(static_cast<uint16_t>(r.s)));
                *reinterpret_cast<float*>(base + kSbOff + ((quarter >> 1) * kTile + prow) * 4) = sc;
            }
            if (sa_slot < kSlots) *reinterpret_cast<uint32_t*>(base + kSaOff + t * 4) = r.sa;
        }
    };
    // The products scale_a[row] * scale_b[column] of the wave's two 32x32 tiles for the block in scale slot `slot`,
    // as one outer-product MFMA (two blocks of 32x32x1: lanes 0..31 carry tile 0's columns, lanes 32..63 tile 1's; both
    // halves carry the wave's 32 rows). Its result has the accumulators' layout, tile j in components 16 j .. 16 j + 15.
    // The matrix cores are mostly idle in this kernel and the vector ALUs are not: this takes one multiply per
    // accumulator and block off them.
    auto scale_tiles = [&](int buf, int slot) -> float32_v {
        const unsigned char* base = smem + buf * kBufBytes;
        const float sa = *reinterpret_cast<const float*>(base + kSaOff + (slot * kTile + wm * 32 + (lane & 31)) * 4);
        const float sb = *reinterpret_cast<const float*>(base + kSbOff + (slot * kTile + wn * 64 + lane) * 4);
        const float32_v zero = {};
        return __builtin_amdgcn_mfma_f32_32x32x1f32(sa, sb, zero, 0, 0, 0);
    };
    // y[j] += f32(tile) * (scale_a[row] * scale_b[column]) for 32x32 tile j.
    auto flush_tile = [&](const int16_t_v& tile, const float32_v& sc, int j) {
#pragma unroll
        for (int i = 0; i < 16; ++i) y[j][i] = fmaf(static_cast<float>(tile[i]), sc[j * 16 + i], y[j][i]);
    };
    // PROBE: the finished int32 tile j of block `blk`, stored before its scale products are formed (fewer registers live
    // than at the flush itself; the integers are final once the block's last MFMA has written them).
    auto probe_tile = [&](const int16_t_v& tile, int j, int64_t blk) {
        if constexpr (PROBE) {
            // lane l holds column l % 32 and rows 8 q + 4 (l / 32) + r of the 32 x 32 tile in component 4 q + r. One vector
            // offset per lane (its first row, tile 0's column), everything else in the scalar offset; a row or column past
            // the matrix gets an offset beyond the buffer's range, which stores nothing.
            const bool col_ok = n_base + wn * 64 + j * 32 + (lane & 31) < p.n && blk < p.kb;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int rowoff = (i >> 2) * 8 + (i & 3);
                const bool ok = col_ok && probe_row + rowoff < p.m;
                const uint32_t soff = static_cast<uint32_t>((static_cast<int64_t>(rowoff) * p.n + j * 32) * p.kb + blk) * 4u;
                __builtin_amdgcn_raw_buffer_store_b32(tile[i], srd_probe, static_cast<int>(ok ? probe_voff : kOutOfRange), static_cast<int>(soff), 0);
            }
        }
    };
    auto mfma = [](const u32x4_t& a, const u32x4_t& b, const int16_t_v& c) {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(int4_t, a), __builtin_bit_cast(int4_t, b), c, 0, 0, 0);
    };
    auto compute = [&](int buf, int kt_in_slice, const Regs& next, bool store_next) {
        const int kt = kt_base + kt_in_slice;
        const unsigned char* la = smem + buf * kBufBytes + wm * (32 * kPitch8) + frag_off;
        const unsigned char* lb = smem + buf * kBufBytes + kTile * kPitch8 + wn * (64 * kPitch8) + frag_off;
        u32x4_t fa[2], fb[2][TN];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            fa[kk] = *reinterpret_cast<const u32x4_t*>(la + kk * 32);
#pragma unroll
            for (int j = 0; j < TN; ++j) fb[kk][j] = *reinterpret_cast<const u32x4_t*>(lb + j * 32 * kPitch8 + kk * 32);
        }
        const int16_t_v zero = {};
        if constexpr (NBS == 1) {
            // One block per step: the integer accumulators live only from the MFMAs to the flush.
            int16_t_v t0 = mfma(fa[0], fb[0][0], zero);
            int16_t_v t1 = mfma(fa[0], fb[0][1], zero);
            t0 = mfma(fa[1], fb[1][0], t0);
            t1 = mfma(fa[1], fb[1][1], t1);
            probe_tile(t0, 0, kt);
            probe_tile(t1, 1, kt);
            const float32_v sc = scale_tiles(buf, 0);
            if (store_next) store_part(next, buf ^ 1, 0);
            flush_tile(t0, sc, 0);
            if (store_next) store_part(next, buf ^ 1, 1);
            flush_tile(t1, sc, 1);
        } else if constexpr (NBS == 2) {
            const bool second = static_cast<int64_t>(kt) * 2 + 1 < p.kb;   // the step's second block exists
            const int16_t_v t0 = mfma(fa[0], fb[0][0], zero);
            const int16_t_v t1 = mfma(fa[0], fb[0][1], zero);
            const int16_t_v u0 = mfma(fa[1], fb[1][0], zero);
            const int16_t_v u1 = mfma(fa[1], fb[1][1], zero);
            probe_tile(t0, 0, 2 * static_cast<int64_t>(kt));
            probe_tile(t1, 1, 2 * static_cast<int64_t>(kt));
            probe_tile(u0, 0, 2 * static_cast<int64_t>(kt) + 1);           // (a second block past K is not stored: blk < kb)
            probe_tile(u1, 1, 2 * static_cast<int64_t>(kt) + 1);
            const float32_v sc0 = scale_tiles(buf, 0);
            const float32_v sc1 = scale_tiles(buf, 1);
            if (store_next) store_part(next, buf ^ 1, 0);
            flush_tile(t0, sc0, 0);
            flush_tile(t1, sc0, 1);
            if (store_next) store_part(next, buf ^ 1, 1);
            if (second) {
                flush_tile(u0, sc1, 0);
                flush_tile(u1, sc1, 1);
            }
        } else {
            // Block size >= 128: the step opens and / or closes a block (wave-uniform).
            const bool opens = ((kt * kStep) & ((1 << p.bs_log2) - 1)) == 0;
            const bool closes = (((kt + 1) * kStep) & ((1 << p.bs_log2) - 1)) == 0;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if (opens) acc[j] = mfma(fa[0], fb[0][j], zero);
                else acc[j] = mfma(fa[0], fb[0][j], acc[j]);
                acc[j] = mfma(fa[1], fb[1][j], acc[j]);
                if (store_next) store_part(next, buf ^ 1, j);
            }
            if (closes) {
#pragma unroll
                for (int j = 0; j < TN; ++j) probe_tile(acc[j], j, (static_cast<int64_t>(kt) * kStep) >> p.bs_log2);
                const float32_v sc = scale_tiles(buf, 0);
#pragma unroll
                for (int j = 0; j < TN; ++j) flush_tile(acc[j], sc, j);
            }
        }
    };

    // Every load is issued unconditionally (past the end of K it reads in-range garbage or range-checked zeros that
    // are never stored): with a fixed number of loads per step the compiler can wait for exactly the step it needs.
#pragma unroll
    for (int s0 = 0; s0 < D - 1; ++s0) load_global(regs[s0], s0);
    store_part(regs[0], 0, 0);
    store_part(regs[0], 0, 1);
    __syncthreads();
    // Main loop: whole rounds of D steps with no branch on the step count inside, so that the wait before each
    // step counts loads exactly and the newer ones stay in flight. The last round runs with the conditions.
    int kt0 = 0;
    for (; kt0 + D < steps; kt0 += D) {
#pragma unroll
        for (int s0 = 0; s0 < D; ++s0) {
            load_global(regs[(s0 + D - 1) % D], kt0 + s0 + D - 1);
            compute(s0 & 1, kt0 + s0, regs[(s0 + 1) % D], true);
            __syncthreads();
        }
    }
#pragma unroll
    for (int s0 = 0; s0 < D; ++s0) {
        const int kt = kt0 + s0;
        load_global(regs[(s0 + D - 1) % D], kt + D - 1);
        if (kt < steps) {
            compute(s0 & 1, kt, regs[(s0 + 1) % D], kt + 1 < steps);
            __syncthreads();
        }
    }

    // Epilogue. A 32x32 accumulator holds, in lane l, column l % 32 and rows 8 q + 4 (l / 32) + r (q, r = 0..3).
    const int col_in_tile = lane & 31;
    const int row_group = (lane >> 5) * 4;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int64_t col = n_base + wn * 64 + j * 32 + col_in_tile;
        if (col >= p.n) continue;
        const void* bias_ptr = p.partial ? nullptr : p.bias;                                   // slices: the reduce kernel adds it
        const bool per_row = (p.bias_dtype & ROCM_BIAS_PER_ROW) != 0;
        const BiasTerm bias = load_bias(bias_ptr, p.bias_dtype, 0, p.n, col);
        float* part = p.partial ? p.partial + static_cast<int64_t>(blockIdx.z) * p.m * p.n : nullptr;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int64_t row = m_base + wm * 32 + q * 8 + row_group + r;
                if (row >= p.m) continue;
                if (part) part[row * p.n + col] = y[j][q * 4 + r];
                else store_from_f32(p.y, p.y_dtype, row * p.n + col, add_bias(y[j][q * 4 + r], per_row ? load_bias(bias_ptr, p.bias_dtype, row, p.n, col) : bias, p.y_dtype));
            }
        }
    }
}

// Slices of K for a grid that leaves CUs idle. Two workgroups of the two-set variant share a CU, so up to 512 run at
// once (block size 32 keeps four register sets: one workgroup per CU, 256 at once): slices bring the grid to at most
// that, with at least 8 steps each, a whole number of blocks per slice, at most 8.
static int acc4_prefill_slices(int64_t m, int64_t n, int64_t padded_k, int block_size)
{
    const int64_t tiles = ((n + kTile - 1) / kTile) * ((m + kTile - 1) / kTile);
    const int64_t steps = (padded_k + kStep - 1) / kStep;
    const int64_t cus = rocm_ffi_compute_units();
    const int64_t resident = block_size < 64 ? cus : 2 * cus;
    // Two slices pay at block size 32 (4096 -> 14336, 17..128 rows: 70-78 -> 44-56 us) and not from 64 up, where they
    // fill the second workgroup slot of each CU (8192 -> 28672 at block 64, 64 / 128 rows: 112 -> 120 us, 123 -> 137 us).
    if (tiles > (block_size < 64 ? resident / 2 : resident / 3)) return 1;
    int64_t want = resident / tiles;
    if (want > 8) want = 8;
    if (want > steps / 8) want = steps / 8;
    return want < 2 ? 1 : static_cast<int>(want);
}

static int acc4_steps_per_slice(int64_t padded_k, int block_size, int slices)
{
    const int64_t steps = (padded_k + kStep - 1) / kStep;
    const int64_t unit = block_size > kStep ? block_size / kStep : 1;            // steps per block
    int64_t per = (steps + slices - 1) / slices;
    per = (per + unit - 1) / unit * unit;
    return static_cast<int>(per);
}

template <int NBS, bool SF32>
static int launch_acc4_prefill(const Acc4PrefillParams& p, int slices, hipStream_t stream)
{
    const dim3 grid(static_cast<unsigned>((p.n + kTile - 1) / kTile), static_cast<unsigned>((p.m + kTile - 1) / kTile), static_cast<unsigned>(slices));
    const size_t lds = 2 * (2 * kTile * kPitch8 + 2 * (NBS == 2 ? 2 : 1) * kTile * 4);
    const bool deep = NBS == 2 || static_cast<uint64_t>(grid.x) * grid.y * grid.z <= static_cast<uint64_t>(rocm_ffi_compute_units());    // at most one workgroup per CU anyway
    if (p.acc_probe) {
        // (block size 32 with four register sets in flight has no room left for the probe's stores: its probe build keeps two -
        // the depth of the load pipeline changes when a step's operands arrive, not what is computed from them)
        if constexpr (NBS == 2) {
            hipLaunchKernelGGL((acc4_prefill_kernel<NBS, SF32, 2, true>), grid, dim3(512), lds, stream, p);
        } else {
            if (deep) hipLaunchKernelGGL((acc4_prefill_kernel<NBS, SF32, 4, true>), grid, dim3(512), lds, stream, p);
            else hipLaunchKernelGGL((acc4_prefill_kernel<NBS, SF32, 2, true>), grid, dim3(512), lds, stream, p);
        }
    } else if (deep) hipLaunchKernelGGL((acc4_prefill_kernel<NBS, SF32, 4, false>), grid, dim3(512), lds, stream, p);
    else hipLaunchKernelGGL((acc4_prefill_kernel<NBS, SF32, NBS == 2 ? 4 : 2, false>), grid, dim3(512), lds, stream, p);
    return static_cast<int>(hipGetLastError());
}

}  // namespace mnb

extern "C" int rocm_acc4_mfma_eligible(const RocmMatMulNBitsArgs* a)
{
    if (a->m < 1 || a->n < 1 || a->block_size < 32) return 0;
    const int64_t kb = (a->k + a->block_size - 1) / a->block_size;
    const int64_t padded_k = kb * a->block_size;
    if ((reinterpret_cast<uintptr_t>(a->b) & 15) != 0 || (reinterpret_cast<uintptr_t>(a->scales) & 3) != 0) return 0;
    if (a->m <= 16) {
        const bool bs_ok = a->block_size == 32 || a->block_size == 64 || a->block_size == 128;
        return bs_ok && padded_k / 2 * 16 < 0x7fffffff && a->m * padded_k < 0x7ffffff0;
    }
    // prefill: 32-bit offsets inside one 128-row / 128-column window and inside the block-major scales
    return padded_k / 2 * 128 < 0x7fffffff && padded_k * 128 < 0x7fffffff && kb * a->m * 4 < 0x7fffffff;
}

extern "C" uint64_t rocm_acc4_mfma_scratch_bytes(const RocmMatMulNBitsArgs* a)
{
    if (a->m <= 16 || a->block_size < 32) return 0;
    const int64_t padded_k = (a->k + a->block_size - 1) / a->block_size * a->block_size;
    const int slices = mnb::acc4_prefill_slices(a->m, a->n, padded_k, a->block_size);
    return slices > 1 ? static_cast<uint64_t>(slices) * static_cast<uint64_t>(a->m) * static_cast<uint64_t>(a->n) * 4 : 0;
}

extern "C" int rocm_launch_acc4_mfma(const RocmMatMulNBitsArgs* a, const RocmAcc4Workspace* ws, int waves, rocm_stream_t stream)
{
    if (!rocm_acc4_mfma_eligible(a)) return -1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (a->m > 16) {
        mnb::Acc4PrefillParams q;
        q.qa = ws->qa;
        q.sa_t = ws->aux;
        q.b = a->b;
        q.scales = a->scales;
        q.zp = a->zp;
        q.bias = a->bias;
        q.y = a->y;
        q.m = a->m;
        q.n = a->n;
        q.kb = (a->k + a->block_size - 1) / a->block_size;
        q.padded_k = q.kb * a->block_size;
        q.row_bytes = q.padded_k / 2;
        q.zp_row = (q.kb + 1) / 2;
        q.bs_log2 = __builtin_ctz(static_cast<unsigned>(a->block_size));
        q.scales_bf16 = a->scale_dtype == ROCM_DT_BF16;
        q.bias_dtype = a->bias_dtype;
        q.y_dtype = a->y_dtype;
        q.acc_probe = a->acc_probe;
        if (q.acc_probe && q.m * q.n * q.kb * 4 >= 0x7fffffff) return -1;            // the probe is addressed with 32-bit offsets
        const bool sf32 = a->scale_dtype == ROCM_DT_F32;
        // slices of K when the grid is small and the workspace has room for their partial sums
        int slices = mnb::acc4_prefill_slices(a->m, a->n, q.padded_k, a->block_size);
        const uint64_t per_slice = static_cast<uint64_t>(a->m) * static_cast<uint64_t>(a->n) * 4;
        if (!ws->partial || ws->partial_bytes < 2 * per_slice) slices = 1;
        else if (ws->partial_bytes < slices * per_slice) slices = static_cast<int>(ws->partial_bytes / per_slice);
        const int64_t steps = (q.padded_k + mnb::kStep - 1) / mnb::kStep;
        q.steps_per_slice = mnb::acc4_steps_per_slice(q.padded_k, a->block_size, slices);
        slices = static_cast<int>((steps + q.steps_per_slice - 1) / q.steps_per_slice);          // no empty slice after rounding to blocks
        q.partial = slices > 1 ? ws->partial : nullptr;
        int rc;
        if (a->block_size == 32) rc = sf32 ? mnb::launch_acc4_prefill<2, true>(q, slices, s) : mnb::launch_acc4_prefill<2, false>(q, slices, s);
        else if (a->block_size == 64) rc = sf32 ? mnb::launch_acc4_prefill<1, true>(q, slices, s) : mnb::launch_acc4_prefill<1, false>(q, slices, s);
        else rc = sf32 ? mnb::launch_acc4_prefill<0, true>(q, slices, s) : mnb::launch_acc4_prefill<0, false>(q, slices, s);
        if (rc != 0 || slices == 1) return rc;
        return rocm_launch_slice_reduce(ws->partial, slices, a->m, a->n, a->bias, a->bias_dtype, a->y, a->y_dtype, stream);
    }
    mnb::Acc4DecodeParams p;
    p.qa = ws->qa;
    p.aq = ws->aq;
    p.aux16 = ws->aux;
    p.b = a->b;
    p.scales = a->scales;
    p.zp = a->zp;
    p.bias = a->bias;
    p.y = a->y;
    p.m = a->m;
    p.n = a->n;
    p.kb = (a->k + a->block_size - 1) / a->block_size;
    p.padded_k = p.kb * a->block_size;
    p.row_bytes = p.padded_k / 2;
    p.zp_row = (p.kb + 1) / 2;
    p.tiles = static_cast<int>((p.padded_k + 127) / 128);
    p.bias_dtype = a->bias_dtype;
    p.y_dtype = a->y_dtype;
    p.scales_bf16 = a->scale_dtype == ROCM_DT_BF16;
    p.acc_probe = a->acc_probe;

    const int group_tiles = a->m <= 1 ? 4 : 2;
    const int64_t wgs = (a->n + 15) / 16;
    int w = waves;
    if (w <= 0) {
        const int want = static_cast<int>((8192 + wgs - 1) / wgs);
        int by_work = p.tiles / group_tiles;
        if (by_work < 1) by_work = 1;
        w = want < by_work ? want : by_work;
        if (wgs * 4 >= 6144 && a->m <= 1) w = by_work;     // many column groups: short waves, no prefetch (see SETS)
        if (w < 1) w = 1;
    }
    if (w > 8) w = 8;
    int tpw = (p.tiles + w - 1) / w;
    tpw = (tpw + group_tiles - 1) / group_tiles * group_tiles;
    w = (p.tiles + tpw - 1) / tpw;
    p.tiles_per_wave = tpw;

    const bool single_set = a->m <= 1 && wgs * w >= 6144;
    if (a->scale_dtype == ROCM_DT_F32) return mnb::launch_acc4_decode_bs<float>(p, a->block_size, w, single_set, s);
    return mnb::launch_acc4_decode_bs<uint16_t>(p, a->block_size, w, single_set, s);
}
