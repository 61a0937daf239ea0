// Decode path of MatMulNBits (M <= 16, f16/bf16 activations): a split-K GEMV on the matrix cores.
//
// Work split. A workgroup owns 16*CG output columns; its waves split K between them in runs of
// 128-element tiles and meet once at the end in LDS, in wave order, so the result is deterministic.
//
// Streaming. Lane (c = lane % 16, g = lane / 16) reads, per tile, one 16-byte piece of packed
// column c: 32 nibbles that never leave registers. Each of its four dwords becomes the eight
// 16-bit operands one v_mfma_f32_16x16x32 wants from that lane, by OR-ing the nibble under a
// constant exponent ("magic" value: 1024+q as f16, 128+q as bf16 - both exact). The activation
// rows are the other MFMA operand (rows beyond M are zero). A second MFMA per dword, whose weight
// operand is the constant -(magic+zp), removes magic and zero point inside the f32 accumulator, so
// the accumulator holds sum a*(q-zp) for the block and is scaled once per block:
//     y += scale[n, block] * acc.
// For block sizes below 128 the four lane groups first swap dwords (two v_permlane*_swap stages,
// a 4x4 transpose) so that one MFMA never mixes two blocks.
#include "common.hiph"

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
    int tiles;              // ceil(kb * BS / 128)
    int tiles_per_wave;     // multiple of max(1, BS / 128)
    int bias_dtype, y_dtype;
};

template <bool BF16> struct Magic;
template <> struct Magic<false> { static constexpr uint32_t pos = 0x64006400u, neg = 0xE400E400u; };
template <> struct Magic<true> { static constexpr uint32_t pos = 0x43004300u, neg = 0xC300C300u; };

template <bool BF16>
__device__ __forceinline__ float4_t mfma16(const uint4& act, const uint4& wgt, float4_t acc)
{
    if constexpr (BF16) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, act), __builtin_bit_cast(bf16x8_t, wgt), acc, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, act), __builtin_bit_cast(half8_t, wgt), acc, 0, 0, 0);
    }
}

// Eight nibbles of `w` (k ascending from bit 0) -> four registers of two 16-bit floats (magic + q),
// element 2i in the low half and 2i+1 in the high half: the order activations lie in memory.
template <bool BF16>
__device__ __forceinline__ uint4 unpack8(uint32_t w)
{
    const uint32_t w4 = w >> 4;
    constexpr uint32_t mask = 0x000F000Fu, mg = Magic<BF16>::pos;
    uint4 r;
    r.x = (__builtin_amdgcn_perm(w4, w, 0x0c040c00u) & mask) | mg;
    r.y = (__builtin_amdgcn_perm(w4, w, 0x0c050c01u) & mask) | mg;
    r.z = (__builtin_amdgcn_perm(w4, w, 0x0c060c02u) & mask) | mg;
    r.w = (__builtin_amdgcn_perm(w4, w, 0x0c070c03u) & mask) | mg;
    return r;
}

// 4x4 transpose of dwords across the four 16-lane groups: afterwards group g holds, in component d,
// what group d held in component g.
__device__ __forceinline__ void transpose_groups(uint4& v)
{
    auto s0 = __builtin_amdgcn_permlane32_swap(v.x, v.z, false, false);
    auto s1 = __builtin_amdgcn_permlane32_swap(v.y, v.w, false, false);
    auto t0 = __builtin_amdgcn_permlane16_swap(s0[0], s1[0], false, false);
    auto t1 = __builtin_amdgcn_permlane16_swap(s0[1], s1[1], false, false);
    v.x = t0[0];
    v.y = t0[1];
    v.z = t1[0];
    v.w = t1[1];
}

template <typename ST> __device__ __forceinline__ float scale_to_f32(ST s, bool bf16);
template <> __device__ __forceinline__ float scale_to_f32<float>(float s, bool) { return s; }
template <> __device__ __forceinline__ float scale_to_f32<uint16_t>(uint16_t s, bool bf16) { return bf16 ? bf16_bits_to_f32(s) : f16_bits_to_f32(s); }

// BF16: activation element type. BS: block size (32, 64, 128, 256). CG: 16-column groups per workgroup.
// ST: storage type of the scales (uint16_t = same 16-bit type as the activations, float = f32).
template <bool BF16, int BS, int CG, typename ST, int U>
__global__ __launch_bounds__(1024) void decode_mfma_kernel(DecodeParams p)
{
    constexpr bool kTranspose = BS < 128;      // several blocks inside one 128-element tile
    constexpr int kBsLog2 = BS == 32 ? 5 : BS == 64 ? 6 : BS == 128 ? 7 : 8;
    extern __shared__ float red[];             // [waves][CG][4][64]

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int waves = blockDim.x >> 6;
    const int c = lane & 15;
    const int g = lane >> 4;
    const int64_t n_base = static_cast<int64_t>(blockIdx.x) * (16 * CG);

    const uint8_t* brow[CG];
    const ST* srow[CG];
    const uint8_t* zrow[CG];
#pragma unroll
    for (int cg = 0; cg < CG; ++cg) {
        int64_t col = n_base + cg * 16 + c;
        if (col >= p.n) col = p.n - 1;          // stay inside the tensor; the store is masked
        brow[cg] = p.b + col * p.row_bytes;
        srow[cg] = static_cast<const ST*>(p.scales) + col * p.kb;
        zrow[cg] = p.zp ? p.zp + col * p.zp_row : nullptr;
    }
    const bool row_ok = c < p.m;
    const uint16_t* arow = p.a + static_cast<int64_t>(row_ok ? c : 0) * p.k;

    float4_t y[CG];
    float4_t acc[CG];
#pragma unroll
    for (int cg = 0; cg < CG; ++cg) {
        y[cg] = float4_t{0.f, 0.f, 0.f, 0.f};
        acc[cg] = float4_t{0.f, 0.f, 0.f, 0.f};
    }

    const int t_begin = wave * p.tiles_per_wave;
    const int t_end = min(t_begin + p.tiles_per_wave, p.tiles);

    for (int t0 = t_begin; t0 < t_end; t0 += U) {
        uint4 wq[U][CG];
        uint4 av[U][4];
        ST sc[U][CG];
        uint32_t zq[U][CG];
        // ---- issue every load of this batch before touching any of them ----
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int kt = t0 + u;
            const bool tile_ok = kt < t_end;
            const int64_t boff = static_cast<int64_t>(kt) * 64 + g * 16;
            const bool w_ok = tile_ok && boff < p.row_bytes;
            const int64_t blk = (static_cast<int64_t>(kt) * 128 + g * 32) >> kBsLog2;
#pragma unroll
            for (int cg = 0; cg < CG; ++cg) {
                wq[u][cg] = w_ok ? *reinterpret_cast<const uint4*>(brow[cg] + boff) : make_uint4(0, 0, 0, 0);
                sc[u][cg] = w_ok ? srow[cg][blk] : ST(0);
                zq[u][cg] = (w_ok && zrow[cg]) ? ((zrow[cg][blk >> 1] >> ((blk & 1) * 4)) & 0xfu) : 8u;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int64_t k0 = static_cast<int64_t>(kt) * 128 + (kTranspose ? j * 32 + g * 8 : g * 32 + j * 8);
                av[u][j] = (tile_ok && row_ok && k0 + 8 <= p.k) ? *reinterpret_cast<const uint4*>(arow + k0) : make_uint4(0, 0, 0, 0);
            }
        }
        // ---- compute ----
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int kt = t0 + u;
            if (kt < t_end) {
#pragma unroll
                for (int cg = 0; cg < CG; ++cg) {
                    uint4 w = wq[u][cg];
                    if constexpr (kTranspose) transpose_groups(w);
                    const uint32_t wd[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        // zero point and scale of the block MFMA j works on
                        uint32_t z = zq[u][cg];
                        ST s = sc[u][cg];
                        if constexpr (kTranspose) {
                            const int src = c + 16 * ((j * 32) / BS) * (BS / 32);
                            z = __shfl(z, src, kWave);
                            if constexpr (sizeof(ST) == 4) s = __shfl(s, src, kWave);
                            else s = static_cast<ST>(__shfl(static_cast<uint32_t>(s), src, kWave));
                        }
                        const uint32_t zpair = Magic<BF16>::neg | (z * 0x00010001u);
                        const uint4 zc = make_uint4(zpair, zpair, zpair, zpair);
                        acc[cg] = mfma16<BF16>(av[u][j], unpack8<BF16>(wd[j]), acc[cg]);
                        acc[cg] = mfma16<BF16>(av[u][j], zc, acc[cg]);
                        const int k_done = kt * 128 + (j + 1) * 32;
                        const bool flush = kTranspose ? (k_done % BS == 0) : (j == 3 && (k_done % BS == 0 || kt + 1 == t_end));
                        if (flush) {
                            const float sf = scale_to_f32<ST>(s, BF16);
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
                                y[cg][r] = fmaf(sf, acc[cg][r], y[cg][r]);
                                acc[cg][r] = 0.f;
                            }
                        }
                    }
                }
            }
        }
    }

    // ---- split-K reduction across the waves of this workgroup, in wave order ----
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
            if (p.bias) total += load_as_f32(p.bias, p.bias_dtype, col);
            store_from_f32(p.y, p.y_dtype, static_cast<int64_t>(row) * p.n + col, total);
        }
    }
}

template <bool BF16, int BS, int CG, typename ST>
static int launch_cfg(const DecodeParams& p, int waves, hipStream_t stream)
{
    constexpr int U = CG >= 4 ? 1 : (CG == 2 ? 2 : 4);
    const unsigned grid = static_cast<unsigned>((p.n + 16 * CG - 1) / (16 * CG));
    const size_t lds = static_cast<size_t>(waves) * CG * 256 * sizeof(float);
    hipLaunchKernelGGL((decode_mfma_kernel<BF16, BS, CG, ST, U>), dim3(grid), dim3(waves * 64), lds, stream, p);
    return static_cast<int>(hipGetLastError());
}

template <bool BF16, int BS, typename ST>
static int launch_cg(const DecodeParams& p, int waves, int cg, hipStream_t stream)
{
    switch (cg) {
        case 1: return launch_cfg<BF16, BS, 1, ST>(p, waves, stream);
        case 2: return launch_cfg<BF16, BS, 2, ST>(p, waves, stream);
        default: return launch_cfg<BF16, BS, 4, ST>(p, waves, stream);
    }
}

template <bool BF16, typename ST>
static int launch_bs(const DecodeParams& p, int bs, int waves, int cg, hipStream_t stream)
{
    switch (bs) {
        case 32: return launch_cg<BF16, 32, ST>(p, waves, cg, stream);
        case 64: return launch_cg<BF16, 64, ST>(p, waves, cg, stream);
        case 128: return launch_cg<BF16, 128, ST>(p, waves, cg, stream);
        default: return launch_cg<BF16, 256, ST>(p, waves, cg, stream);
    }
}

}  // namespace mnb

extern "C" int rocm_decode_mfma_eligible(const RocmMatMulNBitsArgs* a)
{
    const bool half_in = a->a_dtype == ROCM_DT_F16 || a->a_dtype == ROCM_DT_BF16;
    const bool scale_ok = a->scale_dtype == a->a_dtype || a->scale_dtype == ROCM_DT_F32;
    const bool bs_ok = a->block_size == 32 || a->block_size == 64 || a->block_size == 128 || a->block_size == 256;
    return half_in && scale_ok && bs_ok && a->m >= 1 && a->m <= 16 && a->n >= 1 && a->k % 8 == 0 &&
           (reinterpret_cast<uintptr_t>(a->a) & 15) == 0 && (reinterpret_cast<uintptr_t>(a->b) & 15) == 0;
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
    p.tiles = static_cast<int>((p.kb * a->block_size + 127) / 128);
    p.bias_dtype = a->bias_dtype;
    p.y_dtype = a->y_dtype;

    const int tiles_per_block = a->block_size > 128 ? a->block_size / 128 : 1;
    // Heuristic: enough waves to cover the chip several times, at least ~4 tiles of work each.
    int cg = col_groups;
    if (cg != 1 && cg != 2 && cg != 4) {
        const int64_t groups = (a->n + 15) / 16;
        cg = (a->m > 4 && groups >= 4096) ? 2 : 1;
    }
    int w = waves;
    if (w <= 0) {
        const int64_t wgs = (a->n + 16 * cg - 1) / (16 * cg);
        int want = static_cast<int>((8192 + wgs - 1) / wgs);   // waves per workgroup to reach ~8k waves
        int by_work = p.tiles / (4 * tiles_per_block);          // keep >= 4 tiles per wave
        if (by_work < 1) by_work = 1;
        w = want < by_work ? want : by_work;
        if (w < 1) w = 1;
    }
    if (w > 16) w = 16;
    int tpw = (p.tiles + w - 1) / w;
    tpw = (tpw + tiles_per_block - 1) / tiles_per_block * tiles_per_block;
    w = (p.tiles + tpw - 1) / tpw;
    p.tiles_per_wave = tpw;

    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool bf16 = a->a_dtype == ROCM_DT_BF16;
    const bool f32_scales = a->scale_dtype == ROCM_DT_F32;
    if (bf16) return f32_scales ? mnb::launch_bs<true, float>(p, a->block_size, w, cg, s) : mnb::launch_bs<true, uint16_t>(p, a->block_size, w, cg, s);
    return f32_scales ? mnb::launch_bs<false, float>(p, a->block_size, w, cg, s) : mnb::launch_bs<false, uint16_t>(p, a->block_size, w, cg, s);
}
