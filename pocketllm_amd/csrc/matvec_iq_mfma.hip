// Decode matvec over raw IQ2_XXS / IQ1_M super-blocks with the integer dots on the matrix cores.
//
// A wave owns a tile of 16 consecutive output rows (or, for short matrices, a share of the tile's
// super-blocks; the shares meet in a small LDS reduction); the activation image (two int8 terms per
// value) sits in LDS.  For one super-block index the wave forms
//     C[m][n] = sum_k A[m][k] * B[k][n],     v_mfma_i32_16x16x64_i8,
// with n = output row, B = the weights' integer codes and A = activation bytes arranged so that row
// m collects one scale group of the block (the format structs below say which).  Lane (n, s)
// supplies B for the 16-weight slice s of each MFMA from its own 64 weights of the block, and the
// slices are assigned to A rows such that the lane finds the results for exactly those 64 weights
// in its own C registers: C[4 s .. 4 s + 3][n].
//
// The codebook lookups happen once per weight and feed 16 rows of dots each, where the v_dot4 form
// repeats the activation reads and the dots per lane.
#include "block_dot4.h"
#include "pllm_internal.h"

namespace pllm {
namespace {

constexpr int kRowsPerTile = 16;
constexpr int kWaves = 8;
constexpr int kMaxRounds = 16;           // row-tile groups one workgroup works through at most

typedef int v4i __attribute__((ext_vector_type(4)));

__device__ __forceinline__ v4i as_v4i(uint32_t x, uint32_t y, uint32_t z, uint32_t w) {
    v4i r;
    r.x = static_cast<int>(x); r.y = static_cast<int>(y); r.z = static_cast<int>(z); r.w = static_cast<int>(w);
    return r;
}

// LDS offsets of a lane's A operands: slot i of block b is read at off[i] + b * step[i]; slots whose
// A row is not the lane's point at 16 zero bytes with step 0.
template <int SLOTS>
struct AMap { int off[SLOTS]; int step[SLOTS]; };

// ------------------------------------------------------------------------------------------------
// IQ2_XXS: 66 B = d(2) + 8 sub-blocks of 8 B (four grid ids, then a u32: four 7-bit sign indices and
// a 4-bit scale).  Lane (n, s) holds sub-blocks 2 s and 2 s + 1 (two 32-weight groups).
// A rows: m = 2 * group + term; MFMA t, slice s carries half t % 2 of group 2 s + t / 2, so
// C[4 s .. 4 s + 3][n] = groups 2 s and 2 s + 1, both terms, in the lane's own registers.
// LDS tables: 256 x 8 magnitude bytes g, 128 x 8 sign masks m (0xff where the weight is negative).
// The signed code is (g ^ m) - m bytewise; instead of finishing that per byte, the wave runs two
// MFMAs per slice, with B = g ^ m and with B = m, and subtracts the accumulators.
// ------------------------------------------------------------------------------------------------
struct IQ2XXSm {
    static constexpr int kBlockBytes = 66;
    static constexpr int kTableBytes = IQ2XXS::kTableBytes;
    static constexpr int kSlots = 4;
    struct Regs { uint4 q; uint32_t d; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int s) {
        r.q = load16_a2(blk + 2 + 16 * s);
        r.d = *reinterpret_cast<const uint16_t*>(blk);
    }
    static __device__ __forceinline__ void stage_tables(unsigned char* lds) { IQ2XXS::stage_tables(lds); }
    static __device__ __forceinline__ void a_map(AMap<kSlots>& am, int col, int ks, int kpad, int zero_off) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int g = 2 * ks + (t >> 1);
            const bool active = (col >> 1) == g;
            am.off[t] = active ? ((col & 1) ? kpad : 0) + 32 * g + 16 * (t & 1) : zero_off;
            am.step[t] = active ? 256 : 0;
        }
    }
    static __device__ __forceinline__ float block(const Regs& r, int s, int b, const unsigned char* smem, const AMap<kSlots>& am,
                                                  const StagedX& sx, const unsigned char* tables) {
        const uint2* grid = reinterpret_cast<const uint2*>(tables);
        const uint2* sign = grid + 256;
        v4i c = {0, 0, 0, 0}, cm = {0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t ids = (t < 2) ? r.q.x : r.q.z, aux = (t < 2) ? r.q.y : r.q.w;
            const int e = 2 * (t & 1);                                         // grid entries e and e + 1 of the sub-block
            const uint2 g0 = grid[(ids >> (8 * e)) & 0xffu], m0 = sign[(aux >> (7 * e)) & 127u];
            const uint2 g1 = grid[(ids >> (8 * e + 8)) & 0xffu], m1 = sign[(aux >> (7 * e + 7)) & 127u];
            const uint4 a = *reinterpret_cast<const uint4*>(smem + am.off[t] + b * am.step[t]);
            const v4i av = as_v4i(a.x, a.y, a.z, a.w);
            c = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, as_v4i(g0.x ^ m0.x, g0.y ^ m0.y, g1.x ^ m1.x, g1.y ^ m1.y), c, 0, 0, 0);
            cm = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, as_v4i(m0.x, m0.y, m1.x, m1.y), cm, 0, 0, 0);
        }
        const float v0 = static_cast<float>(__mul24(c.x - cm.x, 254) + (c.y - cm.y));   // group 2 s: 254 * high term + low term
        const float v1 = static_cast<float>(__mul24(c.z - cm.z, 254) + (c.w - cm.w));   // group 2 s + 1
        const float4 g2 = *reinterpret_cast<const float4*>(sx.gs + b * 8 + 2 * s);   // {xs0 / 254, sum0, xs1 / 254, sum1}
        const float ls0 = static_cast<float>(2 * (r.q.y >> 28) + 1), ls1 = static_cast<float>(2 * (r.q.w >> 28) + 1);
        return 0.125f * f16_bits_to_float(r.d) * (ls0 * g2.x * v0 + ls1 * g2.z * v1);
    }
};

// ------------------------------------------------------------------------------------------------
// IQ1_M: 56 B = qs(32) qh(16) scales(8); w = dl (c - 1 + delta) with c in {0, 1, 2} from the
// codebook (index: qs byte plus the low three bits of its qh nibble), dl = d (2 s3 + 1) per 16
// weights, delta = -+1/8 per 8 weights (bit 3 of the nibble).  Lane (n, s) holds entries 8 s .. 8 s + 7
// = four 16-weight groups.  With integer codes 8 c +- 1 = 8 (c + delta),
//     sum w x = d sum over 16-groups j of (2 s3_j + 1) [ dot(8 c +- 1, x)_j / 8 - sum16(x)_j ].
// A rows: m = 16-group of the block, one MFMA set per activation term; MFMA t, slice s carries group
// 4 s + t, so C[4 s .. 4 s + 3][n] = the lane's own four groups.  sum16 comes from the image.
// LDS table: 4096 x 8 code bytes, index = qs byte | nibble << 8 (the delta bit selects the half).
// ------------------------------------------------------------------------------------------------
struct alignas(16) Iq1DeltaCodes { uint64_t v[4096]; };
constexpr Iq1DeltaCodes make_iq1_delta_codes() {
    Iq1DeltaCodes t{};
    for (int i = 0; i < 4096; ++i) {
        const uint32_t p = PLLM_IQ1_GRID_PACKED[i & 2047];      // element e in bits [2e, 2e+1], value + 1
        uint64_t v = 0;
        for (int e = 0; e < 8; ++e) {
            const int code = 8 * static_cast<int>((p >> (2 * e)) & 3u) + ((i & 2048) ? -1 : 1);
            v |= static_cast<uint64_t>(static_cast<uint8_t>(code)) << (8 * e);
        }
        t.v[i] = v;
    }
    return t;
}
static __device__ const Iq1DeltaCodes PLLM_IQ1_DELTA_CODES = make_iq1_delta_codes();

struct IQ1Mm {
    static constexpr int kBlockBytes = 56;
    static constexpr int kTableBytes = 32768;
    static constexpr int kSlots = 8;                           // [term][t]
    struct Regs { uint2 qs; uint32_t qh; uint2 sc; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int s) {
        r.qs = *reinterpret_cast<const uint2*>(blk + 8 * s);                   // blocks are 8-byte aligned
        r.qh = *reinterpret_cast<const uint32_t*>(blk + 32 + 4 * s);
        r.sc = *reinterpret_cast<const uint2*>(blk + 48);
    }
    static __device__ __forceinline__ void stage_tables(unsigned char* lds) {
        copy_to_lds(lds, reinterpret_cast<const unsigned char*>(PLLM_IQ1_DELTA_CODES.v), kTableBytes);
    }
    static __device__ __forceinline__ void a_map(AMap<kSlots>& am, int col, int ks, int kpad, int zero_off) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const bool active = col == 4 * ks + t;
            am.off[t] = active ? 16 * col : zero_off;
            am.off[4 + t] = active ? kpad + 16 * col : zero_off;
            am.step[t] = am.step[4 + t] = active ? 256 : 0;
        }
    }
    static __device__ __forceinline__ float block(const Regs& r, int s, int b, const unsigned char* smem, const AMap<kSlots>& am,
                                                  const StagedX& sx, const unsigned char* tables) {
        const uint2* table = reinterpret_cast<const uint2*>(tables);
        const uint32_t s01 = r.sc.x, s23 = r.sc.y;
        const uint32_t dbits = ((s01 >> 12) & 0xfu) | ((s01 >> 24) & 0xf0u) | ((s23 >> 4) & 0xf00u) | ((s23 >> 16) & 0xf000u);
        // the lane's four 16-weight scales are the low 12 bits of scale word s
        const uint32_t word = ((s & 2) ? s23 : s01) >> (16 * (s & 1));
        v4i ch = {0, 0, 0, 0}, cl = {0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 4; ++t) {                                          // 16-weight group t of the lane = entries 2 t, 2 t + 1
            const uint32_t qw = (t < 2) ? r.qs.x : r.qs.y;
            const uint2 w0 = table[((qw >> (16 * (t & 1))) & 0xffu) | (((r.qh >> (8 * t)) & 15u) << 8)];
            const uint2 w1 = table[((qw >> (16 * (t & 1) + 8)) & 0xffu) | (((r.qh >> (8 * t + 4)) & 15u) << 8)];
            const v4i bw = as_v4i(w0.x, w0.y, w1.x, w1.y);
            const uint4 ah = *reinterpret_cast<const uint4*>(smem + am.off[t] + b * am.step[t]);
            const uint4 al = *reinterpret_cast<const uint4*>(smem + am.off[4 + t] + b * am.step[4 + t]);
            ch = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(ah.x, ah.y, ah.z, ah.w), bw, ch, 0, 0, 0);
            cl = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(al.x, al.y, al.z, al.w), bw, cl, 0, 0, 0);
        }
        const float4 g2 = *reinterpret_cast<const float4*>(sx.gs + b * 8 + 2 * s);   // {xs0 / 254, sum0, xs1 / 254, sum1}
        const float4 s16 = *reinterpret_cast<const float4*>(sx.sum16 + b * 16 + 4 * s);
        const float x0 = 0.125f * g2.x, x1 = 0.125f * g2.z;
        const float ls0 = static_cast<float>(2 * (word & 7u) + 1), ls1 = static_cast<float>(2 * ((word >> 3) & 7u) + 1);
        const float ls2 = static_cast<float>(2 * ((word >> 6) & 7u) + 1), ls3 = static_cast<float>(2 * ((word >> 9) & 7u) + 1);
        const float v = ls0 * (x0 * static_cast<float>(__mul24(ch.x, 254) + cl.x) - s16.x) + ls1 * (x0 * static_cast<float>(__mul24(ch.y, 254) + cl.y) - s16.y) +
                        ls2 * (x1 * static_cast<float>(__mul24(ch.z, 254) + cl.z) - s16.z) + ls3 * (x1 * static_cast<float>(__mul24(ch.w, 254) + cl.w) - s16.w);
        return f16_bits_to_float(dbits) * v;
    }
};

// The lane's share of ITERS super-blocks of one row tile: blocks part + (pass * ITERS + it) * split
// (clamped: always a valid address)
template <typename FMT, int ITERS>
__device__ __forceinline__ void load_unit(typename FMT::Regs (&regs)[ITERS], const uint8_t* __restrict__ w, int n, int bpr,
                                          int tile, int col, int ks, int part, int split, int pass) {
    const int row = tile * kRowsPerTile + col;
    const uint8_t* wrow = w + static_cast<size_t>(row < n ? row : 0) * bpr * FMT::kBlockBytes;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int b = min(part + (pass * ITERS + it) * split, bpr - 1);
        FMT::load(regs[it], wrow + static_cast<size_t>(b) * FMT::kBlockBytes, ks);
    }
}

// A workgroup of 8 waves stages the activation image and the codebooks once and then works through
// `rounds` groups of row tiles (group = blockIdx.x + round * gridDim.x, 8 / split tiles of 16 rows
// each): `split` waves share a tile's super-blocks.  The blocks of the next unit of work are loaded
// while the current one is computed.
template <typename FMT, int ITERS>
__global__ __launch_bounds__(64 * kWaves) void iq_mfma_matvec_kernel(
    const unsigned char* __restrict__ image, size_t image_stride, const uint8_t* __restrict__ w,
    void* __restrict__ y, int y_dtype, int n, int bpr, int split, int groups) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    const StagedX sx = carve_staged_x(smem, kpad);
    const int zero_off = image_bytes;                                        // 16 zero bytes
    unsigned char* tables = smem + image_bytes + 16;
    float* partial = reinterpret_cast<float*>(tables + FMT::kTableBytes);   // [rounds][waves][16]

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int col = lane & 15;        // B/C column = output row within the tile; also A's row index m
    const int ks = lane >> 4;         // k slice of A and B, row quad of C
    const int tiles_per_group = kWaves / split;
    const int tile_in_group = wave / split, part = wave % split;
    const int passes = (bpr + split * ITERS - 1) / (split * ITERS);
    const int rounds = (groups - static_cast<int>(blockIdx.x) + static_cast<int>(gridDim.x) - 1) / static_cast<int>(gridDim.x);
    const int units = rounds * passes;
    const int tile0 = blockIdx.x * tiles_per_group + tile_in_group, tile_step = gridDim.x * tiles_per_group;

    // A side: this lane supplies row m = col of every MFMA, slice ks; the format says which rows are its
    AMap<FMT::kSlots> am;
    FMT::a_map(am, col, ks, kpad, zero_off);

    typename FMT::Regs cur[ITERS], nxt[ITERS];
    load_unit<FMT, ITERS>(cur, w, n, bpr, tile0, col, ks, part, split, 0);
    copy_to_lds(smem, image + static_cast<size_t>(blockIdx.y) * image_stride, image_bytes);
    if (tid < 4) reinterpret_cast<uint32_t*>(smem + zero_off)[tid] = 0;
    FMT::stage_tables(tables);
    __syncthreads();

    float acc = 0.0f;
    int round = 0, pass = 0;
    for (int u = 0; u < units; ++u) {
        int next_round = round, next_pass = pass + 1;
        if (next_pass == passes) { next_pass = 0; ++next_round; }
        if (u + 1 < units) load_unit<FMT, ITERS>(nxt, w, n, bpr, tile0 + next_round * tile_step, col, ks, part, split, next_pass);
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            // no branch around a block past the row's end (its registers hold the clamped block's data):
            // the blocks of a unit are then free to overlap; its result is dropped
            const int b = part + (pass * ITERS + it) * split;
            const float v = FMT::block(cur[it], ks, min(b, bpr - 1), smem, am, sx, tables);
            acc += b < bpr ? v : 0.0f;
        }
        if (next_pass == 0) {                                                // the tile's last pass
            acc += __shfl_xor(acc, 16, 64);
            acc += __shfl_xor(acc, 32, 64);
            if (split == 1) {
                const int row = (tile0 + round * tile_step) * kRowsPerTile + col;
                if (ks == 0 && row < n) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + row, acc);
            } else if (ks == 0) {
                partial[(round * kWaves + wave) * kRowsPerTile + col] = acc;
            }
            acc = 0.0f;
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) cur[it] = nxt[it];
        round = next_round; pass = next_pass;
    }
    if (split == 1) return;
    __syncthreads();
    // thread i sums the `split` partials of (round, tile in group, row) = i
    for (int i = tid; i < rounds * tiles_per_group * kRowsPerTile; i += blockDim.x) {
        const int r = i / (tiles_per_group * kRowsPerTile), rest = i % (tiles_per_group * kRowsPerTile);
        const int t = rest / kRowsPerTile, c = rest % kRowsPerTile;
        float total = 0.0f;
        for (int v = 0; v < split; ++v) total += partial[(r * kWaves + t * split + v) * kRowsPerTile + c];
        const int row = ((blockIdx.x + r * gridDim.x) * tiles_per_group + t) * kRowsPerTile + c;
        if (row < n) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + row, total);
    }
}

template <typename FMT, int ITERS>
int launch_one(const unsigned char* image, size_t image_stride, const uint8_t* w, void* y, int y_dtype,
               int rows, int n, int bpr, int split, hipStream_t stream) {
    auto kern = iq_mfma_matvec_kernel<FMT, ITERS>;
    const size_t fixed = staged_x_bytes(bpr * 256) + 16 + FMT::kTableBytes;
    // workgroups that fit the device at once (per kernel, asked once)
    static int resident = 0;
    if (resident == 0) {
        int per_cu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, 64 * kWaves, fixed + 4096) != hipSuccess || per_cu < 1) per_cu = 2;
        resident = per_cu * compute_units();
    }
    const int tiles = (n + kRowsPerTile - 1) / kRowsPerTile;
    const int groups = (tiles * split + kWaves - 1) / kWaves;
    int grid = groups;
    if (groups > resident) {
        const int rounds = min(kMaxRounds, (groups + resident - 1) / resident);
        grid = (groups + rounds - 1) / rounds;
    }
    const int rounds = (groups + grid - 1) / grid;
    const size_t smem = fixed + (split > 1 ? static_cast<size_t>(rounds) * kWaves * kRowsPerTile * sizeof(float) : 0);
    if (smem > 64 * 1024) {
        if (smem > 160 * 1024) return PLLM_ERR_UNSUPPORTED;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(smem)) != hipSuccess)
            return PLLM_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL(kern, dim3(grid, rows), dim3(64 * kWaves), smem, stream, image, image_stride, w, y, y_dtype, n, bpr, split, groups);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

template <typename FMT>
int launch_fmt(const unsigned char* image, size_t image_stride, const uint8_t* w, void* y, int y_dtype,
               int rows, int n, int bpr, hipStream_t stream) {
    // waves per row tile: one when there are tiles enough to keep every wave of the device busy
    // several times over, more (each with at least two super-blocks) for short matrices
    const int tiles = (n + kRowsPerTile - 1) / kRowsPerTile;
    const int want = 6 * compute_units();
    int split = 1;
    while (split < kWaves && split * 4 <= bpr && (tiles * split + kWaves - 1) / kWaves * rows < want) split *= 2;
    const int niter = (bpr + split - 1) / split;
    const int passes = (niter + 3) / 4;
    const int iters = (niter + passes - 1) / passes;
#define PLLM_CASE(I) case I: return launch_one<FMT, I>(image, image_stride, w, y, y_dtype, rows, n, bpr, split, stream)
    switch (iters) {
        PLLM_CASE(1); PLLM_CASE(2); PLLM_CASE(3);
        default: return launch_one<FMT, 4>(image, image_stride, w, y, y_dtype, rows, n, bpr, split, stream);
    }
#undef PLLM_CASE
}

}  // namespace

int iq_mfma_matvec_from_image(const unsigned char* image, size_t stride, const uint8_t* w, int type_id, void* y, int y_dtype,
                              int rows, int n, int bpr, hipStream_t stream) {
    switch (type_id) {
        case PLLM_TYPE_IQ2_XXS: return launch_fmt<IQ2XXSm>(image, stride, w, y, y_dtype, rows, n, bpr, stream);
        case PLLM_TYPE_IQ1_M: return launch_fmt<IQ1Mm>(image, stride, w, y, y_dtype, rows, n, bpr, stream);
        default: return PLLM_ERR_UNSUPPORTED;
    }
}

}  // namespace pllm
