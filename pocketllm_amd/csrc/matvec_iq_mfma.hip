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
    static constexpr int kHoldBlocks = 3;                      // block indices whose activation side a wave may keep in registers
    struct Regs { uint4 q; uint32_t d; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int s) {
        r.q = load16_a2(blk + 2 + 16 * s);
        r.d = *reinterpret_cast<const uint16_t*>(blk);
    }
    // the same share from a copy of the block in LDS (2-byte aligned there as in memory): five
    // aligned dwords, shifted down by 16 bits where the share starts in the middle of a dword
    static __device__ __forceinline__ void load_lds(Regs& r, const unsigned char* base, int off, int s) {   // base 4-byte aligned
        const int a = off + 2 + 16 * s;
        const uint32_t* p = reinterpret_cast<const uint32_t*>(base + (a & ~3));
        const uint32_t sh = (static_cast<uint32_t>(a) & 2u) << 3;
        const uint32_t d0 = p[0], d1 = p[1], d2 = p[2], d3 = p[3], d4 = p[4];
        r.q = make_uint4(__builtin_amdgcn_alignbit(d1, d0, sh), __builtin_amdgcn_alignbit(d2, d1, sh),
                         __builtin_amdgcn_alignbit(d3, d2, sh), __builtin_amdgcn_alignbit(d4, d3, sh));
        r.d = *reinterpret_cast<const uint16_t*>(base + off);
    }
    static __device__ __forceinline__ void stage_tables(unsigned char* lds) { IQ2XXS::stage_tables(lds); }
    static __device__ __forceinline__ void dma_tables(uint32_t lds_base, int wave, int lane);
    static __device__ __forceinline__ void a_map(AMap<kSlots>& am, int col, int ks, int kpad, int zero_off) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int g = 2 * ks + (t >> 1);
            const bool active = (col >> 1) == g;
            am.off[t] = active ? ((col & 1) ? kpad : 0) + 32 * g + 16 * (t & 1) : zero_off;
            am.step[t] = active ? 256 : 0;
        }
    }
    // what a block index contributes from the activation side: the lane's A operands and its two
    // groups' scales; a wave that meets the same block index in tile after tile keeps them in registers
    struct Held { uint4 a[4]; float xs0, xs1; };
    static __device__ __forceinline__ void hold(Held& h, int s, int b, const unsigned char* smem, const AMap<kSlots>& am, const StagedX& sx) {
#pragma unroll
        for (int t = 0; t < 4; ++t) h.a[t] = *reinterpret_cast<const uint4*>(smem + am.off[t] + b * am.step[t]);
        const float4 g2 = *reinterpret_cast<const float4*>(sx.gs + b * 8 + 2 * s);   // {xs0 / 254, sum0, xs1 / 254, sum1}
        h.xs0 = g2.x; h.xs1 = g2.z;
    }
    static __device__ __forceinline__ float block_held(const Regs& r, int, int, const Held& h, const unsigned char*, const AMap<kSlots>&,
                                                       const unsigned char* tables) {
        const uint2* grid = reinterpret_cast<const uint2*>(tables);
        const uint2* sign = grid + 256;
        v4i c = {0, 0, 0, 0}, cm = {0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t ids = (t < 2) ? r.q.x : r.q.z, aux = (t < 2) ? r.q.y : r.q.w;
            const int e = 2 * (t & 1);                                         // grid entries e and e + 1 of the sub-block
            const uint2 g0 = grid[(ids >> (8 * e)) & 0xffu], m0 = sign[(aux >> (7 * e)) & 127u];
            const uint2 g1 = grid[(ids >> (8 * e + 8)) & 0xffu], m1 = sign[(aux >> (7 * e + 7)) & 127u];
            const v4i av = as_v4i(h.a[t].x, h.a[t].y, h.a[t].z, h.a[t].w);
            c = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, as_v4i(g0.x ^ m0.x, g0.y ^ m0.y, g1.x ^ m1.x, g1.y ^ m1.y), c, 0, 0, 0);
            cm = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, as_v4i(m0.x, m0.y, m1.x, m1.y), cm, 0, 0, 0);
        }
        const float v0 = static_cast<float>(__mul24(c.x - cm.x, 254) + (c.y - cm.y));   // group 2 s: 254 * high term + low term
        const float v1 = static_cast<float>(__mul24(c.z - cm.z, 254) + (c.w - cm.w));   // group 2 s + 1
        const float ls0 = static_cast<float>(2 * (r.q.y >> 28) + 1), ls1 = static_cast<float>(2 * (r.q.w >> 28) + 1);
        return 0.125f * f16_bits_to_float(r.d) * (ls0 * h.xs0 * v0 + ls1 * h.xs1 * v1);
    }
    static __device__ __forceinline__ float block(const Regs& r, int s, int b, const unsigned char* smem, const AMap<kSlots>& am,
                                                  const StagedX& sx, const unsigned char* tables) {
        Held h;
        hold(h, s, b, smem, am, sx);
        return block_held(r, s, b, h, smem, am, tables);
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
    static constexpr int kHoldBlocks = 0;                      // (its held operands would cost a workgroup per compute unit)
    struct Regs { uint2 qs; uint32_t qh; uint2 sc; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int s) {
        r.qs = *reinterpret_cast<const uint2*>(blk + 8 * s);                   // blocks are 8-byte aligned
        r.qh = *reinterpret_cast<const uint32_t*>(blk + 32 + 4 * s);
        r.sc = *reinterpret_cast<const uint2*>(blk + 48);
    }
    static __device__ __forceinline__ void load_lds(Regs& r, const unsigned char* base, int off, int s) { load(r, base + off, s); }
    static __device__ __forceinline__ void stage_tables(unsigned char* lds) {
        copy_to_lds(lds, reinterpret_cast<const unsigned char*>(PLLM_IQ1_DELTA_CODES.v), kTableBytes);
    }
    static __device__ __forceinline__ void dma_tables(uint32_t lds_base, int wave, int lane);
    static __device__ __forceinline__ void a_map(AMap<kSlots>& am, int col, int ks, int kpad, int zero_off) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const bool active = col == 4 * ks + t;
            am.off[t] = active ? 16 * col : zero_off;
            am.off[4 + t] = active ? kpad + 16 * col : zero_off;
            am.step[t] = am.step[4 + t] = active ? 256 : 0;
        }
    }
    // activation side of a block index (see IQ2XXSm::Held): the high-term A operands, the groups'
    // scales (already over 8) and the 16-value sums; the low-term operands are read when needed
    struct Held { uint4 a[4]; float x0, x1; float4 s16; };
    static __device__ __forceinline__ void hold(Held& h, int s, int b, const unsigned char* smem, const AMap<kSlots>& am, const StagedX& sx) {
#pragma unroll
        for (int t = 0; t < 4; ++t) h.a[t] = *reinterpret_cast<const uint4*>(smem + am.off[t] + b * am.step[t]);
        const float4 g2 = *reinterpret_cast<const float4*>(sx.gs + b * 8 + 2 * s);   // {xs0 / 254, sum0, xs1 / 254, sum1}
        h.x0 = 0.125f * g2.x; h.x1 = 0.125f * g2.z;
        h.s16 = *reinterpret_cast<const float4*>(sx.sum16 + b * 16 + 4 * s);
    }
    static __device__ __forceinline__ float block_held(const Regs& r, int s, int b, const Held& h, const unsigned char* smem,
                                                       const AMap<kSlots>& am, const unsigned char* tables) {
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
            const uint4 al = *reinterpret_cast<const uint4*>(smem + am.off[4 + t] + b * am.step[4 + t]);
            ch = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(h.a[t].x, h.a[t].y, h.a[t].z, h.a[t].w), bw, ch, 0, 0, 0);
            cl = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(al.x, al.y, al.z, al.w), bw, cl, 0, 0, 0);
        }
        const float ls0 = static_cast<float>(2 * (word & 7u) + 1), ls1 = static_cast<float>(2 * ((word >> 3) & 7u) + 1);
        const float ls2 = static_cast<float>(2 * ((word >> 6) & 7u) + 1), ls3 = static_cast<float>(2 * ((word >> 9) & 7u) + 1);
        const float v = ls0 * (h.x0 * static_cast<float>(__mul24(ch.x, 254) + cl.x) - h.s16.x) + ls1 * (h.x0 * static_cast<float>(__mul24(ch.y, 254) + cl.y) - h.s16.y) +
                        ls2 * (h.x1 * static_cast<float>(__mul24(ch.z, 254) + cl.z) - h.s16.z) + ls3 * (h.x1 * static_cast<float>(__mul24(ch.w, 254) + cl.w) - h.s16.w);
        return f16_bits_to_float(dbits) * v;
    }
    static __device__ __forceinline__ float block(const Regs& r, int s, int b, const unsigned char* smem, const AMap<kSlots>& am,
                                                  const StagedX& sx, const unsigned char* tables) {
        Held h;
        hold(h, s, b, smem, am, sx);
        return block_held(r, s, b, h, smem, am, tables);
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

// ------------------------------------------------------------------------------------------------
// Streamed form.  The rows of consecutive tiles are one contiguous run of memory, but a lane's share
// of a block is 16 + 2 bytes at a 2-byte-aligned address and the 16 rows of a tile lie a whole row
// apart: loading shares straight into registers asks the memory system for many small unaligned
// pieces.  Here the workgroup copies a chunk of `tiles_per_chunk` whole tiles into LDS with
// direct-to-LDS loads (global_load_lds_dwordx4: every wave instruction moves 1 KB that is contiguous
// in memory and in LDS, aligned, no registers involved) and the waves pick their shares out of LDS.
// Workgroups walk chunks blockIdx.x, blockIdx.x + gridDim.x, ...; several share a compute unit, so
// some multiply while others wait for their chunk.  Needs n % 16 == 0 and a 16-byte aligned matrix.
// ------------------------------------------------------------------------------------------------
typedef __attribute__((address_space(3))) unsigned char* lds_byte_ptr;

// 16 bytes per lane from memory to LDS[lds_base + 16 * lane] (lds_base wave-uniform), no registers in
// between.  Issued through inline assembly so that the compiler does not put a wait for it in front
// of every later LDS read: the kernel waits for its chunks itself (wait_vm).
__device__ __forceinline__ void lds_dma16(const void* src, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(lds_base) : "memory", "m0");
}
template <int N> __device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory"); }
// until at most `newest` of this wave's memory operations are outstanding (they complete in order)
__device__ __forceinline__ void wait_vm_all_but(int newest) {
    switch (newest) {
        case 1: wait_vm<1>(); break;
        case 2: wait_vm<2>(); break;
        case 3: wait_vm<3>(); break;
        case 4: wait_vm<4>(); break;
        default: wait_vm<0>(); break;
    }
}
// the wave's share of a workgroup-wide copy of `bytes` (a multiple of 16) to LDS address lds_base:
// 1 KB pieces wave, wave + 8, ...; returns the number of instructions issued
__device__ __forceinline__ int dma_share(const unsigned char* src, uint32_t lds_base, int bytes, int wave, int lane) {
    int issued = 0;
    for (int o = wave * 1024; o < bytes; o += kWaves * 1024) {
        if (o + lane * 16 < bytes) lds_dma16(src + o + lane * 16, lds_base + o);
        ++issued;
    }
    return issued;
}

__device__ __forceinline__ void IQ2XXSm::dma_tables(uint32_t lds_base, int wave, int lane) {
    dma_share(reinterpret_cast<const unsigned char*>(PLLM_IQ2XXS_GRID), lds_base, 2048, wave, lane);
    dma_share(reinterpret_cast<const unsigned char*>(PLLM_IQ2XXS_SIGN_MASKS.v), lds_base + 2048, 1024, wave, lane);
}
__device__ __forceinline__ void IQ1Mm::dma_tables(uint32_t lds_base, int wave, int lane) {
    dma_share(reinterpret_cast<const unsigned char*>(PLLM_IQ1_DELTA_CODES.v), lds_base, kTableBytes, wave, lane);
}

constexpr int kChunkBudget = 28 * 1024;

// NB > 0: a wave meets at most NB block indices (part, part + split, ...) and keeps their activation
// side in registers across all its chunks; NB == 0: any number, read from LDS every time.
template <typename FMT, int NB>
__global__ __launch_bounds__(64 * kWaves) void iq_stream_matvec_kernel(
    const unsigned char* __restrict__ image, size_t image_stride, const uint8_t* __restrict__ w,
    void* __restrict__ y, int y_dtype, int n, int bpr, int split, int chunks, int chunk_off, int chunk_stride) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    const StagedX sx = carve_staged_x(smem, kpad);
    const int zero_off = image_bytes;                                        // 16 zero bytes
    const int table_off = image_bytes + 16;
    const unsigned char* tables = smem + table_off;
    float* partial = reinterpret_cast<float*>(smem + table_off + FMT::kTableBytes);   // [waves][16]
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte_ptr)smem));

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int col = lane & 15, ks = lane >> 4;
    const int tiles_per_chunk = kWaves / split;
    const int tile_in_chunk = wave / split, part = wave % split;
    const int row_bytes = bpr * FMT::kBlockBytes;
    const int chunk_rows = tiles_per_chunk * kRowsPerTile;

    // activation image, codebooks and the first chunk: all in flight together
    dma_share(image + static_cast<size_t>(blockIdx.y) * image_stride, lds0, image_bytes, wave, lane);
    FMT::dma_tables(lds0 + table_off, wave, lane);
    if (tid < 4) reinterpret_cast<uint32_t*>(smem + zero_off)[tid] = 0;
    AMap<FMT::kSlots> am;
    FMT::a_map(am, col, ks, kpad, zero_off);

    int c = blockIdx.x, buf = 0;
    dma_share(w + static_cast<size_t>(c) * chunk_rows * row_bytes, lds0 + chunk_off, min(chunk_rows, n - c * chunk_rows) * row_bytes, wave, lane);
    typename FMT::Held held[NB > 0 ? NB : 1];
    bool holding = false;
    while (c < chunks) {
        const int row0 = c * chunk_rows;
        const int valid_rows = min(chunk_rows, n - row0);                    // a multiple of 16
        // the next chunk goes to the other buffer while this one is multiplied
        const int cn = c + gridDim.x;
        int newest = 0;
        if (cn < chunks)
            newest = dma_share(w + static_cast<size_t>(cn) * chunk_rows * row_bytes, lds0 + chunk_off + (buf ^ 1) * chunk_stride,
                               min(chunk_rows, n - cn * chunk_rows) * row_bytes, wave, lane);
        wait_vm_all_but(newest);             // this wave's pieces of chunk c (and of the image and tables) have landed ...
        __syncthreads();                     // ... and everybody else's too
        if (NB > 0 && !holding) {
#pragma unroll
            for (int i = 0; i < NB; ++i) FMT::hold(held[i], ks, min(part + i * split, bpr - 1), smem, am, sx);
            holding = true;
        }

        const unsigned char* chunk = smem + chunk_off + buf * chunk_stride;
        float acc = 0.0f;
        if (tile_in_chunk * kRowsPerTile < valid_rows) {                     // wave-uniform
            const int row_off = (tile_in_chunk * kRowsPerTile + col) * row_bytes;
            if (NB > 0) {
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    const int b = part + i * split;
                    if (b < bpr) {                                           // wave-uniform
                        typename FMT::Regs regs;
                        FMT::load_lds(regs, chunk, row_off + b * FMT::kBlockBytes, ks);
                        acc += FMT::block_held(regs, ks, b, held[i], smem, am, tables);
                    }
                }
            } else {
                for (int b = part; b < bpr; b += split) {
                    typename FMT::Regs regs;
                    FMT::load_lds(regs, chunk, row_off + b * FMT::kBlockBytes, ks);
                    acc += FMT::block(regs, ks, b, smem, am, sx, tables);
                }
            }
            acc += __shfl_xor(acc, 16, 64);
            acc += __shfl_xor(acc, 32, 64);
            if (split == 1) {
                if (ks == 0) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + row0 + tile_in_chunk * kRowsPerTile + col, acc);
            } else if (ks == 0) {
                partial[wave * kRowsPerTile + col] = acc;
            }
        }
        __syncthreads();                     // this buffer may be overwritten, the partial sums are complete
        if (split > 1 && tid < valid_rows) {
            const int t = tid / kRowsPerTile, cc = tid % kRowsPerTile;
            float total = 0.0f;
            for (int v = 0; v < split; ++v) total += partial[(t * split + v) * kRowsPerTile + cc];
            store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + row0 + tid, total);
        }
        c = cn;
        buf ^= 1;
    }
}

// 0 when the streamed form does not apply
template <typename FMT>
int stream_split(const uint8_t* w, int n, int bpr) {
    if (n % kRowsPerTile != 0 || (reinterpret_cast<uintptr_t>(w) & 15u)) return 0;
    const int tile_bytes = kRowsPerTile * bpr * FMT::kBlockBytes;
    // the most waves per tile first (smallest chunk) that leaves every wave at least three blocks
    for (int split = kWaves; split >= 1; split /= 2)
        if ((split == 1 || bpr >= 3 * split) && (kWaves / split) * tile_bytes <= kChunkBudget) return split;
    return 0;
}

template <typename FMT, int NB>
int launch_stream_nb(const unsigned char* image, size_t image_stride, const uint8_t* w, void* y, int y_dtype,
                     int rows, int n, int bpr, int split, hipStream_t stream) {
    auto kern = iq_stream_matvec_kernel<FMT, NB>;
    const int tiles_per_chunk = kWaves / split;
    const int chunk_bytes = tiles_per_chunk * kRowsPerTile * bpr * FMT::kBlockBytes;
    const size_t head = staged_x_bytes(bpr * 256) + 16 + FMT::kTableBytes + kWaves * kRowsPerTile * sizeof(float);
    const int chunk_off = static_cast<int>((head + 1023) & ~static_cast<size_t>(1023));
    const int chunk_stride = chunk_bytes + 16;                               // shares are read as aligned dwords: a few bytes past the end
    const size_t smem = static_cast<size_t>(chunk_off) + 2 * chunk_stride;
    if (smem > 160 * 1024) return PLLM_ERR_UNSUPPORTED;
    static size_t attr_smem = 0;
    if (smem > 64 * 1024 && smem > attr_smem) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(smem)) != hipSuccess)
            return PLLM_ERR_UNSUPPORTED;
        attr_smem = smem;
    }
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, 64 * kWaves, smem) != hipSuccess || per_cu < 1) per_cu = 1;
    const int chunks = (n / kRowsPerTile + tiles_per_chunk - 1) / tiles_per_chunk;
    const int resident = per_cu * compute_units();
    int grid = chunks;
    if (chunks > resident) {
        const int rounds = (chunks + resident - 1) / resident;
        grid = (chunks + rounds - 1) / rounds;
    }
    hipLaunchKernelGGL(kern, dim3(grid, rows), dim3(64 * kWaves), smem, stream, image, image_stride, w, y, y_dtype, n, bpr, split, chunks,
                       chunk_off, chunk_stride);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

template <typename FMT>
int launch_stream(const unsigned char* image, size_t image_stride, const uint8_t* w, void* y, int y_dtype,
                  int rows, int n, int bpr, int split, hipStream_t stream) {
    const int per_wave = (bpr + split - 1) / split;                          // block indices a wave meets
    if (FMT::kHoldBlocks >= 2 && per_wave <= 2) return launch_stream_nb<FMT, 2>(image, image_stride, w, y, y_dtype, rows, n, bpr, split, stream);
    if (FMT::kHoldBlocks >= 3 && per_wave == 3) return launch_stream_nb<FMT, 3>(image, image_stride, w, y, y_dtype, rows, n, bpr, split, stream);
    return launch_stream_nb<FMT, 0>(image, image_stride, w, y, y_dtype, rows, n, bpr, split, stream);
}

template <typename FMT>
int launch_fmt(const unsigned char* image, size_t image_stride, const uint8_t* w, void* y, int y_dtype,
               int rows, int n, int bpr, hipStream_t stream) {
    if (const int split = stream_split<FMT>(w, n, bpr)) return launch_stream<FMT>(image, image_stride, w, y, y_dtype, rows, n, bpr, split, stream);
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
