// FP8 x FP8 block-scaled matmul on the matrix cores' native OCP-FP8 path:
//     y[t, r] = sum over 128-wide K blocks kb of  a_s[t, kb] * b_s[r / 128, kb] * sum_{c in kb} f32(a[t, c]) * f32(b[r, c])
// with E4M3 codes on both sides (activations as written by the 128-wide activation quantizer, weights
// with their 128 x 128 block scales) and float32 accumulation.
//
// A workgroup of four waves (2 x 2) owns a 128 x 128 output tile and walks K one scale block (128
// codes) at a time.  Codes need no decoding: 16-byte global loads go to registers one step ahead and
// from there into a double-buffered LDS tile (rows padded to 144 bytes: 16-byte reads of 32 rows at
// the same offset never share a bank).  Every wave runs v_mfma_scale_f32_32x32x64_f8f6f4 (both operands
// E4M3, unit block scales) on its 64 x 64 sub-tile: two K halves of 64 into a fresh accumulator, which is then scaled
// into the running sums with the product of the row's activation scale and the block's weight
// scale.  Which code of a 64-chunk sits in which byte of a lane's operand does not matter as long
// as both operands agree: lanes 0..31 take bytes [0, 32) and lanes 32..63 bytes [32, 64) of the
// chunk on both sides.
#include <algorithm>

#include "block_mfma.h"
#include "pllm_device.h"
#include "pllm_internal.h"

namespace pllm {
namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kTile = 128;                // rows of both operands per workgroup tile
constexpr int kStep = 128;                // codes along K per step = one scale block
constexpr int kRow = kStep + 16;          // LDS row stride in bytes

__device__ __forceinline__ v8i operand(const unsigned char* p) {
    const uint4 lo = *reinterpret_cast<const uint4*>(p);
    const uint4 hi = *reinterpret_cast<const uint4*>(p + 16);
    v8i r;
    r[0] = static_cast<int>(lo.x); r[1] = static_cast<int>(lo.y); r[2] = static_cast<int>(lo.z); r[3] = static_cast<int>(lo.w);
    r[4] = static_cast<int>(hi.x); r[5] = static_cast<int>(hi.y); r[6] = static_cast<int>(hi.z); r[7] = static_cast<int>(hi.w);
    return r;
}

// both operands E4M3 (format selectors 0), both block scales 2^0 (E8M0 code 127)
__device__ __forceinline__ floatx16 mfma_e4m3(const v8i& a, const v8i& b, const floatx16& c) {
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 127, 0, 127);
}

// Workgroups [0, full_tiles) take whole tiles (tile = its index, column tiles fastest) and store scaled results into y.
// Workgroup full_tiles + r takes K steps [slice * per, (slice + 1) * per) of tile full_tiles + r / slices, slice = r % slices, and
// stores its float32 sums into partial[r][128][128]: the tiles that would occupy a fraction of the machine for a full round of
// K are cut along K (block scales are per K step, so every slice's sums are final values) and added in slice order afterwards.
__global__ __launch_bounds__(256, 2) void fp8_gemm_kernel(
    const uint8_t* __restrict__ a, const float* __restrict__ a_s, const uint8_t* __restrict__ b, const float* __restrict__ b_s,
    void* __restrict__ y, int y_dtype, int rows, int n, int k, int tiles_n, int full_tiles, int slices, int per, float* __restrict__ partial) {
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char* a_tile = smem;                                         // [2][kTile * kRow]
    unsigned char* b_tile = smem + 2 * kTile * kRow;                      // [2][kTile * kRow]
    float* a_scale = reinterpret_cast<float*>(smem + 4 * kTile * kRow);   // [2][kTile]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int wg = blockIdx.x;
    const bool whole = wg < full_tiles;
    const int rest = wg - full_tiles;
    const int tile = whole ? wg : full_tiles + rest / slices;
    const int n0 = (tile % tiles_n) * kTile, t0 = (tile / tiles_n) * kTile;
    const int steps = k / kStep;                                          // row pitch of the scale tables
    const int s_begin = whole ? 0 : (rest % slices) * per;
    const int s_end = whole ? steps : min(steps, s_begin + per);

    // staging: piece q = tid + 256 i is bytes [16 (q % 8), +16) of tile row q / 8
    const int prow = tid >> 3, pcol = 16 * (tid & 7);
    // (named variables, not arrays: indexed through the lambdas below, arrays end up in scratch memory)
    auto arow = [&](int i) { return a + static_cast<size_t>(min(t0 + prow + 32 * i, rows - 1)) * k + pcol; };
    auto brow = [&](int i) { return b + static_cast<size_t>(min(n0 + prow + 32 * i, n - 1)) * k + pcol; };
    const uint8_t* const as0 = arow(0); const uint8_t* const as1 = arow(1); const uint8_t* const as2 = arow(2); const uint8_t* const as3 = arow(3);
    const uint8_t* const bs0 = brow(0); const uint8_t* const bs1 = brow(1); const uint8_t* const bs2 = brow(2); const uint8_t* const bs3 = brow(3);
    const float* as_src = a_s + static_cast<size_t>(min(t0 + (tid & 127), rows - 1)) * steps;
    // the wave's 64 weight rows lie inside one 128-row scale block
    const float* bs_src = b_s + static_cast<size_t>(min(n0 + wn * 64, n - 1) >> 7) * steps;

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    uint4 ra0, ra1, ra2, ra3, rb0, rb1, rb2, rb3;
    float rs = 0.0f, rws = 0.0f;
    // the step's codes and both scales: everything a step needs from memory is requested one step ahead (loads return in
    // order, so a scale asked for inside the step would arrive behind the next step's codes)
    auto fetch = [&](int s) {
        const size_t off = static_cast<size_t>(s) * kStep;
        rws = bs_src[s];
        ra0 = *reinterpret_cast<const uint4*>(as0 + off); ra1 = *reinterpret_cast<const uint4*>(as1 + off);
        ra2 = *reinterpret_cast<const uint4*>(as2 + off); ra3 = *reinterpret_cast<const uint4*>(as3 + off);
        rb0 = *reinterpret_cast<const uint4*>(bs0 + off); rb1 = *reinterpret_cast<const uint4*>(bs1 + off);
        rb2 = *reinterpret_cast<const uint4*>(bs2 + off); rb3 = *reinterpret_cast<const uint4*>(bs3 + off);
        if (tid < kTile) rs = as_src[s];
    };
    auto stage = [&](int buf) {
        unsigned char* ad = a_tile + buf * kTile * kRow + prow * kRow + pcol;
        unsigned char* bd = b_tile + buf * kTile * kRow + prow * kRow + pcol;
        *reinterpret_cast<uint4*>(ad) = ra0; *reinterpret_cast<uint4*>(ad + 32 * kRow) = ra1;
        *reinterpret_cast<uint4*>(ad + 64 * kRow) = ra2; *reinterpret_cast<uint4*>(ad + 96 * kRow) = ra3;
        *reinterpret_cast<uint4*>(bd) = rb0; *reinterpret_cast<uint4*>(bd + 32 * kRow) = rb1;
        *reinterpret_cast<uint4*>(bd + 64 * kRow) = rb2; *reinterpret_cast<uint4*>(bd + 96 * kRow) = rb3;
        if (tid < kTile) a_scale[buf * kTile + tid] = rs;
    };

    fetch(s_begin);
    stage(0);
    __syncthreads();
    for (int s = s_begin; s < s_end; ++s) {
        const int buf = (s - s_begin) & 1;
        const float ws = rws;
        fetch(min(s + 1, s_end - 1));        // (no branch around the loads: the last step fetches itself again and drops it)
        const unsigned char* at = a_tile + buf * kTile * kRow + (wm * 64 + (lane & 31)) * kRow + 32 * (lane >> 5);
        const unsigned char* bt = b_tile + buf * kTile * kRow + (wn * 64 + (lane & 31)) * kRow + 32 * (lane >> 5);
        floatx16 c[2][2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const v8i a0 = operand(at + 64 * h), a1 = operand(at + 32 * kRow + 64 * h);
            const v8i b0 = operand(bt + 64 * h), b1 = operand(bt + 32 * kRow + 64 * h);
            if (h == 0) {
                const floatx16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                c[0][0] = mfma_e4m3(a0, b0, zero);
                c[0][1] = mfma_e4m3(a0, b1, zero);
                c[1][0] = mfma_e4m3(a1, b0, zero);
                c[1][1] = mfma_e4m3(a1, b1, zero);
            } else {
                c[0][0] = mfma_e4m3(a0, b0, c[0][0]);
                c[0][1] = mfma_e4m3(a0, b1, c[0][1]);
                c[1][0] = mfma_e4m3(a1, b0, c[1][0]);
                c[1][1] = mfma_e4m3(a1, b1, c[1][1]);
            }
        }
        // D[m][n]: lane holds column n = lane % 32 and rows 8 * (v / 4) + 4 * (lane / 32) + v % 4
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float4 sa = *reinterpret_cast<const float4*>(a_scale + buf * kTile + wm * 64 + mi * 32 + 8 * q + 4 * (lane >> 5));
                const float f0 = sa.x * ws, f1 = sa.y * ws, f2 = sa.z * ws, f3 = sa.w * ws;
#pragma unroll
                for (int ni = 0; ni < 2; ++ni) {
                    acc[mi][ni][4 * q + 0] += c[mi][ni][4 * q + 0] * f0;
                    acc[mi][ni][4 * q + 1] += c[mi][ni][4 * q + 1] * f1;
                    acc[mi][ni][4 * q + 2] += c[mi][ni][4 * q + 2] * f2;
                    acc[mi][ni][4 * q + 3] += c[mi][ni][4 * q + 3] * f3;
                }
            }
        if (s + 1 < s_end) stage(buf ^ 1);
        __syncthreads();
    }
    if (!whole) {                            // raw sums of this slice, [row of the tile][column of the tile]
        float* dst = partial + static_cast<size_t>(rest) * kTile * kTile;
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) {
                const int col = wn * 64 + ni * 32 + (lane & 31);
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = wm * 64 + mi * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                    dst[row * kTile + col] = acc[mi][ni][v];
                }
            }
        return;
    }

#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
            const int col = n0 + wn * 64 + ni * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = t0 + wm * 64 + mi * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (row < rows && col < n) store_any(y, y_dtype, static_cast<size_t>(row) * n + col, acc[mi][ni][v]);
            }
        }
}

// y[t, n] = sum over the slices, in slice order, of the split tiles' partial sums; one workgroup per 1024 elements of a tile
__global__ __launch_bounds__(256) void fp8_gemm_reduce_kernel(const float* __restrict__ partial, void* __restrict__ y, int y_dtype, int rows, int n,
                                                              int tiles_n, int full_tiles, int slices) {
    const int tile = full_tiles + blockIdx.y;
    const int n0 = (tile % tiles_n) * kTile, t0 = (tile / tiles_n) * kTile;
    const int i = (blockIdx.x * 256 + threadIdx.x) * 4;                    // four neighbouring columns of one row
    const int row = i / kTile, col = i % kTile;
    const float* src = partial + static_cast<size_t>(blockIdx.y) * slices * kTile * kTile + i;
    float4 total = *reinterpret_cast<const float4*>(src);
    for (int sl = 1; sl < slices; ++sl) {
        const float4 v = *reinterpret_cast<const float4*>(src + static_cast<size_t>(sl) * kTile * kTile);
        total.x += v.x; total.y += v.y; total.z += v.z; total.w += v.w;
    }
    if (t0 + row >= rows) return;
    const size_t o = static_cast<size_t>(t0 + row) * n + n0 + col;
    if (n0 + col < n) store_any(y, y_dtype, o, total.x);
    if (n0 + col + 1 < n) store_any(y, y_dtype, o + 1, total.y);
    if (n0 + col + 2 < n) store_any(y, y_dtype, o + 2, total.z);
    if (n0 + col + 3 < n) store_any(y, y_dtype, o + 3, total.w);
}

// ------------------------------------------------------------------------------------------------
// More than 128 tokens: a tile of 256 tokens x 128 weight rows per workgroup of eight waves (4 x 2, 64 x 64 each), fed by a
// ring of three LDS stages that direct-to-LDS loads fill two steps ahead: no registers in between, and nothing of a step
// waits for memory that was asked for one step earlier.
//  * Rows lie 128 bytes apart in LDS, unpadded, because a wave instruction of such a load writes one contiguous kilobyte
//    (eight rows); instead the 16-byte pieces of row r are stored at position piece ^ ((r / 2) % 8), which spreads the
//    sixteen rows that one pass of a 16-byte LDS read touches over all banks.
//  * The weights are the matrix instruction's A rows and the tokens its columns, so a lane's sums belong to two tokens
//    and the activation scale is one factor per lane and token block.
//  * The activation scales of four steps are one 16-byte load per token (a 4-byte gather per step asks the memory system
//    for as many separate lines as all the codes of the step), in a ring of two groups.
//  * The scaling of a step's sums runs on the vector ALU while the matrix cores work on the next instructions; the last
//    block of a step is scaled during the first instructions of the next step.
//  * Tile index -> (token tile, row tile): the workgroups that share a block of weight rows are neighbours on one XCD
//    (hardware deals workgroups to the eight XCDs in turn), so the block reaches that L2 once.
// What bounds it: a compute unit keeps a limited number of cache requests outstanding, so bytes per step and unit, not
// the L2's bandwidth, cap the rate at which a tile's codes arrive.
// ------------------------------------------------------------------------------------------------
constexpr int kRingM = 256, kRingN = 128, kRingStages = 3, kRingWaves = 8;
constexpr int kRingA = kRingM * kStep;                        // bytes of a stage's activation codes
constexpr int kRingB = kRingN * kStep;
constexpr int kRingStage = kRingA + kRingB;
constexpr int kRingScales = 2 * kRingM * 16;                   // two groups of four steps' activation scales
constexpr int kRingLoads = 6;                                  // code loads per wave and stage

__device__ __forceinline__ void ring_tile_origin(int tile, int tiles_m, int& t0, int& n0) {
    const int xcd = tile & 7, local = tile >> 3;
    n0 = ((local / tiles_m) * 8 + xcd) * kRingN;
    t0 = (local % tiles_m) * kRingM;
}

// sums of one 32 x 32 block times one factor into the running sums
__device__ __forceinline__ void ring_scale_into(floatx16& acc, const floatx16& c, float f) {
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = __builtin_fmaf(c[v], f, acc[v]);
}

// four neighbouring outputs of one token
__device__ __forceinline__ void ring_store4(void* y, int y_dtype, size_t at, float v0, float v1, float v2, float v3, bool vector_ok, int valid) {
    if (vector_ok && valid == 4) {
        if (y_dtype == PLLM_F32) {
            *reinterpret_cast<float4*>(static_cast<float*>(y) + at) = make_float4(v0, v1, v2, v3);
        } else if (y_dtype == PLLM_BF16) {
            const uint32_t lo = from_float<bf16_t>(v0).bits | (static_cast<uint32_t>(from_float<bf16_t>(v1).bits) << 16);
            const uint32_t hi = from_float<bf16_t>(v2).bits | (static_cast<uint32_t>(from_float<bf16_t>(v3).bits) << 16);
            *reinterpret_cast<uint2*>(static_cast<uint16_t*>(y) + at) = make_uint2(lo, hi);
        } else {
            typedef _Float16 half4 __attribute__((ext_vector_type(4)));
            half4 h = {static_cast<_Float16>(v0), static_cast<_Float16>(v1), static_cast<_Float16>(v2), static_cast<_Float16>(v3)};
            *reinterpret_cast<half4*>(static_cast<_Float16*>(y) + at) = h;
        }
        return;
    }
    if (valid > 0) store_any(y, y_dtype, at, v0);
    if (valid > 1) store_any(y, y_dtype, at + 1, v1);
    if (valid > 2) store_any(y, y_dtype, at + 2, v2);
    if (valid > 3) store_any(y, y_dtype, at + 3, v3);
}

__global__ __launch_bounds__(64 * kRingWaves) void fp8_gemm_ring_kernel(
    const uint8_t* __restrict__ a, const float* __restrict__ a_s, const uint8_t* __restrict__ b, const float* __restrict__ b_s,
    void* __restrict__ y, int y_dtype, int rows, int n, int k, int tiles_m, int full_tiles, int slices, int per, float* __restrict__ partial) {
    extern __shared__ __align__(1024) unsigned char smem[];
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte_ptr)smem));
    constexpr int kScaleOff = kRingStages * kRingStage;
    float* w_scale = reinterpret_cast<float*>(smem + kScaleOff + kRingScales);     // [steps of this workgroup]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wt = wave >> 1, wr = wave & 1;                              // the wave's 64 tokens and 64 weight rows of the tile
    const int wg = blockIdx.x;
    const bool whole = wg < full_tiles;
    const int rest = wg - full_tiles;
    int t0, n0;
    ring_tile_origin(whole ? wg : full_tiles + rest / slices, tiles_m, t0, n0);
    if (n0 >= n) return;                                                  // (row tiles are dealt in eights)
    const int steps = k / kStep;                                          // a multiple of four
    const int s_begin = whole ? 0 : (rest % slices) * per;
    const int s_end = whole ? steps : min(steps, s_begin + per);

    // the weight block's scales of all steps, through ordinary loads, before the first direct-to-LDS load is issued
    for (int i = tid; i < s_end - s_begin; i += 64 * kRingWaves) w_scale[i] = b_s[static_cast<size_t>(n0 >> 7) * steps + s_begin + i];

    // this wave's pieces of a stage: kilobytes 4 wave .. 4 wave + 3 of the token tile and 2 wave, 2 wave + 1 of the weight
    // tile (eight rows each; lane = row in the piece, position in the row); waves 0 .. 3: the scales of 64 tokens
    const int pr = lane >> 3, pc = lane & 7;
    auto piece_src = [&](const uint8_t* base, int row0, int limit, int piece) {
        const int row = 8 * piece + pr;
        return base + static_cast<size_t>(min(row0 + row, limit - 1)) * k + 16 * (pc ^ ((row >> 1) & 7));
    };
    const uint8_t* const as0 = piece_src(a, t0, rows, 4 * wave); const uint8_t* const as1 = piece_src(a, t0, rows, 4 * wave + 1);
    const uint8_t* const as2 = piece_src(a, t0, rows, 4 * wave + 2); const uint8_t* const as3 = piece_src(a, t0, rows, 4 * wave + 3);
    const uint8_t* const bs0 = piece_src(b, n0, n, 2 * wave); const uint8_t* const bs1 = piece_src(b, n0, n, 2 * wave + 1);
    const float* const ss = a_s + static_cast<size_t>(min(t0 + (wave & 3) * 64 + lane, rows - 1)) * steps;
    auto issue = [&](int s, int buf) {
        const size_t off = static_cast<size_t>(s) * kStep;
        const uint32_t base = lds0 + buf * kRingStage;
        lds_dma16(as0 + off, base + (4 * wave) * 1024); lds_dma16(as1 + off, base + (4 * wave + 1) * 1024);
        lds_dma16(as2 + off, base + (4 * wave + 2) * 1024); lds_dma16(as3 + off, base + (4 * wave + 3) * 1024);
        lds_dma16(bs0 + off, base + kRingA + (2 * wave) * 1024); lds_dma16(bs1 + off, base + kRingA + (2 * wave + 1) * 1024);
    };
    // scales of steps 4 g .. 4 g + 3 (g clamped to the last group); always issued AHEAD of a stage's code loads, so that
    // "all but the newest six loads have landed" covers them
    auto issue_scales = [&](int g) {
        if (wave < 4) {
            const int gc = min(g, steps / 4 - 1);
            lds_dma16(ss + 4 * gc, lds0 + kScaleOff + (g & 1) * (kRingM * 16) + wave * 1024);
        }
    };

    floatx16 acc[2][2];                      // [32 weight rows i][32 tokens j]
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // operand reads: lane (row l of a 32-row block, K half hs) takes pieces 4 h + 2 hs and + 1 of its row; the rows of
    // both operands are l plus multiples of 16, so one set of swizzled positions serves all of them
    const int l = lane & 31, hs = lane >> 5, x = (l >> 1) & 7;
    const int o00 = 16 * ((2 * hs) ^ x), o01 = 16 * ((2 * hs + 1) ^ x), o10 = 16 * ((4 + 2 * hs) ^ x), o11 = 16 * ((5 + 2 * hs) ^ x);
    auto operand2 = [&](const unsigned char* row, int lo, int hi) {
        const uint4 u = *reinterpret_cast<const uint4*>(row + lo);
        const uint4 w = *reinterpret_cast<const uint4*>(row + hi);
        v8i r;
        r[0] = static_cast<int>(u.x); r[1] = static_cast<int>(u.y); r[2] = static_cast<int>(u.z); r[3] = static_cast<int>(u.w);
        r[4] = static_cast<int>(w.x); r[5] = static_cast<int>(w.y); r[6] = static_cast<int>(w.z); r[7] = static_cast<int>(w.w);
        return r;
    };
    const floatx16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

    issue_scales(s_begin >> 2);
    issue_scales((s_begin >> 2) + 1);
    issue(s_begin, 0);
    issue(min(s_begin + 1, s_end - 1), 1);
    issue(min(s_begin + 2, s_end - 1), 2);
    wait_vm<2 * kRingLoads>();               // the first stage (and the scales, which are older)
    __syncthreads();
    // The loop is cut in the middle of a step: the K half h = 0 of a step's operands is read during the step before, so the
    // matrix instructions of a step start at once; the one barrier per step sits behind the first four of them, which keep the
    // matrix cores busy while the waves meet, and the second half's operands are in registers before it.
    const unsigned char* tk = smem + (wt * 64 + l) * kStep;
    const unsigned char* wg_rows = smem + kRingA + (wr * 64 + l) * kStep;
    v8i t0h0 = operand2(tk, o00, o01), t1h0 = operand2(tk + 32 * kStep, o00, o01);
    v8i w0h0 = operand2(wg_rows, o00, o01), w1h0 = operand2(wg_rows + 32 * kStep, o00, o01);
    int buf = 0;
    floatx16 c11 = zero;                     // weight rows 32 .. 63 x tokens 32 .. 63 of the previous step, not yet scaled
    float late_f = 0.0f;
    for (int s = s_begin; s < s_end; ++s) {
        const float* tok_scale = reinterpret_cast<const float*>(smem + kScaleOff + ((s >> 2) & 1) * (kRingM * 16)) + (s & 3);
        const float ws = w_scale[s - s_begin];
        const float f0 = tok_scale[4 * (wt * 64 + l)] * ws, f1 = tok_scale[4 * (wt * 64 + 32 + l)] * ws;
        const v8i t0h1 = operand2(tk, o10, o11), t1h1 = operand2(tk + 32 * kStep, o10, o11);
        const v8i w0h1 = operand2(wg_rows, o10, o11), w1h1 = operand2(wg_rows + 32 * kStep, o10, o11);
        floatx16 c00 = mfma_e4m3(w0h0, t0h0, zero);
        floatx16 c01 = mfma_e4m3(w0h0, t1h0, zero);
        floatx16 c10 = mfma_e4m3(w1h0, t0h0, zero);
        ring_scale_into(acc[1][1], c11, late_f);
        c11 = mfma_e4m3(w1h0, t1h0, zero);
        asm volatile("" : "+v"(c00), "+v"(c01), "+v"(c10), "+v"(c11));   // the four instructions above are issued before the wave waits

        wait_vm<kRingLoads>();               // this wave's loads of stage s + 1 have landed (stage s + 2 may be on its way) ...
        __syncthreads();                     // ... and everybody's; every read of stage s has returned
        if ((s & 3) == 0) issue_scales((s >> 2) + 1);
        issue(min(s + 3, s_end - 1), buf);   // (no branch around the loads: past the end a step is fetched again and dropped)
        buf = buf == 2 ? 0 : buf + 1;
        tk = smem + buf * kRingStage + (wt * 64 + l) * kStep;
        wg_rows = smem + buf * kRingStage + kRingA + (wr * 64 + l) * kStep;
        t0h0 = operand2(tk, o00, o01); t1h0 = operand2(tk + 32 * kStep, o00, o01);
        w0h0 = operand2(wg_rows, o00, o01); w1h0 = operand2(wg_rows + 32 * kStep, o00, o01);

        c00 = mfma_e4m3(w0h1, t0h1, c00);
        c01 = mfma_e4m3(w0h1, t1h1, c01);
        c10 = mfma_e4m3(w1h1, t0h1, c10);
        c11 = mfma_e4m3(w1h1, t1h1, c11);
        ring_scale_into(acc[0][0], c00, f0);
        ring_scale_into(acc[0][1], c01, f1);
        ring_scale_into(acc[1][0], c10, f0);
        late_f = f1;
    }
    ring_scale_into(acc[1][1], c11, late_f);
    wait_vm<0>();                            // the dropped loads past the end: nothing may arrive in LDS after the workgroup has left

    // D[m][n]: lane holds column n = token l of block j and rows m = weight rows 8 * (v / 4) + 4 * hs + v % 4 of block i
    float* const dst = whole ? nullptr : partial + static_cast<size_t>(rest) * kRingM * kRingN;   // a slice's sums: [token of the tile][row of the tile]
    const bool vector_ok = (n & 3) == 0 && !(y_dtype & 0x100);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int tok = wt * 64 + j * 32 + l;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int col = wr * 64 + i * 32 + 8 * q + 4 * hs;
                const float v0 = acc[i][j][4 * q], v1 = acc[i][j][4 * q + 1], v2 = acc[i][j][4 * q + 2], v3 = acc[i][j][4 * q + 3];
                if (!whole) *reinterpret_cast<float4*>(dst + tok * kRingN + col) = make_float4(v0, v1, v2, v3);
                else if (t0 + tok < rows) ring_store4(y, y_dtype, static_cast<size_t>(t0 + tok) * n + n0 + col, v0, v1, v2, v3, vector_ok, min(4, n - n0 - col));
            }
    }
}

// the split tiles of the ring kernel: sums over the slices in slice order; one workgroup per 1024 elements of a tile
__global__ __launch_bounds__(256) void fp8_gemm_ring_reduce_kernel(const float* __restrict__ partial, void* __restrict__ y, int y_dtype, int rows, int n,
                                                                   int tiles_m, int full_tiles, int slices) {
    int t0, n0;
    ring_tile_origin(full_tiles + blockIdx.y, tiles_m, t0, n0);
    const int i = (blockIdx.x * 256 + threadIdx.x) * 4;                    // four neighbouring columns of one row
    const int row = i / kRingN, col = i % kRingN;
    const float* src = partial + static_cast<size_t>(blockIdx.y) * slices * kRingM * kRingN + i;
    float4 total = *reinterpret_cast<const float4*>(src);
    for (int sl = 1; sl < slices; ++sl) {
        const float4 v = *reinterpret_cast<const float4*>(src + static_cast<size_t>(sl) * kRingM * kRingN);
        total.x += v.x; total.y += v.y; total.z += v.z; total.w += v.w;
    }
    if (t0 + row >= rows || n0 >= n) return;
    const size_t o = static_cast<size_t>(t0 + row) * n + n0 + col;
    if (n0 + col < n) store_any(y, y_dtype, o, total.x);
    if (n0 + col + 1 < n) store_any(y, y_dtype, o + 1, total.y);
    if (n0 + col + 2 < n) store_any(y, y_dtype, o + 2, total.z);
    if (n0 + col + 3 < n) store_any(y, y_dtype, o + 3, total.w);
}


struct Fp8GemmPlan { bool ring; int tiles_m, tiles_n, tiles, full_tiles, slices, per; size_t partial_bytes; };

// Whole rounds of tiles run unsplit; the left-over tiles (all tiles, when there is less than one round) are cut along K so that
// their workgroups fill the machine about once, as long as the partial sums stay under 64 MB and a slice keeps two steps (five
// in the ring kernel).
// More than 128 tokens take the ring kernel's 256 x 128 tiles (one workgroup per compute unit, row tiles dealt in eights).
Fp8GemmPlan plan_fp8_gemm(int rows, int k, int n, bool allow_ring) {
    Fp8GemmPlan p;
    p.ring = allow_ring && rows > kTile && (k / kStep) % 4 == 0;       // (scales of four steps are one load)
    const int tile_m = p.ring ? kRingM : kTile;
    p.tiles_m = (rows + tile_m - 1) / tile_m;
    p.tiles_n = (n + kTile - 1) / kTile;
    if (p.ring) p.tiles_n = (p.tiles_n + 7) / 8 * 8;
    p.tiles = p.tiles_n * p.tiles_m;
    const int resident = (p.ring ? 1 : 2) * compute_units();
    const int steps = k / kStep;
    const size_t tile_bytes = static_cast<size_t>(tile_m) * kTile * sizeof(float);
    p.full_tiles = (p.tiles / resident) * resident;
    const int rem = p.tiles - p.full_tiles;
    p.slices = 1;
    p.per = steps;
    if (rem > 0 && rem * 2 <= resident) {
        // (the ring kernel's slices keep five steps: fewer, longer slices move fewer partial sums; 78 -> 73 us at 17408x5120, T=512)
        int slices = std::min(resident / rem, std::max(1, steps / (p.ring ? 5 : 2)));
        slices = std::min<int>(slices, static_cast<int>((static_cast<size_t>(64) << 20) / (static_cast<size_t>(rem) * tile_bytes)));
        if (slices >= 2) {
            p.per = (steps + slices - 1) / slices;
            p.slices = (steps + p.per - 1) / p.per;
        }
    }
    if (p.slices == 1) p.full_tiles = p.tiles;
    p.partial_bytes = p.slices > 1 ? static_cast<size_t>(p.tiles - p.full_tiles) * p.slices * tile_bytes : 0;
    return p;
}

}  // namespace

size_t fp8_gemm_native_workspace_bytes(int rows, int k, int n) {
    if (k % kStep != 0 || k <= 0 || rows <= 0 || n <= 0) return 0;
    return std::max(plan_fp8_gemm(rows, k, n, true).partial_bytes, plan_fp8_gemm(rows, k, n, false).partial_bytes);
}

int fp8_gemm_native(const uint8_t* a, const float* a_s, const uint8_t* b, const float* b_s, void* y, int y_dtype,
                    int rows, int k, int n, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    if (k % kStep != 0 || k <= 0) return PLLM_ERR_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15u) return PLLM_ERR_UNSUPPORTED;
    const size_t steps_bytes = static_cast<size_t>(k / kStep) * sizeof(float);
    const bool ring_ok = (reinterpret_cast<uintptr_t>(a_s) & 15u) == 0 && static_cast<size_t>(kRingStages) * kRingStage + kRingScales + steps_bytes <= 160 * 1024;
    Fp8GemmPlan p = plan_fp8_gemm(rows, k, n, ring_ok);
    const size_t ring_smem = static_cast<size_t>(kRingStages) * kRingStage + kRingScales + static_cast<size_t>(k / kStep) * sizeof(float);
    const size_t smem = p.ring ? ring_smem : static_cast<size_t>(4) * kTile * kRow + 2 * kTile * sizeof(float);
    const void* kern = p.ring ? reinterpret_cast<const void*>(fp8_gemm_ring_kernel) : reinterpret_cast<const void*>(fp8_gemm_kernel);
    if (hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem)) != hipSuccess) return PLLM_ERR_UNSUPPORTED;
    if (p.slices > 1 && (!workspace || workspace_bytes < p.partial_bytes)) {  // no room for partial sums: every tile whole
        p.slices = 1;
        p.per = k / kStep;
        p.full_tiles = p.tiles;
    }
    const int rem = p.tiles - p.full_tiles;
    const dim3 grid(p.full_tiles + rem * p.slices);
    if (p.ring) {
        hipLaunchKernelGGL(fp8_gemm_ring_kernel, grid, dim3(64 * kRingWaves), smem, stream, a, a_s, b, b_s, y, y_dtype, rows, n, k, p.tiles_m,
                           p.full_tiles, p.slices, p.per, static_cast<float*>(workspace));
        if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
        if (rem > 0)
            hipLaunchKernelGGL(fp8_gemm_ring_reduce_kernel, dim3(kRingM * kRingN / 1024, rem), dim3(256), 0, stream, static_cast<const float*>(workspace),
                               y, y_dtype, rows, n, p.tiles_m, p.full_tiles, p.slices);
        return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(fp8_gemm_kernel, grid, dim3(256), smem, stream, a, a_s, b, b_s, y, y_dtype, rows, n, k,
                       p.tiles_n, p.full_tiles, p.slices, p.per, static_cast<float*>(workspace));
    if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
    if (rem > 0)
        hipLaunchKernelGGL(fp8_gemm_reduce_kernel, dim3(kTile * kTile / 1024, rem), dim3(256), 0, stream, static_cast<const float*>(workspace), y,
                           y_dtype, rows, n, p.tiles_n, p.full_tiles, p.slices);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

}  // namespace pllm
