// Decode matvec over raw Q4_K / Q5_K super-blocks (bandwidth-bound, wave64).
//
// A wave owns 16 consecutive output rows and walks their super-blocks; the W waves of a workgroup
// split a row's super-blocks between them (wave w takes blocks w, w + W, ...) and meet in a small
// LDS reduction.  All weight loads of a pass are issued first; while they are in flight the
// workgroup brings the activation image (two int8 terms per value) into LDS: copied from the image
// act_quant.hip wrote, or, for calls of a few rows, quantized from the raw row on the spot.
//
// The integer dots run on the matrix cores.  For one super-block index the wave forms
//     C[m][n] = sum_k A[m][k] * B[k][n],     v_mfma_i32_16x16x64_i8, four of them per block,
// with B = the 4/5-bit codes of the 16 rows (n = row, straight from the 16-byte global loads after
// a nibble split) and A = the activation codes spread over 16 rows m = 2 * group + term, row m
// holding the codes of 32-weight group `group` (term 0 = high int8 term, 1 = low term) and zeros
// elsewhere.  One accumulator tile then holds, for every row, the eight per-group integer dots of
// both terms; the lane that holds C[4s .. 4s+3][n] owns groups 2s and 2s+1 of row n and applies
// their 6-bit scales and mins in float.  Which k sits where inside an MFMA is irrelevant as long
// as A and B agree, and both are built per (lane / 16, byte) from the same positions.
#include "block_mfma.h"
#include "pllm_device.h"
#include "pllm_internal.h"

namespace pllm {
namespace {

constexpr int kRowsPerWg = 16;
constexpr int kMaxWaves = 8;

typedef int v4i __attribute__((ext_vector_type(4)));

__device__ __forceinline__ v4i as_v4i(const uint4& u) {
    v4i r;
    r.x = static_cast<int>(u.x); r.y = static_cast<int>(u.y); r.z = static_cast<int>(u.z); r.w = static_cast<int>(u.w);
    return r;
}

// 16 bytes of a weight matrix.  A plain load on purpose: the header and the code chunks of a block share cache lines, between
// the loads of one lane and between neighbouring waves, and a non-temporal load gives that reuse up (measured: Q4_K 17408x5120
// 14.2 -> 18.7 us).
__device__ __forceinline__ uint4 stream16(const uint8_t* p) {
    return *reinterpret_cast<const uint4*>(p);
}

// Eight 6-bit scales / mins of a K-quant header as bytes: lo word = entries 0..3, hi word = 4..7.
struct K4Scales { uint32_t sc_lo, sc_hi, mn_lo, mn_hi; };
__device__ __forceinline__ K4Scales k4_unpack(const uint4& hdr) {
    const uint32_t u0 = hdr.y, u1 = hdr.z, u2 = hdr.w;
    K4Scales r;
    r.sc_lo = u0 & 0x3f3f3f3fu;
    r.mn_lo = u1 & 0x3f3f3f3fu;
    r.sc_hi = (u2 & 0x0f0f0f0fu) | (((u0 >> 6) & 0x03030303u) << 4);
    r.mn_hi = ((u2 >> 4) & 0x0f0f0f0fu) | (((u1 >> 6) & 0x03030303u) << 4);
    return r;
}

__device__ __forceinline__ uint4 nib_lo(const uint4& q) {
    return make_uint4(q.x & 0x0f0f0f0fu, q.y & 0x0f0f0f0fu, q.z & 0x0f0f0f0fu, q.w & 0x0f0f0f0fu);
}
__device__ __forceinline__ uint4 nib_hi(const uint4& q) {
    return make_uint4((q.x >> 4) & 0x0f0f0f0fu, (q.y >> 4) & 0x0f0f0f0fu, (q.z >> 4) & 0x0f0f0f0fu, (q.w >> 4) & 0x0f0f0f0fu);
}
// bit `bit` of every byte of qh moves to bit 4 of the same byte by one rotation (a rotation only
// wraps bits that the mask drops) and is merged into the nibble codes
__device__ __forceinline__ uint4 fifth_bit(const uint4& w, const uint4& qh, int bit) {
    const uint32_t r = static_cast<uint32_t>(bit + 28) & 31u;
    return make_uint4(w.x | (__builtin_amdgcn_alignbit(qh.x, qh.x, r) & 0x10101010u), w.y | (__builtin_amdgcn_alignbit(qh.y, qh.y, r) & 0x10101010u),
                      w.z | (__builtin_amdgcn_alignbit(qh.z, qh.z, r) & 0x10101010u), w.w | (__builtin_amdgcn_alignbit(qh.w, qh.w, r) & 0x10101010u));
}

// Which 32-weight group MFMA t's k slice ks carries for the two nibble formats, and the float epilogue of the lane that
// holds the integer dots v0, v1 (both activation terms folded: 254 * hi + lo) of groups 2 ks and 2 ks + 1 of its row;
// g2 = {xs0 / 254, sum0, xs1 / 254, sum1} of those groups' activations.
__device__ __forceinline__ int k45_group_of(int t, int ks) { return 4 * (t >> 1) + 2 * (ks >> 1) + (t & 1); }
__device__ __forceinline__ float k45_combine(const uint4& hdr, int ks, float v0, float v1, const float4& g2) {
    const K4Scales sc = k4_unpack(hdr);
    const uint32_t scw = ((ks & 2) ? sc.sc_hi : sc.sc_lo) >> (16 * (ks & 1));
    const uint32_t mnw = ((ks & 2) ? sc.mn_hi : sc.mn_lo) >> (16 * (ks & 1));
    const float d = f16_bits_to_float(hdr.x & 0xffffu);
    const float dmin = f16_bits_to_float(hdr.x >> 16);
    const float s0 = static_cast<float>(scw & 0xffu), s1 = static_cast<float>((scw >> 8) & 0xffu);
    const float m0 = static_cast<float>(mnw & 0xffu), m1 = static_cast<float>((mnw >> 8) & 0xffu);
    // explicit fused multiply-adds: every kernel that calls this rounds the same way, whatever the compiler would contract
    const float pos = __builtin_fmaf(s1 * g2.z, v1, (s0 * g2.x) * v0);
    const float neg = __builtin_fmaf(m1, g2.w, m0 * g2.y);
    return __builtin_fmaf(d, pos, -(dmin * neg));
}

// ------------------------------------------------------------------------------------------------
// Q4_K: 144 B = d(2) dmin(2) scales(12) qs(128).  Lane (n, ks) holds qs[16 ks, +16) and
// qs[64 + 16 ks, +16).  With p = ks >> 1, h = ks & 1 the first chunk carries weights 16h + (0..15)
// of group 2p in its low nibbles and of group 2p+1 in its high nibbles; the second chunk is the
// same for groups 2p+4 and 2p+5.
// Q5_K: 176 B = d dmin scales(12) qh(32) qs(128); same plus qh[16h, +16): bit g of qh byte 16h + t
// is the fifth bit of weight 16h + t of group g.
// ------------------------------------------------------------------------------------------------
struct Q4K {
    static constexpr int kBlockBytes = 144;
    static constexpr int kDepth = 5;                          // blocks in flight per wave that fit 128 registers (four waves per SIMD)
    struct Regs { uint4 hdr; uint4 qa; uint4 qb; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int ks) {
        r.hdr = stream16(blk);
        r.qa = stream16(blk + 16 + 16 * ks);
        r.qb = stream16(blk + 80 + 16 * ks);
    }
    // B operands of the four MFMAs of a block: groups 2p, 2p+1, 2p+4, 2p+5
    static __device__ __forceinline__ void codes(const Regs& r, int, uint4 b[4]) {
        b[0] = nib_lo(r.qa); b[1] = nib_hi(r.qa); b[2] = nib_lo(r.qb); b[3] = nib_hi(r.qb);
    }
    static __device__ __forceinline__ int group_of(int t, int ks) { return k45_group_of(t, ks); }
    static __device__ __forceinline__ int half_of(int, int ks) { return ks & 1; }   // which 16 weights of the group the slice carries
    static __device__ __forceinline__ float combine(const Regs& r, int ks, float v0, float v1, const float4& g2) { return k45_combine(r.hdr, ks, v0, v1, g2); }
};

struct Q5K {
    static constexpr int kBlockBytes = 176;
    static constexpr int kDepth = 4;
    struct Regs { uint4 hdr; uint4 qh; uint4 qa; uint4 qb; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int ks) {
        r.hdr = stream16(blk);
        r.qh = stream16(blk + 16 + 16 * (ks & 1));
        r.qa = stream16(blk + 48 + 16 * ks);
        r.qb = stream16(blk + 112 + 16 * ks);
    }
    static __device__ __forceinline__ void codes(const Regs& r, int ks, uint4 b[4]) {
        const int g = 2 * (ks >> 1);
        b[0] = fifth_bit(nib_lo(r.qa), r.qh, g);
        b[1] = fifth_bit(nib_hi(r.qa), r.qh, g + 1);
        b[2] = fifth_bit(nib_lo(r.qb), r.qh, g + 4);
        b[3] = fifth_bit(nib_hi(r.qb), r.qh, g + 5);
    }
    static __device__ __forceinline__ int group_of(int t, int ks) { return k45_group_of(t, ks); }
    static __device__ __forceinline__ int half_of(int, int ks) { return ks & 1; }
    static __device__ __forceinline__ float combine(const Regs& r, int ks, float v0, float v1, const float4& g2) { return k45_combine(r.hdr, ks, v0, v1, g2); }
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// ------------------------------------------------------------------------------------------------
// IQ4_XS: 136 B = d(2) scales_h(2) scales_l(4) qs(128), blocks 8-byte aligned; w = d (ls - 32) kvalues[code],
// ls six bits per 32 weights (low four in a nibble of scales_l, high two in scales_h); group g = qs[16 g, +16),
// weights 0..15 in the low and 16..31 in the high nibbles.  Lane (n, ks) holds qs[32 ks, +32) = groups 2 ks and
// 2 ks + 1; MFMA t, slice ks carries half t % 2 of group 2 ks + t / 2.  The 16-entry code table sits in four
// constants; a byte permute picks from its lower and upper half and a third one chooses by bit 3 of the code.
// ------------------------------------------------------------------------------------------------
struct IQ4XS {
    static constexpr int kBlockBytes = 136;
    static constexpr int kDepth = 5;
    struct Regs { uint2 hdr; uint4 q0, q1; };
    struct __attribute__((packed, aligned(8))) Words { u32x4 v; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int ks) {
        r.hdr = *reinterpret_cast<const uint2*>(blk);
        const Words a = *reinterpret_cast<const Words*>(blk + 8 + 32 * ks);
        const Words b = *reinterpret_cast<const Words*>(blk + 24 + 32 * ks);
        r.q0 = make_uint4(a.v.x, a.v.y, a.v.z, a.v.w);
        r.q1 = make_uint4(b.v.x, b.v.y, b.v.z, b.v.w);
    }
    // four codes (one per byte, 0..15) -> four table values
    static __device__ __forceinline__ uint32_t values4(uint32_t codes) {
        const uint32_t low3 = codes & 0x07070707u;
        const uint32_t lower = __builtin_amdgcn_perm(0xF6EADDCFu, 0xBFAD9881u, low3);   // -127 -104 -83 -65 | -49 -35 -22 -10
        const uint32_t upper = __builtin_amdgcn_perm(0x71594535u, 0x26190D01u, low3);   // 1 13 25 38 | 53 69 89 113
        return __builtin_amdgcn_perm(upper, lower, ((codes >> 1) & 0x04040404u) | 0x03020100u);
    }
    static __device__ __forceinline__ uint4 values16(const uint4& q, int sh) {
        return make_uint4(values4((q.x >> sh) & 0x0f0f0f0fu), values4((q.y >> sh) & 0x0f0f0f0fu),
                          values4((q.z >> sh) & 0x0f0f0f0fu), values4((q.w >> sh) & 0x0f0f0f0fu));
    }
    static __device__ __forceinline__ void codes(const Regs& r, int, uint4 b[4]) {
        b[0] = values16(r.q0, 0); b[1] = values16(r.q0, 4); b[2] = values16(r.q1, 0); b[3] = values16(r.q1, 4);
    }
    static __device__ __forceinline__ int group_of(int t, int ks) { return 2 * ks + (t >> 1); }
    static __device__ __forceinline__ int half_of(int t, int) { return t & 1; }
    static __device__ __forceinline__ float combine(const Regs& r, int ks, float v0, float v1, const float4& g2) {
        const uint32_t scales_h = r.hdr.x >> 16, sl = (r.hdr.y >> (8 * ks)) & 0xffu;
        const int ls0 = static_cast<int>((sl & 15u) | (((scales_h >> (4 * ks)) & 3u) << 4)) - 32;
        const int ls1 = static_cast<int>((sl >> 4) | (((scales_h >> (4 * ks + 2)) & 3u) << 4)) - 32;
        return f16_bits_to_float(r.hdr.x & 0xffffu) * (static_cast<float>(ls0) * g2.x * v0 + static_cast<float>(ls1) * g2.z * v1);
    }
};

// R activation rows per workgroup (1, 2 or 4): the weights of a super-block are loaded and split into codes once and multiplied
// with the images of R rows, which sit side by side in LDS; grid row blockIdx.y serves activation rows R * blockIdx.y ...
template <typename FMT, int ITERS, bool RAW, int R>
__global__ __launch_bounds__(64 * kMaxWaves) void k45_mfma_matvec_kernel(
    const ActRows act, const WeightRoute route, const uint8_t* __restrict__ w, void* __restrict__ y, int y_dtype, int n, int bpr, int total_rows) {
    fetch_together(act);
    fetch_together(route);
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));          // a multiple of 16
    const StagedX sx = carve_staged_x(smem, kpad);
    const int zero_off = R * image_bytes;                                    // 16 zero bytes
    float* partial = reinterpret_cast<float*>(smem + R * image_bytes + 16); // [R][waves][16]

    const int tid = threadIdx.x;
    const int waves = blockDim.x >> 6;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int col = lane & 15;        // B/C column = output row within the tile; also A's row index m
    const int ks = lane >> 4;         // k slice of A and B, row quad of C
    const size_t woff = route_offset(route, blockIdx.y);
    w += woff;
    if (blockIdx.z) {                        // several projections in one launch: this one's matrix (of the same expert), row count and output
        const int m = blockIdx.z - 1;
        w = route.more_w[m] + woff;
        y = route.more_y[m];
        n = route.more_n[m];
    }
    if (static_cast<int>(blockIdx.x) * kRowsPerWg >= n) return;             // the grid covers the tallest matrix
    const int row0 = blockIdx.y * R;                                         // first activation row of this workgroup
    const int row = blockIdx.x * kRowsPerWg + col;
    const uint8_t* wrow = w + static_cast<size_t>(row < n ? row : 0) * bpr * FMT::kBlockBytes;

    // A side: this lane supplies row m = col = 2 * group + term of MFMA t, slice ks; it is non-zero
    // only when MFMA t's slice ks belongs to `group`: G(t, ks) = 4 * (t >> 1) + 2 * (ks >> 1) + (t & 1)
    int a_off[4], a_step[4], a_row[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int g = FMT::group_of(t, ks);
        const bool active = (col >> 1) == g;
        a_off[t] = active ? ((col & 1) ? kpad : 0) + 32 * g + 16 * (ks & 1) : zero_off;
        a_step[t] = active ? 256 : 0;
        a_row[t] = active ? image_bytes : 0;                                 // distance to the next activation row's image
    }

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.0f;
    bool staged = false;
    if constexpr (RAW) {                     // quantize before the loads take their registers
#pragma unroll 1
        for (int r = 0; r < R; ++r)          // rows past the end: the last row again, result dropped
            quantize_row_to_lds(smem + r * image_bytes, act.x, act.x_dtype, raw_row_of(act, min(row0 + r, total_rows - 1)) * act.k, act.k, kpad,
                                RowNorm{act.gamma, act.eps, act.round_f16});
        if (tid < 4) reinterpret_cast<uint32_t*>(smem + zero_off)[tid] = 0;
        __syncthreads();
        staged = true;
    }
    for (int b0 = wave; b0 < bpr || !staged; b0 += waves * ITERS) {
        typename FMT::Regs regs[ITERS];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int b = min(b0 + it * waves, bpr - 1);                    // clamped: always a valid address
            FMT::load(regs[it], wrow + static_cast<size_t>(b) * FMT::kBlockBytes, ks);
        }
        if (!staged) {                       // first trip of every thread of the workgroup
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int arow = min(row0 + r, total_rows - 1);
                const size_t image_row = act.row_token ? static_cast<size_t>(act.row_token[arow]) : static_cast<size_t>(arow);
                copy_to_lds(smem + r * image_bytes, act.image + image_row * act.stride, image_bytes);
            }
            if (tid < 4) reinterpret_cast<uint32_t*>(smem + zero_off)[tid] = 0;
            __syncthreads();
            staged = true;
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int b = b0 + it * waves;
            if (b < bpr) {                                                   // wave-uniform
                uint4 bw[4];
                FMT::codes(regs[it], ks, bw);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    v4i c = {0, 0, 0, 0};
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const uint4 a = *reinterpret_cast<const uint4*>(smem + a_off[t] + b * a_step[t] + r * a_row[t]);
                        c = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(a), as_v4i(bw[t]), c, 0, 0, 0);
                    }
                    // c = {group 2ks: hi, lo; group 2ks+1: hi, lo} for output row `col`
                    const float v0 = static_cast<float>(__mul24(c.x, 254) + c.y);
                    const float v1 = static_cast<float>(__mul24(c.z, 254) + c.w);
                    const float4 g2 = *reinterpret_cast<const float4*>(reinterpret_cast<const unsigned char*>(sx.gs + b * 8 + 2 * ks) + r * image_bytes);   // {xs0, sum0, xs1, sum1}
                    acc[r] += FMT::combine(regs[it], ks, v0, v1, g2);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        float a = acc[r];
        a = quad_rows_sum(a);
        if (ks == 0) partial[(r * waves + wave) * kRowsPerWg + col] = a;
    }
    __syncthreads();
    if (tid < kRowsPerWg * R) {
        const int r = tid / kRowsPerWg, c = tid % kRowsPerWg;
        float total = 0.0f;
        for (int v = 0; v < waves; ++v) total += partial[(r * waves + v) * kRowsPerWg + c];
        const int out_row = blockIdx.x * kRowsPerWg + c;
        if (out_row < n && row0 + r < total_rows) store_any(y, y_dtype, static_cast<size_t>(row0 + r) * n + out_row, total);
    }
}

// ------------------------------------------------------------------------------------------------
// The single-launch form for calls of a few raw activation rows: no workgroup-wide image and no barrier ahead of the
// matrix-core work.  A wave needs the activations of its own super-blocks only (wave w of W takes blocks w, w + W, ...), so it
// requests those 256-value slices first, then all its weights, and quantizes the slices (the same two-term image, bit for
// bit) into its own LDS slots while the weights are on their way; memory returns a wave's loads in the order they were
// issued, so the slices are there long before the first block.  Slot = hi[256] | lo[256] | float2 gs[8] (576 B).  The waves
// meet only in the final sum.
constexpr int kSlotBytes = 576;

template <bool X16> struct RawX;
template <> struct RawX<true> { uint2 v; };                    // four fp16 / bf16 values
template <> struct RawX<false> { uint4 v; };                   // four float32 values

// Values e0 .. e0 + 3 of the row at element offset xoff, zeros from k on (k >= 4 or k == 0), in two steps so that nothing
// waits between the requests of consecutive blocks.  request_raw4 is branch-free and only issues the load: four values from
// an address clamped into the row (the row's last four values for a lane at or past its end; any alignment).  settle_raw4,
// called where the values are used, shifts them down by the number of values the clamp moved the address.
__device__ __forceinline__ int raw4_start(int e0, int k) { return max(min(e0, k - 4), 0); }
template <bool X16>
__device__ __forceinline__ void request_raw4(RawX<X16>& r, const void* __restrict__ x, size_t xoff, int e0, int k) {
    const int start = raw4_start(e0, k);
    if constexpr (X16) {
        struct __attribute__((packed, aligned(2))) U { uint32_t a, b; };
        const U u = *reinterpret_cast<const U*>(static_cast<const uint16_t*>(x) + xoff + start);
        r.v = make_uint2(u.a, u.b);
    } else {
        struct __attribute__((packed, aligned(4))) U { u32x4 v; };
        const U u = *reinterpret_cast<const U*>(static_cast<const uint32_t*>(x) + xoff + start);
        r.v = make_uint4(u.v.x, u.v.y, u.v.z, u.v.w);
    }
}
template <bool X16>
__device__ __forceinline__ void settle_raw4(RawX<X16>& r, int e0, int k) {
    const int moved = k == 0 ? 4 : min(e0 - raw4_start(e0, k), 4);          // 0: all four values lie inside the row; 4: none does
    if constexpr (X16) {
        const uint64_t both = (static_cast<uint64_t>(r.v.y) << 32) | r.v.x;
        const uint64_t kept = moved >= 4 ? 0ull : both >> (16 * moved);
        r.v = make_uint2(static_cast<uint32_t>(kept), static_cast<uint32_t>(kept >> 32));
    } else {
        const uint4 u = r.v;
        r.v.x = moved == 0 ? u.x : moved == 1 ? u.y : moved == 2 ? u.z : moved == 3 ? u.w : 0u;
        r.v.y = moved == 0 ? u.y : moved == 1 ? u.z : moved == 2 ? u.w : 0u;
        r.v.z = moved == 0 ? u.z : moved == 1 ? u.w : 0u;
        r.v.w = moved == 0 ? u.w : 0u;
    }
}
template <bool X16>
__device__ __forceinline__ void raw_to_float4(const RawX<X16>& r, int x_dtype, float v[4]) {
    if constexpr (X16) {
        if (x_dtype == PLLM_BF16) {
            v[0] = __uint_as_float(r.v.x << 16); v[1] = __uint_as_float(r.v.x & 0xffff0000u);
            v[2] = __uint_as_float(r.v.y << 16); v[3] = __uint_as_float(r.v.y & 0xffff0000u);
        } else {
            v[0] = f16_bits_to_float(r.v.x & 0xffffu); v[1] = f16_bits_to_float(r.v.x >> 16);
            v[2] = f16_bits_to_float(r.v.y & 0xffffu); v[3] = f16_bits_to_float(r.v.y >> 16);
        }
    } else {
        v[0] = __uint_as_float(r.v.x); v[1] = __uint_as_float(r.v.y); v[2] = __uint_as_float(r.v.z); v[3] = __uint_as_float(r.v.w);
    }
}

// ITERS = blocks a wave walks per pass, DEPTH <= ITERS = blocks it keeps in flight (a block's activation slice is requested
// right ahead of its weights, so it arrives first).
// PLAIN: one matrix, one output, activation row = grid row (no routing, no further projections, no row map): the arguments the
// other forms test one after the other (a scalar load and a wait each) are not read at all.
// RSUM (the down projection of one token's routed experts): wave v is route v.  It takes ALL blocks of its own expert's 16 rows
// against its own activation row, which it forms on the way as SiLU(min(gate, L)) * clamp(up, +-L) * route weight from the gate
// (x) and up (x_up) products [routes, k]; the sum over the waves at the end is the sum over the routes, in route order.
// ROWS > 1 (dense calls of two to four rows): the wave multiplies every block it fetches and unpacks into all ROWS rows, one
// after the other through the same LDS slot; one grid row.  The call's row count travels in round_f16 (no normalisation here):
// rows past it repeat the last row and are not stored.
template <typename FMT, int ITERS, int DEPTH, bool X16, bool NORM, bool PLAIN = false, bool RSUM = false, int ROWS = 1>
__global__ __launch_bounds__(64 * kMaxWaves) void wave_image_matvec_kernel(
    const void* __restrict__ x, int x_dtype, int k, const WeightRoute route, const uint8_t* __restrict__ w, void* __restrict__ y,
    int y_dtype, int n, int bpr, const float* __restrict__ gamma, float eps, int round_f16, const int64_t* __restrict__ row_token, int x_broadcast) {
    // RSUM has no normalisation and no row map, and its own inputs travel in their arguments (one signature for all forms: three
    // arguments more made every short call of the other forms 0.2 us slower, with the same instructions; putting the arguments
    // the dense form reads first and the routing struct last changed nothing, and a dense form without the routing struct in its
    // argument block was 0.2 us slower too):
    // gamma = the route weights, row_token = the up products, eps = the SwiGLU limit
    const float* route_w = gamma;
    const void* x_up = row_token;
    const float limit = eps;
    if constexpr (!PLAIN) {
        fetch_together(route);
        asm volatile("" : : "s"(static_cast<int>(row_token != nullptr)), "s"(x_broadcast));
    }
    asm volatile("" : : "s"(x), "s"(k), "s"(w), "s"(y), "s"(n), "s"(bpr));   // the arguments in one batch of scalar loads, one wait
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    const int waves = blockDim.x >> 6;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int col = lane & 15;
    const int ks = lane >> 4;
    constexpr int kWaveBytes = kSlotBytes + 16;                               // the wave's slot, then its 16 zero bytes
    unsigned char* slot = smem + wave * kWaveBytes;
    float* partial = reinterpret_cast<float*>(smem + waves * kWaveBytes);    // [16][kMaxWaves]: a row's shares side by side
    if constexpr (!PLAIN) {
        const size_t woff = route_offset(route, RSUM ? __builtin_amdgcn_readfirstlane(wave) : static_cast<int>(blockIdx.y));   // routed calls: the grid row's expert
        w += woff;
        if (blockIdx.z) {                    // several projections in one launch: this one's matrix, row count and output
            const int m = blockIdx.z - 1;
            w = route.more_w[m] + woff;
            y = route.more_y[m];
            n = route.more_n[m];
        }
        if (static_cast<int>(blockIdx.x) * kRowsPerWg >= n) return;         // the grid covers the tallest matrix
    }
    const int row = blockIdx.x * kRowsPerWg + col;
    const uint8_t* wrow = w + static_cast<size_t>(row < n ? row : 0) * bpr * FMT::kBlockBytes;
    const size_t xoff = (PLAIN ? static_cast<size_t>(blockIdx.y) : RSUM ? static_cast<size_t>(wave)
                               : x_broadcast ? 0 : row_token ? static_cast<size_t>(row_token[blockIdx.y]) : static_cast<size_t>(blockIdx.y)) * k;
    const int bstep = RSUM ? 1 : waves;                                       // distance between a wave's blocks
    const float rw = RSUM ? route_w[__builtin_amdgcn_readfirstlane(wave)] : 1.0f;

    if (lane < 4) reinterpret_cast<uint32_t*>(slot + kSlotBytes)[lane] = 0;
    float acc = 0.0f;
    constexpr int kMore = ROWS > 1 ? ROWS - 1 : 1;                            // further rows of a ROWS call
    const int total_rows = ROWS > 1 ? round_f16 : 1;
    float acc_more[kMore];
#pragma unroll
    for (int j = 0; j < kMore; ++j) acc_more[j] = 0.0f;
    // NORM (the row passes through an RMS normalisation first, one pass of the loop below): the wave's slices of all its blocks
    // are requested at once, with the weights of the first blocks behind them; their squares are the wave's share of the row's
    // sum, the shares meet in LDS, and the slices are scaled as they are quantized.  No extra pass over the row, one barrier.
    constexpr int kHeldX = NORM ? ITERS : DEPTH;
    RawX<X16> raw[kHeldX];
    RawX<X16> raw_up[RSUM ? kHeldX : 1];                                       // RSUM: the up products
    RawX<X16> raw_more[kMore][ROWS > 1 ? kHeldX : 1];                         // ROWS: the further rows' slices
    RawX<false> graw[NORM ? ITERS : 1];
    float rstd = 1.0f;
    for (int b0 = RSUM ? 0 : wave; b0 < bpr; b0 += bstep * ITERS) {
        typename FMT::Regs regs[DEPTH];
        auto request_x = [&](int it) {
            const int b = b0 + it * bstep;
            request_raw4<X16>(raw[it % kHeldX], x, xoff, 256 * b + 4 * lane, b < bpr ? k : 0);
            if constexpr (RSUM) request_raw4<X16>(raw_up[it % kHeldX], x_up, xoff, 256 * b + 4 * lane, b < bpr ? k : 0);
            if constexpr (ROWS > 1) {
#pragma unroll
                for (int j = 0; j < kMore; ++j)
                    request_raw4<X16>(raw_more[j][it % kHeldX], x, xoff + static_cast<size_t>(min(j + 1, total_rows - 1)) * k, 256 * b + 4 * lane, b < bpr ? k : 0);
            }
        };
        auto request_w = [&](int it) {
            const int b = b0 + it * bstep;
            FMT::load(regs[it % DEPTH], wrow + static_cast<size_t>(min(b, bpr - 1)) * FMT::kBlockBytes, ks);   // clamped: always a valid address
        };
        auto request = [&](int it) {
            if constexpr (!NORM) request_x(it);
            __builtin_amdgcn_sched_barrier(0);                              // keep the issue order: memory returns a wave's loads in it
            request_w(it);
            __builtin_amdgcn_sched_barrier(0);
        };
        // the activation slices first: they are small, arrive first and are quantized while the weights are on their way
#pragma unroll
        for (int it = 0; it < kHeldX; ++it) request_x(it);
        if constexpr (NORM) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int b = b0 + it * bstep;
                request_raw4<false>(graw[it], gamma, 0, 256 * b + 4 * lane, b < bpr ? k : 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int it = 0; it < DEPTH; ++it) request_w(it);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (NORM) {
            float ss = 0.0f;
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int b = b0 + it * bstep;
                if (k != 256 * bpr) {                                        // rows that end inside their last block
                    settle_raw4<X16>(raw[it], 256 * b + 4 * lane, b < bpr ? k : 0);
                    settle_raw4<false>(graw[it], 256 * b + 4 * lane, b < bpr ? k : 0);
                }
                float v[4];
                raw_to_float4<X16>(raw[it], x_dtype, v);
                if (b < bpr) ss += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
            }
            ss = group_sum<64>(ss);
            float* shares = partial + kMaxWaves * kRowsPerWg;                // [waves]
            if (lane == 0) shares[wave] = ss;
            __syncthreads();
            float total = 0.0f;
            for (int v = 0; v < waves; ++v) total += shares[v];
            rstd = rsqrtf(total / static_cast<float>(k) + eps);
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int b = b0 + it * bstep;
            if (b < bpr) {                                                   // wave-uniform
                // the block's activation slice into the wave's slot: the same two-term image the pre-pass kernel writes
                float v[4];
                if constexpr (!NORM)
                    if (k != 256 * bpr) settle_raw4<X16>(raw[it % kHeldX], 256 * b + 4 * lane, k);   // rows that end inside their last block
                raw_to_float4<X16>(raw[it % kHeldX], x_dtype, v);
                if constexpr (RSUM) {
                    float u[4];
                    if (k != 256 * bpr) settle_raw4<X16>(raw_up[it % kHeldX], 256 * b + 4 * lane, k);
                    raw_to_float4<X16>(raw_up[it % kHeldX], x_dtype, u);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float g = v[i], uu = u[i];
                        if (limit > 0.0f) {
                            uu = fminf(fmaxf(uu, -limit), limit);
                            g = fminf(g, limit);
                        }
                        v[i] = g / (1.0f + expf(-g)) * uu * rw;              // values past k are zeros on both sides
                    }
                }
                if constexpr (NORM) {
                    const float g[4] = {__uint_as_float(graw[it].v.x), __uint_as_float(graw[it].v.y), __uint_as_float(graw[it].v.z), __uint_as_float(graw[it].v.w)};
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float t = v[i] * rstd * g[i];                        // values past k are zeros on both sides
                        if (round_f16) t = static_cast<float>(static_cast<_Float16>(t));
                        v[i] = t;
                    }
                }
                uint32_t qh, ql;
                float scale;
                float sum4;                                                 // the four values as the image holds them, summed (exact): the
                quantize4_pow2(v, qh, ql, scale, &sum4);                    // min terms cancel against dots of these same rounded values
                reinterpret_cast<uint32_t*>(slot)[lane] = qh;
                reinterpret_cast<uint32_t*>(slot + 256)[lane] = ql;
                const float sum = group_sum<4>(sum4);
                const float sum32 = sum + butterfly_peer<4>(sum);
                if ((lane & 7) == 0) reinterpret_cast<float2*>(slot + 512)[lane >> 3] = make_float2(scale, sum32);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();                            // LDS serves a wave's requests in order
                uint4 bw[4];
                FMT::codes(regs[it % DEPTH], ks, bw);
                v4i c = {0, 0, 0, 0};
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    // this lane supplies row m = col = 2 * group + term of MFMA t's A operand, slice ks: codes only where that
                    // slice belongs to `group`, the zero bytes elsewhere
                    const int g = FMT::group_of(t, ks);
                    const int off = (col >> 1) == g ? ((col & 1) ? 256 : 0) + 32 * g + 16 * FMT::half_of(t, ks) : kSlotBytes;
                    const uint4 a = *reinterpret_cast<const uint4*>(slot + off);
                    c = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(a), as_v4i(bw[t]), c, 0, 0, 0);
                }
                const float v0 = static_cast<float>((c.x << 8) + c.y);       // both terms of the image joined: 256 hi + lo
                const float v1 = static_cast<float>((c.z << 8) + c.w);
                const float4 g2 = *reinterpret_cast<const float4*>(slot + 512 + 16 * ks);   // {xs0, sum0, xs1, sum1}
                acc += FMT::combine(regs[it % DEPTH], ks, v0, v1, g2);
                __builtin_amdgcn_wave_barrier();                            // the next block's slice overwrites the slot
                if constexpr (ROWS > 1) {
#pragma unroll
                  for (int j = 0; j < kMore; ++j) {
                    // the next row's slice through the same slot, against the codes already unpacked
                    float u[4];
                    if (k != 256 * bpr) settle_raw4<X16>(raw_more[j][it % kHeldX], 256 * b + 4 * lane, k);
                    raw_to_float4<X16>(raw_more[j][it % kHeldX], x_dtype, u);
                    uint32_t qh2, ql2;
                    float scale2, sum4b;
                    quantize4_pow2(u, qh2, ql2, scale2, &sum4b);
                    reinterpret_cast<uint32_t*>(slot)[lane] = qh2;
                    reinterpret_cast<uint32_t*>(slot + 256)[lane] = ql2;
                    const float sum_b = group_sum<4>(sum4b);
                    const float sum32_b = sum_b + butterfly_peer<4>(sum_b);
                    if ((lane & 7) == 0) reinterpret_cast<float2*>(slot + 512)[lane >> 3] = make_float2(scale2, sum32_b);
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    v4i c2 = {0, 0, 0, 0};
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const int g = FMT::group_of(t, ks);
                        const int off = (col >> 1) == g ? ((col & 1) ? 256 : 0) + 32 * g + 16 * FMT::half_of(t, ks) : kSlotBytes;
                        const uint4 a = *reinterpret_cast<const uint4*>(slot + off);
                        c2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(a), as_v4i(bw[t]), c2, 0, 0, 0);
                    }
                    const float w0 = static_cast<float>((c2.x << 8) + c2.y);
                    const float w1 = static_cast<float>((c2.z << 8) + c2.w);
                    const float4 h2 = *reinterpret_cast<const float4*>(slot + 512 + 16 * ks);
                    acc_more[j] += FMT::combine(regs[it % DEPTH], ks, w0, w1, h2);
                    __builtin_amdgcn_wave_barrier();
                  }
                }
            }
            if (it + DEPTH < ITERS) request(it + DEPTH);
        }
    }
    acc = quad_rows_sum(acc);
    if (ks == 0) partial[col * kMaxWaves + wave] = acc;
    if constexpr (ROWS > 1) {
#pragma unroll
        for (int j = 0; j < kMore; ++j) {
            const float more = quad_rows_sum(acc_more[j]);
            if (ks == 0) partial[((j + 1) * kRowsPerWg + col) * kMaxWaves + wave] = more;   // (behind the first row's shares; the launcher sizes for it)
        }
    }
    __syncthreads();
    // the waves' shares in wave order, fetched together (a workgroup of one wave walks the rows of an eight-row call in two steps)
    for (int e = tid; e < ROWS * kRowsPerWg; e += (ROWS * kRowsPerWg > 64 ? 64 * waves : ROWS * kRowsPerWg)) {
        const float4 lo4 = *reinterpret_cast<const float4*>(partial + e * kMaxWaves);
        const float4 hi4 = *reinterpret_cast<const float4*>(partial + e * kMaxWaves + 4);
        const float p[kMaxWaves] = {lo4.x, lo4.y, lo4.z, lo4.w, hi4.x, hi4.y, hi4.z, hi4.w};
        float total = p[0];
#pragma unroll
        for (int v = 1; v < kMaxWaves; ++v) total = v < waves ? total + p[v] : total;
        const int out_row = blockIdx.x * kRowsPerWg + (e & (kRowsPerWg - 1));
        const int y_row = ROWS > 1 ? e / kRowsPerWg : static_cast<int>(blockIdx.y);
        if (out_row < n && (ROWS == 1 || y_row < total_rows)) store_any(y, y_dtype, static_cast<size_t>(y_row) * n + out_row, total);
    }
}

// ------------------------------------------------------------------------------------------------
template <typename KERN>
int launch_kernel(KERN kern, const ActRows& act, const WeightRoute& route, const uint8_t* w, void* y, int y_dtype,
                  int rows, int n, int bpr, int waves, int rows_per_wg, hipStream_t stream) {
    const size_t smem = rows_per_wg * staged_x_bytes(bpr * 256) + 16 + static_cast<size_t>(rows_per_wg) * waves * kRowsPerWg * sizeof(float);
    if (smem > 64 * 1024) {
        if (smem > 160 * 1024) return PLLM_ERR_UNSUPPORTED;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(smem)) != hipSuccess)
            return PLLM_ERR_UNSUPPORTED;
    }
    int tallest = n;
    for (int m = 0; m < route.extra; ++m) tallest = tallest > route.more_n[m] ? tallest : route.more_n[m];
    dim3 grid((tallest + kRowsPerWg - 1) / kRowsPerWg, (rows + rows_per_wg - 1) / rows_per_wg, 1 + route.extra);
    hipLaunchKernelGGL(kern, grid, dim3(64 * waves), smem, stream, act, route, w, y, y_dtype, n, bpr, rows);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

template <typename KERN>
int launch_wave_kernel(KERN kern, const ActRows& act, const WeightRoute& route, const uint8_t* w, void* y, int y_dtype,
                       int rows, int n, int bpr, int waves, hipStream_t stream, int rows_per_pass = 1) {
    const size_t smem = static_cast<size_t>(waves) * (kSlotBytes + 16) + static_cast<size_t>(rows_per_pass * kMaxWaves * kRowsPerWg + waves) * sizeof(float);
    int tallest = n;
    for (int m = 0; m < route.extra; ++m) tallest = tallest > route.more_n[m] ? tallest : route.more_n[m];
    dim3 grid((tallest + kRowsPerWg - 1) / kRowsPerWg, rows, 1 + route.extra);
    hipLaunchKernelGGL(kern, grid, dim3(64 * waves), smem, stream, act.x, act.x_dtype, act.k, route, w, y, y_dtype, n, bpr, act.gamma, act.eps,
                       act.round_f16, act.row_token, act.x_broadcast);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

// float32 activation quads take twice the registers: one block less in flight keeps four waves per SIMD
template <typename FMT>
constexpr int wave_depth(int iters, bool x16) {
    const int cap = FMT::kDepth - (x16 ? 0 : 1);
    return iters < cap ? iters : cap;
}

// waves per workgroup and blocks in flight per wave for a row of bpr super-blocks
void split_blocks(int bpr, int work_items, int& waves, int& iters) {
    waves = 1;
    while (waves < kMaxWaves && bpr / (waves * 2) >= 3) waves *= 2;
    // few tiles (less than two workgroups per compute unit): twice the waves with half the blocks each keep more loads in flight
    if (waves < kMaxWaves && bpr / (waves * 2) >= 2 && work_items < 2 * compute_units()) waves *= 2;
    const int niter = (bpr + waves - 1) / waves;
    const int passes = (niter + 7) / 8;
    iters = (niter + passes - 1) / passes;
    if (iters == 7) iters = 8;
}

// the single-launch form: raw rows (with or without an RMS normalisation ahead), no routing
template <typename FMT, bool NORM>
int launch_wave(const ActRows& act, const WeightRoute& route, const uint8_t* w, void* y, int y_dtype, int rows, int n, int bpr, hipStream_t stream) {
    int waves, iters;
    int tiles = (n + kRowsPerWg - 1) / kRowsPerWg;
    for (int m = 0; m < route.extra; ++m) tiles += (route.more_n[m] + kRowsPerWg - 1) / kRowsPerWg;
    const bool plain = !NORM && !routed(route) && route.extra == 0 && !act.row_token && !act.x_broadcast;
    const bool pair = plain && rows == 2, quad = plain && (rows == 3 || rows == 4), oct = plain && rows >= 5 && rows <= 8;   // all rows in one pass over the weights
    split_blocks(bpr, tiles * (pair || quad || oct ? 1 : rows), waves, iters);   // (one grid row then: the single-row call's split, so the same bits per row)
    if (NORM && waves * iters < bpr) return PLLM_ERR_UNSUPPORTED;             // the normalised form holds a wave's slices of the whole row
    ActRows few = act;
    few.round_f16 = rows;                                                     // (where these forms expect the row count)
#define PLLM_CASE(I) case I: \
        if constexpr (!NORM) if (pair) \
            return act.x_dtype == PLLM_F32 ? launch_wave_kernel(wave_image_matvec_kernel<FMT, I, wave_depth<FMT>(I, false), false, false, true, false, 2>, few, route, w, y, y_dtype, 1, n, bpr, waves, stream, 2) \
                                           : launch_wave_kernel(wave_image_matvec_kernel<FMT, I, wave_depth<FMT>(I, false), true, false, true, false, 2>, few, route, w, y, y_dtype, 1, n, bpr, waves, stream, 2); \
        if constexpr (!NORM) if (quad) \
            return act.x_dtype == PLLM_F32 ? launch_wave_kernel(wave_image_matvec_kernel<FMT, I, (I < 2 ? I : 2), false, false, true, false, 4>, few, route, w, y, y_dtype, 1, n, bpr, waves, stream, 4) \
                                           : launch_wave_kernel(wave_image_matvec_kernel<FMT, I, wave_depth<FMT>(I, false), true, false, true, false, 4>, few, route, w, y, y_dtype, 1, n, bpr, waves, stream, 4); \
        if constexpr (!NORM) if (oct) \
            return act.x_dtype == PLLM_F32 ? launch_wave_kernel(wave_image_matvec_kernel<FMT, I, 1, false, false, true, false, 8>, few, route, w, y, y_dtype, 1, n, bpr, waves, stream, 8) \
                                           : launch_wave_kernel(wave_image_matvec_kernel<FMT, I, (I < 2 ? I : 2), true, false, true, false, 8>, few, route, w, y, y_dtype, 1, n, bpr, waves, stream, 8); \
        if constexpr (!NORM) if (plain) \
            return act.x_dtype == PLLM_F32 ? launch_wave_kernel(wave_image_matvec_kernel<FMT, I, wave_depth<FMT>(I, false), false, false, true>, act, route, w, y, y_dtype, rows, n, bpr, waves, stream) \
                                           : launch_wave_kernel(wave_image_matvec_kernel<FMT, I, wave_depth<FMT>(I, true), true, false, true>, act, route, w, y, y_dtype, rows, n, bpr, waves, stream); \
        return act.x_dtype == PLLM_F32 ? launch_wave_kernel(wave_image_matvec_kernel<FMT, I, wave_depth<FMT>(I, false), false, NORM>, act, route, w, y, y_dtype, rows, n, bpr, waves, stream) \
                                       : launch_wave_kernel(wave_image_matvec_kernel<FMT, I, wave_depth<FMT>(I, true), true, NORM>, act, route, w, y, y_dtype, rows, n, bpr, waves, stream)
    switch (iters) {
        PLLM_CASE(1); PLLM_CASE(2); PLLM_CASE(3); PLLM_CASE(4); PLLM_CASE(5); PLLM_CASE(6);
        default: PLLM_CASE(8);
    }
#undef PLLM_CASE
}

// the routes of one token as the waves of a workgroup (RSUM): float32 gate / up products [routes, k], routes <= kMaxWaves
template <typename FMT>
int launch_wave_route_sum(const float* gate, const float* up, const float* route_w, float limit, int k, const WeightRoute& route, const uint8_t* w,
                          void* y, int y_dtype, int n, int bpr, int routes, hipStream_t stream) {
    const int passes = (bpr + 5) / 6, iters = (bpr + passes - 1) / passes;
    const size_t smem = static_cast<size_t>(routes) * (kSlotBytes + 16) + static_cast<size_t>(kMaxWaves * kRowsPerWg + routes) * sizeof(float);
    const dim3 grid((n + kRowsPerWg - 1) / kRowsPerWg, 1, 1);
#define PLLM_CASE(I) case I: \
        hipLaunchKernelGGL((wave_image_matvec_kernel<FMT, I, wave_depth<FMT>(I, false), false, false, false, true>), grid, dim3(64 * routes), smem, stream, \
                           static_cast<const void*>(gate), PLLM_F32, k, route, w, y, y_dtype, n, bpr, route_w, limit, 0, \
                           reinterpret_cast<const int64_t*>(up), 0); \
        break
    switch (iters) {
        PLLM_CASE(1); PLLM_CASE(2); PLLM_CASE(3); PLLM_CASE(4); PLLM_CASE(5);
        default: PLLM_CASE(6);
    }
#undef PLLM_CASE
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

// ------------------------------------------------------------------------------------------------
// Q2_K and Q6_K in the same single-launch frame: formats of sixteen groups of 16 weights.
// A rows = the 16 groups, one MFMA set per activation term; lane (n, ks) supplies as B the 16 weights of
// one group per MFMA t (the format says which) and, where its A row (= lane % 16) is that group, the
// group's 16 activation bytes as A.  C[4 ks .. 4 ks + 3][n] = groups 4 ks .. 4 ks + 3 of weight row n,
// whose scales the lane applies.  The wave's LDS slot adds the sums per 16 activations (Q2_K: min
// terms; Q6_K: codes are left unsigned and the - 32 goes through the sums).
//   Q2_K, 84 B = scales(16) qs(64) d(2) dmin(2): 2-bit codes; group g lies in bytes qs[16 j, 16 j + 16),
//     j = 2 (g / 8) + g % 2, at bit 2 ((g % 8) / 2); scale byte g = scale (low nibble), min (high nibble);
//     y = d sum_g sc_g dot(q_g, x_g) - dmin sum_g m_g sum(x_g).  MFMA t, slice ks: group 4 t + ks.
//   Q6_K, 210 B = ql(128) qh(64) scales(16 x int8) d(2), blocks 2-byte aligned: code = low nibble | two
//     high bits << 4, minus 32; lane (n, ks) holds ql[64 h + 16 p ..], ql[64 h + 32 + 16 p ..] and
//     qh[32 h + 16 p ..] with h = ks / 2, p = ks % 2; MFMA t, slice ks: group 8 h + 2 t + p.
// ------------------------------------------------------------------------------------------------
constexpr int kQ2SlotBytes = kSlotBytes + 64;       // ... | float sum16[16]
struct __attribute__((packed, aligned(4))) Dwords4 { u32x4 v; };
struct __attribute__((packed, aligned(2))) Words16 { u32x4 v; };          // blocks on a 2-byte boundary: still one 16-byte load
struct __attribute__((packed, aligned(2))) Words4 { uint32_t v; };
__device__ __forceinline__ uint4 load16_a2(const uint8_t* p) {
    const Words16 u = *reinterpret_cast<const Words16*>(p);
    return make_uint4(u.v.x, u.v.y, u.v.z, u.v.w);
}

struct WaveQ2K {
    static constexpr int kBlockBytes = 84;
    static constexpr int kAlign = 4;
    struct Regs { uint32_t sc; uint4 qa, qb; uint32_t dd; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int ks) {
        r.sc = *reinterpret_cast<const uint32_t*>(blk + 4 * ks);               // scale bytes of groups 4 ks .. 4 ks + 3
        const Dwords4 a = *reinterpret_cast<const Dwords4*>(blk + 16 + 16 * (ks & 1));
        const Dwords4 b = *reinterpret_cast<const Dwords4*>(blk + 48 + 16 * (ks & 1));
        r.qa = make_uint4(a.v.x, a.v.y, a.v.z, a.v.w);                        // groups 0 .. 7 with the lane's parity
        r.qb = make_uint4(b.v.x, b.v.y, b.v.z, b.v.w);                        // groups 8 .. 15
        r.dd = *reinterpret_cast<const uint32_t*>(blk + 80);
    }
    // the MFMA and slice that carry group `col`
    static __device__ __forceinline__ int slice_of(int col) { return col & 3; }
    static __device__ __forceinline__ int mfma_of(int col) { return col >> 2; }
    static __device__ __forceinline__ uint4 codes(const Regs& r, int t, int ks) {
        const uint4 piece = t < 2 ? r.qa : r.qb;
        const int sh = 2 * (ks >> 1) + 4 * (t & 1);                             // codes of MFMA t sit at bit 2 (2 (t % 2) + ks / 2)
        return make_uint4((piece.x >> sh) & 0x03030303u, (piece.y >> sh) & 0x03030303u, (piece.z >> sh) & 0x03030303u, (piece.w >> sh) & 0x03030303u);
    }
    // dots[j], xs[j], sums[j]: integer dot (both terms joined), activation scale and activation sum of group 4 ks + j
    static __device__ __forceinline__ float finish(const Regs& r, const float (&dots)[4], const float (&xs)[4], const float (&sums)[4]) {
        float pos = 0.0f, neg = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t sb = (r.sc >> (8 * j)) & 0xffu;
            pos += static_cast<float>(sb & 15u) * xs[j] * dots[j];
            neg += static_cast<float>(sb >> 4) * sums[j];
        }
        return f16_bits_to_float(r.dd & 0xffffu) * pos - f16_bits_to_float(r.dd >> 16) * neg;
    }
};

struct WaveQ6K {
    static constexpr int kBlockBytes = 210;
    static constexpr int kAlign = 2;
    struct Regs { uint4 qa, qb, qh; uint32_t sc, d; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int ks) {
        const int half = ks >> 1, part = ks & 1;
        r.qa = load16_a2(blk + 64 * half + 16 * part);
        r.qb = load16_a2(blk + 64 * half + 32 + 16 * part);
        r.qh = load16_a2(blk + 128 + 32 * half + 16 * part);
        r.sc = reinterpret_cast<const Words4*>(blk + 192 + 4 * ks)->v;     // int8 scales of groups 4 ks .. 4 ks + 3
        r.d = *reinterpret_cast<const uint16_t*>(blk + 208);
    }
    static __device__ __forceinline__ int slice_of(int col) { return 2 * (col >> 3) + (col & 1); }
    static __device__ __forceinline__ int mfma_of(int col) { return (col >> 1) & 3; }
    static __device__ __forceinline__ uint32_t code4(uint32_t ql, uint32_t qh, int t) {
        const uint32_t lo = (t < 2 ? ql : ql >> 4) & 0x0f0f0f0fu;
        const uint32_t hi = (t == 0 ? qh << 4 : t == 1 ? qh << 2 : t == 2 ? qh : qh >> 2) & 0x30303030u;
        return lo | hi;
    }
    static __device__ __forceinline__ uint4 codes(const Regs& r, int t, int) {
        const uint4 ql = (t & 1) ? r.qb : r.qa;
        return make_uint4(code4(ql.x, r.qh.x, t), code4(ql.y, r.qh.y, t), code4(ql.z, r.qh.z, t), code4(ql.w, r.qh.w, t));
    }
    static __device__ __forceinline__ float finish(const Regs& r, const float (&dots)[4], const float (&xs)[4], const float (&sums)[4]) {
        const int sc = static_cast<int>(r.sc);
        const float v = static_cast<float>(static_cast<int8_t>(sc)) * (xs[0] * dots[0] - 32.0f * sums[0]) +
                        static_cast<float>(static_cast<int8_t>(sc >> 8)) * (xs[1] * dots[1] - 32.0f * sums[1]) +
                        static_cast<float>(static_cast<int8_t>(sc >> 16)) * (xs[2] * dots[2] - 32.0f * sums[2]) +
                        static_cast<float>(sc >> 24) * (xs[3] * dots[3] - 32.0f * sums[3]);
        return f16_bits_to_float(r.d) * v;
    }
};

// NORM (one pass of the block loop, as in wave_image_matvec_kernel): the wave requests the slices of all its blocks at once, their
// squares are its share of the row's sum, the shares meet in LDS behind one barrier and the slices are scaled by rstd * gamma
// as they are quantized.
// RSUM: as in wave_image_matvec_kernel (wave = route of one token's experts, SwiGLU formed on the way, ordered sum at the end).
// ROWS > 1: as in wave_image_matvec_kernel (dense calls of two to four rows in one pass over the weights; the row count in round_f16).
template <typename FMT, int ITERS, int DEPTH, bool X16, bool PLAIN = false, bool NORM = false, bool RSUM = false, int ROWS = 1>
__global__ __launch_bounds__(64 * kMaxWaves) void wave_groups16_matvec_kernel(
    const void* __restrict__ x, int x_dtype, int k, const WeightRoute route, const uint8_t* __restrict__ w, void* __restrict__ y,
    int y_dtype, int n, int bpr, const int64_t* __restrict__ row_token, int x_broadcast, const float* __restrict__ gamma, float eps, int round_f16) {
    // (RSUM's own inputs in the arguments it has no use for, as in wave_image_matvec_kernel: gamma = the route weights,
    // row_token = the up products, eps = the SwiGLU limit)
    const float* route_w = gamma;
    const void* x_up = row_token;
    const float limit = eps;
    if constexpr (!PLAIN) {
        fetch_together(route);
        asm volatile("" : : "s"(static_cast<int>(row_token != nullptr)), "s"(x_broadcast));
    }
    asm volatile("" : : "s"(x), "s"(k), "s"(w), "s"(y), "s"(n), "s"(bpr));   // the arguments in one batch of scalar loads, one wait
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    const int waves = blockDim.x >> 6;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int col = lane & 15;
    const int ks = lane >> 4;
    constexpr int kWaveBytes = kQ2SlotBytes + 16;                            // the wave's slot, then its 16 zero bytes
    unsigned char* slot = smem + wave * kWaveBytes;
    float* partial = reinterpret_cast<float*>(smem + waves * kWaveBytes);    // [16][kMaxWaves]: a row's shares side by side
    if constexpr (!PLAIN) {
        const size_t woff = route_offset(route, RSUM ? __builtin_amdgcn_readfirstlane(wave) : static_cast<int>(blockIdx.y));   // routed calls: the grid row's expert
        w += woff;
        if (blockIdx.z) {                    // several projections in one launch: this one's matrix, row count and output
            const int m = blockIdx.z - 1;
            w = route.more_w[m] + woff;
            y = route.more_y[m];
            n = route.more_n[m];
        }
        if (static_cast<int>(blockIdx.x) * kRowsPerWg >= n) return;
    }
    const int row = blockIdx.x * kRowsPerWg + col;
    const uint8_t* wrow = w + static_cast<size_t>(row < n ? row : 0) * bpr * FMT::kBlockBytes;
    const size_t xoff = (PLAIN ? static_cast<size_t>(blockIdx.y) : RSUM ? static_cast<size_t>(wave)
                               : x_broadcast ? 0 : row_token ? static_cast<size_t>(row_token[blockIdx.y]) : static_cast<size_t>(blockIdx.y)) * k;
    const int bstep = RSUM ? 1 : waves;                                       // distance between a wave's blocks
    const float rw = RSUM ? route_w[__builtin_amdgcn_readfirstlane(wave)] : 1.0f;
    // the lane's A operand: group `col` of the block, in the one MFMA whose slice ks carries that group
    const bool mine = FMT::slice_of(col) == ks;
    const int my_t = FMT::mfma_of(col);

    if (lane < 4) reinterpret_cast<uint32_t*>(slot + kQ2SlotBytes)[lane] = 0;
    float acc = 0.0f;
    constexpr int kMore = ROWS > 1 ? ROWS - 1 : 1;                            // further rows of a ROWS call
    const int total_rows = ROWS > 1 ? round_f16 : 1;
    float acc_more[kMore];
#pragma unroll
    for (int j = 0; j < kMore; ++j) acc_more[j] = 0.0f;
    constexpr int kHeldX = NORM ? ITERS : DEPTH;
    float rstd = 1.0f;
    for (int b0 = RSUM ? 0 : wave; b0 < bpr; b0 += bstep * ITERS) {
        RawX<X16> raw[kHeldX];
        RawX<X16> raw_up[RSUM ? kHeldX : 1];
        RawX<X16> raw_more[kMore][ROWS > 1 ? kHeldX : 1];
        RawX<false> graw[NORM ? ITERS : 1];
        typename FMT::Regs regs[DEPTH];
        auto request_x = [&](int it) {
            const int b = b0 + it * bstep;
            request_raw4<X16>(raw[it % kHeldX], x, xoff, 256 * b + 4 * lane, b < bpr ? k : 0);
            if constexpr (RSUM) request_raw4<X16>(raw_up[it % kHeldX], x_up, xoff, 256 * b + 4 * lane, b < bpr ? k : 0);
            if constexpr (ROWS > 1) {
#pragma unroll
                for (int j = 0; j < kMore; ++j)
                    request_raw4<X16>(raw_more[j][it % kHeldX], x, xoff + static_cast<size_t>(min(j + 1, total_rows - 1)) * k, 256 * b + 4 * lane, b < bpr ? k : 0);
            }
        };
        auto request_w = [&](int it) {
            const int b = b0 + it * bstep;
            FMT::load(regs[it % DEPTH], wrow + static_cast<size_t>(min(b, bpr - 1)) * FMT::kBlockBytes, ks);   // clamped: always a valid address
        };
#pragma unroll
        for (int it = 0; it < kHeldX; ++it) request_x(it);
        if constexpr (NORM) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int b = b0 + it * bstep;
                request_raw4<false>(graw[it], gamma, 0, 256 * b + 4 * lane, b < bpr ? k : 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);                                  // keep the issue order: memory returns a wave's loads in it
#pragma unroll
        for (int it = 0; it < DEPTH; ++it) request_w(it);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (NORM) {
            float ss = 0.0f;
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int b = b0 + it * bstep;
                if (k != 256 * bpr) {                                        // rows that end inside their last block
                    settle_raw4<X16>(raw[it], 256 * b + 4 * lane, b < bpr ? k : 0);
                    settle_raw4<false>(graw[it], 256 * b + 4 * lane, b < bpr ? k : 0);
                }
                float v[4];
                raw_to_float4<X16>(raw[it], x_dtype, v);
                if (b < bpr) ss += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
            }
            ss = group_sum<64>(ss);
            float* shares = partial + kMaxWaves * kRowsPerWg;                // [waves]
            if (lane == 0) shares[wave] = ss;
            __syncthreads();
            float total = 0.0f;
            for (int v = 0; v < waves; ++v) total += shares[v];
            rstd = rsqrtf(total / static_cast<float>(k) + eps);
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int b = b0 + it * bstep;
            if (b < bpr) {                                                   // wave-uniform
                float v[4];
                if constexpr (!NORM)
                    if (k != 256 * bpr) settle_raw4<X16>(raw[it % kHeldX], 256 * b + 4 * lane, k);
                raw_to_float4<X16>(raw[it % kHeldX], x_dtype, v);
                if constexpr (RSUM) {
                    float u[4];
                    if (k != 256 * bpr) settle_raw4<X16>(raw_up[it % kHeldX], 256 * b + 4 * lane, k);
                    raw_to_float4<X16>(raw_up[it % kHeldX], x_dtype, u);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float g = v[i], uu = u[i];
                        if (limit > 0.0f) {
                            uu = fminf(fmaxf(uu, -limit), limit);
                            g = fminf(g, limit);
                        }
                        v[i] = g / (1.0f + expf(-g)) * uu * rw;              // values past k are zeros on both sides
                    }
                }
                if constexpr (NORM) {
                    const float g[4] = {__uint_as_float(graw[it].v.x), __uint_as_float(graw[it].v.y), __uint_as_float(graw[it].v.z), __uint_as_float(graw[it].v.w)};
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float t = v[i] * rstd * g[i];                        // values past k are zeros on both sides
                        if (round_f16) t = static_cast<float>(static_cast<_Float16>(t));
                        v[i] = t;
                    }
                }
                uint32_t qh, ql;
                float scale;
                float sum4;                                                 // the four values as the image holds them, summed (exact): the
                quantize4_pow2(v, qh, ql, scale, &sum4);                    // offset terms cancel against dots of these same rounded values
                reinterpret_cast<uint32_t*>(slot)[lane] = qh;
                reinterpret_cast<uint32_t*>(slot + 256)[lane] = ql;
                const float sum = group_sum<4>(sum4);
                const float sum32 = sum + butterfly_peer<4>(sum);
                if ((lane & 7) == 0) reinterpret_cast<float2*>(slot + 512)[lane >> 3] = make_float2(scale, sum32);
                if ((lane & 3) == 0) reinterpret_cast<float*>(slot + kSlotBytes)[lane >> 2] = sum;
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();                            // LDS serves a wave's requests in order
                const typename FMT::Regs& r = regs[it % DEPTH];
                v4i ch = {0, 0, 0, 0}, cl = {0, 0, 0, 0};
                uint4 kept[ROWS > 1 ? 4 : 1];                                 // the unpacked codes, for the further rows
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const uint4 bw = FMT::codes(r, t, ks);
                    if constexpr (ROWS > 1) kept[t] = bw;
                    const int off = (mine && t == my_t) ? 16 * col : kQ2SlotBytes;
                    const uint4 ah = *reinterpret_cast<const uint4*>(slot + off);
                    const uint4 al = *reinterpret_cast<const uint4*>(slot + off + ((mine && t == my_t) ? 256 : 0));
                    ch = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(ah), as_v4i(bw), ch, 0, 0, 0);
                    cl = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(al), as_v4i(bw), cl, 0, 0, 0);
                }
                const float4 g2 = *reinterpret_cast<const float4*>(slot + 512 + 16 * ks);          // {xs, sum} of 32-groups 2 ks, 2 ks + 1
                const float4 s16 = *reinterpret_cast<const float4*>(slot + kSlotBytes + 16 * ks);  // sums of groups 4 ks .. 4 ks + 3
                const float vv[4] = {static_cast<float>((ch.x << 8) + cl.x), static_cast<float>((ch.y << 8) + cl.y),
                                     static_cast<float>((ch.z << 8) + cl.z), static_cast<float>((ch.w << 8) + cl.w)};
                const float xsv[4] = {g2.x, g2.x, g2.z, g2.z};
                const float smv[4] = {s16.x, s16.y, s16.z, s16.w};
                acc += FMT::finish(r, vv, xsv, smv);
                __builtin_amdgcn_wave_barrier();                            // the next block's slice overwrites the slot
                if constexpr (ROWS > 1) {
#pragma unroll
                  for (int j = 0; j < kMore; ++j) {
                    // the next row's slice through the same slot, against the codes already unpacked
                    float u[4];
                    if (k != 256 * bpr) settle_raw4<X16>(raw_more[j][it % kHeldX], 256 * b + 4 * lane, k);
                    raw_to_float4<X16>(raw_more[j][it % kHeldX], x_dtype, u);
                    uint32_t qh2, ql2;
                    float scale2, sum4b;
                    quantize4_pow2(u, qh2, ql2, scale2, &sum4b);
                    reinterpret_cast<uint32_t*>(slot)[lane] = qh2;
                    reinterpret_cast<uint32_t*>(slot + 256)[lane] = ql2;
                    const float sum_b = group_sum<4>(sum4b);
                    const float sum32_b = sum_b + butterfly_peer<4>(sum_b);
                    if ((lane & 7) == 0) reinterpret_cast<float2*>(slot + 512)[lane >> 3] = make_float2(scale2, sum32_b);
                    if ((lane & 3) == 0) reinterpret_cast<float*>(slot + kSlotBytes)[lane >> 2] = sum_b;
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    v4i ch2 = {0, 0, 0, 0}, cl2 = {0, 0, 0, 0};
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const int off = (mine && t == my_t) ? 16 * col : kQ2SlotBytes;
                        const uint4 ah = *reinterpret_cast<const uint4*>(slot + off);
                        const uint4 al = *reinterpret_cast<const uint4*>(slot + off + ((mine && t == my_t) ? 256 : 0));
                        ch2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(ah), as_v4i(kept[t]), ch2, 0, 0, 0);
                        cl2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(al), as_v4i(kept[t]), cl2, 0, 0, 0);
                    }
                    const float4 g2b = *reinterpret_cast<const float4*>(slot + 512 + 16 * ks);
                    const float4 s16b = *reinterpret_cast<const float4*>(slot + kSlotBytes + 16 * ks);
                    const float vvb[4] = {static_cast<float>((ch2.x << 8) + cl2.x), static_cast<float>((ch2.y << 8) + cl2.y),
                                          static_cast<float>((ch2.z << 8) + cl2.z), static_cast<float>((ch2.w << 8) + cl2.w)};
                    const float xsvb[4] = {g2b.x, g2b.x, g2b.z, g2b.z};
                    const float smvb[4] = {s16b.x, s16b.y, s16b.z, s16b.w};
                    acc_more[j] += FMT::finish(r, vvb, xsvb, smvb);
                    __builtin_amdgcn_wave_barrier();
                  }
                }
            }
            if (it + DEPTH < ITERS) {
                if constexpr (!NORM) request_x(it + DEPTH);
                __builtin_amdgcn_sched_barrier(0);
                request_w(it + DEPTH);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    acc = quad_rows_sum(acc);
    if (ks == 0) partial[col * kMaxWaves + wave] = acc;
    if constexpr (ROWS > 1) {
#pragma unroll
        for (int j = 0; j < kMore; ++j) {
            const float more = quad_rows_sum(acc_more[j]);
            if (ks == 0) partial[((j + 1) * kRowsPerWg + col) * kMaxWaves + wave] = more;   // (behind the first row's shares; the launcher sizes for it)
        }
    }
    __syncthreads();
    // the waves' shares in wave order, fetched together (more than 64 results only in the eight-row form, whose workgroup may be one wave)
    for (int e = tid; e < ROWS * kRowsPerWg; e += (ROWS * kRowsPerWg > 64 ? 64 * waves : ROWS * kRowsPerWg)) {
        const float4 lo4 = *reinterpret_cast<const float4*>(partial + e * kMaxWaves);
        const float4 hi4 = *reinterpret_cast<const float4*>(partial + e * kMaxWaves + 4);
        const float p[kMaxWaves] = {lo4.x, lo4.y, lo4.z, lo4.w, hi4.x, hi4.y, hi4.z, hi4.w};
        float total = p[0];
#pragma unroll
        for (int v = 1; v < kMaxWaves; ++v) total = v < waves ? total + p[v] : total;
        const int out_row = blockIdx.x * kRowsPerWg + (e & (kRowsPerWg - 1));
        const int y_row = ROWS > 1 ? e / kRowsPerWg : static_cast<int>(blockIdx.y);
        if (out_row < n && (ROWS == 1 || y_row < total_rows)) store_any(y, y_dtype, static_cast<size_t>(y_row) * n + out_row, total);
    }
}

template <typename KERN>
int launch_q2k_kernel(KERN kern, const ActRows& act, const WeightRoute& route, const uint8_t* w, void* y, int y_dtype,
                      int rows, int n, int bpr, int waves, hipStream_t stream, int rows_per_pass = 1) {
    const size_t smem = static_cast<size_t>(waves) * (kQ2SlotBytes + 16) + static_cast<size_t>(rows_per_pass * kMaxWaves * kRowsPerWg + waves) * sizeof(float);
    int tallest = n;
    for (int m = 0; m < route.extra; ++m) tallest = tallest > route.more_n[m] ? tallest : route.more_n[m];
    dim3 grid((tallest + kRowsPerWg - 1) / kRowsPerWg, rows, 1 + route.extra);
    hipLaunchKernelGGL(kern, grid, dim3(64 * waves), smem, stream, act.x, act.x_dtype, act.k, route, w, y, y_dtype, n, bpr, act.row_token, act.x_broadcast,
                       act.gamma, act.eps, act.round_f16);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

// the routes of one token as the waves of a workgroup (RSUM): float32 gate / up products [routes, k], routes <= kMaxWaves
template <typename FMT>
int launch_groups16_route_sum(const float* gate, const float* up, const float* route_w, float limit, int k, const WeightRoute& route, const uint8_t* w,
                              void* y, int y_dtype, int n, int bpr, int routes, hipStream_t stream) {
    const int passes = (bpr + 5) / 6, iters = (bpr + passes - 1) / passes;
    const size_t smem = static_cast<size_t>(routes) * (kQ2SlotBytes + 16) + static_cast<size_t>(kMaxWaves * kRowsPerWg + routes) * sizeof(float);
    const dim3 grid((n + kRowsPerWg - 1) / kRowsPerWg, 1, 1);
#define PLLM_CASE(I) case I: \
        hipLaunchKernelGGL((wave_groups16_matvec_kernel<FMT, I, (I < 2 ? I : 2), false, false, false, true>), grid, dim3(64 * routes), smem, stream, \
                           static_cast<const void*>(gate), PLLM_F32, k, route, w, y, y_dtype, n, bpr, reinterpret_cast<const int64_t*>(up), 0, \
                           route_w, limit, 0); \
        break
    switch (iters) {
        PLLM_CASE(1); PLLM_CASE(2); PLLM_CASE(3); PLLM_CASE(4); PLLM_CASE(5);
        default: PLLM_CASE(6);
    }
#undef PLLM_CASE
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

template <typename FMT, int R>
int launch_k45_rows(const ActRows& act, const WeightRoute& route, const uint8_t* w, void* y, int y_dtype, int rows, int n, int bpr, hipStream_t stream) {
    if constexpr (R == 1)
        if (act.x && act.k >= 4 && (!act.gamma || (!routed(route) && !act.row_token && !act.x_broadcast))) {
            if (!act.gamma) return launch_wave<FMT, false>(act, route, w, y, y_dtype, rows, n, bpr, stream);
            const int st = launch_wave<FMT, true>(act, route, w, y, y_dtype, rows, n, bpr, stream);
            if (st != PLLM_ERR_UNSUPPORTED) return st;                       // (rows too long for it: the workgroup-wide quantizer below)
        }
    int waves, iters;
    int tiles = (n + kRowsPerWg - 1) / kRowsPerWg;
    for (int m = 0; m < route.extra; ++m) tiles += (route.more_n[m] + kRowsPerWg - 1) / kRowsPerWg;
    split_blocks(bpr, tiles * ((rows + R - 1) / R), waves, iters);
#define PLLM_CASE(I) case I: \
        if constexpr (R == 1) if (act.x) return launch_kernel(k45_mfma_matvec_kernel<FMT, I, true, 1>, act, route, w, y, y_dtype, rows, n, bpr, waves, 1, stream); \
        return launch_kernel(k45_mfma_matvec_kernel<FMT, I, false, R>, act, route, w, y, y_dtype, rows, n, bpr, waves, R, stream)
    switch (iters) {
        PLLM_CASE(1); PLLM_CASE(2); PLLM_CASE(3); PLLM_CASE(4); PLLM_CASE(5); PLLM_CASE(6);
        default: PLLM_CASE(8);
    }
#undef PLLM_CASE
}

// Activation rows per workgroup: routed calls address experts and image rows per grid row and stay at one, and so do calls that
// quantize their rows in the kernel (measured: four rows quantized one after the other cost more than the shared weight pass
// saves, Q4_K 5120x5120 at 4 rows 16.9 us against 14.2); calls on pre-quantized images take pairs at two rows and fours
// from three on (three rows as two pairs: 31.5 us against 28.4 as one four), as long as the images leave room in LDS for three workgroups per compute unit (Q4_K 17408x5120: 24.8 -> 21.9 us
// at 2 rows, 39.5 -> 29.1 us at 4).
template <typename FMT>
int launch_k45(const ActRows& act, const WeightRoute& route, const uint8_t* w, void* y, int y_dtype, int rows, int n, int bpr, hipStream_t stream) {
    const size_t image = staged_x_bytes(bpr * 256);
    const bool plain = !routed(route) && !act.row_token && !act.x;
    if (plain && rows >= 3 && 4 * image <= 52 * 1024) return launch_k45_rows<FMT, 4>(act, route, w, y, y_dtype, rows, n, bpr, stream);
    if (plain && rows >= 2 && 2 * image <= 52 * 1024) return launch_k45_rows<FMT, 2>(act, route, w, y, y_dtype, rows, n, bpr, stream);
    return launch_k45_rows<FMT, 1>(act, route, w, y, y_dtype, rows, n, bpr, stream);
}

template <typename FMT>
int launch_groups16(const ActRows& act, const WeightRoute& route, const uint8_t* w, void* y, int y_dtype, int rows, int n, int bpr, hipStream_t stream) {
    // raw rows, blocks (of every expert) on the format's boundary; a normalisation ahead only on unrouted rows; everything else stays
    // with the other kernels
    if (!act.x || act.k < 4 || ((reinterpret_cast<uintptr_t>(w) | route.expert_stride) & (FMT::kAlign - 1))) return PLLM_ERR_UNSUPPORTED;
    if (act.gamma && (routed(route) || act.row_token || act.x_broadcast)) return PLLM_ERR_UNSUPPORTED;
    for (int m = 0; m < route.extra; ++m)
        if (reinterpret_cast<uintptr_t>(route.more_w[m]) & (FMT::kAlign - 1)) return PLLM_ERR_UNSUPPORTED;
    int waves, iters;
    int tiles = (n + kRowsPerWg - 1) / kRowsPerWg;
    for (int m = 0; m < route.extra; ++m) tiles += (route.more_n[m] + kRowsPerWg - 1) / kRowsPerWg;
    const bool plain = !routed(route) && route.extra == 0 && !act.row_token && !act.x_broadcast;
    const bool pair = plain && !act.gamma && rows == 2, quad = plain && !act.gamma && (rows == 3 || rows == 4);   // all rows in one pass over the weights
    // eight rows for Q6_K only, one block in flight per wave: the caller sends these while the matrix is small (5120x5120 23.7 us against
    // 29.4 on the tiles); for Q2_K eight rows lost to one grid row per row (5120x5120 22.2 against 16.6 us at five rows)
    const bool oct = plain && !act.gamma && rows >= 5 && rows <= 8 && FMT::kBlockBytes == 210;
    split_blocks(bpr, tiles * (pair || quad || oct ? 1 : rows), waves, iters);       // (one grid row then: the single-row call's split, so the same bits per row)
    if (act.gamma && waves * iters < bpr) return PLLM_ERR_UNSUPPORTED;        // the normalised form holds a wave's slices of the whole row
    ActRows few = act;
    few.round_f16 = rows;                                                     // (where the few-row forms expect the row count)
    constexpr int kMaxDepth = 2;            // blocks in flight per wave: five waves per SIMD fit with 2 (Q6_K with 2, 3, 4 and 5 ran within 3 % of each other, Q2_K 14.6 us with 2 against 15.2 with 5)
#define PLLM_OCT_CASE(I) if constexpr (FMT::kBlockBytes == 210) if (oct) \
            return act.x_dtype == PLLM_F32 ? launch_q2k_kernel(wave_groups16_matvec_kernel<FMT, I, 1, false, true, false, false, 8>, few, route, w, y, y_dtype, 1, n, bpr, waves, stream, 8) \
                                           : launch_q2k_kernel(wave_groups16_matvec_kernel<FMT, I, 1, true, true, false, false, 8>, few, route, w, y, y_dtype, 1, n, bpr, waves, stream, 8);
#define PLLM_CASE(I) case I: { \
        constexpr int D = I < kMaxDepth ? I : kMaxDepth; \
        if (pair) \
            return act.x_dtype == PLLM_F32 ? launch_q2k_kernel(wave_groups16_matvec_kernel<FMT, I, D, false, true, false, false, 2>, few, route, w, y, y_dtype, 1, n, bpr, waves, stream, 2) \
                                           : launch_q2k_kernel(wave_groups16_matvec_kernel<FMT, I, D, true, true, false, false, 2>, few, route, w, y, y_dtype, 1, n, bpr, waves, stream, 2); \
        if (quad) \
            return act.x_dtype == PLLM_F32 ? launch_q2k_kernel(wave_groups16_matvec_kernel<FMT, I, D, false, true, false, false, 4>, few, route, w, y, y_dtype, 1, n, bpr, waves, stream, 4) \
                                           : launch_q2k_kernel(wave_groups16_matvec_kernel<FMT, I, D, true, true, false, false, 4>, few, route, w, y, y_dtype, 1, n, bpr, waves, stream, 4); \
        PLLM_OCT_CASE(I) \
        if (act.gamma) \
            return act.x_dtype == PLLM_F32 ? launch_q2k_kernel(wave_groups16_matvec_kernel<FMT, I, D, false, false, true>, act, route, w, y, y_dtype, rows, n, bpr, waves, stream) \
                                           : launch_q2k_kernel(wave_groups16_matvec_kernel<FMT, I, D, true, false, true>, act, route, w, y, y_dtype, rows, n, bpr, waves, stream); \
        if (plain) \
            return act.x_dtype == PLLM_F32 ? launch_q2k_kernel(wave_groups16_matvec_kernel<FMT, I, D, false, true>, act, route, w, y, y_dtype, rows, n, bpr, waves, stream) \
                                           : launch_q2k_kernel(wave_groups16_matvec_kernel<FMT, I, D, true, true>, act, route, w, y, y_dtype, rows, n, bpr, waves, stream); \
        return act.x_dtype == PLLM_F32 ? launch_q2k_kernel(wave_groups16_matvec_kernel<FMT, I, D, false>, act, route, w, y, y_dtype, rows, n, bpr, waves, stream) \
                                       : launch_q2k_kernel(wave_groups16_matvec_kernel<FMT, I, D, true>, act, route, w, y, y_dtype, rows, n, bpr, waves, stream); }
    switch (iters) {
        PLLM_CASE(1) PLLM_CASE(2) PLLM_CASE(3) PLLM_CASE(4) PLLM_CASE(5) PLLM_CASE(6)
        default: PLLM_CASE(8)
    }
#undef PLLM_CASE
#undef PLLM_OCT_CASE
}

// ------------------------------------------------------------------------------------------------
// Q4_K / Q5_K, 2 - 16 rows of bf16 or fp16 activations in one pass over the weights: the activation rows are the ROWS of a
// half-precision matrix-core product and go in as they are (no quantization, no pre-pass).
//   v_mfma_f32_16x16x32_{bf16,f16}: A = 16 activation rows x the 32 columns of one scale group, B = the group's 32 codes x 16 weight
//   rows, C[activation row 4 q .. 4 q + 3][weight row n] in lane (n, q), float32.
// The codes enter B as the exact values M + code (bf16: M = 16 for 4-bit codes, bits 0x4180 | code << 3; M = 32 for 5-bit codes,
// 0x4200 | code << 2; fp16: 0x4c00 | code << 6 and 0x5000 | code << 5), built from the code bytes with a byte permute and a shift;
// a second MFMA per group with B = 1 gives the group's activation sums S, which take M back out and carry the min term:
//   y += d sc_g (C' - M S) - dmin m_g S = (d sc_g) C' - (M d sc_g + dmin m_g) S       per group g, activation row and weight row.
// Lane (n, q) holds bytes [8 q, 8 q + 8) of each 32-byte chunk j of the block's codes (codes 8 q .. 8 q + 7 of groups 2 j, low
// nibbles, and 2 j + 1, high nibbles) and reads the activations at the same columns.  A workgroup owns TILES x 16 weight rows per
// wave, its WAVES waves split the row's super-blocks and meet in LDS; the activation operands and the sums are shared by a
// wave's tiles.  Weights of kRows16Depth blocks in flight per wave, activations one block ahead.
// ------------------------------------------------------------------------------------------------
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8hf __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
constexpr int kRows16Depth = 3;

template <bool BF16>
__device__ __forceinline__ v4f half_mfma(const uint4& a, const uint4& b, v4f c) {
    if constexpr (BF16) {
        union { uint4 u; v8bf v; } av, bv;
        av.u = a; bv.u = b;
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(av.v, bv.v, c, 0, 0, 0);
    } else {
        union { uint4 u; v8hf v; } av, bv;
        av.u = a; bv.u = b;
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(av.v, bv.v, c, 0, 0, 0);
    }
}

// eight code bytes (two dwords) -> eight halves M + code
template <bool BF16, bool FIVE>
__device__ __forceinline__ uint4 code_halves(uint32_t c0, uint32_t c1) {
    constexpr uint32_t kMagic = BF16 ? (FIVE ? 0x42004200u : 0x41804180u) : (FIVE ? 0x50005000u : 0x4c004c00u);
    constexpr int kShift = BF16 ? (FIVE ? 2 : 3) : (FIVE ? 5 : 6);
    // bytes [b0, 0, b1, 0] and [b2, 0, b3, 0], then (x << kShift) | magic per half
    const uint32_t a0 = __builtin_amdgcn_perm(0u, c0, 0x04010400u), a1 = __builtin_amdgcn_perm(0u, c0, 0x04030402u);
    const uint32_t a2 = __builtin_amdgcn_perm(0u, c1, 0x04010400u), a3 = __builtin_amdgcn_perm(0u, c1, 0x04030402u);
    return make_uint4((a0 << kShift) | kMagic, (a1 << kShift) | kMagic, (a2 << kShift) | kMagic, (a3 << kShift) | kMagic);
}

struct Rows16Q4K {
    static constexpr int kBlockBytes = 144;
    static constexpr bool kFive = false;
    struct Regs { uint4 hdr; uint2 q[4]; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int q) {
        r.hdr = *reinterpret_cast<const uint4*>(blk);
#pragma unroll
        for (int j = 0; j < 4; ++j) r.q[j] = *reinterpret_cast<const uint2*>(blk + 16 + 32 * j + 8 * q);
    }
    // code bytes of group g = 2 j + nib
    static __device__ __forceinline__ uint2 codes(const Regs& r, int j, int nib, int) {
        return nib ? make_uint2((r.q[j].x >> 4) & 0x0f0f0f0fu, (r.q[j].y >> 4) & 0x0f0f0f0fu) : make_uint2(r.q[j].x & 0x0f0f0f0fu, r.q[j].y & 0x0f0f0f0fu);
    }
};

struct Rows16Q5K {
    static constexpr int kBlockBytes = 176;
    static constexpr bool kFive = true;
    struct Regs { uint4 hdr; uint2 qh; uint2 q[4]; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int q) {
        r.hdr = *reinterpret_cast<const uint4*>(blk);
        r.qh = *reinterpret_cast<const uint2*>(blk + 16 + 8 * q);           // bit g of byte i: the fifth bit of code 8 q + i of group g
#pragma unroll
        for (int j = 0; j < 4; ++j) r.q[j] = *reinterpret_cast<const uint2*>(blk + 48 + 32 * j + 8 * q);
    }
    static __device__ __forceinline__ uint2 codes(const Regs& r, int j, int nib, int) {
        const int g = 2 * j + nib;
        const uint32_t lo = nib ? (r.q[j].x >> 4) & 0x0f0f0f0fu : r.q[j].x & 0x0f0f0f0fu;
        const uint32_t hi = nib ? (r.q[j].y >> 4) & 0x0f0f0f0fu : r.q[j].y & 0x0f0f0f0fu;
        // bit g of every qh byte to bit 4: a rotation only wraps bits that the mask drops
        const uint32_t rot = static_cast<uint32_t>(g + 28) & 31u;
        return make_uint2(lo | (__builtin_amdgcn_alignbit(r.qh.x, r.qh.x, rot) & 0x10101010u), hi | (__builtin_amdgcn_alignbit(r.qh.y, r.qh.y, rot) & 0x10101010u));
    }
};

// k = 256 bpr, weights and activation rows 16-byte aligned; grid (ceil(n / (16 TILES)), ceil(rows / 16)).
// ITERS = blocks per wave and pass (wave v: blocks v, v + WAVES, ...); every load is issued outside the branches.
template <typename FMT, bool BF16, int TILES, int WAVES, int ITERS>
__global__ __launch_bounds__(64 * WAVES) void k45_rows16_kernel(
    const uint16_t* __restrict__ x, const uint8_t* __restrict__ w, void* __restrict__ y, int y_dtype, int k, int n, int bpr, int total_rows) {
    __shared__ float partial[WAVES][TILES][64][4];
    constexpr int DEPTH = ITERS < kRows16Depth ? ITERS : kRows16Depth;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int col = lane & 15, q = lane >> 4;
    const int arow = min(static_cast<int>(blockIdx.y) * 16 + col, total_rows - 1);   // rows past the end: the last row again, result dropped
    const uint16_t* xp = x + static_cast<size_t>(arow) * k + 8 * q;
    const uint8_t* wp[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        const int wrow = min((static_cast<int>(blockIdx.x) * TILES + t) * 16 + col, n - 1);
        wp[t] = w + static_cast<size_t>(wrow) * bpr * FMT::kBlockBytes;
    }
    constexpr float kM = FMT::kFive ? 32.0f : 16.0f;
    constexpr uint32_t kOnes = BF16 ? 0x3f803f80u : 0x3c003c00u;
    const uint4 ones = make_uint4(kOnes, kOnes, kOnes, kOnes);

    v4f total[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t) total[t] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    for (int b0 = wave; b0 < bpr; b0 += WAVES * ITERS) {
        typename FMT::Regs regs[DEPTH][TILES];
        uint4 areg[2][8];
        auto request_w = [&](int it) {
            const int b = min(b0 + it * WAVES, bpr - 1);                      // (past the last block: that one again, not used)
#pragma unroll
            for (int t = 0; t < TILES; ++t) FMT::load(regs[it % DEPTH][t], wp[t] + static_cast<size_t>(b) * FMT::kBlockBytes, q);
        };
        auto request_a = [&](int it) {
            const int b = min(b0 + it * WAVES, bpr - 1);
#pragma unroll
            for (int g = 0; g < 8; ++g) areg[it & 1][g] = *reinterpret_cast<const uint4*>(xp + 256 * b + 32 * g);
        };
        request_a(0);
#pragma unroll
        for (int it = 0; it < DEPTH; ++it) request_w(it);
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            if (it + 1 < ITERS) request_a(it + 1);
            if (b0 + it * WAVES < bpr) {                                     // wave-uniform
                K4Scales sc[TILES];
                float dd[TILES], dmin[TILES];
#pragma unroll
                for (int t = 0; t < TILES; ++t) {
                    sc[t] = k4_unpack(regs[it % DEPTH][t].hdr);
                    dd[t] = f16_bits_to_float(regs[it % DEPTH][t].hdr.x & 0xffffu);
                    dmin[t] = f16_bits_to_float(regs[it % DEPTH][t].hdr.x >> 16);
                }
#pragma unroll
                for (int g = 0; g < 8; ++g) {
                    const uint4 a = areg[it & 1][g];
                    const v4f sums = half_mfma<BF16>(a, ones, v4f{0.0f, 0.0f, 0.0f, 0.0f});
#pragma unroll
                    for (int t = 0; t < TILES; ++t) {
                        const uint2 cb = FMT::codes(regs[it % DEPTH][t], g >> 1, g & 1, q);
                        const v4f c = half_mfma<BF16>(a, code_halves<BF16, FMT::kFive>(cb.x, cb.y), v4f{0.0f, 0.0f, 0.0f, 0.0f});
                        const uint32_t scw = (g < 4 ? sc[t].sc_lo : sc[t].sc_hi) >> (8 * (g & 3));
                        const uint32_t mnw = (g < 4 ? sc[t].mn_lo : sc[t].mn_hi) >> (8 * (g & 3));
                        const float ca = dd[t] * static_cast<float>(scw & 0xffu);
                        const float cs = __builtin_fmaf(kM, ca, dmin[t] * static_cast<float>(mnw & 0xffu));
                        total[t] += c * ca - sums * cs;
                    }
                }
            }
            if (it + DEPTH < ITERS) request_w(it + DEPTH);
        }
    }
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) partial[wave][t][lane][r] = total[t][r];
    __syncthreads();
    for (int e = tid; e < TILES * 256; e += 64 * WAVES) {
        const int t = e >> 8, l = (e >> 2) & 63, r = e & 3;
        float sum = 0.0f;
#pragma unroll
        for (int v = 0; v < WAVES; ++v) sum += partial[v][t][l][r];
        const int out_row = static_cast<int>(blockIdx.y) * 16 + 4 * (l >> 4) + r, out_col = (static_cast<int>(blockIdx.x) * TILES + t) * 16 + (l & 15);
        if (out_row < total_rows && out_col < n) store_any(y, y_dtype, static_cast<size_t>(out_row) * n + out_col, sum);
    }
}

template <typename FMT, int TILES, int WAVES, int ITERS>
int launch_rows16_it(const void* x, int x_dtype, const uint8_t* w, void* y, int y_dtype, int rows, int k, int n, int bpr, hipStream_t stream) {
    const dim3 grid((n + 16 * TILES - 1) / (16 * TILES), (rows + 15) / 16);
    if (x_dtype == PLLM_BF16)
        hipLaunchKernelGGL((k45_rows16_kernel<FMT, true, TILES, WAVES, ITERS>), grid, dim3(64 * WAVES), 0, stream, static_cast<const uint16_t*>(x), w, y, y_dtype, k, n, bpr, rows);
    else
        hipLaunchKernelGGL((k45_rows16_kernel<FMT, false, TILES, WAVES, ITERS>), grid, dim3(64 * WAVES), 0, stream, static_cast<const uint16_t*>(x), w, y, y_dtype, k, n, bpr, rows);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

template <typename FMT, int TILES, int WAVES>
int launch_rows16(const void* x, int x_dtype, const uint8_t* w, void* y, int y_dtype, int rows, int k, int n, int bpr, hipStream_t stream) {
    const int niter = (bpr + WAVES - 1) / WAVES;
    const int passes = (niter + 5) / 6;
    switch ((niter + passes - 1) / passes) {
        case 1: return launch_rows16_it<FMT, TILES, WAVES, 1>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream);
        case 2: return launch_rows16_it<FMT, TILES, WAVES, 2>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream);
        case 3: return launch_rows16_it<FMT, TILES, WAVES, 3>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream);
        case 4: return launch_rows16_it<FMT, TILES, WAVES, 4>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream);
        case 5: return launch_rows16_it<FMT, TILES, WAVES, 5>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream);
        default: return launch_rows16_it<FMT, TILES, WAVES, 6>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream);
    }
}

// ------------------------------------------------------------------------------------------------
// Q4_K / Q5_K, 17 - 64 activation rows (the kernel serves up to 128): the token counts between decode and the large tiles.  At these
// counts the call is bound by streaming and decoding the weights once, so every super-block is fetched by one wave, decoded once in
// its registers and multiplied into ALL activation rows; the rows reach the waves through LDS, staged once per workgroup and block.
//   v_mfma_f32_16x16x32_f16: A = 16 activation rows x the 32 columns of a scale group as fp16 values, B = 32 weights x 16 weight rows.
// B carries sc_g * code as an exact fp16 integer (at most 63 * 31 = 1953 < 2048): the code enters as 1024 + code (bits
// 0x6400 | code, one byte permute per two codes) and one packed fused multiply-add, (1024 + code) * sc - 1024 * sc, leaves
// sc * code with a single rounding, i.e. exactly.  A second B with m_g in every position accumulates m_g times the group's
// activation sum.  Both accumulate over the eight groups of a block inside the matrix core, so a block costs per 16 rows
//   y += d * C1 - dmin * C2
// and no per-group float arithmetic at all.  Workgroup = eight waves = eight tiles of 16 weight rows on one range of blocks; RG
// groups of 16 activation rows.  LDS per block: [RG][8 groups][64 lanes][16 B] in operand order (a wave's read is one contiguous
// kilobyte), two blocks at a time.  The matrix is cut along K into `slices` until two workgroups per compute unit exist; the
// partial sums leave in the order the lanes hold them and are added in slice order by k45_rows64_reduce_kernel (deterministic).
// ------------------------------------------------------------------------------------------------
constexpr int kR64Waves = 8;
typedef _Float16 v2hf __attribute__((ext_vector_type(2)));

// eight code bytes (two dwords) and the group's 6-bit scale -> eight fp16 values sc * code
__device__ __forceinline__ uint4 scaled_code_halves(uint32_t c0, uint32_t c1, uint32_t scale) {
    union { uint32_t u; v2hf h; } s2, off, in, out;
    const _Float16 sh = static_cast<_Float16>(static_cast<unsigned short>(scale));
    s2.h = v2hf{sh, sh};
    off.h = s2.h * static_cast<_Float16>(-1024.0f);                          // exact: at most 63 * 2^10
    uint32_t r[4];
    const uint32_t pairs[4] = {__builtin_amdgcn_perm(0x64646464u, c0, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, c0, 0x04030402u),
                               __builtin_amdgcn_perm(0x64646464u, c1, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, c1, 0x04030402u)};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        in.u = pairs[i];
        out.h = __builtin_elementwise_fma(in.h, s2.h, off.h);
        r[i] = out.u;
    }
    return make_uint4(r[0], r[1], r[2], r[3]);
}

// A workgroup's partial sums leave in the order the lanes hold them: [slice][row group z][column group][wave][i][lane] float4s
// (rows 4 q .. 4 q + 3 of row group i against one weight row), one contiguous kilobyte per wave and store.
template <int RG>
__device__ __forceinline__ void rows64_store_partial(float* __restrict__ partial, const v4f (&acc)[RG], int wave, int lane) {
    const size_t wg = (static_cast<size_t>(blockIdx.y) * gridDim.z + blockIdx.z) * gridDim.x + blockIdx.x;
    v4f* dst = reinterpret_cast<v4f*>(partial) + (wg * kR64Waves + wave) * (RG * 64) + lane;
#pragma unroll
    for (int i = 0; i < RG; ++i) dst[i * 64] = acc[i];
}

// y[t, c] = xscale[t] * sum over the slices, in slice order, of the partial sums; thread = one float4 of the lane-order layout
// (four rows of one column), per_slice = float4s per slice
template <int RG>
__global__ __launch_bounds__(256) void k45_rows64_reduce_kernel(const float* __restrict__ partial, const float* __restrict__ xscale, void* __restrict__ y,
                                                                int y_dtype, int t_rows, int n, int cols, int per_slice, int slices) {
    const int idx = static_cast<int>(blockIdx.x) * 256 + static_cast<int>(threadIdx.x);
    if (idx >= per_slice) return;
    const int lane = idx & 63, i = (idx >> 6) % RG, wave = (idx / (64 * RG)) % kR64Waves;
    const int wg = idx / (64 * RG * kR64Waves), cg = wg % cols, z = wg / cols;
    const int c = (cg * kR64Waves + wave) * 16 + (lane & 15), t = (z * RG + i) * 16 + 4 * (lane >> 4);
    if (c >= n || t >= t_rows) return;
    const v4f* src = reinterpret_cast<const v4f*>(partial) + idx;
    // eight slices requested at a time, added in slice order
    v4f s = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    int k = 0;
    for (; k + 8 <= slices; k += 8) {
        v4f part[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) part[j] = src[static_cast<size_t>(k + j) * per_slice];
#pragma unroll
        for (int j = 0; j < 8; ++j) s += part[j];
    }
    {
        v4f part[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) part[j] = src[static_cast<size_t>(min(k + j, slices - 1)) * per_slice];
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (k + j < slices) s += part[j];
    }
#pragma unroll
    for (int r = 0; r < 4; ++r)
        if (t + r < t_rows) store_plain(y, y_dtype, static_cast<size_t>(t + r) * n + c, xscale ? s[r] * xscale[t + r] : s[r]);
}

// The rows are 16-bit values, 256 bpr to a row, 16-byte aligned: fp16 rows (the caller's own, or rows staged by a launch before
// this one under one power of two per row, xscale, which the stores multiply back in) go into the operand-order LDS buffers
// unchanged.  bf16 rows (BF16, the caller's own: no staging launch) become fp16 on the way: every trip (two blocks) scales each of
// its rows by the power of two that brings the row's largest magnitude IN THAT TRIP to [2^14, 2^15) (the waves meet in an LDS
// maximum per row), so the conversion is exact for every value within 2^-28 of that maximum, and the trip's sums are scaled back
// per row before they join the accumulators.  Four waves per SIMD (two workgroups per compute unit) are what hides a trip's round
// trip to memory, hence the register bound; the few values it pushes to scratch are loop-invariant addresses.
template <typename FMT, int RG, bool BF16>
__global__ __launch_bounds__(64 * kR64Waves, 4) void k45_rows64_kernel(
    const uint16_t* __restrict__ x, const float* __restrict__ xscale, const uint8_t* __restrict__ w, void* __restrict__ y, int y_dtype,
    float* __restrict__ partial, int t_rows, int n, int bpr, int blocks_per_slice) {
    __shared__ __align__(16) unsigned char abuf[2][RG * 8 * 1024];
    __shared__ __align__(16) uint32_t rmax[2][16 * RG];                      // float32 bits of a trip's row maxima (sign dropped); trips alternate
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int col = lane & 15, q = lane >> 4;
    const int wrow = min((static_cast<int>(blockIdx.x) * kR64Waves + wave) * 16 + col, n - 1);   // rows past the end: the last row again, dropped at the store
    const uint8_t* wp = w + static_cast<size_t>(wrow) * bpr * FMT::kBlockBytes;
    const int b_begin = static_cast<int>(blockIdx.y) * blocks_per_slice, b_end = min(bpr, b_begin + blocks_per_slice);
    const int t0 = static_cast<int>(blockIdx.z) * 16 * RG;
    // wave v brings the pieces (rg, g) = (i, v) of a block, i < RG; lane (col, q): 8 values of activation row 16 rg + col
    uint32_t ao[RG];                                                         // (element offsets: at most 128 rows of bpr blocks)
#pragma unroll
    for (int i = 0; i < RG; ++i) ao[i] = static_cast<uint32_t>(min(t0 + 16 * i + col, t_rows - 1)) * (256u * bpr) + 32u * wave + 8u * q;
    if constexpr (BF16) {
        if (tid < 2 * 16 * RG) (&rmax[0][0])[tid] = 0u;
        __syncthreads();
    }

    v4f acc[RG];
#pragma unroll
    for (int i = 0; i < RG; ++i) acc[i] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    auto multiply = [&](const typename FMT::Regs& r, int buf, int trip) {
        const K4Scales sc = k4_unpack(r.hdr);
        v4f c1[RG], c2[RG];
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            const uint2 cb = FMT::codes(r, g >> 1, g & 1, q);
            const uint32_t scg = ((g < 4 ? sc.sc_lo : sc.sc_hi) >> (8 * (g & 3))) & 0xffu;
            const uint32_t mng = ((g < 4 ? sc.mn_lo : sc.mn_hi) >> (8 * (g & 3))) & 0xffu;
            const uint4 bc = scaled_code_halves(cb.x, cb.y, scg);
            union { uint32_t u; v2hf h; } m2;
            const _Float16 mh = static_cast<_Float16>(static_cast<unsigned short>(mng));
            m2.h = v2hf{mh, mh};
            const uint4 bm = make_uint4(m2.u, m2.u, m2.u, m2.u);
#pragma unroll
            for (int i = 0; i < RG; ++i) {
                const uint4 a = *reinterpret_cast<const uint4*>(&abuf[buf][(i * 8 + g) * 1024 + lane * 16]);
                c1[i] = half_mfma<false>(a, bc, g == 0 ? v4f{0.0f, 0.0f, 0.0f, 0.0f} : c1[i]);
                c2[i] = half_mfma<false>(a, bm, g == 0 ? v4f{0.0f, 0.0f, 0.0f, 0.0f} : c2[i]);
            }
        }
        const float dd = f16_bits_to_float(r.hdr.x & 0xffffu), dmin = f16_bits_to_float(r.hdr.x >> 16);
#pragma unroll
        for (int i = 0; i < RG; ++i) {
            if constexpr (BF16) {
                // the sums of rows 4 q .. 4 q + 3 go back by 2^(E - 141), E as at the conversion
                const uint4 mr = *reinterpret_cast<const uint4*>(&rmax[trip][16 * i + 4 * q]);
                const v4f back = v4f{__uint_as_float((max(mr.x >> 23, 15u) - 14u) << 23), __uint_as_float((max(mr.y >> 23, 15u) - 14u) << 23),
                                     __uint_as_float((max(mr.z >> 23, 15u) - 14u) << 23), __uint_as_float((max(mr.w >> 23, 15u) - 14u) << 23)};
                acc[i] += (c1[i] * dd - c2[i] * dmin) * back;
            } else {
                acc[i] += c1[i] * dd - c2[i] * dmin;
            }
        }
    };
    // two bf16 values in a dword -> two fp16 values, both times `mult`
    auto halves = [](uint32_t pair, float mult) -> uint32_t {
        union { __fp16 __attribute__((ext_vector_type(2))) h; uint32_t u; } o;
        o.h = __builtin_amdgcn_cvt_pkrtz(__uint_as_float(pair << 16) * mult, __uint_as_float(pair & 0xffff0000u) * mult);
        return o.u;
    };
    // Two blocks per trip, everything a trip needs requested at once; the two workgroups of a compute unit overlap their trips.
    int trip = 0;
    for (int b = b_begin; b < b_end; b += 2, trip ^= 1) {
        const int b1 = min(b + 1, b_end - 1);                                // (past the last block: that one again, not used)
        typename FMT::Regs r0, r1;
        u32x4 a0[RG], a1[RG];
        FMT::load(r0, wp + static_cast<size_t>(b) * FMT::kBlockBytes, q);
        FMT::load(r1, wp + static_cast<size_t>(b1) * FMT::kBlockBytes, q);
#pragma unroll
        for (int i = 0; i < RG; ++i) {
            a0[i] = *reinterpret_cast<const u32x4*>(x + (ao[i] + 256u * b));
            a1[i] = *reinterpret_cast<const u32x4*>(x + (ao[i] + 256u * b1));
        }
        if constexpr (BF16) {
#pragma unroll
            for (int i = 0; i < RG; ++i) {
                // the larger of two packed magnitudes per half, then of the halves; as float32 bits the comparison is the values'
                uint32_t m = 0u;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t u0 = a0[i][j] & 0x7fff7fffu, u1 = a1[i][j] & 0x7fff7fffu;
                    m = max(m, max(max(u0 << 16, u0 & 0xffff0000u), max(u1 << 16, u1 & 0xffff0000u)));
                }
                atomicMax(&rmax[trip][16 * i + col], m);
            }
            __syncthreads();                                                 // the maxima are whole; everybody has left the buffers of the trip before
            if (tid < 16 * RG) rmax[trip ^ 1][tid] = 0u;                     // (last read before this barrier, next written after the one below)
#pragma unroll
            for (int i = 0; i < RG; ++i) {
                // exponent field E of the row maximum (at least 15, so that this power of two and the one the sums go back by are
                // ordinary numbers): the row is multiplied by 2^(141 - E)
                const uint32_t e = max(rmax[trip][16 * i + col] >> 23, 15u);
                const float mult = __uint_as_float((268u - e) << 23);
                u32x4 h0, h1;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    h0[j] = halves(a0[i][j], mult);
                    h1[j] = halves(a1[i][j], mult);
                }
                *reinterpret_cast<u32x4*>(&abuf[0][(i * 8 + wave) * 1024 + lane * 16]) = h0;
                *reinterpret_cast<u32x4*>(&abuf[1][(i * 8 + wave) * 1024 + lane * 16]) = h1;
            }
        } else {
            if (b > b_begin) __syncthreads();                                // everybody has left the buffers of the trip before
#pragma unroll
            for (int i = 0; i < RG; ++i) {
                *reinterpret_cast<u32x4*>(&abuf[0][(i * 8 + wave) * 1024 + lane * 16]) = a0[i];
                *reinterpret_cast<u32x4*>(&abuf[1][(i * 8 + wave) * 1024 + lane * 16]) = a1[i];
            }
        }
        __syncthreads();
        multiply(r0, 0, trip);
        if (b + 1 < b_end) multiply(r1, 1, trip);
    }

    if (partial) {
        rows64_store_partial<RG>(partial, acc, wave, lane);
        return;
    }
    const int out_col = (static_cast<int>(blockIdx.x) * kR64Waves + wave) * 16 + col;
    if (out_col >= n) return;
#pragma unroll
    for (int i = 0; i < RG; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = t0 + 16 * i + 4 * q + r;
            if (row < t_rows) store_plain(y, y_dtype, static_cast<size_t>(row) * n + out_col, xscale ? acc[i][r] * xscale[row] : acc[i][r]);
        }
}

// column groups of 128 weight rows, cut along K until about two workgroups per compute unit exist
struct Rows64Plan { int rg, zs, t_pad, cols, slices, bps; };
Rows64Plan plan_rows64(int rows, int n, int bpr) {
    Rows64Plan p;
    p.rg = rows <= 32 ? 2 : 4;
    p.zs = (rows + 16 * p.rg - 1) / (16 * p.rg);
    p.t_pad = p.zs * 16 * p.rg;
    p.cols = (n + 16 * kR64Waves - 1) / (16 * kR64Waves);
    const int want = 2 * compute_units() / (p.cols * p.zs);                 // all workgroups resident at once, two per compute unit
    int slices = want < 1 ? 1 : (want > bpr ? bpr : want);
    p.bps = (bpr + slices - 1) / slices;
    p.slices = (bpr + p.bps - 1) / p.bps;
    return p;
}

template <typename FMT, bool BF16>
int launch_rows64(const Rows64Plan& p, const uint16_t* x, const float* xscale, const uint8_t* w, void* y, int y_dtype, float* partial,
                      int rows, int n, int bpr, hipStream_t stream) {
    const dim3 grid(p.cols, p.slices, p.zs);
    float* part = p.slices > 1 ? partial : nullptr;
    if (p.rg == 2) hipLaunchKernelGGL((k45_rows64_kernel<FMT, 2, BF16>), grid, dim3(64 * kR64Waves), 0, stream, x, xscale, w, y, y_dtype, part, rows, n, bpr, p.bps);
    else hipLaunchKernelGGL((k45_rows64_kernel<FMT, 4, BF16>), grid, dim3(64 * kR64Waves), 0, stream, x, xscale, w, y, y_dtype, part, rows, n, bpr, p.bps);
    if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
    if (p.slices > 1) {
        const int per_slice = p.zs * p.cols * kR64Waves * p.rg * 64;
        if (p.rg == 2) hipLaunchKernelGGL(k45_rows64_reduce_kernel<2>, dim3((per_slice + 255) / 256), dim3(256), 0, stream, partial, xscale, y, y_dtype, rows, n, p.cols, per_slice, p.slices);
        else hipLaunchKernelGGL(k45_rows64_reduce_kernel<4>, dim3((per_slice + 255) / 256), dim3(256), 0, stream, partial, xscale, y, y_dtype, rows, n, p.cols, per_slice, p.slices);
        if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
    }
    return PLLM_OK;
}

}  // namespace

size_t kquant_matvec_workspace_bytes(int rows, int bpr) { return act_image_256_bytes(bpr) * static_cast<size_t>(rows); }

int kquant_matvec_from_image(const ActRows& act, const uint8_t* w, int type_id, void* y, int y_dtype,
                             int rows, int n, int bpr, hipStream_t stream, WeightRoute route) {
    switch (type_id) {
        case PLLM_TYPE_Q4_K: return launch_k45<Q4K>(act, route, w, y, y_dtype, rows, n, bpr, stream);
        case PLLM_TYPE_Q5_K: return launch_k45<Q5K>(act, route, w, y, y_dtype, rows, n, bpr, stream);
        default: return PLLM_ERR_UNSUPPORTED;
    }
}

// Down projection of one token's routed experts with the SwiGLU ahead of it and the ordered sum over the routes behind it in one
// launch: y[n] (+)= sum over routes r, in route order, of W_{e(r)} (SiLU(gate[r]) * up[r] * route_w[r]); Q4_K, Q5_K, IQ4_XS, Q6_K
// and Q2_K, up to kMaxWaves routes (PLLM_ERR_UNSUPPORTED otherwise).  route carries the expert numbers and the expert stride.
bool kquant_route_sum_supports(int type_id, int routes, int k, const uint8_t* w, size_t expert_stride) {
    if (routes < 1 || routes > kMaxWaves || k < 4) return false;
    unsigned need;                                                            // the formats' block boundaries
    switch (type_id) {
        case PLLM_TYPE_Q4_K: case PLLM_TYPE_Q5_K: need = 15u; break;
        case PLLM_TYPE_IQ4_XS: need = 7u; break;
        case PLLM_TYPE_Q2_K: need = 3u; break;
        case PLLM_TYPE_Q6_K: need = 1u; break;
        default: return false;
    }
    return ((reinterpret_cast<uintptr_t>(w) | expert_stride) & need) == 0;
}
int kquant_route_sum_matvec(const float* gate, const float* up, const float* route_w, float limit, int k, const WeightRoute& route, const uint8_t* w,
                            int type_id, void* y, int y_dtype, int n, int bpr, int routes, hipStream_t stream) {
    if (!routed(route) || route.extra != 0 || !kquant_route_sum_supports(type_id, routes, k, w, route.expert_stride)) return PLLM_ERR_UNSUPPORTED;
    switch (type_id) {
        case PLLM_TYPE_Q4_K: return launch_wave_route_sum<Q4K>(gate, up, route_w, limit, k, route, w, y, y_dtype, n, bpr, routes, stream);
        case PLLM_TYPE_Q5_K: return launch_wave_route_sum<Q5K>(gate, up, route_w, limit, k, route, w, y, y_dtype, n, bpr, routes, stream);
        case PLLM_TYPE_IQ4_XS: return launch_wave_route_sum<IQ4XS>(gate, up, route_w, limit, k, route, w, y, y_dtype, n, bpr, routes, stream);
        case PLLM_TYPE_Q6_K: return launch_groups16_route_sum<WaveQ6K>(gate, up, route_w, limit, k, route, w, y, y_dtype, n, bpr, routes, stream);
        case PLLM_TYPE_Q2_K: return launch_groups16_route_sum<WaveQ2K>(gate, up, route_w, limit, k, route, w, y, y_dtype, n, bpr, routes, stream);
        default: return PLLM_ERR_UNSUPPORTED;
    }
}

int iq4xs_wave_matvec(const ActRows& act, const uint8_t* w, void* y, int y_dtype, int rows, int n, int bpr, hipStream_t stream, WeightRoute route) {
    // raw rows, blocks (of every expert) on an 8-byte boundary, no normalisation in routed calls; everything else stays with the tile-frame kernel
    if (!act.x || act.k < 4 || ((reinterpret_cast<uintptr_t>(w) | route.expert_stride) & 7u)) return PLLM_ERR_UNSUPPORTED;
    if (act.gamma && (routed(route) || act.row_token || act.x_broadcast)) return PLLM_ERR_UNSUPPORTED;
    for (int m = 0; m < route.extra; ++m)
        if (reinterpret_cast<uintptr_t>(route.more_w[m]) & 7u) return PLLM_ERR_UNSUPPORTED;
    return act.gamma ? launch_wave<IQ4XS, true>(act, route, w, y, y_dtype, rows, n, bpr, stream)
                     : launch_wave<IQ4XS, false>(act, route, w, y, y_dtype, rows, n, bpr, stream);
}

int groups16_wave_matvec(const ActRows& act, const uint8_t* w, int type_id, void* y, int y_dtype, int rows, int n, int bpr, hipStream_t stream, WeightRoute route) {
    if (type_id == PLLM_TYPE_Q2_K) return launch_groups16<WaveQ2K>(act, route, w, y, y_dtype, rows, n, bpr, stream);
    if (type_id == PLLM_TYPE_Q6_K) return launch_groups16<WaveQ6K>(act, route, w, y, y_dtype, rows, n, bpr, stream);
    return PLLM_ERR_UNSUPPORTED;
}

// Q4_K / Q5_K on 2 - 16 raw rows of bf16 / fp16 activations whose length is a whole number of super-blocks (PLLM_ERR_UNSUPPORTED otherwise)
int k45_rows16_matvec(const void* x, int x_dtype, const uint8_t* w, int type_id, void* y, int y_dtype, int rows, int k, int n, int bpr, hipStream_t stream) {
    if ((type_id != PLLM_TYPE_Q4_K && type_id != PLLM_TYPE_Q5_K) || (x_dtype != PLLM_BF16 && x_dtype != PLLM_F16)) return PLLM_ERR_UNSUPPORTED;
    if (rows < 2 || k != 256 * bpr || ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15u)) return PLLM_ERR_UNSUPPORTED;
    // one tile per wave and four waves on matrices of many tiles of short rows; long rows and matrices of few tiles run two tiles per
    // wave (which share the activation operands) on eight waves (Q4_K, us at 2 / 4 / 8 / 16 rows: 17408x5120 22.7 / 23.8 / 26.3 / 33.9
    // against 28.4 / 29.6 / 31.4 / 37.4; 5120x17408 30.5 / 32.0 / 36.0 / 46.6 against 30.3 / 31.4 / 33.3 / 38.6; 5120x5120 11.3 / 11.7 /
    // 12.9 / 15.7 against 10.6 / 10.9 / 11.5 / 13.7)
    const bool two_tiles = k >= 8192 || n < 8192;
    if (type_id == PLLM_TYPE_Q4_K)
        return two_tiles ? launch_rows16<Rows16Q4K, 2, 8>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream)
                         : launch_rows16<Rows16Q4K, 1, 4>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream);
    return two_tiles ? launch_rows16<Rows16Q5K, 2, 8>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream)
                     : launch_rows16<Rows16Q5K, 1, 4>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream);
}

}  // namespace pllm

namespace pllm {
// Q4_K / Q5_K on 17 - 48 activation rows (float32 rows, and bf16 rows on large matrices, are staged as scaled fp16 rows by a launch
// of their own first; fp16 rows, and bf16 rows on matrices of up to kRows64SmallWeights weights, are read as the caller holds
// them).  Operator calls in us, Q4_K, 17 / 32 / 48 / 64 rows:
//   5120x5120    staged 19.1 / 21.4 / - / 27.9     bf16 as held 16.4 / 18.2 / 24.9 / 25.8     fp16 as held 15.4 / 17.1 / 21.3 / 23.3     tile kernel 26.2 / 26.2 / - / 27.7
//   17408x5120   staged 31.0 / 32.8 / - / 44.6     bf16 as held 32.1 / 33.3 / 52.0 / 51.6     fp16 as held 27.4 / 29.6 / 40.9 / 43.4     tile kernel 40.9 / 41.0 / - / 43.0
// (converting bf16 rows inside the kernel repeats the conversion in every column group: 136 of them at 17408 weight rows), so rows
// read as held are served up to 64 on the small matrices and everything else up to 48; the kernels themselves take up to 128.
constexpr int64_t kRows64SmallWeights = int64_t{48} << 20;
bool k45_rows64_reads_raw(const void* x, int x_dtype, int k, int n, int bpr) {
    if (k != 256 * bpr || (reinterpret_cast<uintptr_t>(x) & 15u) != 0) return false;
    return x_dtype == PLLM_F16 || (x_dtype == PLLM_BF16 && static_cast<int64_t>(n) * k <= kRows64SmallWeights);
}
bool k45_rows64_supports(int type_id, int rows, int n, int bpr, const uint8_t* w, bool raw16) {
    const int most = raw16 && static_cast<int64_t>(n) * bpr * 256 <= kRows64SmallWeights ? 64 : 48;
    return (type_id == PLLM_TYPE_Q4_K || type_id == PLLM_TYPE_Q5_K) && rows > 16 && rows <= most && n >= 16 && bpr >= 1 &&
           (reinterpret_cast<uintptr_t>(w) & 15u) == 0;
}
size_t k45_rows64_workspace_bytes(int rows, int n, int bpr) {
    const Rows64Plan p = plan_rows64(rows, n, bpr);
    const size_t part = p.slices > 1 ? align256(static_cast<size_t>(p.slices) * p.t_pad * p.cols * (16 * kR64Waves) * sizeof(float)) : 0;
    return gemm_f16_staged_bytes(rows, bpr) + part;
}
int k45_rows64_gemm(const void* x, int x_dtype, const uint8_t* w, int type_id, void* y, int y_dtype, int rows, int k, int n, int bpr,
                    void* workspace, size_t workspace_bytes, hipStream_t stream) {
    const bool raw16 = k45_rows64_reads_raw(x, x_dtype, k, n, bpr);
    if (!k45_rows64_supports(type_id, rows, n, bpr, w, raw16) || (y_dtype & kAccumulateInto)) return PLLM_ERR_UNSUPPORTED;
    if (!workspace || workspace_bytes < k45_rows64_workspace_bytes(rows, n, bpr)) return PLLM_ERR_WORKSPACE;
    const Rows64Plan p = plan_rows64(rows, n, bpr);
    float* partial = reinterpret_cast<float*>(static_cast<unsigned char*>(workspace) + gemm_f16_staged_bytes(rows, bpr));
    const uint16_t* xr = static_cast<const uint16_t*>(x);
    const float* xscale = nullptr;
    bool bf16 = x_dtype == PLLM_BF16;
    if (!raw16) {
        // staged as fp16 rows of 256 bpr values, each under one power of two (xscale), which the kernel then reads like fp16 rows
        const int st = gemm_f16_stage_rows(x, x_dtype, nullptr, rows, k, bpr, workspace, stream);
        if (st != PLLM_OK) return st;
        xr = static_cast<const uint16_t*>(workspace);
        xscale = reinterpret_cast<const float*>(static_cast<const unsigned char*>(workspace) + align256(static_cast<size_t>(rows) * bpr * 256 * sizeof(_Float16)));
        bf16 = false;
    }
    if (type_id == PLLM_TYPE_Q4_K)
        return bf16 ? launch_rows64<Rows16Q4K, true>(p, xr, xscale, w, y, y_dtype, partial, rows, n, bpr, stream)
                    : launch_rows64<Rows16Q4K, false>(p, xr, xscale, w, y, y_dtype, partial, rows, n, bpr, stream);
    return bf16 ? launch_rows64<Rows16Q5K, true>(p, xr, xscale, w, y, y_dtype, partial, rows, n, bpr, stream)
                : launch_rows64<Rows16Q5K, false>(p, xr, xscale, w, y, y_dtype, partial, rows, n, bpr, stream);
}
}  // namespace pllm
