// Prefill matmul y[T, N] = x[T, K] . dequant(W)[N, K]^T over raw super-blocks, on f16 MFMA.
//
// A workgroup of eight waves owns a BM (tokens, 64 / 128 / 256) x 256 (weight rows) output tile and
// walks K in chunks of 32 weights (one sub-block).  Per pair of chunks every thread pulls 16 bytes of
// codes plus the block header straight from the raw tensor and its share of the activations; per
// chunk it decodes 16 weights in float32 exactly as the block decoders do, rounds them once to fp16
// and stores them in LDS.  The activations arrive as fp16 (a pre-pass scales every token row by a
// power of two so that its largest value sits just below 2^14, which keeps bf16 inputs exact and
// cannot overflow).  The waves (2 x 4) run v_mfma_f32_32x32x16_f16 on (BM/2) x 64 sub-tiles with
// float32 accumulators: with BM = 256 a wave feeds eight MFMAs from six 16-byte LDS reads.  LDS is
// double buffered and the raw registers come in two sets, so the loads of the chunk pair after next
// and the decode of chunk c+1 overlap the MFMAs of chunk c, with one barrier per chunk; inside a
// step the decode instructions are woven between the MFMAs so that both units stay busy.
//
// The grid is one-dimensional.  Tiles that fill whole rounds of the machine (one workgroup per
// compute unit) run over all of K and store their result directly; the tiles left over, which
// would occupy a fraction of the machine for a full round, are cut along K in slices: every slice
// writes a float32 partial tile and a second kernel adds them in slice order, which keeps the
// result independent of scheduling.  Small token counts consist of left-over tiles only.
//
// Why fp16 tiles and not int8 MFMA here: with int8 activations every 32-wide group needs a float
// fix-up per output (two scales that change along K), which costs more vector instructions than
// the MFMA saves, and a single int8 activation term sits at ~5e-3 from the float statement of the
// operator.  Decoded-to-fp16 tiles need no fix-up, keep bf16 activations exact and land at ~2e-4.
#include "block_dot4.h"
#include "pllm_internal.h"

namespace pllm {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kBN = 256, kBK = 32, kThreads = 512;
constexpr int kLds = kBK + 8;                       // halves per LDS row: 80 bytes, conflict-free for 16-byte reads

// ---- activation pre-pass --------------------------------------------------------------------------
// xh[t, 0..kp) = fp16(x[t, :] * 2^-e_t) (zero beyond k), scale[t] = 2^e_t, amax_t * 2^-e_t in [2^13, 2^14)
__global__ __launch_bounds__(256) void act_f16_kernel(const void* __restrict__ x, int x_dtype, _Float16* __restrict__ xh,
                                                      float* __restrict__ scale, int k, int kp, const int64_t* __restrict__ row_map) {
    __shared__ float red[4];
    const size_t xoff = static_cast<size_t>(row_map ? row_map[blockIdx.x] : blockIdx.x) * k;      // row_map gathers source rows
    float am = 0.0f;
    for (int i = threadIdx.x; i < k; i += 256) am = fmaxf(am, fabsf(load_any(x, x_dtype, xoff + i)));
    am = group_max<64>(am);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = am;
    __syncthreads();
    am = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    int e = 0;
    if (am > 0.0f && am < __uint_as_float(0x7f800000u)) {
        (void)frexpf(am, &e);                       // am = m * 2^e, m in [0.5, 1)
        e -= 14;
    }
    const float down = ldexpf(1.0f, -e);
    _Float16* out = xh + static_cast<size_t>(blockIdx.x) * kp;
    for (int i = threadIdx.x; i < kp; i += 256)
        out[i] = static_cast<_Float16>(i < k ? load_any(x, x_dtype, xoff + i) * down : 0.0f);
    if (threadIdx.x == 0) scale[blockIdx.x] = ldexpf(1.0f, e);
}

// The same for rows of at most 8192 values with 16-bit inputs (the usual case): one wave per row
// keeps the row in registers between the maximum and the conversion, so x is read once.
// bits(v) = the value as float32: bf16 is the high half of a float32, fp16 converts in hardware.
// WPR = waves per row: 1 (four rows per workgroup) or 4 (one row per workgroup, for calls of few rows: four times the
// workgroups, a quarter of the row per wave; the waves meet in LDS for the maximum).
template <bool BF16, int WPR>
__global__ __launch_bounds__(256) void act_f16_rows_kernel(const uint16_t* __restrict__ x, _Float16* __restrict__ xh,
                                                           float* __restrict__ scale, int rows, int k, int kp, const int64_t* __restrict__ row_map) {
    __shared__ float wave_max[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = WPR == 1 ? blockIdx.x * 4 + wave : blockIdx.x, part = WPR == 1 ? 0 : wave;
    if (row >= rows) return;                       // (a whole workgroup when WPR = 4)
    const uint16_t* src = x + static_cast<size_t>(row_map ? row_map[row] : row) * k;
    constexpr int kMaxPieces = 16 / WPR;           // 16 pieces x 64 lanes x 8 values per row
    uint4 piece[kMaxPieces];
    float am = 0.0f;
    auto value = [](uint32_t word, int hi) -> float {
        const uint32_t h = hi ? (word >> 16) : (word & 0xffffu);
        if (BF16) return __uint_as_float(h << 16);
        return f16_bits_to_float(h);
    };
#pragma unroll
    for (int i = 0; i < kMaxPieces; ++i) {
        const int e0 = ((i * WPR + part) * 64 + lane) * 8;
        piece[i] = make_uint4(0, 0, 0, 0);
        if (e0 < k) piece[i] = *reinterpret_cast<const uint4*>(src + e0);          // k is a multiple of 8 here
        const uint32_t wds[4] = {piece[i].x, piece[i].y, piece[i].z, piece[i].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) am = fmaxf(am, fmaxf(fabsf(value(wds[j], 0)), fabsf(value(wds[j], 1))));
    }
    am = group_max<64>(am);
    if constexpr (WPR > 1) {
        if (lane == 0) wave_max[wave] = am;
        __syncthreads();
        am = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
    }
    int e = 0;
    if (am > 0.0f && am < __uint_as_float(0x7f800000u)) {
        (void)frexpf(am, &e);
        e -= 14;
    }
    const float down = ldexpf(1.0f, -e);
    _Float16* out = xh + static_cast<size_t>(row) * kp;
#pragma unroll
    for (int i = 0; i < kMaxPieces; ++i) {
        const int e0 = ((i * WPR + part) * 64 + lane) * 8;
        if (e0 >= kp) continue;
        const uint32_t wds[4] = {piece[i].x, piece[i].y, piece[i].z, piece[i].w};
        half8 o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            o[2 * j] = static_cast<_Float16>(value(wds[j], 0) * down);
            o[2 * j + 1] = static_cast<_Float16>(value(wds[j], 1) * down);
        }
        *reinterpret_cast<half8*>(out + e0) = o;
    }
    if (lane == 0 && part == 0) scale[row] = ldexpf(1.0f, e);
}

// Hidden activations of the routed experts, one wave per route: h = silu(min(g, L)) * clamp(u, +-L) * w_r
// (L <= 0: no clamp) from the float32 gate / up products, written as fp16 rows scaled like the ones above.
__global__ __launch_bounds__(256) void swiglu_f16_rows_kernel(const float* __restrict__ g, const float* __restrict__ u,
                                                              const float* __restrict__ route_weights, float limit, _Float16* __restrict__ hh,
                                                              float* __restrict__ scale, int rows, int inter, int kp) {
    const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* gr = g + static_cast<size_t>(row) * inter;
    const float* ur = u + static_cast<size_t>(row) * inter;
    const float rw = route_weights[row];
    auto hidden = [&](int i) {
        float gv = gr[i], uv = ur[i];
        if (limit > 0.0f) {
            uv = fminf(fmaxf(uv, -limit), limit);
            gv = fminf(gv, limit);
        }
        return gv / (1.0f + expf(-gv)) * uv * rw;
    };
    float am = 0.0f;
    for (int i = lane; i < inter; i += 64) am = fmaxf(am, fabsf(hidden(i)));
    am = group_max<64>(am);
    int e = 0;
    if (am > 0.0f && am < __uint_as_float(0x7f800000u)) {
        (void)frexpf(am, &e);
        e -= 14;
    }
    const float down = ldexpf(1.0f, -e);
    _Float16* out = hh + static_cast<size_t>(row) * kp;
    for (int i = lane; i < kp; i += 64) out[i] = static_cast<_Float16>(i < inter ? hidden(i) * down : 0.0f);
    if (lane == 0) scale[row] = ldexpf(1.0f, e);
}

// ---- per-format decode of one 32-weight chunk -----------------------------------------------------
// Staging thread (row, h) decodes weights [32 j + 16 h, +16) of its row for sub-block j = 2 p + e.
struct K4Scale { float d_sc, dm; };
__device__ __forceinline__ K4Scale k4_scale(const uint4& hdr, int p, int e) {
    const uint32_t u0 = hdr.y, u1 = hdr.z, u2 = hdr.w;
    uint32_t scw, mnw;
    if (p < 2) {
        scw = (u0 & 0x3f3f3f3fu) >> (16 * p);
        mnw = (u1 & 0x3f3f3f3fu) >> (16 * p);
    } else {
        scw = ((u2 & 0x0f0f0f0fu) | (((u0 >> 6) & 0x03030303u) << 4)) >> (16 * (p - 2));
        mnw = (((u2 >> 4) & 0x0f0f0f0fu) | (((u1 >> 6) & 0x03030303u) << 4)) >> (16 * (p - 2));
    }
    const float d = f16_bits_to_float(hdr.x & 0xffffu), dmin = f16_bits_to_float(hdr.x >> 16);
    K4Scale r;
    r.d_sc = d * static_cast<float>((scw >> (8 * e)) & 0xffu);
    r.dm = dmin * static_cast<float>((mnw >> (8 * e)) & 0xffu);
    return r;
}

// four byte-sized codes of one word -> fp16(scale * code - minus)
__device__ __forceinline__ half4 affine4(uint32_t codes, float scale, float minus) {
    half4 r;
    r.x = static_cast<_Float16>(scale * static_cast<float>(codes & 0xffu) - minus);
    r.y = static_cast<_Float16>(scale * static_cast<float>((codes >> 8) & 0xffu) - minus);
    r.z = static_cast<_Float16>(scale * static_cast<float>((codes >> 16) & 0xffu) - minus);
    r.w = static_cast<_Float16>(scale * static_cast<float>(codes >> 24) - minus);
    return r;
}

struct Half16 { half4 a, b, c, d; };

struct GQ4K {
    static constexpr int kTableBytes = 0;
    static __device__ __forceinline__ void stage_table(unsigned char*) {}
    static constexpr int kBlockBytes = 144;
    struct Regs { uint4 hdr; uint4 qs; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, const float*, int, int p, int h) {
        r.hdr = *reinterpret_cast<const uint4*>(blk);
        r.qs = *reinterpret_cast<const uint4*>(blk + 16 + 32 * p + 16 * h);
    }
    static __device__ __forceinline__ void decode(const Regs& r, int p, int e, int, const unsigned char*, Half16& o) {
        const K4Scale s = k4_scale(r.hdr, p, e);
        const int sft = 4 * e;
        o.a = affine4((r.qs.x >> sft) & 0x0f0f0f0fu, s.d_sc, s.dm);
        o.b = affine4((r.qs.y >> sft) & 0x0f0f0f0fu, s.d_sc, s.dm);
        o.c = affine4((r.qs.z >> sft) & 0x0f0f0f0fu, s.d_sc, s.dm);
        o.d = affine4((r.qs.w >> sft) & 0x0f0f0f0fu, s.d_sc, s.dm);
    }
};

struct GQ5K {
    static constexpr int kTableBytes = 0;
    static __device__ __forceinline__ void stage_table(unsigned char*) {}
    static constexpr int kBlockBytes = 176;
    struct Regs { uint4 hdr; uint4 qh; uint4 qs; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, const float*, int, int p, int h) {
        r.hdr = *reinterpret_cast<const uint4*>(blk);
        r.qh = *reinterpret_cast<const uint4*>(blk + 16 + 16 * h);
        r.qs = *reinterpret_cast<const uint4*>(blk + 48 + 32 * p + 16 * h);
    }
    static __device__ __forceinline__ uint32_t codes(uint32_t q, uint32_t g, int sft, int bit) {
        return ((q >> sft) & 0x0f0f0f0fu) | (((g >> bit) & 0x01010101u) << 4);
    }
    static __device__ __forceinline__ void decode(const Regs& r, int p, int e, int, const unsigned char*, Half16& o) {
        const K4Scale s = k4_scale(r.hdr, p, e);
        const int sft = 4 * e, bit = 2 * p + e;
        o.a = affine4(codes(r.qs.x, r.qh.x, sft, bit), s.d_sc, s.dm);
        o.b = affine4(codes(r.qs.y, r.qh.y, sft, bit), s.d_sc, s.dm);
        o.c = affine4(codes(r.qs.z, r.qh.z, sft, bit), s.d_sc, s.dm);
        o.d = affine4(codes(r.qs.w, r.qh.w, sft, bit), s.d_sc, s.dm);
    }
};

// Q2_K: 84 B = scales(16) qs(64) d(2) dmin(2).  Chunk c = 2 p + e holds weights [32 c, +32): byte
// qs[32 (c / 4) + l] >> 2 (c % 4), l = 0..31, so both chunks of a pair read the same 16 bytes per
// thread at two shifts; the thread's 16 weights are group 2 c + h with scale byte scales[2 c + h]
// (low nibble scale, high nibble min).
struct GQ2K {
    static constexpr int kTableBytes = 0;
    static __device__ __forceinline__ void stage_table(unsigned char*) {}
    static constexpr int kBlockBytes = 84;
    struct Regs { uint4 sc; uint4 qs; uint32_t dd; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, const float*, int, int p, int h) {
        const uint32_t* w = reinterpret_cast<const uint32_t*>(blk);           // blocks are 4-byte aligned
        r.sc = make_uint4(w[0], w[1], w[2], w[3]);
        const uint32_t* q = w + 4 + 8 * (p >> 1) + 4 * h;
        r.qs = make_uint4(q[0], q[1], q[2], q[3]);
        r.dd = w[20];
    }
    static __device__ __forceinline__ void decode(const Regs& r, int p, int e, int h, const unsigned char*, Half16& o) {
        const int c = 2 * p + e, sft = 2 * (c & 3), g = 2 * c + h;
        const uint32_t word = (g < 4) ? r.sc.x : (g < 8) ? r.sc.y : (g < 12) ? r.sc.z : r.sc.w;
        const uint32_t sb = (word >> (8 * (g & 3))) & 0xffu;
        const float scale = f16_bits_to_float(r.dd & 0xffffu) * static_cast<float>(sb & 15u);
        const float minus = f16_bits_to_float(r.dd >> 16) * static_cast<float>(sb >> 4);
        o.a = affine4((r.qs.x >> sft) & 0x03030303u, scale, minus);
        o.b = affine4((r.qs.y >> sft) & 0x03030303u, scale, minus);
        o.c = affine4((r.qs.z >> sft) & 0x03030303u, scale, minus);
        o.d = affine4((r.qs.w >> sft) & 0x03030303u, scale, minus);
    }
};

typedef _Float16 half2v __attribute__((ext_vector_type(2)));

// two fp16 values in a dword, sign bits flipped by `flip`, times a float32 scale, rounded once to fp16
// (mixed-precision multiplies: the scale keeps its float32 bits)
__device__ __forceinline__ uint32_t scaled_pair(uint32_t bits, uint32_t flip, float scale) {
    const half2v v = __builtin_bit_cast(half2v, bits ^ flip);
    const half2v r = {static_cast<_Float16>(static_cast<float>(v.x) * scale), static_cast<_Float16>(static_cast<float>(v.y) * scale)};
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ half4 half4_of(uint32_t lo, uint32_t hi) {
    return __builtin_bit_cast(half4, make_uint2(lo, hi));
}

// Q6_K: 210 B = ql(128) qh(64) scales int8(16) d(2); weight 128 half + 32 j + l takes nibble j / 2 of ql[64 half + 32 (j % 2) + l], bit
// pair j of qh[32 half + l] and scale 8 half + 2 j + l / 16; w = d * scale * (q - 32).  Here half = p / 2, j = 2 (p % 2) + e, l = 16 h + ...
// Blocks are only 2-byte aligned.
struct __attribute__((packed, aligned(2))) UnalignedWord { uint32_t v; };
struct GQ6K {
    static constexpr int kTableBytes = 0;
    static __device__ __forceinline__ void stage_table(unsigned char*) {}
    static constexpr int kBlockBytes = 210;
    struct Regs { uint4 qa, qb, qh; uint32_t sc, d; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, const float*, int, int p, int h) {
        const int half = p >> 1;
        r.qa = load16_a2(blk + 64 * half + 16 * h);
        r.qb = load16_a2(blk + 64 * half + 32 + 16 * h);
        r.qh = load16_a2(blk + 128 + 32 * half + 16 * h);
        r.sc = reinterpret_cast<const UnalignedWord*>(blk + 192 + 8 * half + 4 * (p & 1))->v;   // scales 8 half + 4 (p % 2) + 0..3
        r.d = *reinterpret_cast<const uint16_t*>(blk + 208);
    }
    static __device__ __forceinline__ uint32_t codes(uint32_t ql, uint32_t qh, int nib, int pair) {
        return ((ql >> nib) & 0x0f0f0f0fu) | (((qh >> pair) & 0x03030303u) << 4);
    }
    static __device__ __forceinline__ void decode(const Regs& r, int p, int e, int h, const unsigned char*, Half16& o) {
        const int nib = 4 * (p & 1), pair = 2 * (2 * (p & 1) + e);
        const uint4 ql = e ? r.qb : r.qa;
        const float scale = f16_bits_to_float(r.d) * static_cast<float>(static_cast<int8_t>(r.sc >> (8 * (2 * e + h))));
        const float minus = 32.0f * scale;
        o.a = affine4(codes(ql.x, r.qh.x, nib, pair), scale, minus);
        o.b = affine4(codes(ql.y, r.qh.y, nib, pair), scale, minus);
        o.c = affine4(codes(ql.z, r.qh.z, nib, pair), scale, minus);
        o.d = affine4(codes(ql.w, r.qh.w, nib, pair), scale, minus);
    }
};

// IQ4_XS: 136 B = d(2) scales_h(2) scales_l(4) qs(128); group g = 2 p + e of 32 weights: bytes qs[16 g, +16), low nibbles = its first
// 16 weights (h = 0), high nibbles the others; w = d * (ls - 32) * kvalues[code].  The 16-entry table sits in four constants, biased
// by 128 so that the codes stay unsigned bytes; three byte permutes pick four values.
struct GIQ4XS {
    static constexpr int kTableBytes = 0;
    static __device__ __forceinline__ void stage_table(unsigned char*) {}
    static constexpr int kBlockBytes = 136;
    struct Regs { uint2 hdr; uint4 q0, q1; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, const float*, int, int p, int) {
        const uint2* w = reinterpret_cast<const uint2*>(blk);                 // blocks are 8-byte aligned
        r.hdr = w[0];
        r.q0 = make_uint4(w[1 + 4 * p].x, w[1 + 4 * p].y, w[2 + 4 * p].x, w[2 + 4 * p].y);
        r.q1 = make_uint4(w[3 + 4 * p].x, w[3 + 4 * p].y, w[4 + 4 * p].x, w[4 + 4 * p].y);
    }
    static __device__ __forceinline__ uint32_t biased4(uint32_t codes) {     // kvalues[code] + 128, four at a time
        const uint32_t low3 = codes & 0x07070707u;
        const uint32_t lower = __builtin_amdgcn_perm(0x766A5D4Fu, 0x3F2D1801u, low3);   // 1 24 45 63 | 79 93 106 118
        const uint32_t upper = __builtin_amdgcn_perm(0xF1D9C5B5u, 0xA6998D81u, low3);   // 129 141 153 166 | 181 197 217 241
        return __builtin_amdgcn_perm(upper, lower, ((codes >> 1) & 0x04040404u) | 0x03020100u);
    }
    static __device__ __forceinline__ void decode(const Regs& r, int p, int e, int h, const unsigned char*, Half16& o) {
        const uint4 q = e ? r.q1 : r.q0;
        const int g = 2 * p + e, sft = 4 * h;
        const uint32_t scales_h = r.hdr.x >> 16;
        const int ls = static_cast<int>(((r.hdr.y >> (8 * p + 4 * e)) & 15u) | (((scales_h >> (2 * g)) & 3u) << 4)) - 32;
        const float scale = f16_bits_to_float(r.hdr.x & 0xffffu) * static_cast<float>(ls);
        const float minus = 128.0f * scale;
        o.a = affine4(biased4((q.x >> sft) & 0x0f0f0f0fu), scale, minus);
        o.b = affine4(biased4((q.y >> sft) & 0x0f0f0f0fu), scale, minus);
        o.c = affine4(biased4((q.z >> sft) & 0x0f0f0f0fu), scale, minus);
        o.d = affine4(biased4((q.w >> sft) & 0x0f0f0f0fu), scale, minus);
    }
};

// IQ2_XXS: 66 B = d(2) + 8 sub-blocks of 8 B (four grid ids, then a u32: four 7-bit sign indices and a
// 4-bit scale).  A pair is sub-blocks 2 p and 2 p + 1; the thread takes grid entries 2 h and 2 h + 1 of
// its sub-block.  w = d (2 s + 1) / 8 * magnitude, negated where the sign pattern (seven bits plus
// their parity) says so.  The workgroup keeps two LDS tables in fp16: the 256 x 8 magnitudes (8, 25
// and 43 are exact) and the 128 x 8 sign-bit masks, so eight weights cost two 16-byte LDS reads, four
// XORs and eight mixed-precision multiplies by the float32 scale.
struct GIQ2XXS {
    static constexpr int kBlockBytes = 66;
    struct Regs { uint4 q; uint32_t d; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, const float*, int, int p, int) {
        r.q = load16_a2(blk + 2 + 16 * p);
        r.d = *reinterpret_cast<const uint16_t*>(blk);
    }
    static constexpr int kTableBytes = 4096 + 2048;
    static __device__ __forceinline__ void stage_table(unsigned char* lds) {
        _Float16* mag = reinterpret_cast<_Float16*>(lds);
        uint16_t* sgn = reinterpret_cast<uint16_t*>(lds + 4096);
        for (int i = threadIdx.x; i < 256 * 8; i += kThreads)
            mag[i] = static_cast<_Float16>(static_cast<float>((PLLM_IQ2XXS_GRID[i >> 3] >> (8 * (i & 7))) & 0xffull));
        for (int i = threadIdx.x; i < 128 * 8; i += kThreads) {
            const uint32_t s7 = static_cast<uint32_t>(i >> 3);
            const uint32_t s8 = s7 | ((__popc(s7) & 1u) << 7);
            sgn[i] = ((s8 >> (i & 7)) & 1u) ? 0x8000u : 0u;
        }
    }
    static __device__ __forceinline__ void entry(const unsigned char* table, uint32_t id, uint32_t s7, float scale, half4& lo, half4& hi) {
        const uint4 m = *reinterpret_cast<const uint4*>(table + 16 * id);
        const uint4 f = *reinterpret_cast<const uint4*>(table + 4096 + 16 * s7);
        lo = half4_of(scaled_pair(m.x, f.x, scale), scaled_pair(m.y, f.y, scale));
        hi = half4_of(scaled_pair(m.z, f.z, scale), scaled_pair(m.w, f.w, scale));
    }
    static __device__ __forceinline__ void decode(const Regs& r, int, int e, int h, const unsigned char* table, Half16& o) {
        const uint32_t ids = e ? r.q.z : r.q.x, aux = e ? r.q.w : r.q.y;
        const float scale = 0.125f * f16_bits_to_float(r.d) * static_cast<float>(2 * (aux >> 28) + 1);
        entry(table, (ids >> (16 * h)) & 0xffu, (aux >> (14 * h)) & 127u, scale, o.a, o.b);
        entry(table, (ids >> (16 * h + 8)) & 0xffu, (aux >> (14 * h + 7)) & 127u, scale, o.c, o.d);
    }
};

// IQ2_XS: 74 B = d(2) qs u16[32] scales(8).  Entry (8 weights) = 9-bit grid id + 7-bit sign index; two 4-bit scales per 32
// weights (low nibble: first 16).  The thread's 16 weights are entries 8 p + 4 e + 2 h and the next one.  LDS tables as for
// IQ2_XXS with 512 grid entries.
struct GIQ2XS {
    static constexpr int kBlockBytes = 74;
    struct Regs { uint32_t q0, q1, sc, d; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, const float*, int, int p, int h) {
        r.q0 = reinterpret_cast<const UnalignedWord*>(blk + 2 + 16 * p + 4 * h)->v;
        r.q1 = reinterpret_cast<const UnalignedWord*>(blk + 10 + 16 * p + 4 * h)->v;
        r.sc = *reinterpret_cast<const uint16_t*>(blk + 66 + 2 * p);
        r.d = *reinterpret_cast<const uint16_t*>(blk);
    }
    static constexpr int kTableBytes = 8192 + 2048;
    static __device__ __forceinline__ void stage_table(unsigned char* lds) {
        _Float16* mag = reinterpret_cast<_Float16*>(lds);
        uint16_t* sgn = reinterpret_cast<uint16_t*>(lds + 8192);
        for (int i = threadIdx.x; i < 512 * 8; i += kThreads)
            mag[i] = static_cast<_Float16>(static_cast<float>((PLLM_IQ2XS_GRID[i >> 3] >> (8 * (i & 7))) & 0xffull));
        for (int i = threadIdx.x; i < 128 * 8; i += kThreads) {
            const uint32_t s7 = static_cast<uint32_t>(i >> 3);
            const uint32_t s8 = s7 | ((__popc(s7) & 1u) << 7);
            sgn[i] = ((s8 >> (i & 7)) & 1u) ? 0x8000u : 0u;
        }
    }
    static __device__ __forceinline__ void entry(const unsigned char* table, uint32_t q16, float scale, half4& lo, half4& hi) {
        const uint4 m = *reinterpret_cast<const uint4*>(table + 16 * (q16 & 511u));
        const uint4 f = *reinterpret_cast<const uint4*>(table + 8192 + 16 * (q16 >> 9));
        lo = half4_of(scaled_pair(m.x, f.x, scale), scaled_pair(m.y, f.y, scale));
        hi = half4_of(scaled_pair(m.z, f.z, scale), scaled_pair(m.w, f.w, scale));
    }
    static __device__ __forceinline__ void decode(const Regs& r, int, int e, int h, const unsigned char* table, Half16& o) {
        const uint32_t pair = e ? r.q1 : r.q0;
        const uint32_t ls = (r.sc >> (8 * e + 4 * h)) & 15u;
        const float scale = 0.125f * f16_bits_to_float(r.d) * static_cast<float>(2 * ls + 1);
        entry(table, pair & 0xffffu, scale, o.a, o.b);
        entry(table, pair >> 16, scale, o.c, o.d);
    }
};

// IQ3_XXS: 98 B = d(2) grid ids(64) aux u32[8].  An id gives four weights; aux of a 32-weight sub-block = four 7-bit sign indices
// (one per 8 weights) and a 4-bit scale.  The thread's 16 weights are ids 8 (2 p + e) + 4 h .. + 3 with sign indices 2 h, 2 h + 1.
// LDS tables: 256 x 4 magnitudes as fp16, then the 128 x 8 sign bits.
struct GIQ3XXS {
    static constexpr int kBlockBytes = 98;
    struct Regs { uint32_t i0, i1, a0, a1, d; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, const float*, int, int p, int h) {
        r.i0 = reinterpret_cast<const UnalignedWord*>(blk + 2 + 16 * p + 4 * h)->v;
        r.i1 = reinterpret_cast<const UnalignedWord*>(blk + 10 + 16 * p + 4 * h)->v;
        r.a0 = reinterpret_cast<const UnalignedWord*>(blk + 66 + 8 * p)->v;
        r.a1 = reinterpret_cast<const UnalignedWord*>(blk + 70 + 8 * p)->v;
        r.d = *reinterpret_cast<const uint16_t*>(blk);
    }
    static constexpr int kTableBytes = 2048 + 2048;
    static __device__ __forceinline__ void stage_table(unsigned char* lds) {
        _Float16* mag = reinterpret_cast<_Float16*>(lds);
        uint16_t* sgn = reinterpret_cast<uint16_t*>(lds + 2048);
        for (int i = threadIdx.x; i < 256 * 4; i += kThreads)
            mag[i] = static_cast<_Float16>(static_cast<float>((PLLM_IQ3XXS_GRID[i >> 2] >> (8 * (i & 3))) & 0xffu));
        for (int i = threadIdx.x; i < 128 * 8; i += kThreads) {
            const uint32_t s7 = static_cast<uint32_t>(i >> 3);
            const uint32_t s8 = s7 | ((__popc(s7) & 1u) << 7);
            sgn[i] = ((s8 >> (i & 7)) & 1u) ? 0x8000u : 0u;
        }
    }
    static __device__ __forceinline__ half4 four(const unsigned char* table, uint32_t id, uint32_t flip_lo, uint32_t flip_hi, float scale) {
        const uint2 m = *reinterpret_cast<const uint2*>(table + 8 * id);
        return half4_of(scaled_pair(m.x, flip_lo, scale), scaled_pair(m.y, flip_hi, scale));
    }
    static __device__ __forceinline__ void decode(const Regs& r, int, int e, int h, const unsigned char* table, Half16& o) {
        const uint32_t ids = e ? r.i1 : r.i0, aux = e ? r.a1 : r.a0;
        const float scale = 0.25f * f16_bits_to_float(r.d) * static_cast<float>(2 * (aux >> 28) + 1);
        const uint4 f0 = *reinterpret_cast<const uint4*>(table + 2048 + 16 * ((aux >> (14 * h)) & 127u));
        const uint4 f1 = *reinterpret_cast<const uint4*>(table + 2048 + 16 * ((aux >> (14 * h + 7)) & 127u));
        o.a = four(table, ids & 0xffu, f0.x, f0.y, scale);
        o.b = four(table, (ids >> 8) & 0xffu, f0.z, f0.w, scale);
        o.c = four(table, (ids >> 16) & 0xffu, f1.x, f1.y, scale);
        o.d = four(table, ids >> 24, f1.z, f1.w, scale);
    }
};

// IQ1_M: 56 B = qs(32) qh(16) scales(8).  One codebook index per 8 weights (qs byte plus the low three
// bits of its qh nibble; bit 3 of the nibble picks delta = -+0.125); sixteen 3-bit scales, one per 16
// weights, in the low 12 bits of four u16 words whose top nibbles spell the fp16 block scale.
// The thread's 16 weights are entries 8 p + 4 e + 2 h and the next one, scale group 4 p + 2 e + h.
// LDS holds the 2048 x 16-bit codebook (two bits per element, value + 1) and a 2 x 16 table of fp16
// pairs: for a delta and the four bits of two neighbouring elements, the pair (c0 - 1 + delta,
// c1 - 1 + delta), all of them exact in fp16; mixed-precision multiplies by the float32 scale finish them.
struct GIQ1M {
    static constexpr int kBlockBytes = 56;
    struct Regs { uint2 qs; uint32_t qh; uint2 sc; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, const float*, int, int p, int) {
        r.qs = *reinterpret_cast<const uint2*>(blk + 8 * p);                  // blocks are 8-byte aligned
        r.qh = *reinterpret_cast<const uint32_t*>(blk + 32 + 4 * p);
        r.sc = *reinterpret_cast<const uint2*>(blk + 48);
    }
    static constexpr int kTableBytes = 4096 + 128;
    static __device__ __forceinline__ void stage_table(unsigned char* lds) {
        uint16_t* t = reinterpret_cast<uint16_t*>(lds);
        for (int i = threadIdx.x; i < 2048; i += kThreads) t[i] = PLLM_IQ1_GRID_PACKED[i];
        half2v* pairs = reinterpret_cast<half2v*>(lds + 4096);
        for (int i = threadIdx.x; i < 32; i += kThreads) {
            const float delta = (i & 16) ? -0.125f : 0.125f;
            pairs[i] = half2v{static_cast<_Float16>(static_cast<float>(i & 3) - 1.0f + delta),
                              static_cast<_Float16>(static_cast<float>((i >> 2) & 3) - 1.0f + delta)};
        }
    }
    static __device__ __forceinline__ void entry(const unsigned char* table, uint32_t qb, uint32_t nib, float scale, half4& lo, half4& hi) {
        const uint32_t packed = reinterpret_cast<const uint16_t*>(table)[qb | ((nib & 7u) << 8)];      // element k in bits [2k, 2k+1], value + 1
        const uint32_t* pairs = reinterpret_cast<const uint32_t*>(table + 4096) + ((nib & 8u) << 1);  // the delta's half of the pair table
        const uint32_t w0 = scaled_pair(pairs[packed & 15u], 0u, scale), w1 = scaled_pair(pairs[(packed >> 4) & 15u], 0u, scale);
        const uint32_t w2 = scaled_pair(pairs[(packed >> 8) & 15u], 0u, scale), w3 = scaled_pair(pairs[(packed >> 12) & 15u], 0u, scale);
        lo = half4_of(w0, w1);
        hi = half4_of(w2, w3);
    }
    static __device__ __forceinline__ void decode(const Regs& r, int p, int e, int h, const unsigned char* table, Half16& o) {
        const uint32_t s01 = r.sc.x, s23 = r.sc.y;
        const uint32_t dbits = ((s01 >> 12) & 0xfu) | ((s01 >> 24) & 0xf0u) | ((s23 >> 4) & 0xf00u) | ((s23 >> 16) & 0xf000u);
        const int grp = 4 * p + 2 * e + h;                                     // 16-weight scale group of the block
        const uint32_t word = ((grp & 8) ? s23 : s01) >> (16 * ((grp >> 2) & 1));
        const float scale = f16_bits_to_float(dbits) * static_cast<float>(2 * ((word >> (3 * (grp & 3))) & 7u) + 1);
        const int en = 4 * e + 2 * h;                                          // entry inside the pair, 0..7
        const uint32_t qw = (en < 4) ? r.qs.x : r.qs.y;
        const uint32_t q0 = (qw >> (8 * (en & 3))) & 0xffu, q1 = (qw >> (8 * (en & 3) + 8)) & 0xffu;
        entry(table, q0, (r.qh >> (4 * en)) & 15u, scale, o.a, o.b);
        entry(table, q1, (r.qh >> (4 * en + 4)) & 15u, scale, o.c, o.d);
    }
};

// FP8 E4M3 (OCP) codes, one byte per weight, rows of k bytes with k a multiple of 256 here; a
// "block" is 256 consecutive codes of a row and carries no header.  The float32 scale of the
// 128 x 128 block is folded into the fp16 weight: fp16(f32(code) * scale).
struct GFP8 {
    static constexpr int kTableBytes = 0;
    static __device__ __forceinline__ void stage_table(unsigned char*) {}
    static constexpr int kBlockBytes = 256;
    struct Regs { uint4 q0, q1; float scale; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, const float* srow, int b, int p, int h) {
        r.q0 = *reinterpret_cast<const uint4*>(blk + 64 * p + 16 * h);
        r.q1 = *reinterpret_cast<const uint4*>(blk + 64 * p + 32 + 16 * h);
        r.scale = srow[2 * b + (p >> 1)];
    }
    static __device__ __forceinline__ half4 word(uint32_t q, float sc) {
        typedef float v2f __attribute__((ext_vector_type(2)));
        const v2f lo = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(q), false);
        const v2f hi = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(q), true);
        half4 o;
        o.x = static_cast<_Float16>(lo.x * sc); o.y = static_cast<_Float16>(lo.y * sc);
        o.z = static_cast<_Float16>(hi.x * sc); o.w = static_cast<_Float16>(hi.y * sc);
        return o;
    }
    static __device__ __forceinline__ void decode(const Regs& r, int, int e, int, const unsigned char*, Half16& o) {
        const uint4 q = e ? r.q1 : r.q0;
        o.a = word(q.x, r.scale); o.b = word(q.y, r.scale); o.c = word(q.z, r.scale); o.d = word(q.w, r.scale);
    }
};

// MI = 32-row MFMA tiles per wave along the tokens; the workgroup tile is (64 MI) x 256.
// Workgroups [0, full_tiles) take whole tiles and store scaled results into y; workgroup
// full_tiles + r takes slice r % slices of tile full_tiles + r / slices and stores raw float32 sums
// into partial[r][kBM][kBN].  Tiles are numbered along N first.
// With `seg` the launch is a batch of matmuls (routed experts): grid.y counts the groups, every group
// has its own weight matrix and a run of activation / output rows, and its tiles along the tokens are
// counted from the start of that run (workgroups past the end of a short run leave at once).
template <typename FMT, int MI>
__global__ __launch_bounds__(kThreads) void gemm_f16_kernel(
    const _Float16* __restrict__ xh, const float* __restrict__ xscale, const uint8_t* __restrict__ w,
    void* __restrict__ y, int y_dtype, float* __restrict__ partial, int t_rows, int n, int bpr,
    int tiles_n, int full_tiles, int slices, const float* __restrict__ wscale, int scale_kb,
    const int32_t* __restrict__ seg, size_t group_stride) {
    constexpr int kBM = 64 * MI;
    constexpr int kXTile = kBM * kLds, kWTile = kBN * kLds;
    extern __shared__ __align__(16) unsigned char smem[];
    _Float16* xs_buf = reinterpret_cast<_Float16*>(smem);                 // [2][kBM][kLds]
    _Float16* ws_buf = xs_buf + 2 * kXTile;                               // [2][kBN][kLds]
    unsigned char* table = reinterpret_cast<unsigned char*>(ws_buf + 2 * kWTile);   // the format's codebook, if any

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 2, wn = wave & 3;                              // 2 x 4 waves, (32 MI) x 64 each
    const int wg = blockIdx.x;
    const bool whole = wg < full_tiles;
    const int rest = wg - full_tiles;
    const int tile = whole ? wg : full_tiles + rest / slices;
    const int slice = whole ? 0 : rest % slices, nsl = whole ? 1 : slices;
    const int n0 = (tile % tiles_n) * kBN;
    int t0 = (tile / tiles_n) * kBM;
    if (seg) {
        // grouped: group blockIdx.y owns activation rows [seg[g], seg[g + 1]) and the matrix at w + g * group_stride
        const int g = blockIdx.y;
        t0 += seg[g];
        t_rows = seg[g + 1];
        if (t0 >= t_rows) return;
        w += static_cast<size_t>(g) * group_stride;
    }
    const int kp = bpr * 256;
    const int b0 = static_cast<int>(static_cast<long long>(slice) * bpr / nsl);
    const int b1 = static_cast<int>(static_cast<long long>(slice + 1) * bpr / nsl);

    // staging roles.  Weights: thread (row, h) owns 16 of the 32 weights of its row in every chunk.
    // Activations: per chunk the tile has 4 pieces of 16 bytes per row; a thread moves piece
    // tid % 4 of rows tid / 4 and tid / 4 + 128 (MI = 4), of row tid / 4 (MI = 2), and the first
    // four waves of row tid / 4 (MI = 1).  Both chunks of a pair are fetched together, so the two
    // halves of every 128-byte line are requested back to back.
    // (named variables, not arrays: indexed through the lambdas below, arrays end up in scratch memory)
    const int srow = tid >> 1, sh = tid & 1;
    const uint8_t* wrow = w + static_cast<size_t>(min(n0 + srow, n - 1)) * bpr * FMT::kBlockBytes;
    const float* srow_scale = wscale + static_cast<size_t>(min(n0 + srow, n - 1) >> 7) * scale_kb;      // FP8 only
    constexpr int kXRows = MI == 4 ? 2 : 1;                 // pieces per thread and chunk
    const bool xmover = MI > 1 || tid < 256;
    auto xaddr = [&](int i) { return xh + static_cast<size_t>(min(t0 + (tid >> 2) + 128 * i, t_rows - 1)) * kp + 8 * (tid & 3); };
    const _Float16* const xsrc0 = xaddr(0);
    const _Float16* const xsrc1 = xaddr(kXRows > 1 ? 1 : 0);
    const int xdst_off = (tid >> 2) * kLds + 8 * (tid & 3);

    floatx16 acc[MI][2];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    typename FMT::Regs wset0 = {}, wset1 = {};
    uint4 xa0, xa1, xa2, xa3, xb0, xb1, xb2, xb3;            // [chunk of the pair][row piece] per set
    // (blk, p) = super-block along K and chunk pair (64 weights) inside it
    auto fetch = [&](int blk, int p, typename FMT::Regs& wr, uint4& x00, uint4& x01, uint4& x10, uint4& x11) {
        FMT::load(wr, wrow + static_cast<size_t>(blk) * FMT::kBlockBytes, srow_scale, blk, p, sh);
        const size_t off = static_cast<size_t>(blk) * 256 + 64 * p;
        if (xmover) {
            x00 = *reinterpret_cast<const uint4*>(xsrc0 + off);
            x10 = *reinterpret_cast<const uint4*>(xsrc0 + off + 32);
            if constexpr (kXRows > 1) {
                x01 = *reinterpret_cast<const uint4*>(xsrc1 + off);
                x11 = *reinterpret_cast<const uint4*>(xsrc1 + off + 32);
            }
        }
    };
    auto stage = [&](int p, int e, int buf, const typename FMT::Regs& wr, const uint4& x0, const uint4& x1) {
        Half16 d;
        FMT::decode(wr, p, e, sh, table, d);
        half4* wdst = reinterpret_cast<half4*>(ws_buf + buf * kWTile + srow * kLds + 16 * sh);
        wdst[0] = d.a; wdst[1] = d.b; wdst[2] = d.c; wdst[3] = d.d;
        if (xmover) {
            uint4* xdst = reinterpret_cast<uint4*>(xs_buf + buf * kXTile + xdst_off);
            xdst[0] = x0;
            if constexpr (kXRows > 1) xdst[128 * kLds * 2 / 16] = x1;
        }
    };
    auto multiply = [&](int buf) {
        const _Float16* xt = xs_buf + buf * kXTile + (wm * 32 * MI + (lane & 31)) * kLds + 8 * (lane >> 5);
        const _Float16* wt = ws_buf + buf * kWTile + (wn * 64 + (lane & 31)) * kLds + 8 * (lane >> 5);
#pragma unroll
        for (int ks = 0; ks < kBK / 16; ++ks) {
            const half8 b0 = *reinterpret_cast<const half8*>(wt + 16 * ks);
            const half8 b1 = *reinterpret_cast<const half8*>(wt + 32 * kLds + 16 * ks);
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) {
                const half8 a = *reinterpret_cast<const half8*>(xt + mi * 32 * kLds + 16 * ks);
                acc[mi][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b0, acc[mi][0], 0, 0, 0);
                acc[mi][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b1, acc[mi][1], 0, 0, 0);
            }
        }
    };
    // Asks the scheduler to weave one step's decode (vector ALU) and LDS reads between its MFMAs:
    // a wave that issues its MFMAs in one run and decodes afterwards leaves each unit idle in turn.
    auto weave = [&]() {
        constexpr int kMfma = 4 * MI, kValuPer = 112 / kMfma, kReads = 2 * (2 + MI);
        __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);                 // b0, b1, a0 of the first k-step
#pragma unroll
        for (int i = 0; i < kMfma; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);             // one MFMA
            if (i < kReads - 3) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read ahead
            __builtin_amdgcn_sched_group_barrier(0x002, kValuPer, 0);      // a slice of the decode
        }
    };

    // One turn of the loop is one super-block: eight chunks = four pairs, pairs 0 and 2 through
    // register set a, pairs 1 and 3 through set b, so that the pair index is a compile-time constant
    // in every step.  Even chunks use the low nibbles of their pair's codes, odd chunks the high ones.
    // Past the end the loop re-fetches and re-stages the last block instead of branching: nobody reads it.
    fetch(b0, 0, wset0, xa0, xa1, xa2, xa3);
    fetch(b0, 1, wset1, xb0, xb1, xb2, xb3);
    if constexpr (FMT::kTableBytes > 0) {
        FMT::stage_table(table);
        __syncthreads();
    }
    stage(0, 0, 0, wset0, xa0, xa1);
    __syncthreads();
    for (int blk = b0; blk < b1; ++blk) {
        const int nxt = min(blk + 1, b1 - 1);
        multiply(0); stage(0, 1, 1, wset0, xa2, xa3); weave();
        __syncthreads();
        fetch(blk, 2, wset0, xa0, xa1, xa2, xa3);
        multiply(1); stage(1, 0, 0, wset1, xb0, xb1); weave();
        __syncthreads();
        multiply(0); stage(1, 1, 1, wset1, xb2, xb3); weave();
        __syncthreads();
        fetch(blk, 3, wset1, xb0, xb1, xb2, xb3);
        multiply(1); stage(2, 0, 0, wset0, xa0, xa1); weave();
        __syncthreads();
        multiply(0); stage(2, 1, 1, wset0, xa2, xa3); weave();
        __syncthreads();
        fetch(nxt, 0, wset0, xa0, xa1, xa2, xa3);
        multiply(1); stage(3, 0, 0, wset1, xb0, xb1); weave();
        __syncthreads();
        multiply(0); stage(3, 1, 1, wset1, xb2, xb3); weave();
        __syncthreads();
        fetch(nxt, 1, wset1, xb0, xb1, xb2, xb3);
        multiply(1); stage(0, 0, 0, wset0, xa0, xa1); weave();
        __syncthreads();
    }

    // D[m][n]: lane holds column n = lane % 32 and rows 8 * (v / 4) + 4 * (lane / 32) + v % 4
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
            const int lcol = wn * 64 + ni * 32 + (lane & 31), col = n0 + lcol;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int lrow = wm * 32 * MI + mi * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3), row = t0 + lrow;
                if (!whole) partial[(static_cast<size_t>(rest) * kBM + lrow) * kBN + lcol] = acc[mi][ni][v];
                else if (row < t_rows && col < n) store_any(y, y_dtype, static_cast<size_t>(row) * n + col, acc[mi][ni][v] * xscale[row]);
            }
        }
}

// Split tile number blockIdx.y (tile full_tiles + blockIdx.y of the grid above), 1024 of its
// elements per workgroup: y[t, n] = xscale[t] * sum over its slices, in slice order, of their
// partial tiles.
__global__ __launch_bounds__(256) void gemm_reduce_kernel(const float* __restrict__ partial, const float* __restrict__ xscale,
                                                          void* __restrict__ y, int y_dtype, int t_rows, int n,
                                                          int bm, int tiles_n, int full_tiles, int slices) {
    const int tile = full_tiles + blockIdx.y;
    const int n0 = (tile % tiles_n) * kBN, t0 = (tile / tiles_n) * bm;
    const size_t tile_elems = static_cast<size_t>(bm) * kBN;
    const int i = (blockIdx.x * 256 + threadIdx.x) * 4;
    const int row = t0 + i / kBN, col = n0 + i % kBN;
    if (row >= t_rows || col >= n) return;
    const float* src = partial + static_cast<size_t>(blockIdx.y) * slices * tile_elems + i;
    float4 s = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    for (int k = 0; k < slices; ++k) {
        const float4 v = *reinterpret_cast<const float4*>(src + k * tile_elems);
        s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    const float sc = xscale[row];
    const size_t o = static_cast<size_t>(row) * n + col;
    store_any(y, y_dtype, o, s.x * sc);
    if (col + 1 < n) store_any(y, y_dtype, o + 1, s.y * sc);
    if (col + 2 < n) store_any(y, y_dtype, o + 2, s.z * sc);
    if (col + 3 < n) store_any(y, y_dtype, o + 3, s.w * sc);
}

struct GemmPlan { int mi; int tiles_n; int tiles; int full_tiles; int slices; };

// Tile height by token count.  The tiles beyond the last whole round of the machine are cut in the
// number of K slices that minimises rounds per slice plus the cost of moving the partial tiles.
GemmPlan plan_gemm(int t_rows, int n, int bpr) {
    GemmPlan p;
    const int cus = compute_units();
    p.tiles_n = (n + kBN - 1) / kBN;
    p.mi = t_rows <= 64 ? 1 : (t_rows <= 128 ? 2 : 4);
    if (t_rows > 128) {
        // 128-row tiles instead of 256-row ones where those would leave the machine mostly empty (a quarter of the compute units or
        // less: half the partial-tile traffic per slice, twice the workgroups before slicing), and where the last 256-row tile
        // would be half padding while the 128-row tiles still fit one round.  Q4_K, us, 256- / 128-row tiles: 5120x5120 T=129
        // 49.8 / 42.9, T=256 52.1 / 44.1, T=384 60.9 / 50.8, T=512 64.3 / 63.7, T=1024 92.7 / 114.0; 17408x5120 T=256 83.1 / 107.4,
        // T=384 152.3 / 138.5, T=512 159.8 / 167.7
        const int tiles128 = (t_rows + 127) / 128, tiles256 = (t_rows + 255) / 256;
        if (tiles256 * p.tiles_n * 4 <= cus || ((tiles128 & 1) && tiles128 * p.tiles_n <= cus)) p.mi = 2;
    }
    const int bm = 64 * p.mi;
    p.tiles = ((t_rows + bm - 1) / bm) * p.tiles_n;
    p.full_tiles = (p.tiles / cus) * cus;
    const int rem = p.tiles - p.full_tiles;
    p.slices = 1;
    if (rem > 0) {
        // time of one unsplit tile in microseconds (about 1.1 per 32-weight step) against the
        // write-plus-read of rem * s partial tiles at about 5 TB/s
        const double tile_us = 8.8 * bpr;
        double best = 1e30;
        for (int s = 1; s <= 16 && s <= bpr; ++s) {
            const double rounds = static_cast<double>((static_cast<long long>(rem) * s + cus - 1) / cus) / s;
            const double move_us = s > 1 ? 2.0 * rem * s * bm * kBN * 4.0 / 5.0e6 : 0.0;
            const double cost = rounds * tile_us + move_us;
            if (cost < best - 1e-9) { best = cost; p.slices = s; }
        }
    }
    return p;
}

template <typename FMT, int MI>
int launch_gemm(const GemmPlan& p, const _Float16* xh, const float* xscale, const uint8_t* w, void* y, int y_dtype, float* partial,
                int t_rows, int n, int bpr, const float* wscale, int scale_kb, const int32_t* seg, size_t group_stride, int groups,
                hipStream_t stream) {
    const size_t smem = static_cast<size_t>(2) * (64 * MI + kBN) * kLds * sizeof(_Float16) + FMT::kTableBytes;
    auto kern = gemm_f16_kernel<FMT, MI>;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem)) != hipSuccess)
        return PLLM_ERR_UNSUPPORTED;
    const int rem = p.tiles - p.full_tiles;
    const int full = p.slices > 1 ? p.full_tiles : p.tiles;             // unsplit left-over tiles are whole tiles too
    const int grid = full + (p.slices > 1 ? rem * p.slices : 0);
    hipLaunchKernelGGL(kern, dim3(grid, seg ? groups : 1), dim3(kThreads), smem, stream, xh, xscale, w, y, y_dtype, partial, t_rows, n, bpr,
                       p.tiles_n, full, p.slices, wscale, scale_kb, seg, group_stride);
    if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
    if (p.slices > 1) {
        hipLaunchKernelGGL(gemm_reduce_kernel, dim3(64 * MI * kBN / 1024, rem), dim3(256), 0, stream, partial, xscale, y, y_dtype, t_rows, n,
                           64 * MI, p.tiles_n, full, p.slices);
        if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
    }
    return PLLM_OK;
}

template <typename FMT>
int launch_gemm_mi(const GemmPlan& p, const _Float16* xh, const float* xscale, const uint8_t* w, void* y, int y_dtype, float* partial,
                   int t_rows, int n, int bpr, const float* wscale, int scale_kb, const int32_t* seg, size_t group_stride, int groups,
                   hipStream_t stream) {
    switch (p.mi) {
        case 1: return launch_gemm<FMT, 1>(p, xh, xscale, w, y, y_dtype, partial, t_rows, n, bpr, wscale, scale_kb, seg, group_stride, groups, stream);
        case 2: return launch_gemm<FMT, 2>(p, xh, xscale, w, y, y_dtype, partial, t_rows, n, bpr, wscale, scale_kb, seg, group_stride, groups, stream);
        default: return launch_gemm<FMT, 4>(p, xh, xscale, w, y, y_dtype, partial, t_rows, n, bpr, wscale, scale_kb, seg, group_stride, groups, stream);
    }
}


}  // namespace

bool gemm_f16_supports(int type_id) {
    return type_id == PLLM_TYPE_Q4_K || type_id == PLLM_TYPE_Q5_K || type_id == PLLM_TYPE_Q2_K || type_id == PLLM_TYPE_IQ2_XXS ||
           type_id == PLLM_TYPE_IQ1_M || type_id == PLLM_TYPE_Q6_K || type_id == PLLM_TYPE_IQ4_XS || type_id == PLLM_TYPE_IQ2_XS ||
           type_id == PLLM_TYPE_IQ3_XXS;
}

size_t gemm_f16_workspace_bytes(int rows, int n, int bpr) {
    const GemmPlan p = plan_gemm(rows, n, bpr);
    const size_t part = p.slices > 1 ? align256(static_cast<size_t>(p.tiles - p.full_tiles) * p.slices * 64 * p.mi * kBN * sizeof(float)) : 0;
    return align256(static_cast<size_t>(rows) * bpr * 256 * sizeof(_Float16)) + align256(static_cast<size_t>(rows) * sizeof(float)) + part;
}

namespace {
// activations -> fp16 rows + per-row scales at the head of the workspace; returns the partial-tile area
float* stage_activations(const void* x, int x_dtype, int rows, int k, int bpr, void* workspace, const _Float16*& xh_out, const float*& xscale_out,
                         hipStream_t stream, const int64_t* row_map = nullptr) {
    unsigned char* base = static_cast<unsigned char*>(workspace);
    _Float16* xh = reinterpret_cast<_Float16*>(base);
    base += align256(static_cast<size_t>(rows) * bpr * 256 * sizeof(_Float16));
    float* xscale = reinterpret_cast<float*>(base);
    base += align256(static_cast<size_t>(rows) * sizeof(float));
    const bool narrow = (x_dtype == PLLM_BF16 || x_dtype == PLLM_F16) && k % 8 == 0 && bpr * 256 <= 8192 &&
                        reinterpret_cast<uintptr_t>(x) % 16 == 0;
    const bool few = rows <= 512;                  // one row per workgroup while that leaves the grid small
    const uint16_t* x16 = static_cast<const uint16_t*>(x);
    if (narrow && x_dtype == PLLM_BF16 && few)
        hipLaunchKernelGGL((act_f16_rows_kernel<true, 4>), dim3(rows), dim3(256), 0, stream, x16, xh, xscale, rows, k, bpr * 256, row_map);
    else if (narrow && x_dtype == PLLM_BF16)
        hipLaunchKernelGGL((act_f16_rows_kernel<true, 1>), dim3((rows + 3) / 4), dim3(256), 0, stream, x16, xh, xscale, rows, k, bpr * 256, row_map);
    else if (narrow && few)
        hipLaunchKernelGGL((act_f16_rows_kernel<false, 4>), dim3(rows), dim3(256), 0, stream, x16, xh, xscale, rows, k, bpr * 256, row_map);
    else if (narrow)
        hipLaunchKernelGGL((act_f16_rows_kernel<false, 1>), dim3((rows + 3) / 4), dim3(256), 0, stream, x16, xh, xscale, rows, k, bpr * 256, row_map);
    else
        hipLaunchKernelGGL(act_f16_kernel, dim3(rows), dim3(256), 0, stream, x, x_dtype, xh, xscale, k, bpr * 256, row_map);
    xh_out = xh;
    xscale_out = xscale;
    return reinterpret_cast<float*>(base);
}
}  // namespace

int gemm_f16(const void* x, int x_dtype, const uint8_t* w, int type_id, void* y, int y_dtype,
             int rows, int k, int n, int bpr, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    if (!workspace || workspace_bytes < gemm_f16_workspace_bytes(rows, n, bpr)) return PLLM_ERR_WORKSPACE;
    const GemmPlan p = plan_gemm(rows, n, bpr);
    const _Float16* xh;
    const float* xscale;
    float* partial = stage_activations(x, x_dtype, rows, k, bpr, workspace, xh, xscale, stream);
    if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
    switch (type_id) {
        case PLLM_TYPE_Q4_K: return launch_gemm_mi<GQ4K>(p, xh, xscale, w, y, y_dtype, partial, rows, n, bpr, nullptr, 0, nullptr, 0, 1, stream);
        case PLLM_TYPE_Q5_K: return launch_gemm_mi<GQ5K>(p, xh, xscale, w, y, y_dtype, partial, rows, n, bpr, nullptr, 0, nullptr, 0, 1, stream);
        case PLLM_TYPE_Q2_K: return launch_gemm_mi<GQ2K>(p, xh, xscale, w, y, y_dtype, partial, rows, n, bpr, nullptr, 0, nullptr, 0, 1, stream);
        case PLLM_TYPE_IQ2_XXS: return launch_gemm_mi<GIQ2XXS>(p, xh, xscale, w, y, y_dtype, partial, rows, n, bpr, nullptr, 0, nullptr, 0, 1, stream);
        case PLLM_TYPE_IQ1_M: return launch_gemm_mi<GIQ1M>(p, xh, xscale, w, y, y_dtype, partial, rows, n, bpr, nullptr, 0, nullptr, 0, 1, stream);
        case PLLM_TYPE_Q6_K: return launch_gemm_mi<GQ6K>(p, xh, xscale, w, y, y_dtype, partial, rows, n, bpr, nullptr, 0, nullptr, 0, 1, stream);
        case PLLM_TYPE_IQ4_XS: return launch_gemm_mi<GIQ4XS>(p, xh, xscale, w, y, y_dtype, partial, rows, n, bpr, nullptr, 0, nullptr, 0, 1, stream);
        case PLLM_TYPE_IQ2_XS: return launch_gemm_mi<GIQ2XS>(p, xh, xscale, w, y, y_dtype, partial, rows, n, bpr, nullptr, 0, nullptr, 0, 1, stream);
        case PLLM_TYPE_IQ3_XXS: return launch_gemm_mi<GIQ3XXS>(p, xh, xscale, w, y, y_dtype, partial, rows, n, bpr, nullptr, 0, nullptr, 0, 1, stream);
        default: return PLLM_ERR_UNSUPPORTED;
    }
}

// FP8 weights [n, k] (k a multiple of 256), scales [ceil(n/128), k/128]
int gemm_f16_fp8(const void* x, int x_dtype, const uint8_t* w, const float* wscale, void* y, int y_dtype,
                 int rows, int k, int n, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    if (k % 256 != 0) return PLLM_ERR_UNSUPPORTED;
    const int bpr = k / 256;
    if (!workspace || workspace_bytes < gemm_f16_workspace_bytes(rows, n, bpr)) return PLLM_ERR_WORKSPACE;
    const GemmPlan p = plan_gemm(rows, n, bpr);
    const _Float16* xh;
    const float* xscale;
    float* partial = stage_activations(x, x_dtype, rows, k, bpr, workspace, xh, xscale, stream);
    if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
    return launch_gemm_mi<GFP8>(p, xh, xscale, w, y, y_dtype, partial, rows, n, bpr, wscale, k / 128, nullptr, 0, 1, stream);
}

// ---- routed experts as a batch of tile matmuls ---------------------------------------------------------
size_t gemm_f16_staged_bytes(int rows, int bpr) {
    return align256(static_cast<size_t>(rows) * bpr * 256 * sizeof(_Float16)) + align256(static_cast<size_t>(rows) * sizeof(float));
}

// x rows gathered through row_map (route -> token) into fp16 rows + scales at `staged` (gemm_f16_staged_bytes bytes)
int gemm_f16_stage_rows(const void* x, int x_dtype, const int64_t* row_map, int rows, int k, int bpr, void* staged, hipStream_t stream) {
    const _Float16* xh;
    const float* xscale;
    (void)stage_activations(x, x_dtype, rows, k, bpr, staged, xh, xscale, stream, row_map);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

int gemm_f16_stage_swiglu(const float* g, const float* u, const float* route_weights, float limit, int rows, int inter, int bpr, void* staged,
                          hipStream_t stream) {
    _Float16* hh = static_cast<_Float16*>(staged);
    float* hscale = reinterpret_cast<float*>(static_cast<unsigned char*>(staged) + align256(static_cast<size_t>(rows) * bpr * 256 * sizeof(_Float16)));
    hipLaunchKernelGGL(swiglu_f16_rows_kernel, dim3((rows + 3) / 4), dim3(256), 0, stream, g, u, route_weights, limit, hh, hscale, rows, inter, bpr * 256);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

// y[r, :] (float32 [rows, n]) = staged row r . dequant(W_g)^T for r in [seg[g], seg[g + 1]); no group has more than max_group_rows rows
int gemm_f16_grouped(const void* staged, const uint8_t* w, int type_id, size_t group_stride, const int32_t* seg, int groups,
                     float* y, int rows, int max_group_rows, int n, int bpr, hipStream_t stream) {
    const _Float16* xh = static_cast<const _Float16*>(staged);
    const float* xscale = reinterpret_cast<const float*>(static_cast<const unsigned char*>(staged) + align256(static_cast<size_t>(rows) * bpr * 256 * sizeof(_Float16)));
    const int avg = (rows + groups - 1) / groups;
    GemmPlan p;
    p.mi = avg <= 48 ? 1 : (avg <= 128 ? 2 : 4);
    p.tiles_n = (n + kBN - 1) / kBN;
    p.tiles = p.tiles_n * ((max_group_rows + 64 * p.mi - 1) / (64 * p.mi));
    p.full_tiles = p.tiles;
    p.slices = 1;
    switch (type_id) {
        case PLLM_TYPE_Q4_K: return launch_gemm_mi<GQ4K>(p, xh, xscale, w, y, PLLM_F32, nullptr, rows, n, bpr, nullptr, 0, seg, group_stride, groups, stream);
        case PLLM_TYPE_Q5_K: return launch_gemm_mi<GQ5K>(p, xh, xscale, w, y, PLLM_F32, nullptr, rows, n, bpr, nullptr, 0, seg, group_stride, groups, stream);
        case PLLM_TYPE_Q2_K: return launch_gemm_mi<GQ2K>(p, xh, xscale, w, y, PLLM_F32, nullptr, rows, n, bpr, nullptr, 0, seg, group_stride, groups, stream);
        case PLLM_TYPE_IQ2_XXS: return launch_gemm_mi<GIQ2XXS>(p, xh, xscale, w, y, PLLM_F32, nullptr, rows, n, bpr, nullptr, 0, seg, group_stride, groups, stream);
        case PLLM_TYPE_IQ1_M: return launch_gemm_mi<GIQ1M>(p, xh, xscale, w, y, PLLM_F32, nullptr, rows, n, bpr, nullptr, 0, seg, group_stride, groups, stream);
        case PLLM_TYPE_Q6_K: return launch_gemm_mi<GQ6K>(p, xh, xscale, w, y, PLLM_F32, nullptr, rows, n, bpr, nullptr, 0, seg, group_stride, groups, stream);
        case PLLM_TYPE_IQ4_XS: return launch_gemm_mi<GIQ4XS>(p, xh, xscale, w, y, PLLM_F32, nullptr, rows, n, bpr, nullptr, 0, seg, group_stride, groups, stream);
        case PLLM_TYPE_IQ2_XS: return launch_gemm_mi<GIQ2XS>(p, xh, xscale, w, y, PLLM_F32, nullptr, rows, n, bpr, nullptr, 0, seg, group_stride, groups, stream);
        case PLLM_TYPE_IQ3_XXS: return launch_gemm_mi<GIQ3XXS>(p, xh, xscale, w, y, PLLM_F32, nullptr, rows, n, bpr, nullptr, 0, seg, group_stride, groups, stream);
        default: return PLLM_ERR_UNSUPPORTED;
    }
}

}  // namespace pllm
