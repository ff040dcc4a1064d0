// Per-format pieces of the v_dot4_i32_i8 kernels: Q2_K, IQ2_XXS and IQ1_M super-blocks.
//
// Common lane map: four adjacent lanes share one 256-weight super-block, lane j owning 64 of its
// weights; each format below says which.  A format provides
//   Regs / load(regs, block pointer, j)      the lane's share of the block, in registers
//   kTableBytes / stage_tables(lds)          codebooks the workgroup keeps in LDS
//   lane_dot(regs, j, block index, sx, lds)  the lane's partial dot against the staged activations
// Activations come from the image described in pllm_device.h (two int8 terms per value).
#pragma once

#include "pllm_device.h"

namespace pllm {

#define PLLM_TABLE_U64(name, n) alignas(16) static __device__ constexpr uint64_t name[n] = {
#define PLLM_TABLE_U32(name, n) alignas(16) static __device__ constexpr uint32_t name[n] = {
#define PLLM_TABLE_U16(name, n) alignas(16) static __device__ constexpr uint16_t name[n] = {
#define PLLM_TABLE_END };
#include "ggml_codebooks.inc"
#undef PLLM_TABLE_U64
#undef PLLM_TABLE_U32
#undef PLLM_TABLE_U16
#undef PLLM_TABLE_END

// Derived tables in the form the kernels keep in LDS, built at compile time so that staging them is
// a plain copy.
//   PLLM_IQ2XXS_SIGN_MASKS[s7]: 0xff in byte b where bit b of the 8-bit sign pattern is set (bit 7
//     of a pattern is the parity of the other seven).
//   PLLM_IQ1_GRID_NIBBLES[i]: the eight codes c = grid value + 1 in {0, 1, 2} of codebook entry i,
//     nibble 2b = element b and nibble 2b + 1 = element 4 + b, so that two masks give the two dwords
//     of int8 codes.
struct alignas(16) Iq2xxsSignMasks { uint64_t v[128]; };
struct alignas(16) Iq1GridNibbles { uint32_t v[2048]; };
constexpr Iq2xxsSignMasks make_iq2xxs_sign_masks() {
    Iq2xxsSignMasks t{};
    for (uint32_t i = 0; i < 128; ++i) {
        uint32_t parity = 0;
        for (int b = 0; b < 7; ++b) parity ^= (i >> b) & 1u;
        const uint32_t s8 = i | (parity << 7);
        uint64_t m = 0;
        for (int b = 0; b < 8; ++b) m |= ((s8 >> b) & 1u) ? (0xffull << (8 * b)) : 0ull;
        t.v[i] = m;
    }
    return t;
}
constexpr Iq1GridNibbles make_iq1_grid_nibbles() {
    Iq1GridNibbles t{};
    for (int i = 0; i < 2048; ++i) {
        const uint32_t p = PLLM_IQ1_GRID_PACKED[i];          // element e in bits [2e, 2e+1]
        uint32_t v = 0;
        for (int b = 0; b < 4; ++b) {
            v |= ((p >> (2 * b)) & 3u) << (8 * b);
            v |= ((p >> (2 * (4 + b))) & 3u) << (8 * b + 4);
        }
        t.v[i] = v;
    }
    return t;
}
static __device__ const Iq2xxsSignMasks PLLM_IQ2XXS_SIGN_MASKS = make_iq2xxs_sign_masks();
static __device__ const Iq1GridNibbles PLLM_IQ1_GRID_NIBBLES = make_iq1_grid_nibbles();

// 16 bytes from an address that is only 2-byte aligned.  The vector member keeps it one 16-byte load instruction (global
// memory takes any alignment); four separate words would become four loads.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
struct __attribute__((packed, aligned(2))) Unaligned16 { u32x4 v; };
__device__ __forceinline__ uint4 load16_a2(const uint8_t* p) {
    const Unaligned16 u = *reinterpret_cast<const Unaligned16*>(p);
    return make_uint4(u.v.x, u.v.y, u.v.z, u.v.w);
}

// ------------------------------------------------------------------------------------------------
// Q2_K: 84 B = scales(16) qs(64) d(2) dmin(2).  Lane j holds qs[16j, 16j+16): shift 2s of those
// bytes is group g = 8 * (j >> 1) + 2s + (j & 1), 16 weights each.
// ------------------------------------------------------------------------------------------------
struct Q2K {
    static constexpr int kBlockBytes = 84;
    static constexpr int kTableBytes = 0;
    struct Regs { uint4 sc; uint4 qs; uint32_t dd; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int j) {
        const uint32_t* p = reinterpret_cast<const uint32_t*>(blk);      // blocks are 4-byte aligned
        r.sc = make_uint4(p[0], p[1], p[2], p[3]);
        const uint32_t* q = p + 4 + 4 * j;
        r.qs = make_uint4(q[0], q[1], q[2], q[3]);
        r.dd = p[20];
    }
    static __device__ __forceinline__ void stage_tables(unsigned char*) {}
    static __device__ __forceinline__ float lane_dot(const Regs& r, int j, int blk, const StagedX& sx, const unsigned char*) {
        const int half = j >> 1, odd = j & 1;
        const float d = f16_bits_to_float(r.dd & 0xffffu);
        const float dmin = f16_bits_to_float(r.dd >> 16);
        // scale bytes of groups 8*half + 2s + odd, s = 0..3, live in dwords 2*half and 2*half+1
        const uint32_t slo = half ? r.sc.z : r.sc.x;
        const uint32_t shi = half ? r.sc.w : r.sc.y;
        float pos = 0.0f, neg = 0.0f;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const uint32_t word = s < 2 ? slo : shi;
            const uint32_t sb = (word >> (16 * (s & 1) + 8 * odd)) & 0xffu;
            const int g = 8 * half + 2 * s + odd;
            const int base = blk * 256 + 16 * g;
            const uint4 ah = *reinterpret_cast<const uint4*>(sx.hi + base);
            const uint4 al = *reinterpret_cast<const uint4*>(sx.lo + base);
            const uint32_t w0 = (r.qs.x >> (2 * s)) & 0x03030303u;
            const uint32_t w1 = (r.qs.y >> (2 * s)) & 0x03030303u;
            const uint32_t w2 = (r.qs.z >> (2 * s)) & 0x03030303u;
            const uint32_t w3 = (r.qs.w >> (2 * s)) & 0x03030303u;
            int sh = dot4(w0, ah.x, 0); sh = dot4(w1, ah.y, sh); sh = dot4(w2, ah.z, sh); sh = dot4(w3, ah.w, sh);
            int sl = dot4(w0, al.x, 0); sl = dot4(w1, al.y, sl); sl = dot4(w2, al.z, sl); sl = dot4(w3, al.w, sl);
            const float xs = sx.gs[blk * 8 + (g >> 1)].x;
            pos += static_cast<float>(sb & 15u) * xs * static_cast<float>(__mul24(sh, 254) + sl);
            neg += static_cast<float>(sb >> 4) * sx.sum16[blk * 16 + g];
        }
        return d * pos - dmin * neg;
    }
};

// ------------------------------------------------------------------------------------------------
// IQ2_XXS: 66 B = d(2) + 8 sub-blocks of 8 B (four grid ids, then a u32: four 7-bit sign indices
// and a 4-bit scale).  Lane j holds sub-blocks 2j and 2j+1 (weights 64j .. 64j+63).
// LDS tables: 256 x 8 magnitude bytes, then 128 x 8 sign masks (0xff where the weight is negative;
// bit 7 of a sign pattern is the parity of the other seven).
// ------------------------------------------------------------------------------------------------
struct IQ2XXS {
    static constexpr int kBlockBytes = 66;
    static constexpr int kTableBytes = 2048 + 1024;
    struct Regs { uint4 q; uint32_t d; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int j) {
        r.q = load16_a2(blk + 2 + 16 * j);
        r.d = *reinterpret_cast<const uint16_t*>(blk);
    }
    static __device__ __forceinline__ void stage_tables(unsigned char* lds) {
        copy_to_lds(lds, reinterpret_cast<const unsigned char*>(PLLM_IQ2XXS_GRID), 2048);
        copy_to_lds(lds + 2048, reinterpret_cast<const unsigned char*>(PLLM_IQ2XXS_SIGN_MASKS.v), 1024);
    }
    static __device__ __forceinline__ float sub_block(uint32_t ids, uint32_t aux, int base, const StagedX& sx, const uint2* grid,
                                                       const uint2* sign) {
        int sh = 0, sl = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint2 g = grid[(ids >> (8 * k)) & 0xffu];
            const uint2 m = sign[(aux >> (7 * k)) & 127u];
            // negate the masked bytes: (g ^ 0xff) + 1 never carries out of a byte because g >= 8
            const uint32_t w0 = (g.x ^ m.x) + (m.x & 0x01010101u);
            const uint32_t w1 = (g.y ^ m.y) + (m.y & 0x01010101u);
            const uint2 ah = *reinterpret_cast<const uint2*>(sx.hi + base + 8 * k);
            const uint2 al = *reinterpret_cast<const uint2*>(sx.lo + base + 8 * k);
            sh = dot4(w0, ah.x, sh); sh = dot4(w1, ah.y, sh);
            sl = dot4(w0, al.x, sl); sl = dot4(w1, al.y, sl);
        }
        const float ls = static_cast<float>(2 * (aux >> 28) + 1);
        return ls * sx.gs[base >> 5].x * static_cast<float>(__mul24(sh, 254) + sl);
    }
    static __device__ __forceinline__ float lane_dot(const Regs& r, int j, int blk, const StagedX& sx, const unsigned char* lds) {
        const uint2* grid = reinterpret_cast<const uint2*>(lds);
        const uint2* sign = grid + 256;
        const int base = blk * 256 + 64 * j;
        const float v = sub_block(r.q.x, r.q.y, base, sx, grid, sign) + sub_block(r.q.z, r.q.w, base + 32, sx, grid, sign);
        return 0.125f * f16_bits_to_float(r.d) * v;
    }
};

// ------------------------------------------------------------------------------------------------
// IQ1_M: 56 B = qs(32) qh(16) scales(8).  One codebook index per 8 weights: qs byte plus the low
// three bits of its qh nibble; bit 3 of the nibble picks the shift delta = -+0.125.  Sixteen 3-bit
// scales (one per 16 weights) fill the low 12 bits of four u16 words whose top nibbles spell the
// fp16 super-block scale.  Lane j holds entries 8j .. 8j+7 (weights 64j .. 64j+63).
// LDS table: 2048 x u32 of eight nibbles c = grid value + 1 in {0,1,2}, nibble 2b = element b and
// nibble 2b+1 = element 4+b, so that two masks give the two dwords of int8 codes.
//   w = dl * (c - 1 + delta)   =>   sum w x = dl * (dot(c, x) + (delta - 1) * sum x).
// ------------------------------------------------------------------------------------------------
struct IQ1M {
    static constexpr int kBlockBytes = 56;
    static constexpr int kTableBytes = 8192;
    struct Regs { uint2 qs; uint32_t qh; uint2 sc; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int j) {
        r.qs = *reinterpret_cast<const uint2*>(blk + 8 * j);          // blocks are 8-byte aligned
        r.qh = *reinterpret_cast<const uint32_t*>(blk + 32 + 4 * j);
        r.sc = *reinterpret_cast<const uint2*>(blk + 48);
    }
    static __device__ __forceinline__ void stage_tables(unsigned char* lds) {
        copy_to_lds(lds, reinterpret_cast<const unsigned char*>(PLLM_IQ1_GRID_NIBBLES.v), 8192);
    }
    static __device__ __forceinline__ float lane_dot(const Regs& r, int j, int blk, const StagedX& sx, const unsigned char* lds) {
        const uint32_t* table = reinterpret_cast<const uint32_t*>(lds);
        const uint32_t s01 = r.sc.x, s23 = r.sc.y;
        const uint32_t dbits = ((s01 >> 12) & 0xfu) | ((s01 >> 24) & 0xf0u) | ((s23 >> 4) & 0xf00u) | ((s23 >> 16) & 0xf000u);
        // the lane's four 3-bit scales are the low 12 bits of scale word j
        const uint32_t word = ((j & 2) ? s23 : s01) >> (16 * (j & 1));
        float acc = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t qb = ((e < 4 ? r.qs.x : r.qs.y) >> (8 * (e & 3))) & 0xffu;
            const uint32_t h = (r.qh >> (4 * e)) & 15u;
            const uint32_t packed = table[qb | ((h & 7u) << 8)];
            const uint32_t w0 = packed & 0x0f0f0f0fu;
            const uint32_t w1 = (packed >> 4) & 0x0f0f0f0fu;
            const int base = blk * 256 + 64 * j + 8 * e;
            const uint2 ah = *reinterpret_cast<const uint2*>(sx.hi + base);
            const uint2 al = *reinterpret_cast<const uint2*>(sx.lo + base);
            const int dh = dot4(w1, ah.y, dot4(w0, ah.x, 0));
            const int dl = dot4(w1, al.y, dot4(w0, al.x, 0));
            const int th = dot4(0x01010101u, ah.y, dot4(0x01010101u, ah.x, 0));
            const int tl = dot4(0x01010101u, al.y, dot4(0x01010101u, al.x, 0));
            const float shift = (h & 8u) ? -1.125f : -0.875f;
            const float v = static_cast<float>(__mul24(dh, 254) + dl) + shift * static_cast<float>(__mul24(th, 254) + tl);
            const float ls = static_cast<float>(2 * ((word >> (3 * (e >> 1))) & 7u) + 1);
            acc += ls * sx.gs[base >> 5].x * v;
        }
        return f16_bits_to_float(dbits) * acc;
    }
};

}  // namespace pllm
