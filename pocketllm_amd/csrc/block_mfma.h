// Per-format pieces of the matrix-core kernels over IQ2_XXS, IQ2_XS, IQ3_XXS, IQ1_M, IQ4_XS and Q6_K super-blocks, and the
// direct-to-LDS copy helpers they share.
//
// Lane map: lane (n, s) = (lane % 16, lane / 16) of a wave works on output row n of a 16-row tile and
// owns the 64 weights [64 s, 64 s + 64) of a super-block.  For one super-block index the wave forms
//     C[m][n] = sum_k A[m][k] * B[k][n],     v_mfma_i32_16x16x64_i8,
// with B = the weights' integer codes and A = activation bytes (from the image described in
// pllm_device.h, two int8 terms per value) arranged so that row m collects one scale group of the
// block; the slices are assigned to A rows such that the lane finds the results for exactly its own
// 64 weights in its own C registers, C[4 s .. 4 s + 3][n].  A format provides
//   Regs / load(regs, block pointer, s) / load_lds(regs, LDS base, offset, s)   the lane's share of a block
//   kTableBytes / stage_tables / dma_tables                                      codebooks kept in LDS
//   a_map(am, n, s, kpad, zero offset)           LDS offsets of the lane's A operands
//   block(regs, s, block index, ...)             the lane's partial result for the block
//   Held / hold / block_held                     the same with the activation side kept in registers
#pragma once

#include "block_dot4.h"

namespace pllm {

typedef __attribute__((address_space(3))) unsigned char* lds_byte_ptr;

// 16 bytes per lane from memory to LDS[lds_base + 16 * lane] (lds_base wave-uniform), no registers in
// between.  Issued through inline assembly so that the compiler does not put a wait for it in front
// of every later LDS read: the kernel waits for its chunks itself (wait_vm).
__device__ __forceinline__ void lds_dma16(const void* src, uint32_t lds_base) {
    // (lds_base is wave-uniform by contract; the readfirstlane only tells the compiler so)
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(__builtin_amdgcn_readfirstlane(lds_base)) : "memory", "m0");
}
// the same with the source as a wave-uniform base (scalar registers) plus a 32-bit byte offset per lane: no 64-bit vector
// arithmetic per copy; lds_base must be a scalar value too (computed from readfirstlane'd or launch-wide quantities only)
__device__ __forceinline__ void lds_dma16_at(const void* uniform_base, uint32_t lane_off, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(lane_off), "s"(uniform_base), "s"(lds_base) : "memory", "m0");
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
// 1 KB pieces wave, wave + WAVES, ...; returns the number of instructions issued
template <int WAVES>
__device__ __forceinline__ int dma_share(const unsigned char* src, uint32_t lds_base, int bytes, int wave, int lane) {
    int issued = 0;
    for (int o = wave * 1024; o < bytes; o += WAVES * 1024) {
        if (o + lane * 16 < bytes) lds_dma16(src + o + lane * 16, lds_base + o);
        ++issued;
    }
    return issued;
}

typedef int v4i __attribute__((ext_vector_type(4)));

__device__ __forceinline__ v4i as_v4i(uint32_t x, uint32_t y, uint32_t z, uint32_t w) {
    v4i r;
    r.x = static_cast<int>(x); r.y = static_cast<int>(y); r.z = static_cast<int>(z); r.w = static_cast<int>(w);
    return r;
}

// LDS offsets of a lane's A operands: slot i of block b is read at off[i] + b * step[i]; slots whose
// A row is not the lane's point at 16 zero bytes with step 0 (on[i] false).
template <int SLOTS>
struct AMap { int off[SLOTS]; int step[SLOTS]; bool on[SLOTS]; };

// A operands in registers.  Three quarters or more of a wave's lanes hold zero rows of A: cleared
// once, they are never read again, and only the lanes a slot belongs to touch LDS (a 16-byte read of
// every lane costs the LDS as much as a whole kilobyte of data, zeros included).
template <int SLOTS>
struct AOps { uint4 a[SLOTS]; };
template <int SLOTS>
__device__ __forceinline__ void clear_a(AOps<SLOTS>& ops) {
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) ops.a[i] = make_uint4(0u, 0u, 0u, 0u);
}
template <int SLOTS>
__device__ __forceinline__ void load_a(AOps<SLOTS>& ops, const AMap<SLOTS>& am, const unsigned char* base, int b) {
#pragma unroll
    for (int i = 0; i < SLOTS; ++i)
        if (am.on[i]) ops.a[i] = *reinterpret_cast<const uint4*>(base + am.off[i] + b * 256);
}

// ------------------------------------------------------------------------------------------------
// IQ2_XXS: 66 B = d(2) + 8 sub-blocks of 8 B (four grid ids, then a u32: four 7-bit sign indices and
// a 4-bit scale).  Lane (n, s) holds sub-blocks 2 s and 2 s + 1 (two 32-weight groups).
// A rows: m = 2 * group + term; MFMA t, slice s carries half t % 2 of group 2 s + t / 2, so
// C[4 s .. 4 s + 3][n] = groups 2 s and 2 s + 1, both terms, in the lane's own registers.
// LDS tables: 256 x 8 magnitude bytes g, 128 x 8 sign masks m (0xff where the weight is negative).
// The signed code is (g ^ m) - m bytewise; instead of finishing that per byte, the wave runs two
// MFMAs per slice, with B = g ^ m and with B = m, and subtracts the accumulators.
// ------------------------------------------------------------------------------------------------
// COPIES > 1: every table entry is stored COPIES times side by side (entry e, copy c at 8 * (e * COPIES + c)) and lane l
// reads copy l % COPIES, i.e. `tables` is the lane's own pointer (lane_tables).  With 16 copies the 16 lanes that the LDS
// serves together read from 16 different pairs of banks whatever their indices are: a random 8-byte lookup then costs about 5
// cycles of the LDS per wave instruction instead of about 12 from a single copy (8.4 with 8 copies), measured on the box.
template <int COPIES>
struct IQ2XXSmT {
    static constexpr int kBlockBytes = 66;
    static constexpr int kCopies = COPIES;
    static constexpr int kTableBytes = IQ2XXS::kTableBytes * COPIES;
    static constexpr int kSlots = 4;
    static constexpr bool kStreamed = true;                    // has LDS loaders and table copies for the streamed kernel
    static constexpr int kRowsPerPass = 1;                     // (two rows go through the streamed kernel's own form)
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
    static __device__ __forceinline__ void stage_tables(unsigned char* lds) { static_assert(COPIES == 1, "single copy only"); IQ2XXS::stage_tables(lds); }
    template <int WAVES> static __device__ __forceinline__ void dma_tables(uint32_t lds_base, int wave, int lane);
    // the lane's view of the tables at `tables` (its copy of every entry)
    static __device__ __forceinline__ const unsigned char* lane_tables(const unsigned char* tables, int lane) { return tables + 8 * (lane % COPIES); }
    // the replicated tables, written by the whole workgroup (a barrier must follow): thread e takes entry e from memory
    static __device__ __forceinline__ void stage_replicated(unsigned char* lds, int tid, int threads) {
        for (int e = tid; e < 256 + 128; e += threads) {
            const uint64_t v = e < 256 ? PLLM_IQ2XXS_GRID[e] : PLLM_IQ2XXS_SIGN_MASKS.v[e - 256];
            const uint32_t lo = static_cast<uint32_t>(v), hi = static_cast<uint32_t>(v >> 32);
            uint4* dst = reinterpret_cast<uint4*>(lds + static_cast<size_t>(e) * 8 * COPIES);
#pragma unroll
            for (int c = 0; c < COPIES / 2; ++c) dst[c] = make_uint4(lo, hi, lo, hi);
        }
    }
    static __device__ __forceinline__ void a_map(AMap<kSlots>& am, int col, int ks, int kpad, int zero_off) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int g = 2 * ks + (t >> 1);
            const bool active = (col >> 1) == g;
            am.off[t] = active ? ((col & 1) ? kpad : 0) + 32 * g + 16 * (t & 1) : zero_off;
            am.step[t] = active ? 256 : 0;
            am.on[t] = active;
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
        const uint2* sign = grid + 256 * COPIES;
        v4i c = {0, 0, 0, 0}, cm = {0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t ids = (t < 2) ? r.q.x : r.q.z, aux = (t < 2) ? r.q.y : r.q.w;
            const int e = 2 * (t & 1);                                         // grid entries e and e + 1 of the sub-block
            const uint2 g0 = grid[((ids >> (8 * e)) & 0xffu) * COPIES], m0 = sign[((aux >> (7 * e)) & 127u) * COPIES];
            const uint2 g1 = grid[((ids >> (8 * e + 8)) & 0xffu) * COPIES], m1 = sign[((aux >> (7 * e + 7)) & 127u) * COPIES];
            const v4i av = as_v4i(h.a[t].x, h.a[t].y, h.a[t].z, h.a[t].w);
            c = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, as_v4i(g0.x ^ m0.x, g0.y ^ m0.y, g1.x ^ m1.x, g1.y ^ m1.y), c, 0, 0, 0);
            cm = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, as_v4i(m0.x, m0.y, m1.x, m1.y), cm, 0, 0, 0);
        }
        const float v0 = static_cast<float>(__mul24(c.x - cm.x, 254) + (c.y - cm.y));   // group 2 s: 254 * high term + low term
        const float v1 = static_cast<float>(__mul24(c.z - cm.z, 254) + (c.w - cm.w));   // group 2 s + 1
        const float ls0 = static_cast<float>(2 * (r.q.y >> 28) + 1), ls1 = static_cast<float>(2 * (r.q.w >> 28) + 1);
        return 0.125f * f16_bits_to_float(r.d) * (ls0 * h.xs0 * v0 + ls1 * h.xs1 * v1);
    }
    // A block decoded once for several activation vectors: finished signed codes (B operands of the
    // four MFMAs) and the two groups' scales times d / 8.
    struct Decoded { v4i b[4]; float ls0, ls1; };
    static __device__ __forceinline__ void decode(const Regs& r, int, const unsigned char* tables, Decoded& o) {
        const uint2* grid = reinterpret_cast<const uint2*>(tables);
        const uint2* sign = grid + 256 * COPIES;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t ids = (t < 2) ? r.q.x : r.q.z, aux = (t < 2) ? r.q.y : r.q.w;
            const int e = 2 * (t & 1);
            const uint2 g0 = grid[((ids >> (8 * e)) & 0xffu) * COPIES], m0 = sign[((aux >> (7 * e)) & 127u) * COPIES];
            const uint2 g1 = grid[((ids >> (8 * e + 8)) & 0xffu) * COPIES], m1 = sign[((aux >> (7 * e + 7)) & 127u) * COPIES];
            // negate the masked bytes: (g ^ 0xff) + 1 never carries out of a byte because g >= 8
            o.b[t] = as_v4i((g0.x ^ m0.x) + (m0.x & 0x01010101u), (g0.y ^ m0.y) + (m0.y & 0x01010101u),
                            (g1.x ^ m1.x) + (m1.x & 0x01010101u), (g1.y ^ m1.y) + (m1.y & 0x01010101u));
        }
        const float d8 = 0.125f * f16_bits_to_float(r.d);
        o.ls0 = d8 * static_cast<float>(2 * (r.q.y >> 28) + 1);
        o.ls1 = d8 * static_cast<float>(2 * (r.q.w >> 28) + 1);
    }
    // the decoded block against one activation image (img = its first byte in LDS, offsets of am relative to it)
    static __device__ __forceinline__ float route_block(const Decoded& o, int s, int b, const unsigned char* img, const AMap<kSlots>& am, int kpad,
                                                        AOps<kSlots>& ops) {
        load_a(ops, am, img, b);
        v4i c = {0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 4; ++t)
            c = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(ops.a[t].x, ops.a[t].y, ops.a[t].z, ops.a[t].w), o.b[t], c, 0, 0, 0);
        const float4 g2 = *reinterpret_cast<const float4*>(img + 2 * kpad + (b * 8 + 2 * s) * 8);   // {xs0 / 254, sum0, xs1 / 254, sum1}
        return o.ls0 * g2.x * static_cast<float>(__mul24(c.x, 254) + c.y) + o.ls1 * g2.z * static_cast<float>(__mul24(c.z, 254) + c.w);
    }
    static __device__ __forceinline__ float block(const Regs& r, int s, int b, const unsigned char* smem, const AMap<kSlots>& am,
                                                  const StagedX& sx, const unsigned char* tables) {
        Held h;
        hold(h, s, b, smem, am, sx);
        return block_held(r, s, b, h, smem, am, tables);
    }
};

using IQ2XXSm = IQ2XXSmT<1>;

// ------------------------------------------------------------------------------------------------
// IQ1_M: 56 B = qs(32) qh(16) scales(8); w = dl (c - 1 + delta) with c in {0, 1, 2} from the
// codebook (index: qs byte plus the low three bits of its qh nibble), dl = d (2 s3 + 1) per 16
// weights, delta = -+1/8 per 8 weights (bit 3 of the nibble).  Lane (n, s) holds entries 8 s .. 8 s + 7
// = four 16-weight groups.  With signed integer codes 8 (c - 1) +- 1 = 8 (c - 1 + delta) in {-9, -7, -1, 1, 7, 9},
//     sum w x = d / 8 sum over 16-groups j of (2 s3_j + 1) dot(code, x)_j.
// A rows: m = 16-group of the block, one MFMA set per activation term; MFMA t, slice s carries group
// 4 s + t, so C[4 s .. 4 s + 3][n] = the lane's own four groups.
// LDS table: 4096 x 8 code bytes, index = qs byte | nibble << 8 (the delta bit selects the half).
// ------------------------------------------------------------------------------------------------
struct alignas(16) Iq1DeltaCodes { uint64_t v[4096]; };
constexpr Iq1DeltaCodes make_iq1_delta_codes() {
    Iq1DeltaCodes t{};
    for (int i = 0; i < 4096; ++i) {
        const uint32_t p = PLLM_IQ1_GRID_PACKED[i & 2047];      // element e in bits [2e, 2e+1], value + 1
        uint64_t v = 0;
        for (int e = 0; e < 8; ++e) {
            const int code = 8 * (static_cast<int>((p >> (2 * e)) & 3u) - 1) + ((i & 2048) ? -1 : 1);
            v |= static_cast<uint64_t>(static_cast<uint8_t>(code)) << (8 * e);
        }
        t.v[i] = v;
    }
    return t;
}
static __device__ const Iq1DeltaCodes PLLM_IQ1_DELTA_CODES = make_iq1_delta_codes();

struct IQ1Mm {
    static constexpr int kBlockBytes = 56;
    static constexpr int kCopies = 1;
    static constexpr int kTableBytes = 32768;
    static __device__ __forceinline__ const unsigned char* lane_tables(const unsigned char* tables, int) { return tables; }
    static constexpr int kSlots = 8;                           // [term][t]
    static constexpr bool kStreamed = true;
    static constexpr int kRowsPerPass = 1;
    static constexpr int kHoldBlocks = 3;                      // (109 registers in the streamed kernels: four waves per SIMD; 23.1 -> 21.3 us at 196608x1536)
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
    template <int WAVES> static __device__ __forceinline__ void dma_tables(uint32_t lds_base, int wave, int lane);
    static __device__ __forceinline__ void a_map(AMap<kSlots>& am, int col, int ks, int kpad, int zero_off) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const bool active = col == 4 * ks + t;
            am.off[t] = active ? 16 * col : zero_off;
            am.off[4 + t] = active ? kpad + 16 * col : zero_off;
            am.step[t] = am.step[4 + t] = active ? 256 : 0;
            am.on[t] = am.on[4 + t] = active;
        }
    }
    // activation side of a block index (see IQ2XXSm::Held): the high-term A operands, the groups'
    // scales (already over 8); the low-term operands are read when needed
    struct Held { uint4 a[4]; float x0, x1; };
    static __device__ __forceinline__ void hold(Held& h, int s, int b, const unsigned char* smem, const AMap<kSlots>& am, const StagedX& sx) {
#pragma unroll
        for (int t = 0; t < 4; ++t) h.a[t] = *reinterpret_cast<const uint4*>(smem + am.off[t] + b * am.step[t]);
        const float4 g2 = *reinterpret_cast<const float4*>(sx.gs + b * 8 + 2 * s);   // {xs0 / 254, sum0, xs1 / 254, sum1}
        h.x0 = 0.125f * g2.x; h.x1 = 0.125f * g2.z;
    }
    // lookups and MFMAs of one block: ch / cl = the lane's four 16-weight groups against the high / low term
    static __device__ __forceinline__ void group_dots(const Regs& r, int b, const uint4 (&ah)[4], const unsigned char* smem, const AMap<kSlots>& am,
                                                      const unsigned char* tables, v4i& ch, v4i& cl) {
        const uint2* table = reinterpret_cast<const uint2*>(tables);
        ch = v4i{0, 0, 0, 0}; cl = v4i{0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 4; ++t) {                                          // 16-weight group t of the lane = entries 2 t, 2 t + 1
            const uint32_t qw = (t < 2) ? r.qs.x : r.qs.y;
            const uint2 w0 = table[((qw >> (16 * (t & 1))) & 0xffu) | (((r.qh >> (8 * t)) & 15u) << 8)];
            const uint2 w1 = table[((qw >> (16 * (t & 1) + 8)) & 0xffu) | (((r.qh >> (8 * t + 4)) & 15u) << 8)];
            const v4i bw = as_v4i(w0.x, w0.y, w1.x, w1.y);
            const uint4 al = *reinterpret_cast<const uint4*>(smem + am.off[4 + t] + b * am.step[4 + t]);
            ch = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(ah[t].x, ah[t].y, ah[t].z, ah[t].w), bw, ch, 0, 0, 0);
            cl = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(al.x, al.y, al.z, al.w), bw, cl, 0, 0, 0);
        }
    }
    // scales: x8 = the four groups' activation scales / (254 * 8)
    static __device__ __forceinline__ float finish(const Regs& r, int s, const v4i& ch, const v4i& cl, const float4& x8) {
        const uint32_t s01 = r.sc.x, s23 = r.sc.y;
        const uint32_t dbits = ((s01 >> 12) & 0xfu) | ((s01 >> 24) & 0xf0u) | ((s23 >> 4) & 0xf00u) | ((s23 >> 16) & 0xf000u);
        // the lane's four 16-weight scales are the low 12 bits of scale word s
        const uint32_t word = ((s & 2) ? s23 : s01) >> (16 * (s & 1));
        const float ls0 = static_cast<float>(2 * (word & 7u) + 1), ls1 = static_cast<float>(2 * ((word >> 3) & 7u) + 1);
        const float ls2 = static_cast<float>(2 * ((word >> 6) & 7u) + 1), ls3 = static_cast<float>(2 * ((word >> 9) & 7u) + 1);
        const float v = ls0 * x8.x * static_cast<float>(__mul24(ch.x, 254) + cl.x) + ls1 * x8.y * static_cast<float>(__mul24(ch.y, 254) + cl.y) +
                        ls2 * x8.z * static_cast<float>(__mul24(ch.z, 254) + cl.z) + ls3 * x8.w * static_cast<float>(__mul24(ch.w, 254) + cl.w);
        return f16_bits_to_float(dbits) * v;
    }
    // the same when each pair of groups shares an activation scale (xa for groups 0 and 1, xb for 2 and 3): the group scales go in as
    // integers.  |254 ch + cl| <= 16 * 127 * 9 * 255 < 2^23 and the scales are at most 15, so the 24-bit multiplies are exact.
    static __device__ __forceinline__ float finish_pairs(const Regs& r, int s, const v4i& ch, const v4i& cl, float xa, float xb) {
        const uint32_t s01 = r.sc.x, s23 = r.sc.y;
        const uint32_t dbits = ((s01 >> 12) & 0xfu) | ((s01 >> 24) & 0xf0u) | ((s23 >> 4) & 0xf00u) | ((s23 >> 16) & 0xf000u);
        const uint32_t word = ((s & 2) ? s23 : s01) >> (16 * (s & 1));
        const int l0 = static_cast<int>(2 * (word & 7u) + 1), l1 = static_cast<int>(2 * ((word >> 3) & 7u) + 1);
        const int l2 = static_cast<int>(2 * ((word >> 6) & 7u) + 1), l3 = static_cast<int>(2 * ((word >> 9) & 7u) + 1);
        const int ta = __mul24(l0, __mul24(ch.x, 254) + cl.x) + __mul24(l1, __mul24(ch.y, 254) + cl.y);
        const int tb = __mul24(l2, __mul24(ch.z, 254) + cl.z) + __mul24(l3, __mul24(ch.w, 254) + cl.w);
        return f16_bits_to_float(dbits) * (xa * static_cast<float>(ta) + xb * static_cast<float>(tb));
    }
    static __device__ __forceinline__ float block_held(const Regs& r, int s, int b, const Held& h, const unsigned char* smem,
                                                       const AMap<kSlots>& am, const unsigned char* tables) {
        v4i ch, cl;
        group_dots(r, b, h.a, smem, am, tables, ch, cl);
        return finish_pairs(r, s, ch, cl, h.x0, h.x1);
    }
    // A block decoded once for several activation vectors: the codes of the lane's four 16-weight
    // groups and their scales times d / 8.
    struct Decoded { v4i b[4]; float l0, l1, l2, l3; };
    static __device__ __forceinline__ void decode(const Regs& r, int s, const unsigned char* tables, Decoded& o) {
        const uint2* table = reinterpret_cast<const uint2*>(tables);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t qw = (t < 2) ? r.qs.x : r.qs.y;
            const uint2 w0 = table[((qw >> (16 * (t & 1))) & 0xffu) | (((r.qh >> (8 * t)) & 15u) << 8)];
            const uint2 w1 = table[((qw >> (16 * (t & 1) + 8)) & 0xffu) | (((r.qh >> (8 * t + 4)) & 15u) << 8)];
            o.b[t] = as_v4i(w0.x, w0.y, w1.x, w1.y);
        }
        const uint32_t s01 = r.sc.x, s23 = r.sc.y;
        const uint32_t dbits = ((s01 >> 12) & 0xfu) | ((s01 >> 24) & 0xf0u) | ((s23 >> 4) & 0xf00u) | ((s23 >> 16) & 0xf000u);
        const uint32_t word = ((s & 2) ? s23 : s01) >> (16 * (s & 1));
        const float d8 = 0.125f * f16_bits_to_float(dbits);
        o.l0 = d8 * static_cast<float>(2 * (word & 7u) + 1); o.l1 = d8 * static_cast<float>(2 * ((word >> 3) & 7u) + 1);
        o.l2 = d8 * static_cast<float>(2 * ((word >> 6) & 7u) + 1); o.l3 = d8 * static_cast<float>(2 * ((word >> 9) & 7u) + 1);
    }
    static __device__ __forceinline__ float route_dots(const Decoded& o, int b, const unsigned char* img, const AMap<kSlots>& am, const float4& xs,
                                                       AOps<kSlots>& ops) {
        load_a(ops, am, img, b);
        v4i ch = {0, 0, 0, 0}, cl = {0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            ch = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(ops.a[t].x, ops.a[t].y, ops.a[t].z, ops.a[t].w), o.b[t], ch, 0, 0, 0);
            cl = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(ops.a[4 + t].x, ops.a[4 + t].y, ops.a[4 + t].z, ops.a[4 + t].w), o.b[t], cl, 0, 0, 0);
        }
        return o.l0 * xs.x * static_cast<float>(__mul24(ch.x, 254) + cl.x) + o.l1 * xs.y * static_cast<float>(__mul24(ch.y, 254) + cl.y) +
               o.l2 * xs.z * static_cast<float>(__mul24(ch.z, 254) + cl.z) + o.l3 * xs.w * static_cast<float>(__mul24(ch.w, 254) + cl.w);
    }
    // against an activation image with one scale per 32 values (pllm_device.h) ...
    static __device__ __forceinline__ float route_block(const Decoded& o, int s, int b, const unsigned char* img, const AMap<kSlots>& am, int kpad,
                                                        AOps<kSlots>& ops) {
        const float4 g2 = *reinterpret_cast<const float4*>(img + 2 * kpad + (b * 8 + 2 * s) * 8);   // {xs0 / 254, sum0, xs1 / 254, sum1}
        return route_dots(o, b, img, am, make_float4(g2.x, g2.x, g2.z, g2.z), ops);
    }
    // ... and against one with a scale per 16 values (float xs16[kpad / 16] after the two int8 planes)
    static __device__ __forceinline__ float route_block16(const Decoded& o, int s, int b, const unsigned char* img, const AMap<kSlots>& am, int kpad,
                                                          AOps<kSlots>& ops) {
        return route_dots(o, b, img, am, *reinterpret_cast<const float4*>(img + 2 * kpad + (b * 16 + 4 * s) * 4), ops);
    }
    static __device__ __forceinline__ float block(const Regs& r, int s, int b, const unsigned char* smem, const AMap<kSlots>& am,
                                                  const StagedX& sx, const unsigned char* tables) {
        Held h;
        hold(h, s, b, smem, am, sx);
        return block_held(r, s, b, h, smem, am, tables);
    }
};

// ------------------------------------------------------------------------------------------------
// Q6_K: 210 B = ql(128) qh(64) scales int8(16) d(2); w = d * scale[i / 16] * (q - 32), q = a nibble of ql
// plus two bits of qh.  Lane (n, s), half = s / 2, part = s % 2, holds ql[64 half + 16 part, +16),
// ql[64 half + 32 + 16 part, +16) and qh[32 half + 16 part, +16): the 16-weight groups
// 8 half + 2 t + part, t = 0..3 (low nibbles of the first piece, of the second, then their high
// nibbles, with bit pair t of qh).  A rows: m = 16-group, one MFMA set per activation term; MFMA t,
// slice s carries that group.  The codes stay unsigned (0..63): the "- 32" leaves through the
// image's 16-value sums.  C[4 s .. 4 s + 3][n] are groups 4 s .. 4 s + 3, scale bytes = dword s of scales.
// Blocks are only 2-byte aligned.
// ------------------------------------------------------------------------------------------------
struct __attribute__((packed, aligned(2))) Unaligned4 { uint32_t v; };

struct Q6Km {
    static constexpr int kBlockBytes = 210;
    static constexpr int kTableBytes = 0;
    static constexpr int kSlots = 8;                           // [term][t]
    static constexpr bool kStreamed = false;
    static constexpr int kRowsPerPass = 1;
    struct Regs { uint4 qa, qb, qh; uint32_t sc, d; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int s) {
        const int half = s >> 1, part = s & 1;
        r.qa = load16_a2(blk + 64 * half + 16 * part);
        r.qb = load16_a2(blk + 64 * half + 32 + 16 * part);
        r.qh = load16_a2(blk + 128 + 32 * half + 16 * part);
        r.sc = reinterpret_cast<const Unaligned4*>(blk + 192 + 4 * s)->v;
        r.d = *reinterpret_cast<const uint16_t*>(blk + 208);
    }
    static __device__ __forceinline__ void stage_tables(unsigned char*) {}
    static __device__ __forceinline__ void a_map(AMap<kSlots>& am, int col, int ks, int kpad, int zero_off) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const bool active = col == 8 * (ks >> 1) + 2 * t + (ks & 1);
            am.off[t] = active ? 16 * col : zero_off;
            am.off[4 + t] = active ? kpad + 16 * col : zero_off;
            am.step[t] = am.step[4 + t] = active ? 256 : 0;
            am.on[t] = am.on[4 + t] = active;
        }
    }
    static __device__ __forceinline__ uint32_t code4(uint32_t ql, uint32_t qh, int t) {
        const uint32_t lo = (t < 2 ? ql : ql >> 4) & 0x0f0f0f0fu;
        const uint32_t hi = (t == 0 ? qh << 4 : t == 1 ? qh << 2 : t == 2 ? qh : qh >> 2) & 0x30303030u;
        return lo | hi;
    }
    static __device__ __forceinline__ float block(const Regs& r, int s, int b, const unsigned char* smem, const AMap<kSlots>& am,
                                                  const StagedX& sx, const unsigned char*) {
        v4i ch = {0, 0, 0, 0}, cl = {0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint4 ql = (t & 1) ? r.qb : r.qa;
            const v4i bw = as_v4i(code4(ql.x, r.qh.x, t), code4(ql.y, r.qh.y, t), code4(ql.z, r.qh.z, t), code4(ql.w, r.qh.w, t));
            const uint4 ah = *reinterpret_cast<const uint4*>(smem + am.off[t] + b * am.step[t]);
            const uint4 al = *reinterpret_cast<const uint4*>(smem + am.off[4 + t] + b * am.step[4 + t]);
            ch = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(ah.x, ah.y, ah.z, ah.w), bw, ch, 0, 0, 0);
            cl = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(al.x, al.y, al.z, al.w), bw, cl, 0, 0, 0);
        }
        const float4 g2 = *reinterpret_cast<const float4*>(sx.gs + b * 8 + 2 * s);   // {xs0 / 254, sum0, xs1 / 254, sum1}
        const float4 s16 = *reinterpret_cast<const float4*>(sx.sum16 + b * 16 + 4 * s);
        const int sc = static_cast<int>(r.sc);
        const float v = static_cast<float>(static_cast<int8_t>(sc)) * (g2.x * static_cast<float>(__mul24(ch.x, 254) + cl.x) - 32.0f * s16.x) +
                        static_cast<float>(static_cast<int8_t>(sc >> 8)) * (g2.x * static_cast<float>(__mul24(ch.y, 254) + cl.y) - 32.0f * s16.y) +
                        static_cast<float>(static_cast<int8_t>(sc >> 16)) * (g2.z * static_cast<float>(__mul24(ch.z, 254) + cl.z) - 32.0f * s16.z) +
                        static_cast<float>(sc >> 24) * (g2.z * static_cast<float>(__mul24(ch.w, 254) + cl.w) - 32.0f * s16.w);
        return f16_bits_to_float(r.d) * v;
    }
};

// ------------------------------------------------------------------------------------------------
// IQ4_XS: 136 B = d(2) scales_h(2) scales_l(4) qs(128); w = d * (ls - 32) * kvalues[code], ls six bits per
// 32 weights (low four in a nibble of scales_l, high two in scales_h), 16 bytes per group with
// weights 0..15 in the low and 16..31 in the high nibbles.  Lane (n, s) holds qs[32 s, 32 s + 32) =
// groups 2 s and 2 s + 1.  A rows as for IQ2_XXS: m = 2 * group + term; MFMA t, slice s carries half
// t % 2 of group 2 s + t / 2.  The 16-entry code table sits in four registers; a byte permute picks
// from its lower and upper half and a third one chooses between them by bit 3 of the code.
// ------------------------------------------------------------------------------------------------
struct IQ4XSm {
    static constexpr int kBlockBytes = 136;
    static constexpr int kTableBytes = 0;
    static constexpr int kSlots = 4;
    static constexpr bool kStreamed = false;
    static constexpr int kRowsPerPass = 1;
    struct Regs { uint4 q0, q1; uint2 hdr; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int s) {
        const uint2* p = reinterpret_cast<const uint2*>(blk);                  // blocks are 8-byte aligned
        r.hdr = p[0];
        r.q0 = make_uint4(p[1 + 4 * s].x, p[1 + 4 * s].y, p[2 + 4 * s].x, p[2 + 4 * s].y);
        r.q1 = make_uint4(p[3 + 4 * s].x, p[3 + 4 * s].y, p[4 + 4 * s].x, p[4 + 4 * s].y);
    }
    static __device__ __forceinline__ void stage_tables(unsigned char*) {}
    static __device__ __forceinline__ void a_map(AMap<kSlots>& am, int col, int ks, int kpad, int zero_off) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int g = 2 * ks + (t >> 1);
            const bool active = (col >> 1) == g;
            am.off[t] = active ? ((col & 1) ? kpad : 0) + 32 * g + 16 * (t & 1) : zero_off;
            am.step[t] = active ? 256 : 0;
            am.on[t] = active;
        }
    }
    // four codes (one per byte, 0..15) -> four table values
    static __device__ __forceinline__ uint32_t values4(uint32_t codes) {
        const uint32_t low3 = codes & 0x07070707u;
        const uint32_t lower = __builtin_amdgcn_perm(0xF6EADDCFu, 0xBFAD9881u, low3);   // -127 -104 -83 -65 | -49 -35 -22 -10
        const uint32_t upper = __builtin_amdgcn_perm(0x71594535u, 0x26190D01u, low3);   // 1 13 25 38 | 53 69 89 113
        return __builtin_amdgcn_perm(upper, lower, ((codes >> 1) & 0x04040404u) | 0x03020100u);
    }
    static __device__ __forceinline__ float block(const Regs& r, int s, int b, const unsigned char* smem, const AMap<kSlots>& am,
                                                  const StagedX& sx, const unsigned char*) {
        v4i c = {0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint4 q = (t < 2) ? r.q0 : r.q1;
            const int sh = 4 * (t & 1);
            const v4i bw = as_v4i(values4((q.x >> sh) & 0x0f0f0f0fu), values4((q.y >> sh) & 0x0f0f0f0fu),
                                  values4((q.z >> sh) & 0x0f0f0f0fu), values4((q.w >> sh) & 0x0f0f0f0fu));
            const uint4 a = *reinterpret_cast<const uint4*>(smem + am.off[t] + b * am.step[t]);
            c = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(a.x, a.y, a.z, a.w), bw, c, 0, 0, 0);
        }
        const float v0 = static_cast<float>(__mul24(c.x, 254) + c.y);         // group 2 s: 254 * high term + low term
        const float v1 = static_cast<float>(__mul24(c.z, 254) + c.w);         // group 2 s + 1
        const float4 g2 = *reinterpret_cast<const float4*>(sx.gs + b * 8 + 2 * s);   // {xs0 / 254, sum0, xs1 / 254, sum1}
        const uint32_t scales_h = r.hdr.x >> 16, sl = (r.hdr.y >> (8 * s)) & 0xffu;
        const int ls0 = static_cast<int>((sl & 15u) | (((scales_h >> (4 * s)) & 3u) << 4)) - 32;
        const int ls1 = static_cast<int>((sl >> 4) | (((scales_h >> (4 * s + 2)) & 3u) << 4)) - 32;
        return f16_bits_to_float(r.hdr.x & 0xffffu) * (static_cast<float>(ls0) * g2.x * v0 + static_cast<float>(ls1) * g2.z * v1);
    }
};

// ------------------------------------------------------------------------------------------------
// IQ2_XS: 74 B = d(2) qs u16[32] scales(8).  Entry e (8 weights): grid id = low 9 bits of qs[e], sign
// index = high 7 bits; two 4-bit scales per 32 weights (low nibble: first 16); w = d (2 ls + 1) / 8 *
// grid * sign.  Lane (n, s) holds qs[8 s, 8 s + 8) = four 16-weight groups and scale bytes 2 s, 2 s + 1.
// A rows as for IQ1_M: m = 16-group, one MFMA set per activation term, MFMA t, slice s carries group
// 4 s + t.  LDS tables: 512 x 8 magnitude bytes, then the 128 x 8 sign masks.  Blocks are 2-byte aligned.
// ------------------------------------------------------------------------------------------------
struct IQ2XSm {
    static constexpr int kBlockBytes = 74;
    static constexpr int kTableBytes = 4096 + 1024;
    static constexpr int kSlots = 8;                           // [term][t]
    static constexpr bool kStreamed = false;
    struct Regs { uint4 q; uint32_t sc, d; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int s) {
        r.q = load16_a2(blk + 2 + 16 * s);
        r.sc = *reinterpret_cast<const uint16_t*>(blk + 66 + 2 * s);
        r.d = *reinterpret_cast<const uint16_t*>(blk);
    }
    static __device__ __forceinline__ void stage_tables(unsigned char* lds) {
        copy_to_lds(lds, reinterpret_cast<const unsigned char*>(PLLM_IQ2XS_GRID), 4096);
        copy_to_lds(lds + 4096, reinterpret_cast<const unsigned char*>(PLLM_IQ2XXS_SIGN_MASKS.v), 1024);
    }
    static __device__ __forceinline__ void a_map(AMap<kSlots>& am, int col, int ks, int kpad, int zero_off) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const bool active = col == 4 * ks + t;
            am.off[t] = active ? 16 * col : zero_off;
            am.off[4 + t] = active ? kpad + 16 * col : zero_off;
            am.step[t] = am.step[4 + t] = active ? 256 : 0;
            am.on[t] = am.on[4 + t] = active;
        }
    }
    static __device__ __forceinline__ uint2 signed8(const uint2* grid, const uint2* sign, uint32_t q16) {
        const uint2 g = grid[q16 & 511u], m = sign[q16 >> 9];
        // negate the masked bytes: (g ^ 0xff) + 1 never carries out of a byte because g >= 8
        return make_uint2((g.x ^ m.x) + (m.x & 0x01010101u), (g.y ^ m.y) + (m.y & 0x01010101u));
    }
    static __device__ __forceinline__ float block(const Regs& r, int s, int b, const unsigned char* smem, const AMap<kSlots>& am,
                                                  const StagedX& sx, const unsigned char* tables) {
        const uint2* grid = reinterpret_cast<const uint2*>(tables);
        const uint2* sign = grid + 512;
        v4i ch = {0, 0, 0, 0}, cl = {0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 4; ++t) {                                          // 16-weight group t of the lane = entries 2 t, 2 t + 1
            const uint32_t pair = t == 0 ? r.q.x : t == 1 ? r.q.y : t == 2 ? r.q.z : r.q.w;
            const uint2 w0 = signed8(grid, sign, pair & 0xffffu), w1 = signed8(grid, sign, pair >> 16);
            const v4i bw = as_v4i(w0.x, w0.y, w1.x, w1.y);
            const uint4 ah = *reinterpret_cast<const uint4*>(smem + am.off[t] + b * am.step[t]);
            const uint4 al = *reinterpret_cast<const uint4*>(smem + am.off[4 + t] + b * am.step[4 + t]);
            ch = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(ah.x, ah.y, ah.z, ah.w), bw, ch, 0, 0, 0);
            cl = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(al.x, al.y, al.z, al.w), bw, cl, 0, 0, 0);
        }
        const float4 g2 = *reinterpret_cast<const float4*>(sx.gs + b * 8 + 2 * s);   // {xs0 / 254, sum0, xs1 / 254, sum1}
        const float l0 = static_cast<float>(2 * (r.sc & 15u) + 1), l1 = static_cast<float>(2 * ((r.sc >> 4) & 15u) + 1);
        const float l2 = static_cast<float>(2 * ((r.sc >> 8) & 15u) + 1), l3 = static_cast<float>(2 * (r.sc >> 12) + 1);
        const float v = l0 * g2.x * static_cast<float>(__mul24(ch.x, 254) + cl.x) + l1 * g2.x * static_cast<float>(__mul24(ch.y, 254) + cl.y) +
                        l2 * g2.z * static_cast<float>(__mul24(ch.z, 254) + cl.z) + l3 * g2.z * static_cast<float>(__mul24(ch.w, 254) + cl.w);
        return 0.125f * f16_bits_to_float(r.d) * v;
    }
    // The block against R activation images that lie image_stride apart (each with its zero bytes behind it, offsets of am
    // relative to the image): the signed codes are looked up once; per image the same products and the same float steps as block().
    static constexpr int kRowsPerPass = 2;                     // (every further row costs as much as the lookups: 8 MFMAs per block)
    template <int R>
    static __device__ __forceinline__ void block_rows(const Regs& r, int s, int b, const unsigned char* img0, int image_stride,
                                                      const AMap<kSlots>& am, int kpad, const unsigned char* tables, float (&acc)[R]) {
        const uint2* grid = reinterpret_cast<const uint2*>(tables);
        const uint2* sign = grid + 512;
        v4i ch[R], cl[R];
#pragma unroll
        for (int i = 0; i < R; ++i) { ch[i] = v4i{0, 0, 0, 0}; cl[i] = v4i{0, 0, 0, 0}; }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t pair = t == 0 ? r.q.x : t == 1 ? r.q.y : t == 2 ? r.q.z : r.q.w;
            const uint2 w0 = signed8(grid, sign, pair & 0xffffu), w1 = signed8(grid, sign, pair >> 16);
            const v4i bw = as_v4i(w0.x, w0.y, w1.x, w1.y);
#pragma unroll
            for (int i = 0; i < R; ++i) {
                const unsigned char* img = img0 + i * image_stride;
                const uint4 ah = *reinterpret_cast<const uint4*>(img + am.off[t] + b * am.step[t]);
                const uint4 al = *reinterpret_cast<const uint4*>(img + am.off[4 + t] + b * am.step[4 + t]);
                ch[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(ah.x, ah.y, ah.z, ah.w), bw, ch[i], 0, 0, 0);
                cl[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(al.x, al.y, al.z, al.w), bw, cl[i], 0, 0, 0);
            }
        }
        const float l0 = static_cast<float>(2 * (r.sc & 15u) + 1), l1 = static_cast<float>(2 * ((r.sc >> 4) & 15u) + 1);
        const float l2 = static_cast<float>(2 * ((r.sc >> 8) & 15u) + 1), l3 = static_cast<float>(2 * (r.sc >> 12) + 1);
        const float d8 = 0.125f * f16_bits_to_float(r.d);
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const float4 g2 = *reinterpret_cast<const float4*>(img0 + i * image_stride + 2 * kpad + (b * 8 + 2 * s) * 8);
            const float v = l0 * g2.x * static_cast<float>(__mul24(ch[i].x, 254) + cl[i].x) + l1 * g2.x * static_cast<float>(__mul24(ch[i].y, 254) + cl[i].y) +
                            l2 * g2.z * static_cast<float>(__mul24(ch[i].z, 254) + cl[i].z) + l3 * g2.z * static_cast<float>(__mul24(ch[i].w, 254) + cl[i].w);
            acc[i] += d8 * v;
        }
    }
};

// ------------------------------------------------------------------------------------------------
// IQ3_XXS: 98 B = d(2) grid ids(64) aux u32[8].  An id gives four weights from a 256-entry grid; aux of a
// sub-block (32 weights) holds four 7-bit sign indices (one per 8 weights) and a 4-bit scale;
// w = d (2 ls + 1) / 4 * grid * sign.  Lane (n, s) holds ids [16 s, 16 s + 16) = groups 2 s, 2 s + 1 and their
// two aux words.  A rows as for IQ2_XXS.  LDS tables: 256 x 4 magnitude bytes, then the 128 x 8 sign
// masks.  Blocks are 2-byte aligned.
// ------------------------------------------------------------------------------------------------
struct IQ3XXSm {
    static constexpr int kBlockBytes = 98;
    static constexpr int kTableBytes = 1024 + 1024;
    static constexpr int kSlots = 4;
    static constexpr bool kStreamed = false;
    struct Regs { uint4 ids; uint32_t aux0, aux1, d; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int s) {
        r.ids = load16_a2(blk + 2 + 16 * s);
        r.aux0 = reinterpret_cast<const Unaligned4*>(blk + 66 + 8 * s)->v;
        r.aux1 = reinterpret_cast<const Unaligned4*>(blk + 70 + 8 * s)->v;
        r.d = *reinterpret_cast<const uint16_t*>(blk);
    }
    static __device__ __forceinline__ void stage_tables(unsigned char* lds) {
        copy_to_lds(lds, reinterpret_cast<const unsigned char*>(PLLM_IQ3XXS_GRID), 1024);
        copy_to_lds(lds + 1024, reinterpret_cast<const unsigned char*>(PLLM_IQ2XXS_SIGN_MASKS.v), 1024);
    }
    static __device__ __forceinline__ void a_map(AMap<kSlots>& am, int col, int ks, int kpad, int zero_off) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int g = 2 * ks + (t >> 1);
            const bool active = (col >> 1) == g;
            am.off[t] = active ? ((col & 1) ? kpad : 0) + 32 * g + 16 * (t & 1) : zero_off;
            am.step[t] = active ? 256 : 0;
            am.on[t] = active;
        }
    }
    static __device__ __forceinline__ uint32_t signed4(uint32_t g, uint32_t m) { return (g ^ m) + (m & 0x01010101u); }   // g >= 4: no carry
    static __device__ __forceinline__ float block(const Regs& r, int s, int b, const unsigned char* smem, const AMap<kSlots>& am,
                                                  const StagedX& sx, const unsigned char* tables) {
        const uint32_t* grid = reinterpret_cast<const uint32_t*>(tables);
        const uint2* sign = reinterpret_cast<const uint2*>(tables + 1024);
        v4i c = {0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 4; ++t) {                                          // half t % 2 of group 2 s + t / 2: four ids, two sign indices
            const uint32_t ids = t == 0 ? r.ids.x : t == 1 ? r.ids.y : t == 2 ? r.ids.z : r.ids.w;
            const uint32_t aux = (t < 2) ? r.aux0 : r.aux1;
            const uint2 m0 = sign[(aux >> (14 * (t & 1))) & 127u], m1 = sign[(aux >> (14 * (t & 1) + 7)) & 127u];
            const v4i bw = as_v4i(signed4(grid[ids & 0xffu], m0.x), signed4(grid[(ids >> 8) & 0xffu], m0.y),
                                  signed4(grid[(ids >> 16) & 0xffu], m1.x), signed4(grid[ids >> 24], m1.y));
            const uint4 a = *reinterpret_cast<const uint4*>(smem + am.off[t] + b * am.step[t]);
            c = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(a.x, a.y, a.z, a.w), bw, c, 0, 0, 0);
        }
        const float v0 = static_cast<float>(__mul24(c.x, 254) + c.y);         // group 2 s: 254 * high term + low term
        const float v1 = static_cast<float>(__mul24(c.z, 254) + c.w);         // group 2 s + 1
        const float4 g2 = *reinterpret_cast<const float4*>(sx.gs + b * 8 + 2 * s);   // {xs0 / 254, sum0, xs1 / 254, sum1}
        const float ls0 = static_cast<float>(2 * (r.aux0 >> 28) + 1), ls1 = static_cast<float>(2 * (r.aux1 >> 28) + 1);
        return 0.25f * f16_bits_to_float(r.d) * (ls0 * g2.x * v0 + ls1 * g2.z * v1);
    }
    // The block against R activation images (as IQ2XSm::block_rows): ids and signs looked up once.
    static constexpr int kRowsPerPass = 2;                     // (four rows lost: 17408x5120 55.7 us against 44.8 on the tile kernel, every workgroup quantizes all rows)
    template <int R>
    static __device__ __forceinline__ void block_rows(const Regs& r, int s, int b, const unsigned char* img0, int image_stride,
                                                      const AMap<kSlots>& am, int kpad, const unsigned char* tables, float (&acc)[R]) {
        const uint32_t* grid = reinterpret_cast<const uint32_t*>(tables);
        const uint2* sign = reinterpret_cast<const uint2*>(tables + 1024);
        v4i c[R];
#pragma unroll
        for (int i = 0; i < R; ++i) c[i] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t ids = t == 0 ? r.ids.x : t == 1 ? r.ids.y : t == 2 ? r.ids.z : r.ids.w;
            const uint32_t aux = (t < 2) ? r.aux0 : r.aux1;
            const uint2 m0 = sign[(aux >> (14 * (t & 1))) & 127u], m1 = sign[(aux >> (14 * (t & 1) + 7)) & 127u];
            const v4i bw = as_v4i(signed4(grid[ids & 0xffu], m0.x), signed4(grid[(ids >> 8) & 0xffu], m0.y),
                                  signed4(grid[(ids >> 16) & 0xffu], m1.x), signed4(grid[ids >> 24], m1.y));
#pragma unroll
            for (int i = 0; i < R; ++i) {
                const uint4 a = *reinterpret_cast<const uint4*>(img0 + i * image_stride + am.off[t] + b * am.step[t]);
                c[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(a.x, a.y, a.z, a.w), bw, c[i], 0, 0, 0);
            }
        }
        const float ls0 = static_cast<float>(2 * (r.aux0 >> 28) + 1), ls1 = static_cast<float>(2 * (r.aux1 >> 28) + 1);
        const float d4 = 0.25f * f16_bits_to_float(r.d);
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const float v0 = static_cast<float>(__mul24(c[i].x, 254) + c[i].y);
            const float v1 = static_cast<float>(__mul24(c[i].z, 254) + c[i].w);
            const float4 g2 = *reinterpret_cast<const float4*>(img0 + i * image_stride + 2 * kpad + (b * 8 + 2 * s) * 8);
            acc[i] += d4 * (ls0 * g2.x * v0 + ls1 * g2.z * v1);
        }
    }
};

template <int COPIES>
template <int WAVES>
__device__ __forceinline__ void IQ2XXSmT<COPIES>::dma_tables(uint32_t lds_base, int wave, int lane) {
    static_assert(COPIES == 1, "single copy only");
    dma_share<WAVES>(reinterpret_cast<const unsigned char*>(PLLM_IQ2XXS_GRID), lds_base, 2048, wave, lane);
    dma_share<WAVES>(reinterpret_cast<const unsigned char*>(PLLM_IQ2XXS_SIGN_MASKS.v), lds_base + 2048, 1024, wave, lane);
}
template <int WAVES>
__device__ __forceinline__ void IQ1Mm::dma_tables(uint32_t lds_base, int wave, int lane) {
    dma_share<WAVES>(reinterpret_cast<const unsigned char*>(PLLM_IQ1_DELTA_CODES.v), lds_base, kTableBytes, wave, lane);
}

}  // namespace pllm
