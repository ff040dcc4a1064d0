// Decode matvec over raw Q4_K / Q5_K / Q2_K super-blocks (bandwidth-bound, wave64).
//
// Work split: a "team" of LPB adjacent lanes owns one 256-weight super-block at a time, every lane
// loading 16 bytes of quants with one global_load_dwordx4 plus the block header shared by the team.
// TPR teams stride over the super-blocks of one output row; a 256-thread workgroup therefore covers
// (256 / LPB) / TPR rows.  All weight loads of a pass are issued before the workgroup quantizes the
// activation row into LDS (two int8 terms per value), so the quantization hides under the HBM
// latency.  Dots are v_dot4_i32_i8; scales and mins are unpacked in registers; the per-row sum is a
// cross-lane reduction over the LPB * TPR lanes that share the row.
#include "pllm_device.h"

namespace pllm {
namespace {

constexpr int kThreads = 256;

// ------------------------------------------------------------------------------------------------
// Q4_K: 144 B = d(2) dmin(2) scales(12) qs(128).  8 lanes per block; lane j holds qs[16j, 16j+16):
// low nibbles are weights 64p + 16h + i of group 2p, high nibbles the same offsets of group 2p+1
// (p = j >> 1, h = j & 1).
// ------------------------------------------------------------------------------------------------
struct Q4K {
    static constexpr int kLanesPerBlock = 8;
    static constexpr int kBlockBytes = 144;
    struct Regs { uint4 hdr; uint4 qs; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int j) {
        r.hdr = *reinterpret_cast<const uint4*>(blk);
        r.qs = *reinterpret_cast<const uint4*>(blk + 16 + 16 * j);
    }
    static __device__ __forceinline__ void zero(Regs& r) { r.hdr = make_uint4(0, 0, 0, 0); r.qs = r.hdr; }
};

// Q5_K: 176 B = d dmin scales(12) qh(32) qs(128).  Same lane map as Q4_K plus qh[16h, 16h+16):
// bit 2p of qh byte i is the fifth bit of the low-nibble weight, bit 2p+1 that of the high nibble.
struct Q5K {
    static constexpr int kLanesPerBlock = 8;
    static constexpr int kBlockBytes = 176;
    struct Regs { uint4 hdr; uint4 qh; uint4 qs; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int j) {
        r.hdr = *reinterpret_cast<const uint4*>(blk);
        r.qh = *reinterpret_cast<const uint4*>(blk + 16 + 16 * (j & 1));
        r.qs = *reinterpret_cast<const uint4*>(blk + 48 + 16 * j);
    }
    static __device__ __forceinline__ void zero(Regs& r) { r.hdr = make_uint4(0, 0, 0, 0); r.qh = r.hdr; r.qs = r.hdr; }
};

// Eight 6-bit scales and mins of a K-quant header -> scale/min of groups 2p and 2p+1 as floats.
__device__ __forceinline__ void k4_scales(const uint4& hdr, int p, float& sc0, float& sc1, float& m0, float& m1) {
    const uint32_t u0 = hdr.y, u1 = hdr.z, u2 = hdr.w;
    const uint32_t sc_lo = u0 & 0x3f3f3f3fu;
    const uint32_t mn_lo = u1 & 0x3f3f3f3fu;
    const uint32_t sc_hi = (u2 & 0x0f0f0f0fu) | (((u0 >> 6) & 0x03030303u) << 4);
    const uint32_t mn_hi = ((u2 >> 4) & 0x0f0f0f0fu) | (((u1 >> 6) & 0x03030303u) << 4);
    const uint32_t scw = (p < 2 ? sc_lo : sc_hi) >> ((p & 1) * 16);
    const uint32_t mnw = (p < 2 ? mn_lo : mn_hi) >> ((p & 1) * 16);
    sc0 = static_cast<float>(scw & 0xffu);
    sc1 = static_cast<float>((scw >> 8) & 0xffu);
    m0 = static_cast<float>(mnw & 0xffu);
    m1 = static_cast<float>((mnw >> 8) & 0xffu);
}

__device__ __forceinline__ float k45_finish(const uint4& hdr, int p, int h, int blk, const StagedX& sx,
                                            const uint4& w0, const uint4& w1) {
    const int base = blk * 256 + 64 * p + 16 * h;
    const uint4 a0h = *reinterpret_cast<const uint4*>(sx.hi + base);
    const uint4 a1h = *reinterpret_cast<const uint4*>(sx.hi + base + 32);
    const uint4 a0l = *reinterpret_cast<const uint4*>(sx.lo + base);
    const uint4 a1l = *reinterpret_cast<const uint4*>(sx.lo + base + 32);
    int s0h = dot4(w0.x, a0h.x, 0); s0h = dot4(w0.y, a0h.y, s0h); s0h = dot4(w0.z, a0h.z, s0h); s0h = dot4(w0.w, a0h.w, s0h);
    int s0l = dot4(w0.x, a0l.x, 0); s0l = dot4(w0.y, a0l.y, s0l); s0l = dot4(w0.z, a0l.z, s0l); s0l = dot4(w0.w, a0l.w, s0l);
    int s1h = dot4(w1.x, a1h.x, 0); s1h = dot4(w1.y, a1h.y, s1h); s1h = dot4(w1.z, a1h.z, s1h); s1h = dot4(w1.w, a1h.w, s1h);
    int s1l = dot4(w1.x, a1l.x, 0); s1l = dot4(w1.y, a1l.y, s1l); s1l = dot4(w1.z, a1l.z, s1l); s1l = dot4(w1.w, a1l.w, s1l);
    float sc0, sc1, m0, m1;
    k4_scales(hdr, p, sc0, sc1, m0, m1);
    const float d = f16_bits_to_float(hdr.x & 0xffffu);
    const float dmin = f16_bits_to_float(hdr.x >> 16);
    const float xs0 = sx.xs[blk * 8 + 2 * p];
    const float xs1 = sx.xs[blk * 8 + 2 * p + 1];
    const float t0 = sx.sum16[blk * 16 + 4 * p + h];
    const float t1 = sx.sum16[blk * 16 + 4 * p + 2 + h];
    const float v0 = static_cast<float>(s0h) + static_cast<float>(s0l) * kLoInv;
    const float v1 = static_cast<float>(s1h) + static_cast<float>(s1l) * kLoInv;
    return d * (sc0 * xs0 * v0 + sc1 * xs1 * v1) - dmin * (m0 * t0 + m1 * t1);
}

__device__ __forceinline__ float lane_dot(const Q4K::Regs& r, int j, int blk, const StagedX& sx) {
    const uint4 q = r.qs;
    const uint4 w0 = make_uint4(q.x & 0x0f0f0f0fu, q.y & 0x0f0f0f0fu, q.z & 0x0f0f0f0fu, q.w & 0x0f0f0f0fu);
    const uint4 w1 = make_uint4((q.x >> 4) & 0x0f0f0f0fu, (q.y >> 4) & 0x0f0f0f0fu, (q.z >> 4) & 0x0f0f0f0fu, (q.w >> 4) & 0x0f0f0f0fu);
    return k45_finish(r.hdr, j >> 1, j & 1, blk, sx, w0, w1);
}

__device__ __forceinline__ float lane_dot(const Q5K::Regs& r, int j, int blk, const StagedX& sx) {
    const int p = j >> 1;
    const uint4 q = r.qs;
    const uint4 b = r.qh;
    const int s0 = 2 * p, s1 = 2 * p + 1;
    const uint4 w0 = make_uint4((q.x & 0x0f0f0f0fu) | (((b.x >> s0) & 0x01010101u) << 4),
                                (q.y & 0x0f0f0f0fu) | (((b.y >> s0) & 0x01010101u) << 4),
                                (q.z & 0x0f0f0f0fu) | (((b.z >> s0) & 0x01010101u) << 4),
                                (q.w & 0x0f0f0f0fu) | (((b.w >> s0) & 0x01010101u) << 4));
    const uint4 w1 = make_uint4(((q.x >> 4) & 0x0f0f0f0fu) | (((b.x >> s1) & 0x01010101u) << 4),
                                ((q.y >> 4) & 0x0f0f0f0fu) | (((b.y >> s1) & 0x01010101u) << 4),
                                ((q.z >> 4) & 0x0f0f0f0fu) | (((b.z >> s1) & 0x01010101u) << 4),
                                ((q.w >> 4) & 0x0f0f0f0fu) | (((b.w >> s1) & 0x01010101u) << 4));
    return k45_finish(r.hdr, p, j & 1, blk, sx, w0, w1);
}

// ------------------------------------------------------------------------------------------------
// Q2_K: 84 B = scales(16) qs(64) d(2) dmin(2).  4 lanes per block; lane j holds qs[16j, 16j+16):
// shift 2s of those bytes is group g = 8 * (j >> 1) + 2s + (j & 1), 16 weights each.
// ------------------------------------------------------------------------------------------------
struct Q2K {
    static constexpr int kLanesPerBlock = 4;
    static constexpr int kBlockBytes = 84;
    struct Regs { uint4 sc; uint4 qs; uint32_t dd; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int j) {
        // blocks are only 4-byte aligned: the loads below are dword-aligned vector loads
        const uint32_t* p = reinterpret_cast<const uint32_t*>(blk);
        r.sc = make_uint4(p[0], p[1], p[2], p[3]);
        const uint32_t* q = p + 4 + 4 * j;
        r.qs = make_uint4(q[0], q[1], q[2], q[3]);
        r.dd = p[20];
    }
    static __device__ __forceinline__ void zero(Regs& r) { r.sc = make_uint4(0, 0, 0, 0); r.qs = r.sc; r.dd = 0; }
};

__device__ __forceinline__ float lane_dot(const Q2K::Regs& r, int j, int blk, const StagedX& sx) {
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
        const float xs = sx.xs[blk * 8 + (g >> 1)];
        pos += static_cast<float>(sb & 15u) * xs * (static_cast<float>(sh) + static_cast<float>(sl) * kLoInv);
        neg += static_cast<float>(sb >> 4) * sx.sum16[blk * 16 + g];
    }
    return d * pos - dmin * neg;
}

// ------------------------------------------------------------------------------------------------
template <typename FMT, int ITERS>
__global__ __launch_bounds__(kThreads) void kquant_matvec_kernel(
    const void* __restrict__ x, int x_dtype, const uint8_t* __restrict__ w, void* __restrict__ y, int y_dtype,
    int k, int n, int bpr, int tpr_log2) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int LPB = FMT::kLanesPerBlock;
    const int kpad = bpr * 256;
    const StagedX sx = carve_staged_x(smem, kpad);

    const int tid = threadIdx.x;
    const int j = tid % LPB;
    const int team = tid / LPB;
    const int tpr = 1 << tpr_log2;
    const int rows_per_wg = (kThreads / LPB) >> tpr_log2;
    const int row = blockIdx.x * rows_per_wg + (team >> tpr_log2);
    const int slice = team & (tpr - 1);
    const bool row_ok = row < n;
    const uint8_t* wrow = w + static_cast<size_t>(row_ok ? row : 0) * bpr * FMT::kBlockBytes;
    const size_t xoff = static_cast<size_t>(blockIdx.y) * k;

    float acc = 0.0f;
    bool staged = false;
    for (int b0 = slice; b0 < bpr || !staged; b0 += tpr * ITERS) {
        typename FMT::Regs regs[ITERS];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int b = b0 + it * tpr;
            if (row_ok && b < bpr) FMT::load(regs[it], wrow + static_cast<size_t>(b) * FMT::kBlockBytes, j);
            else FMT::zero(regs[it]);
        }
        if (!staged) {                       // uniform across the workgroup: first trip of every thread
            stage_activations_any(x, x_dtype, xoff, k, kpad, sx);
            __syncthreads();
            staged = true;
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int b = b0 + it * tpr;
            if (row_ok && b < bpr) acc += lane_dot(regs[it], j, b, sx);
        }
    }
    // lanes sharing the row are LPB * tpr consecutive lanes
    const int width = LPB << tpr_log2;
    for (int off = 1; off < width; off <<= 1) acc += __shfl_xor(acc, off, 64);
    if (row_ok && (tid & (width - 1)) == 0) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + row, acc);
}

template <typename FMT, int ITERS>
int launch_one(const void* x, int x_dtype, const uint8_t* w, void* y, int y_dtype, int rows, int k, int n, int bpr,
               int tpr_log2, hipStream_t stream) {
    const int rows_per_wg = (kThreads / FMT::kLanesPerBlock) >> tpr_log2;
    const size_t smem = staged_x_bytes(bpr * 256);
    auto kern = kquant_matvec_kernel<FMT, ITERS>;
    if (smem > 64 * 1024) {
        if (smem > 160 * 1024) return PLLM_ERR_UNSUPPORTED;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(smem)) != hipSuccess)
            return PLLM_ERR_UNSUPPORTED;
    }
    dim3 grid((n + rows_per_wg - 1) / rows_per_wg, rows);
    hipLaunchKernelGGL(kern, grid, dim3(kThreads), smem, stream, x, x_dtype, w, y, y_dtype, k, n, bpr, tpr_log2);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

template <typename FMT>
int launch_fmt(const void* x, int x_dtype, const uint8_t* w, void* y, int y_dtype, int rows, int k, int n, int bpr,
               hipStream_t stream) {
    // teams per row: enough that a row's blocks are spread over lanes, few enough that every team
    // still has several blocks in flight
    int tpr_log2 = 0;
    while (tpr_log2 < 3 && (bpr >> (tpr_log2 + 1)) >= 3) ++tpr_log2;
    const int tpr = 1 << tpr_log2;
    const int niter = (bpr + tpr - 1) / tpr;
    const int passes = (niter + 7) / 8;
    const int iters = (niter + passes - 1) / passes;
#define PLLM_CASE(I) return launch_one<FMT, I>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, tpr_log2, stream)
    switch (iters) {
        case 1: PLLM_CASE(1);
        case 2: PLLM_CASE(2);
        case 3: PLLM_CASE(3);
        case 4: PLLM_CASE(4);
        case 5: PLLM_CASE(5);
        case 6: PLLM_CASE(6);
        default: PLLM_CASE(8);
    }
#undef PLLM_CASE
}

}  // namespace

int kquant_matvec(const void* x, int x_dtype, const uint8_t* w, int type_id, void* y, int y_dtype,
                  int rows, int k, int n, int bpr, hipStream_t stream) {
    switch (type_id) {
        case PLLM_TYPE_Q4_K: return launch_fmt<Q4K>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream);
        case PLLM_TYPE_Q5_K: return launch_fmt<Q5K>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream);
        case PLLM_TYPE_Q2_K: return launch_fmt<Q2K>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream);
        default: return PLLM_ERR_UNSUPPORTED;
    }
}

}  // namespace pllm
