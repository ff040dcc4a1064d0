// Prefill matmul y[T, N] = x[T, K] . dequant(W)[N, K]^T over raw super-blocks, on f16 MFMA.
//
// A workgroup owns a 128 (tokens) x 128 (weight rows) output tile and walks K in chunks of 64
// weights (one quarter of a super-block).  Per chunk every thread pulls 16 bytes of codes plus the
// block header straight from the raw tensor, decodes 32 weights in float32 exactly as the block
// decoders do, rounds them once to fp16 and stores them in LDS; the activations arrive as fp16
// (a pre-pass scales every token row by a power of two so that its largest value sits just below
// 2^14, which keeps bf16 inputs exact and cannot overflow).  The four waves then run
// v_mfma_f32_32x32x16_f16 on 64 x 64 sub-tiles with float32 accumulators.  LDS is double buffered:
// the loads and the decode of chunk c+1 overlap the MFMAs of chunk c.
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
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kBM = 128, kBN = 128, kBK = 64;
constexpr int kLds = kBK + 8;                       // halves per LDS row: 144 bytes, conflict-free for 16-byte reads
constexpr int kTileHalves = 128 * kLds;

// ---- activation pre-pass --------------------------------------------------------------------------
// xh[t, 0..kp) = fp16(x[t, :] * 2^-e_t) (zero beyond k), scale[t] = 2^e_t, amax_t * 2^-e_t in [2^13, 2^14)
__global__ __launch_bounds__(256) void act_f16_kernel(const void* __restrict__ x, int x_dtype, _Float16* __restrict__ xh,
                                                      float* __restrict__ scale, int k, int kp) {
    __shared__ float red[4];
    const size_t xoff = static_cast<size_t>(blockIdx.x) * k;
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

// ---- per-format decode of one 64-weight chunk ----------------------------------------------------
// Thread (row, h) of the staging step decodes weights [64 c + 16 h, +16) and [64 c + 32 + 16 h, +16)
// of its row (c = chunk index along K) into lo[16] and hi[16].
struct K4Pair { float d_sc0, d_sc1, dm0, dm1; };
__device__ __forceinline__ K4Pair k4_pair(const uint4& hdr, int p) {
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
    K4Pair r;
    r.d_sc0 = d * static_cast<float>(scw & 0xffu);
    r.d_sc1 = d * static_cast<float>((scw >> 8) & 0xffu);
    r.dm0 = dmin * static_cast<float>(mnw & 0xffu);
    r.dm1 = dmin * static_cast<float>((mnw >> 8) & 0xffu);
    return r;
}

typedef _Float16 half4 __attribute__((ext_vector_type(4)));
struct Half32 { half4 lo[4], hi[4]; };            // lo = weights [16 h, +16), hi = weights [32 + 16 h, +16) of the chunk

__device__ __forceinline__ half4 affine4(uint32_t b0, uint32_t b1, uint32_t b2, uint32_t b3, float scale, float minus) {
    half4 r;
    r.x = static_cast<_Float16>(scale * static_cast<float>(b0) - minus);
    r.y = static_cast<_Float16>(scale * static_cast<float>(b1) - minus);
    r.z = static_cast<_Float16>(scale * static_cast<float>(b2) - minus);
    r.w = static_cast<_Float16>(scale * static_cast<float>(b3) - minus);
    return r;
}

struct GQ4K {
    static constexpr int kBlockBytes = 144;
    struct Regs { uint4 hdr; uint4 qs; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int p, int h) {
        r.hdr = *reinterpret_cast<const uint4*>(blk);
        r.qs = *reinterpret_cast<const uint4*>(blk + 16 + 32 * p + 16 * h);
    }
    static __device__ __forceinline__ void word(uint32_t q, const K4Pair& s, half4& lo, half4& hi) {
        lo = affine4(q & 15u, (q >> 8) & 15u, (q >> 16) & 15u, (q >> 24) & 15u, s.d_sc0, s.dm0);
        hi = affine4((q >> 4) & 15u, (q >> 12) & 15u, (q >> 20) & 15u, q >> 28, s.d_sc1, s.dm1);
    }
    static __device__ __forceinline__ void decode(const Regs& r, int p, Half32& o) {
        const K4Pair s = k4_pair(r.hdr, p);
        word(r.qs.x, s, o.lo[0], o.hi[0]);
        word(r.qs.y, s, o.lo[1], o.hi[1]);
        word(r.qs.z, s, o.lo[2], o.hi[2]);
        word(r.qs.w, s, o.lo[3], o.hi[3]);
    }
};

struct GQ5K {
    static constexpr int kBlockBytes = 176;
    struct Regs { uint4 hdr; uint4 qh; uint4 qs; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int p, int h) {
        r.hdr = *reinterpret_cast<const uint4*>(blk);
        r.qh = *reinterpret_cast<const uint4*>(blk + 16 + 16 * h);
        r.qs = *reinterpret_cast<const uint4*>(blk + 48 + 32 * p + 16 * h);
    }
    // g = the high-bit bytes shifted so that bit 0 of every byte belongs to the low nibble's weight
    // and bit 1 to the high nibble's weight
    static __device__ __forceinline__ void word(uint32_t q, uint32_t g, const K4Pair& s, half4& lo, half4& hi) {
        const uint32_t l = (q & 0x0f0f0f0fu) | ((g & 0x01010101u) << 4);
        const uint32_t u = ((q >> 4) & 0x0f0f0f0fu) | ((g & 0x02020202u) << 3);
        lo = affine4(l & 31u, (l >> 8) & 31u, (l >> 16) & 31u, l >> 24, s.d_sc0, s.dm0);
        hi = affine4(u & 31u, (u >> 8) & 31u, (u >> 16) & 31u, u >> 24, s.d_sc1, s.dm1);
    }
    static __device__ __forceinline__ void decode(const Regs& r, int p, Half32& o) {
        const K4Pair s = k4_pair(r.hdr, p);
        const int sft = 2 * p;
        word(r.qs.x, r.qh.x >> sft, s, o.lo[0], o.hi[0]);
        word(r.qs.y, r.qh.y >> sft, s, o.lo[1], o.hi[1]);
        word(r.qs.z, r.qh.z >> sft, s, o.lo[2], o.hi[2]);
        word(r.qs.w, r.qh.w >> sft, s, o.lo[3], o.hi[3]);
    }
};

template <typename FMT>
__global__ __launch_bounds__(256) void gemm_f16_kernel(
    const _Float16* __restrict__ xh, const float* __restrict__ xscale, const uint8_t* __restrict__ w,
    void* __restrict__ y, int y_dtype, int t_rows, int n, int bpr) {
    extern __shared__ __align__(16) unsigned char smem[];
    _Float16* xs_buf = reinterpret_cast<_Float16*>(smem);                 // [2][128][kLds]
    _Float16* ws_buf = xs_buf + 2 * kTileHalves;                          // [2][128][kLds]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;                              // 2 x 2 waves, 64 x 64 each
    const int n0 = blockIdx.x * kBN, t0 = blockIdx.y * kBM;
    const int kp = bpr * 256;
    const int chunks = bpr * 4;

    // staging roles: thread (row, h)
    const int srow = tid >> 1, sh = tid & 1;
    const uint8_t* wrow = w + static_cast<size_t>(min(n0 + srow, n - 1)) * bpr * FMT::kBlockBytes;
    const _Float16* xrow = xh + static_cast<size_t>(min(t0 + srow, t_rows - 1)) * kp + 32 * sh;

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // two register sets: while chunk c is multiplied, chunk c+1 is decoded into the other LDS buffer
    // from one set and chunk c+2 is already being fetched into the other
    typename FMT::Regs wreg0, wreg1;
    // (the activation registers are separate variables on purpose: grouped in an aggregate the four
    // copies fuse into one block copy that the compiler then keeps in scratch memory)
    uint4 xa0, xb0, xc0, xd0, xa1, xb1, xc1, xd1;
    auto fetch = [&](int c, typename FMT::Regs& wr, uint4& xa, uint4& xb, uint4& xc, uint4& xd) {
        FMT::load(wr, wrow + static_cast<size_t>(c >> 2) * FMT::kBlockBytes, c & 3, sh);
        const uint4* xp = reinterpret_cast<const uint4*>(xrow + static_cast<size_t>(c) * kBK);
        xa = xp[0]; xb = xp[1]; xc = xp[2]; xd = xp[3];
    };
    auto stage = [&](int c, const typename FMT::Regs& wr, const uint4& xa, const uint4& xb, const uint4& xc, const uint4& xd, int buf) {
        Half32 d;
        FMT::decode(wr, c & 3, d);
        half4* wlo = reinterpret_cast<half4*>(ws_buf + buf * kTileHalves + srow * kLds + 16 * sh);
        wlo[0] = d.lo[0]; wlo[1] = d.lo[1]; wlo[2] = d.lo[2]; wlo[3] = d.lo[3];
        wlo[8] = d.hi[0]; wlo[9] = d.hi[1]; wlo[10] = d.hi[2]; wlo[11] = d.hi[3];
        uint4* xdst = reinterpret_cast<uint4*>(xs_buf + buf * kTileHalves + srow * kLds + 32 * sh);
        xdst[0] = xa; xdst[1] = xb; xdst[2] = xc; xdst[3] = xd;
    };
    auto multiply = [&](int buf) {
        const _Float16* xt = xs_buf + buf * kTileHalves + (wm * 64 + (lane & 31)) * kLds + 8 * (lane >> 5);
        const _Float16* wt = ws_buf + buf * kTileHalves + (wn * 64 + (lane & 31)) * kLds + 8 * (lane >> 5);
#pragma unroll
        for (int ks = 0; ks < kBK / 16; ++ks) {
            const half8 a0 = *reinterpret_cast<const half8*>(xt + 16 * ks);
            const half8 a1 = *reinterpret_cast<const half8*>(xt + 32 * kLds + 16 * ks);
            const half8 b0 = *reinterpret_cast<const half8*>(wt + 16 * ks);
            const half8 b1 = *reinterpret_cast<const half8*>(wt + 32 * kLds + 16 * ks);
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, b1, acc[1][1], 0, 0, 0);
        }
    };

    // chunks is a multiple of 4, so the loop below runs in pairs with compile-time set/buffer indices
    fetch(0, wreg0, xa0, xb0, xc0, xd0);
    fetch(1, wreg1, xa1, xb1, xc1, xd1);
    stage(0, wreg0, xa0, xb0, xc0, xd0, 0);
    __syncthreads();
    for (int c = 0; c < chunks; c += 2) {
        if (c + 2 < chunks) fetch(c + 2, wreg0, xa0, xb0, xc0, xd0);
        multiply(0);
        stage(c + 1, wreg1, xa1, xb1, xc1, xd1, 1);
        __syncthreads();
        if (c + 3 < chunks) fetch(c + 3, wreg1, xa1, xb1, xc1, xd1);
        multiply(1);
        if (c + 2 < chunks) stage(c + 2, wreg0, xa0, xb0, xc0, xd0, 0);
        __syncthreads();
    }

    // D[m][n]: lane holds column n = lane % 32 and rows 8 * (v / 4) + 4 * (lane / 32) + v % 4
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
            const int col = n0 + wn * 64 + ni * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = t0 + wm * 64 + mi * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (row < t_rows && col < n) store_any(y, y_dtype, static_cast<size_t>(row) * n + col, acc[mi][ni][v] * xscale[row]);
            }
        }
}

template <typename FMT>
int launch_gemm(const _Float16* xh, const float* xscale, const uint8_t* w, void* y, int y_dtype, int t_rows, int n, int bpr, hipStream_t stream) {
    const size_t smem = static_cast<size_t>(4) * kTileHalves * sizeof(_Float16);          // 73 728 bytes
    auto kern = gemm_f16_kernel<FMT>;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem)) != hipSuccess)
        return PLLM_ERR_UNSUPPORTED;
    dim3 grid((n + kBN - 1) / kBN, (t_rows + kBM - 1) / kBM);
    hipLaunchKernelGGL(kern, grid, dim3(256), smem, stream, xh, xscale, w, y, y_dtype, t_rows, n, bpr);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

size_t align256(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }

}  // namespace

bool gemm_f16_supports(int type_id) { return type_id == PLLM_TYPE_Q4_K || type_id == PLLM_TYPE_Q5_K; }

size_t gemm_f16_workspace_bytes(int rows, int bpr) {
    return align256(static_cast<size_t>(rows) * bpr * 256 * sizeof(_Float16)) + align256(static_cast<size_t>(rows) * sizeof(float));
}

int gemm_f16(const void* x, int x_dtype, const uint8_t* w, int type_id, void* y, int y_dtype,
             int rows, int k, int n, int bpr, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    if (!workspace || workspace_bytes < gemm_f16_workspace_bytes(rows, bpr)) return PLLM_ERR_WORKSPACE;
    _Float16* xh = static_cast<_Float16*>(workspace);
    float* xscale = reinterpret_cast<float*>(static_cast<unsigned char*>(workspace) + align256(static_cast<size_t>(rows) * bpr * 256 * sizeof(_Float16)));
    hipLaunchKernelGGL(act_f16_kernel, dim3(rows), dim3(256), 0, stream, x, x_dtype, xh, xscale, k, bpr * 256);
    if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
    switch (type_id) {
        case PLLM_TYPE_Q4_K: return launch_gemm<GQ4K>(xh, xscale, w, y, y_dtype, rows, n, bpr, stream);
        case PLLM_TYPE_Q5_K: return launch_gemm<GQ5K>(xh, xscale, w, y, y_dtype, rows, n, bpr, stream);
        default: return PLLM_ERR_UNSUPPORTED;
    }
}

}  // namespace pllm
