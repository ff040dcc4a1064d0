// Decode matvec over raw Q8_0 blocks (34 B = fp16 scale + 32 int8), bandwidth-bound, wave64.
//
// 34-byte blocks are only 2-byte aligned, so lanes do not own blocks.  Instead a wave reads a row as
// an aligned byte stream, lane l taking 16 bytes at offset 16 * (c0 + l) with one
// global_load_dwordx4.  The activations are laid out in LDS as an IMAGE OF THE SAME STREAM: for
// every block two zero bytes where the weight stream has its scale, then the 32 int8 activation
// codes.  A dword of weights and the dword of the image at the same offset then line up byte for
// byte, and v_dot4_i32_i8 of the two is a partial dot that belongs to exactly one block (the scale
// bytes meet zeros).  The stream repeats every 17 dwords (two blocks): dwords 0..8 of a pair belong
// to the even block, 9..16 to the odd one, so four consecutive dwords touch at most two blocks.
// The fp16 scale of a lane's first block sits at most two lanes back and comes over with one
// ds_bpermute; only the first two lanes of a pass fetch theirs from memory.
#include "pllm_device.h"

namespace pllm {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;

struct Q8Image {
    int8_t* hi;   // [bpr * 34]
    int8_t* lo;   // [bpr * 34]
    float* xs;    // [bpr]
};

__device__ __forceinline__ void stage_q8_image(const void* x, int x_dtype, size_t xoff, int k, int bpr, const Q8Image& im) {
    const int kpad = bpr * 32;
    for (int e0 = threadIdx.x * 4; e0 < kpad; e0 += kThreads * 4) {
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = (e0 + i < k) ? load_any(x, x_dtype, xoff + e0 + i) : 0.0f;
        uint32_t hi, lo;
        float scale;
        quantize4(v, hi, lo, scale);
        const int b = e0 >> 5;
        const int j = (e0 & 31) >> 2;
        const int off = 34 * b + 2 + 4 * j;                       // 2-byte aligned
        *reinterpret_cast<uint16_t*>(im.hi + off) = static_cast<uint16_t>(hi);
        *reinterpret_cast<uint16_t*>(im.hi + off + 2) = static_cast<uint16_t>(hi >> 16);
        *reinterpret_cast<uint16_t*>(im.lo + off) = static_cast<uint16_t>(lo);
        *reinterpret_cast<uint16_t*>(im.lo + off + 2) = static_cast<uint16_t>(lo >> 16);
        if (j == 0) {
            *reinterpret_cast<uint16_t*>(im.hi + 34 * b) = 0;
            *reinterpret_cast<uint16_t*>(im.lo + 34 * b) = 0;
            im.xs[b] = scale;
        }
    }
}

// Contribution of one 16-byte chunk (index c in the row stream) held in w.
__device__ __forceinline__ float chunk_dot(const uint4& w, int c, int lane, uint32_t head_scale_bits, int bpr, const Q8Image& im) {
    const int g0 = 4 * c;
    const int pair = g0 / 17;
    const int t0 = g0 - 17 * pair;
    const int block_a = 2 * pair + (t0 >= 9 ? 1 : 0);
    const int k_a = min(4, (t0 < 9 ? 9 : 17) - t0);           // dwords of this chunk inside block A

    // the scale this lane carries, if any: low half of the dword at t == 0, high half of t == 8
    const bool in_hi = (t0 >= 5 && t0 <= 8);
    const int sel = (t0 == 0) ? 0 : (in_hi ? 8 - t0 : 17 - t0);
    const uint32_t wsel = sel == 0 ? w.x : sel == 1 ? w.y : sel == 2 ? w.z : w.w;
    const uint32_t own_bits = in_hi ? (wsel >> 16) : (wsel & 0xffffu);

    // scale of block A: own (t0 == 0) or one/two lanes back
    const int back = (t0 < 9) ? t0 : t0 - 8;                  // dwords back to the scale, 0..8
    const int dlanes = (back + 3) >> 2;
    const int src = lane - dlanes;
    const uint32_t got = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute((src & 63) << 2, static_cast<int>(own_bits)));
    const uint32_t a_bits = (t0 == 0) ? own_bits : (src >= 0 ? got : head_scale_bits);

    const uint4 ah = *reinterpret_cast<const uint4*>(im.hi + 16 * c);
    const uint4 al = *reinterpret_cast<const uint4*>(im.lo + 16 * c);
    const int h0 = dot4(w.x, ah.x, 0), h1 = dot4(w.y, ah.y, 0), h2 = dot4(w.z, ah.z, 0), h3 = dot4(w.w, ah.w, 0);
    const int l0 = dot4(w.x, al.x, 0), l1 = dot4(w.y, al.y, 0), l2 = dot4(w.z, al.z, 0), l3 = dot4(w.w, al.w, 0);
    const int ha = h0 + (k_a > 1 ? h1 : 0) + (k_a > 2 ? h2 : 0) + (k_a > 3 ? h3 : 0);
    const int la = l0 + (k_a > 1 ? l1 : 0) + (k_a > 2 ? l2 : 0) + (k_a > 3 ? l3 : 0);
    const int hb = (h0 + h1 + h2 + h3) - ha;
    const int lb = (l0 + l1 + l2 + l3) - la;

    const float xs_a = im.xs[block_a];
    float out = f16_bits_to_float(a_bits) * xs_a * (static_cast<float>(ha) + static_cast<float>(la) * kLoInv);
    if (k_a < 4) {
        const float xs_b = im.xs[min(block_a + 1, bpr - 1)];
        out += f16_bits_to_float(own_bits) * xs_b * (static_cast<float>(hb) + static_cast<float>(lb) * kLoInv);
    }
    return out;
}

template <int ITERS, int RW>
__global__ __launch_bounds__(kThreads) void q8_0_stream_kernel(
    const void* __restrict__ x, int x_dtype, const uint8_t* __restrict__ w, void* __restrict__ y, int y_dtype,
    int k, int n, int bpr) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int row_bytes = bpr * 34;                               // multiple of 272
    Q8Image im;
    im.hi = reinterpret_cast<int8_t*>(smem);
    im.lo = im.hi + row_bytes;
    im.xs = reinterpret_cast<float*>(im.lo + row_bytes);
    const int chunks = row_bytes >> 4;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int row0 = (blockIdx.x * kWaves + wave) * RW;
    const size_t xoff = static_cast<size_t>(blockIdx.y) * k;

    float acc[RW];
#pragma unroll
    for (int r = 0; r < RW; ++r) acc[r] = 0.0f;

    bool staged = false;
    for (int c0 = 0; c0 < chunks; c0 += 64 * ITERS) {
        uint4 regs[RW][ITERS];
        uint32_t head[RW][ITERS];
#pragma unroll
        for (int r = 0; r < RW; ++r) {
            const int row = row0 + r;
            const uint8_t* wrow = w + static_cast<size_t>(row < n ? row : 0) * row_bytes;
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int c = c0 + it * 64 + lane;
                const int cc = c < chunks ? c : 0;
                regs[r][it] = *reinterpret_cast<const uint4*>(wrow + 16 * cc);
                head[r][it] = 0;
                if (lane < 2) {
                    const int g0 = 4 * cc;
                    const int pair = g0 / 17;
                    const int t0 = g0 - 17 * pair;
                    const int block_a = 2 * pair + (t0 >= 9 ? 1 : 0);
                    head[r][it] = *reinterpret_cast<const uint16_t*>(wrow + 34 * block_a);
                }
            }
        }
        if (!staged) {
            stage_q8_image(x, x_dtype, xoff, k, bpr, im);
            __syncthreads();
            staged = true;
        }
#pragma unroll
        for (int r = 0; r < RW; ++r) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int c = c0 + it * 64 + lane;
                const bool ok = c < chunks;
                const float v = chunk_dot(regs[r][it], ok ? c : 0, lane, head[r][it], bpr, im);
                acc[r] += ok ? v : 0.0f;
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RW; ++r) {
        const float total = group_sum<64>(acc[r]);
        const int row = row0 + r;
        if (lane == 0 && row < n) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + row, total);
    }
}

// Any shape, any alignment: one wave per output row, one lane per block, byte loads.  Used when the
// rows are not 16-byte aligned streams (blocks_per_row not a multiple of 8, or an offset base).
__global__ __launch_bounds__(kThreads) void q8_0_generic_kernel(
    const void* __restrict__ x, int x_dtype, const uint8_t* __restrict__ w, void* __restrict__ y, int y_dtype,
    int k, int n, int bpr) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * kWaves + (threadIdx.x >> 6);
    const size_t xoff = static_cast<size_t>(blockIdx.y) * k;
    float acc = 0.0f;
    if (row < n) {
        const uint8_t* wrow = w + static_cast<size_t>(row) * bpr * 34;
        for (int b = lane; b < bpr; b += 64) {
            const uint8_t* blk = wrow + 34 * b;
            const float d = f16_bits_to_float(static_cast<uint32_t>(blk[0]) | (static_cast<uint32_t>(blk[1]) << 8));
            float s = 0.0f;
            for (int i = 0; i < 32; ++i) {
                const int e = 32 * b + i;
                if (e < k) s += load_any(x, x_dtype, xoff + e) * static_cast<float>(static_cast<int8_t>(blk[2 + i]));
            }
            acc += d * s;
        }
    }
    acc = group_sum<64>(acc);
    if (lane == 0 && row < n) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + row, acc);
}

template <int ITERS, int RW>
int launch_stream(const void* x, int x_dtype, const uint8_t* w, void* y, int y_dtype, int rows, int k, int n, int bpr,
                  hipStream_t stream) {
    const size_t smem = static_cast<size_t>(bpr) * 34 * 2 + static_cast<size_t>(bpr) * 4;
    auto kern = q8_0_stream_kernel<ITERS, RW>;
    if (smem > 64 * 1024) {
        if (smem > 160 * 1024) return PLLM_ERR_UNSUPPORTED;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(smem)) != hipSuccess)
            return PLLM_ERR_UNSUPPORTED;
    }
    const int rows_per_wg = kWaves * RW;
    dim3 grid((n + rows_per_wg - 1) / rows_per_wg, rows);
    hipLaunchKernelGGL(kern, grid, dim3(kThreads), smem, stream, x, x_dtype, w, y, y_dtype, k, n, bpr);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

template <int RW>
int launch_stream_rw(const void* x, int x_dtype, const uint8_t* w, void* y, int y_dtype, int rows, int k, int n, int bpr,
                     hipStream_t stream) {
    const int chunks = bpr * 34 / 16;
    const int niter = (chunks + 63) / 64;
    const int passes = (niter + 7) / 8;
    const int iters = (niter + passes - 1) / passes;
#define PLLM_CASE(I) return launch_stream<I, RW>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream)
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

int q8_0_matvec(const void* x, int x_dtype, const uint8_t* w, void* y, int y_dtype,
                int rows, int k, int n, int bpr, hipStream_t stream) {
    const bool stream_ok = (bpr % 8 == 0) && ((reinterpret_cast<uintptr_t>(w) & 15u) == 0);
    if (!stream_ok) {
        dim3 grid((n + kWaves - 1) / kWaves, rows);
        hipLaunchKernelGGL(q8_0_generic_kernel, grid, dim3(kThreads), 0, stream, x, x_dtype, w, y, y_dtype, k, n, bpr);
        return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
    }
    if (n >= 16384) return launch_stream_rw<4>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream);
    if (n >= 2048) return launch_stream_rw<2>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream);
    return launch_stream_rw<1>(x, x_dtype, w, y, y_dtype, rows, k, n, bpr, stream);
}

}  // namespace pllm
