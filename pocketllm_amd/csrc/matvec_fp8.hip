// Decode matvec over FP8 E4M3 (OCP) weights with float32 scales per 128 x 128 block.
//
// One byte per weight, rows contiguous: a wave reads a row as a stream, lane l taking 16 bytes at
// offset 16 * (l + 64 * it) with one global_load_dwordx4, two rows in flight per wave.  The
// activation row sits in LDS as float32 (no quantization on this path: y = x . (f32(code) * scale),
// the reference's dequantize-then-matmul statement).  Codes become floats with v_cvt_pk_f32_fp8,
// 16 FMAs per lane and chunk; a chunk lies inside one 128-wide scale block, so the block scale is
// applied once per chunk.  Row sums are 64-lane reductions.
#include "pllm_device.h"
#include "pllm_internal.h"
#include <algorithm>

namespace pllm {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kRowsPerWave = 2;

typedef float v2f __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float chunk_dot(const uint4& w, const float* xp) {
    const float4 x0 = *reinterpret_cast<const float4*>(xp);
    const float4 x1 = *reinterpret_cast<const float4*>(xp + 4);
    const float4 x2 = *reinterpret_cast<const float4*>(xp + 8);
    const float4 x3 = *reinterpret_cast<const float4*>(xp + 12);
    v2f a;
    float s;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.x), false); s = a.x * x0.x; s += a.y * x0.y;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.x), true);  s += a.x * x0.z; s += a.y * x0.w;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.y), false); s += a.x * x1.x; s += a.y * x1.y;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.y), true);  s += a.x * x1.z; s += a.y * x1.w;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.z), false); s += a.x * x2.x; s += a.y * x2.y;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.z), true);  s += a.x * x2.z; s += a.y * x2.w;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.w), false); s += a.x * x3.x; s += a.y * x3.y;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.w), true);  s += a.x * x3.z; s += a.y * x3.w;
    return s;
}

// k a multiple of 16, weight base 16-byte aligned
template <int ITERS>
__global__ __launch_bounds__(kThreads) void fp8_stream_matvec_kernel(
    const void* __restrict__ x, int x_dtype, const uint8_t* __restrict__ w, const float* __restrict__ scale,
    void* __restrict__ y, int y_dtype, int k, int n, int kb) {
    extern __shared__ __align__(16) unsigned char smem[];
    float* xs = reinterpret_cast<float*>(smem);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int chunks = k >> 4;
    const int row0 = (blockIdx.x * kWaves + wave) * kRowsPerWave;
    const size_t xoff = static_cast<size_t>(blockIdx.y) * k;

    float acc[kRowsPerWave];
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) acc[r] = 0.0f;

    bool staged = false;
    for (int c0 = 0; c0 < chunks; c0 += 64 * ITERS) {
        uint4 regs[kRowsPerWave][ITERS];
#pragma unroll
        for (int r = 0; r < kRowsPerWave; ++r) {
            const uint8_t* wrow = w + static_cast<size_t>(min(row0 + r, n - 1)) * k;
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int c = min(c0 + it * 64 + lane, chunks - 1);
                regs[r][it] = *reinterpret_cast<const uint4*>(wrow + 16 * c);
            }
        }
        if (!staged) {
            for (int i = tid; i < k; i += kThreads) xs[i] = load_any(x, x_dtype, xoff + i);
            __syncthreads();
            staged = true;
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int c = c0 + it * 64 + lane;
            const bool ok = c < chunks;
            const int cc = ok ? c : 0;
#pragma unroll
            for (int r = 0; r < kRowsPerWave; ++r) {
                const float s = chunk_dot(regs[r][it], xs + 16 * cc);
                const float sc = scale[(min(row0 + r, n - 1) >> 7) * kb + (cc >> 3)];
                acc[r] += ok ? s * sc : 0.0f;
            }
        }
    }
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        const float total = group_sum<64>(acc[r]);
        if (lane == 0 && row0 + r < n) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + row0 + r, total);
    }
}

// The same, persistent: the grid is sized to be resident at once, a workgroup stages the activation
// row once and then walks groups of 8 weight rows (two per wave), always holding the loads of its
// next group in a second register set while it multiplies the current one.  Rows of at most
// 64 * 16 * ITERS bytes.
template <int ITERS>
__device__ __forceinline__ void fp8_fetch_group(uint4 (&r)[kRowsPerWave][ITERS], const uint8_t* __restrict__ w, int row0, int n, int k, int chunks, int lane) {
#pragma unroll
    for (int q = 0; q < kRowsPerWave; ++q) {
        const uint8_t* wrow = w + static_cast<size_t>(min(row0 + q, n - 1)) * k;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) r[q][it] = *reinterpret_cast<const uint4*>(wrow + 16 * min(it * 64 + lane, chunks - 1));
    }
}

template <int ITERS>
__device__ __forceinline__ void fp8_finish_group(const uint4 (&r)[kRowsPerWave][ITERS], const float* xs, const float* __restrict__ scale,
                                                 void* __restrict__ y, int y_dtype, size_t yoff, int row0, int n, int kb, int chunks, int lane) {
    float acc[kRowsPerWave];
#pragma unroll
    for (int q = 0; q < kRowsPerWave; ++q) acc[q] = 0.0f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int c = it * 64 + lane;
        const bool ok = c < chunks;
        const int cc = ok ? c : 0;
#pragma unroll
        for (int q = 0; q < kRowsPerWave; ++q) {
            const float d = chunk_dot(r[q][it], xs + 16 * cc);
            const float sc = scale[(min(row0 + q, n - 1) >> 7) * kb + (cc >> 3)];
            acc[q] += ok ? d * sc : 0.0f;
        }
    }
#pragma unroll
    for (int q = 0; q < kRowsPerWave; ++q) {
        const float total = group_sum<64>(acc[q]);
        if (lane == 0 && row0 + q < n) store_any(y, y_dtype, yoff + row0 + q, total);
    }
}

template <int ITERS>
__global__ __launch_bounds__(kThreads) void fp8_persistent_matvec_kernel(
    const void* __restrict__ x, int x_dtype, const uint8_t* __restrict__ w, const float* __restrict__ scale,
    void* __restrict__ y, int y_dtype, int k, int n, int kb, int groups) {
    extern __shared__ __align__(16) unsigned char smem[];
    float* xs = reinterpret_cast<float*>(smem);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int chunks = k >> 4;
    const size_t xoff = static_cast<size_t>(blockIdx.y) * k;
    const size_t yoff = static_cast<size_t>(blockIdx.y) * n;
    const int rows_per_group = kWaves * kRowsPerWave, wave_row = wave * kRowsPerWave;

    uint4 a[kRowsPerWave][ITERS], b[kRowsPerWave][ITERS];
    int g = blockIdx.x;
    const int step = gridDim.x;
    fp8_fetch_group<ITERS>(a, w, g * rows_per_group + wave_row, n, k, chunks, lane);
    for (int i = tid; i < k; i += kThreads) xs[i] = load_any(x, x_dtype, xoff + i);
    __syncthreads();
    while (g < groups) {
        if (g + step < groups) fp8_fetch_group<ITERS>(b, w, (g + step) * rows_per_group + wave_row, n, k, chunks, lane);
        fp8_finish_group<ITERS>(a, xs, scale, y, y_dtype, yoff, g * rows_per_group + wave_row, n, kb, chunks, lane);
        g += step;
        if (g >= groups) break;
        if (g + step < groups) fp8_fetch_group<ITERS>(a, w, (g + step) * rows_per_group + wave_row, n, k, chunks, lane);
        fp8_finish_group<ITERS>(b, xs, scale, y, y_dtype, yoff, g * rows_per_group + wave_row, n, kb, chunks, lane);
        g += step;
    }
}

__device__ __forceinline__ float fp8_to_float_sw(uint32_t c) {
    const uint32_t e = (c >> 3) & 15u, m = c & 7u;
    float v;
    if (e == 0) v = static_cast<float>(m) * 0.001953125f;
    else if (e == 15 && m == 7) v = __uint_as_float(0x7fc00000u);
    else v = __uint_as_float(((e + 120u) << 23) | (m << 20));
    return (c & 0x80u) ? -v : v;
}

// any k, any alignment: one wave per row, byte loads
__global__ __launch_bounds__(kThreads) void fp8_generic_matvec_kernel(
    const void* __restrict__ x, int x_dtype, const uint8_t* __restrict__ w, const float* __restrict__ scale,
    void* __restrict__ y, int y_dtype, int k, int n, int kb) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * kWaves + (threadIdx.x >> 6);
    const size_t xoff = static_cast<size_t>(blockIdx.y) * k;
    float acc = 0.0f;
    if (row < n) {
        const uint8_t* wrow = w + static_cast<size_t>(row) * k;
        for (int c = lane; c < k; c += 64)
            acc += load_any(x, x_dtype, xoff + c) * (fp8_to_float_sw(wrow[c]) * scale[(row >> 7) * kb + (c >> 7)]);
    }
    acc = group_sum<64>(acc);
    if (lane == 0 && row < n) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + row, acc);
}

template <int ITERS>
int launch_stream(const void* x, int x_dtype, const uint8_t* w, const float* scale, void* y, int y_dtype,
                  int rows, int k, int n, hipStream_t stream) {
    const size_t smem = static_cast<size_t>(k) * sizeof(float);
    auto kern = fp8_stream_matvec_kernel<ITERS>;
    if (smem > 64 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(smem)) != hipSuccess)
            return PLLM_ERR_UNSUPPORTED;
    }
    const int rows_per_wg = kWaves * kRowsPerWave;
    dim3 grid((n + rows_per_wg - 1) / rows_per_wg, rows);
    hipLaunchKernelGGL(kern, grid, dim3(kThreads), smem, stream, x, x_dtype, w, scale, y, y_dtype, k, n, (k + 127) / 128);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

}  // namespace

int fp8_matvec(const void* x, int x_dtype, const uint8_t* w, const float* scale, void* y, int y_dtype,
               int rows, int k, int n, hipStream_t stream) {
    const bool stream_ok = (k % 16 == 0) && ((reinterpret_cast<uintptr_t>(w) & 15u) == 0) && (static_cast<size_t>(k) * 4 <= 160 * 1024);
    if (!stream_ok) {
        dim3 grid((n + kWaves - 1) / kWaves, rows);
        hipLaunchKernelGGL(fp8_generic_matvec_kernel, grid, dim3(kThreads), 0, stream, x, x_dtype, w, scale, y, y_dtype, k, n,
                           (k + 127) / 128);
        return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
    }
    const int niter = ((k >> 4) + 63) / 64;
    if (niter <= 6) {
        const int groups = (n + kWaves * kRowsPerWave - 1) / (kWaves * kRowsPerWave);
        const int grid_x = std::min(groups, 2 * compute_units());   // two resident workgroups per compute unit (register-bound), groups dealt round-robin
        const size_t smem = static_cast<size_t>(k) * sizeof(float);
#define PLLM_PCASE(I) case I: hipLaunchKernelGGL(fp8_persistent_matvec_kernel<I>, dim3(grid_x, rows), dim3(kThreads), smem, stream, x, x_dtype, w, scale, y, y_dtype, k, n, (k + 127) / 128, groups); break
        switch (niter) {
            PLLM_PCASE(1); PLLM_PCASE(2); PLLM_PCASE(3); PLLM_PCASE(4); PLLM_PCASE(5);
            default: hipLaunchKernelGGL(fp8_persistent_matvec_kernel<6>, dim3(grid_x, rows), dim3(kThreads), smem, stream, x, x_dtype, w, scale, y, y_dtype, k, n, (k + 127) / 128, groups); break;
        }
#undef PLLM_PCASE
        return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
    }
    const int passes = (niter + 5) / 6;
    const int iters = (niter + passes - 1) / passes;
#define PLLM_CASE(I) case I: return launch_stream<I>(x, x_dtype, w, scale, y, y_dtype, rows, k, n, stream)
    switch (iters) {
        PLLM_CASE(1); PLLM_CASE(2); PLLM_CASE(3); PLLM_CASE(4); PLLM_CASE(5);
        default: return launch_stream<6>(x, x_dtype, w, scale, y, y_dtype, rows, k, n, stream);
    }
#undef PLLM_CASE
}

}  // namespace pllm
