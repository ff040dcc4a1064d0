// Activation pre-quantization: float / fp16 / bf16 rows -> int8 "images" the matvec kernels copy
// into LDS (layouts in pllm_device.h and matvec_q8_0.hip).  One thread quantizes four values; the
// eight threads of an aligned group share a 32-value block (amax by cross-lane max).
#include "pllm_device.h"
#include "pllm_internal.h"

namespace pllm {
namespace {

constexpr int kThreads = 256;

__global__ __launch_bounds__(kThreads) void act_image_256_kernel(
    const void* __restrict__ x, int x_dtype, unsigned char* __restrict__ image, int k, int kpad, size_t image_stride) {
    const int e0 = (blockIdx.x * kThreads + threadIdx.x) * 4;
    if (e0 >= kpad) return;                                   // kpad is a multiple of 256: whole groups leave together
    const size_t xoff = static_cast<size_t>(blockIdx.y) * k;
    unsigned char* base = image + static_cast<size_t>(blockIdx.y) * image_stride;
    int8_t* hi = reinterpret_cast<int8_t*>(base);
    int8_t* lo = hi + kpad;
    float2* gs = reinterpret_cast<float2*>(lo + kpad);
    float* sum16 = reinterpret_cast<float*>(gs + kpad / 32);
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = (e0 + i < k) ? load_any(x, x_dtype, xoff + e0 + i) : 0.0f;
    quantize4_to_image(v, e0, hi, lo, gs, sum16);
}

// The image of h = SiLU(g) * u (g capped at L from above and u clamped to +-L when L > 0), optionally rounded through a 16-bit
// type first, as the two-operator chain "activation in the model's dtype, then the down projection" rounds it.
__global__ __launch_bounds__(kThreads) void swiglu_image_256_kernel(
    const void* __restrict__ gate, const void* __restrict__ up, int gu_dtype, float limit, int round_dtype,
    unsigned char* __restrict__ image, int k, int kpad, size_t image_stride) {
    const int e0 = (blockIdx.x * kThreads + threadIdx.x) * 4;
    if (e0 >= kpad) return;
    const size_t xoff = static_cast<size_t>(blockIdx.y) * k;
    unsigned char* base = image + static_cast<size_t>(blockIdx.y) * image_stride;
    int8_t* hi = reinterpret_cast<int8_t*>(base);
    int8_t* lo = hi + kpad;
    float2* gs = reinterpret_cast<float2*>(lo + kpad);
    float* sum16 = reinterpret_cast<float*>(gs + kpad / 32);
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float h = 0.0f;
        if (e0 + i < k) {
            float g = load_any(gate, gu_dtype, xoff + e0 + i), u = load_any(up, gu_dtype, xoff + e0 + i);
            if (limit > 0.0f) {
                u = fminf(fmaxf(u, -limit), limit);
                g = fminf(g, limit);
            }
            h = g / (1.0f + expf(-g)) * u;
            if (round_dtype == PLLM_F16) h = to_float(from_float<f16_t>(h));
            else if (round_dtype == PLLM_BF16) h = to_float(from_float<bf16_t>(h));
        }
        v[i] = h;
    }
    quantize4_to_image(v, e0, hi, lo, gs, sum16);
}

// Q8_0 pair image: per pair of 32-value blocks 80 bytes that mirror the weight stream,
//   [0,0, q0..q31, 0,0, q32..q63, 12 x 0],  then after all pairs: float xs[2 * pairs].
__global__ __launch_bounds__(kThreads) void act_image_q8pair_kernel(
    const void* __restrict__ x, int x_dtype, unsigned char* __restrict__ image, int k, int pairs, size_t image_stride) {
    const int e0 = (blockIdx.x * kThreads + threadIdx.x) * 4;
    if (e0 >= pairs * 64) return;
    const size_t xoff = static_cast<size_t>(blockIdx.y) * k;
    unsigned char* base = image + static_cast<size_t>(blockIdx.y) * image_stride;
    unsigned char* hi = base;
    unsigned char* lo = base + static_cast<size_t>(pairs) * 80;
    float* xs = reinterpret_cast<float*>(lo + static_cast<size_t>(pairs) * 80);
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = (e0 + i < k) ? load_any(x, x_dtype, xoff + e0 + i) : 0.0f;
    quantize4_to_pair_image(v, e0, hi, lo, xs);
}

// RMS normalisation of rows: one workgroup per row.  Rows of up to 4 x kRmsHeld x kThreads values are read once, four values per
// lane and trip with all trips' loads in flight together, and kept in registers for the scaling (a loop of dependent scalar
// loads costs a cache round trip per trip: 10 us for a row of 3072); wider rows are read twice.
constexpr int kRmsHeld = 4;
__global__ __launch_bounds__(kThreads) void rms_norm_rows_kernel(
    const void* __restrict__ x, int x_dtype, const float* __restrict__ weight, void* __restrict__ y, int y_dtype, int dim, float eps) {
    __shared__ float red[kThreads / 64];
    const size_t off = static_cast<size_t>(blockIdx.x) * dim;
    const bool held = dim <= 4 * kRmsHeld * kThreads;
    const bool vec = (dim % 4 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15u) == 0);
    const bool wvec = (dim % 4 == 0) && ((reinterpret_cast<uintptr_t>(weight) & 15u) == 0);
    float v[kRmsHeld][4], g[kRmsHeld][4];
    float ss = 0.0f;
    if (held) {
        int e0[kRmsHeld];                                                   // beyond the row: its first piece again, not counted
#pragma unroll
        for (int j = 0; j < kRmsHeld; ++j) e0[j] = 4 * (static_cast<int>(threadIdx.x) + kThreads * j) < dim ? 4 * (static_cast<int>(threadIdx.x) + kThreads * j) : 0;
        // (the weights are requested first: the row's loads sit behind a branch on its type, and what is requested after that
        // branch, or after the barrier, costs a round trip of its own)
#pragma unroll
        for (int j = 0; j < kRmsHeld; ++j) load_row4(g[j], weight, PLLM_F32, 0, e0[j], dim, wvec);
        if (vec) {
            load_rows4_batch(v, x, x_dtype, off, e0);
        } else {
#pragma unroll
            for (int j = 0; j < kRmsHeld; ++j) load_row4(v[j], x, x_dtype, off, e0[j], dim, false);
        }
#pragma unroll
        for (int j = 0; j < kRmsHeld; ++j)
            if (4 * (threadIdx.x + kThreads * j) < dim) ss += (v[j][0] * v[j][0] + v[j][1] * v[j][1]) + (v[j][2] * v[j][2] + v[j][3] * v[j][3]);
    } else {
        for (int i = threadIdx.x; i < dim; i += kThreads) {
            const float w = load_any(x, x_dtype, off + i);
            ss += w * w;
        }
    }
    ss = group_sum<64>(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < kThreads / 64; ++w) total += red[w];
    const float rstd = rsqrtf(total / static_cast<float>(dim) + eps);
    if (held) {
#pragma unroll
        for (int j = 0; j < kRmsHeld; ++j) {
            const int e0 = 4 * (threadIdx.x + kThreads * j);
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (e0 + i < dim) store_any(y, y_dtype, off + e0 + i, v[j][i] * rstd * g[j][i]);
        }
    } else {
        for (int i = threadIdx.x; i < dim; i += kThreads) store_any(y, y_dtype, off + i, load_any(x, x_dtype, off + i) * rstd * weight[i]);
    }
}

}  // namespace

int rms_norm_rows(const void* x, int x_dtype, const float* weight, void* y, int y_dtype, int rows, int dim, float eps, hipStream_t stream) {
    hipLaunchKernelGGL(rms_norm_rows_kernel, dim3(rows), dim3(kThreads), 0, stream, x, x_dtype, weight, y, y_dtype, dim, eps);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

size_t act_image_256_bytes(int bpr) { return (staged_x_bytes(bpr * 256) + 255) & ~static_cast<size_t>(255); }

int act_image_256(const void* x, int x_dtype, int rows, int k, int bpr, void* image, hipStream_t stream) {
    const int kpad = bpr * 256;
    dim3 grid((kpad / 4 + kThreads - 1) / kThreads, rows);
    hipLaunchKernelGGL(act_image_256_kernel, grid, dim3(kThreads), 0, stream, x, x_dtype,
                       static_cast<unsigned char*>(image), k, kpad, act_image_256_bytes(bpr));
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

int swiglu_image_256(const void* gate, const void* up, int gu_dtype, float limit, int round_dtype, int rows, int k, int bpr, void* image,
                     hipStream_t stream) {
    const int kpad = bpr * 256;
    dim3 grid((kpad / 4 + kThreads - 1) / kThreads, rows);
    hipLaunchKernelGGL(swiglu_image_256_kernel, grid, dim3(kThreads), 0, stream, gate, up, gu_dtype, limit, round_dtype,
                       static_cast<unsigned char*>(image), k, kpad, act_image_256_bytes(bpr));
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

size_t act_image_q8pair_bytes(int pairs) {
    return (static_cast<size_t>(pairs) * 160 + static_cast<size_t>(pairs) * 8 + 255) & ~static_cast<size_t>(255);
}

int act_image_q8pair(const void* x, int x_dtype, int rows, int k, int pairs, void* image, hipStream_t stream) {
    dim3 grid((pairs * 16 + kThreads - 1) / kThreads, rows);
    hipLaunchKernelGGL(act_image_q8pair_kernel, grid, dim3(kThreads), 0, stream, x, x_dtype,
                       static_cast<unsigned char*>(image), k, pairs, act_image_q8pair_bytes(pairs));
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

}  // namespace pllm
