// Device-side helpers shared by the raw-block kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/pllm_hip.h"

namespace pllm {

// ---- scalar conversions -------------------------------------------------------------------
struct bf16_t { uint16_t bits; };
struct f16_t { _Float16 v; };

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return __uint_as_float(static_cast<uint32_t>(v.bits) << 16); }
__device__ __forceinline__ float to_float(f16_t v) { return static_cast<float>(v.v); }

__device__ __forceinline__ float f16_bits_to_float(uint32_t bits) {
    union { uint16_t u; _Float16 h; } c;
    c.u = static_cast<uint16_t>(bits);
    return static_cast<float>(c.h);
}

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ f16_t from_float<f16_t>(float v) { f16_t r; r.v = static_cast<_Float16>(v); return r; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float v) {
    // round to nearest even; NaN stays NaN
    uint32_t u = __float_as_uint(v);
    bf16_t r;
    if ((u & 0x7fffffffu) > 0x7f800000u) { r.bits = static_cast<uint16_t>((u >> 16) | 0x40u); return r; }
    u += 0x7fffu + ((u >> 16) & 1u);
    r.bits = static_cast<uint16_t>(u >> 16);
    return r;
}

// ---- integer dot and cross-lane ------------------------------------------------------------
__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4(static_cast<int>(a), static_cast<int>(b), c, false);
}

// Sum over aligned groups of WIDTH lanes (WIDTH a power of two <= 64); every lane gets the total.
template <int WIDTH>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
    for (int off = 1; off < WIDTH; off <<= 1) v += __shfl_xor(v, off, 64);
    return v;
}
template <int WIDTH>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
    for (int off = 1; off < WIDTH; off <<= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// ---- activation images ----------------------------------------------------------------------
// Activations reach the matvec kernels pre-quantized, as an "image" a tiny kernel writes once per
// call and every workgroup copies into LDS.  Per 32 values two int8 terms are kept,
//     x[i] ~= xs[g] * (hi[i] + lo[i] / 254),   xs[g] = amax_g / 127,
// so that integer dot products against the weight codes carry ~15 bits of each activation, enough
// to stay far below 1e-3 relative error against float activations.  sum16[] holds the exact float
// sum of every 16 activations for the "minus dmin * m" terms of the K-quants.
//
// Layout of one row's image for 256-weight super-block types (kpad = blocks_per_row * 256):
//     int8 hi[kpad] | int8 lo[kpad] | float2 gs[kpad / 32] | float sum16[kpad / 16]
// with gs[g] = { xs[g] / 254, exact float sum of the 32 activations of group g }, so that
// xs * (hi + lo / 254) dotted with integer codes is gs.x * (254 * dot_hi + dot_lo).
constexpr float kLoInv = 1.0f / 254.0f;

struct StagedX {
    const int8_t* hi;
    const int8_t* lo;
    const float2* gs;
    const float* sum16;
};

__host__ __device__ inline size_t staged_x_bytes(int kpad) {
    return static_cast<size_t>(kpad) * 2 + static_cast<size_t>(kpad / 32) * 8 + static_cast<size_t>(kpad / 16) * 4;
}

__device__ __forceinline__ StagedX carve_staged_x(const unsigned char* base, int kpad) {
    StagedX s;
    s.hi = reinterpret_cast<const int8_t*>(base);
    s.lo = s.hi + kpad;
    s.gs = reinterpret_cast<const float2*>(s.lo + kpad);
    s.sum16 = reinterpret_cast<const float*>(s.gs + kpad / 32);
    return s;
}

// Quantize four activations of one lane; the eight lanes of an aligned group share a 32-block.
__device__ __forceinline__ void quantize4(const float v[4], uint32_t& hi, uint32_t& lo, float& scale) {
    float am = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
    am = group_max<8>(am);
    const float inv = am > 0.0f ? 127.0f / am : 0.0f;
    scale = am * (1.0f / 127.0f);
    hi = 0; lo = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float q = fminf(fmaxf(rintf(v[i] * inv), -127.0f), 127.0f);
        float r = v[i] - q * scale;
        float l = fminf(fmaxf(rintf(r * inv * 254.0f), -127.0f), 127.0f);
        hi |= (static_cast<uint32_t>(static_cast<int>(q)) & 0xffu) << (8 * i);
        lo |= (static_cast<uint32_t>(static_cast<int>(l)) & 0xffu) << (8 * i);
    }
}

// Runtime-dtype front ends (the dtype is uniform, so the switch costs one scalar branch).
__device__ __forceinline__ float load_any(const void* x, int x_dtype, size_t i) {
    if (x_dtype == PLLM_BF16) return to_float(static_cast<const bf16_t*>(x)[i]);
    if (x_dtype == PLLM_F16) return to_float(static_cast<const f16_t*>(x)[i]);
    return static_cast<const float*>(x)[i];
}

__device__ __forceinline__ void store_any(void* y, int y_dtype, size_t i, float v) {
    if (y_dtype == PLLM_BF16) static_cast<bf16_t*>(y)[i] = from_float<bf16_t>(v);
    else if (y_dtype == PLLM_F16) static_cast<f16_t*>(y)[i] = from_float<f16_t>(v);
    else static_cast<float*>(y)[i] = v;
}

// Workgroup-wide quantization of one activation row straight into LDS, the same image the
// pre-pass kernel writes to memory (blockDim.x a multiple of 8, kpad a multiple of 256).  Four
// consecutive values per lane: one 8-byte load for 16-bit inputs when the row allows it.
__device__ __forceinline__ void quantize_row_to_lds(unsigned char* lds, const void* __restrict__ x, int x_dtype, size_t xoff, int k, int kpad) {
    int8_t* hi = reinterpret_cast<int8_t*>(lds);
    int8_t* lo = hi + kpad;
    float2* gs = reinterpret_cast<float2*>(lo + kpad);
    float* sum16 = reinterpret_cast<float*>(gs + kpad / 32);
    const bool narrow = x_dtype != PLLM_F32 && ((reinterpret_cast<uintptr_t>(x) + 2 * xoff) & 7u) == 0;
    for (int e0 = static_cast<int>(threadIdx.x) * 4; e0 < kpad; e0 += static_cast<int>(blockDim.x) * 4) {
        float v[4];
        if (narrow && e0 + 3 < k) {
            const uint2 w = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(x) + xoff + e0);
            if (x_dtype == PLLM_BF16) {
                v[0] = __uint_as_float(w.x << 16); v[1] = __uint_as_float(w.x & 0xffff0000u);
                v[2] = __uint_as_float(w.y << 16); v[3] = __uint_as_float(w.y & 0xffff0000u);
            } else {
                v[0] = f16_bits_to_float(w.x & 0xffffu); v[1] = f16_bits_to_float(w.x >> 16);
                v[2] = f16_bits_to_float(w.y & 0xffffu); v[3] = f16_bits_to_float(w.y >> 16);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = (e0 + i < k) ? load_any(x, x_dtype, xoff + e0 + i) : 0.0f;
        }
        uint32_t qh, ql;
        float scale;
        quantize4(v, qh, ql, scale);
        *reinterpret_cast<uint32_t*>(hi + e0) = qh;
        *reinterpret_cast<uint32_t*>(lo + e0) = ql;
        const float sum = group_sum<4>((v[0] + v[1]) + (v[2] + v[3]));
        const float sum32 = sum + __shfl_xor(sum, 4, 64);
        if ((threadIdx.x & 3) == 0) sum16[e0 >> 4] = sum;
        if ((threadIdx.x & 7) == 0) gs[e0 >> 5] = make_float2(scale * kLoInv, sum32);
    }
}

// Workgroup-wide copy of nbytes (a multiple of 16, both pointers 16-byte aligned) into LDS.
__device__ __forceinline__ void copy_to_lds(unsigned char* dst, const unsigned char* __restrict__ src, int nbytes) {
    const uint4* s = reinterpret_cast<const uint4*>(src);
    uint4* d = reinterpret_cast<uint4*>(dst);
    for (int i = threadIdx.x; i < (nbytes >> 4); i += blockDim.x) d[i] = s[i];
}

}  // namespace pllm
