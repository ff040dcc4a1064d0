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

// One step of a butterfly reduction without the LDS crossbar: the value lane (id ^ OFF) holds,
// for a v that is already equal over aligned groups of OFF lanes (which is what step OFF of a
// butterfly sees).  Steps 1 and 2 swap inside the quad, 4 and 8 mirror the half row / the row,
// which pairs each group with its partner group; wider steps go through ds_bpermute.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
template <int OFF>
__device__ __forceinline__ float butterfly_peer(float v) {
    if constexpr (OFF == 1) return dpp_move<0xB1>(v);            // quad_perm:[1,0,3,2]
    else if constexpr (OFF == 2) return dpp_move<0x4E>(v);       // quad_perm:[2,3,0,1]
    else if constexpr (OFF == 4) return dpp_move<0x141>(v);      // row_half_mirror
    else if constexpr (OFF == 8) return dpp_move<0x140>(v);      // row_mirror
    else return __shfl_xor(v, OFF, 64);
}

// v summed over the four lanes (l % 16) + {0, 16, 32, 48}, in every lane: the two wide steps of a butterfly (lane ^ 16, then
// lane ^ 32, the order and therefore the bits of the shuffle form) through gfx950's row swaps: v_permlane16_swap exchanges the odd
// rows of one operand with the even rows of the other, v_permlane32_swap the upper half with the lower half; one vector
// instruction each and no LDS crossbar.
__device__ __forceinline__ float quad_rows_sum(float v) {
    const uint32_t b = __float_as_uint(v);
    const auto h = __builtin_amdgcn_permlane16_swap(b, b, false, false);      // {rows 0 0 2 2, rows 1 1 3 3}
    const uint32_t s = __float_as_uint(__uint_as_float(h[0]) + __uint_as_float(h[1]));
    const auto r = __builtin_amdgcn_permlane32_swap(s, s, false, false);      // {lower half twice, upper half twice}
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Sum / maximum over aligned groups of WIDTH lanes (WIDTH a power of two <= 64); every lane gets the result.
// the wide steps (lane ^ 16, lane ^ 32) of a commutative reduction through the row swaps: both halves of the swapped pair hold
// the two values every lane needs, in one order or the other
template <int OFF>
__device__ __forceinline__ void swapped_pair(float v, float& a, float& b) {
    const uint32_t bits = __float_as_uint(v);
    if constexpr (OFF == 16) {
        const auto h = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
        a = __uint_as_float(h[0]); b = __uint_as_float(h[1]);
    } else {
        const auto h = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
        a = __uint_as_float(h[0]); b = __uint_as_float(h[1]);
    }
}
template <int WIDTH>
__device__ __forceinline__ float group_sum(float v) {
    if constexpr (WIDTH > 1) v += butterfly_peer<1>(v);
    if constexpr (WIDTH > 2) v += butterfly_peer<2>(v);
    if constexpr (WIDTH > 4) v += butterfly_peer<4>(v);
    if constexpr (WIDTH > 8) v += butterfly_peer<8>(v);
    float a, b;
    if constexpr (WIDTH > 16) { swapped_pair<16>(v, a, b); v = a + b; }
    if constexpr (WIDTH > 32) { swapped_pair<32>(v, a, b); v = a + b; }
    return v;
}
template <int WIDTH>
__device__ __forceinline__ float group_max(float v) {
    if constexpr (WIDTH > 1) v = fmaxf(v, butterfly_peer<1>(v));
    if constexpr (WIDTH > 2) v = fmaxf(v, butterfly_peer<2>(v));
    if constexpr (WIDTH > 4) v = fmaxf(v, butterfly_peer<4>(v));
    if constexpr (WIDTH > 8) v = fmaxf(v, butterfly_peer<8>(v));
    float a, b;
    if constexpr (WIDTH > 16) { swapped_pair<16>(v, a, b); v = fmaxf(a, b); }
    if constexpr (WIDTH > 32) { swapped_pair<32>(v, a, b); v = fmaxf(a, b); }
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

__host__ __device__ constexpr size_t staged_x_bytes(int kpad) {
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
// First term: q = rint(fl(v / scale)) with scale = fl(amax / 127), the correctly rounded float32 quotient rounded to the nearest
// even integer, which is the reference's 32-value activation quantizer (src/csrc/cuda_kernel_impl.cu:7102-7116) bit for bit;
// |v / scale| <= 127 * (1 + 2^-23), so the clamp of the reference never acts.  Second term: the residual v - q * scale in
// units of scale / 254 (|r / scale * 254| <= 127.01 by construction, no clamp either).  An all-zero group stores scale 0, codes 0.
//
// How the quotients stay exact without four IEEE divisions per lane:
//   * scale: q0 = amax * c, scale = fma(fma(-q0, 127, amax), c, q0) with c = fl(1 / 127) is the correctly rounded amax / 127
//     for every finite float32 (checked exhaustively on the host, tests/test_quantizer_identities.py).
//   * codes: q = rint(v * y) with y ~= 1 / scale from v_rcp_f32 can differ from rint(fl(v / scale)) only when v / scale lies
//     within 127 * 2^-21 of a rounding tie.  The residual r = fma(-q, scale, v), which the second term needs anyway, shows it:
//     |r| < scale * (0.5 - 1e-4) proves q right whatever y was.  If any lane of the wave fails that test (about one
//     32-block in a hundred), or amax is so small that the products above could leave the normal range, the whole wave
//     redoes its four codes with true divisions.
// The rounding and the int8 cast ride on one addition: for |t| < 2^22 the float t + 1.5 * 2^23 has round-to-nearest-even(t)
// in its low mantissa bits, two's complement included, so its low byte is the code and (sum - 1.5 * 2^23) the rounded value.
__device__ __forceinline__ uint32_t pack_low_bytes(uint32_t b0, uint32_t b1, uint32_t b2, uint32_t b3) {
    const uint32_t lo = __builtin_amdgcn_perm(b1, b0, 0x0c0c0400u);
    const uint32_t hi = __builtin_amdgcn_perm(b3, b2, 0x0c0c0400u);
    return __builtin_amdgcn_perm(hi, lo, 0x05040100u);
}
__device__ __forceinline__ void quantize4(const float v[4], uint32_t& hi, uint32_t& lo, float& scale) {
    constexpr float kRound = 12582912.0f;                       // 1.5 * 2^23
    constexpr float kInv127 = 1.0f / 127.0f;
    float am = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
    am = group_max<8>(am);
    const float s0 = am * kInv127;
    scale = __builtin_fmaf(__builtin_fmaf(-s0, 127.0f, am), kInv127, s0);
    const bool normal = am > 1e-30f && am < 1e30f;
    const float y = normal ? __builtin_amdgcn_rcpf(scale) : 0.0f;
    const float thr = scale * (0.5f - 1e-4f);
    float qm[4], r[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        qm[i] = __builtin_fmaf(v[i], y, kRound);
        r[i] = __builtin_fmaf(kRound - qm[i], scale, v[i]);     // v - q * scale
    }
    // one comparison on the largest residual (a NaN among the values has the same code either way and drops out of the maximum)
    const bool sure = normal && fmaxf(fmaxf(fabsf(r[0]), fabsf(r[1])), fmaxf(fabsf(r[2]), fabsf(r[3]))) < thr;
    if (__builtin_amdgcn_ballot_w64(am > 0.0f && !sure) != 0) {  // wave-uniform: a quotient next to a rounding tie, or an extreme amax
        scale = am / 127.0f;
        const float divisor = am > 0.0f ? scale : 1.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            qm[i] = v[i] / divisor + kRound;
            r[i] = __builtin_fmaf(kRound - qm[i], scale, v[i]);
        }
    }
    const float inv_lo = am > 0.0f ? (127.0f * 254.0f) * __builtin_amdgcn_rcpf(am) : 0.0f;
    uint32_t qb[4], lb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        qb[i] = __float_as_uint(qm[i]);
        lb[i] = __float_as_uint(__builtin_fmaf(r[i], inv_lo, kRound));
    }
    hi = pack_low_bytes(qb[0], qb[1], qb[2], qb[3]);
    lo = pack_low_bytes(lb[0], lb[1], lb[2], lb[3]);
}

// The same two-term image on a power-of-two scale, for kernels that quantize a slice per wave and block and cannot afford the
// exact quotients above: x ~= xs * (256 * hi + lo) with xs = 2^(E - 13), E the exponent of the group's largest magnitude, so that
// |x / xs| < 2^14, hi in [-64, 64], lo in [-128, 127].  No division and no tie test: x / xs is an exponent shift, exact for every
// value whose lowest mantissa bit is worth xs or more (all bf16 values within 2^-6 of the group's largest; fp16 within 2^-3);
// smaller values round to the nearest multiple of xs (error <= amax * 2^-15).  One fused multiply-add with 1.5 * 2^23 + 128
// rounds to nearest even and leaves (q + 128) in the low mantissa bits: byte 1 is hi, byte 0 is lo with its top bit flipped.
// image_sum: the sum of the four values as the image holds them (exact).  The K-quants' offset terms (- dmin m sum(x), Q6_K's
// - 32 sum(x)) cancel most of the dot of the unsigned codes; taken from the image the two carry the same rounding and the result
// is the weights applied to the rounded activations, with the unrounded sums the rounding error is amplified by that cancellation.
__device__ __forceinline__ void quantize4_pow2(const float v[4], uint32_t& hi, uint32_t& lo, float& xs, float* image_sum) {
    constexpr float kRound = 12582912.0f + 128.0f;
    float am = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
    am = group_max<8>(am);
    const uint32_t e = max(__float_as_uint(am) >> 23, 14u);     // groups below 2^-113 quantize to zeros
    const float mult = __uint_as_float((267u - e) << 23);       // 2^(13 - (e - 127))
    xs = __uint_as_float((e - 13u) << 23);
    uint32_t t[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) t[i] = __float_as_uint(__builtin_fmaf(v[i], mult, kRound));
    const uint32_t w01 = __builtin_amdgcn_perm(t[1], t[0], 0x05010400u);   // lo0 lo1 hi0 hi1
    const uint32_t w23 = __builtin_amdgcn_perm(t[3], t[2], 0x05010400u);
    lo = __builtin_amdgcn_perm(w23, w01, 0x05040100u) ^ 0x80808080u;
    hi = __builtin_amdgcn_perm(w23, w01, 0x07060302u);
    *image_sum = xs * (((__uint_as_float(t[0]) - kRound) + (__uint_as_float(t[1]) - kRound)) + ((__uint_as_float(t[2]) - kRound) + (__uint_as_float(t[3]) - kRound)));
}

// Runtime-dtype front ends (the dtype is uniform, so the switch costs one scalar branch).
__device__ __forceinline__ float load_any(const void* x, int x_dtype, size_t i) {
    if (x_dtype == PLLM_BF16) return to_float(static_cast<const bf16_t*>(x)[i]);
    if (x_dtype == PLLM_F16) return to_float(static_cast<const f16_t*>(x)[i]);
    return static_cast<const float*>(x)[i];
}

// Output element i.  With bit 0x100 (kAccumulateInto of pllm_internal.h) set in y_dtype the value is added to what y holds
// (in float32, rounded once): the residual connection y += W x of the operators that state it.
__device__ __forceinline__ void store_any(void* y, int y_dtype, size_t i, float v) {
    if (y_dtype & 0x100) {
        y_dtype &= ~0x100;
        v += load_any(y, y_dtype, i);
    }
    if (y_dtype == PLLM_BF16) static_cast<bf16_t*>(y)[i] = from_float<bf16_t>(v);
    else if (y_dtype == PLLM_F16) static_cast<f16_t*>(y)[i] = from_float<f16_t>(v);
    else static_cast<float*>(y)[i] = v;
}

// the same for callers that never accumulate (y_dtype is one of the three plain codes)
__device__ __forceinline__ void store_plain(void* y, int y_dtype, size_t i, float v) {
    if (y_dtype == PLLM_BF16) static_cast<bf16_t*>(y)[i] = from_float<bf16_t>(v);
    else if (y_dtype == PLLM_F16) static_cast<f16_t*>(y)[i] = from_float<f16_t>(v);
    else static_cast<float*>(y)[i] = v;
}

// Workgroup-wide quantization of one activation row straight into LDS, the same image the
// pre-pass kernel writes to memory (blockDim.x a multiple of 8, kpad a multiple of 256).  Four
// consecutive values per lane and trip, fetched by one vector load when the row's alignment allows it.
// The loads of BATCH trips are issued together so that a row costs one or two memory round trips.
__device__ __forceinline__ void load_row4(float v[4], const void* __restrict__ x, int x_dtype, size_t xoff, int e0, int k, bool vec) {
    if (vec && e0 + 3 < k && x_dtype == PLLM_F32) {
        const float4 w = *reinterpret_cast<const float4*>(static_cast<const float*>(x) + xoff + e0);
        v[0] = w.x; v[1] = w.y; v[2] = w.z; v[3] = w.w;
    } else if (vec && e0 + 3 < k) {
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
}

// N pieces of four consecutive values (piece j at element e0[j], whole and 8- / 16-byte aligned: the caller checks), all loads in
// flight together.  The type is told apart once around the batch: a branch per piece would end every load in a wait of its own.
template <int N>
__device__ __forceinline__ void load_rows4_batch(float (&v)[N][4], const void* __restrict__ x, int x_dtype, size_t xoff, const int (&e0)[N]) {
    if (x_dtype == PLLM_F32) {
        float4 w[N];
#pragma unroll
        for (int j = 0; j < N; ++j) w[j] = *reinterpret_cast<const float4*>(static_cast<const float*>(x) + xoff + e0[j]);
#pragma unroll
        for (int j = 0; j < N; ++j) { v[j][0] = w[j].x; v[j][1] = w[j].y; v[j][2] = w[j].z; v[j][3] = w[j].w; }
    } else {
        uint2 w[N];
#pragma unroll
        for (int j = 0; j < N; ++j) w[j] = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(x) + xoff + e0[j]);
        if (x_dtype == PLLM_BF16) {
#pragma unroll
            for (int j = 0; j < N; ++j) {
                v[j][0] = __uint_as_float(w[j].x << 16); v[j][1] = __uint_as_float(w[j].x & 0xffff0000u);
                v[j][2] = __uint_as_float(w[j].y << 16); v[j][3] = __uint_as_float(w[j].y & 0xffff0000u);
            }
        } else {
#pragma unroll
            for (int j = 0; j < N; ++j) {
                v[j][0] = f16_bits_to_float(w[j].x & 0xffffu); v[j][1] = f16_bits_to_float(w[j].x >> 16);
                v[j][2] = f16_bits_to_float(w[j].y & 0xffffu); v[j][3] = f16_bits_to_float(w[j].y >> 16);
            }
        }
    }
}

// One lane's four values into the image at e0 (hi, lo, and the group figures from the lanes that own them).
__device__ __forceinline__ void quantize4_to_image(const float v[4], int e0, int8_t* hi, int8_t* lo, float2* gs, float* sum16) {
    uint32_t qh, ql;
    float scale;
    quantize4(v, qh, ql, scale);
    *reinterpret_cast<uint32_t*>(hi + e0) = qh;
    *reinterpret_cast<uint32_t*>(lo + e0) = ql;
    const float sum = group_sum<4>((v[0] + v[1]) + (v[2] + v[3]));
    const float sum32 = sum + butterfly_peer<4>(sum);
    if ((threadIdx.x & 3) == 0) sum16[e0 >> 4] = sum;
    if ((threadIdx.x & 7) == 0) gs[e0 >> 5] = make_float2(scale * kLoInv, sum32);
}

// Optional RMS normalisation ahead of the quantization: v = x * rsqrt(mean(x^2) + eps) * gamma, optionally rounded through fp16
// (what a separate normalisation kernel with an fp16 output would hand over).  gamma == nullptr: none.
struct RowNorm {
    const float* gamma;
    float eps;
    int round_f16;
};

// BATCH pieces of four values at base, base + trip, ... of a row of k values padded to kpad (zeros beyond k, pieces beyond kpad
// untouched): one batch of vector loads when all pieces lie inside the row, piece by piece otherwise (the row's last trips,
// rows that do not start on a vector boundary).
template <int BATCH>
__device__ __forceinline__ void load_row_pieces(float (&v)[BATCH][4], const void* __restrict__ x, int x_dtype, size_t xoff, int base, int trip, int k,
                                                int kpad, bool vec) {
    if (vec && base + (BATCH - 1) * trip + 3 < k) {
        int e0[BATCH];
#pragma unroll
        for (int j = 0; j < BATCH; ++j) e0[j] = base + j * trip;
        load_rows4_batch(v, x, x_dtype, xoff, e0);
    } else {
#pragma unroll
        for (int j = 0; j < BATCH; ++j)
            if (base + j * trip < kpad) load_row4(v[j], x, x_dtype, xoff, base + j * trip, k, vec);
    }
}

template <int BATCH = 6>
__device__ __forceinline__ void quantize_row_to_lds(unsigned char* lds, const void* __restrict__ x, int x_dtype, size_t xoff, int k, int kpad,
                                                    const RowNorm norm = RowNorm{nullptr, 0.0f, 0}) {
    int8_t* hi = reinterpret_cast<int8_t*>(lds);
    int8_t* lo = hi + kpad;
    float2* gs = reinterpret_cast<float2*>(lo + kpad);
    float* sum16 = reinterpret_cast<float*>(gs + kpad / 32);
    // one 8-byte (16-bit inputs) or 16-byte (float32) load per lane and trip when the row starts on that boundary
    const bool vec = x_dtype == PLLM_F32 ? ((reinterpret_cast<uintptr_t>(x) + 4 * xoff) & 15u) == 0
                                         : ((reinterpret_cast<uintptr_t>(x) + 2 * xoff) & 7u) == 0;
    const bool gvec = (reinterpret_cast<uintptr_t>(norm.gamma) & 15u) == 0;
    const int trip = static_cast<int>(blockDim.x) * 4;
    const int first = static_cast<int>(threadIdx.x) * 4;
    const bool one_batch = kpad <= trip * BATCH;                             // the whole row in one batch: read once, also for the norm
    float v[BATCH][4], g[BATCH][4];
    float rstd = 1.0f;
    if (norm.gamma) {
        // sum of squares of the row: per-wave sums meet in the first floats of the image area, which nobody has written yet
        float ss = 0.0f;
        if (one_batch) {
            // (the weights first: the row's loads sit behind a branch on its type, and what is requested after that branch, or
            // after the barriers, costs a round trip of its own)
            load_row_pieces<BATCH>(g, norm.gamma, PLLM_F32, 0, first, trip, k, kpad, gvec);
            load_row_pieces<BATCH>(v, x, x_dtype, xoff, first, trip, k, kpad, vec);
#pragma unroll
            for (int j = 0; j < BATCH; ++j)
                if (first + j * trip < kpad) ss += (v[j][0] * v[j][0] + v[j][1] * v[j][1]) + (v[j][2] * v[j][2] + v[j][3] * v[j][3]);
        } else {
            for (int e0 = first; e0 < k; e0 += trip) {
                float w[4];
                load_row4(w, x, x_dtype, xoff, e0, k, vec);
                ss += (w[0] * w[0] + w[1] * w[1]) + (w[2] * w[2] + w[3] * w[3]);
            }
        }
        ss = group_sum<64>(ss);
        float* red = reinterpret_cast<float*>(lds);
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
        __syncthreads();
        float total = 0.0f;
        for (int w = 0; w < static_cast<int>(blockDim.x >> 6); ++w) total += red[w];
        __syncthreads();                                                     // read by everybody before the image overwrites it
        rstd = rsqrtf(total / static_cast<float>(k) + norm.eps);
    }
    for (int base = first; base < kpad; base += trip * BATCH) {
        if (!(norm.gamma && one_batch)) load_row_pieces<BATCH>(v, x, x_dtype, xoff, base, trip, k, kpad, vec);
        if (norm.gamma) {
            if (!one_batch) load_row_pieces<BATCH>(g, norm.gamma, PLLM_F32, 0, base, trip, k, kpad, gvec);
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                if (base + j * trip < kpad) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float t = v[j][i] * rstd * g[j][i];                  // values past k are zeros on both sides
                        if (norm.round_f16) t = static_cast<float>(static_cast<_Float16>(t));
                        v[j][i] = t;
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < BATCH; ++j)
            if (base + j * trip < kpad) quantize4_to_image(v[j], base + j * trip, hi, lo, gs, sum16);
    }
}

// The Q8_0 pair image (layout in matvec_q8_0.hip): per pair of 32-value blocks 80 bytes that mirror the
// weight stream, [0,0, q0..q31, 0,0, q32..q63, 12 x 0], hi term then lo term, then float xs[2 * pairs].
__device__ __forceinline__ void quantize4_to_pair_image(const float v[4], int e0, unsigned char* hi, unsigned char* lo, float* xs) {
    uint32_t qh, ql;
    float scale;
    quantize4(v, qh, ql, scale);
    const int b = e0 >> 5;
    const int j = (e0 & 31) >> 2;
    const int off = (b >> 1) * 80 + ((b & 1) ? 36 : 2) + 4 * j;   // 2-byte aligned
    *reinterpret_cast<uint16_t*>(hi + off) = static_cast<uint16_t>(qh);
    *reinterpret_cast<uint16_t*>(hi + off + 2) = static_cast<uint16_t>(qh >> 16);
    *reinterpret_cast<uint16_t*>(lo + off) = static_cast<uint16_t>(ql);
    *reinterpret_cast<uint16_t*>(lo + off + 2) = static_cast<uint16_t>(ql >> 16);
    if (j == 0) {
        const int p0 = (b >> 1) * 80;
        if (b & 1) {
            *reinterpret_cast<uint16_t*>(hi + p0 + 34) = 0;
            *reinterpret_cast<uint16_t*>(lo + p0 + 34) = 0;
#pragma unroll
            for (int z = 68; z < 80; z += 4) {
                *reinterpret_cast<uint32_t*>(hi + p0 + z) = 0;
                *reinterpret_cast<uint32_t*>(lo + p0 + z) = 0;
            }
        } else {
            *reinterpret_cast<uint16_t*>(hi + p0) = 0;
            *reinterpret_cast<uint16_t*>(lo + p0) = 0;
        }
        xs[b] = scale;
    }
}

// Workgroup-wide copy of nbytes (a multiple of 16, both pointers 16-byte aligned) into LDS.
__device__ __forceinline__ void copy_to_lds(unsigned char* dst, const unsigned char* __restrict__ src, int nbytes) {
    const uint4* s = reinterpret_cast<const uint4*>(src);
    uint4* d = reinterpret_cast<uint4*>(dst);
    for (int i = threadIdx.x; i < (nbytes >> 4); i += blockDim.x) d[i] = s[i];
}

}  // namespace pllm
