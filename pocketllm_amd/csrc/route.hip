// Expert routing of the fused expert path's callers: gate logits, scores, top-k and renormalised
// route weights in two launches instead of six framework ops.
//
//   logits[t, e] = x[t, :] . gate_weight[e, :]                (float32 accumulate)
//   sigmoid mode: p = sigmoid(logits); pick the top_k of p + bias (bias optional); weight = p / max(sum of picked p, 1e-20)
//   softmax mode: pick the top_k logits; weight = softmax over the picked logits (= softmax probabilities renormalised)
//
// Launch 1: one wave per (expert, group of 4 tokens), 16-byte loads, the gate row held in registers, the tokens side by side, 64-lane sums;
// from 80 tokens on 16 x 16 blocks of logits on the float32 matrix cores instead.  Launch 2: one
// wave per token, every lane keeps E / 64 candidates in registers, top_k rounds of a wave-wide
// argmax (larger score first, lower expert id on equal scores), picked in descending order.
#include "pllm_device.h"
#include "pllm_internal.h"

namespace pllm {
namespace {

constexpr int kThreads = 256;
constexpr int kWavesPerWg = kThreads / 64;
constexpr int kMaxPerLane = 16;          // experts per lane: up to 1024 experts

// One wave per (expert, group of kTokensPerWave tokens): the gate row is read once per group (its
// first kHeld float4 pieces per lane stay in registers), the tokens' rows come from cache.
constexpr int kTokensPerWave = 4;        // their x loads are in flight together; a single token (decode) runs alone
constexpr int kMfmaMinTokens = 80;       // from here on the logits are formed block by block on the matrix cores
constexpr int kHeld = 12;                // 12 x 256 floats: gate rows up to 3072 wide are held whole

template <int NT>
__global__ __launch_bounds__(kThreads) void route_logits_kernel(
    const void* __restrict__ x, int x_dtype, const float* __restrict__ gate, float* __restrict__ logits, int dim, int n_experts, int tokens) {
    const int lane = threadIdx.x & 63;
    const int e = blockIdx.x * kWavesPerWg + (threadIdx.x >> 6);
    if (e >= n_experts) return;                                             // whole waves leave together
    const float* grow = gate + static_cast<size_t>(e) * dim;
    const int t0 = blockIdx.y * NT, t1 = min(tokens, t0 + NT);
    const bool vec = (dim % 4 == 0) && ((reinterpret_cast<uintptr_t>(gate) & 15u) == 0);
    if (!vec) {
        for (int t = t0; t < t1; ++t) {
            float acc = 0.0f;
            for (int c = lane; c < dim; c += 64) acc += grow[c] * load_any(x, x_dtype, static_cast<size_t>(t) * dim + c);
            acc = group_sum<64>(acc);
            if (lane == 0) logits[static_cast<size_t>(t) * n_experts + e] = acc;
        }
        return;
    }
    float4 held[kHeld];
#pragma unroll
    for (int i = 0; i < kHeld; ++i) {
        const int c = lane * 4 + 256 * i;
        const float4 gv = *reinterpret_cast<const float4*>(grow + min(c, dim - 4));
        held[i] = c < dim ? gv : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
    // all tokens of the group side by side: their loads are independent and go out together
    const bool xvec = ((reinterpret_cast<uintptr_t>(x) & 15u) == 0) && (x_dtype != PLLM_F32 ? dim % 4 == 0 : true);
    float acc[NT];
    size_t xoff[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        acc[j] = 0.0f;
        xoff[j] = static_cast<size_t>(min(t0 + j, t1 - 1)) * dim;            // past the end: the last token again, result dropped
    }
    // (no branch around the loads: pieces beyond the row read its last piece again and are dropped; a branch per piece would
    // make every piece wait for its own round trip)
    int cpos[kHeld];
#pragma unroll
    for (int i = 0; i < kHeld; ++i) cpos[i] = min(lane * 4 + 256 * i, max(dim - 4, 0));
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        float v[kHeld][4];
        if (xvec) {
            load_rows4_batch(v, x, x_dtype, xoff[j], cpos);
        } else {
#pragma unroll
            for (int i = 0; i < kHeld; ++i) load_row4(v[i], x, x_dtype, xoff[j], cpos[i], dim, false);
        }
#pragma unroll
        for (int i = 0; i < kHeld; ++i) {
            const float d = held[i].x * v[i][0] + held[i].y * v[i][1] + held[i].z * v[i][2] + held[i].w * v[i][3];
            acc[j] += (lane * 4 + 256 * i < dim) ? d : 0.0f;
        }
    }
    for (int c = lane * 4 + 256 * kHeld; c < dim; c += 256) {               // rows wider than the held part
        const float4 g = *reinterpret_cast<const float4*>(grow + c);
#pragma unroll
        for (int j = 0; j < NT; ++j)
            acc[j] += g.x * load_any(x, x_dtype, xoff[j] + c) + g.y * load_any(x, x_dtype, xoff[j] + c + 1) +
                      g.z * load_any(x, x_dtype, xoff[j] + c + 2) + g.w * load_any(x, x_dtype, xoff[j] + c + 3);
    }
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const float total = group_sum<64>(acc[j]);
        if (lane == 0 && t0 + j < t1) logits[static_cast<size_t>(t0 + j) * n_experts + e] = total;
    }
}

// Decode rows that are RMS-normalized first (the block's normalisation ahead of its experts): one wave per (expert, token).
// Every wave holds the whole row, so every wave forms the row's sum of squares itself; v = x * rsqrt(mean(x^2) + eps) * weight is
// rounded to xn_dtype (what a normalisation launch of its own would have stored) and the logit is formed on the rounded values.
// The wave of expert 0 also writes the normalized row out for the operators that follow.  dim <= 256 * kHeld, dim % 4 == 0,
// 16-byte aligned rows.
template <int XN>
__device__ __forceinline__ float round_to(float v) {
    if constexpr (XN == PLLM_F16) return static_cast<float>(static_cast<_Float16>(v));
    if constexpr (XN == PLLM_BF16) return to_float(from_float<bf16_t>(v));
    return v;
}
template <int XN>
__global__ __launch_bounds__(kThreads) void route_logits_norm_kernel(
    const void* __restrict__ x, int x_dtype, const float* __restrict__ norm_weight, float eps, void* __restrict__ xn,
    const float* __restrict__ gate, float* __restrict__ logits, int dim, int n_experts) {
    const int lane = threadIdx.x & 63;
    const int e = blockIdx.x * kWavesPerWg + (threadIdx.x >> 6);
    if (e >= n_experts) return;                                             // whole waves leave together
    const int t = blockIdx.y;
    const float* grow = gate + static_cast<size_t>(e) * dim;
    int cpos[kHeld];
#pragma unroll
    for (int i = 0; i < kHeld; ++i) cpos[i] = min(lane * 4 + 256 * i, dim - 4);   // beyond the row: its last piece again, not counted
    // gate row and norm weights first: the row's loads sit behind a branch on its type, and what is requested after that branch
    // would wait for a round trip of its own
    float4 held[kHeld], g[kHeld];
#pragma unroll
    for (int i = 0; i < kHeld; ++i) {
        held[i] = *reinterpret_cast<const float4*>(grow + cpos[i]);
        g[i] = *reinterpret_cast<const float4*>(norm_weight + cpos[i]);
    }
    float v[kHeld][4];
    load_rows4_batch(v, x, x_dtype, static_cast<size_t>(t) * dim, cpos);
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < kHeld; ++i)
        if (lane * 4 + 256 * i < dim) ss += (v[i][0] * v[i][0] + v[i][1] * v[i][1]) + (v[i][2] * v[i][2] + v[i][3] * v[i][3]);
    const float rstd = rsqrtf(group_sum<64>(ss) / static_cast<float>(dim) + eps);
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < kHeld; ++i) {
        v[i][0] = round_to<XN>(v[i][0] * rstd * g[i].x);
        v[i][1] = round_to<XN>(v[i][1] * rstd * g[i].y);
        v[i][2] = round_to<XN>(v[i][2] * rstd * g[i].z);
        v[i][3] = round_to<XN>(v[i][3] * rstd * g[i].w);
        const float d = held[i].x * v[i][0] + held[i].y * v[i][1] + held[i].z * v[i][2] + held[i].w * v[i][3];
        acc += (lane * 4 + 256 * i < dim) ? d : 0.0f;
    }
    // the normalized row leaves piece by piece: the wave of expert i (of expert 0 where there are fewer experts than pieces)
    // stores piece i, one 8- or 16-byte store per lane
#pragma unroll
    for (int i = 0; i < kHeld; ++i) {
        if (e == (n_experts >= kHeld ? i : 0) && lane * 4 + 256 * i < dim) {
            const size_t o = static_cast<size_t>(t) * dim + lane * 4 + 256 * i;
            if constexpr (XN == PLLM_F32) {
                *reinterpret_cast<float4*>(static_cast<float*>(xn) + o) = make_float4(v[i][0], v[i][1], v[i][2], v[i][3]);
            } else if constexpr (XN == PLLM_F16) {
                union { _Float16 h[4]; uint2 u; } pk;
#pragma unroll
                for (int c = 0; c < 4; ++c) pk.h[c] = static_cast<_Float16>(v[i][c]);
                *reinterpret_cast<uint2*>(static_cast<uint16_t*>(xn) + o) = pk.u;
            } else {
                // (already bf16 values: the high halves are exact)
                const uint2 pk = make_uint2((__float_as_uint(v[i][0]) >> 16) | (__float_as_uint(v[i][1]) & 0xffff0000u),
                                            (__float_as_uint(v[i][2]) >> 16) | (__float_as_uint(v[i][3]) & 0xffff0000u));
                *reinterpret_cast<uint2*>(static_cast<uint16_t*>(xn) + o) = pk;
            }
        }
    }
    acc = group_sum<64>(acc);
    if (lane == 0) logits[static_cast<size_t>(t) * n_experts + e] = acc;
}

// Many tokens: a workgroup forms the 16 x 16 block logits[t0 .. t0 + 15, e0 .. e0 + 15] on the float32 matrix cores
// (v_mfma_f32_16x16x4_f32, C[m][n] = sum_k A[m][k] B[k][n] with m = token, n = expert).  Lane (r, q) = (lane % 16, lane / 16)
// loads four consecutive values of token row r and of gate row r at column k0 + 4 q; value i of both goes to MFMA i of the step,
// where the lane's k index is q on either side.  The four waves split the row's columns and meet in LDS.  A block reads
// 16 gate rows and 16 token rows once: an eighth of the cache traffic of the one-wave-per-expert form.  dim % 16 == 0.
typedef float v4f __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(kThreads) void route_logits_mfma_kernel(
    const void* __restrict__ x, int x_dtype, const float* __restrict__ gate, float* __restrict__ logits, int dim, int n_experts, int tokens) {
    __shared__ float partial[kWavesPerWg][16 * 16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, q = lane >> 4;
    const int e0 = blockIdx.x * 16, t0 = blockIdx.y * 16;
    const float* grow = gate + static_cast<size_t>(min(e0 + r, n_experts - 1)) * dim;       // past the end: a valid row, result dropped
    const size_t xoff = static_cast<size_t>(min(t0 + r, tokens - 1)) * dim;
    const bool xvec = ((reinterpret_cast<uintptr_t>(x) & 15u) == 0);
    const int per_wave = (dim / 16 + kWavesPerWg - 1) / kWavesPerWg * 16;                    // columns per wave, a multiple of 16
    const int k_begin = wave * per_wave, k_end = min(dim, k_begin + per_wave);
    v4f c = {0.0f, 0.0f, 0.0f, 0.0f};
    constexpr int kUnroll = 4;
    for (int k0 = k_begin; k0 < k_end; k0 += 16 * kUnroll) {
        float4 g[kUnroll];
        float xv[kUnroll][4];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int col = min(k0 + 16 * u, k_end - 16) + 4 * q;                            // a step past the end repeats the last one ...
            g[u] = *reinterpret_cast<const float4*>(grow + col);
            load_row4(xv[u], x, x_dtype, xoff, col, dim, xvec);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            if (k0 + 16 * u < k_end) {                                                       // ... and is not multiplied (wave-uniform)
                c = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[u][0], g[u].x, c, 0, 0, 0);
                c = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[u][1], g[u].y, c, 0, 0, 0);
                c = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[u][2], g[u].z, c, 0, 0, 0);
                c = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[u][3], g[u].w, c, 0, 0, 0);
            }
        }
    }
    // lane (n = r, quad q) holds C[4 q + i][n], i = 0..3: token t0 + 4 q + i, expert e0 + r
#pragma unroll
    for (int i = 0; i < 4; ++i) partial[wave][(4 * q + i) * 16 + r] = c[i];
    __syncthreads();
    const int m = threadIdx.x >> 4, n = threadIdx.x & 15;                                    // 256 threads, 256 outputs
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < kWavesPerWg; ++w) total += partial[w][m * 16 + n];
    if (t0 + m < tokens && e0 + n < n_experts) logits[static_cast<size_t>(t0 + m) * n_experts + e0 + n] = total;
}

__device__ __forceinline__ float wave_max(float v) { return group_max<64>(v); }

// the maximum over the wave as a wave-uniform value: butterflies inside the rows of 16 lanes, then the four rows' results
// through scalar registers (no LDS crossbar)
__device__ __forceinline__ float wave_max_uniform(float v) {
    v = group_max<16>(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0)), r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32)), r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// PER = candidates per lane (expert lane + 64 i)
template <int PER>
__global__ __launch_bounds__(64) void route_topk_kernel(
    const float* __restrict__ logits, const float* __restrict__ bias, int n_experts, int top_k, int softmax_mode,
    int64_t* __restrict__ indices, float* __restrict__ weights) {
    const int lane = threadIdx.x;
    const size_t t = blockIdx.x;
    const float* row = logits + t * n_experts;
    constexpr float kGone = -3.0e38f;
    float score[PER], prob[PER], l[PER], bv[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {                                         // all loads first, past the end the last expert again
        const int e = min(lane + 64 * i, n_experts - 1);
        l[i] = row[e];
        bv[i] = bias ? bias[e] : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const bool live = lane + 64 * i < n_experts;
        const float p = softmax_mode ? l[i] : 1.0f / (1.0f + expf(-l[i]));
        prob[i] = live ? p : 0.0f;
        score[i] = live ? (softmax_mode ? p : p + bv[i]) : kGone;
    }
    // top_k rounds; lane r keeps the r-th pick
    int my_pick = -1;
    float my_prob = 0.0f;
    for (int r = 0; r < top_k; ++r) {
        float best = kGone;
        int best_e = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < PER; ++i) {                                     // ascending expert id inside the lane: strict > keeps the lowest
            if (score[i] > best) { best = score[i]; best_e = lane + 64 * i; }
        }
        const float top = wave_max_uniform(best);
        // the lowest expert id among the lanes that hold the maximum: one lane almost always, else a wave-wide minimum
        const unsigned long long holders = __ballot(best == top);
        int cand;
        if (__popcll(holders) == 1) {
            cand = __builtin_amdgcn_readlane(best_e, static_cast<int>(__ffsll(static_cast<long long>(holders))) - 1);
        } else {
            cand = (best == top) ? best_e : 0x7fffffff;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) cand = min(cand, __shfl_xor(cand, off, 64));
            cand = __builtin_amdgcn_readfirstlane(cand);
        }
        const int owner = cand & 63, slot = cand >> 6;
        float p = 0.0f;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            if (i == slot) p = prob[i];                                     // (wave-uniform slot)
            if (lane == owner && i == slot) score[i] = kGone;
        }
        p = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), owner));
        if (lane == r) { my_pick = cand; my_prob = p; }
    }
    // renormalise over the picks (lanes 0 .. top_k - 1)
    float w;
    if (softmax_mode) {
        const float m = wave_max(lane < top_k ? my_prob : kGone);
        const float ex = lane < top_k ? expf(my_prob - m) : 0.0f;
        w = ex / group_sum<64>(ex);
    } else {
        const float total = group_sum<64>(lane < top_k ? my_prob : 0.0f);
        w = my_prob / fmaxf(total, 1.0e-20f);
    }
    if (lane < top_k) {
        indices[t * top_k + lane] = my_pick;
        weights[t * top_k + lane] = w;
    }
}

}  // namespace
}  // namespace pllm

extern "C" {

int pllm_moe_route(const void* x, int x_dtype, int64_t tokens, int64_t dim, const float* gate_weight, const float* gate_bias,
                   int64_t n_experts, int64_t top_k, int softmax_mode, float* logits, int64_t* indices, float* weights, void* stream) {
    using namespace pllm;
    if (!x || !gate_weight || !logits || !indices || !weights) return PLLM_ERR_INVALID_ARGUMENT;
    if (x_dtype != PLLM_F32 && x_dtype != PLLM_F16 && x_dtype != PLLM_BF16) return PLLM_ERR_INVALID_ARGUMENT;
    if (tokens <= 0 || dim <= 0 || n_experts <= 0 || top_k <= 0 || top_k > n_experts) return PLLM_ERR_INVALID_ARGUMENT;
    if (n_experts > 64 * kMaxPerLane || top_k > 64 || tokens > 65535 || dim > 0x7fffffffLL) return PLLM_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 wgs(static_cast<unsigned>((n_experts + kWavesPerWg - 1) / kWavesPerWg),
                   static_cast<unsigned>(tokens == 1 ? 1 : (tokens + kTokensPerWave - 1) / kTokensPerWave));
    if (tokens >= kMfmaMinTokens && dim % 16 == 0 && dim >= 16 && ((reinterpret_cast<uintptr_t>(gate_weight) & 15u) == 0))
        hipLaunchKernelGGL(route_logits_mfma_kernel, dim3(static_cast<unsigned>((n_experts + 15) / 16), static_cast<unsigned>((tokens + 15) / 16)),
                           dim3(kThreads), 0, s, x, x_dtype, gate_weight, logits, static_cast<int>(dim), static_cast<int>(n_experts),
                           static_cast<int>(tokens));
    else if (tokens == 1)
        hipLaunchKernelGGL(route_logits_kernel<1>, wgs, dim3(kThreads), 0, s, x, x_dtype, gate_weight, logits, static_cast<int>(dim),
                           static_cast<int>(n_experts), static_cast<int>(tokens));
    else
        hipLaunchKernelGGL(route_logits_kernel<kTokensPerWave>, wgs, dim3(kThreads), 0, s, x, x_dtype, gate_weight, logits, static_cast<int>(dim),
                           static_cast<int>(n_experts), static_cast<int>(tokens));
    if (n_experts <= 256)
        hipLaunchKernelGGL(route_topk_kernel<4>, dim3(static_cast<unsigned>(tokens)), dim3(64), 0, s, logits, gate_bias, static_cast<int>(n_experts),
                           static_cast<int>(top_k), softmax_mode, indices, weights);
    else
        hipLaunchKernelGGL(route_topk_kernel<kMaxPerLane>, dim3(static_cast<unsigned>(tokens)), dim3(64), 0, s, logits, gate_bias,
                           static_cast<int>(n_experts), static_cast<int>(top_k), softmax_mode, indices, weights);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

int pllm_moe_route_rmsnorm(const void* x, int x_dtype, const float* norm_weight, float eps, void* x_normed, int x_normed_dtype,
                           int64_t tokens, int64_t dim, const float* gate_weight, const float* gate_bias, int64_t n_experts, int64_t top_k,
                           int softmax_mode, float* logits, int64_t* indices, float* weights, void* stream) {
    using namespace pllm;
    if (!x || !norm_weight || !x_normed || !gate_weight || !logits || !indices || !weights) return PLLM_ERR_INVALID_ARGUMENT;
    if (x_dtype != PLLM_F32 && x_dtype != PLLM_F16 && x_dtype != PLLM_BF16) return PLLM_ERR_INVALID_ARGUMENT;
    if (x_normed_dtype != PLLM_F32 && x_normed_dtype != PLLM_F16 && x_normed_dtype != PLLM_BF16) return PLLM_ERR_INVALID_ARGUMENT;
    if (tokens <= 0 || dim <= 0 || n_experts <= 0 || top_k <= 0 || top_k > n_experts) return PLLM_ERR_INVALID_ARGUMENT;
    if (n_experts > 64 * kMaxPerLane || top_k > 64) return PLLM_ERR_UNSUPPORTED;
    // decode rows that a wave can hold whole, everything on vector boundaries; other calls: normalisation and routing as two operators
    const uintptr_t align = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(norm_weight) | reinterpret_cast<uintptr_t>(gate_weight) |
                            reinterpret_cast<uintptr_t>(x_normed);
    if (tokens > 4 || dim > 256 * kHeld || dim < 4 || dim % 4 != 0 || (align & 15u) != 0) return PLLM_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 wgs(static_cast<unsigned>((n_experts + kWavesPerWg - 1) / kWavesPerWg), static_cast<unsigned>(tokens));
    const int d = static_cast<int>(dim), ne = static_cast<int>(n_experts);
    if (x_normed_dtype == PLLM_F16)
        hipLaunchKernelGGL(route_logits_norm_kernel<PLLM_F16>, wgs, dim3(kThreads), 0, s, x, x_dtype, norm_weight, eps, x_normed, gate_weight, logits, d, ne);
    else if (x_normed_dtype == PLLM_BF16)
        hipLaunchKernelGGL(route_logits_norm_kernel<PLLM_BF16>, wgs, dim3(kThreads), 0, s, x, x_dtype, norm_weight, eps, x_normed, gate_weight, logits, d, ne);
    else
        hipLaunchKernelGGL(route_logits_norm_kernel<PLLM_F32>, wgs, dim3(kThreads), 0, s, x, x_dtype, norm_weight, eps, x_normed, gate_weight, logits, d, ne);
    if (n_experts <= 256)
        hipLaunchKernelGGL(route_topk_kernel<4>, dim3(static_cast<unsigned>(tokens)), dim3(64), 0, s, logits, gate_bias, static_cast<int>(n_experts),
                           static_cast<int>(top_k), softmax_mode, indices, weights);
    else
        hipLaunchKernelGGL(route_topk_kernel<kMaxPerLane>, dim3(static_cast<unsigned>(tokens)), dim3(64), 0, s, logits, gate_bias,
                           static_cast<int>(n_experts), static_cast<int>(top_k), softmax_mode, indices, weights);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

}  // extern "C"
