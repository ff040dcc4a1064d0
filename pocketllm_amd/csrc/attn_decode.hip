// Attention of one new token per sequence against a key/value store (decode step), two launches:
//     RMS normalisation of q and k over the whole projection width, rotary phases, store of the new key / value row,
//     scores against up to 64 stored keys per workgroup, softmax statistics and the weighted value sum of that slice;
//     then the slices of a head are merged (the usual running-maximum form of a split softmax).
// What the reference does between its q / k / v projections and its output projection (src/models/minimax_m2/
// architecture.py:158-266: q_norm, k_norm, apply_rotary_emb, cache update, scaled_dot_product_attention with the key/value
// heads shared by groups of query heads), for one query position.  None of it is quantized; it is here because a decoder
// block's step was dominated by the ~17 small framework launches this replaces, not by its matmuls.
//
// Layout: q [batch, heads * 128], k_new / v_new [batch, kv_heads * 128] in fp16 or bf16; stores [batch, kv_heads, capacity, 128]
// of the same type (batch and head strides in elements); out [batch, heads * 128].  Head dimension 128, up to 8 query heads per
// key/value head.  Arithmetic in float32 on the stored 16-bit values; the new key is rounded to the store's type before it is
// used, so a later step reads the same bits this step multiplied with.  HBM-bound on the store: 2 x length x kv_heads x 256 B.
#include "pllm_device.h"
#include "pllm_internal.h"

namespace pllm {
namespace {

constexpr int kHeadDim = 128;
constexpr int kSliceKeys = 64;
constexpr int kMaxGroup = 8;
constexpr int kMaxHeads = 64;                  // q rows of up to 64 x 128 values (four 16-byte pieces per thread)
constexpr int kQPieces = kMaxHeads * kHeadDim / (8 * 256), kKPieces = 2;   // k rows of up to 32 x 128 values
constexpr int kPartFloats = kHeadDim + 2;     // a slice's result per query head: 128 weighted sums, running maximum, sum of weights

template <bool BF16> struct HalfBits {
    static __device__ __forceinline__ float to_float(uint32_t bits) {
        if constexpr (BF16) return __uint_as_float(bits << 16);
        else return f16_bits_to_float(bits);
    }
    static __device__ __forceinline__ uint16_t from(float v) {
        if constexpr (BF16) return from_float<bf16_t>(v).bits;
        else {
            union { _Float16 h; uint16_t u; } c;
            c.h = static_cast<_Float16>(v);
            return c.u;
        }
    }
};
#define half_bits_to_float(bits, bf16) HalfBits<bf16>::to_float(bits)
#define float_to_half_bits(v, bf16) HalfBits<bf16>::from(v)
template <bool bf16>
__device__ __forceinline__ void unpack8(const uint4& u, float v[8]) {
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = half_bits_to_float(w[i] & 0xffffu, bf16);
        v[2 * i + 1] = half_bits_to_float(w[i] >> 16, bf16);
    }
}

// the rotary partner of value d of a head: the other half of the rotary part, itself behind it
__device__ __forceinline__ int rotary_partner(int d, int half) { return d < half ? d + half : (d < 2 * half ? d - half : d); }

// sum over the workgroup (256 threads) of two values at once; everybody gets both
__device__ __forceinline__ void block_sum2(float& a, float& b, float* red) {
    a = group_sum<64>(a);
    b = group_sum<64>(b);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { red[wave] = a; red[4 + wave] = b; }
    __syncthreads();
    a = (red[0] + red[1]) + (red[2] + red[3]);
    b = (red[4] + red[5]) + (red[6] + red[7]);
}

__device__ const float kOne = 1.0f;

struct DecodeArgs {
    const uint16_t* q; const uint16_t* k_new; const uint16_t* v_new;
    const float* q_weight; const float* k_weight;               // RMS normalisation weights over the whole q / k width, or null
    const float* cos_row; const float* sin_row;                 // 128 floats each for this position, or null (no rotary part)
    uint16_t* k_store; uint16_t* v_store;
    size_t batch_stride, head_stride;                           // of the stores, in elements
    float* part;                                                // [batch][heads][slices][kPartFloats]
    uint16_t* out;
    float eps, scale;
    int bf16, heads, kv_heads, rope_half, pos, slices;
};

// GROUP: the query heads per key/value head the loops are unrolled for (at least the launch's heads / kv_heads)
template <bool bf16, int GROUP>
__global__ __launch_bounds__(256) void attn_decode_slice_kernel(const DecodeArgs a) {
    __shared__ float red[8];
    __shared__ __align__(16) float qn[kMaxGroup][kHeadDim];                   // normalized, turned, scaled queries of this key/value head's group
    __shared__ __align__(16) uint16_t new_key[kHeadDim], new_value[kHeadDim]; // the new row as the store holds it
    __shared__ __align__(16) uint16_t raw_q[kMaxGroup * kHeadDim], raw_k[kHeadDim];   // the group's q heads and this head's k as they came
    __shared__ float w_q[kMaxGroup * kHeadDim], w_k[kHeadDim], rot_cos[kHeadDim], rot_sin[kHeadDim];
    __shared__ float weight[kMaxGroup][kSliceKeys];                           // scores, then softmax weights
    __shared__ float stats[kMaxGroup][2];
    __shared__ __align__(16) float sums[8][kMaxGroup][kHeadDim];              // weighted value sums per group of eight keys

    const int slice = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x;
    const int group = a.heads / a.kv_heads;
    const int length = a.pos + 1;
    const int j0 = slice * kSliceKeys;
    const int nkeys = min(kSliceKeys, length - j0);
    const bool has_new = a.pos >= j0 && a.pos < j0 + kSliceKeys;              // this slice holds the new position: it writes the stores

    const uint16_t* kbase = a.k_store + static_cast<size_t>(b) * a.batch_stride + static_cast<size_t>(kvh) * a.head_stride;
    const uint16_t* vbase = a.v_store + static_cast<size_t>(b) * a.batch_stride + static_cast<size_t>(kvh) * a.head_stride;

    // stored keys and values of the slice first: they are the long round trip.  Keys: thread (key tid / 4, quarter tid % 4) holds
    // 32 values; values: thread (keys 8 (tid / 32) .. + 7, columns 4 (tid % 32) .. + 3).  The new position is not in memory yet.
    // Every load has a valid address whatever the thread's share (row numbers clamped to the new position, whose row exists and is
    // replaced below): no load stands under a condition, so all of them are in flight together.
    const int key = tid >> 2, quarter = tid & 3;
    uint4 kreg[4];
    {
        const uint4* src = reinterpret_cast<const uint4*>(kbase + static_cast<size_t>(min(j0 + key, a.pos)) * kHeadDim + 32 * quarter);
#pragma unroll
        for (int i = 0; i < 4; ++i) kreg[i] = src[i];
    }
    const int kg = tid >> 5, dpart = tid & 31;
    uint2 vreg[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
        vreg[i] = *reinterpret_cast<const uint2*>(vbase + static_cast<size_t>(min(j0 + 8 * kg + i, a.pos)) * kHeadDim + 4 * dpart);

    // the q row, this head's k row, the group's normalisation weights and the rotary rows: requested in one batch behind the
    // stores' rows, staged in LDS as they are, so that the whole prologue costs one round trip to memory
    const uint16_t* qrow = a.q + static_cast<size_t>(b) * a.heads * kHeadDim;
    const uint16_t* krow = a.k_new + static_cast<size_t>(b) * a.kv_heads * kHeadDim;
    const int q_width = a.heads * kHeadDim, k_width = a.kv_heads * kHeadDim;
    uint4 qpiece[kQPieces], kpiece[kKPieces];
#pragma unroll
    for (int r = 0; r < kQPieces; ++r) qpiece[r] = *reinterpret_cast<const uint4*>(qrow + min(8 * (tid + 256 * r), q_width - 8));
#pragma unroll
    for (int r = 0; r < kKPieces; ++r) kpiece[r] = *reinterpret_cast<const uint4*>(krow + min(8 * (tid + 256 * r), k_width - 8));
    const float* qw_src = a.q_weight ? a.q_weight + kvh * group * kHeadDim : &kOne;    // null weights: read a one, stride zero
    const int qw_last = a.q_weight ? group * kHeadDim - 1 : 0;
    float qw_reg[kMaxGroup * kHeadDim / 256];
#pragma unroll
    for (int r = 0; r < kMaxGroup * kHeadDim / 256; ++r) qw_reg[r] = qw_src[min(tid + 256 * r, qw_last)];
    const float kw_reg = a.k_weight ? a.k_weight[kvh * kHeadDim + (tid & (kHeadDim - 1))] : 1.0f;
    const float rot_reg = a.cos_row ? (tid < kHeadDim ? a.cos_row[tid] : a.sin_row[tid - kHeadDim]) : (tid < kHeadDim ? 1.0f : 0.0f);
    const uint16_t v_bits = a.v_new[static_cast<size_t>(b) * k_width + kvh * kHeadDim + (tid & (kHeadDim - 1))];

    // sums of squares of the whole q and k rows; the group's part of q and this head's k go to LDS on the way
    float ssq = 0.0f, ssk = 0.0f;
#pragma unroll
    for (int r = 0; r < kQPieces; ++r) {
        float v[8];
        unpack8<bf16>(qpiece[r], v);
        if (8 * (tid + 256 * r) < q_width)
#pragma unroll
            for (int e = 0; e < 8; ++e) ssq += v[e] * v[e];
        const int at = 8 * (tid + 256 * r) - kvh * group * kHeadDim;          // position inside the group's part
        if (at >= 0 && at < group * kHeadDim) *reinterpret_cast<uint4*>(&raw_q[at]) = qpiece[r];
    }
#pragma unroll
    for (int r = 0; r < kKPieces; ++r) {
        float v[8];
        unpack8<bf16>(kpiece[r], v);
        if (8 * (tid + 256 * r) < k_width)
#pragma unroll
            for (int e = 0; e < 8; ++e) ssk += v[e] * v[e];
        const int at = 8 * (tid + 256 * r) - kvh * kHeadDim;
        if (at >= 0 && at < kHeadDim) *reinterpret_cast<uint4*>(&raw_k[at]) = kpiece[r];
    }
#pragma unroll
    for (int r = 0; r < kMaxGroup * kHeadDim / 256; ++r)
        if (tid + 256 * r < group * kHeadDim) w_q[tid + 256 * r] = qw_reg[r];
    if (tid < kHeadDim) { w_k[tid] = kw_reg; rot_cos[tid] = rot_reg; }
    else rot_sin[tid - kHeadDim] = rot_reg;
    block_sum2(ssq, ssk, red);                                                // (its barrier also covers the staging above)
    const float rstd_q = a.q_weight ? rsqrtf(ssq / static_cast<float>(q_width) + a.eps) : 1.0f;
    const float rstd_k = a.k_weight ? rsqrtf(ssk / static_cast<float>(k_width) + a.eps) : 1.0f;

    // one normalized value: x * rstd * weight, rounded to the activations' type like a separate normalisation's output; then the
    // turn out = x cos + partner sin, rounded again like a separate rotary operator's output
    auto normed = [&](const uint16_t* raw, const float* w, bool on, float rstd, int i) {
        const float x = half_bits_to_float(raw[i], bf16);
        return on ? half_bits_to_float(float_to_half_bits(x * rstd * w[i], bf16), bf16) : x;
    };
    auto turned = [&](const uint16_t* raw, const float* w, bool on, float rstd, int head_at, int d) {
        const float x = normed(raw, w, on, rstd, head_at + d);
        if (!a.cos_row) return x;
        const float xp = normed(raw, w, on, rstd, head_at + rotary_partner(d, a.rope_half));
        return half_bits_to_float(float_to_half_bits(__builtin_fmaf(xp, rot_sin[d], x * rot_cos[d]), bf16), bf16);
    };
    for (int e = tid; e < GROUP * kHeadDim; e += 256) {
        const int g = e / kHeadDim, d = e % kHeadDim;
        qn[g][d] = g < group ? turned(raw_q, w_q, a.q_weight != nullptr, rstd_q, g * kHeadDim, d) * a.scale : 0.0f;
    }
    if (has_new && tid < kHeadDim) {
        const uint16_t kb = float_to_half_bits(turned(raw_k, w_k, a.k_weight != nullptr, rstd_k, 0, tid), bf16);
        new_key[tid] = kb;
        new_value[tid] = v_bits;
        const size_t at = static_cast<size_t>(b) * a.batch_stride + static_cast<size_t>(kvh) * a.head_stride + static_cast<size_t>(a.pos) * kHeadDim + tid;
        a.k_store[at] = kb;
        a.v_store[at] = v_bits;
    }
    __syncthreads();

    // scores: 32 columns per thread, the four quarters of a key meet through the quad
    if (key < nkeys && j0 + key == a.pos) {
        const uint4* src = reinterpret_cast<const uint4*>(new_key + 32 * quarter);
#pragma unroll
        for (int i = 0; i < 4; ++i) kreg[i] = src[i];
    }
    {
        float kv[32];
#pragma unroll
        for (int i = 0; i < 4; ++i) unpack8<bf16>(kreg[i], kv + 8 * i);
        // the heads side by side: GROUP independent sums per pass over the key's values (rows of qn beyond the group hold
        // zeros and are not stored)
        float s[GROUP];
#pragma unroll
        for (int g = 0; g < GROUP; ++g) s[g] = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int g = 0; g < GROUP; ++g) {
                const float4 q4 = *reinterpret_cast<const float4*>(&qn[g][32 * quarter + 4 * i]);
                s[g] = __builtin_fmaf(q4.x, kv[4 * i], s[g]);
                s[g] = __builtin_fmaf(q4.y, kv[4 * i + 1], s[g]);
                s[g] = __builtin_fmaf(q4.z, kv[4 * i + 2], s[g]);
                s[g] = __builtin_fmaf(q4.w, kv[4 * i + 3], s[g]);
            }
#pragma unroll
        for (int g = 0; g < GROUP; ++g) {
            const float t = group_sum<4>(s[g]);
            if (quarter == 0 && g < group) weight[g][key] = key < nkeys ? t : -INFINITY;
        }
    }
    __syncthreads();

    // softmax statistics of the slice: wave w takes heads w, w + 4
    {
        const int lane = tid & 63, wave = tid >> 6;
        for (int g = wave; g < group; g += 4) {
            const float s = weight[g][lane];
            const float m = group_max<64>(s);
            const float p = lane < nkeys ? expf(s - m) : 0.0f;
            weight[g][lane] = p;
            const float l = group_sum<64>(p);
            if (lane == 0) { stats[g][0] = m; stats[g][1] = l; }
        }
    }
    __syncthreads();

    // weighted sums of the values: eight keys and four columns per thread
    {
        float acc[GROUP][4] = {};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int j = 8 * kg + i;
            if (j < nkeys) {                 // uniform over the 32 threads of a key group
                const uint2 fresh = *reinterpret_cast<const uint2*>(new_value + 4 * dpart);
                const uint2 bits = j0 + j == a.pos ? fresh : vreg[i];
                const float v0 = half_bits_to_float(bits.x & 0xffffu, bf16), v1 = half_bits_to_float(bits.x >> 16, bf16);
                const float v2 = half_bits_to_float(bits.y & 0xffffu, bf16), v3 = half_bits_to_float(bits.y >> 16, bf16);
#pragma unroll
                for (int g = 0; g < GROUP; ++g) {
                    {
                        const float p = g < group ? weight[g][j] : 0.0f;
                        acc[g][0] = __builtin_fmaf(p, v0, acc[g][0]);
                        acc[g][1] = __builtin_fmaf(p, v1, acc[g][1]);
                        acc[g][2] = __builtin_fmaf(p, v2, acc[g][2]);
                        acc[g][3] = __builtin_fmaf(p, v3, acc[g][3]);
                    }
                }
            }
        }
#pragma unroll
        for (int g = 0; g < GROUP; ++g)
            if (g < group) *reinterpret_cast<float4*>(&sums[kg][g][4 * dpart]) = make_float4(acc[g][0], acc[g][1], acc[g][2], acc[g][3]);
    }
    __syncthreads();
    for (int e = tid; e < group * kHeadDim; e += 256) {
        const int g = e / kHeadDim, d = e % kHeadDim;
        float o = 0.0f;
#pragma unroll
        for (int r = 0; r < 8; ++r) o += sums[r][g][d];
        const int head = kvh * group + g;
        if (a.slices == 1) {
            a.out[(static_cast<size_t>(b) * a.heads + head) * kHeadDim + d] = float_to_half_bits(o / stats[g][1], bf16);
        } else {
            float* dst = a.part + ((static_cast<size_t>(b) * a.heads + head) * a.slices + slice) * kPartFloats;
            dst[d] = o;
            if (d == 0) { dst[kHeadDim] = stats[g][0]; dst[kHeadDim + 1] = stats[g][1]; }
        }
    }
}

// out[b, head, :] = sum over slices of sums * exp(m - M) / sum over slices of l * exp(m - M), slices in order.
// The slices' statistics are fetched side by side (one round trip), the sums in batches of eight.
constexpr int kMaxSlices = 2048;                // stores of up to 131072 positions
__global__ __launch_bounds__(kHeadDim) void attn_decode_merge_kernel(const float* __restrict__ part, uint16_t* __restrict__ out, int slices, int bf16) {
    __shared__ float factor[kMaxSlices];
    __shared__ float wave_top[2], wave_den[2];
    const size_t row = blockIdx.x;                                            // b * heads + head
    const float* src = part + row * slices * kPartFloats;
    const int d = threadIdx.x;
    float top = -INFINITY;
    for (int s = d; s < slices; s += kHeadDim) { const float m = src[s * kPartFloats + kHeadDim]; factor[s] = m; top = fmaxf(top, m); }
    top = group_max<64>(top);
    if ((d & 63) == 0) wave_top[d >> 6] = top;
    __syncthreads();
    top = fmaxf(wave_top[0], wave_top[1]);
    float den = 0.0f;
    for (int s = d; s < slices; s += kHeadDim) {
        const float f = expf(factor[s] - top);
        factor[s] = f;
        den = __builtin_fmaf(src[s * kPartFloats + kHeadDim + 1], f, den);
    }
    den = group_sum<64>(den);
    if ((d & 63) == 0) wave_den[d >> 6] = den;
    __syncthreads();
    den = wave_den[0] + wave_den[1];
    float num = 0.0f;
    int s = 0;
    for (; s + 8 <= slices; s += 8) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = src[(s + i) * kPartFloats + d];
#pragma unroll
        for (int i = 0; i < 8; ++i) num = __builtin_fmaf(v[i], factor[s + i], num);
    }
    for (; s < slices; ++s) num = __builtin_fmaf(src[s * kPartFloats + d], factor[s], num);
    out[row * kHeadDim + d] = bf16 ? HalfBits<true>::from(num / den) : HalfBits<false>::from(num / den);
}

}  // namespace

size_t attention_decode_workspace_bytes(int batch, int heads, int pos) {
    const int slices = pos / kSliceKeys + 1;
    return slices == 1 ? 0 : align256(static_cast<size_t>(batch) * heads * slices * kPartFloats * sizeof(float));
}

bool attention_decode_supports(int heads, int kv_heads, int head_dim, int rope_dim) {
    return head_dim == kHeadDim && kv_heads >= 1 && heads % kv_heads == 0 && heads / kv_heads <= kMaxGroup && heads <= kMaxHeads &&
           kv_heads * kHeadDim <= kKPieces * 8 * 256 && rope_dim >= 0 && rope_dim <= kHeadDim && rope_dim % 2 == 0;
}

int attention_decode(const void* q, const void* k_new, const void* v_new, int dtype, const float* q_weight, const float* k_weight, float eps,
                     const float* cos_row, const float* sin_row, int rope_dim, void* k_store, void* v_store, size_t batch_stride,
                     size_t head_stride, int batch, int heads, int kv_heads, int pos, void* out, void* workspace, hipStream_t stream) {
    DecodeArgs a;
    a.q = static_cast<const uint16_t*>(q); a.k_new = static_cast<const uint16_t*>(k_new); a.v_new = static_cast<const uint16_t*>(v_new);
    a.q_weight = q_weight; a.k_weight = k_weight;
    a.cos_row = rope_dim > 0 ? cos_row : nullptr; a.sin_row = rope_dim > 0 ? sin_row : nullptr;
    a.k_store = static_cast<uint16_t*>(k_store); a.v_store = static_cast<uint16_t*>(v_store);
    a.batch_stride = batch_stride; a.head_stride = head_stride;
    a.part = static_cast<float*>(workspace);
    a.out = static_cast<uint16_t*>(out);
    a.eps = eps; a.scale = 1.0f / sqrtf(static_cast<float>(kHeadDim));
    a.bf16 = dtype == PLLM_BF16; a.heads = heads; a.kv_heads = kv_heads; a.rope_half = rope_dim / 2; a.pos = pos;
    a.slices = pos / kSliceKeys + 1;
    if (a.slices > kMaxSlices) return PLLM_ERR_UNSUPPORTED;
    const int group = heads / kv_heads;
    const dim3 grid(a.slices, kv_heads, batch);
#define PLLM_CASE(G) \
    if (group <= G) { \
        if (a.bf16) hipLaunchKernelGGL((attn_decode_slice_kernel<true, G>), grid, dim3(256), 0, stream, a); \
        else hipLaunchKernelGGL((attn_decode_slice_kernel<false, G>), grid, dim3(256), 0, stream, a); \
    } else
    PLLM_CASE(1) PLLM_CASE(2) PLLM_CASE(4) PLLM_CASE(6) PLLM_CASE(8) return PLLM_ERR_UNSUPPORTED;
#undef PLLM_CASE
    if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
    if (a.slices > 1) {
        hipLaunchKernelGGL(attn_decode_merge_kernel, dim3(batch * heads), dim3(kHeadDim), 0, stream, a.part, a.out, a.slices, a.bf16);
        if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
    }
    return PLLM_OK;
}

}  // namespace pllm
