// Block dequantization to float: selected rows of a raw-block matrix (the embedding operator) and
// whole FP8 matrices.  One thread per weight, byte loads, the reference decoders' operand order.
// Every product below is exact in float32, so only the K-quants' final subtraction rounds and the
// results are bit-identical to the numpy decoders whatever the compiler contracts.
#include "block_dot4.h"
#include "pllm_internal.h"

namespace pllm {
namespace {

__device__ __forceinline__ float f16_at(const uint8_t* p) {
    return f16_bits_to_float(static_cast<uint32_t>(p[0]) | (static_cast<uint32_t>(p[1]) << 8));
}

__device__ __forceinline__ void scale_min_k4(const uint8_t* s, int j, int& sc, int& mn) {
    if (j < 4) {
        sc = s[j] & 63;
        mn = s[j + 4] & 63;
    } else {
        sc = (s[j + 4] & 0x0f) | ((s[j - 4] >> 6) << 4);
        mn = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
    }
}

__device__ float dequant_q4_k(const uint8_t* b, int e) {
    const int pair = e >> 6, in_pair = e & 63, hi = in_pair >> 5;
    int sc, mn;
    scale_min_k4(b + 4, 2 * pair + hi, sc, mn);
    const int byte = b[16 + 32 * pair + (in_pair & 31)];
    const int q = hi ? (byte >> 4) : (byte & 15);
    return f16_at(b) * static_cast<float>(sc) * static_cast<float>(q) - f16_at(b + 2) * static_cast<float>(mn);
}

__device__ float dequant_q5_k(const uint8_t* b, int e) {
    const int pair = e >> 6, in_pair = e & 63, hi = in_pair >> 5, pos = in_pair & 31;
    int sc, mn;
    scale_min_k4(b + 4, 2 * pair + hi, sc, mn);
    const int byte = b[48 + 32 * pair + pos];
    const int q = (hi ? (byte >> 4) : (byte & 15)) + (((b[16 + pos] >> (2 * pair + hi)) & 1) ? 16 : 0);
    return f16_at(b) * static_cast<float>(sc) * static_cast<float>(q) - f16_at(b + 2) * static_cast<float>(mn);
}

__device__ float dequant_q2_k(const uint8_t* b, int e) {
    const int group = e >> 4, half = group >> 3, gi = group & 7;
    const int q = (b[16 + 32 * half + 16 * (gi & 1) + (e & 15)] >> (2 * (gi >> 1))) & 3;
    const int s = b[group];
    return f16_at(b + 80) * static_cast<float>(s & 15) * static_cast<float>(q) - f16_at(b + 82) * static_cast<float>(s >> 4);
}

__device__ float dequant_iq2_xxs(const uint8_t* b, int e) {
    const int sub = e >> 5, part = (e >> 3) & 3, j = e & 7;
    const uint8_t* c = b + 2 + 8 * sub;
    const uint32_t aux = static_cast<uint32_t>(c[4]) | (static_cast<uint32_t>(c[5]) << 8) | (static_cast<uint32_t>(c[6]) << 16) |
                         (static_cast<uint32_t>(c[7]) << 24);
    const uint32_t sidx = (aux >> (7 * part)) & 127u;
    const uint32_t sign8 = sidx | ((__popc(sidx) & 1u) << 7);
    const float mag = static_cast<float>((PLLM_IQ2XXS_GRID[c[part]] >> (8 * j)) & 0xffull);
    const float val = ((sign8 >> j) & 1u) ? -mag : mag;
    return 0.125f * f16_at(b) * static_cast<float>(2 * (aux >> 28) + 1) * val;
}

__device__ float dequant_iq1_m(const uint8_t* b, int e) {
    const int ent = e >> 3, t = e & 7, s = ent >> 1;
    uint32_t sc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) sc[i] = static_cast<uint32_t>(b[48 + 2 * i]) | (static_cast<uint32_t>(b[49 + 2 * i]) << 8);
    const uint32_t dbits = (sc[0] >> 12) | ((sc[1] >> 12) << 4) | ((sc[2] >> 12) << 8) | (sc[3] & 0xf000u);
    const uint32_t ls = (sc[s >> 2] >> (3 * (s & 3))) & 7u;
    const float dl = f16_bits_to_float(dbits) * static_cast<float>(2 * ls + 1);
    const uint32_t h = (b[32 + (ent >> 1)] >> (4 * (ent & 1))) & 15u;
    const uint32_t idx = b[ent] | ((h & 7u) << 8);
    const float g = static_cast<float>(static_cast<int>((PLLM_IQ1_GRID_PACKED[idx] >> (2 * t)) & 3u) - 1);
    return dl * (g + ((h & 8u) ? -0.125f : 0.125f));
}

// sign of weight j under a 7-bit sign index (bit 7 = parity of the other seven)
__device__ __forceinline__ float sign_of(uint32_t s7, int j) {
    const uint32_t s8 = s7 | ((__popc(s7) & 1u) << 7);
    return ((s8 >> j) & 1u) ? -1.0f : 1.0f;
}

// IQ2_XS: d, qs u16[32] (9-bit grid id, 7-bit sign index per 8 weights), scales(8): two 4-bit scales per 32 weights
__device__ float dequant_iq2_xs(const uint8_t* b, int e) {
    const int ent = e >> 3, j = e & 7;
    const uint32_t q = static_cast<uint32_t>(b[2 + 2 * ent]) | (static_cast<uint32_t>(b[3 + 2 * ent]) << 8);
    const uint32_t ls = (b[66 + (ent >> 2)] >> (4 * ((ent >> 1) & 1))) & 15u;
    const float mag = static_cast<float>((PLLM_IQ2XS_GRID[q & 511u] >> (8 * j)) & 0xffull);
    return 0.25f * f16_at(b) * (static_cast<float>(ls) + 0.5f) * (mag * sign_of(q >> 9, j));
}

// IQ3_XXS: d, grid ids(64: four weights each), aux u32[8] (four 7-bit sign indices per 32 weights, 4-bit scale)
__device__ float dequant_iq3_xxs(const uint8_t* b, int e) {
    const int sub = e >> 5, part = (e >> 2) & 7, j = e & 3;
    const uint8_t* a = b + 66 + 4 * sub;
    const uint32_t aux = static_cast<uint32_t>(a[0]) | (static_cast<uint32_t>(a[1]) << 8) | (static_cast<uint32_t>(a[2]) << 16) | (static_cast<uint32_t>(a[3]) << 24);
    const float mag = static_cast<float>((PLLM_IQ3XXS_GRID[b[2 + 8 * sub + part]] >> (8 * j)) & 0xffu);
    const float sgn = sign_of((aux >> (7 * (part >> 1))) & 127u, 4 * (part & 1) + j);
    return 0.5f * f16_at(b) * (static_cast<float>(aux >> 28) + 0.5f) * (mag * sgn);
}

// Q6_K: ql(128) qh(64) scales int8(16) d; weight e = 128 half + 32 j + l takes nibble j / 2 of ql[64 half + 32 (j % 2) + l],
// bit pair j of qh[32 half + l] and scale e / 16
__device__ float dequant_q6_k(const uint8_t* b, int e) {
    const int half = e >> 7, j = (e >> 5) & 3, l = e & 31;
    const uint32_t lo = (b[64 * half + 32 * (j & 1) + l] >> (4 * (j >> 1))) & 15u;
    const uint32_t hi = (b[128 + 32 * half + l] >> (2 * j)) & 3u;
    const int q = static_cast<int>(lo | (hi << 4)) - 32;
    const float d = f16_at(b + 208);
    return d * static_cast<float>(static_cast<int8_t>(b[192 + (e >> 4)])) * static_cast<float>(q);
}

__device__ const int8_t kIq4Values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

// IQ4_XS: d, scales_h u16, scales_l(4), qs(128); group g = e / 32: 6-bit scale - 32, byte 16 g + e % 16, low nibble for the
// first 16 weights of the group and high nibble for the others
__device__ float dequant_iq4_xs(const uint8_t* b, int e) {
    const int g = e >> 5, i = e & 31;
    const uint32_t sh = static_cast<uint32_t>(b[2]) | (static_cast<uint32_t>(b[3]) << 8);
    const int ls = static_cast<int>(((b[4 + (g >> 1)] >> (4 * (g & 1))) & 15u) | (((sh >> (2 * g)) & 3u) << 4)) - 32;
    const uint32_t code = (b[8 + 16 * g + (i & 15)] >> (4 * (i >> 4))) & 15u;
    return f16_at(b) * static_cast<float>(ls) * static_cast<float>(kIq4Values[code]);
}

// Q3_K as the reference's reader decodes it (src/loader/gguf/tensor_reader.py:746-776): 110 B = hmask(32) qs(64) scales(12) d(2);
// group g = e / 16: scale = nibble g of the first eight scale bytes - 8; two low bits from qs[4 g + j % 4] at 2 (j / 4), minus 4
// when bit j % 8 of hmask[2 g + j / 8] is clear; (d * scale) * q.
__device__ float dequant_q3_k(const uint8_t* b, int e) {
    const int g = e >> 4, j = e & 15;
    const int nib = g < 8 ? (b[96 + g] & 15) : (b[96 + g - 8] >> 4);
    const int low = (b[32 + 4 * g + (j & 3)] >> (2 * (j >> 2))) & 3;
    const int bit = (b[2 * g + (j >> 3)] >> (j & 7)) & 1;
    const float ds = f16_at(b + 108) * static_cast<float>(nib - 8);
    return ds * static_cast<float>(low - (bit ? 0 : 4));
}

// grid (selected rows, ceil(k / 256)), 256 threads
__global__ __launch_bounds__(256) void dequant_rows_kernel(
    const int64_t* __restrict__ row_ids, const uint8_t* __restrict__ blocks, int type_id, void* __restrict__ out, int out_dtype,
    int k, int bpr, int block_bytes, int64_t n_rows) {
    const int64_t row = row_ids ? row_ids[blockIdx.x] : static_cast<int64_t>(blockIdx.x);
    const int e = threadIdx.x;
    const int col = blockIdx.y * 256 + e;
    if (col >= k) return;
    float v = 0.0f;
    if (row >= 0 && row < n_rows) {
        if (type_id < 0) {                                                  // Q8_0: bpr counts 32-weight blocks
            const uint8_t* b = blocks + (static_cast<size_t>(row) * bpr + (col >> 5)) * 34;
            v = f16_at(b) * static_cast<float>(static_cast<int8_t>(b[2 + (col & 31)]));
        } else {
            const uint8_t* b = blocks + (static_cast<size_t>(row) * bpr + blockIdx.y) * block_bytes;
            switch (type_id) {
                case PLLM_TYPE_Q4_K: v = dequant_q4_k(b, e); break;
                case PLLM_TYPE_Q5_K: v = dequant_q5_k(b, e); break;
                case PLLM_TYPE_Q2_K: v = dequant_q2_k(b, e); break;
                case PLLM_TYPE_IQ2_XXS: v = dequant_iq2_xxs(b, e); break;
                case PLLM_TYPE_Q6_K: v = dequant_q6_k(b, e); break;
                case PLLM_TYPE_IQ2_XS: v = dequant_iq2_xs(b, e); break;
                case PLLM_TYPE_IQ3_XXS: v = dequant_iq3_xxs(b, e); break;
                case PLLM_TYPE_IQ4_XS: v = dequant_iq4_xs(b, e); break;
                case PLLM_TYPE_Q3_K: v = dequant_q3_k(b, e); break;
                default: v = dequant_iq1_m(b, e); break;
            }
        }
    }
    store_any(out, out_dtype, static_cast<size_t>(blockIdx.x) * k + col, v);
}

__device__ __forceinline__ float fp8_e4m3_to_float(uint32_t c) {
    const uint32_t e = (c >> 3) & 15u, m = c & 7u;
    float v;
    if (e == 0) v = static_cast<float>(m) * 0.001953125f;                           // m / 8 * 2^-6
    else if (e == 15 && m == 7) v = __uint_as_float(0x7fc00000u);
    else v = __uint_as_float(((e + 120u) << 23) | (m << 20));                       // (1 + m / 8) * 2^(e - 7)
    return (c & 0x80u) ? -v : v;
}

__global__ __launch_bounds__(256) void dequant_fp8_kernel(
    const uint8_t* __restrict__ w, const float* __restrict__ scale, void* __restrict__ out, int out_dtype, int n, int k, int kb) {
    const int col = blockIdx.y * 256 + threadIdx.x;
    const int row = blockIdx.x;
    if (col >= k) return;
    const float v = fp8_e4m3_to_float(w[static_cast<size_t>(row) * k + col]) * scale[(row >> 7) * kb + (col >> 7)];
    store_any(out, out_dtype, static_cast<size_t>(row) * k + col, v);
}

}  // namespace
}  // namespace pllm

extern "C" {

int pllm_gguf_dequantize_rows(const int64_t* row_ids, int64_t n_selected, const uint8_t* blocks, int type_id,
                              int64_t n_rows, int64_t k, int64_t blocks_per_row, void* out, int out_dtype, void* stream) {
    if (!blocks || !out || n_selected < 0 || n_rows <= 0 || k <= 0 || blocks_per_row <= 0) return PLLM_ERR_INVALID_ARGUMENT;
    if (out_dtype != PLLM_F32 && out_dtype != PLLM_F16 && out_dtype != PLLM_BF16) return PLLM_ERR_INVALID_ARGUMENT;
    const bool q8 = type_id == PLLM_TYPE_Q8_0;
    const int block_bytes = type_id == PLLM_TYPE_Q3_K ? 110 : pllm_gguf_block_bytes(type_id);   // (Q3_K: this entry point only)
    if (!q8 && block_bytes == 0) return PLLM_ERR_UNSUPPORTED;
    if (blocks_per_row * (q8 ? 32 : 256) < k) return PLLM_ERR_INVALID_ARGUMENT;
    if (n_selected == 0) return PLLM_OK;
    if (n_selected > 0x7fffffffLL || (k + 255) / 256 > 65535 || k > 0x7fffffffLL) return PLLM_ERR_UNSUPPORTED;
    dim3 grid(static_cast<unsigned>(n_selected), static_cast<unsigned>((k + 255) / 256));
    hipLaunchKernelGGL(pllm::dequant_rows_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), row_ids, blocks,
                       q8 ? -1 : type_id, out, out_dtype, static_cast<int>(k), static_cast<int>(blocks_per_row),
                       q8 ? 34 : block_bytes, n_rows);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

int pllm_fp8_block_dequantize(const uint8_t* weight, const float* scale, int64_t n, int64_t k, void* out, int out_dtype, void* stream) {
    if (!weight || !scale || !out || n <= 0 || k <= 0) return PLLM_ERR_INVALID_ARGUMENT;
    if (out_dtype != PLLM_F32 && out_dtype != PLLM_F16 && out_dtype != PLLM_BF16) return PLLM_ERR_INVALID_ARGUMENT;
    if (n > 0x7fffffffLL || (k + 255) / 256 > 65535) return PLLM_ERR_UNSUPPORTED;
    dim3 grid(static_cast<unsigned>(n), static_cast<unsigned>((k + 255) / 256));
    hipLaunchKernelGGL(pllm::dequant_fp8_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), weight, scale, out,
                       out_dtype, static_cast<int>(n), static_cast<int>(k), static_cast<int>((k + 127) / 128));
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

}  // extern "C"
