/* CPU restatement in plain C of the raw-block matvec: y[t][r] = sum_k x[t][k] * w[r][k], the weights decoded block by block
 * on the fly (no float copy of the matrix), float32 accumulation, OpenMP over output rows.
 *
 * TEST INFRASTRUCTURE ONLY: the benchmark's CPU-baseline leg times it and tests/ compares it with the numpy oracle; nothing in
 * the shipped package links or loads it.
 *
 * What it follows in the reference (paths relative to the reference checkout):
 *   - block layouts and decode arithmetic: src/loader/gguf/tensor_reader.py:543-550 (Q8_0), 786-821 (Q4_K), 823-866 (Q5_K),
 *     135-146 (the 6-bit scale / min unpacking);
 *   - the loop shape (one OpenMP thread per output row, block dots in float32): src/csrc/deepseek_cpu_moe_ext.cpp:2759-2803
 *     (gguf_quantized_matmul), which serves IQ2_XXS and Q2_K only; this file states the same operator for the three formats of
 *     BASELINE configs 1 and 2.
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>

static float f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {                                   /* subnormal: normalise */
            int shift = 0;
            while (!(man & 0x400u)) { man <<= 1; ++shift; }
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static uint16_t load_u16(const uint8_t* p) { return (uint16_t)(p[0] | (p[1] << 8)); }

/* scale and min j (0..7) of a Q4_K / Q5_K header's 12 scale bytes */
static void scale_min_k4(const uint8_t* s, int j, int* sc, int* mn) {
    if (j < 4) {
        *sc = s[j] & 63;
        *mn = s[j + 4] & 63;
    } else {
        *sc = (s[j + 4] & 15) | ((s[j - 4] >> 6) << 4);
        *mn = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
    }
}

static float dot_q8_0(const uint8_t* row, const float* x, int k) {
    float acc = 0.0f;
    const int blocks = (k + 31) / 32;
    for (int b = 0; b < blocks; ++b) {
        const uint8_t* blk = row + (size_t)b * 34;
        const float d = f16_to_f32(load_u16(blk));
        const int8_t* q = (const int8_t*)(blk + 2);
        const int n = k - 32 * b < 32 ? k - 32 * b : 32;
        float part = 0.0f;
        for (int i = 0; i < n; ++i) part += (float)q[i] * x[32 * b + i];
        acc += d * part;
    }
    return acc;
}

/* five_bits != 0: Q5_K (176-byte blocks with 32 bytes of fifth bits ahead of the nibbles), else Q4_K (144-byte blocks) */
static float dot_q45_k(const uint8_t* row, const float* x, int k, int five_bits) {
    const int bb = five_bits ? 176 : 144;
    const int blocks = (k + 255) / 256;
    float acc = 0.0f;
    for (int b = 0; b < blocks; ++b) {
        const uint8_t* blk = row + (size_t)b * bb;
        const float d = f16_to_f32(load_u16(blk));
        const float dmin = f16_to_f32(load_u16(blk + 2));
        const uint8_t* scales = blk + 4;
        const uint8_t* qh = blk + 16;
        const uint8_t* qs = blk + (five_bits ? 48 : 16);
        for (int pair = 0; pair < 4; ++pair) {
            int sc0, mn0, sc1, mn1;
            scale_min_k4(scales, 2 * pair, &sc0, &mn0);
            scale_min_k4(scales, 2 * pair + 1, &sc1, &mn1);
            float dot0 = 0.0f, dot1 = 0.0f, sum0 = 0.0f, sum1 = 0.0f;
            const int base = 256 * b + 64 * pair;
            for (int i = 0; i < 32; ++i) {
                int lo = qs[32 * pair + i] & 15, hi = qs[32 * pair + i] >> 4;
                if (five_bits) {
                    lo += 16 * ((qh[i] >> (2 * pair)) & 1);
                    hi += 16 * ((qh[i] >> (2 * pair + 1)) & 1);
                }
                const float x0 = base + i < k ? x[base + i] : 0.0f;
                const float x1 = base + 32 + i < k ? x[base + 32 + i] : 0.0f;
                dot0 += (float)lo * x0; sum0 += x0;
                dot1 += (float)hi * x1; sum1 += x1;
            }
            acc += d * ((float)sc0 * dot0 + (float)sc1 * dot1) - dmin * ((float)mn0 * sum0 + (float)mn1 * sum1);
        }
    }
    return acc;
}

/* format: 0 = Q8_0 (34-byte blocks of 32), 3 = Q4_K, 4 = Q5_K (the type ids of src/loader/gguf/quant_types.py:3-13 for the
 * two super-block formats).  blocks: uint8 [n][blocks_per_row][block_bytes] row-major; x float32 [t][k]; y float32 [t][n].
 * Returns 0, or -1 for an unknown format. */
int rawblock_matvec_f32(const uint8_t* blocks, int format, const float* x, float* y, int t, int n, int k, int blocks_per_row) {
    int bb;
    if (format == 0) bb = 34;
    else if (format == 3) bb = 144;
    else if (format == 4) bb = 176;
    else return -1;
    const size_t row_bytes = (size_t)blocks_per_row * bb;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < n; ++r) {
        const uint8_t* row = blocks + (size_t)r * row_bytes;
        for (int tt = 0; tt < t; ++tt) {
            const float* xr = x + (size_t)tt * k;
            y[(size_t)tt * n + r] = format == 0 ? dot_q8_0(row, xr, k) : dot_q45_k(row, xr, k, format == 4);
        }
    }
    return 0;
}

/* float32 copy of a Q8_0 matrix (src/kernels/ops.py:734-741, q8_0_weight_dequantize): out [n][blocks_per_row * 32] */
void rawblock_q8_0_dequantize(const uint8_t* blocks, float* out, int n, int blocks_per_row) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < n; ++r)
        for (int b = 0; b < blocks_per_row; ++b) {
            const uint8_t* blk = blocks + ((size_t)r * blocks_per_row + b) * 34;
            const float d = f16_to_f32(load_u16(blk));
            const int8_t* q = (const int8_t*)(blk + 2);
            float* o = out + ((size_t)r * blocks_per_row + b) * 32;
            for (int i = 0; i < 32; ++i) o[i] = d * (float)q[i];
        }
}
