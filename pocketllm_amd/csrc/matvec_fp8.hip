// Decode matvec over FP8 E4M3 (OCP) weights with one scale per 128 x 128 block (float32, or IEEE
// fp16 bits with a row pitch for the scale table, the form the reference's C++ engine uploads), and
// the fused gate/up form y = silu(G x) * (U x) of the same kernels.
//
// One byte per weight, rows contiguous: a wave reads a row as a stream, lane l taking 16 bytes at
// offset 16 * (l + 64 * it) with one global_load_dwordx4, the current and the next pass in registers.  The
// activation row sits in LDS as float32 (no quantization on this path: y = x . (f32(code) * scale),
// the reference's dequantize-then-matmul statement).  Codes become floats with v_cvt_pk_f32_fp8,
// 16 FMAs per lane and chunk; a chunk lies inside one 128-wide scale block, so the block scale is
// applied once per chunk.  Row sums are 64-lane reductions.
#include "block_mfma.h"
#include "pllm_internal.h"
#include <algorithm>

namespace pllm {
namespace {

constexpr int kWaves = 4;
constexpr int kThreads = 64 * kWaves;
// register slots per wave: the fused gate/up form holds the same row of both matrices, the plain form one row (two rows per wave
// cost 0.8 us at 17408x5120: 19.6 against 18.9 us)
// (calls on several activation rows keep two rows per wave: 25.8 us against 29.5 at two rows)
template <bool SWIGLU, int R> constexpr int kSlots = (SWIGLU || R > 1) ? 2 : 1;

typedef float v2f __attribute__((ext_vector_type(2)));

// One weight matrix as the kernels see it: codes with a row pitch, scale table with a row pitch.
struct Fp8Mat {
    const uint8_t* w;
    const void* scale;      // float32, fp16 bits or bf16 bits, chosen by the kernels' F16S parameter
    size_t wstride;         // bytes between rows of codes
    int sstride;            // entries between rows of the scale table
};

// scale storage: 0 float32, 1 IEEE fp16 bits, 2 bf16 bits
template <int F16S>
__device__ __forceinline__ float scale_at(const void* __restrict__ scale, size_t i) {
    if constexpr (F16S == 1) return f16_bits_to_float(static_cast<const uint16_t*>(scale)[i]);
    else if constexpr (F16S == 2) return __uint_as_float(static_cast<uint32_t>(static_cast<const uint16_t*>(scale)[i]) << 16);
    else return static_cast<const float*>(scale)[i];
}

// a scale entry as loaded (no conversion yet, so that the load can stay in flight) and its value
template <int F16S>
__device__ __forceinline__ uint32_t scale_raw_at(const void* __restrict__ scale, size_t i) {
    if constexpr (F16S == 0) return __float_as_uint(static_cast<const float*>(scale)[i]);
    else return static_cast<const uint16_t*>(scale)[i];
}
template <int F16S>
__device__ __forceinline__ float scale_value(uint32_t raw) {
    if constexpr (F16S == 1) return f16_bits_to_float(raw);
    else if constexpr (F16S == 2) return __uint_as_float(raw << 16);
    else return __uint_as_float(raw);
}

__device__ __forceinline__ float silu(float v) { return v / (1.0f + __expf(-v)); }

// The activation row as float32 in LDS (k a multiple of 16 on the callers' path): four values per lane and trip, one vector
// load each where the row's alignment allows, all trips of a pass issued together.
__device__ __forceinline__ void stage_row_f32(float* xs, const void* __restrict__ x, int x_dtype, size_t xoff, int k) {
    const bool vec = x_dtype == PLLM_F32 ? ((reinterpret_cast<uintptr_t>(x) + 4 * xoff) & 15u) == 0
                                         : ((reinterpret_cast<uintptr_t>(x) + 2 * xoff) & 7u) == 0;
    constexpr int kBatch = 6;
    for (int base = static_cast<int>(threadIdx.x) * 4; base < k; base += kThreads * 4 * kBatch) {
        float v[kBatch][4];
#pragma unroll
        for (int j = 0; j < kBatch; ++j)
            if (base + j * kThreads * 4 < k) load_row4(v[j], x, x_dtype, xoff, base + j * kThreads * 4, k, vec);
#pragma unroll
        for (int j = 0; j < kBatch; ++j)
            if (base + j * kThreads * 4 < k) *reinterpret_cast<float4*>(xs + base + j * kThreads * 4) = make_float4(v[j][0], v[j][1], v[j][2], v[j][3]);
    }
}

// The first batch of stage_row_f32 in two halves, so that the row's loads can be issued ahead of the weight loads (loads return
// in order: a row requested after the weights would arrive after all of them) and stored once the weights are on their way.
constexpr int kStageBatch = 6;
__device__ __forceinline__ void stage_row_request(float (&v)[kStageBatch][4], const void* __restrict__ x, int x_dtype, size_t xoff, int k) {
    const bool vec = x_dtype == PLLM_F32 ? ((reinterpret_cast<uintptr_t>(x) + 4 * xoff) & 15u) == 0
                                         : ((reinterpret_cast<uintptr_t>(x) + 2 * xoff) & 7u) == 0;
    const int base = static_cast<int>(threadIdx.x) * 4;
#pragma unroll
    for (int j = 0; j < kStageBatch; ++j)
        if (base + j * kThreads * 4 < k) load_row4(v[j], x, x_dtype, xoff, base + j * kThreads * 4, k, vec);
}
__device__ __forceinline__ void stage_row_finish(float* xs, const float (&v)[kStageBatch][4], const void* __restrict__ x, int x_dtype, size_t xoff, int k) {
    const int base = static_cast<int>(threadIdx.x) * 4;
#pragma unroll
    for (int j = 0; j < kStageBatch; ++j)
        if (base + j * kThreads * 4 < k) *reinterpret_cast<float4*>(xs + base + j * kThreads * 4) = make_float4(v[j][0], v[j][1], v[j][2], v[j][3]);
    // rows longer than one batch: the rest the ordinary way
    const bool vec = x_dtype == PLLM_F32 ? ((reinterpret_cast<uintptr_t>(x) + 4 * xoff) & 15u) == 0
                                         : ((reinterpret_cast<uintptr_t>(x) + 2 * xoff) & 7u) == 0;
    for (int e0 = base + kStageBatch * kThreads * 4; e0 < k; e0 += kThreads * 4) {
        float t[4];
        load_row4(t, x, x_dtype, xoff, e0, k, vec);
        *reinterpret_cast<float4*>(xs + e0) = make_float4(t[0], t[1], t[2], t[3]);
    }
}

// Register slots of a wave: one row of the matrix, or (SWIGLU) the same row of the gate and of the up matrix.
template <bool SWIGLU>
__device__ __forceinline__ const Fp8Mat& slot_mat(const Fp8Mat& a, const Fp8Mat& b, int q) { return (SWIGLU && q == 1) ? b : a; }
// (plain form with two slots: the second slot's row lies rstride rows behind the first one's, in the workgroup's next group of rows)
__device__ __forceinline__ int slot_row(int row0, int q, int rstride, int n) { return min(row0 + q * rstride, n - 1); }

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

// The same with the 16 activations as the caller's bf16 / fp16 values (the row lies in LDS as it came from memory): the values are
// widened here, which costs vector instructions the kernel has to spare, and the row takes half the LDS reads.  Same products
// and the same summation order as chunk_dot, so the same bits.
template <bool BF16>
__device__ __forceinline__ float chunk_dot16(const uint4& w, const uint16_t* xp) {
    const uint4 xa = *reinterpret_cast<const uint4*>(xp);
    const uint4 xb = *reinterpret_cast<const uint4*>(xp + 8);
    auto lo = [](uint32_t u) { return BF16 ? __uint_as_float(u << 16) : f16_bits_to_float(u & 0xffffu); };
    auto hi = [](uint32_t u) { return BF16 ? __uint_as_float(u & 0xffff0000u) : f16_bits_to_float(u >> 16); };
    v2f a;
    float s;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.x), false); s = a.x * lo(xa.x); s += a.y * hi(xa.x);
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.x), true);  s += a.x * lo(xa.y); s += a.y * hi(xa.y);
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.y), false); s += a.x * lo(xa.z); s += a.y * hi(xa.z);
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.y), true);  s += a.x * lo(xa.w); s += a.y * hi(xa.w);
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.z), false); s += a.x * lo(xb.x); s += a.y * hi(xb.x);
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.z), true);  s += a.x * lo(xb.y); s += a.y * hi(xb.y);
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.w), false); s += a.x * lo(xb.z); s += a.y * hi(xb.z);
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.w), true);  s += a.x * lo(xb.w); s += a.y * hi(xb.w);
    return s;
}

// k a multiple of 16, weight base and row pitch 16-byte aligned.  Persistent: the grid is sized to be resident at once, a workgroup stages the activation
// row once and then walks groups of 4 weight rows (one per wave) in passes of 64 * 16 * ITERS bytes
// per row, always holding the loads of its next pass (of the same group or of its next group) in a
// second register set while it multiplies the current one.
// The block scales of a pass travel with its weights, requested ahead of them: loads return in order, so a scale asked for
// while the pass is multiplied would arrive behind the weights of the pass after it and hold the arithmetic until those are in.
template <int ITERS, int F16S, bool SWIGLU, int SLOTS>
__device__ __forceinline__ void fp8_fetch_pass(uint4 (&r)[SLOTS][ITERS], uint32_t (&sc)[SLOTS][ITERS], const Fp8Mat& ma, const Fp8Mat& mb,
                                               int row0, int rstride, int n, int chunks, int c0, int lane) {
#pragma unroll
    for (int q = 0; q < SLOTS; ++q) {
        const Fp8Mat& m = slot_mat<SWIGLU>(ma, mb, q);
        const size_t srow = static_cast<size_t>(slot_row(row0, q, rstride, n) >> 7) * m.sstride;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) sc[q][it] = scale_raw_at<F16S>(m.scale, srow + (min(c0 + it * 64 + lane, chunks - 1) >> 3));
    }
#pragma unroll
    for (int q = 0; q < SLOTS; ++q) {
        const uint8_t* wrow = slot_mat<SWIGLU>(ma, mb, q).w + static_cast<size_t>(slot_row(row0, q, rstride, n)) * slot_mat<SWIGLU>(ma, mb, q).wstride;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) r[q][it] = *reinterpret_cast<const uint4*>(wrow + 16 * min(c0 + it * 64 + lane, chunks - 1));
    }
}

// 16 codes as floats, converted once for all activation rows
__device__ __forceinline__ void chunk_floats(float (&f)[16], const uint4& w) {
    v2f a;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.x), false); f[0] = a.x; f[1] = a.y;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.x), true);  f[2] = a.x; f[3] = a.y;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.y), false); f[4] = a.x; f[5] = a.y;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.y), true);  f[6] = a.x; f[7] = a.y;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.z), false); f[8] = a.x; f[9] = a.y;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.z), true);  f[10] = a.x; f[11] = a.y;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.w), false); f[12] = a.x; f[13] = a.y;
    a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w.w), true);  f[14] = a.x; f[15] = a.y;
}

// the same summation order as chunk_dot
__device__ __forceinline__ float floats_dot(const float (&f)[16], const float* xp) {
    const float4 x0 = *reinterpret_cast<const float4*>(xp);
    const float4 x1 = *reinterpret_cast<const float4*>(xp + 4);
    const float4 x2 = *reinterpret_cast<const float4*>(xp + 8);
    const float4 x3 = *reinterpret_cast<const float4*>(xp + 12);
    float s = f[0] * x0.x; s += f[1] * x0.y; s += f[2] * x0.z; s += f[3] * x0.w;
    s += f[4] * x1.x; s += f[5] * x1.y; s += f[6] * x1.z; s += f[7] * x1.w;
    s += f[8] * x2.x; s += f[9] * x2.y; s += f[10] * x2.z; s += f[11] * x2.w;
    s += f[12] * x3.x; s += f[13] * x3.y; s += f[14] * x3.z; s += f[15] * x3.w;
    return s;
}

// R activation rows (xs holds them k floats apart) against the pass's weights: the codes are converted once per chunk
// XT: what xs holds: 0 / 3 float32 values, 1 bf16 and 2 fp16 values as they came from memory (one activation row only)
template <int ITERS, int F16S, bool SWIGLU, int R, int XT, int SLOTS>
__device__ __forceinline__ void fp8_multiply_pass(float (&acc)[SLOTS][R], const uint4 (&r)[SLOTS][ITERS],
                                                  const uint32_t (&scales)[SLOTS][ITERS], const float* xs, int k, int chunks, int c0, int lane) {
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int c = c0 + it * 64 + lane;
        const bool ok = c < chunks;
        const int cc = ok ? c : 0;
#pragma unroll
        for (int q = 0; q < SLOTS; ++q) {
            const float sc = scale_value<F16S>(scales[q][it]);
            if constexpr (R == 1) {
                float d;
                if constexpr (XT == 0 || XT == 3) d = chunk_dot(r[q][it], xs + 16 * cc);
                else d = chunk_dot16<XT == 1>(r[q][it], reinterpret_cast<const uint16_t*>(xs) + 16 * cc);
                acc[q][0] += ok ? d * sc : 0.0f;
            } else {
                float f[16];
                chunk_floats(f, r[q][it]);
#pragma unroll
                for (int a = 0; a < R; ++a) {
                    const float d = floats_dot(f, xs + static_cast<size_t>(a) * k + 16 * cc);
                    acc[q][a] += ok ? d * sc : 0.0f;
                }
            }
        }
    }
}

// activation rows arow0 .. arow0 + R - 1 (those below total_rows) of output row(s) row0
template <bool SWIGLU, int R, int SLOTS>
__device__ __forceinline__ void fp8_store_rows(float (&acc)[SLOTS][R], void* __restrict__ y, int y_dtype, size_t y_stride, int arow0, int total_rows,
                                               int row0, int rstride, int n, int lane) {
#pragma unroll
    for (int a = 0; a < R; ++a) {
        float total[SLOTS];
#pragma unroll
        for (int q = 0; q < SLOTS; ++q) { total[q] = group_sum<64>(acc[q][a]); acc[q][a] = 0.0f; }
        if (arow0 + a >= total_rows) continue;
        const size_t yoff = static_cast<size_t>(arow0 + a) * y_stride;
        if constexpr (SWIGLU) {
            if (lane == 0 && row0 < n) store_any(y, y_dtype, yoff + row0, silu(total[0]) * total[1]);
        } else {
#pragma unroll
            for (int q = 0; q < SLOTS; ++q)
                if (lane == 0 && row0 + q * rstride < n) store_any(y, y_dtype, yoff + row0 + q * rstride, total[q]);
        }
    }
}

template <int ITERS, int F16S, bool SWIGLU, bool LONG_ROWS, int R, int XT = 0>
__global__ __launch_bounds__(kThreads) void fp8_persistent_matvec_kernel(
    const void* __restrict__ x, int x_dtype, size_t x_stride, const Fp8Mat ma, const Fp8Mat mb,
    void* __restrict__ y, int y_dtype, size_t y_stride, int k, int n, int groups, int passes_of_long_rows, int total_rows) {
    const int passes = LONG_ROWS ? passes_of_long_rows : 1;                  // a constant for rows that fit one pass
    extern __shared__ __align__(16) unsigned char smem[];
    float* xs = reinterpret_cast<float*>(smem);                              // R activation rows, k floats apart
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int chunks = k >> 4;
    const int arow0 = blockIdx.y * R;                                        // this workgroup's first activation row
    constexpr int kPassChunks = 64 * ITERS;
    // A group = kWaves rows, one per wave, groups dealt round-robin over the workgroups.  SWIGLU: the wave's two slots hold its
    // row of the gate and of the up matrix.
    constexpr int rows_per_group = kWaves;
    const int wave_row = wave;
    // two plain slots: the wave's rows of this workgroup's current and next group (groups are dealt round-robin)
    constexpr bool kTwoPlain = !SWIGLU && kSlots<SWIGLU, R> == 2;
    const int step = kTwoPlain ? 2 * gridDim.x : gridDim.x;
    const int rstride = kTwoPlain ? rows_per_group * static_cast<int>(gridDim.x) : 0;

    uint4 a[kSlots<SWIGLU, R>][ITERS], b[kSlots<SWIGLU, R>][ITERS];
    uint32_t sa[kSlots<SWIGLU, R>][ITERS], sb[kSlots<SWIGLU, R>][ITERS];
    float acc[kSlots<SWIGLU, R>][R];
#pragma unroll
    for (int q = 0; q < kSlots<SWIGLU, R>; ++q)
#pragma unroll
        for (int r = 0; r < R; ++r) acc[q][r] = 0.0f;
    int g = blockIdx.x, p = 0;               // the pass being multiplied
    int gn = g, pn = 0;                      // the pass being fetched
    if constexpr (R == 1 && XT != 0) {
        // the row as it is (XT 1, 2: 16-bit values; 3: float32; row start on a 16-byte boundary) straight to LDS, requested ahead of
        // the weights; loads complete in order, so once no more than the pass's weight loads are outstanding the row (and the
        // pass's scales, which stand between them) has landed
        const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte_ptr)smem));
        constexpr int kValueBytes = XT == 3 ? 4 : 2;
        dma_share<kWaves>(static_cast<const unsigned char*>(x) + static_cast<size_t>(arow0) * x_stride * kValueBytes, lds0, k * kValueBytes, wave, lane);
        fp8_fetch_pass<ITERS, F16S, SWIGLU>(a, sa, ma, mb, g * rows_per_group + wave_row, rstride, n, chunks, 0, lane);
        wait_vm<ITERS * kSlots<SWIGLU, R>>();
    } else if constexpr (R == 1) {           // the activation row is requested first and stored once the weights are on their way
        float head[kStageBatch][4];
        const size_t xoff = static_cast<size_t>(arow0) * x_stride;
        stage_row_request(head, x, x_dtype, xoff, k);
        fp8_fetch_pass<ITERS, F16S, SWIGLU>(a, sa, ma, mb, g * rows_per_group + wave_row, rstride, n, chunks, 0, lane);
        stage_row_finish(xs, head, x, x_dtype, xoff, k);
    } else {
        fp8_fetch_pass<ITERS, F16S, SWIGLU>(a, sa, ma, mb, g * rows_per_group + wave_row, rstride, n, chunks, 0, lane);
#pragma unroll 1
        for (int r = 0; r < R; ++r)          // rows past the end: the last row again, result dropped
            stage_row_f32(xs + static_cast<size_t>(r) * k, x, x_dtype, static_cast<size_t>(min(arow0 + r, total_rows - 1)) * x_stride, k);
    }
    __syncthreads();
    while (g < groups) {
        if (++pn == passes) { pn = 0; gn += step; }
        // (fetched without a condition, past the last group its rows again: a branch around the loads would make the compiler wait
        // for them at the join, ahead of the arithmetic on the other register set)
        fp8_fetch_pass<ITERS, F16S, SWIGLU>(b, sb, ma, mb, min(gn, groups - 1) * rows_per_group + wave_row, rstride, n, chunks, pn * kPassChunks, lane);
        fp8_multiply_pass<ITERS, F16S, SWIGLU, R, XT>(acc, a, sa, xs, k, chunks, p * kPassChunks, lane);
        if (p == passes - 1) fp8_store_rows<SWIGLU, R>(acc, y, y_dtype, y_stride, arow0, total_rows, g * rows_per_group + wave_row, rstride, n, lane);
        g = gn; p = pn;
        if (g >= groups) break;
        if (++pn == passes) { pn = 0; gn += step; }
        fp8_fetch_pass<ITERS, F16S, SWIGLU>(a, sa, ma, mb, min(gn, groups - 1) * rows_per_group + wave_row, rstride, n, chunks, pn * kPassChunks, lane);
        fp8_multiply_pass<ITERS, F16S, SWIGLU, R, XT>(acc, b, sb, xs, k, chunks, p * kPassChunks, lane);
        if (p == passes - 1) fp8_store_rows<SWIGLU, R>(acc, y, y_dtype, y_stride, arow0, total_rows, g * rows_per_group + wave_row, rstride, n, lane);
        g = gn; p = pn;
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
template <int F16S, bool SWIGLU>
__global__ __launch_bounds__(kThreads) void fp8_generic_matvec_kernel(
    const void* __restrict__ x, int x_dtype, size_t x_stride, const Fp8Mat ma, const Fp8Mat mb,
    void* __restrict__ y, int y_dtype, size_t y_stride, int k, int n) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * kWaves + (threadIdx.x >> 6);
    const size_t xoff = static_cast<size_t>(blockIdx.y) * x_stride;
    float acc = 0.0f, acc_up = 0.0f;
    if (row < n) {
        const uint8_t* wrow = ma.w + static_cast<size_t>(row) * ma.wstride;
        for (int c = lane; c < k; c += 64) {
            const float xv = load_any(x, x_dtype, xoff + c);
            acc += xv * (fp8_to_float_sw(wrow[c]) * scale_at<F16S>(ma.scale, static_cast<size_t>(row >> 7) * ma.sstride + (c >> 7)));
            if constexpr (SWIGLU)
                acc_up += xv * (fp8_to_float_sw(mb.w[static_cast<size_t>(row) * mb.wstride + c]) *
                                scale_at<F16S>(mb.scale, static_cast<size_t>(row >> 7) * mb.sstride + (c >> 7)));
        }
    }
    acc = group_sum<64>(acc);
    if constexpr (SWIGLU) acc = silu(acc) * group_sum<64>(acc_up);
    if (lane == 0 && row < n) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * y_stride + row, acc);
}

// ------------------------------------------------------------------------------------------------
// Two to sixteen activation rows of bf16 or fp16 in one pass over the weights, on the matrix cores.
// E4M3 codes are exact in bf16 and in fp16 (v_cvt_scalef32_pk_{bf16,f16}_fp8 with scale 1), the activations go in as they are,
// products and sums are float32: v_mfma_f32_16x16x32_{bf16,f16} with A = 16 activation rows x 32 columns, B = 32 columns x 16
// weight rows, C[row 4 q .. 4 q + 3][weight row n] in lane (n, q).  A workgroup owns 16 or 32 weight rows (one or two tiles per wave);
// its eight or four waves split the row's 128-column scale blocks (wave v: blocks v, v + WAVES, ...).  Per block a lane loads its weight row's bytes [32 q, 32 q + 32)
// (whole cache lines per row) and, for each of the block's four MFMAs j, the activations of its row at columns 32 q + 8 j .. + 8 -
// the MFMA's column order is the lanes' own, the same on both sides.  The block's sum is scaled by the block scale and added to
// the wave's total; the waves meet in LDS.  The activations come from cache (16 rows x k x 2 bytes); they are requested one
// block ahead, the weights of a pass of up to kRows16Blocks blocks all at once.
// ------------------------------------------------------------------------------------------------
constexpr int kRows16Blocks = 5;                    // scale blocks per wave and pass
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef _Float16 v8hf __attribute__((ext_vector_type(8)));
typedef _Float16 v2hf __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));

template <bool BF16>
__device__ __forceinline__ v4f rows16_mfma(const uint4& a, uint32_t w_lo, uint32_t w_hi, v4f c) {
    if constexpr (BF16) {
        const v2bf p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w_lo, 1.0f, false), p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w_lo, 1.0f, true);
        const v2bf p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w_hi, 1.0f, false), p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w_hi, 1.0f, true);
        const v8bf b = {p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
        union { uint4 u; v8bf v; } av;
        av.u = a;
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(av.v, b, c, 0, 0, 0);
    } else {
        const v2hf p0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w_lo, 1.0f, false), p1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w_lo, 1.0f, true);
        const v2hf p2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w_hi, 1.0f, false), p3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w_hi, 1.0f, true);
        const v8hf b = {p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
        union { uint4 u; v8hf v; } av;
        av.u = a;
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(av.v, b, c, 0, 0, 0);
    }
}

// k a multiple of 128, weight base / pitch and activation base / pitch 16-byte aligned; grid (ceil(n / (16 TILES)), ceil(rows / 16)).
// TILES tiles of 16 weight rows per wave share the wave's activation operands.
template <int F16S, bool BF16, int TILES, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void fp8_rows16_matvec_kernel(
    const uint16_t* __restrict__ x, size_t x_stride, const Fp8Mat m, void* __restrict__ y, int y_dtype, size_t y_stride,
    int k, int n, int total_rows) {
    __shared__ float partial[WAVES][TILES][64][4];
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int col = lane & 15, q = lane >> 4;                                // B column (weight row) and A row (activation row); column quarter
    const int blocks = k >> 7;
    const int arow = min(static_cast<int>(blockIdx.y) * 16 + col, total_rows - 1);   // rows past the end: the last row again, result dropped
    const uint16_t* xp = x + static_cast<size_t>(arow) * x_stride + 32 * q;
    const uint8_t* wp[TILES];
    size_t srow[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        const int wrow = min((static_cast<int>(blockIdx.x) * TILES + t) * 16 + col, n - 1);
        wp[t] = m.w + static_cast<size_t>(wrow) * m.wstride + 32 * q;
        srow[t] = static_cast<size_t>(wrow >> 7) * m.sstride;
    }

    v4f total[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t) total[t] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    for (int b0 = wave; b0 < blocks; b0 += WAVES * kRows16Blocks) {
        uint4 wreg[kRows16Blocks][TILES][2];
        uint32_t sraw[kRows16Blocks][TILES];
#pragma unroll
        for (int i = 0; i < kRows16Blocks; ++i) {                            // (past the last block: that one again, not used)
            const int b = min(b0 + i * WAVES, blocks - 1);
#pragma unroll
            for (int t = 0; t < TILES; ++t) sraw[i][t] = scale_raw_at<F16S>(m.scale, srow[t] + b);
        }
#pragma unroll
        for (int i = 0; i < kRows16Blocks; ++i) {
            const int b = min(b0 + i * WAVES, blocks - 1);
#pragma unroll
            for (int t = 0; t < TILES; ++t) {
                wreg[i][t][0] = *reinterpret_cast<const uint4*>(wp[t] + 128 * b);
                wreg[i][t][1] = *reinterpret_cast<const uint4*>(wp[t] + 128 * b + 16);
            }
        }
        uint4 areg[2][4];
#pragma unroll
        for (int j = 0; j < 4; ++j) areg[0][j] = *reinterpret_cast<const uint4*>(xp + 128 * min(b0, blocks - 1) + 8 * j);
#pragma unroll
        for (int i = 0; i < kRows16Blocks; ++i) {
            if (i + 1 < kRows16Blocks) {
                const int bn = min(b0 + (i + 1) * WAVES, blocks - 1);
#pragma unroll
                for (int j = 0; j < 4; ++j) areg[(i + 1) & 1][j] = *reinterpret_cast<const uint4*>(xp + 128 * bn + 8 * j);
            }
            if (b0 + i * WAVES < blocks) {                                   // wave-uniform
#pragma unroll
                for (int t = 0; t < TILES; ++t) {
                    v4f c = {0.0f, 0.0f, 0.0f, 0.0f};
                    c = rows16_mfma<BF16>(areg[i & 1][0], wreg[i][t][0].x, wreg[i][t][0].y, c);
                    c = rows16_mfma<BF16>(areg[i & 1][1], wreg[i][t][0].z, wreg[i][t][0].w, c);
                    c = rows16_mfma<BF16>(areg[i & 1][2], wreg[i][t][1].x, wreg[i][t][1].y, c);
                    c = rows16_mfma<BF16>(areg[i & 1][3], wreg[i][t][1].z, wreg[i][t][1].w, c);
                    total[t] += c * scale_value<F16S>(sraw[i][t]);
                }
            }
        }
    }
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) partial[wave][t][lane][r] = total[t][r];
    __syncthreads();
    for (int e = tid; e < TILES * 256; e += 64 * WAVES) {
        const int t = e >> 8, l = (e >> 2) & 63, r = e & 3;
        float sum = 0.0f;
#pragma unroll
        for (int v = 0; v < WAVES; ++v) sum += partial[v][t][l][r];
        const int out_row = static_cast<int>(blockIdx.y) * 16 + 4 * (l >> 4) + r, out_col = (static_cast<int>(blockIdx.x) * TILES + t) * 16 + (l & 15);
        if (out_row < total_rows && out_col < n) store_any(y, y_dtype, static_cast<size_t>(out_row) * y_stride + out_col, sum);
    }
}

template <int F16S, bool BF16, int TILES, int WAVES>
int launch_rows16(const void* x, size_t x_stride, const Fp8Mat& ma, void* y, int y_dtype, size_t y_stride, int rows, int k, int n, hipStream_t stream) {
    const dim3 grid((n + 16 * TILES - 1) / (16 * TILES), (rows + 15) / 16);
    hipLaunchKernelGGL((fp8_rows16_matvec_kernel<F16S, BF16, TILES, WAVES>), grid, dim3(64 * WAVES), 0, stream, static_cast<const uint16_t*>(x), x_stride,
                       ma, y, y_dtype, y_stride, k, n, rows);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

// fp16 scale table with a row pitch -> dense float32 table (what the tile kernel reads)
__global__ __launch_bounds__(kThreads) void f16_scale_table_kernel(const uint16_t* __restrict__ src, int src_stride, float* __restrict__ dst,
                                                                   int table_rows, int table_cols) {
    const int i = blockIdx.x * kThreads + threadIdx.x;
    if (i < table_rows * table_cols) dst[i] = f16_bits_to_float(src[static_cast<size_t>(i / table_cols) * src_stride + i % table_cols]);
}

template <int F16S, bool SWIGLU>
int launch_any(const void* x, int x_dtype, size_t x_stride, const Fp8Mat& ma, const Fp8Mat& mb, void* y, int y_dtype, size_t y_stride,
               int rows, int k, int n, hipStream_t stream) {
    const bool aligned = (k % 16 == 0) && (static_cast<size_t>(k) * 4 <= 160 * 1024) &&
                         ((reinterpret_cast<uintptr_t>(ma.w) | ma.wstride) & 15u) == 0 &&
                         (!SWIGLU || ((reinterpret_cast<uintptr_t>(mb.w) | mb.wstride) & 15u) == 0);
    if (!aligned) {
        dim3 grid((n + kWaves - 1) / kWaves, rows);
        hipLaunchKernelGGL((fp8_generic_matvec_kernel<F16S, SWIGLU>), grid, dim3(kThreads), 0, stream, x, x_dtype, x_stride, ma, mb,
                           y, y_dtype, y_stride, k, n);
        return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
    }
    if constexpr (!SWIGLU)
        if (rows >= 2 && (x_dtype == PLLM_BF16 || x_dtype == PLLM_F16) && k % 128 == 0 &&
            ((reinterpret_cast<uintptr_t>(x) | (x_stride * 2)) & 15u) == 0) {
            // two tiles per wave halve the activation operands fetched per weight byte; they pay from 8 rows on, on long rows and
            // on matrices of few tiles (17408x5120 at 2 / 16 rows: 23.5 / 38.4 us with one tile and eight waves, 25.1 / 37.1 with two
            // and four; 5120x17408: 34.9 / 57.8 against 30.6 / 40.0)
            const bool two_tiles = rows >= 8 || k >= 8192 || n < 8192;
            if (two_tiles)
                return x_dtype == PLLM_BF16 ? launch_rows16<F16S, true, 2, 4>(x, x_stride, ma, y, y_dtype, y_stride, rows, k, n, stream)
                                            : launch_rows16<F16S, false, 2, 4>(x, x_stride, ma, y, y_dtype, y_stride, rows, k, n, stream);
            return x_dtype == PLLM_BF16 ? launch_rows16<F16S, true, 1, 8>(x, x_stride, ma, y, y_dtype, y_stride, rows, k, n, stream)
                                        : launch_rows16<F16S, false, 1, 8>(x, x_stride, ma, y, y_dtype, y_stride, rows, k, n, stream);
        }
    const int groups = (n + kWaves - 1) / kWaves;                            // one row per wave; a workgroup multiplies two groups at a time (SWIGLU: one, both matrices)
    const int niter = ((k >> 4) + 63) / 64;
    const int passes = (niter + 5) / 6;
    const int iters = (niter + passes - 1) / passes;
    // activation rows per workgroup: pairs from two rows on and fours from three on share one pass over the weights, as long as two
    // workgroups' rows fit LDS
    const int share = (rows >= 3 && static_cast<size_t>(k) * 4 * 4 <= 80 * 1024) ? 4 : (rows >= 2 && static_cast<size_t>(k) * 4 * 2 <= 80 * 1024) ? 2 : 1;
    const size_t smem = static_cast<size_t>(share) * k * sizeof(float);
    // persistent: the workgroups that fit a compute unit at once (two by registers, fewer when the activation rows fill LDS),
    // groups dealt round-robin
    const int per_cu = std::max(1, std::min(2, static_cast<int>((160 * 1024) / std::max<size_t>(smem, 1))));
    const int grid_x = std::min((!SWIGLU && share > 1) ? (groups + 1) / 2 : groups, per_cu * compute_units());
    const dim3 grid(grid_x, (rows + share - 1) / share);
    // (the form with the pass count as a variable needs 70 registers against 168 and is slower on rows of one pass: 21.5 against 18.9 us;
    // the form with a compile-time pass count keeps both register sets and all accumulators of several rows live at once and spills;
    // several activation rows always run the form with the pass count as a variable)
    // one activation row that starts on a 16-byte boundary goes to LDS as it is (rows of one pass): 1 bf16, 2 fp16, 3 float32
    const size_t value_bytes = x_dtype == PLLM_F32 ? 4 : 2;
    const int xt = (share == 1 && passes == 1 && ((reinterpret_cast<uintptr_t>(x) | (x_stride * value_bytes)) & 15u) == 0)
                       ? (x_dtype == PLLM_BF16 ? 1 : x_dtype == PLLM_F16 ? 2 : 3) : 0;
#define PLLM_LAUNCH(I, RR) { \
        auto kern = (passes > 1 || RR > 1) ? fp8_persistent_matvec_kernel<I, F16S, SWIGLU, true, RR> : fp8_persistent_matvec_kernel<I, F16S, SWIGLU, false, 1>; \
        if constexpr (RR == 1) { \
            if (xt == 1) kern = fp8_persistent_matvec_kernel<I, F16S, SWIGLU, false, 1, 1>; \
            else if (xt == 2) kern = fp8_persistent_matvec_kernel<I, F16S, SWIGLU, false, 1, 2>; \
            else if (xt == 3) kern = fp8_persistent_matvec_kernel<I, F16S, SWIGLU, false, 1, 3>; \
        } \
        if (smem > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, \
                                                    static_cast<int>(smem)) != hipSuccess) return PLLM_ERR_UNSUPPORTED; \
        hipLaunchKernelGGL(kern, grid, dim3(kThreads), smem, stream, x, x_dtype, x_stride, ma, mb, y, y_dtype, y_stride, k, n, groups, passes, rows); }
#define PLLM_PCASE(I) case I: if (share == 4) PLLM_LAUNCH(I, 4) else if (share == 2) PLLM_LAUNCH(I, 2) else PLLM_LAUNCH(I, 1) break;
    switch (iters) {
        PLLM_PCASE(1) PLLM_PCASE(2) PLLM_PCASE(3) PLLM_PCASE(4) PLLM_PCASE(5)
        default: PLLM_PCASE(6)
    }
#undef PLLM_PCASE
#undef PLLM_LAUNCH
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

}  // namespace

int fp8_matvec(const void* x, int x_dtype, const uint8_t* w, const float* scale, void* y, int y_dtype,
               int rows, int k, int n, hipStream_t stream) {
    const Fp8Mat m{w, scale, static_cast<size_t>(k), (k + 127) / 128};
    return launch_any<0, false>(x, x_dtype, static_cast<size_t>(k), m, m, y, y_dtype, static_cast<size_t>(n), rows, k, n, stream);
}

int fp8_f16scale_matvec(const void* x, int x_dtype, size_t x_stride, const uint8_t* w, const uint16_t* scale, size_t weight_stride,
                        int scale_stride, void* y, int y_dtype, size_t y_stride, int rows, int k, int n, hipStream_t stream) {
    const Fp8Mat m{w, scale, weight_stride, scale_stride};
    return launch_any<1, false>(x, x_dtype, x_stride, m, m, y, y_dtype, y_stride, rows, k, n, stream);
}

int fp8_bf16scale_matvec(const void* x, int x_dtype, size_t x_stride, const uint8_t* w, const uint16_t* scale, size_t weight_stride,
                         int scale_stride, void* y, int y_dtype, size_t y_stride, int rows, int k, int n, hipStream_t stream) {
    const Fp8Mat m{w, scale, weight_stride, scale_stride};
    return launch_any<2, false>(x, x_dtype, x_stride, m, m, y, y_dtype, y_stride, rows, k, n, stream);
}

int fp8_f16scale_table_to_f32(const uint16_t* scale, int scale_stride, float* out, int n, int k, hipStream_t stream) {
    const int tr = (n + 127) / 128, tc = (k + 127) / 128;
    hipLaunchKernelGGL(f16_scale_table_kernel, dim3((tr * tc + kThreads - 1) / kThreads), dim3(kThreads), 0, stream, scale, scale_stride, out, tr, tc);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

int fp8_f16scale_swiglu_matvec(const void* x, int x_dtype, size_t x_stride, const uint8_t* gate_w, const uint16_t* gate_scale,
                               const uint8_t* up_w, const uint16_t* up_scale, size_t weight_stride, int scale_stride,
                               void* y, int y_dtype, size_t y_stride, int rows, int k, int n, hipStream_t stream) {
    const Fp8Mat g{gate_w, gate_scale, weight_stride, scale_stride};
    const Fp8Mat u{up_w, up_scale, weight_stride, scale_stride};
    return launch_any<1, true>(x, x_dtype, x_stride, g, u, y, y_dtype, y_stride, rows, k, n, stream);
}

}  // namespace pllm
