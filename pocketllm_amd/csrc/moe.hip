// Routed experts over raw GGUF super-blocks: route grouping and the fused expert matmul
//     y[t] = sum over routes r of token t:  W2_e ( silu(W1_e x_t) * (W3_e x_t) * w_r ),   e = expert of r.
//
// Stages, all on one stream:
//   1. act_image_256 quantizes every token's activations once (two int8 terms per value).
//   2. moe_w13_kernel: one workgroup per (32 intermediate rows, route).  Waves 0/1 take the gate rows,
//      waves 2/3 the up rows, v_dot4 block dots against the token's image in LDS.  The epilogue
//      applies the clamp, SiLU and the route weight and QUANTIZES the 32 hidden values in place,
//      writing the route's hidden activations straight into the image format the down projection
//      reads: no float gate/up/hidden tensors are materialised.
//   3. the routed matvec of matvec_dot4.hip computes W2_e h_r per route into a float32 [R, D] scratch.
//   4. moe_reduce_kernel sums each token's routes in ascending route order: the result does not
//      depend on scheduling (the reference accumulates with atomicAdd).
#include <algorithm>

#include "block_dot4.h"
#include "pllm_internal.h"

namespace pllm {
// from this many tokens on, an expert's routes are multiplied as one tile matmul on the matrix cores
constexpr int kMoeGemmMinTokens = 16;
constexpr int kMoeTileMinRoutesPerExpert = 4;   // (128 experts top-8, 2048 -> 768, Q4_K: 66 / 117 us route by route at 16 / 32 tokens, ~175 / ~230 at 48 / 64, against 190 / 211 / 216 / 220 us as tile matmuls)
// up to this many routes per expert on average the grouped matrix-core kernels (cost per route: MFMAs and a short
// epilogue after one decode per expert; measured ~180 us + 0.5 us per route at 256 experts of 1536 x 3072) run ahead
// of the tile matmuls (cost per expert: the fp16 decode of every weight, ~1450 us for the same experts)
constexpr int kMoeGroupedMaxRoutesPerExpert = 8;
// The half-precision form with the routes as matrix rows pays a fixed price per expert that has routes at all (its decode costs
// more than the integer one, its multiply next to nothing): measured at 256 experts of 1536 x 3072 it overtakes the form above
// between 1 and 2 routes per expert (32 tokens, top 8: 375 vs 316 us; 64 tokens: 381 vs 472 us; 256 tokens: 500 vs 1126 us).
// It has no upper limit: an expert with more than 16 routes is decoded once per batch of 16, and that still beats the tile matmuls,
// which run every expert's few rows through 64-row tiles (256 experts, top 8, 512 / 1024 / 2048 / 4096 tokens: 0.97 / 1.41 / 2.39 /
// 4.37 ms against 2.85 / 4.57 / 7.25 / 8.50 ms, routing included).
constexpr int kMoeRowsMinRoutesPerExpertX2 = 3;

namespace {

constexpr int kW13Iters = 6;
constexpr int kW13Split = 2;               // waves that share one row's super-blocks in the per-route gate/up kernel

// Epilogue of one 32-row tile of one route, run by lanes 0..31 of a wave (lane = row inside the tile):
// clamp, SiLU, route weight, then the 32 hidden values are quantized in place into the image format
// the down projection reads (one activation group).
__device__ __forceinline__ void store_hidden(float g, float u, float limit, float route_weight, int i, int inter,
                                             unsigned char* img, int h_kpad, int lane) {
    if (limit > 0.0f) {
        u = fminf(fmaxf(u, -limit), limit);
        g = fminf(g, limit);
    }
    const float h = (i < inter) ? g / (1.0f + expf(-g)) * u * route_weight : 0.0f;
    float am = fabsf(h);
#pragma unroll
    for (int off = 1; off < 32; off <<= 1) am = fmaxf(am, __shfl_xor(am, off, 64));
    const float inv = am > 0.0f ? 127.0f / am : 0.0f;
    const float scale = am * (1.0f / 127.0f);
    const float q = fminf(fmaxf(rintf(h * inv), -127.0f), 127.0f);
    const float l = fminf(fmaxf(rintf((h - q * scale) * inv * 254.0f), -127.0f), 127.0f);
    float s16 = h;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) s16 += __shfl_xor(s16, off, 64);
    const float s32 = s16 + __shfl_xor(s16, 16, 64);
    if (i < h_kpad) {
        reinterpret_cast<int8_t*>(img)[i] = static_cast<int8_t>(static_cast<int>(q));
        reinterpret_cast<int8_t*>(img + h_kpad)[i] = static_cast<int8_t>(static_cast<int>(l));
        float2* gs = reinterpret_cast<float2*>(img + 2 * static_cast<size_t>(h_kpad));
        float* sum16 = reinterpret_cast<float*>(gs + h_kpad / 32);
        if ((lane & 15) == 0) sum16[i >> 4] = s16;
        if (lane == 0) gs[i >> 5] = make_float2(scale * kLoInv, s32);
    }
}


// Hidden images of the route-by-route path: h = SiLU(min(g, L)) * clamp(u, +-L) * route weight (the clamp only for L > 0)
// from the float32 gate and up products [routes, inter], quantized into the image the down projection reads.
__global__ __launch_bounds__(256) void swiglu_image_kernel(
    const float* __restrict__ gate, const float* __restrict__ up, const float* __restrict__ route_weights, float limit, int inter, int h_kpad,
    unsigned char* __restrict__ h_image, size_t h_stride) {
    const int e0 = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (e0 >= h_kpad) return;                                   // h_kpad is a multiple of 256: whole groups leave together
    const size_t r = blockIdx.y;
    unsigned char* base = h_image + r * h_stride;
    int8_t* hi = reinterpret_cast<int8_t*>(base);
    int8_t* lo = hi + h_kpad;
    float2* gs = reinterpret_cast<float2*>(lo + h_kpad);
    float* sum16 = reinterpret_cast<float*>(gs + h_kpad / 32);
    const float rw = route_weights[r];
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float h = 0.0f;
        if (e0 + i < inter) {
            float g = gate[r * inter + e0 + i], u = up[r * inter + e0 + i];
            if (limit > 0.0f) {
                u = fminf(fmaxf(u, -limit), limit);
                g = fminf(g, limit);
            }
            h = g / (1.0f + expf(-g)) * u * rw;
        }
        v[i] = h;
    }
    quantize4_to_image(v, e0, hi, lo, gs, sum16);
}


template <typename FMT>
__global__ __launch_bounds__(256 * kW13Split) void moe_w13_kernel(
    const unsigned char* __restrict__ x_image, size_t x_image_stride, int bpr,
    const int64_t* __restrict__ route_tokens, const int32_t* __restrict__ route_experts, const float* __restrict__ route_weights,
    const uint8_t* __restrict__ w1, const uint8_t* __restrict__ w3, int inter, float limit,
    unsigned char* __restrict__ h_image, size_t h_image_stride, int h_kpad,
    const void* __restrict__ x_raw, int x_dtype, int dim, const int64_t* __restrict__ route_experts64) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    const StagedX sx = carve_staged_x(smem, kpad);
    unsigned char* tables = smem + image_bytes;
    float* exch = reinterpret_cast<float*>(tables + FMT::kTableBytes);           // [kW13Split][2 matrices][32]

    const int route = blockIdx.y;
    const int64_t token = route_tokens ? route_tokens[route] : 0;
    // single-token calls skip the two helper launches: the expert ids are read as they come (int64)
    // and the workgroup quantizes the activation row into LDS itself (x_raw)
    const int expert = route_experts64 ? static_cast<int>(route_experts64[route]) : route_experts[route];
    const size_t expert_off = static_cast<size_t>(expert) * inter * bpr * FMT::kBlockBytes;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int j = lane & 3, team = lane >> 2;
    // 4 kW13Split waves: (matrix, half of the 32 rows, share of the super-blocks); more waves in
    // flight per row tile hide the latency of the codebook lookups
    const int mat = (wave >> 1) & 1;
    const int bhalf = wave >> 2;
    const int slot = 16 * (wave & 1) + team;                                     // 0..31 inside the tile
    const int row = min(blockIdx.x * 32 + slot, inter - 1);
    const uint8_t* wrow = (mat ? w3 : w1) + expert_off + static_cast<size_t>(row) * bpr * FMT::kBlockBytes;

    float acc = 0.0f;
    bool staged = false;
    for (int b0 = bhalf; b0 < bpr || !staged; b0 += kW13Split * kW13Iters) {
        typename FMT::Regs regs[kW13Iters];
#pragma unroll
        for (int it = 0; it < kW13Iters; ++it)
            FMT::load(regs[it], wrow + static_cast<size_t>(min(b0 + kW13Split * it, bpr - 1)) * FMT::kBlockBytes, j);
        if (!staged) {
            if (x_raw) quantize_row_to_lds(smem, x_raw, x_dtype, static_cast<size_t>(token) * dim, dim, kpad);
            else copy_to_lds(smem, x_image + static_cast<size_t>(token) * x_image_stride, image_bytes);
            FMT::stage_tables(tables);
            __syncthreads();
            staged = true;
        }
#pragma unroll
        for (int it = 0; it < kW13Iters; ++it)
            if (b0 + kW13Split * it < bpr) acc += FMT::lane_dot(regs[it], j, b0 + kW13Split * it, sx, tables);
    }
    acc += __shfl_xor(acc, 1, 64);
    acc += __shfl_xor(acc, 2, 64);
    if (j == 0) exch[bhalf * 64 + mat * 32 + slot] = acc;
    __syncthreads();
    float gsum = 0.0f, usum = 0.0f;
    if (tid < 32) {
#pragma unroll
        for (int v = 0; v < kW13Split; ++v) { gsum += exch[v * 64 + tid]; usum += exch[v * 64 + 32 + tid]; }
    }
    if (tid < 32) store_hidden(gsum, usum, limit, route_weights[route], blockIdx.x * 32 + tid, inter,
                               h_image + static_cast<size_t>(route) * h_image_stride, h_kpad, tid);
}

// Down projection of a single token with the sum over its routes inside the kernel:
//     y[row] = sum over routes r, in route order, of W2_{e_r}[row, :] . h_r
// One workgroup per 16 output rows; its waves split the routes and every expert row's super-blocks between them as
// in the dense matvec, the hidden images of all routes sit in LDS.  No partial buffer, no second launch.
// The sixteen waves' sums are added in wave order, so the result does not depend on scheduling.
constexpr int kSumWaves = 16;             // wave = (route mod 8, super-block parity)
constexpr int kSumIters = 4;

template <typename FMT>
__global__ __launch_bounds__(64 * kSumWaves) void moe_w2_sum_kernel(
    const unsigned char* __restrict__ h_image, size_t h_image_stride, int bpr, const int64_t* __restrict__ route_experts, int routes,
    const uint8_t* __restrict__ w2, size_t expert_stride, float* __restrict__ y, int dim) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    unsigned char* tables = smem + routes * image_bytes;
    float* partial = reinterpret_cast<float*>(tables + FMT::kTableBytes);        // [waves][16]

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int j = lane & 3, team = lane >> 2;
    const int row = blockIdx.x * 16 + team;
    const size_t row_off = static_cast<size_t>(row < dim ? row : 0) * bpr * FMT::kBlockBytes;

    for (int r = 0; r < routes; ++r) copy_to_lds(smem + r * image_bytes, h_image + static_cast<size_t>(r) * h_image_stride, image_bytes);
    FMT::stage_tables(tables);
    __syncthreads();

    float acc = 0.0f;
    for (int r = wave >> 1; r < routes; r += kSumWaves / 2) {
        const uint8_t* wrow = w2 + static_cast<size_t>(route_experts[r]) * expert_stride + row_off;
        const StagedX sx = carve_staged_x(smem + r * image_bytes, kpad);
        for (int b0 = wave & 1; b0 < bpr; b0 += 2 * kSumIters) {
            typename FMT::Regs regs[kSumIters];
#pragma unroll
            for (int it = 0; it < kSumIters; ++it)
                FMT::load(regs[it], wrow + static_cast<size_t>(min(b0 + 2 * it, bpr - 1)) * FMT::kBlockBytes, j);
#pragma unroll
            for (int it = 0; it < kSumIters; ++it)
                if (b0 + 2 * it < bpr) acc += FMT::lane_dot(regs[it], j, b0 + 2 * it, sx, tables);
        }
    }
    acc += __shfl_xor(acc, 1, 64);
    acc += __shfl_xor(acc, 2, 64);
    if (j == 0) partial[wave * 16 + team] = acc;
    __syncthreads();
    if (tid < 16) {
        float total = 0.0f;
#pragma unroll
        for (int v = 0; v < kSumWaves; ++v) total += partial[v * 16 + tid];
        const int out_row = blockIdx.x * 16 + tid;
        if (out_row < dim) y[out_row] = total;
    }
}

// ---- grouped forms: one workgroup per (row tile, expert) -----------------------------------------
// With many tokens an expert serves several routes.  The workgroup brings up to kRouteBatch of the
// expert's activation images into LDS and walks its rows' super-blocks kW13Iters at a time: every
// pass of weights in registers is multiplied with all routes of the batch, so the weights cross the
// memory system once per batch (for the usual handful of routes per expert: once per expert)
// instead of once per route.  Per-route sums collect in LDS between the passes.
constexpr int kRouteBatch = 8;

template <typename FMT>
__global__ __launch_bounds__(256) void moe_w13_grouped_kernel(
    const unsigned char* __restrict__ x_image, size_t x_image_stride, int bpr,
    const int64_t* __restrict__ route_tokens, const int32_t* __restrict__ seg, const float* __restrict__ route_weights,
    const uint8_t* __restrict__ w1, const uint8_t* __restrict__ w3, int inter, float limit,
    unsigned char* __restrict__ h_image, size_t h_image_stride, int h_kpad) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    unsigned char* tables = smem + kRouteBatch * image_bytes;
    float* exch = reinterpret_cast<float*>(tables + FMT::kTableBytes);           // [kRouteBatch][2][32]

    const int expert = blockIdx.y;
    const int r0 = seg[expert], r1 = seg[expert + 1];
    if (r0 >= r1) return;
    const size_t expert_off = static_cast<size_t>(expert) * inter * bpr * FMT::kBlockBytes;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int j = lane & 3, team = lane >> 2;
    const int mat = wave >> 1;
    const int slot = 16 * (wave & 1) + team;
    const int row = min(blockIdx.x * 32 + slot, inter - 1);
    const uint8_t* wrow = (mat ? w3 : w1) + expert_off + static_cast<size_t>(row) * bpr * FMT::kBlockBytes;
    FMT::stage_tables(tables);

    for (int rc = r0; rc < r1; rc += kRouteBatch) {
        const int nr = min(kRouteBatch, r1 - rc);
        for (int q = 0; q < nr; ++q)
            copy_to_lds(smem + q * image_bytes, x_image + static_cast<size_t>(route_tokens[rc + q]) * x_image_stride, image_bytes);
        __syncthreads();
        for (int b0 = 0; b0 < bpr; b0 += kW13Iters) {
            typename FMT::Regs regs[kW13Iters];
#pragma unroll
            for (int it = 0; it < kW13Iters; ++it)
                FMT::load(regs[it], wrow + static_cast<size_t>(min(b0 + it, bpr - 1)) * FMT::kBlockBytes, j);
            for (int q = 0; q < nr; ++q) {
                const StagedX sx = carve_staged_x(smem + q * image_bytes, kpad);
                float acc = 0.0f;
#pragma unroll
                for (int it = 0; it < kW13Iters; ++it)
                    if (b0 + it < bpr) acc += FMT::lane_dot(regs[it], j, b0 + it, sx, tables);
                acc += __shfl_xor(acc, 1, 64);
                acc += __shfl_xor(acc, 2, 64);
                if (j == 0) {                                                    // every (route, row) slot has one owner lane
                    float* dst = exch + q * 64 + mat * 32 + slot;
                    *dst = b0 == 0 ? acc : *dst + acc;
                }
            }
        }
        __syncthreads();
        for (int q = wave; q < nr; q += 4)
            if (lane < 32)
                store_hidden(exch[q * 64 + lane], exch[q * 64 + 32 + lane], limit, route_weights[rc + q], blockIdx.x * 32 + lane, inter,
                             h_image + static_cast<size_t>(rc + q) * h_image_stride, h_kpad, lane);
        __syncthreads();
    }
}

// partial[r, :] = W2_e h_r for the routes r of expert e = blockIdx.y; 64 rows per workgroup, one wave = 16 rows x all blocks
template <typename FMT>
__global__ __launch_bounds__(256) void moe_w2_grouped_kernel(
    const unsigned char* __restrict__ h_image, size_t h_image_stride, int bpr, const int32_t* __restrict__ seg,
    const uint8_t* __restrict__ w2, size_t expert_stride, float* __restrict__ partial, int dim) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    unsigned char* tables = smem + kRouteBatch * image_bytes;

    const int expert = blockIdx.y;
    const int r0 = seg[expert], r1 = seg[expert + 1];
    if (r0 >= r1) return;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int j = lane & 3, team = lane >> 2;
    const int row = blockIdx.x * 64 + wave * 16 + team;
    const uint8_t* wrow = w2 + static_cast<size_t>(expert) * expert_stride + static_cast<size_t>(min(row, dim - 1)) * bpr * FMT::kBlockBytes;
    FMT::stage_tables(tables);

    for (int rc = r0; rc < r1; rc += kRouteBatch) {
        const int nr = min(kRouteBatch, r1 - rc);
        for (int q = 0; q < nr; ++q)
            copy_to_lds(smem + q * image_bytes, h_image + static_cast<size_t>(rc + q) * h_image_stride, image_bytes);
        __syncthreads();
        for (int b0 = 0; b0 < bpr; b0 += kW13Iters) {
            typename FMT::Regs regs[kW13Iters];
#pragma unroll
            for (int it = 0; it < kW13Iters; ++it)
                FMT::load(regs[it], wrow + static_cast<size_t>(min(b0 + it, bpr - 1)) * FMT::kBlockBytes, j);
            for (int q = 0; q < nr; ++q) {
                const StagedX sx = carve_staged_x(smem + q * image_bytes, kpad);
                float acc = 0.0f;
#pragma unroll
                for (int it = 0; it < kW13Iters; ++it)
                    if (b0 + it < bpr) acc += FMT::lane_dot(regs[it], j, b0 + it, sx, tables);
                acc += __shfl_xor(acc, 1, 64);
                acc += __shfl_xor(acc, 2, 64);
                if (j == 0 && row < dim) {                                       // one owner lane per output: plain read-modify-write
                    float* dst = partial + static_cast<size_t>(rc + q) * dim + row;
                    *dst = b0 == 0 ? acc : *dst + acc;
                }
            }
        }
        __syncthreads();
    }
}

// seg_starts [E + 1] -> route_experts [R]
__global__ void expand_segments_kernel(const int32_t* __restrict__ seg, int32_t* __restrict__ route_experts, int n_experts) {
    const int e = blockIdx.x;
    if (e >= n_experts) return;
    for (int r = seg[e] + threadIdx.x; r < seg[e + 1]; r += blockDim.x) route_experts[r] = e;
}

__global__ void zero_fill_kernel(float* __restrict__ p, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.0f;
}

__global__ void narrow_experts_kernel(const int64_t* __restrict__ src, int32_t* __restrict__ dst, int routes) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r < routes) dst[r] = static_cast<int32_t>(src[r]);
}

// y[t, d] = sum_{r : route_tokens[r] == t} partial[r, d], ascending r.  grid (tokens, column groups): a workgroup owns the
// columns blockIdx.y * 256 + tid + k * gridDim.y * 256.  It first lists the routes of its token in LDS (the route table is read in
// pieces of 2048 routes, every thread a contiguous run of a piece; an exclusive scan of the per-thread counts keeps the list in
// route order), then adds them.  route_tokens == nullptr: a single token owns every route.
constexpr int kReduceList = 2048;
__global__ __launch_bounds__(256) void moe_reduce_kernel(const float* __restrict__ partial, const int64_t* __restrict__ route_tokens,
                                                         float* __restrict__ y, int routes, int dim) {
    __shared__ int list[kReduceList];
    __shared__ int wave_total[4];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int d0 = blockIdx.y * 256 + tid, dstep = gridDim.y * 256;
    if (!route_tokens) {
        for (int d = d0; d < dim; d += dstep) {
            float acc = 0.0f;
            for (int r = 0; r < routes; ++r) acc += partial[static_cast<size_t>(r) * dim + d];
            y[static_cast<size_t>(t) * dim + d] = acc;
        }
    } else {
        // The route table is scanned in pieces of kReduceList routes; a token's routes found so far stay listed in LDS in route
        // order.  (A token with more routes than the list holds - more than kReduceList experts - falls back to a scan per column.)
        int listed = 0;
        for (int c0 = 0; c0 < routes; c0 += kReduceList) {
            const int chunk = min(kReduceList, routes - c0);
            const int per = (chunk + 255) / 256;                             // at most kReduceList / 256 = 8
            const int r0 = c0 + min(tid * per, chunk), r1 = min(r0 + per, c0 + chunk);
            // the thread's run of the route table, all loads in flight together (past the run: the table's last entry, not counted)
            int64_t mine[kReduceList / 256];
#pragma unroll
            for (int i = 0; i < kReduceList / 256; ++i) mine[i] = route_tokens[min(r0 + i, routes - 1)];
            int cnt = 0;
#pragma unroll
            for (int i = 0; i < kReduceList / 256; ++i) cnt += (r0 + i < r1) && mine[i] == t;
            int incl = cnt;                                 // inclusive scan over the wave, then over the four waves
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const int v = __shfl_up(incl, off, 64);
                if ((tid & 63) >= off) incl += v;
            }
            __syncthreads();                                // the previous piece's totals have been read by everybody
            if ((tid & 63) == 63) wave_total[tid >> 6] = incl;
            __syncthreads();
            int pos = listed + incl - cnt, total = 0;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                if (w < (tid >> 6)) pos += wave_total[w];
                total += wave_total[w];
            }
#pragma unroll
            for (int i = 0; i < kReduceList / 256; ++i)
                if ((r0 + i < r1) && mine[i] == t) {
                    if (pos < kReduceList) list[pos] = r0 + i;
                    ++pos;
                }
            listed += total;
        }
        __syncthreads();
        if (listed <= kReduceList) {
            for (int d = d0; d < dim; d += dstep) {
                float acc = 0.0f;
                int i = 0;
                for (; i + 8 <= listed; i += 8) {                            // eight routes' values requested together, added in route order
                    float v[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) v[j] = partial[static_cast<size_t>(list[i + j]) * dim + d];
#pragma unroll
                    for (int j = 0; j < 8; ++j) acc += v[j];
                }
                for (; i < listed; ++i) acc += partial[static_cast<size_t>(list[i]) * dim + d];
                y[static_cast<size_t>(t) * dim + d] = acc;
            }
        } else {
            for (int d = d0; d < dim; d += dstep) {
                float acc = 0.0f;
                for (int r = 0; r < routes; ++r)
                    if (route_tokens[r] == t) acc += partial[static_cast<size_t>(r) * dim + d];
                y[static_cast<size_t>(t) * dim + d] = acc;
            }
        }
    }
}

// (with many tokens a workgroup takes several column groups, so that the route table is scanned by about a thousand workgroups at most)
int launch_moe_reduce(const float* partial, const int64_t* route_tokens, float* y, int64_t tokens, int routes, int dim, hipStream_t s) {
    const int col_groups = (dim + 255) / 256;
    const int per_token = static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(col_groups, 1024 / std::max<int64_t>(tokens, 1))));
    hipLaunchKernelGGL(moe_reduce_kernel, dim3(static_cast<unsigned>(tokens), static_cast<unsigned>(per_token)), dim3(256), 0, s, partial, route_tokens, y,
                       routes, dim);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

// ---- route grouping ---------------------------------------------------------------------------
// counts per local expert and exclusive prefix; one workgroup
__global__ __launch_bounds__(1024) void route_count_kernel(const void* __restrict__ indices, int idx_is_i64, int total, int start, int n_local,
                                                           int32_t* __restrict__ seg_starts) {
    extern __shared__ int32_t counts[];
    for (int e = threadIdx.x; e <= n_local; e += blockDim.x) counts[e] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < total; i += blockDim.x) {
        const int64_t ex = idx_is_i64 ? static_cast<const int64_t*>(indices)[i] : static_cast<const int32_t*>(indices)[i];
        const int64_t local = ex - start;
        if (local >= 0 && local < n_local) atomicAdd(&counts[local], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int32_t run = 0;
        for (int e = 0; e < n_local; ++e) {
            const int32_t c = counts[e];
            seg_starts[e] = run;
            run += c;
        }
        seg_starts[n_local] = run;
    }
}

// one wave per local expert: stable compaction of its (token, weight) pairs in (token, k) order
__global__ __launch_bounds__(64) void route_fill_kernel(const void* __restrict__ indices, int idx_is_i64, const float* __restrict__ weights,
                                                        int total, int topk, int start, const int32_t* __restrict__ seg_starts,
                                                        int64_t* __restrict__ route_tokens, float* __restrict__ route_weights,
                                                        int32_t* __restrict__ route_experts) {
    const int e = blockIdx.x;
    const int lane = threadIdx.x;
    int out = seg_starts[e];
    for (int base = 0; base < total; base += 64) {
        const int i = base + lane;
        bool hit = false;
        if (i < total) {
            const int64_t ex = idx_is_i64 ? static_cast<const int64_t*>(indices)[i] : static_cast<const int32_t*>(indices)[i];
            hit = (ex - start) == e;
        }
        const unsigned long long mask = __ballot(hit);
        if (hit) {
            const int pos = out + __popcll(mask & ((1ull << lane) - 1ull));
            route_tokens[pos] = i / topk;
            route_weights[pos] = weights[i];
            route_experts[pos] = e;
        }
        out += __popcll(mask);
    }
}

template <typename FMT>
int launch_w13(const unsigned char* x_image, size_t x_stride, int bpr, const int64_t* route_tokens, const int32_t* route_experts,
               const float* route_weights, const uint8_t* w1, const uint8_t* w3, int inter, float limit, unsigned char* h_image,
               size_t h_stride, int h_kpad, int routes, hipStream_t stream,
               const void* x_raw = nullptr, int x_dtype = 0, int dim = 0, const int64_t* route_experts64 = nullptr) {
    const size_t smem = staged_x_bytes(bpr * 256) + FMT::kTableBytes + kW13Split * 64 * sizeof(float);
    auto kern = moe_w13_kernel<FMT>;
    if (smem > 64 * 1024) {
        if (smem > 160 * 1024) return PLLM_ERR_UNSUPPORTED;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(smem)) != hipSuccess)
            return PLLM_ERR_UNSUPPORTED;
    }
    dim3 grid(h_kpad / 32, routes);
    hipLaunchKernelGGL(kern, grid, dim3(256 * kW13Split), smem, stream, x_image, x_stride, bpr, route_tokens, route_experts, route_weights, w1, w3,
                       inter, limit, h_image, h_stride, h_kpad, x_raw, x_dtype, dim, route_experts64);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

template <typename FMT>
int launch_w2_sum(const unsigned char* h_image, size_t h_stride, int bpr, const int64_t* route_experts64, int routes, const uint8_t* w2,
                  size_t expert_stride, float* y, int dim, hipStream_t stream) {
    const size_t smem = static_cast<size_t>(routes) * staged_x_bytes(bpr * 256) + FMT::kTableBytes + kSumWaves * 16 * sizeof(float);
    auto kern = moe_w2_sum_kernel<FMT>;
    if (smem > 64 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem)) != hipSuccess)
        return PLLM_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(kern, dim3((dim + 15) / 16), dim3(64 * kSumWaves), smem, stream, h_image, h_stride, bpr, route_experts64, routes, w2,
                       expert_stride, y, dim);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

template <typename FMT>
int launch_w13_grouped(const unsigned char* x_image, size_t x_stride, int bpr, const int64_t* route_tokens, const int32_t* seg,
                       const float* route_weights, const uint8_t* w1, const uint8_t* w3, int inter, float limit, unsigned char* h_image,
                       size_t h_stride, int h_kpad, int n_experts, hipStream_t stream) {
    const size_t smem = kRouteBatch * staged_x_bytes(bpr * 256) + FMT::kTableBytes + kRouteBatch * 64 * sizeof(float);
    auto kern = moe_w13_grouped_kernel<FMT>;
    if (smem > 160 * 1024) return PLLM_ERR_UNSUPPORTED;
    if (smem > 64 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem)) != hipSuccess)
        return PLLM_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(kern, dim3(h_kpad / 32, n_experts), dim3(256), smem, stream, x_image, x_stride, bpr, route_tokens, seg, route_weights,
                       w1, w3, inter, limit, h_image, h_stride, h_kpad);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

template <typename FMT>
int launch_w2_grouped(const unsigned char* h_image, size_t h_stride, int bpr, const int32_t* seg, const uint8_t* w2, size_t expert_stride,
                      float* partial, int dim, int n_experts, hipStream_t stream) {
    const size_t smem = kRouteBatch * staged_x_bytes(bpr * 256) + FMT::kTableBytes;
    auto kern = moe_w2_grouped_kernel<FMT>;
    if (smem > 160 * 1024) return PLLM_ERR_UNSUPPORTED;
    if (smem > 64 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem)) != hipSuccess)
        return PLLM_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(kern, dim3((dim + 63) / 64, n_experts), dim3(256), smem, stream, h_image, h_stride, bpr, seg, w2, expert_stride, partial, dim);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

bool dot4_type(int t) { return t == PLLM_TYPE_Q2_K || t == PLLM_TYPE_IQ2_XXS || t == PLLM_TYPE_IQ1_M; }

}  // namespace
}  // namespace pllm

extern "C" {

size_t pllm_gguf_moe_workspace_bytes(int64_t tokens, int64_t routes, int64_t dim, int64_t inter) {
    if (tokens <= 0 || routes < 0 || dim <= 0 || inter <= 0) return 0;
    const int bpr_x = static_cast<int>((dim + 255) / 256), bpr_h = static_cast<int>((inter + 255) / 256);
    // images of the tokens and of the routes' hidden rows, per-route outputs, narrow expert ids, and (route-by-route path of the
    // types without fused expert kernels) the float32 gate and up products
    size_t dot_path = pllm::act_image_256_bytes(bpr_x) * static_cast<size_t>(tokens) + pllm::act_image_256_bytes(bpr_h) * static_cast<size_t>(routes) +
                            pllm::align256(static_cast<size_t>(routes) * dim * sizeof(float)) + pllm::align256(static_cast<size_t>(routes) * sizeof(int32_t)) +
                            2 * pllm::align256(static_cast<size_t>(routes) * inter * sizeof(float)) + 256;
    // (the grouped path with the routes as matrix rows: half-precision activation rows and hidden rows, per-route outputs)
    const size_t rows_path = pllm::moe_rows_x_bytes(tokens, dim) + pllm::moe_rows_h_bytes(routes, inter) +
                             pllm::align256(static_cast<size_t>(routes) * dim * sizeof(float)) + 256;
    if (rows_path > dot_path) dot_path = rows_path;
    if (tokens < pllm::kMoeGemmMinTokens || routes > INT32_MAX) return dot_path;
    const int R = static_cast<int>(routes);
    const size_t tile_path = pllm::gemm_f16_staged_bytes(R, bpr_x) + pllm::gemm_f16_staged_bytes(R, bpr_h) +
                             2 * pllm::align256(static_cast<size_t>(routes) * inter * sizeof(float)) +
                             pllm::align256(static_cast<size_t>(routes) * dim * sizeof(float)) + 256;
    return dot_path > tile_path ? dot_path : tile_path;
}

int pllm_gguf_moe_single_token_accumulate(const void* x, int x_dtype, int64_t dim, int64_t inter, const int64_t* route_experts,
                                          const float* route_weights, int64_t routes, const uint8_t* w1, const uint8_t* w3, int w13_type,
                                          const uint8_t* w2, int w2_type, float swiglu_limit, void* y, int y_dtype, void* workspace,
                                          size_t workspace_bytes, void* stream) {
    using namespace pllm;
    if (!x || !y || dim <= 0 || inter <= 0 || routes < 0) return PLLM_ERR_INVALID_ARGUMENT;
    if (x_dtype != PLLM_F32 && x_dtype != PLLM_F16 && x_dtype != PLLM_BF16) return PLLM_ERR_INVALID_ARGUMENT;
    if (y_dtype != PLLM_F32 && y_dtype != PLLM_F16 && y_dtype != PLLM_BF16) return PLLM_ERR_INVALID_ARGUMENT;
    if (routes == 0) return PLLM_OK;                                          // nothing to add
    if (!w1 || !w3 || !w2 || !route_weights || !route_experts) return PLLM_ERR_INVALID_ARGUMENT;
    if (routes > 65535 || dim > (1 << 24) || inter > (1 << 24)) return PLLM_ERR_UNSUPPORTED;
    if (!workspace || workspace_bytes < pllm_gguf_moe_workspace_bytes(1, routes, dim, inter)) return PLLM_ERR_WORKSPACE;
    const int bpr_h = static_cast<int>((inter + 255) / 256);
    const int R = static_cast<int>(routes), I = static_cast<int>(inter), D = static_cast<int>(dim);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t h_stride = act_image_256_bytes(bpr_h);
    if ((!dot4_type(w13_type) || !dot4_type(w2_type)) && pllm_gguf_block_bytes(w13_type) != 0) {
        // types without fused expert kernels: gate and up as one launch of the routed wave kernels, then the down projection with the
        // routes as its waves, which adds the ordered sum into y itself (the workspace layout of pllm_gguf_moe_forward's same path)
        const int bpr_x = static_cast<int>((dim + 255) / 256);
        const size_t stride2 = static_cast<size_t>(dim) * bpr_h * pllm_gguf_block_bytes(w2_type);
        if (!kquant_route_sum_supports(w2_type, R, I, w2, stride2)) return PLLM_ERR_UNSUPPORTED;
        unsigned char* p = static_cast<unsigned char*>(workspace);
        p += act_image_256_bytes(bpr_x) + h_stride * routes + align256(static_cast<size_t>(routes) * dim * sizeof(float)) +
             align256(static_cast<size_t>(routes) * sizeof(int32_t));
        float* gate = reinterpret_cast<float*>(p);  p += align256(static_cast<size_t>(routes) * inter * sizeof(float));
        float* up = reinterpret_cast<float*>(p);
        WeightRoute r13{};
        r13.expert64 = route_experts;
        WeightRoute r2 = r13;
        r13.expert_stride = static_cast<size_t>(inter) * bpr_x * pllm_gguf_block_bytes(w13_type);
        r13.extra = 1;
        r13.more_w[0] = w3;
        r13.more_y[0] = up;
        r13.more_n[0] = I;
        r2.expert_stride = stride2;
        ActRows xa = act_rows_raw(x, x_dtype, D);
        xa.x_broadcast = 1;
        const int st = superblock_matvec(xa, w1, w13_type, gate, PLLM_F32, R, I, bpr_x, s, r13);
        if (st != PLLM_OK) return st;
        return kquant_route_sum_matvec(gate, up, route_weights, swiglu_limit, I, r2, w2, w2_type, y, y_dtype | kAccumulateInto, D, bpr_h, R, s);
    }
    if (routes * staged_x_bytes(bpr_h * 256) > 96 * 1024 || !moe_single_mfma_supports(w13_type, w2_type, D, I, R, x, w1, w3, w2))
        return PLLM_ERR_UNSUPPORTED;
    unsigned char* himg = static_cast<unsigned char*>(workspace);
    const int st = moe_single_w13_mfma(x, x_dtype, D, route_experts, route_weights, R, w1, w3, w13_type, I, swiglu_limit, himg, h_stride, s);
    if (st != PLLM_OK) return st;
    return moe_single_w2_mfma(himg, h_stride, I, route_experts, R, w2, nullptr, D, s, y, y_dtype);
}

int pllm_gguf_moe_forward(const void* x, int x_dtype, int64_t tokens, int64_t dim, int64_t inter,
                          const int64_t* route_tokens, const int64_t* route_experts, const int32_t* seg_starts, int64_t n_experts,
                          const float* route_weights, int64_t routes,
                          const uint8_t* w1, const uint8_t* w3, int w13_type, const uint8_t* w2, int w2_type,
                          float swiglu_limit, float* y, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace pllm;
    if (!x || !y || tokens <= 0 || dim <= 0 || inter <= 0 || routes < 0 || n_experts <= 0) return PLLM_ERR_INVALID_ARGUMENT;
    if (x_dtype != PLLM_F32 && x_dtype != PLLM_F16 && x_dtype != PLLM_BF16) return PLLM_ERR_INVALID_ARGUMENT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (routes == 0) {
        const size_t count = static_cast<size_t>(tokens) * dim;                // a kernel, not a memset: callers may capture graphs
        hipLaunchKernelGGL(zero_fill_kernel, dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0, s, y, count);
        return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
    }
    if (!w1 || !w3 || !w2 || !route_weights || (!route_experts && !seg_starts)) return PLLM_ERR_INVALID_ARGUMENT;
    if (pllm_gguf_block_bytes(w13_type) == 0 || pllm_gguf_block_bytes(w2_type) == 0) return PLLM_ERR_UNSUPPORTED;
    if (tokens > 65535 || routes > 65535 || dim > (1 << 24) || inter > (1 << 24)) return PLLM_ERR_UNSUPPORTED;
    if (tokens > 1 && !route_tokens) return PLLM_ERR_INVALID_ARGUMENT;
    if (!workspace || workspace_bytes < pllm_gguf_moe_workspace_bytes(tokens, routes, dim, inter)) return PLLM_ERR_WORKSPACE;

    const int bpr_x = static_cast<int>((dim + 255) / 256), bpr_h = static_cast<int>((inter + 255) / 256);
    if (seg_starts && tokens > 1 && 2 * routes >= kMoeRowsMinRoutesPerExpertX2 * n_experts &&
        moe_rows_supports(w13_type, w2_type, static_cast<int>(dim), static_cast<int>(inter), w1, w3, w2)) {
        // a few routes per expert, IQ2_XXS / IQ1_M: every expert's weights are decoded once, in half precision, and multiplied with
        // all its routes at once on the matrix cores
        unsigned char* x_rows = static_cast<unsigned char*>(workspace);
        unsigned char* h_rows = x_rows + moe_rows_x_bytes(tokens, dim);
        float* part = reinterpret_cast<float*>(h_rows + moe_rows_h_bytes(routes, inter));
        const int R = static_cast<int>(routes), E = static_cast<int>(n_experts), I = static_cast<int>(inter), D = static_cast<int>(dim);
        int st = moe_rows_w13(x, x_dtype, static_cast<int>(tokens), D, x_rows, route_tokens, seg_starts, route_weights, w1, w3, I, swiglu_limit, h_rows, E, R, s);
        if (st != PLLM_OK) return st;
        st = moe_rows_w2(h_rows, I, seg_starts, w2, part, D, E, R, s);
        if (st != PLLM_OK) return st;
        return launch_moe_reduce(part, route_tokens, y, tokens, R, D, s);
    }
    if (seg_starts && tokens > 1 && routes <= kMoeGroupedMaxRoutesPerExpert * n_experts &&
        moe_grouped_mfma_supports(w13_type, w2_type, static_cast<int>(dim), static_cast<int>(inter), w1, w3, w2)) {
        // a few routes per expert: every expert's weights are decoded once on the matrix-core path and all its routes pass
        // through; same workspace layout as the v_dot4 forms below
        const size_t xs = act_image_256_bytes(bpr_x), hs = act_image_256_bytes(bpr_h);
        unsigned char* x_img = static_cast<unsigned char*>(workspace);
        unsigned char* h_img = x_img + xs * tokens;
        float* part = reinterpret_cast<float*>(h_img + hs * routes);
        const int R = static_cast<int>(routes), E = static_cast<int>(n_experts), I = static_cast<int>(inter), D = static_cast<int>(dim);
        int st = act_image_256(x, x_dtype, static_cast<int>(tokens), D, bpr_x, x_img, s);
        if (st != PLLM_OK) return st;
        st = moe_grouped_w13_mfma(x_img, xs, D, route_tokens, seg_starts, route_weights, w1, w3, w13_type, I, swiglu_limit, h_img, hs, E, s);
        if (st != PLLM_OK) return st;
        st = moe_grouped_w2_mfma(h_img, hs, I, seg_starts, w2, part, D, E, s);
        if (st != PLLM_OK) return st;
        return launch_moe_reduce(part, route_tokens, y, tokens, R, D, s);
    }
    // (types without fused expert kernels: the tile path decodes every touched expert's three matrices whatever its route count, so
    // below kMoeTileMinRoutesPerExpert routes per expert on average the route-by-route path below stays cheaper)
    const bool few_routes_each = (!dot4_type(w13_type) || !dot4_type(w2_type)) && routes < static_cast<int64_t>(kMoeTileMinRoutesPerExpert) * n_experts;
    if (seg_starts && tokens >= kMoeGemmMinTokens && !few_routes_each) {
        // tile path: gather the routes' activation rows as fp16, gate and up as two batches of tile
        // matmuls (one group per expert), SwiGLU into fp16 hidden rows, down as a third batch, then
        // the ordered sum of every token's routes
        const int R = static_cast<int>(routes), E = static_cast<int>(n_experts), I = static_cast<int>(inter), D = static_cast<int>(dim);
        unsigned char* p = static_cast<unsigned char*>(workspace);
        void* x_staged = p;  p += gemm_f16_staged_bytes(R, bpr_x);
        void* h_staged = p;  p += gemm_f16_staged_bytes(R, bpr_h);
        float* gate = reinterpret_cast<float*>(p);  p += align256(static_cast<size_t>(R) * I * sizeof(float));
        float* up = reinterpret_cast<float*>(p);    p += align256(static_cast<size_t>(R) * I * sizeof(float));
        float* part = reinterpret_cast<float*>(p);
        const int max_group = static_cast<int>(tokens < routes ? tokens : routes);       // an expert sees a token at most once
        const size_t stride13 = static_cast<size_t>(inter) * bpr_x * pllm_gguf_block_bytes(w13_type);
        const size_t stride2 = static_cast<size_t>(dim) * bpr_h * pllm_gguf_block_bytes(w2_type);
        int st = gemm_f16_stage_rows(x, x_dtype, route_tokens, R, D, bpr_x, x_staged, s);
        if (st != PLLM_OK) return st;
        st = gemm_f16_grouped(x_staged, w1, w13_type, stride13, seg_starts, E, gate, R, max_group, I, bpr_x, s);
        if (st != PLLM_OK) return st;
        st = gemm_f16_grouped(x_staged, w3, w13_type, stride13, seg_starts, E, up, R, max_group, I, bpr_x, s);
        if (st != PLLM_OK) return st;
        st = gemm_f16_stage_swiglu(gate, up, route_weights, swiglu_limit, R, I, bpr_h, h_staged, s);
        if (st != PLLM_OK) return st;
        st = gemm_f16_grouped(h_staged, w2, w2_type, stride2, seg_starts, E, part, R, max_group, D, bpr_h, s);
        if (st != PLLM_OK) return st;
        return launch_moe_reduce(part, route_tokens, y, tokens, R, D, s);
    }
    const size_t x_stride = act_image_256_bytes(bpr_x), h_stride = act_image_256_bytes(bpr_h);
    if (!dot4_type(w13_type) || !dot4_type(w2_type)) {
        // Types without fused expert kernels (Q4_K, Q5_K, Q6_K, IQ4_XS, IQ2_XS, IQ3_XXS), below the tile path's token count: route
        // by route through the dense decode kernels in their routed form (grid row = route, matrix = the route's expert, activation
        // row = the route's token, quantized inside the kernel): gate and up as one launch (grid.z picks the matrix), SwiGLU into
        // hidden images, down, ordered sum per token.  Four launches for one token (its int64 expert numbers are read as they are;
        // the SwiGLU inside the down projection's activation quantizer instead of a launch of its own ran 22.3 us against 20.4 in
        // the route-per-workgroup form), two where the down format has the routes-as-waves form.
        unsigned char* p = static_cast<unsigned char*>(workspace);
        p += x_stride * tokens;                                              // (the activation images of the layout: unused here)
        unsigned char* h_image = p;  p += h_stride * routes;
        float* partial = reinterpret_cast<float*>(p);  p += align256(static_cast<size_t>(routes) * dim * sizeof(float));
        int32_t* experts32 = reinterpret_cast<int32_t*>(p);  p += align256(static_cast<size_t>(routes) * sizeof(int32_t));
        float* gate = reinterpret_cast<float*>(p);  p += align256(static_cast<size_t>(routes) * inter * sizeof(float));
        float* up = reinterpret_cast<float*>(p);
        const int R = static_cast<int>(routes), I = static_cast<int>(inter), D = static_cast<int>(dim);
        WeightRoute r13{};
        if (route_experts) {
            r13.expert64 = route_experts;
        } else {
            hipLaunchKernelGGL(expand_segments_kernel, dim3(static_cast<unsigned>(n_experts)), dim3(256), 0, s, seg_starts, experts32, static_cast<int>(n_experts));
            if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
            r13.expert = experts32;
        }
        // one token: every route reads row 0; several: the route's token picks the row
        ActRows xa = act_rows_raw(x, x_dtype, D);
        xa.row_token = tokens > 1 ? route_tokens : nullptr;
        xa.x_broadcast = tokens > 1 ? 0 : 1;
        WeightRoute r2 = r13;
        r13.expert_stride = static_cast<size_t>(inter) * bpr_x * pllm_gguf_block_bytes(w13_type);
        r13.extra = 1;
        r13.more_w[0] = w3;
        r13.more_y[0] = up;
        r13.more_n[0] = I;
        r2.expert_stride = static_cast<size_t>(dim) * bpr_h * pllm_gguf_block_bytes(w2_type);
        int st = superblock_matvec(xa, w1, w13_type, gate, PLLM_F32, R, I, bpr_x, s, r13);
        if (st != PLLM_OK) return st;
        if (tokens == 1) {
            // one token, a down format of the single-launch wave kernels: the routes are the waves of a workgroup, which form their
            // hidden slices from the gate and up products themselves and meet in the ordered sum (two launches in all)
            const int st2 = kquant_route_sum_matvec(gate, up, route_weights, swiglu_limit, I, r2, w2, w2_type, y, PLLM_F32, D, bpr_h, R, s);
            if (st2 != PLLM_ERR_UNSUPPORTED) return st2;
        }
        const int h_kpad = bpr_h * 256;
        hipLaunchKernelGGL(swiglu_image_kernel, dim3((h_kpad / 4 + 255) / 256, R), dim3(256), 0, s, gate, up, route_weights, swiglu_limit, I, h_kpad,
                           h_image, h_stride);
        if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
        st = superblock_matvec(act_rows_from_image(h_image, h_stride), w2, w2_type, partial, PLLM_F32, R, D, bpr_h, s, r2);
        if (st != PLLM_OK) return st;
        return launch_moe_reduce(partial, tokens > 1 ? route_tokens : nullptr, y, tokens, R, D, s);
    }
    if (tokens == 1 && route_experts && routes * staged_x_bytes(bpr_h * 256) <= 96 * 1024) {
        // single token: two launches.  Gate/up read the raw activation row and the int64 expert ids
        // themselves; the down projection sums the routes in order inside the kernel.
        unsigned char* himg = static_cast<unsigned char*>(workspace);
        const int R1 = static_cast<int>(routes), I1 = static_cast<int>(inter), D1 = static_cast<int>(dim);
        if (moe_single_mfma_supports(w13_type, w2_type, D1, I1, R1, x, w1, w3, w2)) {
            const int st = moe_single_w13_mfma(x, x_dtype, D1, route_experts, route_weights, R1, w1, w3, w13_type, I1, swiglu_limit, himg, h_stride, s);
            if (st != PLLM_OK) return st;
            return moe_single_w2_mfma(himg, h_stride, I1, route_experts, R1, w2, y, D1, s);
        }
        int st1;
        switch (w13_type) {
            case PLLM_TYPE_IQ2_XXS: st1 = launch_w13<IQ2XXS>(nullptr, 0, bpr_x, nullptr, nullptr, route_weights, w1, w3, I1, swiglu_limit, himg, h_stride, bpr_h * 256, R1, s, x, x_dtype, D1, route_experts); break;
            case PLLM_TYPE_IQ1_M: st1 = launch_w13<IQ1M>(nullptr, 0, bpr_x, nullptr, nullptr, route_weights, w1, w3, I1, swiglu_limit, himg, h_stride, bpr_h * 256, R1, s, x, x_dtype, D1, route_experts); break;
            default: st1 = launch_w13<Q2K>(nullptr, 0, bpr_x, nullptr, nullptr, route_weights, w1, w3, I1, swiglu_limit, himg, h_stride, bpr_h * 256, R1, s, x, x_dtype, D1, route_experts); break;
        }
        if (st1 != PLLM_OK) return st1;
        const size_t stride2 = static_cast<size_t>(dim) * bpr_h * pllm_gguf_block_bytes(w2_type);
        switch (w2_type) {
            case PLLM_TYPE_IQ2_XXS: return launch_w2_sum<IQ2XXS>(himg, h_stride, bpr_h, route_experts, R1, w2, stride2, y, D1, s);
            case PLLM_TYPE_IQ1_M: return launch_w2_sum<IQ1M>(himg, h_stride, bpr_h, route_experts, R1, w2, stride2, y, D1, s);
            default: return launch_w2_sum<Q2K>(himg, h_stride, bpr_h, route_experts, R1, w2, stride2, y, D1, s);
        }
    }
    unsigned char* ws = static_cast<unsigned char*>(workspace);
    unsigned char* x_image = ws;
    unsigned char* h_image = x_image + x_stride * tokens;
    float* partial = reinterpret_cast<float*>(h_image + h_stride * routes);
    int32_t* experts32 = reinterpret_cast<int32_t*>(reinterpret_cast<unsigned char*>(partial) + align256(static_cast<size_t>(routes) * dim * sizeof(float)));
    const int R = static_cast<int>(routes);

    if (route_experts) {
        hipLaunchKernelGGL(narrow_experts_kernel, dim3((R + 255) / 256), dim3(256), 0, s, route_experts, experts32, R);
    } else {
        hipLaunchKernelGGL(expand_segments_kernel, dim3(static_cast<unsigned>(n_experts)), dim3(256), 0, s, seg_starts, experts32,
                           static_cast<int>(n_experts));
    }
    if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
    int st = act_image_256(x, x_dtype, static_cast<int>(tokens), static_cast<int>(dim), bpr_x, x_image, s);
    if (st != PLLM_OK) return st;

    const int I = static_cast<int>(inter);
    const bool grouped = seg_starts && tokens > 1;                 // several routes per expert: weights once per batch of routes
    if (grouped) {
        const int E = static_cast<int>(n_experts);
        switch (w13_type) {
            case PLLM_TYPE_IQ2_XXS: st = launch_w13_grouped<IQ2XXS>(x_image, x_stride, bpr_x, route_tokens, seg_starts, route_weights, w1, w3, I, swiglu_limit, h_image, h_stride, bpr_h * 256, E, s); break;
            case PLLM_TYPE_IQ1_M: st = launch_w13_grouped<IQ1M>(x_image, x_stride, bpr_x, route_tokens, seg_starts, route_weights, w1, w3, I, swiglu_limit, h_image, h_stride, bpr_h * 256, E, s); break;
            default: st = launch_w13_grouped<Q2K>(x_image, x_stride, bpr_x, route_tokens, seg_starts, route_weights, w1, w3, I, swiglu_limit, h_image, h_stride, bpr_h * 256, E, s); break;
        }
        if (st != PLLM_OK) return st;
        const size_t stride2 = static_cast<size_t>(dim) * bpr_h * pllm_gguf_block_bytes(w2_type);
        switch (w2_type) {
            case PLLM_TYPE_IQ2_XXS: st = launch_w2_grouped<IQ2XXS>(h_image, h_stride, bpr_h, seg_starts, w2, stride2, partial, static_cast<int>(dim), E, s); break;
            case PLLM_TYPE_IQ1_M: st = launch_w2_grouped<IQ1M>(h_image, h_stride, bpr_h, seg_starts, w2, stride2, partial, static_cast<int>(dim), E, s); break;
            default: st = launch_w2_grouped<Q2K>(h_image, h_stride, bpr_h, seg_starts, w2, stride2, partial, static_cast<int>(dim), E, s); break;
        }
        if (st != PLLM_OK) return st;
        return launch_moe_reduce(partial, route_tokens, y, tokens, R, static_cast<int>(dim), s);
    }
    switch (w13_type) {
        case PLLM_TYPE_IQ2_XXS:
            st = launch_w13<IQ2XXS>(x_image, x_stride, bpr_x, route_tokens, experts32, route_weights, w1, w3, I, swiglu_limit, h_image, h_stride, bpr_h * 256, R, s);
            break;
        case PLLM_TYPE_IQ1_M:
            st = launch_w13<IQ1M>(x_image, x_stride, bpr_x, route_tokens, experts32, route_weights, w1, w3, I, swiglu_limit, h_image, h_stride, bpr_h * 256, R, s);
            break;
        default:
            st = launch_w13<Q2K>(x_image, x_stride, bpr_x, route_tokens, experts32, route_weights, w1, w3, I, swiglu_limit, h_image, h_stride, bpr_h * 256, R, s);
            break;
    }
    if (st != PLLM_OK) return st;

    const size_t w2_expert_stride = static_cast<size_t>(dim) * bpr_h * pllm_gguf_block_bytes(w2_type);
    st = dot4_routed_matvec_from_image(h_image, h_stride, w2, w2_type, partial, PLLM_F32, R, static_cast<int>(dim), bpr_h, experts32,
                                       w2_expert_stride, s);
    if (st != PLLM_OK) return st;
    return launch_moe_reduce(partial, tokens > 1 ? route_tokens : nullptr, y, tokens, R, static_cast<int>(dim), s);
}

int pllm_moe_group_routes(const void* indices, int indices_are_i64, const float* weights, int64_t tokens, int64_t topk,
                          int64_t experts_start, int64_t n_local, int32_t* seg_starts, int64_t* route_tokens, float* route_weights,
                          int32_t* route_experts, void* stream) {
    using namespace pllm;
    if (!indices || !weights || !seg_starts || !route_tokens || !route_weights || !route_experts) return PLLM_ERR_INVALID_ARGUMENT;
    if (tokens <= 0 || topk <= 0 || n_local <= 0) return PLLM_ERR_INVALID_ARGUMENT;
    if (tokens * topk > 0x7fffffffLL || n_local > 8192) return PLLM_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int total = static_cast<int>(tokens * topk);
    hipLaunchKernelGGL(route_count_kernel, dim3(1), dim3(1024), (n_local + 1) * sizeof(int32_t), s, indices, indices_are_i64, total,
                       static_cast<int>(experts_start), static_cast<int>(n_local), seg_starts);
    hipLaunchKernelGGL(route_fill_kernel, dim3(static_cast<unsigned>(n_local)), dim3(64), 0, s, indices, indices_are_i64, weights, total,
                       static_cast<int>(topk), static_cast<int>(experts_start), seg_starts, route_tokens, route_weights, route_experts);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

}  // extern "C"
