// Decode matvec over raw IQ2_XXS / IQ2_XS / IQ3_XXS / IQ1_M / IQ4_XS / Q6_K super-blocks with the integer dots on the matrix cores.
//
// A wave owns a tile of 16 consecutive output rows (or, for short matrices, a share of the tile's
// super-blocks; the shares meet in a small LDS reduction); the activation image (two int8 terms per
// value) sits in LDS.  For one super-block index the wave forms
//     C[m][n] = sum_k A[m][k] * B[k][n],     v_mfma_i32_16x16x64_i8,
// with n = output row, B = the weights' integer codes and A = activation bytes arranged so that row
// m collects one scale group of the block (the format structs of block_mfma.h say which).  Lane (n, s)
// supplies B for the 16-weight slice s of each MFMA from its own 64 weights of the block, and the
// slices are assigned to A rows such that the lane finds the results for exactly those 64 weights
// in its own C registers: C[4 s .. 4 s + 3][n].
//
// The codebook lookups happen once per weight and feed 16 rows of dots each, where the v_dot4 form
// repeats the activation reads and the dots per lane.
#include <type_traits>

#include "block_mfma.h"
#include "pllm_internal.h"

namespace pllm {
namespace {

constexpr int kRowsPerTile = 16;
constexpr int kWaves = 8;

// One workgroup per tile of 16 rows: its W waves split the row's super-blocks (wave w takes blocks w,
// w + W, ...) and meet in a small LDS reduction.  All weight loads of a pass are issued first; while
// they are in flight the workgroup fills LDS with the activation image and the format's codebooks.
template <typename FMT, int ITERS, bool RAW>
__global__ __launch_bounds__(64 * kWaves) void mfma_tile_matvec_kernel(
    const ActRows act, const WeightRoute route, const uint8_t* __restrict__ w, void* __restrict__ y, int y_dtype, int n, int bpr) {
    fetch_together(act);
    fetch_together(route);
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    const StagedX sx = carve_staged_x(smem, kpad);
    const int zero_off = image_bytes;                                        // 16 zero bytes
    unsigned char* tables = smem + image_bytes + 16;
    const size_t woff = route_offset(route, blockIdx.y);
    w += woff;
    if (blockIdx.z) {                        // several projections in one launch: this one's matrix (of the same expert), row count and output
        const int m = blockIdx.z - 1;
        w = route.more_w[m] + woff;
        y = route.more_y[m];
        n = route.more_n[m];
    }
    if (static_cast<int>(blockIdx.x) * kRowsPerTile >= n) return;           // the grid covers the tallest matrix
    const size_t image_row = act.row_token ? static_cast<size_t>(act.row_token[blockIdx.y]) : blockIdx.y;
    float* partial = reinterpret_cast<float*>(tables + FMT::kTableBytes);   // [waves][16]

    const int tid = threadIdx.x;
    const int waves = blockDim.x >> 6;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int col = lane & 15;        // B/C column = output row within the tile; also A's row index m
    const int ks = lane >> 4;         // k slice of A and B, row quad of C
    const int row = blockIdx.x * kRowsPerTile + col;
    const uint8_t* wrow = w + static_cast<size_t>(row < n ? row : 0) * bpr * FMT::kBlockBytes;

    // A side: this lane supplies row m = col of every MFMA, slice ks; the format says which rows are its
    AMap<FMT::kSlots> am;
    FMT::a_map(am, col, ks, kpad, zero_off);

    float acc = 0.0f;
    bool staged = false;
    if constexpr (RAW)                       // raw activation row: quantized here, before the loads take their registers
        quantize_row_to_lds(smem, act.x, act.x_dtype, raw_row_of(act, blockIdx.y) * act.k, act.k, kpad, RowNorm{act.gamma, act.eps, act.round_f16});
    for (int b0 = wave; b0 < bpr || !staged; b0 += waves * ITERS) {
        typename FMT::Regs regs[ITERS];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int b = min(b0 + it * waves, bpr - 1);                    // clamped: always a valid address
            FMT::load(regs[it], wrow + static_cast<size_t>(b) * FMT::kBlockBytes, ks);
        }
        if (!staged) {                       // first trip of every thread of the workgroup
            if constexpr (!RAW) copy_to_lds(smem, act.image + image_row * act.stride, image_bytes);
            if (tid < 4) reinterpret_cast<uint32_t*>(smem + zero_off)[tid] = 0;
            FMT::stage_tables(tables);
            __syncthreads();
            staged = true;
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int b = b0 + it * waves;
            if (b < bpr) acc += FMT::block(regs[it], ks, b, smem, am, sx, tables);   // wave-uniform guard
        }
    }
    acc = quad_rows_sum(acc);
    if (ks == 0) partial[wave * kRowsPerTile + col] = acc;
    __syncthreads();
    if (tid < kRowsPerTile) {
        float total = 0.0f;
        for (int v = 0; v < waves; ++v) total += partial[v * kRowsPerTile + tid];
        const int out_row = blockIdx.x * kRowsPerTile + tid;
        if (out_row < n) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + out_row, total);
    }
}

// Two to R raw rows of a dense call in one pass over the weights (formats with block_rows; the row count in act.round_f16): R
// activation images in LDS, each with its zero bytes behind it; per row the same image, products and float steps as in a call
// of its own, so the same bits.  An image the call has no row for is a copy of the last row's (computed, not stored).
template <typename FMT, int ITERS, int R>
__global__ __launch_bounds__(64 * kWaves) void mfma_tile_rows_kernel(
    const ActRows act, const uint8_t* __restrict__ w, void* __restrict__ y, int y_dtype, int n, int bpr) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    const int image_stride = image_bytes + 16;
    unsigned char* tables = smem + R * image_stride;
    float* partial = reinterpret_cast<float*>(tables + FMT::kTableBytes);   // [R][waves][16]
    const int total_rows = act.round_f16;

    const int tid = threadIdx.x;
    const int waves = blockDim.x >> 6;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int col = lane & 15, ks = lane >> 4;
    const int row = blockIdx.x * kRowsPerTile + col;
    const uint8_t* wrow = w + static_cast<size_t>(row < n ? row : 0) * bpr * FMT::kBlockBytes;
    AMap<FMT::kSlots> am;
    FMT::a_map(am, col, ks, kpad, image_bytes);

    float acc[R];
#pragma unroll
    for (int i = 0; i < R; ++i) acc[i] = 0.0f;
    bool staged = false;
    for (int i = 0; i < R; ++i)
        quantize_row_to_lds(smem + i * image_stride, act.x, act.x_dtype, static_cast<size_t>(min(i, total_rows - 1)) * act.k, act.k, kpad);
    for (int b0 = wave; b0 < bpr || !staged; b0 += waves * ITERS) {
        typename FMT::Regs regs[ITERS];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int b = min(b0 + it * waves, bpr - 1);                    // clamped: always a valid address
            FMT::load(regs[it], wrow + static_cast<size_t>(b) * FMT::kBlockBytes, ks);
        }
        if (!staged) {                       // first trip of every thread of the workgroup
            if (tid < 4 * R) reinterpret_cast<uint32_t*>(smem + (tid >> 2) * image_stride + image_bytes)[tid & 3] = 0;
            FMT::stage_tables(tables);
            __syncthreads();
            staged = true;
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int b = b0 + it * waves;
            if (b < bpr) FMT::template block_rows<R>(regs[it], ks, b, smem, image_stride, am, kpad, tables, acc);   // wave-uniform guard
        }
    }
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const float sum = quad_rows_sum(acc[i]);
        if (ks == 0) partial[(i * waves + wave) * kRowsPerTile + col] = sum;
    }
    __syncthreads();
    if (tid < R * kRowsPerTile) {
        const int r = tid / kRowsPerTile, cc = tid % kRowsPerTile;
        float total = 0.0f;
        for (int v = 0; v < waves; ++v) total += partial[(r * waves + v) * kRowsPerTile + cc];
        const int out_row = blockIdx.x * kRowsPerTile + cc;
        if (out_row < n && r < total_rows) store_any(y, y_dtype, static_cast<size_t>(r) * n + out_row, total);
    }
}

template <typename FMT, int ITERS, int R>
int launch_tile_rows(const ActRows& act, const uint8_t* w, void* y, int y_dtype, int rows, int n, int bpr, int waves, hipStream_t stream) {
    const size_t smem = R * (staged_x_bytes(bpr * 256) + 16) + FMT::kTableBytes + static_cast<size_t>(R * waves) * kRowsPerTile * sizeof(float);
    auto kern = mfma_tile_rows_kernel<FMT, ITERS, R>;
    if (smem > 64 * 1024) {
        if (smem > 160 * 1024) return PLLM_ERR_UNSUPPORTED;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem)) != hipSuccess)
            return PLLM_ERR_UNSUPPORTED;
    }
    ActRows few = act;
    few.round_f16 = rows;                    // (where the kernel expects the row count)
    hipLaunchKernelGGL(kern, dim3((n + kRowsPerTile - 1) / kRowsPerTile), dim3(64 * waves), smem, stream, few, w, y, y_dtype, n, bpr);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

template <typename FMT, int ITERS, bool RAW>
int launch_tile(const ActRows& act, const WeightRoute& route, const uint8_t* w, void* y, int y_dtype,
                int rows, int n, int bpr, int waves, hipStream_t stream) {
    const size_t smem = staged_x_bytes(bpr * 256) + 16 + FMT::kTableBytes + static_cast<size_t>(waves) * kRowsPerTile * sizeof(float);
    auto kern = mfma_tile_matvec_kernel<FMT, ITERS, RAW>;
    if (smem > 64 * 1024) {
        if (smem > 160 * 1024) return PLLM_ERR_UNSUPPORTED;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(smem)) != hipSuccess)
            return PLLM_ERR_UNSUPPORTED;
    }
    int tallest = n;
    for (int m = 0; m < route.extra; ++m) tallest = tallest > route.more_n[m] ? tallest : route.more_n[m];
    dim3 grid((tallest + kRowsPerTile - 1) / kRowsPerTile, rows, 1 + route.extra);
    hipLaunchKernelGGL(kern, grid, dim3(64 * waves), smem, stream, act, route, w, y, y_dtype, n, bpr);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

// The pair kernel halves the number of workgroups and doubles the image's share of LDS: taken from 512 tiles on and up to rows of
// 32 super-blocks (IQ3_XXS 17408x5120 32.2 -> 24.7 us, 12288x4096 19.3 -> 15.0, 200064x3072 185 -> 124; IQ2_XS 31.3 -> 29.5,
// 20.4 -> 15.2, 185 -> 144; at 5120x5120 the two were level and at 5120x17408 two grid rows won, 37.4 against 40.5 us)
constexpr int kPairMinRows = 8192;
constexpr int kPairMaxBlocksPerRow = 32;

template <typename FMT>
int launch_tiles(const ActRows& act, const WeightRoute& route, const uint8_t* w, void* y, int y_dtype,
                 int rows, int n, int bpr, hipStream_t stream) {
    // waves per workgroup: split a row's blocks so that every wave keeps a handful in flight
    int waves = 1;
    while (waves < kWaves && bpr / (waves * 2) >= 3) waves *= 2;
    const int niter = (bpr + waves - 1) / waves;
    const int passes = (niter + 5) / 6;
    const int iters = (niter + passes - 1) / passes;
    // two raw rows of a tall dense matrix: one pass over the weights, every block's codes looked up once
    if constexpr (FMT::kRowsPerPass > 1)
        if (act.x && !act.gamma && rows >= 2 && rows <= FMT::kRowsPerPass && !routed(route) && route.extra == 0 && !act.row_token && !act.x_broadcast &&
            n >= kPairMinRows && bpr <= kPairMaxBlocksPerRow) {
#define PLLM_ROWS_CASE(I) case I: return rows == 2 ? launch_tile_rows<FMT, I, 2>(act, w, y, y_dtype, rows, n, bpr, waves, stream) \
                                              : launch_tile_rows<FMT, I, FMT::kRowsPerPass>(act, w, y, y_dtype, rows, n, bpr, waves, stream)
            switch (iters) {
                PLLM_ROWS_CASE(1); PLLM_ROWS_CASE(2); PLLM_ROWS_CASE(3); PLLM_ROWS_CASE(4); PLLM_ROWS_CASE(5);
                default: PLLM_ROWS_CASE(6);
            }
#undef PLLM_ROWS_CASE
        }
#define PLLM_CASE(I) case I: return act.x ? launch_tile<FMT, I, true>(act, route, w, y, y_dtype, rows, n, bpr, waves, stream) \
                                          : launch_tile<FMT, I, false>(act, route, w, y, y_dtype, rows, n, bpr, waves, stream)
    switch (iters) {
        PLLM_CASE(1); PLLM_CASE(2); PLLM_CASE(3); PLLM_CASE(4); PLLM_CASE(5);
        default: PLLM_CASE(6);
    }
#undef PLLM_CASE
}

// ------------------------------------------------------------------------------------------------
// Streamed form.  The rows of consecutive tiles are one contiguous run of memory, but a lane's share
// of a block is 16 + 2 bytes at a 2-byte-aligned address and the 16 rows of a tile lie a whole row
// apart: loading shares straight into registers asks the memory system for many small unaligned
// pieces.  Here the workgroup copies a chunk of `tiles_per_chunk` whole tiles into LDS with
// direct-to-LDS loads (global_load_lds_dwordx4: every wave instruction moves 1 KB that is contiguous
// in memory and in LDS, aligned, no registers involved) and the waves pick their shares out of LDS.
// Workgroups walk chunks blockIdx.x, blockIdx.x + gridDim.x, ...; several share a compute unit, so
// some multiply while others wait for their chunk.  Needs n % 16 == 0 and a 16-byte aligned matrix.
// ------------------------------------------------------------------------------------------------
constexpr int kChunkBudget = 28 * 1024;
constexpr int kLdsBytes = 160 * 1024;

// NB > 0: a wave meets at most NB block indices (part, part + split, ...) and keeps their activation
// side in registers across all its chunks; NB == 0: any number, read from LDS every time.
// WAVES: 8, several workgroups per compute unit, or 16, one workgroup per compute unit around one set of tables (the form for
// replicated tables, FMT::kCopies > 1, which take the LDS of several plain ones).
// ROWS > 1 (dense calls of two raw rows; the row count in act.round_f16, one grid row): ROWS activation images lie one
// behind the other, each with its own zero bytes; every block a wave picks out of a chunk is decoded once and multiplied into
// all of them (the decode, table lookups and sign masks, is what these kernels spend their time on).
template <typename FMT, int NB, bool RAW, int WAVES, int ROWS = 1>
__global__ __launch_bounds__(64 * WAVES) void iq_stream_matvec_kernel(
    const ActRows act, const uint8_t* __restrict__ w,
    void* __restrict__ y, int y_dtype, int n, int bpr, int split, int chunks, int chunk_off, int chunk_stride) {
    static_assert(ROWS == 1 || (NB == 0 && RAW), "the few-row form quantizes its rows itself and holds nothing");
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    const StagedX sx = carve_staged_x(smem, kpad);
    const int zero_off = image_bytes;                                        // 16 zero bytes behind every image
    const int image_stride = image_bytes + 16;
    const int table_off = ROWS * image_stride;
    const int total_rows = ROWS > 1 ? act.round_f16 : 1;
    float* partial = reinterpret_cast<float*>(smem + table_off + FMT::kTableBytes);   // [ROWS][waves][16]
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte_ptr)smem));

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int col = lane & 15, ks = lane >> 4;
    const unsigned char* tables = FMT::lane_tables(smem + table_off, lane);
    const int tiles_per_chunk = WAVES / split;
    const int tile_in_chunk = wave / split, part = wave % split;
    const int row_bytes = bpr * FMT::kBlockBytes;
    const int chunk_rows = tiles_per_chunk * kRowsPerTile;

    // activation image, codebooks and the first chunk: all in flight together
    if constexpr (!RAW) dma_share<WAVES>(act.image + static_cast<size_t>(blockIdx.y) * act.stride, lds0, image_bytes, wave, lane);
    if constexpr (FMT::kCopies == 1) FMT::template dma_tables<WAVES>(lds0 + table_off, wave, lane);
    if (tid < 4 * ROWS) reinterpret_cast<uint32_t*>(smem + (tid >> 2) * image_stride + zero_off)[tid & 3] = 0;
    AMap<FMT::kSlots> am;
    FMT::a_map(am, col, ks, kpad, zero_off);

    int c = blockIdx.x, buf = 0;
    dma_share<WAVES>(w + static_cast<size_t>(c) * chunk_rows * row_bytes, lds0 + chunk_off, min(chunk_rows, n - c * chunk_rows) * row_bytes, wave, lane);
    if constexpr (FMT::kCopies > 1) FMT::stage_replicated(smem + table_off, tid, 64 * WAVES);   // ordinary stores; the loop's first barrier covers them
    if constexpr (ROWS > 1) {
        for (int r = 0; r < total_rows; ++r)
            quantize_row_to_lds(smem + r * image_stride, act.x, act.x_dtype, static_cast<size_t>(r) * act.k, act.k, kpad);
    } else if constexpr (RAW)                // raw activation row: quantized once per workgroup while the first chunk is on its way
        quantize_row_to_lds(smem, act.x, act.x_dtype, static_cast<size_t>(blockIdx.y) * act.k, act.k, kpad, RowNorm{act.gamma, act.eps, act.round_f16});
    typename FMT::Held held[NB > 0 ? NB : 1];
    bool holding = false;
    while (c < chunks) {
        const int row0 = c * chunk_rows;
        const int valid_rows = min(chunk_rows, n - row0);                    // a multiple of 16
        // the next chunk goes to the other buffer while this one is multiplied
        const int cn = c + gridDim.x;
        int newest = 0;
        if (cn < chunks)
            newest = dma_share<WAVES>(w + static_cast<size_t>(cn) * chunk_rows * row_bytes, lds0 + chunk_off + (buf ^ 1) * chunk_stride,
                               min(chunk_rows, n - cn * chunk_rows) * row_bytes, wave, lane);
        wait_vm_all_but(newest);             // this wave's pieces of chunk c (and of the image and tables) have landed ...
        __syncthreads();                     // ... and everybody else's too
        if constexpr (NB > 0) if (!holding) {
#pragma unroll
            for (int i = 0; i < NB; ++i) FMT::hold(held[i], ks, min(part + i * split, bpr - 1), smem, am, sx);
            holding = true;
        }

        const unsigned char* chunk = smem + chunk_off + buf * chunk_stride;
        float acc = 0.0f;
        if constexpr (ROWS > 1) {
            if (tile_in_chunk * kRowsPerTile < valid_rows) {                 // wave-uniform
                const int row_off = (tile_in_chunk * kRowsPerTile + col) * row_bytes;
                float accs[ROWS];
#pragma unroll
                for (int r = 0; r < ROWS; ++r) accs[r] = 0.0f;
                AOps<FMT::kSlots> ops;
                clear_a(ops);                                                // (the slots that are not the lane's stay zero: never loaded)
                for (int b = part; b < bpr; b += split) {
                    typename FMT::Regs regs;
                    FMT::load_lds(regs, chunk, row_off + b * FMT::kBlockBytes, ks);
                    typename FMT::Decoded o;
                    FMT::decode(regs, ks, tables, o);
#pragma unroll
                    for (int r = 0; r < ROWS; ++r)
                        if (r < total_rows) {                                // wave-uniform
                            accs[r] += FMT::route_block(o, ks, b, smem + r * image_stride, am, kpad, ops);
                        }
                }
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    const float sum = quad_rows_sum(accs[r]);
                    if (ks == 0 && r < total_rows) {
                        if (split == 1) store_any(y, y_dtype, static_cast<size_t>(r) * n + row0 + tile_in_chunk * kRowsPerTile + col, sum);
                        else partial[(r * WAVES + wave) * kRowsPerTile + col] = sum;
                    }
                }
            }
            __syncthreads();                 // this buffer may be overwritten, the partial sums are complete
            if (split > 1 && tid < valid_rows) {
                const int t = tid / kRowsPerTile, cc = tid % kRowsPerTile;
                for (int r = 0; r < total_rows; ++r) {
                    float total = 0.0f;
                    for (int v = 0; v < split; ++v) total += partial[(r * WAVES + t * split + v) * kRowsPerTile + cc];
                    store_any(y, y_dtype, static_cast<size_t>(r) * n + row0 + tid, total);
                }
            }
            c = cn;
            buf ^= 1;
            continue;
        }
        if (tile_in_chunk * kRowsPerTile < valid_rows) {                     // wave-uniform
            const int row_off = (tile_in_chunk * kRowsPerTile + col) * row_bytes;
            if constexpr (NB > 0) {
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    const int b = part + i * split;
                    if (b < bpr) {                                           // wave-uniform
                        typename FMT::Regs regs;
                        FMT::load_lds(regs, chunk, row_off + b * FMT::kBlockBytes, ks);
                        acc += FMT::block_held(regs, ks, b, held[i], smem, am, tables);
                    }
                }
            } else {
                for (int b = part; b < bpr; b += split) {
                    typename FMT::Regs regs;
                    FMT::load_lds(regs, chunk, row_off + b * FMT::kBlockBytes, ks);
                    acc += FMT::block(regs, ks, b, smem, am, sx, tables);
                }
            }
            acc = quad_rows_sum(acc);
            if (split == 1) {
                if (ks == 0) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + row0 + tile_in_chunk * kRowsPerTile + col, acc);
            } else if (ks == 0) {
                partial[wave * kRowsPerTile + col] = acc;
            }
        }
        __syncthreads();                     // this buffer may be overwritten, the partial sums are complete
        if (split > 1 && tid < valid_rows) {
            const int t = tid / kRowsPerTile, cc = tid % kRowsPerTile;
            float total = 0.0f;
            for (int v = 0; v < split; ++v) total += partial[(t * split + v) * kRowsPerTile + cc];
            store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + row0 + tid, total);
        }
        c = cn;
        buf ^= 1;
    }
}

// ------------------------------------------------------------------------------------------------
// The streamed form for rows of exactly NB * SPLIT super-blocks (every model shape): the row length is a compile-time constant,
// so are the LDS layout and the number of copy instructions per chunk, and every chunk is whole (the last one is moved back to
// end at row n; rows it shares with its predecessor are computed twice and stored once).  One barrier per chunk:
//     wait for my pieces of chunk c | barrier | sums of chunk c - 1 out | request chunk c + 1 | multiply chunk c
// The barrier says that chunk c has landed AND that everybody has left chunk c - 1, whose buffer the request reuses and whose
// per-wave sums (kept in two alternating sets) can now be added and stored.  These kernels are bound by the number of
// instructions a SIMD issues (a step of 16 rows x 256 weights cost ~190 wave instructions in the general form above, a third of
// them the chunk loop's bookkeeping), not by the LDS or the matrix cores.
// ------------------------------------------------------------------------------------------------
template <typename FMT, int NB, int SPLIT, int WAVES>
struct ExactLayout {
    static constexpr int kBpr = NB * SPLIT;
    static constexpr int kKpad = kBpr * 256;
    static constexpr int kImageBytes = static_cast<int>(staged_x_bytes(kKpad));
    static constexpr int kZeroOff = kImageBytes;
    static constexpr int kTableOff = kImageBytes + 16;
    static constexpr int kPartialOff = kTableOff + FMT::kTableBytes;          // float [2][WAVES][16]
    static constexpr int kChunkOff = (kPartialOff + 2 * WAVES * 16 * 4 + 1023) & ~1023;
    static constexpr int kTiles = WAVES / SPLIT;
    static constexpr int kChunkRows = kTiles * kRowsPerTile;
    static constexpr int kRowBytes = kBpr * FMT::kBlockBytes;
    static constexpr int kChunkBytes = kChunkRows * kRowBytes;                // a multiple of 32
    static constexpr int kChunkStride = kChunkBytes + 16;                     // shares are read as aligned dwords: a few bytes past the end
    static constexpr int kSmem = kChunkOff + 2 * kChunkStride;
    static constexpr int kPieces = (kChunkBytes + 1023) / 1024;               // 1 KB copy instructions per chunk, dealt round the waves
    static constexpr int kPiecesPerWave = (kPieces + WAVES - 1) / WAVES;
};

template <typename FMT, int NB, int SPLIT, bool RAW, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void iq_stream_exact_kernel(
    const ActRows act, const uint8_t* __restrict__ w, void* __restrict__ y, int y_dtype, int n, int chunks) {
    using L = ExactLayout<FMT, NB, SPLIT, WAVES>;
    extern __shared__ __align__(16) unsigned char smem[];
    const StagedX sx = carve_staged_x(smem, L::kKpad);
    float* partial = reinterpret_cast<float*>(smem + L::kPartialOff);
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte_ptr)smem));

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int col = lane & 15, ks = lane >> 4;
    const unsigned char* tables = FMT::lane_tables(smem + L::kTableOff, lane);
    const int tile_in_chunk = wave / SPLIT, part = wave % SPLIT;
    y = static_cast<unsigned char*>(y) + static_cast<size_t>(blockIdx.y) * n * (y_dtype == PLLM_F32 ? 4 : 2);   // this activation row's outputs

    const uint32_t piece_off = wave * 1024 + lane * 16;
    // chunk c covers rows [first_row(c), first_row(c) + kChunkRows); all but the last start at c * kChunkRows
    auto first_row = [&](int c) { return min(c * L::kChunkRows, n - L::kChunkRows); };
    // whole 1 KB pieces wave, wave + WAVES, ... of a chunk, then the last, shorter piece (scalar bases and targets, one lane offset)
    constexpr int kWhole = L::kChunkBytes / 1024, kTail = L::kChunkBytes % 1024;
    auto request = [&](int c, int buf) {
        const uint8_t* src = w + static_cast<size_t>(first_row(c)) * L::kRowBytes;
        const uint32_t dst = lds0 + L::kChunkOff + buf * L::kChunkStride + wave * 1024;
#pragma unroll
        for (int i = 0; i * WAVES < kWhole; ++i)
            if ((i + 1) * WAVES <= kWhole || wave + i * WAVES < kWhole) lds_dma16_at(src + i * (WAVES * 1024), piece_off, dst + i * (WAVES * 1024));
        if constexpr (kTail > 0)
            if (wave == kWhole % WAVES && lane * 16 < kTail)
                lds_dma16_at(src + (kWhole / WAVES) * (WAVES * 1024), piece_off, dst + (kWhole / WAVES) * (WAVES * 1024));
    };
    // sums of the waves that share a tile, in wave order; rows below `skip` belong to the chunk before
    auto sums_out = [&](int set, int row0, int skip) {
        if constexpr (SPLIT > 1) {
            if (tid < L::kChunkRows && tid >= skip) {
                const float* ps = partial + set * (WAVES * 16) + (tid / kRowsPerTile) * (SPLIT * 16) + tid % kRowsPerTile;
                float total = 0.0f;
#pragma unroll
                for (int v = 0; v < SPLIT; ++v) total += ps[v * 16];
                store_plain(y, y_dtype, static_cast<size_t>(row0 + tid), total);
            }
        }
    };

    // activation image, codebooks and the first chunk: all in flight together
    if constexpr (!RAW) dma_share<WAVES>(act.image + static_cast<size_t>(blockIdx.y) * act.stride, lds0, L::kImageBytes, wave, lane);
    if constexpr (FMT::kCopies == 1) FMT::template dma_tables<WAVES>(lds0 + L::kTableOff, wave, lane);
    if (tid < 4) reinterpret_cast<uint32_t*>(smem + L::kZeroOff)[tid] = 0;
    AMap<FMT::kSlots> am;
    FMT::a_map(am, col, ks, L::kKpad, L::kZeroOff);
    int c = blockIdx.x;
    request(c, 0);
    if constexpr (FMT::kCopies > 1) FMT::stage_replicated(smem + L::kTableOff, tid, 64 * WAVES);   // ordinary stores; the loop's first barrier covers them
    if constexpr (RAW)                       // raw activation row: quantized once per workgroup while the first chunk is on its way
        quantize_row_to_lds(smem, act.x, act.x_dtype, static_cast<size_t>(blockIdx.y) * act.k, act.k, L::kKpad, RowNorm{act.gamma, act.eps, act.round_f16});

    constexpr bool kHold = NB <= FMT::kHoldBlocks;
    typename FMT::Held held[kHold ? NB : 1];
    wait_vm<0>();                            // this wave's pieces of the first chunk, of the image and of the tables have landed ...
    __syncthreads();                         // ... and everybody else's
    if constexpr (kHold) {
#pragma unroll
        for (int i = 0; i < NB; ++i) FMT::hold(held[i], ks, part + i * SPLIT, smem, am, sx);
    }
    int buf = 0, set = 0;
    const int row_off = (tile_in_chunk * kRowsPerTile + col) * L::kRowBytes + part * FMT::kBlockBytes;
    while (true) {
        const int cn = c + gridDim.x;
        if (cn < chunks) request(cn, buf ^ 1);   // the other buffer is free: everybody has passed the barrier behind its last use

        const unsigned char* chunk = smem + L::kChunkOff + buf * L::kChunkStride;
        float acc = 0.0f;
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            typename FMT::Regs regs;
            FMT::load_lds(regs, chunk, row_off + i * SPLIT * FMT::kBlockBytes, ks);
            if constexpr (kHold) acc += FMT::block_held(regs, ks, part + i * SPLIT, held[i], smem, am, tables);
            else acc += FMT::block(regs, ks, part + i * SPLIT, smem, am, sx, tables);
            __builtin_amdgcn_sched_barrier(0);                               // one block after the other: interleaved they do not fit the registers
        }
        acc = quad_rows_sum(acc);
        const int row0 = first_row(c), skip = c * L::kChunkRows - row0;
        if constexpr (SPLIT == 1) {
            const int r = tile_in_chunk * kRowsPerTile + col;
            if (ks == 0 && r >= skip) store_plain(y, y_dtype, static_cast<size_t>(row0 + r), acc);
        } else if (ks == 0) {
            partial[set * (WAVES * 16) + wave * 16 + col] = acc;
        }
        wait_vm<0>();                        // this wave's pieces of the next chunk have landed ...
        __syncthreads();                     // ... and everybody else's; everybody has left this chunk, whose sums are complete
        sums_out(set, row0, skip);
        if (cn >= chunks) break;
        c = cn; buf ^= 1; set ^= 1;
    }
}

template <typename FMT, int NB, int SPLIT, int WAVES>
int launch_exact(const ActRows& act, const uint8_t* w, void* y, int y_dtype, int rows, int n, hipStream_t stream) {
    using L = ExactLayout<FMT, NB, SPLIT, WAVES>;
    static_assert(L::kSmem <= kLdsBytes, "does not fit the LDS");
    const void* kern = act.x ? reinterpret_cast<const void*>(iq_stream_exact_kernel<FMT, NB, SPLIT, true, WAVES>)
                             : reinterpret_cast<const void*>(iq_stream_exact_kernel<FMT, NB, SPLIT, false, WAVES>);
    static SmemGrant granted[2];
    if (!grant_dynamic_smem(kern, L::kSmem, granted[act.x ? 1 : 0])) return PLLM_ERR_UNSUPPORTED;
    const int chunks = (n + L::kChunkRows - 1) / L::kChunkRows;
    const int resident = (kLdsBytes / L::kSmem) * compute_units();           // the LDS is what limits residency here
    int grid = chunks;
    if (chunks > resident) {
        const int rounds = (chunks + resident - 1) / resident;
        grid = (chunks + rounds - 1) / rounds;
    }
    if (act.x) hipLaunchKernelGGL((iq_stream_exact_kernel<FMT, NB, SPLIT, true, WAVES>), dim3(grid, rows), dim3(64 * WAVES), L::kSmem, stream, act, w, y, y_dtype, n, chunks);
    else hipLaunchKernelGGL((iq_stream_exact_kernel<FMT, NB, SPLIT, false, WAVES>), dim3(grid, rows), dim3(64 * WAVES), L::kSmem, stream, act, w, y, y_dtype, n, chunks);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

// the exact form for the row lengths it is built for; PLLM_ERR_UNSUPPORTED: take the general one
template <typename FMT>
int launch_exact_for(const ActRows& act, const uint8_t* w, void* y, int y_dtype, int rows, int n, int bpr, hipStream_t stream) {
    if (n % kRowsPerTile != 0 || (reinterpret_cast<uintptr_t>(w) & 15u) || (y_dtype & kAccumulateInto)) return PLLM_ERR_UNSUPPORTED;
#define PLLM_EXACT(F, NB, SPLIT, WAVES) \
    if (bpr == NB * SPLIT && n >= ExactLayout<F, NB, SPLIT, WAVES>::kChunkRows) return launch_exact<F, NB, SPLIT, WAVES>(act, w, y, y_dtype, rows, n, stream)
    if constexpr (std::is_same<FMT, IQ2XXSm>::value) {
        PLLM_EXACT(IQ2XXSmT<16>, 3, 4, 16);        // K = 3072
    } else if constexpr (std::is_same<FMT, IQ1Mm>::value) {
        PLLM_EXACT(IQ1Mm, 3, 2, 8);                // K = 1536
    }
#undef PLLM_EXACT
    return PLLM_ERR_UNSUPPORTED;
}

// What a streamed launch looks like: waves per workgroup, waves per tile, LDS layout.  split == 0: the streamed form does not apply.
struct StreamPlan { int waves, split, chunk_off, chunk_stride; size_t smem; };

template <typename FMT>
StreamPlan stream_plan(const uint8_t* w, int n, int bpr, int waves, int chunk_budget, int rows_per_pass = 1) {
    StreamPlan p{waves, 0, 0, 0, 0};
    if (n % kRowsPerTile != 0 || (reinterpret_cast<uintptr_t>(w) & 15u)) return p;
    const int tile_bytes = kRowsPerTile * bpr * FMT::kBlockBytes;
    const size_t head = rows_per_pass * (staged_x_bytes(bpr * 256) + 16 + waves * kRowsPerTile * sizeof(float)) + FMT::kTableBytes;
    p.chunk_off = static_cast<int>((head + 1023) & ~static_cast<size_t>(1023));
    if (chunk_budget <= 0) chunk_budget = (kLdsBytes - p.chunk_off) / 2 - 16;
    // the most waves per tile first (smallest chunk) that leaves every wave at least two blocks
    for (int split = waves; split >= 1; split /= 2)
        if ((split == 1 || bpr >= 2 * split) && (waves / split) * tile_bytes <= chunk_budget) { p.split = split; break; }
    if (!p.split) return p;
    p.chunk_stride = (waves / p.split) * tile_bytes + 16;                    // shares are read as aligned dwords: a few bytes past the end
    p.smem = static_cast<size_t>(p.chunk_off) + 2 * p.chunk_stride;
    if (p.smem > kLdsBytes) p.split = 0;
    return p;
}

template <typename FMT, int NB, bool RAW, int WAVES, int ROWS = 1>
int launch_stream_raw(const ActRows& act, const uint8_t* w, void* y, int y_dtype, int rows, int n, int bpr, const StreamPlan& p, hipStream_t stream) {
    auto kern = iq_stream_matvec_kernel<FMT, NB, RAW, WAVES, ROWS>;
    const int tiles_per_chunk = WAVES / p.split;
    static SmemGrant granted;
    if (!grant_dynamic_smem(reinterpret_cast<const void*>(kern), p.smem, granted)) return PLLM_ERR_UNSUPPORTED;
    // resident workgroups per compute unit for this LDS size: asked once per size (the query costs microseconds of host time)
    static std::atomic<size_t> occ_smem{~static_cast<size_t>(0)};
    static std::atomic<int> occ_per_cu{1};
    if (p.smem != occ_smem.load(std::memory_order_acquire)) {
        int q = 0;
        occ_per_cu.store((hipOccupancyMaxActiveBlocksPerMultiprocessor(&q, kern, 64 * WAVES, p.smem) == hipSuccess && q >= 1) ? q : 1, std::memory_order_relaxed);
        occ_smem.store(p.smem, std::memory_order_release);
    }
    const int per_cu = occ_per_cu.load(std::memory_order_relaxed);
    const int chunks = (n / kRowsPerTile + tiles_per_chunk - 1) / tiles_per_chunk;
    const int resident = per_cu * compute_units();
    int grid = chunks;
    if (chunks > resident) {
        const int rounds = (chunks + resident - 1) / resident;
        grid = (chunks + rounds - 1) / rounds;
    }
    hipLaunchKernelGGL(kern, dim3(grid, rows), dim3(64 * WAVES), p.smem, stream, act, w, y, y_dtype, n, bpr, p.split, chunks,
                       p.chunk_off, p.chunk_stride);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

// two raw rows through every decoded block: one grid row, the row count where the kernel expects it
template <typename FMT, int WAVES>
int launch_stream_few(const ActRows& act, const uint8_t* w, void* y, int y_dtype, int rows, int n, int bpr, const StreamPlan& p, hipStream_t stream) {
    ActRows few = act;
    few.round_f16 = rows;
    return launch_stream_raw<FMT, 0, true, WAVES, 2>(few, w, y, y_dtype, 1, n, bpr, p, stream);
}

template <typename FMT, int NB, int WAVES>
int launch_stream_nb(const ActRows& act, const uint8_t* w, void* y, int y_dtype, int rows, int n, int bpr, const StreamPlan& p, hipStream_t stream) {
    return act.x ? launch_stream_raw<FMT, NB, true, WAVES>(act, w, y, y_dtype, rows, n, bpr, p, stream)
                 : launch_stream_raw<FMT, NB, false, WAVES>(act, w, y, y_dtype, rows, n, bpr, p, stream);
}

template <typename FMT, int WAVES>
int launch_stream(const ActRows& act, const uint8_t* w, void* y, int y_dtype, int rows, int n, int bpr, const StreamPlan& p, hipStream_t stream) {
    const int per_wave = (bpr + p.split - 1) / p.split;                      // block indices a wave meets
    if constexpr (FMT::kHoldBlocks >= 2) if (per_wave <= 2) return launch_stream_nb<FMT, 2, WAVES>(act, w, y, y_dtype, rows, n, bpr, p, stream);
    if constexpr (FMT::kHoldBlocks >= 3) if (per_wave == 3) return launch_stream_nb<FMT, 3, WAVES>(act, w, y, y_dtype, rows, n, bpr, p, stream);
    return launch_stream_nb<FMT, 0, WAVES>(act, w, y, y_dtype, rows, n, bpr, p, stream);
}

template <typename FMT>
int launch_fmt(const ActRows& act, const WeightRoute& route, const uint8_t* w, void* y, int y_dtype,
               int rows, int n, int bpr, hipStream_t stream) {
    // whole tiles streamed through long-lived workgroups (the codebooks are staged once per workgroup)
    // where shape and alignment allow, else one short workgroup per tile; routed calls and several projections in one launch
    // always take the latter
    if constexpr (FMT::kStreamed)
        if (!routed(route) && !act.row_token && !act.x_broadcast && route.extra == 0) {
            // two raw rows of a large matrix: every block decoded once for both (17408x5120 IQ2_XXS 27.8 -> 22.0 us, IQ1_M 26.3 -> 24.5,
            // 5120x5120 15.5 -> 11.7 and 14.4 -> 13.5, 200064x3072 88.5 -> 78.5 and 111.8 -> 99.4); below 24M weights two grid rows fill
            // the machine better (IQ1_M 8192x1536 5.4 against 8.7 us), and with four rows in this form each further row still cost
            // 6 - 10 us (the multiply side: operand loads and MFMAs per image), level with the tile kernel
            if (act.x && !act.gamma && rows == 2 && static_cast<int64_t>(n) * bpr * 256 >= (int64_t{24} << 20)) {
                constexpr int rp = 2;
                if constexpr (std::is_same<FMT, IQ2XXSm>::value) {
                    const StreamPlan wide = stream_plan<IQ2XXSmT<16>>(w, n, bpr, 16, 0, rp);
                    if (wide.split) return launch_stream_few<IQ2XXSmT<16>, 16>(act, w, y, y_dtype, rows, n, bpr, wide, stream);
                }
                const StreamPlan p = stream_plan<FMT>(w, n, bpr, kWaves, kChunkBudget, rp);
                if (p.split) return launch_stream_few<FMT, kWaves>(act, w, y, y_dtype, rows, n, bpr, p, stream);
            }
            const int exact = launch_exact_for<FMT>(act, w, y, y_dtype, rows, n, bpr, stream);
            if (exact != PLLM_ERR_UNSUPPORTED) return exact;
            if constexpr (std::is_same<FMT, IQ2XXSm>::value) {
                // sixteen table copies (conflict-free lookups) around one 16-wave workgroup per compute unit, where the LDS holds it
                const StreamPlan wide = stream_plan<IQ2XXSmT<16>>(w, n, bpr, 16, 0);
                if (wide.split) return launch_stream<IQ2XXSmT<16>, 16>(act, w, y, y_dtype, rows, n, bpr, wide, stream);
            }
            const StreamPlan p = stream_plan<FMT>(w, n, bpr, kWaves, kChunkBudget);
            if (p.split) return launch_stream<FMT, kWaves>(act, w, y, y_dtype, rows, n, bpr, p, stream);
        }
    return launch_tiles<FMT>(act, route, w, y, y_dtype, rows, n, bpr, stream);
}

}  // namespace

int iq_mfma_matvec_from_image(const ActRows& act, const uint8_t* w, int type_id, void* y, int y_dtype,
                              int rows, int n, int bpr, hipStream_t stream, WeightRoute route) {
    switch (type_id) {
        case PLLM_TYPE_IQ2_XXS: return launch_fmt<IQ2XXSm>(act, route, w, y, y_dtype, rows, n, bpr, stream);
        case PLLM_TYPE_IQ1_M: return launch_fmt<IQ1Mm>(act, route, w, y, y_dtype, rows, n, bpr, stream);
        case PLLM_TYPE_IQ2_XS: return launch_fmt<IQ2XSm>(act, route, w, y, y_dtype, rows, n, bpr, stream);
        case PLLM_TYPE_IQ3_XXS: return launch_fmt<IQ3XXSm>(act, route, w, y, y_dtype, rows, n, bpr, stream);
        case PLLM_TYPE_IQ4_XS: return launch_fmt<IQ4XSm>(act, route, w, y, y_dtype, rows, n, bpr, stream);
        case PLLM_TYPE_Q6_K: return launch_fmt<Q6Km>(act, route, w, y, y_dtype, rows, n, bpr, stream);
        default: return PLLM_ERR_UNSUPPORTED;
    }
}

}  // namespace pllm
