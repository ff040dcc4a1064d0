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
    acc += __shfl_xor(acc, 16, 64);
    acc += __shfl_xor(acc, 32, 64);
    if (ks == 0) partial[wave * kRowsPerTile + col] = acc;
    __syncthreads();
    if (tid < kRowsPerTile) {
        float total = 0.0f;
        for (int v = 0; v < waves; ++v) total += partial[v * kRowsPerTile + tid];
        const int out_row = blockIdx.x * kRowsPerTile + tid;
        if (out_row < n) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + out_row, total);
    }
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

template <typename FMT>
int launch_tiles(const ActRows& act, const WeightRoute& route, const uint8_t* w, void* y, int y_dtype,
                 int rows, int n, int bpr, hipStream_t stream) {
    // waves per workgroup: split a row's blocks so that every wave keeps a handful in flight
    int waves = 1;
    while (waves < kWaves && bpr / (waves * 2) >= 3) waves *= 2;
    const int niter = (bpr + waves - 1) / waves;
    const int passes = (niter + 5) / 6;
    const int iters = (niter + passes - 1) / passes;
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

// NB > 0: a wave meets at most NB block indices (part, part + split, ...) and keeps their activation
// side in registers across all its chunks; NB == 0: any number, read from LDS every time.
template <typename FMT, int NB, bool RAW>
__global__ __launch_bounds__(64 * kWaves) void iq_stream_matvec_kernel(
    const ActRows act, const uint8_t* __restrict__ w,
    void* __restrict__ y, int y_dtype, int n, int bpr, int split, int chunks, int chunk_off, int chunk_stride) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    const StagedX sx = carve_staged_x(smem, kpad);
    const int zero_off = image_bytes;                                        // 16 zero bytes
    const int table_off = image_bytes + 16;
    const unsigned char* tables = smem + table_off;
    float* partial = reinterpret_cast<float*>(smem + table_off + FMT::kTableBytes);   // [waves][16]
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte_ptr)smem));

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int col = lane & 15, ks = lane >> 4;
    const int tiles_per_chunk = kWaves / split;
    const int tile_in_chunk = wave / split, part = wave % split;
    const int row_bytes = bpr * FMT::kBlockBytes;
    const int chunk_rows = tiles_per_chunk * kRowsPerTile;

    // activation image, codebooks and the first chunk: all in flight together
    if constexpr (!RAW) dma_share<kWaves>(act.image + static_cast<size_t>(blockIdx.y) * act.stride, lds0, image_bytes, wave, lane);
    FMT::template dma_tables<kWaves>(lds0 + table_off, wave, lane);
    if (tid < 4) reinterpret_cast<uint32_t*>(smem + zero_off)[tid] = 0;
    AMap<FMT::kSlots> am;
    FMT::a_map(am, col, ks, kpad, zero_off);

    int c = blockIdx.x, buf = 0;
    dma_share<kWaves>(w + static_cast<size_t>(c) * chunk_rows * row_bytes, lds0 + chunk_off, min(chunk_rows, n - c * chunk_rows) * row_bytes, wave, lane);
    if constexpr (RAW)                       // raw activation row: quantized once per workgroup while the first chunk is on its way
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
            newest = dma_share<kWaves>(w + static_cast<size_t>(cn) * chunk_rows * row_bytes, lds0 + chunk_off + (buf ^ 1) * chunk_stride,
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
            acc += __shfl_xor(acc, 16, 64);
            acc += __shfl_xor(acc, 32, 64);
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

// 0 when the streamed form does not apply
template <typename FMT>
int stream_split(const uint8_t* w, int n, int bpr) {
    if (n % kRowsPerTile != 0 || (reinterpret_cast<uintptr_t>(w) & 15u)) return 0;
    const int tile_bytes = kRowsPerTile * bpr * FMT::kBlockBytes;
    // the most waves per tile first (smallest chunk) that leaves every wave at least two blocks
    for (int split = kWaves; split >= 1; split /= 2)
        if ((split == 1 || bpr >= 2 * split) && (kWaves / split) * tile_bytes <= kChunkBudget) return split;
    return 0;
}

template <typename FMT, int NB, bool RAW>
int launch_stream_raw(const ActRows& act, const uint8_t* w, void* y, int y_dtype,
                      int rows, int n, int bpr, int split, hipStream_t stream) {
    auto kern = iq_stream_matvec_kernel<FMT, NB, RAW>;
    const int tiles_per_chunk = kWaves / split;
    const int chunk_bytes = tiles_per_chunk * kRowsPerTile * bpr * FMT::kBlockBytes;
    const size_t head = staged_x_bytes(bpr * 256) + 16 + FMT::kTableBytes + kWaves * kRowsPerTile * sizeof(float);
    const int chunk_off = static_cast<int>((head + 1023) & ~static_cast<size_t>(1023));
    const int chunk_stride = chunk_bytes + 16;                               // shares are read as aligned dwords: a few bytes past the end
    const size_t smem = static_cast<size_t>(chunk_off) + 2 * chunk_stride;
    if (smem > 160 * 1024) return PLLM_ERR_UNSUPPORTED;
    static SmemGrant granted;
    if (!grant_dynamic_smem(reinterpret_cast<const void*>(kern), smem, granted)) return PLLM_ERR_UNSUPPORTED;
    // resident workgroups per compute unit for this LDS size: asked once per size (the query costs microseconds of host time)
    static size_t occ_smem = ~static_cast<size_t>(0);
    static int occ_per_cu = 1;
    if (smem != occ_smem) {
        int q = 0;
        occ_per_cu = (hipOccupancyMaxActiveBlocksPerMultiprocessor(&q, kern, 64 * kWaves, smem) == hipSuccess && q >= 1) ? q : 1;
        occ_smem = smem;
    }
    const int per_cu = occ_per_cu;
    const int chunks = (n / kRowsPerTile + tiles_per_chunk - 1) / tiles_per_chunk;
    const int resident = per_cu * compute_units();
    int grid = chunks;
    if (chunks > resident) {
        const int rounds = (chunks + resident - 1) / resident;
        grid = (chunks + rounds - 1) / rounds;
    }
    hipLaunchKernelGGL(kern, dim3(grid, rows), dim3(64 * kWaves), smem, stream, act, w, y, y_dtype, n, bpr, split, chunks,
                       chunk_off, chunk_stride);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

template <typename FMT, int NB>
int launch_stream_nb(const ActRows& act, const uint8_t* w, void* y, int y_dtype, int rows, int n, int bpr, int split, hipStream_t stream) {
    return act.x ? launch_stream_raw<FMT, NB, true>(act, w, y, y_dtype, rows, n, bpr, split, stream)
                 : launch_stream_raw<FMT, NB, false>(act, w, y, y_dtype, rows, n, bpr, split, stream);
}

template <typename FMT>
int launch_stream(const ActRows& act, const uint8_t* w, void* y, int y_dtype,
                  int rows, int n, int bpr, int split, hipStream_t stream) {
    const int per_wave = (bpr + split - 1) / split;                          // block indices a wave meets
    if constexpr (FMT::kHoldBlocks >= 2) if (per_wave <= 2) return launch_stream_nb<FMT, 2>(act, w, y, y_dtype, rows, n, bpr, split, stream);
    if constexpr (FMT::kHoldBlocks >= 3) if (per_wave == 3) return launch_stream_nb<FMT, 3>(act, w, y, y_dtype, rows, n, bpr, split, stream);
    return launch_stream_nb<FMT, 0>(act, w, y, y_dtype, rows, n, bpr, split, stream);
}

template <typename FMT>
int launch_fmt(const ActRows& act, const WeightRoute& route, const uint8_t* w, void* y, int y_dtype,
               int rows, int n, int bpr, hipStream_t stream) {
    // whole tiles streamed through long-lived workgroups (the codebooks are staged once per workgroup)
    // where shape and alignment allow, else one short workgroup per tile; routed calls and several projections in one launch
    // always take the latter
    if constexpr (FMT::kStreamed)
        if (!routed(route) && !act.row_token && !act.x_broadcast && route.extra == 0)
            if (const int split = stream_split<FMT>(w, n, bpr)) return launch_stream<FMT>(act, w, y, y_dtype, rows, n, bpr, split, stream);
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
