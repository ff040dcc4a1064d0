// Decode matvec over raw IQ2_XXS / IQ1_M super-blocks with the integer dots on the matrix cores.
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
constexpr int kMaxRounds = 16;           // row-tile groups one workgroup works through at most

// The lane's share of ITERS super-blocks of one row tile: blocks part + (pass * ITERS + it) * split
// (clamped: always a valid address)
template <typename FMT, int ITERS>
__device__ __forceinline__ void load_unit(typename FMT::Regs (&regs)[ITERS], const uint8_t* __restrict__ w, int n, int bpr,
                                          int tile, int col, int ks, int part, int split, int pass) {
    const int row = tile * kRowsPerTile + col;
    const uint8_t* wrow = w + static_cast<size_t>(row < n ? row : 0) * bpr * FMT::kBlockBytes;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int b = min(part + (pass * ITERS + it) * split, bpr - 1);
        FMT::load(regs[it], wrow + static_cast<size_t>(b) * FMT::kBlockBytes, ks);
    }
}

// A workgroup of 8 waves stages the activation image and the codebooks once and then works through
// `rounds` groups of row tiles (group = blockIdx.x + round * gridDim.x, 8 / split tiles of 16 rows
// each): `split` waves share a tile's super-blocks.  The blocks of the next unit of work are loaded
// while the current one is computed.
template <typename FMT, int ITERS>
__global__ __launch_bounds__(64 * kWaves) void iq_mfma_matvec_kernel(
    const unsigned char* __restrict__ image, size_t image_stride, const uint8_t* __restrict__ w,
    void* __restrict__ y, int y_dtype, int n, int bpr, int split, int groups) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    const StagedX sx = carve_staged_x(smem, kpad);
    const int zero_off = image_bytes;                                        // 16 zero bytes
    unsigned char* tables = smem + image_bytes + 16;
    float* partial = reinterpret_cast<float*>(tables + FMT::kTableBytes);   // [rounds][waves][16]

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int col = lane & 15;        // B/C column = output row within the tile; also A's row index m
    const int ks = lane >> 4;         // k slice of A and B, row quad of C
    const int tiles_per_group = kWaves / split;
    const int tile_in_group = wave / split, part = wave % split;
    const int passes = (bpr + split * ITERS - 1) / (split * ITERS);
    const int rounds = (groups - static_cast<int>(blockIdx.x) + static_cast<int>(gridDim.x) - 1) / static_cast<int>(gridDim.x);
    const int units = rounds * passes;
    const int tile0 = blockIdx.x * tiles_per_group + tile_in_group, tile_step = gridDim.x * tiles_per_group;

    // A side: this lane supplies row m = col of every MFMA, slice ks; the format says which rows are its
    AMap<FMT::kSlots> am;
    FMT::a_map(am, col, ks, kpad, zero_off);

    typename FMT::Regs cur[ITERS], nxt[ITERS];
    load_unit<FMT, ITERS>(cur, w, n, bpr, tile0, col, ks, part, split, 0);
    copy_to_lds(smem, image + static_cast<size_t>(blockIdx.y) * image_stride, image_bytes);
    if (tid < 4) reinterpret_cast<uint32_t*>(smem + zero_off)[tid] = 0;
    FMT::stage_tables(tables);
    __syncthreads();

    float acc = 0.0f;
    int round = 0, pass = 0;
    for (int u = 0; u < units; ++u) {
        int next_round = round, next_pass = pass + 1;
        if (next_pass == passes) { next_pass = 0; ++next_round; }
        if (u + 1 < units) load_unit<FMT, ITERS>(nxt, w, n, bpr, tile0 + next_round * tile_step, col, ks, part, split, next_pass);
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            // no branch around a block past the row's end (its registers hold the clamped block's data):
            // the blocks of a unit are then free to overlap; its result is dropped
            const int b = part + (pass * ITERS + it) * split;
            const float v = FMT::block(cur[it], ks, min(b, bpr - 1), smem, am, sx, tables);
            acc += b < bpr ? v : 0.0f;
        }
        if (next_pass == 0) {                                                // the tile's last pass
            acc += __shfl_xor(acc, 16, 64);
            acc += __shfl_xor(acc, 32, 64);
            if (split == 1) {
                const int row = (tile0 + round * tile_step) * kRowsPerTile + col;
                if (ks == 0 && row < n) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + row, acc);
            } else if (ks == 0) {
                partial[(round * kWaves + wave) * kRowsPerTile + col] = acc;
            }
            acc = 0.0f;
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) cur[it] = nxt[it];
        round = next_round; pass = next_pass;
    }
    if (split == 1) return;
    __syncthreads();
    // thread i sums the `split` partials of (round, tile in group, row) = i
    for (int i = tid; i < rounds * tiles_per_group * kRowsPerTile; i += blockDim.x) {
        const int r = i / (tiles_per_group * kRowsPerTile), rest = i % (tiles_per_group * kRowsPerTile);
        const int t = rest / kRowsPerTile, c = rest % kRowsPerTile;
        float total = 0.0f;
        for (int v = 0; v < split; ++v) total += partial[(r * kWaves + t * split + v) * kRowsPerTile + c];
        const int row = ((blockIdx.x + r * gridDim.x) * tiles_per_group + t) * kRowsPerTile + c;
        if (row < n) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + row, total);
    }
}

template <typename FMT, int ITERS>
int launch_one(const unsigned char* image, size_t image_stride, const uint8_t* w, void* y, int y_dtype,
               int rows, int n, int bpr, int split, hipStream_t stream) {
    auto kern = iq_mfma_matvec_kernel<FMT, ITERS>;
    const size_t fixed = staged_x_bytes(bpr * 256) + 16 + FMT::kTableBytes;
    // workgroups that fit the device at once (per kernel, asked once)
    static int resident = 0;
    if (resident == 0) {
        int per_cu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, 64 * kWaves, fixed + 4096) != hipSuccess || per_cu < 1) per_cu = 2;
        resident = per_cu * compute_units();
    }
    const int tiles = (n + kRowsPerTile - 1) / kRowsPerTile;
    const int groups = (tiles * split + kWaves - 1) / kWaves;
    int grid = groups;
    if (groups > resident) {
        const int rounds = min(kMaxRounds, (groups + resident - 1) / resident);
        grid = (groups + rounds - 1) / rounds;
    }
    const int rounds = (groups + grid - 1) / grid;
    const size_t smem = fixed + (split > 1 ? static_cast<size_t>(rounds) * kWaves * kRowsPerTile * sizeof(float) : 0);
    if (smem > 64 * 1024) {
        if (smem > 160 * 1024) return PLLM_ERR_UNSUPPORTED;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(smem)) != hipSuccess)
            return PLLM_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL(kern, dim3(grid, rows), dim3(64 * kWaves), smem, stream, image, image_stride, w, y, y_dtype, n, bpr, split, groups);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
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
template <typename FMT, int NB>
__global__ __launch_bounds__(64 * kWaves) void iq_stream_matvec_kernel(
    const unsigned char* __restrict__ image, size_t image_stride, const uint8_t* __restrict__ w,
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
    dma_share<kWaves>(image + static_cast<size_t>(blockIdx.y) * image_stride, lds0, image_bytes, wave, lane);
    FMT::template dma_tables<kWaves>(lds0 + table_off, wave, lane);
    if (tid < 4) reinterpret_cast<uint32_t*>(smem + zero_off)[tid] = 0;
    AMap<FMT::kSlots> am;
    FMT::a_map(am, col, ks, kpad, zero_off);

    int c = blockIdx.x, buf = 0;
    dma_share<kWaves>(w + static_cast<size_t>(c) * chunk_rows * row_bytes, lds0 + chunk_off, min(chunk_rows, n - c * chunk_rows) * row_bytes, wave, lane);
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
        if (NB > 0 && !holding) {
#pragma unroll
            for (int i = 0; i < NB; ++i) FMT::hold(held[i], ks, min(part + i * split, bpr - 1), smem, am, sx);
            holding = true;
        }

        const unsigned char* chunk = smem + chunk_off + buf * chunk_stride;
        float acc = 0.0f;
        if (tile_in_chunk * kRowsPerTile < valid_rows) {                     // wave-uniform
            const int row_off = (tile_in_chunk * kRowsPerTile + col) * row_bytes;
            if (NB > 0) {
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
    // the most waves per tile first (smallest chunk) that leaves every wave at least three blocks
    for (int split = kWaves; split >= 1; split /= 2)
        if ((split == 1 || bpr >= 3 * split) && (kWaves / split) * tile_bytes <= kChunkBudget) return split;
    return 0;
}

template <typename FMT, int NB>
int launch_stream_nb(const unsigned char* image, size_t image_stride, const uint8_t* w, void* y, int y_dtype,
                     int rows, int n, int bpr, int split, hipStream_t stream) {
    auto kern = iq_stream_matvec_kernel<FMT, NB>;
    const int tiles_per_chunk = kWaves / split;
    const int chunk_bytes = tiles_per_chunk * kRowsPerTile * bpr * FMT::kBlockBytes;
    const size_t head = staged_x_bytes(bpr * 256) + 16 + FMT::kTableBytes + kWaves * kRowsPerTile * sizeof(float);
    const int chunk_off = static_cast<int>((head + 1023) & ~static_cast<size_t>(1023));
    const int chunk_stride = chunk_bytes + 16;                               // shares are read as aligned dwords: a few bytes past the end
    const size_t smem = static_cast<size_t>(chunk_off) + 2 * chunk_stride;
    if (smem > 160 * 1024) return PLLM_ERR_UNSUPPORTED;
    static size_t attr_smem = 0;
    if (smem > 64 * 1024 && smem > attr_smem) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(smem)) != hipSuccess)
            return PLLM_ERR_UNSUPPORTED;
        attr_smem = smem;
    }
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, 64 * kWaves, smem) != hipSuccess || per_cu < 1) per_cu = 1;
    const int chunks = (n / kRowsPerTile + tiles_per_chunk - 1) / tiles_per_chunk;
    const int resident = per_cu * compute_units();
    int grid = chunks;
    if (chunks > resident) {
        const int rounds = (chunks + resident - 1) / resident;
        grid = (chunks + rounds - 1) / rounds;
    }
    hipLaunchKernelGGL(kern, dim3(grid, rows), dim3(64 * kWaves), smem, stream, image, image_stride, w, y, y_dtype, n, bpr, split, chunks,
                       chunk_off, chunk_stride);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

template <typename FMT>
int launch_stream(const unsigned char* image, size_t image_stride, const uint8_t* w, void* y, int y_dtype,
                  int rows, int n, int bpr, int split, hipStream_t stream) {
    const int per_wave = (bpr + split - 1) / split;                          // block indices a wave meets
    if (FMT::kHoldBlocks >= 2 && per_wave <= 2) return launch_stream_nb<FMT, 2>(image, image_stride, w, y, y_dtype, rows, n, bpr, split, stream);
    if (FMT::kHoldBlocks >= 3 && per_wave == 3) return launch_stream_nb<FMT, 3>(image, image_stride, w, y, y_dtype, rows, n, bpr, split, stream);
    return launch_stream_nb<FMT, 0>(image, image_stride, w, y, y_dtype, rows, n, bpr, split, stream);
}

template <typename FMT>
int launch_fmt(const unsigned char* image, size_t image_stride, const uint8_t* w, void* y, int y_dtype,
               int rows, int n, int bpr, hipStream_t stream) {
    if (const int split = stream_split<FMT>(w, n, bpr)) return launch_stream<FMT>(image, image_stride, w, y, y_dtype, rows, n, bpr, split, stream);
    // waves per row tile: one when there are tiles enough to keep every wave of the device busy
    // several times over, more (each with at least two super-blocks) for short matrices
    const int tiles = (n + kRowsPerTile - 1) / kRowsPerTile;
    const int want = 6 * compute_units();
    int split = 1;
    while (split < kWaves && split * 4 <= bpr && (tiles * split + kWaves - 1) / kWaves * rows < want) split *= 2;
    const int niter = (bpr + split - 1) / split;
    const int passes = (niter + 3) / 4;
    const int iters = (niter + passes - 1) / passes;
#define PLLM_CASE(I) case I: return launch_one<FMT, I>(image, image_stride, w, y, y_dtype, rows, n, bpr, split, stream)
    switch (iters) {
        PLLM_CASE(1); PLLM_CASE(2); PLLM_CASE(3);
        default: return launch_one<FMT, 4>(image, image_stride, w, y, y_dtype, rows, n, bpr, split, stream);
    }
#undef PLLM_CASE
}

}  // namespace

int iq_mfma_matvec_from_image(const unsigned char* image, size_t stride, const uint8_t* w, int type_id, void* y, int y_dtype,
                              int rows, int n, int bpr, hipStream_t stream) {
    switch (type_id) {
        case PLLM_TYPE_IQ2_XXS: return launch_fmt<IQ2XXSm>(image, stride, w, y, y_dtype, rows, n, bpr, stream);
        case PLLM_TYPE_IQ1_M: return launch_fmt<IQ1Mm>(image, stride, w, y, y_dtype, rows, n, bpr, stream);
        default: return PLLM_ERR_UNSUPPORTED;
    }
}

}  // namespace pllm
