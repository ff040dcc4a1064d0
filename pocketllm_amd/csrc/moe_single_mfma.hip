// Routed experts of a single token with the integer dots on the matrix cores (IQ2_XXS / IQ1_M gate
// and up projections, IQ1_M down projection):
//     y = sum over routes r, in route order, of  W2_e ( silu(W1_e x) * (W3_e x) * w_r ),   e = expert of r.
// Two launches.  Both bring their weights into LDS with direct-to-LDS loads (the 16 rows of a tile
// are one contiguous run of memory) while the workgroup prepares the activation side, and take the
// lanes' block shares from there (lane map and per-format pieces: block_mfma.h).
//
//   moe_single_w13_kernel: one workgroup per (16 intermediate rows, route), eight waves = (matrix,
//     share of the row's super-blocks).  The workgroup quantizes the activation row into LDS itself
//     and reads the int64 expert ids as they come.  The epilogue applies the clamp, SiLU and the route
//     weight and quantizes the 16 hidden values in place, one scale per 16 values.
//   moe_single_w2_kernel: one workgroup per 16 output rows, sixteen waves = (route mod 8, block
//     parity), the hidden images of all routes in LDS; the waves' sums are added in wave order, so the
//     result does not depend on scheduling.
//
// Hidden image of one route (h_kpad = intermediate size rounded up to 256):
//     int8 hi[h_kpad] | int8 lo[h_kpad] | float xs16[h_kpad / 16] | float sum16[h_kpad / 16]
// with h[i] ~= 254 * xs16[i / 16] * (hi[i] + lo[i] / 254) and sum16 the exact sums: the image of
// pllm_device.h with one scale per 16 values instead of one per 32 (same size).
#include "block_mfma.h"
#include "pllm_internal.h"

namespace pllm {
namespace {

constexpr int kW13Waves = 8;
constexpr int kW2Waves = 16;

// Epilogue of one 16-row tile of one route, run by lanes 0..15 of a wave (lane = row inside the tile).
__device__ __forceinline__ void store_hidden16(float g, float u, float limit, float route_weight, int i, int inter,
                                               unsigned char* img, int h_kpad, int lane) {
    if (limit > 0.0f) {
        u = fminf(fmaxf(u, -limit), limit);
        g = fminf(g, limit);
    }
    const float h = (i < inter) ? g / (1.0f + expf(-g)) * u * route_weight : 0.0f;
    float am = fabsf(h), sum = h;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
        am = fmaxf(am, __shfl_xor(am, off, 64));
        sum += __shfl_xor(sum, off, 64);
    }
    const float inv = am > 0.0f ? 127.0f / am : 0.0f;
    const float scale = am * (1.0f / 127.0f);
    const float q = fminf(fmaxf(rintf(h * inv), -127.0f), 127.0f);
    const float l = fminf(fmaxf(rintf((h - q * scale) * inv * 254.0f), -127.0f), 127.0f);
    reinterpret_cast<int8_t*>(img)[i] = static_cast<int8_t>(static_cast<int>(q));
    reinterpret_cast<int8_t*>(img + h_kpad)[i] = static_cast<int8_t>(static_cast<int>(l));
    float* xs16 = reinterpret_cast<float*>(img + 2 * static_cast<size_t>(h_kpad));
    float* sum16 = xs16 + h_kpad / 16;
    if (lane == 0) { xs16[i >> 4] = scale * kLoInv; sum16[i >> 4] = sum; }
}

template <typename FMT>
__global__ __launch_bounds__(64 * kW13Waves) void moe_single_w13_kernel(
    const void* __restrict__ x, int x_dtype, int dim, int bpr, const int64_t* __restrict__ route_experts,
    const float* __restrict__ route_weights, const uint8_t* __restrict__ w1, const uint8_t* __restrict__ w3, int inter, float limit,
    unsigned char* __restrict__ h_image, size_t h_image_stride, int h_kpad, int raw_off, int tile_off, int tile_stride) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    const StagedX sx = carve_staged_x(smem, kpad);
    const int zero_off = image_bytes;                                        // 16 zero bytes
    const int table_off = image_bytes + 16;
    const unsigned char* tables = smem + table_off;
    float* exch = reinterpret_cast<float*>(smem + table_off + FMT::kTableBytes);   // [share][matrix][16]; then the raw activation row at raw_off
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte_ptr)smem));

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int col = lane & 15, ks = lane >> 4;
    const int mat = wave & 1, share = wave >> 1;
    const int route = blockIdx.y;
    const int row_bytes = bpr * FMT::kBlockBytes;
    const int tile_bytes = 16 * row_bytes;
    const size_t tile_pos = (static_cast<size_t>(route_experts[route]) * inter + static_cast<size_t>(blockIdx.x) * 16) * row_bytes;

    if (blockIdx.x * 16 >= inter) {          // padding rows of the hidden image: zeros, no weights behind them
        if (tid < 16) store_hidden16(0.0f, 0.0f, 0.0f, 0.0f, blockIdx.x * 16 + tid, inter, h_image + static_cast<size_t>(route) * h_image_stride, h_kpad, tid);
        return;
    }
    // the raw activation row, both matrices' tiles and the codebooks travel to LDS together
    dma_share<kW13Waves>(static_cast<const unsigned char*>(x), lds0 + raw_off, dim * (x_dtype == PLLM_F32 ? 4 : 2), wave, lane);
    dma_share<kW13Waves>(w1 + tile_pos, lds0 + tile_off, tile_bytes, wave, lane);
    dma_share<kW13Waves>(w3 + tile_pos, lds0 + tile_off + tile_stride, tile_bytes, wave, lane);
    FMT::template dma_tables<kW13Waves>(lds0 + table_off, wave, lane);
    if (tid < 4) reinterpret_cast<uint32_t*>(smem + zero_off)[tid] = 0;
    AMap<FMT::kSlots> am;
    FMT::a_map(am, col, ks, kpad, zero_off);
    wait_vm<0>();
    __syncthreads();
    quantize_row_to_lds(smem, smem + raw_off, x_dtype, 0, dim, kpad);       // LDS to LDS
    __syncthreads();

    const unsigned char* tile = smem + tile_off + mat * tile_stride;
    float acc = 0.0f;
    for (int b = share; b < bpr; b += kW13Waves / 2) {
        typename FMT::Regs regs;
        FMT::load_lds(regs, tile, col * row_bytes + b * FMT::kBlockBytes, ks);
        acc += FMT::block(regs, ks, b, smem, am, sx, tables);
    }
    acc += __shfl_xor(acc, 16, 64);
    acc += __shfl_xor(acc, 32, 64);
    if (ks == 0) exch[(share * 2 + mat) * 16 + col] = acc;
    __syncthreads();
    if (tid < 16) {
        float g = 0.0f, u = 0.0f;
#pragma unroll
        for (int v = 0; v < kW13Waves / 2; ++v) { g += exch[(v * 2) * 16 + tid]; u += exch[(v * 2 + 1) * 16 + tid]; }
        store_hidden16(g, u, limit, route_weights[route], blockIdx.x * 16 + tid, inter,
                       h_image + static_cast<size_t>(route) * h_image_stride, h_kpad, tid);
    }
}

// IQ1_M down projection.  LDS: the routes' hidden images | 16 zero bytes | codebook | partial sums | the routes' tiles.
__global__ __launch_bounds__(64 * kW2Waves) void moe_single_w2_kernel(
    const unsigned char* __restrict__ h_image, size_t h_image_stride, int bpr, const int64_t* __restrict__ route_experts, int routes,
    const uint8_t* __restrict__ w2, size_t expert_stride, float* __restrict__ y, int dim, int tile_off, int tile_stride) {
    using FMT = IQ1Mm;
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    const int zero_off = routes * image_bytes;
    const int table_off = zero_off + 16;
    const unsigned char* tables = smem + table_off;
    float* partial = reinterpret_cast<float*>(smem + table_off + FMT::kTableBytes);   // [waves][16]
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte_ptr)smem));

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int col = lane & 15, ks = lane >> 4;
    const int row_bytes = bpr * FMT::kBlockBytes;
    const int tile_bytes = 16 * row_bytes;
    const size_t tile_pos = static_cast<size_t>(blockIdx.x) * 16 * row_bytes;

    // 1 KB pieces of the routes' tiles and images, dealt round the waves
    const int tile_pieces = (tile_bytes + 1023) / 1024, image_pieces = (image_bytes + 1023) / 1024;
    for (int q = wave; q < routes * tile_pieces; q += kW2Waves) {
        const int r = q / tile_pieces, o = (q % tile_pieces) * 1024;
        if (o + lane * 16 < tile_bytes)
            lds_dma16(w2 + static_cast<size_t>(route_experts[r]) * expert_stride + tile_pos + o + lane * 16, lds0 + tile_off + r * tile_stride + o);
    }
    for (int q = wave; q < routes * image_pieces; q += kW2Waves) {
        const int r = q / image_pieces, o = (q % image_pieces) * 1024;
        if (o + lane * 16 < image_bytes) lds_dma16(h_image + static_cast<size_t>(r) * h_image_stride + o + lane * 16, lds0 + r * image_bytes + o);
    }
    FMT::dma_tables<kW2Waves>(lds0 + table_off, wave, lane);
    if (tid < 4) reinterpret_cast<uint32_t*>(smem + zero_off)[tid] = 0;
    wait_vm<0>();
    __syncthreads();

    float acc = 0.0f;
    for (int r = wave >> 1; r < routes; r += kW2Waves / 2) {
        const unsigned char* img = smem + r * image_bytes;
        AMap<FMT::kSlots> am;
        FMT::a_map(am, col, ks, kpad, zero_off - r * image_bytes);
        const float* xs16 = reinterpret_cast<const float*>(img + 2 * kpad);
        const unsigned char* tile = smem + tile_off + r * tile_stride;
        for (int b = wave & 1; b < bpr; b += 2) {
            FMT::Regs regs;
            FMT::load_lds(regs, tile, col * row_bytes + b * FMT::kBlockBytes, ks);
            uint4 ah[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) ah[t] = *reinterpret_cast<const uint4*>(img + am.off[t] + b * am.step[t]);
            v4i ch, cl;
            FMT::group_dots(regs, b, ah, img, am, tables, ch, cl);
            const float4 xs = *reinterpret_cast<const float4*>(xs16 + b * 16 + 4 * ks);
            acc += FMT::finish(regs, ks, ch, cl, make_float4(0.125f * xs.x, 0.125f * xs.y, 0.125f * xs.z, 0.125f * xs.w));
        }
    }
    acc += __shfl_xor(acc, 16, 64);
    acc += __shfl_xor(acc, 32, 64);
    if (ks == 0) partial[wave * 16 + col] = acc;
    __syncthreads();
    if (tid < 16) {
        float total = 0.0f;
#pragma unroll
        for (int v = 0; v < kW2Waves; ++v) total += partial[v * 16 + tid];
        y[blockIdx.x * 16 + tid] = total;
    }
}

// ---- several tokens: one pass of an expert's weights serves all its routes ---------------------------
// Routes are grouped by expert (seg[e] .. seg[e + 1]).  Workgroups are persistent and walk units =
// (expert, row tile(s)): the unit's weight tiles come to LDS by direct-to-LDS loads, every wave
// decodes its share of the blocks ONCE into registers (finished integer codes = B operands, scales),
// and the expert's routes then pass through in batches: their activation images come to LDS, every
// route costs only its MFMAs and a short epilogue.  The codebook lookups, which bound the single-token
// kernels, are paid once per expert instead of once per route.
constexpr int kGroupWaves = 8;
constexpr int kGroupBatch = 4;            // routes per batch, gate/up (an activation image of the model dimension each)
constexpr int kGroupBatch2 = 8;           // routes per batch, down projection
constexpr int kGroupBlocks = 3;           // block indices a wave may hold decoded, gate/up
constexpr int kGroupBlocks2 = 2;          // the same for the down projection (IQ1_M holds more per block: two workgroups per CU need <= 128 registers)

template <typename FMT, int NB>
__global__ __launch_bounds__(64 * kGroupWaves) void moe_grouped_w13_kernel(
    const unsigned char* __restrict__ x_image, size_t x_image_stride, int bpr, const int64_t* __restrict__ route_tokens,
    const int32_t* __restrict__ seg, const float* __restrict__ route_weights, const uint8_t* __restrict__ w1, const uint8_t* __restrict__ w3,
    int inter, float limit, unsigned char* __restrict__ h_image, size_t h_image_stride, int h_kpad, int n_experts,
    int table_off, int tile_off, int tile_stride) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    const int slot_stride = image_bytes + 16;                               // every image slot ends in 16 zero bytes
    const unsigned char* tables = smem + table_off;
    float* exch = reinterpret_cast<float*>(smem + table_off + FMT::kTableBytes);   // [batch][share][matrix][16]
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte_ptr)smem));

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int col = lane & 15, ks = lane >> 4;
    const int mat = wave & 1, share = wave >> 1;
    constexpr int kShares = kGroupWaves / 2;
    const int row_bytes = bpr * FMT::kBlockBytes;
    const int tile_bytes = 16 * row_bytes;
    const int tiles = h_kpad / 16;

    FMT::template dma_tables<kGroupWaves>(lds0 + table_off, wave, lane);
    if (tid < 4 * kGroupBatch) reinterpret_cast<uint32_t*>(smem + (tid >> 2) * slot_stride + image_bytes)[tid & 3] = 0;
    AMap<FMT::kSlots> am;
    FMT::a_map(am, col, ks, kpad, image_bytes);
    AOps<FMT::kSlots> ops;
    clear_a(ops);

    for (int unit = blockIdx.x; unit < n_experts * tiles; unit += gridDim.x) {
        const int expert = unit / tiles, tile = unit % tiles;
        const int r0 = seg[expert], r1 = seg[expert + 1];
        if (r0 >= r1) continue;
        if (tile * 16 >= inter) {            // padding rows of the hidden images: zeros, no weights behind them
            for (int i = tid; i < 16 * (r1 - r0); i += blockDim.x)
                store_hidden16(0.0f, 0.0f, 0.0f, 0.0f, tile * 16 + (i & 15), inter, h_image + static_cast<size_t>(r0 + (i >> 4)) * h_image_stride, h_kpad, i & 15);
            continue;
        }
        const size_t tile_pos = (static_cast<size_t>(expert) * inter + static_cast<size_t>(tile) * 16) * row_bytes;
        dma_share<kGroupWaves>(w1 + tile_pos, lds0 + tile_off, tile_bytes, wave, lane);
        dma_share<kGroupWaves>(w3 + tile_pos, lds0 + tile_off + tile_stride, tile_bytes, wave, lane);
        wait_vm<0>();
        __syncthreads();
        typename FMT::Decoded dec[NB];
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            typename FMT::Regs regs;
            FMT::load_lds(regs, smem + tile_off + mat * tile_stride, col * row_bytes + min(share + kShares * i, bpr - 1) * FMT::kBlockBytes, ks);
            FMT::decode(regs, ks, tables, dec[i]);
        }
        for (int rc = r0; rc < r1; rc += kGroupBatch) {
            const int nr = min(kGroupBatch, r1 - rc);
            for (int q = 0; q < nr; ++q)
                dma_share<kGroupWaves>(x_image + static_cast<size_t>(route_tokens[rc + q]) * x_image_stride, lds0 + q * slot_stride, image_bytes, wave, lane);
            wait_vm<0>();
            __syncthreads();                 // images landed; every wave has left the previous batch's epilogue and the decode
            for (int q = 0; q < nr; ++q) {
                const unsigned char* img = smem + q * slot_stride;
                float acc = 0.0f;
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    const int b = share + kShares * i;
                    if (b < bpr) acc += FMT::route_block(dec[i], ks, b, img, am, kpad, ops);   // wave-uniform
                }
                acc += __shfl_xor(acc, 16, 64);
                acc += __shfl_xor(acc, 32, 64);
                if (ks == 0) exch[((q * kShares + share) * 2 + mat) * 16 + col] = acc;
            }
            __syncthreads();
            if (tid < 16 * nr) {
                const int q = tid >> 4, c = tid & 15;
                float g = 0.0f, u = 0.0f;
#pragma unroll
                for (int v = 0; v < kShares; ++v) { g += exch[((q * kShares + v) * 2) * 16 + c]; u += exch[((q * kShares + v) * 2 + 1) * 16 + c]; }
                store_hidden16(g, u, limit, route_weights[rc + q], tile * 16 + c, inter, h_image + static_cast<size_t>(rc + q) * h_image_stride, h_kpad, c);
            }
        }
    }
}

// partial[r, :] = W2_e h_r for the routes r of expert e (IQ1_M).  Unit = (expert, group of 8 / shares tiles).
template <int NB>
__global__ __launch_bounds__(64 * kGroupWaves) void moe_grouped_w2_kernel(
    const unsigned char* __restrict__ h_image, size_t h_image_stride, int bpr, const int32_t* __restrict__ seg,
    const uint8_t* __restrict__ w2, size_t expert_stride, float* __restrict__ partial, int dim, int n_experts, int shares,
    int table_off, int tile_off) {
    using FMT = IQ1Mm;
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    const int slot_stride = image_bytes + 16;
    const unsigned char* tables = smem + table_off;
    float* exch = reinterpret_cast<float*>(smem + table_off + FMT::kTableBytes);   // [batch][wave][16]
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte_ptr)smem));

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int col = lane & 15, ks = lane >> 4;
    const int tiles_per_unit = kGroupWaves / shares;
    const int tile_in_unit = wave / shares, share = wave % shares;
    const int row_bytes = bpr * FMT::kBlockBytes;
    const int unit_rows = tiles_per_unit * 16;
    const int units_per_expert = (dim + unit_rows - 1) / unit_rows;

    FMT::dma_tables<kGroupWaves>(lds0 + table_off, wave, lane);
    if (tid < 4 * kGroupBatch2) reinterpret_cast<uint32_t*>(smem + (tid >> 2) * slot_stride + image_bytes)[tid & 3] = 0;
    AMap<FMT::kSlots> am;
    FMT::a_map(am, col, ks, kpad, image_bytes);
    AOps<FMT::kSlots> ops;
    clear_a(ops);

    for (int unit = blockIdx.x; unit < n_experts * units_per_expert; unit += gridDim.x) {
        const int expert = unit / units_per_expert, row0 = (unit % units_per_expert) * unit_rows;
        const int r0 = seg[expert], r1 = seg[expert + 1];
        if (r0 >= r1) continue;
        const int valid_rows = min(unit_rows, dim - row0);                  // a multiple of 16
        dma_share<kGroupWaves>(w2 + static_cast<size_t>(expert) * expert_stride + static_cast<size_t>(row0) * row_bytes, lds0 + tile_off,
                               valid_rows * row_bytes, wave, lane);
        wait_vm<0>();
        __syncthreads();
        const bool live = tile_in_unit * 16 < valid_rows;                   // wave-uniform
        FMT::Decoded dec[NB];
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            FMT::Regs regs;
            FMT::load_lds(regs, smem + tile_off, ((live ? tile_in_unit : 0) * 16 + col) * row_bytes + min(share + shares * i, bpr - 1) * FMT::kBlockBytes, ks);
            FMT::decode(regs, ks, tables, dec[i]);
        }
        for (int rc = r0; rc < r1; rc += kGroupBatch2) {
            const int nr = min(kGroupBatch2, r1 - rc);
            for (int q = 0; q < nr; ++q)
                dma_share<kGroupWaves>(h_image + static_cast<size_t>(rc + q) * h_image_stride, lds0 + q * slot_stride, image_bytes, wave, lane);
            wait_vm<0>();
            __syncthreads();
            if (live)
                for (int q = 0; q < nr; ++q) {
                    const unsigned char* img = smem + q * slot_stride;
                    float acc = 0.0f;
#pragma unroll
                    for (int i = 0; i < NB; ++i) {
                        const int b = share + shares * i;
                        if (b < bpr) acc += FMT::route_block16(dec[i], ks, b, img, am, kpad, ops);
                    }
                    acc += __shfl_xor(acc, 16, 64);
                    acc += __shfl_xor(acc, 32, 64);
                    if (ks == 0) exch[(q * kGroupWaves + wave) * 16 + col] = acc;
                }
            __syncthreads();
            for (int i = tid; i < nr * valid_rows; i += blockDim.x) {
                const int q = i / valid_rows, r = i % valid_rows, t = r >> 4, c = r & 15;
                float total = 0.0f;
                for (int v = 0; v < shares; ++v) total += exch[(q * kGroupWaves + t * shares + v) * 16 + c];
                partial[static_cast<size_t>(rc + q) * dim + row0 + r] = total;
            }
        }
    }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <typename KERN>
bool allow_lds(KERN kern, size_t smem) {
    if (smem > 160 * 1024) return false;
    return smem <= 64 * 1024 ||
           hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem)) == hipSuccess;
}

template <typename FMT>
int launch_single_w13(const void* x, int x_dtype, int dim, int bpr, const int64_t* route_experts, const float* route_weights, int routes,
                      const uint8_t* w1, const uint8_t* w3, int inter, float limit, unsigned char* h_image, size_t h_stride, int h_kpad,
                      hipStream_t stream) {
    const int tile_bytes = 16 * bpr * FMT::kBlockBytes;
    const size_t head = staged_x_bytes(bpr * 256) + 16 + FMT::kTableBytes + (kW13Waves / 2) * 2 * 16 * sizeof(float);
    const int raw_off = static_cast<int>((head + 15) & ~static_cast<size_t>(15));
    const int tile_off = (raw_off + dim * (x_dtype == PLLM_F32 ? 4 : 2) + 1023) & ~1023;
    const int tile_stride = tile_bytes + 16;                                 // shares are read as aligned dwords: a few bytes past the end
    const size_t smem = static_cast<size_t>(tile_off) + 2 * tile_stride;
    auto kern = moe_single_w13_kernel<FMT>;
    if (!allow_lds(kern, smem)) return PLLM_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(kern, dim3(h_kpad / 16, routes), dim3(64 * kW13Waves), smem, stream, x, x_dtype, dim, bpr, route_experts, route_weights,
                       w1, w3, inter, limit, h_image, h_stride, h_kpad, raw_off, tile_off, tile_stride);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

// workgroups of a persistent kernel that fit the device at once
// (asked again only when kernel, threads or LDS size change: the query costs microseconds of host time)
template <typename KERN>
int resident_workgroups(KERN kern, int threads, size_t smem) {
    static const void* asked_kern = nullptr;                 // kernels of one signature share this instantiation
    static size_t asked_smem = ~static_cast<size_t>(0);
    static int asked_threads = 0, per_cu = 1;
    if (reinterpret_cast<const void*>(kern) != asked_kern || smem != asked_smem || threads != asked_threads) {
        int q = 0;
        per_cu = (hipOccupancyMaxActiveBlocksPerMultiprocessor(&q, kern, threads, smem) == hipSuccess && q >= 1) ? q : 1;
        asked_kern = reinterpret_cast<const void*>(kern);
        asked_smem = smem;
        asked_threads = threads;
    }
    return per_cu * compute_units();
}

struct GroupedW13Plan { int nb, table_off, tile_off, tile_stride; size_t smem; };

template <typename FMT>
GroupedW13Plan plan_grouped_w13(int bpr) {
    GroupedW13Plan p;
    p.nb = (bpr + kGroupWaves / 2 - 1) / (kGroupWaves / 2);
    const int slots = kGroupBatch * (static_cast<int>(staged_x_bytes(bpr * 256)) + 16);
    p.table_off = slots;
    const int head = slots + FMT::kTableBytes + kGroupBatch * (kGroupWaves / 2) * 2 * 16 * static_cast<int>(sizeof(float));
    p.tile_off = (head + 1023) & ~1023;
    p.tile_stride = 16 * bpr * FMT::kBlockBytes + 16;
    p.smem = static_cast<size_t>(p.tile_off) + 2 * p.tile_stride;
    return p;
}

template <typename FMT, int NB>
int launch_grouped_w13_nb(const GroupedW13Plan& p, const unsigned char* x_image, size_t x_stride, int bpr, const int64_t* route_tokens, const int32_t* seg,
                          const float* route_weights, const uint8_t* w1, const uint8_t* w3, int inter, float limit, unsigned char* h_image,
                          size_t h_stride, int h_kpad, int n_experts, hipStream_t stream) {
    auto kern = moe_grouped_w13_kernel<FMT, NB>;
    if (!allow_lds(kern, p.smem)) return PLLM_ERR_UNSUPPORTED;
    const int units = n_experts * (h_kpad / 16);
    const int grid = min(units, resident_workgroups(kern, 64 * kGroupWaves, p.smem));
    hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * kGroupWaves), p.smem, stream, x_image, x_stride, bpr, route_tokens, seg, route_weights, w1, w3, inter,
                       limit, h_image, h_stride, h_kpad, n_experts, p.table_off, p.tile_off, p.tile_stride);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

template <typename FMT>
int launch_grouped_w13(const unsigned char* x_image, size_t x_stride, int bpr, const int64_t* route_tokens, const int32_t* seg,
                       const float* route_weights, const uint8_t* w1, const uint8_t* w3, int inter, float limit, unsigned char* h_image,
                       size_t h_stride, int h_kpad, int n_experts, hipStream_t stream) {
    const GroupedW13Plan p = plan_grouped_w13<FMT>(bpr);
#define PLLM_CASE(N) case N: return launch_grouped_w13_nb<FMT, N>(p, x_image, x_stride, bpr, route_tokens, seg, route_weights, w1, w3, inter, limit, h_image, h_stride, h_kpad, n_experts, stream)
    switch (p.nb) {
        PLLM_CASE(1); PLLM_CASE(2); PLLM_CASE(3);
        default: return PLLM_ERR_UNSUPPORTED;
    }
#undef PLLM_CASE
}

struct GroupedW2Plan { int nb, shares, table_off, tile_off; size_t smem; };

GroupedW2Plan plan_grouped_w2(int bpr) {
    GroupedW2Plan p;
    p.shares = 1;
    while (p.shares < kGroupWaves && (bpr + p.shares - 1) / p.shares > kGroupBlocks2) p.shares *= 2;
    p.nb = (bpr + p.shares - 1) / p.shares;
    const int slots = kGroupBatch2 * (static_cast<int>(staged_x_bytes(bpr * 256)) + 16);
    p.table_off = slots;
    const int head = slots + IQ1Mm::kTableBytes + kGroupBatch2 * kGroupWaves * 16 * static_cast<int>(sizeof(float));
    p.tile_off = (head + 1023) & ~1023;
    p.smem = static_cast<size_t>(p.tile_off) + static_cast<size_t>(kGroupWaves / p.shares) * 16 * bpr * IQ1Mm::kBlockBytes + 16;
    return p;
}

template <int NB>
int launch_grouped_w2_nb(const GroupedW2Plan& p, const unsigned char* h_image, size_t h_stride, int bpr, const int32_t* seg, const uint8_t* w2,
                         float* partial, int dim, int n_experts, hipStream_t stream) {
    auto kern = moe_grouped_w2_kernel<NB>;
    if (!allow_lds(kern, p.smem)) return PLLM_ERR_UNSUPPORTED;
    const int unit_rows = (kGroupWaves / p.shares) * 16;
    const int units = n_experts * ((dim + unit_rows - 1) / unit_rows);
    const int grid = min(units, resident_workgroups(kern, 64 * kGroupWaves, p.smem));
    const size_t expert_stride = static_cast<size_t>(dim) * bpr * IQ1Mm::kBlockBytes;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * kGroupWaves), p.smem, stream, h_image, h_stride, bpr, seg, w2, expert_stride, partial, dim, n_experts,
                       p.shares, p.table_off, p.tile_off);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

}  // namespace

bool moe_single_mfma_supports(int w13_type, int w2_type, int dim, int inter, int routes, const void* x, const uint8_t* w1,
                              const uint8_t* w3, const uint8_t* w2) {
    if (w2_type != PLLM_TYPE_IQ1_M || (w13_type != PLLM_TYPE_IQ2_XXS && w13_type != PLLM_TYPE_IQ1_M)) return false;
    // whole 16-row tiles on both sides, 16-byte aligned tiles
    if (dim % 16 != 0 || inter % 16 != 0 || !aligned16(x) || !aligned16(w1) || !aligned16(w3) || !aligned16(w2) || routes < 1) return false;
    const int bpr_x = (dim + 255) / 256, bpr_h = (inter + 255) / 256;
    const int w13_block = w13_type == PLLM_TYPE_IQ2_XXS ? IQ2XXSm::kBlockBytes : IQ1Mm::kBlockBytes;
    const int w13_tables = w13_type == PLLM_TYPE_IQ2_XXS ? IQ2XXSm::kTableBytes : IQ1Mm::kTableBytes;
    const size_t smem13 = staged_x_bytes(bpr_x * 256) + 2048 + w13_tables + 4 * static_cast<size_t>(dim) + 2 * (16 * bpr_x * w13_block + 16);
    const size_t smem2 = static_cast<size_t>(routes) * (staged_x_bytes(bpr_h * 256) + 16 * bpr_h * IQ1Mm::kBlockBytes + 16) + 2048 +
                         IQ1Mm::kTableBytes + kW2Waves * 16 * sizeof(float);
    return smem13 <= 150 * 1024 && smem2 <= 150 * 1024;
}

int moe_single_w13_mfma(const void* x, int x_dtype, int dim, const int64_t* route_experts, const float* route_weights, int routes,
                        const uint8_t* w1, const uint8_t* w3, int w13_type, int inter, float limit, unsigned char* h_image, size_t h_stride,
                        hipStream_t stream) {
    const int bpr = (dim + 255) / 256, h_kpad = (inter + 255) / 256 * 256;
    if (w13_type == PLLM_TYPE_IQ2_XXS)
        return launch_single_w13<IQ2XXSm>(x, x_dtype, dim, bpr, route_experts, route_weights, routes, w1, w3, inter, limit, h_image, h_stride, h_kpad, stream);
    return launch_single_w13<IQ1Mm>(x, x_dtype, dim, bpr, route_experts, route_weights, routes, w1, w3, inter, limit, h_image, h_stride, h_kpad, stream);
}

int moe_single_w2_mfma(const unsigned char* h_image, size_t h_stride, int inter, const int64_t* route_experts, int routes, const uint8_t* w2,
                       float* y, int dim, hipStream_t stream) {
    const int bpr = (inter + 255) / 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(bpr * 256));
    const int tile_bytes = 16 * bpr * IQ1Mm::kBlockBytes;
    const size_t head = static_cast<size_t>(routes) * image_bytes + 16 + IQ1Mm::kTableBytes + kW2Waves * 16 * sizeof(float);
    const int tile_off = static_cast<int>((head + 1023) & ~static_cast<size_t>(1023));
    const int tile_stride = tile_bytes + 16;
    const size_t smem = static_cast<size_t>(tile_off) + static_cast<size_t>(routes) * tile_stride;
    if (!allow_lds(moe_single_w2_kernel, smem)) return PLLM_ERR_UNSUPPORTED;
    const size_t expert_stride = static_cast<size_t>(dim) * bpr * IQ1Mm::kBlockBytes;
    hipLaunchKernelGGL(moe_single_w2_kernel, dim3(dim / 16), dim3(64 * kW2Waves), smem, stream, h_image, h_stride, bpr, route_experts, routes, w2,
                       expert_stride, y, dim, tile_off, tile_stride);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

bool moe_grouped_mfma_supports(int w13_type, int w2_type, int dim, int inter, const uint8_t* w1, const uint8_t* w3, const uint8_t* w2) {
    if (w2_type != PLLM_TYPE_IQ1_M || (w13_type != PLLM_TYPE_IQ2_XXS && w13_type != PLLM_TYPE_IQ1_M)) return false;
    if (dim % 16 != 0 || inter % 16 != 0 || !aligned16(w1) || !aligned16(w3) || !aligned16(w2)) return false;
    const int bpr_x = (dim + 255) / 256, bpr_h = (inter + 255) / 256;
    const GroupedW13Plan p13 = w13_type == PLLM_TYPE_IQ2_XXS ? plan_grouped_w13<IQ2XXSm>(bpr_x) : plan_grouped_w13<IQ1Mm>(bpr_x);
    const GroupedW2Plan p2 = plan_grouped_w2(bpr_h);
    return p13.nb <= kGroupBlocks && p2.nb <= kGroupBlocks2 && p13.smem <= 150 * 1024 && p2.smem <= 150 * 1024;
}

int moe_grouped_w13_mfma(const unsigned char* x_image, size_t x_stride, int dim, const int64_t* route_tokens, const int32_t* seg,
                         const float* route_weights, const uint8_t* w1, const uint8_t* w3, int w13_type, int inter, float limit,
                         unsigned char* h_image, size_t h_stride, int n_experts, hipStream_t stream) {
    const int bpr = (dim + 255) / 256, h_kpad = (inter + 255) / 256 * 256;
    if (w13_type == PLLM_TYPE_IQ2_XXS)
        return launch_grouped_w13<IQ2XXSm>(x_image, x_stride, bpr, route_tokens, seg, route_weights, w1, w3, inter, limit, h_image, h_stride, h_kpad, n_experts, stream);
    return launch_grouped_w13<IQ1Mm>(x_image, x_stride, bpr, route_tokens, seg, route_weights, w1, w3, inter, limit, h_image, h_stride, h_kpad, n_experts, stream);
}

int moe_grouped_w2_mfma(const unsigned char* h_image, size_t h_stride, int inter, const int32_t* seg, const uint8_t* w2, float* partial, int dim,
                        int n_experts, hipStream_t stream) {
    const int bpr = (inter + 255) / 256;
    const GroupedW2Plan p = plan_grouped_w2(bpr);
    switch (p.nb) {
        case 1: return launch_grouped_w2_nb<1>(p, h_image, h_stride, bpr, seg, w2, partial, dim, n_experts, stream);
        case 2: return launch_grouped_w2_nb<2>(p, h_image, h_stride, bpr, seg, w2, partial, dim, n_experts, stream);
        default: return PLLM_ERR_UNSUPPORTED;
    }
}

}  // namespace pllm
