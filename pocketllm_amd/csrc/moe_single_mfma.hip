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
    am = group_max<16>(am);
    sum = group_sum<16>(sum);
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
    // the arguments in one batch of scalar loads, one wait (not the route tables: their reads must stay scalar loads)
    asm volatile("" : : "s"(x), "s"(x_dtype), "s"(dim), "s"(bpr), "s"(w1), "s"(w3), "s"(inter), "s"(h_image), "s"(h_image_stride), "s"(h_kpad),
                 "s"(raw_off), "s"(tile_off), "s"(tile_stride));
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
    // the raw activation row, the codebooks and both matrices' tiles travel to LDS together; the row is requested first and
    // quantized (LDS to LDS) while the tiles are still on their way: loads complete in order, so "all but the tiles'
    // instructions" means the row has landed
    dma_share<kW13Waves>(static_cast<const unsigned char*>(x), lds0 + raw_off, dim * (x_dtype == PLLM_F32 ? 4 : 2), wave, lane);
    FMT::template dma_tables<kW13Waves>(lds0 + table_off, wave, lane);
    const int tile_loads = dma_share<kW13Waves>(w1 + tile_pos, lds0 + tile_off, tile_bytes, wave, lane) +
                           dma_share<kW13Waves>(w3 + tile_pos, lds0 + tile_off + tile_stride, tile_bytes, wave, lane);
    if (tid < 4) reinterpret_cast<uint32_t*>(smem + zero_off)[tid] = 0;
    AMap<FMT::kSlots> am;
    FMT::a_map(am, col, ks, kpad, zero_off);
    wait_vm_all_but(tile_loads);
    __syncthreads();
    quantize_row_to_lds(smem, smem + raw_off, x_dtype, 0, dim, kpad);
    wait_vm<0>();
    __syncthreads();

    const unsigned char* tile = smem + tile_off + mat * tile_stride;
    float acc = 0.0f;
    for (int b = share; b < bpr; b += kW13Waves / 2) {
        typename FMT::Regs regs;
        FMT::load_lds(regs, tile, col * row_bytes + b * FMT::kBlockBytes, ks);
        acc += FMT::block(regs, ks, b, smem, am, sx, tables);
    }
    acc = quad_rows_sum(acc);
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
    const uint8_t* __restrict__ w2, size_t expert_stride, float* __restrict__ y, int dim, int tile_off, int tile_stride,
    void* __restrict__ add_into, int add_dtype) {
    // the arguments in one batch of scalar loads, one wait (not the route table: its reads must stay scalar loads)
    asm volatile("" : : "s"(h_image), "s"(h_image_stride), "s"(bpr), "s"(routes), "s"(w2), "s"(expert_stride), "s"(y), "s"(dim), "s"(tile_off),
                 "s"(tile_stride), "s"(static_cast<int>(add_into != nullptr)), "s"(add_dtype));
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

    // 1 KB pieces of the routes' tiles and images: wave = (route parity, piece mod 8), so that no wave divides to find its share
    for (int r = wave >> 3; r < routes; r += kW2Waves / 8) {
        const uint8_t* tile_src = w2 + static_cast<size_t>(route_experts[r]) * expert_stride + tile_pos;
        for (int o = (wave & 7) * 1024; o < tile_bytes; o += 8 * 1024)
            if (o + lane * 16 < tile_bytes) lds_dma16(tile_src + o + lane * 16, lds0 + tile_off + r * tile_stride + o);
        for (int o = (wave & 7) * 1024; o < image_bytes; o += 8 * 1024)
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
    acc = quad_rows_sum(acc);
    if (ks == 0) partial[wave * 16 + col] = acc;
    __syncthreads();
    if (tid < 16) {
        float total = 0.0f;
#pragma unroll
        for (int v = 0; v < kW2Waves; ++v) total += partial[v * 16 + tid];
        // the routes' sum, or the residual stream with the sum added (float32 addition, one rounding to the stream's type)
        if (add_into) store_any(add_into, add_dtype | 0x100, static_cast<size_t>(blockIdx.x) * 16 + tid, total);
        else y[blockIdx.x * 16 + tid] = total;
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
                acc = quad_rows_sum(acc);
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
                    acc = quad_rows_sum(acc);
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

// ------------------------------------------------------------------------------------------------
// Grouped routes with the ROUTES as matrix rows, in half precision on the matrix cores.
//
// The integer weights of IQ2_XXS, magnitude (8, 25 or 43) times group scale (odd, at most 31), are
// exact in half precision, and so is a bfloat16 / float16 activation once its row is scaled by a power
// of two (float32 rows go in as two half-precision terms).  v_mfma_f32_16x16x32_f16 per 32-weight
// group: A row m = route m of a batch of 16 (or route m / 2, term m % 2, of a batch of 8), B column n =
// weight row n; lane (n, q) = (lane % 16, lane / 16) supplies the eight weights [8 q, 8 q + 8) of the
// group (grid entry q of the sub-block) as B and the same eight positions of its image row as A, and
// finds rows 4 q .. 4 q + 3 for weight row n in its C registers.  The matrix cores accumulate over the
// groups of a block in float32; the block scale goes on per block.  One decode of a block serves the
// whole batch, no integer fix-up follows the MFMA, and the lanes' A operands are the same for every
// tile of a run: they are read from memory once per batch and kept in registers.
//
// Unit = (expert, run of 16-row tiles).  The tiles' weights (gate and up) arrive by direct-to-LDS
// loads, double-buffered, one barrier per tile.  Twelve waves = (matrix, sixth of the row's blocks).
// LDS codebooks: 256 x 8 magnitudes and 128 x 8 sign masks as half-precision vectors, kRowsCopies
// copies of each entry side by side so that lane l reads copy l % 8: eight neighbouring lanes cover
// all banks with their 16-byte reads whatever entries they pick.
// ------------------------------------------------------------------------------------------------
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

constexpr int kRowsWaves = 12;
constexpr int kRowsShares = kRowsWaves / 2;
constexpr int kRowsBlocks = 2;            // blocks of a row per wave
constexpr int kRowsCopies = 8;            // (the kernel shifts entry numbers by 7 = log2(16 * kRowsCopies))
constexpr int kRowsTableBytes = (256 + 128) * 16 * kRowsCopies;

// Activation rows as half-precision images: img[token][term][kpad] = x * s (zero beyond dim), s a
// power of two that brings the row's largest magnitude into [1024, 2048); unscale[token] = 1 / s.
// TERMS = 2 adds the rounding residual as a second row.
// the power of two that brings a row whose largest magnitude is am into [1024, 2048) (1 for rows of zeros or with non-finite values)
__device__ __forceinline__ float rows_scale(float am) {
    if (!(am > 0.0f && am < 3.0e38f)) return 1.0f;
    int ex;
    frexpf(am, &ex);                           // am = m * 2^ex, m in [0.5, 1)
    return ldexpf(1.0f, max(-126, min(11 - ex, 126)));
}

constexpr int kImageHeld = 4;              // pieces of four values a thread keeps: rows up to 4096 values are read once
template <int TERMS>
__global__ __launch_bounds__(256) void rows_image_kernel(const void* __restrict__ x, int x_dtype, int dim, int kpad, _Float16* __restrict__ img,
                                                         float* __restrict__ unscale) {
    __shared__ float part[4];
    const int token = blockIdx.x, tid = threadIdx.x;
    const size_t base = static_cast<size_t>(token) * dim;
    const bool held = kpad <= 4 * kImageHeld * 256 && dim % 4 == 0 &&
                      ((reinterpret_cast<uintptr_t>(x) + base * (x_dtype == PLLM_F32 ? 4 : 2)) & 15u) == 0;
    float v[kImageHeld][4];
    float am = 0.0f;
    if (held) {                                // all of the thread's pieces requested together (beyond the row: its first piece again, dropped)
        int e0[kImageHeld];
#pragma unroll
        for (int j = 0; j < kImageHeld; ++j) e0[j] = 4 * (tid + 256 * j) < dim ? 4 * (tid + 256 * j) : 0;
        load_rows4_batch(v, x, x_dtype, base, e0);
#pragma unroll
        for (int j = 0; j < kImageHeld; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (4 * (tid + 256 * j) >= dim) v[j][i] = 0.0f;
                am = fmaxf(am, fabsf(v[j][i]));
            }
    } else {
        for (int k = tid; k < dim; k += 256) am = fmaxf(am, fabsf(load_any(x, x_dtype, base + k)));
    }
    am = group_max<64>(am);
    if ((tid & 63) == 0) part[tid >> 6] = am;
    __syncthreads();
    am = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
    const float s = rows_scale(am);
    _Float16* row = img + static_cast<size_t>(token) * TERMS * kpad;
    if (held) {
#pragma unroll
        for (int j = 0; j < kImageHeld; ++j) {
            const int k0 = 4 * (tid + 256 * j);
            if (k0 < kpad) {
                union { _Float16 h[4]; uint2 u; } hi, lo;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float w = v[j][i] * s;
                    hi.h[i] = static_cast<_Float16>(w);
                    lo.h[i] = static_cast<_Float16>(w - static_cast<float>(hi.h[i]));
                }
                *reinterpret_cast<uint2*>(row + k0) = hi.u;
                if constexpr (TERMS == 2) *reinterpret_cast<uint2*>(row + kpad + k0) = lo.u;
            }
        }
    } else {
        for (int k = tid; k < kpad; k += 256) {
            const float w = k < dim ? load_any(x, x_dtype, base + k) * s : 0.0f;
            const _Float16 h = static_cast<_Float16>(w);
            row[k] = h;
            if constexpr (TERMS == 2) row[kpad + k] = static_cast<_Float16>(w - static_cast<float>(h));
        }
    }
    if (tid == 0) unscale[token] = 1.0f / s;
}

__device__ __forceinline__ v8h as_v8h(uint4 u) {
    union { uint4 u; v8h h; } c;
    c.u = u;
    return c.h;
}

// the half-precision codebooks of IQ2_XXS, kRowsCopies copies per entry, built by the whole workgroup
__device__ __forceinline__ void rows_tables_iq2xxs(unsigned char* lds, int tid, int threads) {
    for (int i = tid; i < (256 + 128) * kRowsCopies; i += threads) {
        const int e = i / kRowsCopies;
        uint32_t w[4];
        if (e < 256) {
            const uint64_t g = PLLM_IQ2XXS_GRID[e];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                union { _Float16 h[2]; uint32_t u; } c;
                c.h[0] = static_cast<_Float16>(static_cast<float>((g >> (16 * j)) & 0xffu));
                c.h[1] = static_cast<_Float16>(static_cast<float>((g >> (16 * j + 8)) & 0xffu));
                w[j] = c.u;
            }
        } else {
            const uint64_t m = PLLM_IQ2XXS_SIGN_MASKS.v[e - 256];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = (((m >> (16 * j)) & 1u) ? 0x8000u : 0u) | (((m >> (16 * j + 8)) & 1u) ? 0x80000000u : 0u);
        }
        reinterpret_cast<uint4*>(lds)[i] = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

// One hidden value h = silu(g) * u * route weight of a 16-row tile (16 neighbouring lanes = the tile), kept in float32,
// and the tile's largest magnitude: the down projection's rows are scaled per route once all tiles are there.
__device__ __forceinline__ void store_hidden_rows(float g, float u, float limit, float route_weight, int i, int inter, float* row, float* tile_max) {
    if (limit > 0.0f) {
        u = fminf(fmaxf(u, -limit), limit);
        g = fminf(g, limit);
    }
    const float h = (i < inter) ? g / (1.0f + expf(-g)) * u * route_weight : 0.0f;
    row[i] = h;
    // the tile's maximum through DPP row operations (no LDS crossbar); fmaxf drops NaNs, an infinity stays
    const float am = group_max<16>(fabsf(h));
    if ((i & 15) == 0) tile_max[i >> 4] = am;
}

// hidden rows of the down projection: h16[route][k] = h[route][k] * s, s the power of two of rows_scale for the route's
// largest magnitude; unscale[route] = 1 / s.  One workgroup per route.
__global__ __launch_bounds__(256) void rows_hidden_half_kernel(const float* __restrict__ h, const float* __restrict__ tile_max, int h_kpad,
                                                               _Float16* __restrict__ h16, float* __restrict__ unscale) {
    __shared__ float part[4];
    const int route = blockIdx.x, tid = threadIdx.x;
    float am = 0.0f;
    for (int t = tid; t < h_kpad / 16; t += 256) am = fmaxf(am, tile_max[static_cast<size_t>(route) * (h_kpad / 16) + t]);
    am = group_max<64>(am);
    if ((tid & 63) == 0) part[tid >> 6] = am;
    __syncthreads();
    const float s = rows_scale(fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3])));
    const float4* src = reinterpret_cast<const float4*>(h + static_cast<size_t>(route) * h_kpad);
    uint2* dst = reinterpret_cast<uint2*>(h16 + static_cast<size_t>(route) * h_kpad);
    for (int k = tid; k < h_kpad / 4; k += 256) {
        const float4 v = src[k];
        union { _Float16 h[4]; uint2 u; } c;
        c.h[0] = static_cast<_Float16>(v.x * s); c.h[1] = static_cast<_Float16>(v.y * s);
        c.h[2] = static_cast<_Float16>(v.z * s); c.h[3] = static_cast<_Float16>(v.w * s);
        dst[k] = c.u;
    }
    if (tid == 0) unscale[route] = 1.0f / s;
}

template <int NB, int TERMS>
__global__ __launch_bounds__(64 * kRowsWaves) void moe_rows_w13_kernel(
    const _Float16* __restrict__ x_rows, const float* __restrict__ unscale, int bpr, const int64_t* __restrict__ route_tokens,
    const int32_t* __restrict__ seg, const float* __restrict__ route_weights, const uint8_t* __restrict__ w1, const uint8_t* __restrict__ w3,
    int inter, float limit, float* __restrict__ h_rows, float* __restrict__ h_tile_max, int h_kpad, int n_experts, int runs,
    int tile_off, int tile_stride) {
    using FMT = IQ2XXSm;
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int kBatch = 16 / TERMS;
    constexpr int kExchFloats = kBatch * kRowsShares * 2 * 16;              // [route][share][matrix][16]
    const int kpad = bpr * 256;
    float* exch = reinterpret_cast<float*>(smem + kRowsTableBytes);          // two of them, by tile parity
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte_ptr)smem));

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int n = lane & 15, q = lane >> 4;
    const int mat = wave & 1, share = wave >> 1;
    const int row_bytes = bpr * FMT::kBlockBytes;
    const int tile_bytes = 16 * row_bytes;
    const int tiles = (inter + 15) / 16;
    const int tiles_per_run = (tiles + runs - 1) / runs;
    const unsigned char* grid_lane = smem + (lane & (kRowsCopies - 1)) * 16;            // entry e of the lane's copy: + e * 16 * kRowsCopies
    const unsigned char* sign_lane = grid_lane + 256 * 16 * kRowsCopies;
    // every block the lane reads starts at the same offset modulo 4 (66-byte blocks, the wave's blocks
    // an even number of them apart): its sub-blocks are read as aligned dwords and shifted where needed
    const bool dword_aligned = ((n * bpr + share) & 1) != 0;
    uint32_t sh = dword_aligned ? 0u : 16u;
    asm volatile("" : "+v"(sh));               // (kept a plain shift amount: one v_alignbit per use instead of a byte permute and a select)
    const uint32_t id_sel = 0x0c0c0c00u | static_cast<uint32_t>(q + (dword_aligned ? 0 : 2));   // byte q of the sub-block's four grid ids

    rows_tables_iq2xxs(smem, tid, blockDim.x);

    for (int unit = blockIdx.x; unit < n_experts * runs; unit += gridDim.x) {
        const int expert = unit / runs, run = unit % runs;
        const int r0 = seg[expert], r1 = seg[expert + 1];
        if (r0 >= r1) continue;
        if (run == 0)                          // padding of the hidden rows: zeros, no weights behind them
            for (int i = tid; i < (h_kpad - 16 * tiles) * (r1 - r0); i += blockDim.x) {
                const int r = i / (h_kpad - 16 * tiles), c = i % (h_kpad - 16 * tiles);
                h_rows[static_cast<size_t>(r0 + r) * h_kpad + 16 * tiles + c] = 0.0f;
                if ((c & 15) == 0) h_tile_max[static_cast<size_t>(r0 + r) * (h_kpad / 16) + tiles + (c >> 4)] = 0.0f;
            }
        const int t0 = run * tiles_per_run, t1 = min(tiles, t0 + tiles_per_run);
        if (t0 >= t1) continue;
        const size_t expert_pos = static_cast<size_t>(expert) * inter * row_bytes;
        for (int rc = r0; rc < r1; rc += kBatch) {
            const int nr = min(kBatch, r1 - rc);
            {
                const size_t pos = expert_pos + static_cast<size_t>(t0) * tile_bytes;
                dma_share<kRowsWaves>(w1 + pos, lds0 + tile_off, tile_bytes, wave, lane);
                dma_share<kRowsWaves>(w3 + pos, lds0 + tile_off + tile_stride, tile_bytes, wave, lane);
            }
            // the lane's image row: the same for every tile of the run (rows past the batch's end repeat its last route)
            const int my_route = rc + min((TERMS == 2) ? (n >> 1) : n, nr - 1);
            const _Float16* xrow = x_rows + (static_cast<size_t>(route_tokens[my_route]) * TERMS + ((TERMS == 2) ? (n & 1) : 0)) * kpad + 8 * q;
            v8h av[NB][8];
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                const int b = min(share + kRowsShares * i, bpr - 1);
#pragma unroll
                for (int g = 0; g < 8; ++g) av[i][g] = as_v8h(*reinterpret_cast<const uint4*>(xrow + 256 * b + 32 * g));
            }
            // the epilogue's thread (route j, row c of the tile) keeps its route's factors
            float ep_unscale = 0.0f, ep_weight = 0.0f;
            if (tid < 16 * nr) {
                ep_unscale = unscale[route_tokens[rc + (tid >> 4)]];
                ep_weight = route_weights[rc + (tid >> 4)];
            }
            wait_vm<0>();
            __syncthreads();                   // first tile landed; every wave has left the previous batch (and the tables are built)
            for (int tile = t0; tile < t1; ++tile) {
                const int buf = (tile - t0) & 1;
                if (tile + 1 < t1) {           // the other buffer was last read before the previous tile's barrier
                    const size_t pos = expert_pos + static_cast<size_t>(tile + 1) * tile_bytes;
                    const uint32_t dst = lds0 + tile_off + (buf ^ 1) * 2 * tile_stride;
                    dma_share<kRowsWaves>(w1 + pos, dst, tile_bytes, wave, lane);
                    dma_share<kRowsWaves>(w3 + pos, dst + tile_stride, tile_bytes, wave, lane);
                }
                const unsigned char* tb = smem + tile_off + (2 * buf + mat) * tile_stride;
                v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    const int b = share + kRowsShares * i;
                    if (b < bpr) {             // wave-uniform
                        const int off = n * row_bytes + b * FMT::kBlockBytes;
                        const uint32_t* p = reinterpret_cast<const uint32_t*>(tb + ((off + 2) & ~3));
                        uint32_t dw[17];
#pragma unroll
                        for (int j = 0; j < 17; ++j) dw[j] = p[j];
                        const float d8 = 0.125f * f16_bits_to_float(*reinterpret_cast<const uint16_t*>(tb + off));
                        v4f c = {0.0f, 0.0f, 0.0f, 0.0f};
                        // four groups at a time: all their codebook reads are issued before the first is used
#pragma unroll
                        for (int g0 = 0; g0 < 8; g0 += 4) {
                            uint4 mag[4], sgn[4];
                            uint32_t aux[4];
#pragma unroll
                            for (int j = 0; j < 4; ++j) {
                                const int g = g0 + j;
                                const uint32_t id = __builtin_amdgcn_perm(dw[2 * g + 1], dw[2 * g], id_sel);
                                aux[j] = __builtin_amdgcn_alignbit(dw[2 * g + 2], dw[2 * g + 1], sh);
                                mag[j] = *reinterpret_cast<const uint4*>(grid_lane + (id << 7));
                                sgn[j] = *reinterpret_cast<const uint4*>(sign_lane + (__builtin_amdgcn_ubfe(aux[j], 7 * q, 7) << 7));
                            }
                            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                            for (int j = 0; j < 4; ++j) {
                                // the group scale 2 ls + 1 as a pair of halves: 1024 + 2 ls + 1 by integer arithmetic on the bits, then - 1024
                                union { uint32_t u; v2h h; } ls2;
                                ls2.u = (aux[j] >> 28) * 0x00020002u + 0x64016401u;
                                const v2h k1024 = {static_cast<_Float16>(1024.0f), static_cast<_Float16>(1024.0f)};
                                ls2.h = ls2.h - k1024;
                                union { uint4 u; v2h h[4]; } bw;
                                bw.u = make_uint4(mag[j].x ^ sgn[j].x, mag[j].y ^ sgn[j].y, mag[j].z ^ sgn[j].z, mag[j].w ^ sgn[j].w);
#pragma unroll
                                for (int e = 0; e < 4; ++e) bw.h[e] = bw.h[e] * ls2.h;
                                c = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[i][g0 + j], as_v8h(bw.u), c, 0, 0, 0);
                            }
                        }
                        acc += c * d8;
                    }
                }
                float* ex = exch + buf * kExchFloats;
                if constexpr (TERMS == 1) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) ex[(((4 * q + j) * kRowsShares + share) * 2 + mat) * 16 + n] = acc[j];
                } else {
                    ex[(((2 * q) * kRowsShares + share) * 2 + mat) * 16 + n] = acc[0] + acc[1];
                    ex[(((2 * q + 1) * kRowsShares + share) * 2 + mat) * 16 + n] = acc[2] + acc[3];
                }
                wait_vm<0>();
                __syncthreads();               // sums visible, next tile landed, this tile's buffer free
                if (tid < 16 * nr) {
                    const int j = tid >> 4, c = tid & 15;
                    float g = 0.0f, u = 0.0f;
#pragma unroll
                    for (int v = 0; v < kRowsShares; ++v) { g += ex[((j * kRowsShares + v) * 2) * 16 + c]; u += ex[((j * kRowsShares + v) * 2 + 1) * 16 + c]; }
                    store_hidden_rows(g * ep_unscale, u * ep_unscale, limit, ep_weight, tile * 16 + c, inter, h_rows + static_cast<size_t>(rc + j) * h_kpad, h_tile_max + static_cast<size_t>(rc + j) * (h_kpad / 16));
                }
            }
            __syncthreads();                   // the epilogue's readers are done before the next batch overwrites anything
        }
    }
}

// Down projection of grouped routes, the routes as matrix rows (IQ1_M): partial[r, :] = W2_e h_r.
// The codes 8 (c - 1) +- 1 times the 16-weight scale 2 s + 1 (at most 9 * 15) are exact in half
// precision; a 32-weight group = four codebook entries = one MFMA, lane (n, q) supplying entry q with
// its own 16-weight scale.  A rows = the hidden rows of 16 routes (rows_hidden_half_kernel), kept in
// registers for a run of steps.  A step = 64 output rows (four tiles), twelve waves = (tile, third
// of the row's blocks); the step's weights are one contiguous run of memory.
// LDS codebook: 4096 x 8 codes as half-precision vectors, index = qs byte | qh nibble << 8.
constexpr int kRows2Tiles = 4;
constexpr int kRows2Shares = kRowsWaves / kRows2Tiles;
constexpr int kRows2Blocks = 3;           // blocks of a row per wave
constexpr int kRows2TableBytes = 4096 * 16;
constexpr int kRows2Batch = 16;

__device__ __forceinline__ void rows_tables_iq1m(unsigned char* lds, int tid, int threads) {
    for (int i = tid; i < 4096; i += threads) {
        const uint64_t v = PLLM_IQ1_DELTA_CODES.v[i];
        uint32_t w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            union { _Float16 h[2]; uint32_t u; } c;
            c.h[0] = static_cast<_Float16>(static_cast<float>(static_cast<int8_t>(v >> (16 * j))));
            c.h[1] = static_cast<_Float16>(static_cast<float>(static_cast<int8_t>(v >> (16 * j + 8))));
            w[j] = c.u;
        }
        reinterpret_cast<uint4*>(lds)[i] = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

template <int NB>
__global__ __launch_bounds__(64 * kRowsWaves) void moe_rows_w2_kernel(
    const _Float16* __restrict__ h_rows, const float* __restrict__ h_unscale, int bpr, const int32_t* __restrict__ seg, const uint8_t* __restrict__ w2,
    size_t expert_stride, float* __restrict__ partial, int dim, int n_experts, int runs, int tile_off, int step_stride) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int kBlockBytes = IQ1Mm::kBlockBytes;
    constexpr int kStepRows = 16 * kRows2Tiles;
    constexpr int kExchFloats = kRows2Batch * kRows2Shares * kStepRows;     // [route][share][row of the step]
    const int kpad = bpr * 256;
    float* exch = reinterpret_cast<float*>(smem + kRows2TableBytes);         // two of them, by step parity
    float* route_unscale = exch + 2 * kExchFloats;                           // [route of the batch]
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte_ptr)smem));

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int n = lane & 15, q = lane >> 4;
    const int tile_in_step = wave / kRows2Shares, share = wave % kRows2Shares;
    const int row_bytes = bpr * kBlockBytes;
    const int steps = (dim + kStepRows - 1) / kStepRows;
    const int steps_per_run = (steps + runs - 1) / runs;

    rows_tables_iq1m(smem, tid, blockDim.x);

    for (int unit = blockIdx.x; unit < n_experts * runs; unit += gridDim.x) {
        const int expert = unit / runs, run = unit % runs;
        const int r0 = seg[expert], r1 = seg[expert + 1];
        if (r0 >= r1) continue;
        const int s0 = run * steps_per_run, s1 = min(steps, s0 + steps_per_run);
        if (s0 >= s1) continue;
        const uint8_t* wexp = w2 + static_cast<size_t>(expert) * expert_stride;
        for (int rc = r0; rc < r1; rc += kRows2Batch) {
            const int nr = min(kRows2Batch, r1 - rc);
            dma_share<kRowsWaves>(wexp + static_cast<size_t>(s0) * kStepRows * row_bytes, lds0 + tile_off, min(kStepRows, dim - s0 * kStepRows) * row_bytes, wave, lane);
            // the lane's row of the hidden values: the same for every step of the run (rows past the batch's end repeat its last route)
            // (rows scaled into half-precision range by a power of two per route: taken out again when the sums are stored)
            const _Float16* hrow = h_rows + static_cast<size_t>(rc + min(n, nr - 1)) * kpad + 8 * q;
            if (tid < kRows2Batch) route_unscale[tid] = h_unscale[rc + min(tid, nr - 1)];
            v8h av[NB][8];
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                const int b = min(share + kRows2Shares * i, bpr - 1);
#pragma unroll
                for (int g = 0; g < 8; ++g) av[i][g] = as_v8h(*reinterpret_cast<const uint4*>(hrow + 256 * b + 32 * g));
            }
            wait_vm<0>();
            __syncthreads();                   // first step landed; every wave has left the previous batch (and the table is built)
            for (int step = s0; step < s1; ++step) {
                const int buf = (step - s0) & 1;
                const int row0 = step * kStepRows, valid_rows = min(kStepRows, dim - row0);   // a multiple of 16
                if (step + 1 < s1)             // the other buffer was last read before the previous step's barrier
                    dma_share<kRowsWaves>(wexp + static_cast<size_t>(row0 + kStepRows) * row_bytes, lds0 + tile_off + (buf ^ 1) * step_stride,
                                          min(kStepRows, dim - row0 - kStepRows) * row_bytes, wave, lane);
                float* ex = exch + buf * kExchFloats;
                if (tile_in_step * 16 < valid_rows) {                       // wave-uniform
                    const unsigned char* tb = smem + tile_off + buf * step_stride + (tile_in_step * 16 + n) * row_bytes;
                    v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int i = 0; i < NB; ++i) {
                        const int b = share + kRows2Shares * i;
                        if (b < bpr) {         // wave-uniform
                            const uint2* p = reinterpret_cast<const uint2*>(tb + b * kBlockBytes);     // blocks are 8-byte aligned
                            uint32_t dw[14];
#pragma unroll
                            for (int j = 0; j < 7; ++j) { const uint2 v = p[j]; dw[2 * j] = v.x; dw[2 * j + 1] = v.y; }
                            const uint32_t s01 = dw[12], s23 = dw[13];
                            const uint32_t dbits = ((s01 >> 12) & 0xfu) | ((s01 >> 24) & 0xf0u) | ((s23 >> 4) & 0xf00u) | ((s23 >> 16) & 0xf000u);
                            v4f c = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                            for (int g0 = 0; g0 < 8; g0 += 4) {
                                uint4 code[4];
#pragma unroll
                                for (int j = 0; j < 4; ++j) {
                                    const int g = g0 + j;
                                    const uint32_t qs = __builtin_amdgcn_ubfe(dw[g], 8 * q, 8);
                                    const uint32_t nib = __builtin_amdgcn_ubfe(dw[8 + (g >> 1)], 16 * (g & 1) + 4 * q, 4);
                                    code[j] = *reinterpret_cast<const uint4*>(smem + (qs | (nib << 8)) * 16);
                                }
                                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                                for (int j = 0; j < 4; ++j) {
                                    const int g = g0 + j;
                                    // the 16-weight group 2 g + q / 2: field (2 (g % 2) + q / 2) of scale word g / 2
                                    const uint32_t s3 = __builtin_amdgcn_ubfe(dw[12 + (g >> 2)], 16 * ((g >> 1) & 1) + 6 * (g & 1) + 3 * (q >> 1), 3);
                                    union { uint32_t u; v2h h; } ls2;
                                    ls2.u = s3 * 0x00020002u + 0x64016401u;          // 1024 + 2 s + 1 in both halves ...
                                    const v2h k1024 = {static_cast<_Float16>(1024.0f), static_cast<_Float16>(1024.0f)};
                                    ls2.h = ls2.h - k1024;                            // ... minus 1024
                                    union { uint4 u; v2h h[4]; } bw;
                                    bw.u = code[j];
#pragma unroll
                                    for (int e = 0; e < 4; ++e) bw.h[e] = bw.h[e] * ls2.h;
                                    c = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[i][g], as_v8h(bw.u), c, 0, 0, 0);
                                }
                            }
                            acc += c * (0.125f * f16_bits_to_float(dbits));
                        }
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j) ex[((4 * q + j) * kRows2Shares + share) * kStepRows + tile_in_step * 16 + n] = acc[j];
                }
                wait_vm<0>();
                __syncthreads();               // sums visible, next step landed, this step's buffer free
                for (int o = tid; o < nr * kStepRows; o += blockDim.x) {
                    const int j = o / kStepRows, r = o % kStepRows;
                    if (r < valid_rows) {
                        float total = 0.0f;
#pragma unroll
                        for (int v = 0; v < kRows2Shares; ++v) total += ex[(j * kRows2Shares + v) * kStepRows + r];
                        partial[static_cast<size_t>(rc + j) * dim + row0 + r] = total * route_unscale[j];
                    }
                }
            }
            __syncthreads();                   // the epilogue's readers are done before the next batch overwrites anything
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

struct RowsW13Plan { int nb, tile_off, tile_stride; size_t smem; };

RowsW13Plan plan_rows_w13(int bpr) {
    RowsW13Plan p;
    p.nb = (bpr + kRowsShares - 1) / kRowsShares;
    const int head = kRowsTableBytes + 2 * 16 * kRowsShares * 2 * 16 * static_cast<int>(sizeof(float));
    p.tile_off = (head + 1023) & ~1023;
    p.tile_stride = 16 * bpr * IQ2XXSm::kBlockBytes + 16;                    // block shares are read as aligned dwords: a few bytes past the end
    p.smem = static_cast<size_t>(p.tile_off) + 4 * p.tile_stride;
    return p;
}

template <int NB, int TERMS>
int launch_rows_w13_nb(const RowsW13Plan& p, const _Float16* x_rows, const float* unscale, int bpr, const int64_t* route_tokens, const int32_t* seg,
                       const float* route_weights, const uint8_t* w1, const uint8_t* w3, int inter, float limit, float* h_rows,
                       float* h_tile_max, int h_kpad, int n_experts, int routes, hipStream_t stream) {
    auto kern = moe_rows_w13_kernel<NB, TERMS>;
    if (!allow_lds(kern, p.smem)) return PLLM_ERR_UNSUPPORTED;
    const int resident = resident_workgroups(kern, 64 * kRowsWaves, p.smem);
    const int tiles = (inter + 15) / 16;
    const int busy = max(1, min(routes, n_experts));                         // experts that can have routes at all
    const int runs = max(1, min(tiles, (4 * resident + busy - 1) / busy));
    const int grid = min(n_experts * runs, resident);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * kRowsWaves), p.smem, stream, x_rows, unscale, bpr, route_tokens, seg, route_weights, w1, w3, inter,
                       limit, h_rows, h_tile_max, h_kpad, n_experts, runs, p.tile_off, p.tile_stride);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

struct RowsW2Plan { int nb, tile_off, step_stride; size_t smem; };

RowsW2Plan plan_rows_w2(int bpr) {
    RowsW2Plan p;
    p.nb = (bpr + kRows2Shares - 1) / kRows2Shares;
    const int head = kRows2TableBytes + (2 * kRows2Batch * kRows2Shares * 16 * kRows2Tiles + kRows2Batch) * static_cast<int>(sizeof(float));
    p.tile_off = (head + 1023) & ~1023;
    p.step_stride = 16 * kRows2Tiles * bpr * IQ1Mm::kBlockBytes;
    p.smem = static_cast<size_t>(p.tile_off) + 2 * p.step_stride;
    return p;
}

template <int NB>
int launch_rows_w2_nb(const RowsW2Plan& p, const _Float16* h_rows, const float* h_unscale, int bpr, const int32_t* seg, const uint8_t* w2, float* partial, int dim,
                      int n_experts, int routes, hipStream_t stream) {
    auto kern = moe_rows_w2_kernel<NB>;
    if (!allow_lds(kern, p.smem)) return PLLM_ERR_UNSUPPORTED;
    const int resident = resident_workgroups(kern, 64 * kRowsWaves, p.smem);
    const int steps = (dim + 16 * kRows2Tiles - 1) / (16 * kRows2Tiles);
    const int busy = max(1, min(routes, n_experts));
    const int runs = max(1, min(steps, (4 * resident + busy - 1) / busy));
    const int grid = min(n_experts * runs, resident);
    const size_t expert_stride = static_cast<size_t>(dim) * bpr * IQ1Mm::kBlockBytes;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * kRowsWaves), p.smem, stream, h_rows, h_unscale, bpr, seg, w2, expert_stride, partial, dim, n_experts, runs,
                       p.tile_off, p.step_stride);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
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
                       float* y, int dim, hipStream_t stream, void* add_into, int add_dtype) {
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
                       expert_stride, y, dim, tile_off, tile_stride, add_into, add_dtype);
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

bool moe_rows_supports(int w13_type, int w2_type, int dim, int inter, const uint8_t* w1, const uint8_t* w3, const uint8_t* w2) {
    if (w13_type != PLLM_TYPE_IQ2_XXS || w2_type != PLLM_TYPE_IQ1_M || dim % 16 != 0 || inter % 16 != 0) return false;
    if (!aligned16(w1) || !aligned16(w3) || !aligned16(w2)) return false;
    const RowsW13Plan p13 = plan_rows_w13((dim + 255) / 256);
    const RowsW2Plan p2 = plan_rows_w2((inter + 255) / 256);
    return p13.nb <= kRowsBlocks && p13.smem <= 160 * 1024 && p2.nb <= kRows2Blocks && p2.smem <= 160 * 1024;
}

size_t moe_rows_x_bytes(int64_t tokens, int64_t dim) {
    const size_t kpad = static_cast<size_t>((dim + 255) / 256) * 256;
    return align256(static_cast<size_t>(tokens) * 2 * kpad * sizeof(_Float16)) + align256(static_cast<size_t>(tokens) * sizeof(float));
}

// hidden rows of the routes: float32 values [routes][h_kpad], largest magnitudes per 16-row tile, half-precision rows, 1 / scale
struct RowsHidden { float* values; float* tile_max; _Float16* half_rows; float* unscale; size_t bytes; };

static RowsHidden rows_hidden(void* ws, int64_t routes, int64_t inter) {
    const size_t kpad = static_cast<size_t>((inter + 255) / 256) * 256, r = static_cast<size_t>(routes);
    unsigned char* p = static_cast<unsigned char*>(ws);
    RowsHidden h;
    h.values = reinterpret_cast<float*>(p);        p += align256(r * kpad * sizeof(float));
    h.tile_max = reinterpret_cast<float*>(p);      p += align256(r * (kpad / 16) * sizeof(float));
    h.half_rows = reinterpret_cast<_Float16*>(p);  p += align256(r * kpad * sizeof(_Float16));
    h.unscale = reinterpret_cast<float*>(p);       p += align256(r * sizeof(float));
    h.bytes = static_cast<size_t>(p - static_cast<unsigned char*>(ws));
    return h;
}

size_t moe_rows_h_bytes(int64_t routes, int64_t inter) { return rows_hidden(nullptr, routes, inter).bytes; }

int moe_rows_w13(const void* x, int x_dtype, int tokens, int dim, void* x_rows_ws, const int64_t* route_tokens, const int32_t* seg,
                 const float* route_weights, const uint8_t* w1, const uint8_t* w3, int inter, float limit, void* h_rows_ws,
                 int n_experts, int routes, hipStream_t stream) {
    const int bpr = (dim + 255) / 256, kpad = bpr * 256, h_kpad = (inter + 255) / 256 * 256;
    _Float16* x_rows = static_cast<_Float16*>(x_rows_ws);
    const RowsHidden hid = rows_hidden(h_rows_ws, routes, inter);
    float* unscale = reinterpret_cast<float*>(static_cast<unsigned char*>(x_rows_ws) + align256(static_cast<size_t>(tokens) * 2 * kpad * sizeof(_Float16)));
    const bool two_terms = x_dtype == PLLM_F32;
    if (two_terms) hipLaunchKernelGGL(rows_image_kernel<2>, dim3(tokens), dim3(256), 0, stream, x, x_dtype, dim, kpad, x_rows, unscale);
    else hipLaunchKernelGGL(rows_image_kernel<1>, dim3(tokens), dim3(256), 0, stream, x, x_dtype, dim, kpad, x_rows, unscale);
    if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
    const RowsW13Plan p = plan_rows_w13(bpr);
#define PLLM_CASE(N, T) return launch_rows_w13_nb<N, T>(p, x_rows, unscale, bpr, route_tokens, seg, route_weights, w1, w3, inter, limit, hid.values, hid.tile_max, h_kpad, n_experts, routes, stream)
    if (p.nb == 1) { if (two_terms) PLLM_CASE(1, 2); PLLM_CASE(1, 1); }
    if (p.nb == 2) { if (two_terms) PLLM_CASE(2, 2); PLLM_CASE(2, 1); }
#undef PLLM_CASE
    return PLLM_ERR_UNSUPPORTED;
}

int moe_rows_w2(void* h_rows_ws, int inter, const int32_t* seg, const uint8_t* w2, float* partial, int dim, int n_experts, int routes,
                hipStream_t stream) {
    const int bpr = (inter + 255) / 256;
    const RowsW2Plan p = plan_rows_w2(bpr);
    const RowsHidden hid = rows_hidden(const_cast<void*>(h_rows_ws), routes, inter);
    hipLaunchKernelGGL(rows_hidden_half_kernel, dim3(routes), dim3(256), 0, stream, hid.values, hid.tile_max, bpr * 256, hid.half_rows, hid.unscale);
    if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
    switch (p.nb) {
        case 1: return launch_rows_w2_nb<1>(p, hid.half_rows, hid.unscale, bpr, seg, w2, partial, dim, n_experts, routes, stream);
        case 2: return launch_rows_w2_nb<2>(p, hid.half_rows, hid.unscale, bpr, seg, w2, partial, dim, n_experts, routes, stream);
        case 3: return launch_rows_w2_nb<3>(p, hid.half_rows, hid.unscale, bpr, seg, w2, partial, dim, n_experts, routes, stream);
        default: return PLLM_ERR_UNSUPPORTED;
    }
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
