// Decode matvec over raw Q2_K / IQ2_XXS / IQ1_M super-blocks with v_dot4_i32_i8 (wave64).
//
// Four adjacent lanes share one super-block (block_dot4.h says which 64 weights each owns); the 16
// such teams of a wave work on 16 consecutive output rows and on the same super-block index, so LDS
// reads of activations are broadcasts.  The W waves of a workgroup split a row's super-blocks
// between them (wave w takes blocks w, w + W, ...) and meet in a small LDS reduction.  All weight
// loads of a pass are issued first; while they are in flight the workgroup fills LDS with the
// pre-quantized activation image and the format's codebooks.
#include "block_dot4.h"
#include "pllm_internal.h"

namespace pllm {
namespace {

constexpr int kRowsPerWg = 16;
constexpr int kMaxWaves = 8;

template <typename FMT, int ITERS, bool RAW>
__global__ __launch_bounds__(64 * kMaxWaves) void dot4_matvec_kernel(
    const ActRows act, const uint8_t* __restrict__ w,
    void* __restrict__ y, int y_dtype, int n, int bpr, const int32_t* __restrict__ y_expert, size_t expert_stride) {
    fetch_together(act);
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    const StagedX sx = carve_staged_x(smem, kpad);
    unsigned char* tables = smem + image_bytes;
    if (y_expert) w += static_cast<size_t>(y_expert[blockIdx.y]) * expert_stride;   // routed: activation row r meets expert r's matrix
    float* partial = reinterpret_cast<float*>(tables + FMT::kTableBytes);        // [waves][16]

    const int tid = threadIdx.x;
    const int waves = blockDim.x >> 6;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int j = lane & 3;
    const int team = lane >> 2;
    const int row = blockIdx.x * kRowsPerWg + team;
    const uint8_t* wrow = w + static_cast<size_t>(row < n ? row : 0) * bpr * FMT::kBlockBytes;

    float acc = 0.0f;
    bool staged = false;
    if constexpr (RAW)                       // raw activation row: quantized here, before the loads take their registers
        quantize_row_to_lds(smem, act.x, act.x_dtype, static_cast<size_t>(blockIdx.y) * act.k, act.k, kpad, RowNorm{act.gamma, act.eps, act.round_f16});
    for (int b0 = wave; b0 < bpr || !staged; b0 += waves * ITERS) {
        typename FMT::Regs regs[ITERS];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int b = min(b0 + it * waves, bpr - 1);                        // clamped: always a valid address
            FMT::load(regs[it], wrow + static_cast<size_t>(b) * FMT::kBlockBytes, j);
        }
        if (!staged) {                       // first trip of every thread of the workgroup
            if constexpr (!RAW)
                copy_to_lds(smem, act.image + (act.row_token ? static_cast<size_t>(act.row_token[blockIdx.y]) : blockIdx.y) * act.stride, image_bytes);
            FMT::stage_tables(tables);
            __syncthreads();
            staged = true;
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int b = b0 + it * waves;
            if (b < bpr) acc += FMT::lane_dot(regs[it], j, b, sx, tables);      // wave-uniform guard
        }
    }
    acc += __shfl_xor(acc, 1, 64);
    acc += __shfl_xor(acc, 2, 64);
    if (j == 0) partial[wave * kRowsPerWg + team] = acc;
    __syncthreads();
    if (tid < kRowsPerWg) {
        float total = 0.0f;
        for (int v = 0; v < waves; ++v) total += partial[v * kRowsPerWg + tid];
        const int out_row = blockIdx.x * kRowsPerWg + tid;
        if (out_row < n) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + out_row, total);
    }
}

template <typename FMT, int ITERS, bool RAW>
int launch_one(const ActRows& act, const uint8_t* w, void* y, int y_dtype,
               int rows, int n, int bpr, int waves, const int32_t* y_expert, size_t expert_stride, hipStream_t stream) {
    const size_t smem = staged_x_bytes(bpr * 256) + FMT::kTableBytes + static_cast<size_t>(waves) * kRowsPerWg * sizeof(float);
    auto kern = dot4_matvec_kernel<FMT, ITERS, RAW>;
    if (smem > 64 * 1024) {
        if (smem > 160 * 1024) return PLLM_ERR_UNSUPPORTED;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(smem)) != hipSuccess)
            return PLLM_ERR_UNSUPPORTED;
    }
    dim3 grid((n + kRowsPerWg - 1) / kRowsPerWg, rows);
    hipLaunchKernelGGL(kern, grid, dim3(64 * waves), smem, stream, act, w, y, y_dtype, n, bpr, y_expert, expert_stride);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

template <typename FMT>
int launch_fmt(const ActRows& act, const uint8_t* w, void* y, int y_dtype,
               int rows, int n, int bpr, const int32_t* y_expert, size_t expert_stride, hipStream_t stream) {
    // waves per workgroup: split a row's blocks so that every wave keeps a handful in flight
    int waves = 1;
    while (waves < kMaxWaves && bpr / (waves * 2) >= 3) waves *= 2;
    const int niter = (bpr + waves - 1) / waves;
    const int passes = (niter + 5) / 6;
    const int iters = (niter + passes - 1) / passes;
#define PLLM_CASE(I) case I: return act.x ? launch_one<FMT, I, true>(act, w, y, y_dtype, rows, n, bpr, waves, y_expert, expert_stride, stream) \
                                          : launch_one<FMT, I, false>(act, w, y, y_dtype, rows, n, bpr, waves, y_expert, expert_stride, stream)
    switch (iters) {
        PLLM_CASE(1); PLLM_CASE(2); PLLM_CASE(3); PLLM_CASE(4); PLLM_CASE(5);
        default: PLLM_CASE(6);
    }
#undef PLLM_CASE
}

}  // namespace

static int dot4_dispatch(const ActRows& act, const uint8_t* w, int type_id, void* y, int y_dtype,
                         int rows, int n, int bpr, const int32_t* y_expert, size_t expert_stride, hipStream_t stream) {
    switch (type_id) {
        case PLLM_TYPE_Q2_K: return launch_fmt<Q2K>(act, w, y, y_dtype, rows, n, bpr, y_expert, expert_stride, stream);
        case PLLM_TYPE_IQ2_XXS: return launch_fmt<IQ2XXS>(act, w, y, y_dtype, rows, n, bpr, y_expert, expert_stride, stream);
        case PLLM_TYPE_IQ1_M: return launch_fmt<IQ1M>(act, w, y, y_dtype, rows, n, bpr, y_expert, expert_stride, stream);
        default: return PLLM_ERR_UNSUPPORTED;
    }
}

int dot4_matvec_from_image(const ActRows& act, const uint8_t* w, int type_id, void* y, int y_dtype,
                           int rows, int n, int bpr, hipStream_t stream, WeightRoute route) {
    return dot4_dispatch(act, w, type_id, y, y_dtype, rows, n, bpr, route.expert, route.expert_stride, stream);
}

int dot4_routed_matvec_from_image(const unsigned char* image, size_t stride, const uint8_t* w, int type_id, void* y, int y_dtype,
                                  int rows, int n, int bpr, const int32_t* y_expert, size_t expert_stride, hipStream_t stream) {
    return dot4_dispatch(act_rows_from_image(image, stride), w, type_id, y, y_dtype, rows, n, bpr, y_expert, expert_stride, stream);
}

}  // namespace pllm
