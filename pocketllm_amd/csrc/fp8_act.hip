// FP8 activation quantizer: per (row, 128 values) s = max(amax, eps) / 448, optionally rounded up to
// a power of two, code = E4M3 (round to nearest even) of clamp(x / s, +-448).
#include "pllm_device.h"
#include "pllm_internal.h"

namespace pllm {
namespace {

// one wave per (row, 128-block); lane l owns values 2l and 2l+1
__global__ __launch_bounds__(64) void fp8_act_quant_kernel(
    const void* __restrict__ x, int x_dtype, uint8_t* __restrict__ codes, float* __restrict__ scales,
    int k, float eps, int pow2) {
    const int lane = threadIdx.x;
    const int blk = blockIdx.x;
    const size_t base = static_cast<size_t>(blockIdx.y) * k + static_cast<size_t>(blk) * 128 + 2 * lane;
    const float a = load_any(x, x_dtype, base);
    const float b = load_any(x, x_dtype, base + 1);
    const float amax = group_max<64>(fmaxf(fabsf(a), fabsf(b)));
    float s = fmaxf(amax, eps) / 448.0f;
    if (pow2) {
        int e;
        const float m = frexpf(fmaxf(s, 1.17549435e-38f), &e);          // s = m * 2^e, m in [0.5, 1)
        s = ldexpf(1.0f, m == 0.5f ? e - 1 : e);
    }
    const float qa = fminf(fmaxf(a / s, -448.0f), 448.0f);
    const float qb = fminf(fmaxf(b / s, -448.0f), 448.0f);
    const int packed = __builtin_amdgcn_cvt_pk_fp8_f32(qa, qb, 0, false);
    *reinterpret_cast<uint16_t*>(codes + base) = static_cast<uint16_t>(packed & 0xffff);
    if (lane == 0) scales[static_cast<size_t>(blockIdx.y) * (k / 128) + blk] = s;
}

}  // namespace
}  // namespace pllm

extern "C" int pllm_fp8_act_quant(const void* x, int x_dtype, int64_t rows, int64_t k, uint8_t* codes, float* scales,
                                  float eps, int round_scale_pow2, void* stream) {
    if (!x || !codes || !scales || rows <= 0 || k <= 0 || (k % 128) != 0) return PLLM_ERR_INVALID_ARGUMENT;
    if (x_dtype != PLLM_F32 && x_dtype != PLLM_F16 && x_dtype != PLLM_BF16) return PLLM_ERR_INVALID_ARGUMENT;
    if (rows > 65535 || k / 128 > 0x7fffffffLL) return PLLM_ERR_UNSUPPORTED;
    dim3 grid(static_cast<unsigned>(k / 128), static_cast<unsigned>(rows));
    hipLaunchKernelGGL(pllm::fp8_act_quant_kernel, grid, dim3(64), 0, static_cast<hipStream_t>(stream), x, x_dtype, codes, scales,
                       static_cast<int>(k), eps, round_scale_pow2);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}
