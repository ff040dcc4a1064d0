// extern "C" surface of libpllm_hip: argument validation and dispatch by type and shape.
#include "pllm_internal.h"

namespace {

bool dtype_ok(int d) { return d == PLLM_F32 || d == PLLM_F16 || d == PLLM_BF16; }
bool fits_int(int64_t v) { return v > 0 && v <= 0x7fffffffLL; }

}  // namespace

extern "C" {

const char* pllm_status_string(int status) {
    switch (status) {
        case PLLM_OK: return "ok";
        case PLLM_ERR_INVALID_ARGUMENT: return "invalid argument";
        case PLLM_ERR_UNSUPPORTED: return "unsupported type or shape";
        case PLLM_ERR_LAUNCH: return "kernel launch failed";
        case PLLM_ERR_WORKSPACE: return "workspace too small";
        default: return "unknown status";
    }
}

int pllm_abi_version(void) { return 1; }

int pllm_gguf_block_bytes(int type_id) {
    switch (type_id) {
        case PLLM_TYPE_IQ2_XXS: return 66;
        case PLLM_TYPE_Q2_K: return 84;
        case PLLM_TYPE_IQ1_M: return 56;
        case PLLM_TYPE_Q4_K: return 144;
        case PLLM_TYPE_Q5_K: return 176;
        default: return 0;
    }
}

int pllm_q8_0_gemm(const void* x, int x_dtype, const uint8_t* blocks, void* y, int y_dtype,
                   int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row,
                   void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !blocks || !y || !dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return PLLM_ERR_INVALID_ARGUMENT;
    if (!fits_int(rows) || !fits_int(k) || !fits_int(n) || !fits_int(blocks_per_row)) return PLLM_ERR_INVALID_ARGUMENT;
    if (blocks_per_row * 32 < k) return PLLM_ERR_INVALID_ARGUMENT;
    if (rows > 65535) return PLLM_ERR_UNSUPPORTED;
    return pllm::q8_0_matvec(x, x_dtype, blocks, y, y_dtype, static_cast<int>(rows), static_cast<int>(k),
                             static_cast<int>(n), static_cast<int>(blocks_per_row), workspace, workspace_bytes,
                             static_cast<hipStream_t>(stream));
}

size_t pllm_q8_0_gemm_workspace_bytes(int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row) {
    (void)k; (void)n;
    if (!fits_int(rows) || !fits_int(blocks_per_row)) return 0;
    return pllm::q8_0_matvec_workspace_bytes(static_cast<int>(rows), static_cast<int>(blocks_per_row));
}

int pllm_gguf_quant_gemm(const void* x, int x_dtype, const uint8_t* blocks, int type_id, void* y, int y_dtype,
                         int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row,
                         void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !blocks || !y || !dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return PLLM_ERR_INVALID_ARGUMENT;
    if (!fits_int(rows) || !fits_int(k) || !fits_int(n) || !fits_int(blocks_per_row)) return PLLM_ERR_INVALID_ARGUMENT;
    if (blocks_per_row * 256 < k) return PLLM_ERR_INVALID_ARGUMENT;
    if (pllm_gguf_block_bytes(type_id) == 0) return PLLM_ERR_UNSUPPORTED;
    if (rows > 65535) return PLLM_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (type_id) {
        case PLLM_TYPE_Q2_K:
        case PLLM_TYPE_IQ2_XXS:
        case PLLM_TYPE_IQ1_M:
            return pllm::dot4_matvec(x, x_dtype, blocks, type_id, y, y_dtype, static_cast<int>(rows), static_cast<int>(k),
                                     static_cast<int>(n), static_cast<int>(blocks_per_row), workspace, workspace_bytes, s);
        case PLLM_TYPE_Q4_K:
        case PLLM_TYPE_Q5_K:
            return pllm::kquant_matvec(x, x_dtype, blocks, type_id, y, y_dtype, static_cast<int>(rows), static_cast<int>(k),
                                       static_cast<int>(n), static_cast<int>(blocks_per_row), workspace, workspace_bytes, s);
        default:
            return PLLM_ERR_UNSUPPORTED;
    }
}

size_t pllm_gguf_quant_gemm_workspace_bytes(int type_id, int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row) {
    (void)k; (void)n;
    if (!fits_int(rows) || !fits_int(blocks_per_row) || pllm_gguf_block_bytes(type_id) == 0) return 0;
    return pllm::kquant_matvec_workspace_bytes(static_cast<int>(rows), static_cast<int>(blocks_per_row));
}

int pllm_fp8_block_gemm(const void* x, int x_dtype, const uint8_t* weight, const float* scale, void* y, int y_dtype,
                        int64_t rows, int64_t k, int64_t n, void* stream) {
    if (!x || !weight || !scale || !y || !dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return PLLM_ERR_INVALID_ARGUMENT;
    if (!fits_int(rows) || !fits_int(k) || !fits_int(n)) return PLLM_ERR_INVALID_ARGUMENT;
    if (rows > 65535) return PLLM_ERR_UNSUPPORTED;
    return pllm::fp8_matvec(x, x_dtype, weight, scale, y, y_dtype, static_cast<int>(rows), static_cast<int>(k),
                            static_cast<int>(n), static_cast<hipStream_t>(stream));
}

}  // extern "C"
