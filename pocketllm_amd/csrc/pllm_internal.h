// Host-side declarations shared between the kernel translation units and the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/pllm_hip.h"

namespace pllm {

// activation images (act_quant.hip); *_bytes is the per-row stride, a multiple of 256
size_t act_image_256_bytes(int bpr);
int act_image_256(const void* x, int x_dtype, int rows, int k, int bpr, void* image, hipStream_t stream);
size_t act_image_q8pair_bytes(int pairs);
int act_image_q8pair(const void* x, int x_dtype, int rows, int k, int pairs, void* image, hipStream_t stream);

size_t q8_0_matvec_workspace_bytes(int rows, int bpr);
int q8_0_matvec(const void* x, int x_dtype, const uint8_t* w, void* y, int y_dtype,
                int rows, int k, int n, int bpr, void* workspace, size_t workspace_bytes, hipStream_t stream);

size_t kquant_matvec_workspace_bytes(int rows, int bpr);
int kquant_matvec(const void* x, int x_dtype, const uint8_t* w, int type_id, void* y, int y_dtype,
                  int rows, int k, int n, int bpr, void* workspace, size_t workspace_bytes, hipStream_t stream);

// Q2_K / IQ2_XXS / IQ1_M (matvec_dot4.hip); same workspace as kquant_matvec
int dot4_matvec(const void* x, int x_dtype, const uint8_t* w, int type_id, void* y, int y_dtype,
                int rows, int k, int n, int bpr, void* workspace, size_t workspace_bytes, hipStream_t stream);

// FP8 E4M3 weights [n, k] with float32 scales [ceil(n/128), ceil(k/128)] (matvec_fp8.hip)
int fp8_matvec(const void* x, int x_dtype, const uint8_t* w, const float* scale, void* y, int y_dtype,
               int rows, int k, int n, hipStream_t stream);

}  // namespace pllm
