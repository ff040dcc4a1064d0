// Host-side declarations shared between the kernel translation units and the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/pllm_hip.h"

namespace pllm {

int q8_0_matvec(const void* x, int x_dtype, const uint8_t* w, void* y, int y_dtype,
                int rows, int k, int n, int bpr, hipStream_t stream);

int kquant_matvec(const void* x, int x_dtype, const uint8_t* w, int type_id, void* y, int y_dtype,
                  int rows, int k, int n, int bpr, hipStream_t stream);

}  // namespace pllm
