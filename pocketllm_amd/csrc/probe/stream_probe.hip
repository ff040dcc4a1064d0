// Measurement aids, built into their own library (libpllm_probe.so), not into the operator library: a plain streaming copy
// and a streaming read of known size.  They calibrate the HBM counters (bytes a counter reports for a known transfer) and
// show the bandwidth a trivial kernel reaches on the same box; no operator uses them.
//   int pllm_probe_stream_copy(src, dst, nbytes (a multiple of 16), workgroups of 256 threads, stream)   0 = launched
//   int pllm_probe_stream_read(src, sink (4 writable bytes), nbytes, workgroups, stream)
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pllm {
namespace {

__global__ __launch_bounds__(256) void stream_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16) {
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

__global__ __launch_bounds__(256) void stream_read_kernel(const uint4* __restrict__ src, uint32_t* __restrict__ sink, size_t n16) {
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    uint32_t acc = 0;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n16; i += stride) {
        const uint4 v = src[i];
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x9e3779b9u) sink[0] = acc;      // practically never true: keeps the loads alive
}

}  // namespace
}  // namespace pllm

extern "C" {

int pllm_probe_stream_copy(const void* src, void* dst, size_t nbytes, int blocks, void* stream) {
    if (!src || !dst || (nbytes & 15) || blocks <= 0) return -1;
    hipLaunchKernelGGL(pllm::stream_copy_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4*>(src), static_cast<uint4*>(dst), nbytes >> 4);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

int pllm_probe_stream_read(const void* src, void* sink, size_t nbytes, int blocks, void* stream) {
    if (!src || !sink || (nbytes & 15) || blocks <= 0) return -1;
    hipLaunchKernelGGL(pllm::stream_read_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4*>(src), static_cast<uint32_t*>(sink), nbytes >> 4);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

}  // extern "C"
