/*
 * libpllm_hip: C ABI of the MI355X (gfx950) raw-block quantized matmul kernels.
 *
 * Every entry point takes plain device pointers, sizes and an opaque hipStream_t (void*; NULL is
 * the default stream), enqueues its kernels on that stream and returns without synchronizing.
 * Return value: PLLM_OK or a negative pllm_status; nothing throws.  The library never allocates
 * device memory: outputs and workspaces belong to the caller.  Calls on different streams may run
 * concurrently; there is no mutable global state.
 *
 * Each declaration names the reference interface it replaces (paths relative to the PocketLLM
 * checkout).
 */
#ifndef PLLM_HIP_H
#define PLLM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum pllm_status {
    PLLM_OK = 0,
    PLLM_ERR_INVALID_ARGUMENT = -1, /* null pointer, non-positive size, blocks do not cover K, ... */
    PLLM_ERR_UNSUPPORTED = -2,      /* type id or shape outside what the kernels implement */
    PLLM_ERR_LAUNCH = -3,           /* HIP reported an error when the kernel was enqueued */
    PLLM_ERR_WORKSPACE = -4         /* caller's workspace is too small */
} pllm_status;

typedef enum pllm_dtype {
    PLLM_F32 = 0,
    PLLM_F16 = 1,
    PLLM_BF16 = 2
} pllm_dtype;

/* GGUF dense type ids: src/loader/gguf/quant_types.py:3-13, src/csrc/cuda_kernel.cpp:401-412 */
enum {
    PLLM_TYPE_IQ2_XXS = 0, /* 66 B / 256 weights */
    PLLM_TYPE_Q2_K = 1,    /* 84 B */
    PLLM_TYPE_IQ1_M = 2,   /* 56 B */
    PLLM_TYPE_Q4_K = 3,    /* 144 B */
    PLLM_TYPE_Q5_K = 4     /* 176 B */
};

const char* pllm_status_string(int status);
int pllm_abi_version(void);

/* Bytes per 256-weight super-block of a type id, or 0 if the id is unknown.
 * Replaces gguf_quant_block_bytes_for_type (src/csrc/cuda_kernel.cpp:401-412). */
int pllm_gguf_block_bytes(int type_id);

/*
 * y[t, n] = sum_k x[t, k] * dequant(blocks)[n, k]        Q8_0 blocks, 34 B per 32 weights.
 *   x       [rows, k]  x_dtype, contiguous
 *   blocks  [n, blocks_per_row, 34] uint8, blocks_per_row * 32 >= k (the tail is treated as zero
 *           activations)
 *   y       [rows, n]  y_dtype
 *   workspace  device scratch of at least pllm_q8_0_gemm_workspace_bytes(...) bytes, 256-byte
 *           aligned, private to this call until its kernels have run (it receives the
 *           pre-quantized activations); the reference allocates its temporaries through torch in
 *           the same place (src/csrc/cuda_kernel_impl.cu:9172-9175)
 * Replaces q8_0_gemm_forward (src/csrc/cuda_kernel.cpp:524-543, launcher
 * src/csrc/cuda_kernel_impl.cu:8472-8500, kernel 8345-8385).
 */
int pllm_q8_0_gemm(const void* x, int x_dtype, const uint8_t* blocks, void* y, int y_dtype,
                   int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row,
                   void* workspace, size_t workspace_bytes, void* stream);
size_t pllm_q8_0_gemm_workspace_bytes(int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row);

/*
 * Same contraction for 256-weight super-block types (type_id above).
 *   blocks  [n, blocks_per_row, block_bytes(type_id)] uint8, blocks_per_row * 256 >= k
 * Serves every number of activation rows: few rows take the bandwidth-bound matvec, many rows the
 * MFMA tile kernel.
 * Replaces gguf_quant_gemm_forward and gguf_quant_gemm_prefill_forward
 * (src/csrc/cuda_kernel.cpp:566-614; launchers src/csrc/cuda_kernel_impl.cu:8502-8596) and
 * gguf_q2k_gemm_dp4a_forward (cuda_kernel.cpp:545-564).
 */
int pllm_gguf_quant_gemm(const void* x, int x_dtype, const uint8_t* blocks, int type_id, void* y, int y_dtype,
                         int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row,
                         void* workspace, size_t workspace_bytes, void* stream);
size_t pllm_gguf_quant_gemm_workspace_bytes(int type_id, int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row);

/*
 * Measurement aids with no counterpart in the reference: a streaming copy and a streaming read of
 * nbytes (a multiple of 16) with `blocks` workgroups of 256 threads.  They calibrate HBM byte
 * counters against a transfer of known size.  sink: 4 writable bytes.
 */
int pllm_diag_stream_copy(const void* src, void* dst, size_t nbytes, int blocks, void* stream);
int pllm_diag_stream_read(const void* src, void* sink, size_t nbytes, int blocks, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* PLLM_HIP_H */
