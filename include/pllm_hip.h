/*
 * libpllm_hip: C ABI of the MI355X (gfx950) raw-block quantized matmul kernels.
 *
 * Every entry point takes plain device pointers, sizes and an opaque hipStream_t (void*; NULL is
 * the default stream), enqueues its kernels on that stream and returns without synchronizing.
 * Return value: PLLM_OK or a negative pllm_status; nothing throws.  The library never allocates
 * device memory: outputs and workspaces belong to the caller.  Calls on different streams may run
 * concurrently, with one exception: pllm_gguf_quant_gemm_static_scratch keeps its staging in a
 * device array that all its calls on one GPU share, so overlapping calls of THAT entry point race
 * (see its declaration).  The only other state the library keeps is host-side bookkeeping that
 * never changes a result (the device's compute-unit count, LDS sizes already granted to a kernel,
 * the address of that array), each guarded for concurrent callers.
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
    PLLM_TYPE_Q5_K = 4,    /* 176 B */
    PLLM_TYPE_IQ2_XS = 5,  /* 74 B */
    PLLM_TYPE_IQ3_XXS = 6, /* 98 B */
    PLLM_TYPE_IQ4_XS = 7,  /* 136 B */
    PLLM_TYPE_Q6_K = 8,    /* 210 B */
    PLLM_TYPE_Q8_0 = 100,  /* 34 B / 32 weights; the reference gives Q8_0 no id, this one is the library's own */
    PLLM_TYPE_Q3_K = 101   /* 110 B; decoded by the reference's reader only (src/loader/gguf/tensor_reader.py:746-776, no id, no kernel):
                              pllm_gguf_dequantize_rows takes it, the matmul entry points do not */
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
 * Q4_K / Q5_K matmul with the int8 activation semantics of the reference's MMA prefill path: activations quantized to 32-value
 * int8 blocks (xs = amax / 127, code = rint(x / xs)), integer dots per 32-weight group on the int8 matrix cores,
 *   y[t, r] = sum_g xs[t, g] * (d_r sc_{r,g} * dot_g - dmin_r m_{r,g} * sum of the group's activation codes),
 * d * sc and dmin * m in float32.  Up to 65535 rows (more return PLLM_ERR_UNSUPPORTED); built for prefill row counts.  Other
 * type ids return PLLM_ERR_UNSUPPORTED.
 * Where this differs from the reference's MMA path: its activation quantizer (src/csrc/llama_mmq/gguf_mma_wrapper.cu:104-119)
 * stores xs and the group's sum as fp16, the sum being that of the float activations; here xs stays float32 and the min term
 * uses xs * (sum of the int8 codes).  Both are statements of the same operator with one int8 term per activation; they differ
 * by the fp16 rounding of xs (2^-11 relative) and by the quantization residual inside the min term.
 * Replaces the MMA branch of gguf_quant_gemm_prefill_forward (src/csrc/llama_mmq/gguf_mma_wrapper.cu:257-322,
 * src/csrc/llama_mmq/mmq.cuh:1329-1455, 2083-2200; activation quantizer src/csrc/cuda_kernel_impl.cu:7090-7117).
 * pllm_gguf_quant_gemm keeps float-activation semantics (fp16 tiles); this entry point is the reference's other statement of
 * the operator.
 */
int pllm_gguf_quant_gemm_q8(const void* x, int x_dtype, const uint8_t* blocks, int type_id, void* y, int y_dtype,
                            int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row,
                            void* workspace, size_t workspace_bytes, void* stream);
size_t pllm_gguf_quant_gemm_q8_workspace_bytes(int type_id, int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row);

/*
 * pllm_gguf_quant_gemm for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): same arguments without the workspace, same results bit for bit.  It has no counterpart in
 * the reference, whose operators allocate their temporaries through the framework on every call.  The activation image / the
 * tile kernel's staging lives in a device array of PLLM_STATIC_SCRATCH_BYTES that the library holds on every GPU it runs on
 * until the process ends; the call itself calls no hipMalloc, hipFree or other allocating routine.
 *   - calls whose pllm_gguf_quant_gemm_workspace_bytes(...) exceeds PLLM_STATIC_SCRATCH_BYTES return PLLM_ERR_WORKSPACE;
 *   - every call on one GPU shares that GPU's array: calls that overlap on one GPU (two streams, two threads) race;
 *   - the first call on a device looks the array's address up (hipGetSymbolAddress): make it outside graph capture.
 */
#define PLLM_STATIC_SCRATCH_BYTES (16u << 20)
int pllm_gguf_quant_gemm_static_scratch(const void* x, int x_dtype, const uint8_t* blocks, int type_id, void* y, int y_dtype,
                                        int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row, void* stream);

/*
 * The residual form of pllm_gguf_quant_gemm: y[t, r] += sum_c x[t, c] * W[r, c], the sum formed in float32 and rounded to y's
 * type once.  Replaces the matmul followed by the separate addition of the transformer block's residual connection
 * (src/models/minimax_m2/architecture.py:412-413, `x = x + ...` after the output and expert projections) for decode calls.
 * Same arguments and workspace as pllm_gguf_quant_gemm; y is read and written.  Served by the decode kernels only: a row count
 * that pllm_gguf_quant_gemm would hand to the tile kernel returns PLLM_ERR_UNSUPPORTED (the caller then adds separately).
 */
int pllm_gguf_quant_gemm_accumulate(const void* x, int x_dtype, const uint8_t* blocks, int type_id, void* y, int y_dtype,
                                    int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row,
                                    void* workspace, size_t workspace_bytes, void* stream);

/*
 * RMS normalisation of rows, y[r, :] = x[r, :] * rsqrt(mean(x[r, :]^2) + eps) * weight, float32 arithmetic and one rounding to
 * y_dtype (the reference writes fp16).  Replaces fused_rms_norm_forward (src/csrc/cuda_kernel_impl.cu:9639-9730,
 * src/csrc/cuda_kernel.cpp:2012), the normalisation the reference runs ahead of its quantized projections
 * (src/models/minimax_m2/architecture.py:57-85).
 *
 * pllm_gguf_quant_gemm_rmsnorm: pllm_gguf_quant_gemm on the normalized rows without the round trip through memory,
 *     y = W . (x * rsqrt(mean(x^2) + eps) * norm_weight).
 * It has no counterpart in the reference (which runs the two operators one after the other) and is for decode callers: up to
 * 4 rows are normalized and quantized inside the matvec kernel, one launch in all.  round_fp16 != 0 rounds the normalized values
 * through fp16 first, which is what the reference's two-operator chain hands to its projection; 0 keeps float32.  More rows run
 * the normalisation into the workspace (fp16 rows) and then the ordinary operator.
 */
int pllm_fused_rms_norm(const void* x, int x_dtype, const float* weight, void* y, int y_dtype, int64_t rows, int64_t dim, float eps, void* stream);
int pllm_gguf_quant_gemm_rmsnorm(const void* x, int x_dtype, const float* norm_weight, float eps, int round_fp16,
                                 const uint8_t* blocks, int type_id, void* y, int y_dtype,
                                 int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row,
                                 void* workspace, size_t workspace_bytes, void* stream);
size_t pllm_gguf_quant_gemm_rmsnorm_workspace_bytes(int type_id, int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row);

/*
 * Attention of one new token per sequence against a key/value store (a decode step), everything between the q / k / v projections
 * and the output projection: RMS normalisation of q and k over their whole width (weights may be null: none), rotary phases
 * out = x * cos_row + partner(x) * sin_row on the first rope_dim values of every head (partner = the value rope_dim / 2 away;
 * cos_row / sin_row hold head_dim floats for position pos, sin_row with the sign of the first half; rope_dim 0: none), the new
 * key and value rows written to position pos of the stores, softmax(q k^T / sqrt(head_dim)) v over positions 0 .. pos with every
 * key/value head shared by heads / kv_heads query heads.  Replaces, for one query position, what the reference runs as separate
 * framework operators in src/models/minimax_m2/architecture.py:158-266 (q_norm, k_norm, apply_rotary_emb, cache update,
 * scaled_dot_product_attention).  Not a quantized operator: it is here because those ~17 small launches, not the matmuls,
 * dominated a decoder block's step.
 *
 * q [batch, heads * head_dim], k_new / v_new [batch, kv_heads * head_dim], out [batch, heads * head_dim] and the stores
 * [batch, kv_heads, capacity, head_dim] (strides in elements) all have type dtype (PLLM_F16 or PLLM_BF16); 16-byte aligned.
 * head_dim must be 128, heads at most 64, heads / kv_heads at most 8, pos below 131072 (PLLM_ERR_UNSUPPORTED otherwise).  Float32 arithmetic; the normalized and the
 * turned values are rounded to dtype where the separate operators round.  Two launches (one when pos < 64).
 */
size_t pllm_attention_decode_workspace_bytes(int64_t batch, int64_t heads, int64_t pos);
int pllm_attention_decode(const void* q, const void* k_new, const void* v_new, int dtype,
                          const float* q_norm_weight, const float* k_norm_weight, float eps,
                          const float* cos_row, const float* sin_row, int64_t rope_dim,
                          void* k_store, void* v_store, int64_t store_batch_stride, int64_t store_head_stride,
                          int64_t batch, int64_t heads, int64_t kv_heads, int64_t head_dim, int64_t pos,
                          void* out, void* workspace, size_t workspace_bytes, void* stream);

/*
 * The two halves of pllm_gguf_quant_gemm, for callers that feed one activation tensor to several
 * matrices (q/k/v, gate/up): quantize once into `image` (pllm_activation_image_bytes bytes, 256-byte
 * aligned), then run any number of matmuls against it (the decode kernels, whatever the row count).  They have no counterpart in the
 * reference, whose kernels re-read float activations; the reference's q8_1 activation quantizers
 * (src/csrc/cuda_kernel_impl.cu:7090-7117) are the closest relative of the first.
 */
size_t pllm_activation_image_bytes(int64_t rows, int64_t blocks_per_row);
int pllm_quantize_activations(const void* x, int x_dtype, int64_t rows, int64_t k, int64_t blocks_per_row,
                              void* image, size_t image_bytes, void* stream);
int pllm_gguf_quant_gemm_prequantized(const void* image, const uint8_t* blocks, int type_id, void* y, int y_dtype,
                                      int64_t rows, int64_t n, int64_t blocks_per_row, void* stream);

/*
 * The feed-forward tail of a decode step in two launches: the image of h = SiLU(gate) * up straight from the gate and up
 * projections [rows, k] (float16, bfloat16 or float32), then the down projection on that image with the residual added
 * (y += W h).  swiglu_limit > 0 caps gate at the limit and clamps up to +-limit first (src/csrc/cuda_kernel_impl.cu:241-262);
 * round_dtype PLLM_F16 / PLLM_BF16 rounds h through that type before quantizing, which is what the chain
 * "F.silu(gate) * up in the model's dtype, then the down projection" feeds its matmul; PLLM_F32 keeps h in float32.
 * They have no counterpart in the reference, whose dense feed-forward runs activation, multiplication, projection and residual
 * addition as separate framework ops around gguf_quant_gemm_forward (src/components/gguf/quantized_ops.py:9-151).
 * image: pllm_activation_image_bytes(rows, blocks_per_row) bytes, 256-byte aligned.
 */
int pllm_swiglu_quantize_activations(const void* gate, const void* up, int gu_dtype, int64_t rows, int64_t k, int64_t blocks_per_row,
                                     float swiglu_limit, int round_dtype, void* image, size_t image_bytes, void* stream);
int pllm_gguf_quant_gemm_prequantized_accumulate(const void* image, const uint8_t* blocks, int type_id, void* y, int y_dtype,
                                                 int64_t rows, int64_t n, int64_t blocks_per_row, void* stream);

/*
 * Two weight matrices of the same [n, k] against one activation tensor (k/v projections): the
 * activations are quantized once.  y [2, rows, n]; workspace as for pllm_gguf_quant_gemm.
 * Replaces gguf_quant_gemm_pair_forward (src/csrc/cuda_kernel.cpp:615-666, launcher
 * src/csrc/cuda_kernel_impl.cu:8598-8650).
 */
int pllm_gguf_quant_gemm_pair(const void* x, int x_dtype, const uint8_t* blocks0, int type_id0, const uint8_t* blocks1, int type_id1,
                              void* y, int y_dtype, int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row,
                              void* workspace, size_t workspace_bytes, void* stream);

/*
 * Up to four weight matrices of the same row length and format against one activation tensor, in one launch: the q / k / v
 * (or gate / up) projections of a decode step.  y[m] [rows, n[m]] = x (optionally RMS-normalized first, as in
 * pllm_gguf_quant_gemm_rmsnorm; norm_weight may be null) times blocks[m] [n[m], blocks_per_row, block bytes] transposed.
 * `blocks`, `n` and `y` are host arrays of `count` entries.  Generalizes gguf_quant_gemm_pair_forward
 * (src/csrc/cuda_kernel.cpp:615-666), which takes two matrices of equal height, to the unequal heights of q and k / v.
 * One launch exists for every format but Q2_K at decode row counts; Q2_K, row counts of the tile kernel, and a normalisation
 * with more than four rows return PLLM_ERR_UNSUPPORTED (call pllm_gguf_quant_gemm[_rmsnorm] per matrix instead).
 * workspace: pllm_activation_image_bytes(rows, blocks_per_row) bytes (unused when the kernel quantizes the rows itself).
 */
int pllm_gguf_quant_gemm_multi(const void* x, int x_dtype, const float* norm_weight, float eps, int round_fp16,
                               int count, const uint8_t* const* blocks, const int64_t* n, int type_id, void* const* y, int y_dtype,
                               int64_t rows, int64_t k, int64_t blocks_per_row, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Selected-row dequantization: out[i, :] = dequant(blocks[row_ids[i], :, :])[:k]  (row_ids == NULL
 * selects rows 0 .. n_selected-1 in order).  type_id may also be PLLM_TYPE_Q8_0 (blocks_per_row then
 * counts 32-weight blocks) or PLLM_TYPE_Q3_K.  Results are bit-identical to the reference's numpy decoders.
 *   row_ids int64 [n_selected] (ids outside [0, n_rows) produce zero rows), out [n_selected, k]
 * Replaces gguf_quant_embedding_forward (src/csrc/cuda_kernel.cpp:669-687, kernel
 * src/csrc/cuda_kernel_impl.cu:8387-8423, which serves q4_k/q5_k only) and stands in for the
 * decoders of src/loader/gguf/tensor_reader.py:543-1009 and q8_0_weight_dequantize
 * (src/kernels/ops.py:734-741).
 */
int pllm_gguf_dequantize_rows(const int64_t* row_ids, int64_t n_selected, const uint8_t* blocks, int type_id,
                              int64_t n_rows, int64_t k, int64_t blocks_per_row, void* out, int out_dtype, void* stream);

/*
 * FP8 E4M3FN (OCP) weights with one float32 scale per 128 x 128 block.
 *   weight [n, k] uint8 codes, scale [ceil(n/128), ceil(k/128)] float32
 * pllm_fp8_block_dequantize: out[r, c] = f32(code[r, c]) * scale[r / 128, c / 128]
 *   replaces _dequant_fp8_weight_torch (src/kernels/ops.py:144-147).
 * pllm_fp8_block_gemm: y[t, r] = sum_c x[t, c] * out[r, c] without materialising `out`
 *   replaces soft_fp8_blockfp8_gemm (src/kernels/ops.py:641-648, 910-954) on float activations.
 *   Few rows take the bandwidth-bound matvec; 16 rows or more with k a multiple of 256 (5 or more when the matrix has
 *   16M weights, 3 or more when it has 64M) take the MFMA tile kernel, which needs `workspace` (pllm_fp8_block_gemm_workspace_bytes bytes, 256-byte
 *   aligned, private to the call until its kernels have run; the query returns 0 when none is needed).
 *   Precision: the matvec multiplies in float32 (rel-L2 <= 1e-5 against the float statement); the tile kernel rounds both
 *   operands to fp16 (<= 1e-3).  float32 activations therefore lose precision at the row count where the tile kernel takes
 *   over, but never below 16 rows; 16-bit activations of 2 - 16 rows run a matrix-core matvec with exact products.
 */
int pllm_fp8_block_dequantize(const uint8_t* weight, const float* scale, int64_t n, int64_t k, void* out, int out_dtype, void* stream);
int pllm_fp8_block_gemm(const void* x, int x_dtype, const uint8_t* weight, const float* scale, void* y, int y_dtype,
                        int64_t rows, int64_t k, int64_t n, void* workspace, size_t workspace_bytes, void* stream);

/*
 * The residual form of pllm_fp8_block_gemm for decode calls: y[t, r] += sum_c x[t, c] * out[r, c], the sum formed in float32 and
 * rounded to y's type once (no workspace: the matvec kernel only; a row count of the tile kernel returns PLLM_ERR_UNSUPPORTED).
 * Replaces soft_fp8_blockfp8_gemm (src/kernels/ops.py:641-648) followed by the separate addition of a transformer block's
 * residual connection.
 */
int pllm_fp8_block_gemm_accumulate(const void* x, int x_dtype, const uint8_t* weight, const float* scale, void* y, int y_dtype,
                                   int64_t rows, int64_t k, int64_t n, void* stream);
size_t pllm_fp8_block_gemm_workspace_bytes(int64_t rows, int64_t k, int64_t n);

/*
 * FP8 activations times FP8 weights, both block-scaled, on the matrix cores' native OCP-FP8 path:
 *     y[t, r] = sum over 128-wide K blocks kb of a_scale[t, kb] * scale[r / 128, kb] * sum_{c in kb} f32(a[t, c]) * f32(weight[r, c])
 *   a [rows, k] E4M3 codes, a_scale [rows, k / 128] float32: the outputs of pllm_fp8_act_quant (block 128)
 *   weight [n, k] E4M3 codes, scale [ceil(n / 128), k / 128] float32; k a multiple of 128, bases 16-byte aligned
 *   y [rows, n] y_dtype, float32 accumulation
 * Replaces fp8_gemm (src/kernels/ops.py:1043-1051), which dequantizes both sides and multiplies in
 * floating point; together with pllm_fp8_act_quant this is the reference's FP8 linear
 * (act_quant + fp8_gemm, src/models/deepseek_v4/runtime.py:639-643).
 */
int pllm_fp8_gemm(const uint8_t* a, const float* a_scale, const uint8_t* weight, const float* scale, void* y, int y_dtype,
                  int64_t rows, int64_t k, int64_t n, void* stream);
/*
 * The same operator (same reference interface, src/kernels/ops.py:1043-1051) with a caller-provided workspace of
 * pllm_fp8_gemm_workspace_bytes(rows, k, n) bytes: output tiles that would occupy a fraction of the GPU for a full pass
 * over K are cut along K, their float32 partial sums go through the workspace and are added in a fixed order (results do
 * not depend on scheduling).  A null or short workspace runs every tile whole, as pllm_fp8_gemm does.
 */
size_t pllm_fp8_gemm_workspace_bytes(int64_t rows, int64_t k, int64_t n);
int pllm_fp8_gemm_ws(const uint8_t* a, const float* a_scale, const uint8_t* weight, const float* scale, void* y, int y_dtype,
                     int64_t rows, int64_t k, int64_t n, void* workspace, size_t workspace_bytes, void* stream);

/*
 * FP8 E4M3 weights with IEEE fp16 scale bits per 128 x 128 block and explicit pitches: the raw-pointer
 * operators of the reference's C++ engine (cpp_engine/include/qwen_cuda_ops.hpp), which take device
 * pointers, ints and an opaque stream and return false on bad arguments; these return a status.
 * In the reference's naming `rows` counts OUTPUT rows (N) and `cols` is the inner dimension (K):
 *   weight [rows, weight_stride >= cols] codes; scale_fp16 [ceil(rows / 128), scale_stride >= ceil(cols / 128)];
 *   x [batch, x_stride >= cols], y [batch, y_stride >= rows]; float32 accumulation, any x / y dtype code.
 * pllm_fp8_fp16scale_matvec: y[r] = sum_c x[c] * f32(code[r, c]) * f32(scale[r / 128, c / 128])
 *   replaces qwen_fp8_e4m3_fp16scale_matvec_cuda and ..._matvec_f16_cuda (qwen_cuda_ops.hpp:59-69, 102-111;
 *   cpp_engine/cuda/qwen_fp8_ops.cu:959-1007).
 * pllm_fp8_fp16scale_swiglu_matvec: y[b, r] = silu(gate . x_b) * (up . x_b), neither projection written out
 *   replaces ..._swiglu_matvec_cuda, ..._swiglu_matvec_f16_cuda (batch 1) and ..._swiglu_small_batch_f16_cuda
 *   (qwen_cuda_ops.hpp:72-83, 113-140; qwen_fp8_ops.cu:1009-1033).
 * pllm_fp8_fp16scale_matmul_rows: the matvec over `batch` activation rows
 *   replaces ..._matmul_rows_cuda, ..._matmul_rows_f16_cuda and ..._matmul_simt_cuda (qwen_cuda_ops.hpp:85-97,
 *   142-170; qwen_fp8_ops.cu:1035-1124).  16 rows or more (5 / 3 or more from 16M / 64M weights) of fp16 / bf16 activations with dense pitches and cols a
 *   multiple of 256 run on the MFMA tile kernel (fp16 operands, float32 accumulation) when `workspace` holds pllm_fp8_fp16scale_matmul_rows_workspace_bytes bytes (256-byte
 *   aligned, private to the call until its kernels have run); otherwise, or with a null workspace, every
 *   activation row takes the matvec kernel.
 */
int pllm_fp8_fp16scale_matvec(const void* x, int x_dtype, const uint8_t* weight, const uint16_t* scale_fp16, void* y, int y_dtype,
                              int64_t rows, int64_t cols, int64_t weight_stride, int64_t scale_stride, void* stream);
int pllm_fp8_fp16scale_swiglu_matvec(const void* x, int x_dtype, const uint8_t* gate_weight, const uint16_t* gate_scale_fp16,
                                     const uint8_t* up_weight, const uint16_t* up_scale_fp16, void* y, int y_dtype,
                                     int64_t batch, int64_t rows, int64_t cols, int64_t x_stride, int64_t y_stride,
                                     int64_t weight_stride, int64_t scale_stride, void* stream);
int pllm_fp8_fp16scale_matmul_rows(const void* x, int x_dtype, const uint8_t* weight, const uint16_t* scale_fp16, void* y, int y_dtype,
                                   int64_t batch, int64_t rows, int64_t cols, int64_t x_stride, int64_t y_stride,
                                   int64_t weight_stride, int64_t scale_stride, void* workspace, size_t workspace_bytes, void* stream);
size_t pllm_fp8_fp16scale_matmul_rows_workspace_bytes(int64_t batch, int64_t rows, int64_t cols);

/*
 * The same matvec over `batch` rows with the scale table kept as bf16 bits, the checkpoint's own storage:
 * replaces qwen_fp8_e4m3_bf16_matvec_cuda (batch 1, x_stride = cols, y_stride = rows) and
 * qwen_fp8_e4m3_bf16_matmul_rows_cuda (cpp_engine/include/qwen_cuda_ops.hpp:172-197), which the reference keeps
 * as its compatibility path; every row takes the float32 matvec kernel.
 */
int pllm_fp8_bf16scale_matmul_rows(const void* x, int x_dtype, const uint8_t* weight, const uint16_t* scale_bf16, void* y, int y_dtype,
                                   int64_t batch, int64_t rows, int64_t cols, int64_t x_stride, int64_t y_stride,
                                   int64_t weight_stride, int64_t scale_stride, void* stream);

/*
 * Fused routed-expert matmul over raw super-blocks (any of the nine super-block types; gate/up share a
 * type, the down projection may use another, so IQ2_XXS gate/up with IQ1_M down needs no special case;
 * pairs of Q2_K / IQ2_XXS / IQ1_M have fused kernels, the other types run route by route through the
 * dense decode kernels or, from 16 tokens on, as batches of tile matmuls):
 *     y[t] = sum over routes r of token t:  W2_e ( silu(min(W1_e x_t, L)) * clamp(W3_e x_t, +-L) * w_r )
 * with the clamp only when swiglu_limit L > 0.
 *   x [tokens, dim]; w1, w3 [n_experts, inter, ceil(dim/256), bb]; w2 [n_experts, dim, ceil(inter/256), bb]
 *   route_tokens  int64 [routes] token of each route (NULL when tokens == 1)
 *   route_experts int64 [routes] expert of each route, or NULL with seg_starts int32 [n_experts + 1]
 *                 giving expert e the routes [seg_starts[e], seg_starts[e+1])
 *   route_weights float32 [routes];  y float32 [tokens, dim], fully overwritten
 * Each token's routes are summed in ascending route order (deterministic).
 * Replaces gguf_moe_prefill_grouped_forward, gguf_moe_single_token_iq2_q2k_forward and
 * gguf_moe_single_token_iq1m_forward (src/csrc/cuda_kernel.cpp:689-865; launchers
 * src/csrc/cuda_kernel_impl.cu:8688-9385).
 */
size_t pllm_gguf_moe_workspace_bytes(int64_t tokens, int64_t routes, int64_t dim, int64_t inter);
int pllm_gguf_moe_forward(const void* x, int x_dtype, int64_t tokens, int64_t dim, int64_t inter,
                          const int64_t* route_tokens, const int64_t* route_experts, const int32_t* seg_starts, int64_t n_experts,
                          const float* route_weights, int64_t routes,
                          const uint8_t* w1, const uint8_t* w3, int w13_type, const uint8_t* w2, int w2_type,
                          float swiglu_limit, float* y, void* workspace, size_t workspace_bytes, void* stream);

/*
 * The routed experts of ONE token added into y [dim] of y_dtype (the residual stream of a decoder block: y += experts(x),
 * float32 sum of what y holds and the routes' sum, rounded once), for callers that would otherwise convert and add in two
 * further launches (the reference's block does: src/models/minimax_m2/architecture.py:404-413).  Same arguments and workspace as
 * pllm_gguf_moe_forward with tokens == 1.  PLLM_ERR_UNSUPPORTED when the shape or the type pair has no kernel that sums the
 * routes inside the down projection: call pllm_gguf_moe_forward and add.  Such kernels exist for IQ2_XXS or IQ1_M gate / up with
 * IQ1_M down (whole 16-row tiles, 16-byte aligned tensors) and, with any gate / up type outside that family, for Q4_K, Q5_K,
 * IQ4_XS, Q6_K and Q2_K down with up to 8 routes (expert matrices on their block type's boundary).  No routes: y is left as it is.
 */
int pllm_gguf_moe_single_token_accumulate(const void* x, int x_dtype, int64_t dim, int64_t inter, const int64_t* route_experts,
                                          const float* route_weights, int64_t routes, const uint8_t* w1, const uint8_t* w3, int w13_type,
                                          const uint8_t* w2, int w2_type, float swiglu_limit, void* y, int y_dtype, void* workspace,
                                          size_t workspace_bytes, void* stream);

/*
 * Counting sort of the (token, k) routes of indices [tokens, topk] by local expert
 * (local = expert - experts_start, kept when 0 <= local < n_local), stable in (token, k) order.
 *   seg_starts int32 [n_local + 1]; route_tokens int64, route_weights float32, route_experts int32:
 *   capacity tokens * topk each, the first seg_starts[n_local] entries are written.
 * Replaces moe_group_routes (src/csrc/cuda_kernel.cpp:1228-1242, src/csrc/cuda_kernel_impl.cu:295-351,
 * 4306-4377), whose order inside a segment depends on atomics.
 */
int pllm_moe_group_routes(const void* indices, int indices_are_i64, const float* weights, int64_t tokens, int64_t topk,
                          int64_t experts_start, int64_t n_local, int32_t* seg_starts, int64_t* route_tokens, float* route_weights,
                          int32_t* route_experts, void* stream);

/*
 * Expert routing ahead of the fused expert matmul: gate logits, scores, top-k, renormalised route weights.
 *   logits[t, e] = x[t, :] . gate_weight[e, :]   (gate_weight float32 [n_experts, dim], float32 accumulation)
 *   softmax_mode == 0: p = sigmoid(logits); the top_k of p + gate_bias (gate_bias float32 [n_experts] or null) are picked;
 *                      weights = p[picked] / max(sum of p[picked], 1e-20)
 *   softmax_mode != 0: the top_k logits are picked; weights = softmax over the picked logits
 *   indices int64 [tokens, top_k] in descending score order (lower expert id first on equal scores), weights float32 [tokens, top_k];
 *   logits float32 [tokens, n_experts] is caller-provided scratch that holds the logits afterwards.
 * Replaces MiniMaxMoE.route (src/models/minimax_m2/architecture.py:291-298), a chain of six framework ops on the caller's side
 * of the expert operators; the softmax form is the routing of the grouped-expert benchmark (tests/bench_gguf_fused_expert.py).
 * n_experts <= 1024, top_k <= 64.
 */
int pllm_moe_route(const void* x, int x_dtype, int64_t tokens, int64_t dim, const float* gate_weight, const float* gate_bias,
                   int64_t n_experts, int64_t top_k, int softmax_mode, float* logits, int64_t* indices, float* weights, void* stream);

/*
 * pllm_moe_route on rows that are RMS-normalized first, as a decoder block does ahead of its experts
 * (src/models/minimax_m2/architecture.py:405-412: ffn_norm, then MiniMaxMoE.forward's gate): the normalisation
 *     x_normed[t, :] = x[t, :] * rsqrt(mean(x[t, :]^2) + eps) * norm_weight      (float32 arithmetic, one rounding to x_normed_dtype)
 * runs inside the logits launch, the logits are formed on the rounded values, and x_normed [tokens, dim] is written out for the
 * expert operators that follow: pllm_fused_rms_norm + pllm_moe_route in two launches instead of three.
 * For up to 4 rows of at most 3072 values (dim % 4 == 0; x, x_normed, norm_weight and gate_weight 16-byte aligned); PLLM_ERR_UNSUPPORTED
 * otherwise (call the two operators).
 */
int pllm_moe_route_rmsnorm(const void* x, int x_dtype, const float* norm_weight, float eps, void* x_normed, int x_normed_dtype,
                           int64_t tokens, int64_t dim, const float* gate_weight, const float* gate_bias, int64_t n_experts, int64_t top_k,
                           int softmax_mode, float* logits, int64_t* indices, float* weights, void* stream);

/*
 * FP8 activation quantizer: per (row, 128 values) scale = max(amax, eps) / 448 (rounded up to a power
 * of two when round_scale_pow2 != 0), code = E4M3FN round-to-nearest-even of clamp(x / scale, +-448).
 *   x [rows, k] (k a multiple of 128) -> codes uint8 [rows, k], scales float32 [rows, k / 128]
 * Replaces blockfp8_act_quant / act_quant (src/kernels/ops.py:501-516, 982-1001).
 */
int pllm_fp8_act_quant(const void* x, int x_dtype, int64_t rows, int64_t k, uint8_t* codes, float* scales,
                       float eps, int round_scale_pow2, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* PLLM_HIP_H */
