// Host-side declarations shared between the kernel translation units and the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <atomic>

#include "../../include/pllm_hip.h"

namespace pllm {

inline size_t align256(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }

// Dynamic LDS above 64 KB has to be granted to a kernel before its launch, on every device it runs on.  `granted` is the
// caller's per-kernel record (one static instance per launcher): the largest size granted so far per device, so that the
// attribute call is made only when a call needs more than any before it on that device.  Safe from several threads: a
// lost race only repeats the attribute call.
struct SmemGrant { std::atomic<size_t> bytes[16]; };
inline bool grant_dynamic_smem(const void* kernel, size_t smem, SmemGrant& granted) {
    if (smem <= 64 * 1024) return true;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return false;
    std::atomic<size_t>* slot = (dev >= 0 && dev < 16) ? &granted.bytes[dev] : nullptr;
    if (slot && slot->load(std::memory_order_relaxed) >= smem) return true;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem)) != hipSuccess) return false;
    if (slot) slot->store(smem, std::memory_order_relaxed);
    return true;
}

// Set in the output dtype code a matvec launcher receives: the kernels add their result to what y holds (float32 sum,
// rounded once) instead of overwriting it.
constexpr int kAccumulateInto = 0x100;

// activation images (act_quant.hip); *_bytes is the per-row stride, a multiple of 256
size_t act_image_256_bytes(int bpr);
int act_image_256(const void* x, int x_dtype, int rows, int k, int bpr, void* image, hipStream_t stream);
// the image of SiLU(gate) * up (clamped by `limit` when positive, rounded through round_dtype when that is a 16-bit type)
int swiglu_image_256(const void* gate, const void* up, int gu_dtype, float limit, int round_dtype, int rows, int k, int bpr, void* image,
                     hipStream_t stream);
// y[r, :] = x[r, :] * rsqrt(mean(x[r, :]^2) + eps) * weight (float32 arithmetic, one rounding to y_dtype)
int rms_norm_rows(const void* x, int x_dtype, const float* weight, void* y, int y_dtype, int rows, int dim, float eps, hipStream_t stream);
// one decode step of attention (attn_decode.hip): normalisation, rotary phases, store update, grouped-query softmax attention
size_t attention_decode_workspace_bytes(int batch, int heads, int pos);
bool attention_decode_supports(int heads, int kv_heads, int head_dim, int rope_dim);
int attention_decode(const void* q, const void* k_new, const void* v_new, int dtype, const float* q_weight, const float* k_weight, float eps,
                     const float* cos_row, const float* sin_row, int rope_dim, void* k_store, void* v_store, size_t batch_stride,
                     size_t head_stride, int batch, int heads, int kv_heads, int pos, void* out, void* workspace, hipStream_t stream);
size_t act_image_q8pair_bytes(int pairs);
int act_image_q8pair(const void* x, int x_dtype, int rows, int k, int pairs, void* image, hipStream_t stream);

size_t q8_0_matvec_workspace_bytes(int rows, int bpr);
int q8_0_matvec(const void* x, int x_dtype, const uint8_t* w, void* y, int y_dtype,
                int rows, int k, int n, int bpr, void* workspace, size_t workspace_bytes, hipStream_t stream);

// Where a super-block matvec kernel finds its activation rows.  x == nullptr: images written by
// act_image_256, `stride` bytes apart.  Otherwise the raw rows ([rows, k] of x_dtype): every
// workgroup quantizes its row into LDS itself (the same image, bit for bit), which saves the
// pre-pass launch when there are only a few rows.
struct ActRows {
    const unsigned char* image;
    size_t stride;
    const void* x;
    int x_dtype;
    int k;
    const int64_t* row_token;     // routed calls: grid row r reads image (or raw row) row_token[r] (null: row r)
    const float* gamma;           // raw rows only: RMS normalisation ahead of the quantization (null: none)
    float eps;
    int round_f16;
    int x_broadcast;              // raw rows, routed calls on one token: every grid row reads row 0
};
// Routed calls: grid row r multiplies with the matrix at w + expert[r] * expert_stride (null: one matrix for every row).
struct WeightRoute {
    const int32_t* expert;
    size_t expert_stride;
    // several projections of one activation tensor in one launch (kernels that support it): grid.z = 1 + m multiplies with
    // more_w[m] (more_n[m] rows of the same length and format) and writes to more_y[m]; `extra` counts them
    const uint8_t* more_w[3];
    void* more_y[3];
    int more_n[3];
    int extra;
    const int64_t* expert64;      // the expert numbers as int64 (the form the single-token operators receive them in) instead of `expert`
};
inline bool routed(const WeightRoute& r) { return r.expert != nullptr || r.expert64 != nullptr; }
#ifdef __HIPCC__
// byte offset of grid row `row`'s matrix
__device__ __forceinline__ size_t route_offset(const WeightRoute& r, int row) {
    if (r.expert) return static_cast<size_t>(r.expert[row]) * r.expert_stride;
    if (r.expert64) return static_cast<size_t>(r.expert64[row]) * r.expert_stride;
    return 0;
}
// Kernels that take these structs test their fields one after the other (routed? further projections? a row map?), and the
// compiler loads each field where it is first needed: a scalar load and a wait per test, several hundred nanoseconds of a
// short kernel before its first memory request.  Naming the fields as inputs of an empty statement at the top of the kernel
// makes it fetch them together, behind one wait.  Pointers to the per-row tables (expert numbers, row maps) go in as the
// integers the tests compare, not as pointers: a pointer that has been an operand of an asm statement is no longer known to
// point at memory nobody writes, and its reads turn from scalar loads into vector loads with a full wait behind each.
__device__ __forceinline__ void fetch_together(const ActRows& a) {
    asm volatile("" : : "s"(a.image), "s"(a.stride), "s"(a.x), "s"(a.x_dtype), "s"(a.k), "s"(static_cast<int>(a.row_token != nullptr)), "s"(static_cast<int>(a.gamma != nullptr)),
                 "s"(a.round_f16), "s"(a.x_broadcast));
}
__device__ __forceinline__ void fetch_together(const WeightRoute& r) {
    asm volatile("" : : "s"(static_cast<int>(r.expert != nullptr)), "s"(r.expert_stride), "s"(r.extra), "s"(static_cast<int>(r.expert64 != nullptr)));
}
// the activation row (raw rows) that grid row `row` reads
__device__ __forceinline__ size_t raw_row_of(const ActRows& a, int row) {
    return a.x_broadcast ? 0 : (a.row_token ? static_cast<size_t>(a.row_token[row]) : static_cast<size_t>(row));
}
#endif
inline ActRows act_rows_from_image(const unsigned char* image, size_t stride, const int64_t* row_token = nullptr) {
    return ActRows{image, stride, nullptr, 0, 0, row_token, nullptr, 0.0f, 0};
}
inline ActRows act_rows_raw(const void* x, int x_dtype, int k, const float* gamma = nullptr, float eps = 0.0f, int round_f16 = 0) {
    return ActRows{nullptr, 0, x, x_dtype, k, nullptr, gamma, eps, round_f16};
}

// 256-weight super-block types: one activation image (act_image_256) serves any number of matvecs.
// Q4_K / Q5_K run in matvec_kquant.hip, IQ2_XXS / IQ1_M in matvec_iq_mfma.hip (matrix cores),
// Q2_K and the routed forms in matvec_dot4.hip (v_dot4).
int kquant_matvec_from_image(const ActRows& act, const uint8_t* w, int type_id, void* y, int y_dtype,
                             int rows, int n, int bpr, hipStream_t stream, WeightRoute route = WeightRoute{});
int dot4_matvec_from_image(const ActRows& act, const uint8_t* w, int type_id, void* y, int y_dtype,
                           int rows, int n, int bpr, hipStream_t stream, WeightRoute route = WeightRoute{});
// Q2_K / Q6_K and IQ4_XS on raw activation rows in the single-launch frames of matvec_kquant.hip (PLLM_ERR_UNSUPPORTED: take the
// kernels for prepared images)
// Q4_K / Q5_K, 2 - 16 raw rows of bf16 / fp16 activations (k a whole number of super-blocks) as rows of a half-precision matrix-core
// product in one pass over the weights (PLLM_ERR_UNSUPPORTED: not such a call)
int k45_rows16_matvec(const void* x, int x_dtype, const uint8_t* w, int type_id, void* y, int y_dtype, int rows, int k, int n, int bpr, hipStream_t stream);
// Q4_K / Q5_K on 17 - 48 activation rows: every block decoded once in registers and multiplied into all rows (fp16 matrix cores,
// exact weights); workspace = staged fp16 rows + partial sums of the slices along K
bool kquant_route_sum_supports(int type_id, int routes, int k, const uint8_t* w, size_t expert_stride);
int kquant_route_sum_matvec(const float* gate, const float* up, const float* route_w, float limit, int k, const WeightRoute& route, const uint8_t* w,
                            int type_id, void* y, int y_dtype, int n, int bpr, int routes, hipStream_t stream);
bool k45_rows64_reads_raw(const void* x, int x_dtype, int k, int n, int bpr);
bool k45_rows64_supports(int type_id, int rows, int n, int bpr, const uint8_t* w, bool raw16);
size_t k45_rows64_workspace_bytes(int rows, int n, int bpr);
int k45_rows64_gemm(const void* x, int x_dtype, const uint8_t* w, int type_id, void* y, int y_dtype, int rows, int k, int n, int bpr,
                    void* workspace, size_t workspace_bytes, hipStream_t stream);
int iq4xs_wave_matvec(const ActRows& act, const uint8_t* w, void* y, int y_dtype, int rows, int n, int bpr, hipStream_t stream,
                      WeightRoute route = WeightRoute{});
int groups16_wave_matvec(const ActRows& act, const uint8_t* w, int type_id, void* y, int y_dtype, int rows, int n, int bpr, hipStream_t stream,
                    WeightRoute route = WeightRoute{});
int iq_mfma_matvec_from_image(const ActRows& act, const uint8_t* w, int type_id, void* y, int y_dtype,
                              int rows, int n, int bpr, hipStream_t stream, WeightRoute route = WeightRoute{});
// any of the nine super-block types, dense or routed (defined beside the C ABI)
int superblock_matvec(const ActRows& act, const uint8_t* blocks, int type_id, void* y, int y_dtype,
                      int rows, int n, int bpr, hipStream_t stream, WeightRoute route = WeightRoute{});

// routed form: activation row r (image r, output row r) meets the matrix at w + y_expert[r] * expert_stride
int dot4_routed_matvec_from_image(const unsigned char* image, size_t stride, const uint8_t* w, int type_id, void* y, int y_dtype,
                                  int rows, int n, int bpr, const int32_t* y_expert, size_t expert_stride, hipStream_t stream);

// Routed experts of a single token on the matrix cores (moe_single_mfma.hip): IQ2_XXS / IQ1_M gate and
// up projections into per-route hidden images with one scale per 16 values, IQ1_M down projection
// with the sum over the routes inside the kernel.  `supports` says whether types, shapes and
// alignment fit; the hidden images need staged-image bytes per route (h_stride apart).
bool moe_single_mfma_supports(int w13_type, int w2_type, int dim, int inter, int routes, const void* x, const uint8_t* w1,
                              const uint8_t* w3, const uint8_t* w2);
int moe_single_w13_mfma(const void* x, int x_dtype, int dim, const int64_t* route_experts, const float* route_weights, int routes,
                        const uint8_t* w1, const uint8_t* w3, int w13_type, int inter, float limit, unsigned char* h_image, size_t h_stride,
                        hipStream_t stream);
int moe_single_w2_mfma(const unsigned char* h_image, size_t h_stride, int inter, const int64_t* route_experts, int routes, const uint8_t* w2,
                       float* y, int dim, hipStream_t stream, void* add_into = nullptr, int add_dtype = 0);

// Routed experts of several tokens on the matrix cores (same file): routes grouped by expert (seg), x images from
// act_image_256, hidden images with one scale per 16 values, per-route outputs into partial [R, dim].
bool moe_grouped_mfma_supports(int w13_type, int w2_type, int dim, int inter, const uint8_t* w1, const uint8_t* w3, const uint8_t* w2);
int moe_grouped_w13_mfma(const unsigned char* x_image, size_t x_stride, int dim, const int64_t* route_tokens, const int32_t* seg,
                         const float* route_weights, const uint8_t* w1, const uint8_t* w3, int w13_type, int inter, float limit,
                         unsigned char* h_image, size_t h_stride, int n_experts, hipStream_t stream);
// the same two steps with the routes as matrix rows in half precision (IQ2_XXS gate / up, IQ1_M down): x_rows_ws and h_rows_ws
// are moe_rows_x_bytes(tokens, dim) and moe_rows_h_bytes(routes, inter) bytes of workspace (activation rows, hidden rows)
bool moe_rows_supports(int w13_type, int w2_type, int dim, int inter, const uint8_t* w1, const uint8_t* w3, const uint8_t* w2);
size_t moe_rows_x_bytes(int64_t tokens, int64_t dim);
size_t moe_rows_h_bytes(int64_t routes, int64_t inter);
int moe_rows_w13(const void* x, int x_dtype, int tokens, int dim, void* x_rows_ws, const int64_t* route_tokens, const int32_t* seg,
                 const float* route_weights, const uint8_t* w1, const uint8_t* w3, int inter, float limit, void* h_rows_ws,
                 int n_experts, int routes, hipStream_t stream);
int moe_rows_w2(void* h_rows_ws, int inter, const int32_t* seg, const uint8_t* w2, float* partial, int dim, int n_experts, int routes,
                hipStream_t stream);
int moe_grouped_w2_mfma(const unsigned char* h_image, size_t h_stride, int inter, const int32_t* seg, const uint8_t* w2, float* partial, int dim,
                        int n_experts, hipStream_t stream);

// compute units of the current device (read once per process; 256 when no device answers)
int compute_units();

// prefill tile GEMM on f16 MFMA with decoded tiles (gemm_f16.hip)
bool gemm_f16_supports(int type_id);
size_t gemm_f16_workspace_bytes(int rows, int n, int bpr);
// routed experts as a batch of tile matmuls: activation rows staged once (fp16 rows + per-row scales),
// then one launch per projection over all experts
size_t gemm_f16_staged_bytes(int rows, int bpr);
int gemm_f16_stage_rows(const void* x, int x_dtype, const int64_t* row_map, int rows, int k, int bpr, void* staged, hipStream_t stream);
int gemm_f16_stage_swiglu(const float* g, const float* u, const float* route_weights, float limit, int rows, int inter, int bpr, void* staged,
                          hipStream_t stream);
int gemm_f16_grouped(const void* staged, const uint8_t* w, int type_id, size_t group_stride, const int32_t* seg, int groups,
                     float* y, int rows, int max_group_rows, int n, int bpr, hipStream_t stream);
// prefill matmul of Q4_K / Q5_K on the int8 matrix cores, activations quantized to 32-value int8 blocks (gemm_i8.hip)
bool gemm_i8_supports(int type_id);
size_t gemm_i8_workspace_bytes(int rows, int bpr);
int gemm_i8(const void* x, int x_dtype, const uint8_t* w, int type_id, void* y, int y_dtype,
            int rows, int k, int n, int bpr, void* workspace, size_t workspace_bytes, hipStream_t stream);
// FP8 x FP8 block-scaled matmul on the native FP8 matrix path (gemm_fp8.hip); k a multiple of 128
// (workspace: fp8_gemm_native_workspace_bytes for the partial sums of tiles cut along K; without it every tile runs whole)
size_t fp8_gemm_native_workspace_bytes(int rows, int k, int n);
int fp8_gemm_native(const uint8_t* a, const float* a_s, const uint8_t* b, const float* b_s, void* y, int y_dtype,
                    int rows, int k, int n, void* workspace, size_t workspace_bytes, hipStream_t stream);
int gemm_f16_fp8(const void* x, int x_dtype, const uint8_t* w, const float* wscale, void* y, int y_dtype,
                 int rows, int k, int n, void* workspace, size_t workspace_bytes, hipStream_t stream);
int gemm_f16(const void* x, int x_dtype, const uint8_t* w, int type_id, void* y, int y_dtype,
             int rows, int k, int n, int bpr, void* workspace, size_t workspace_bytes, hipStream_t stream);

// FP8 E4M3 weights [n, k] with float32 scales [ceil(n/128), ceil(k/128)] (matvec_fp8.hip)
int fp8_matvec(const void* x, int x_dtype, const uint8_t* w, const float* scale, void* y, int y_dtype,
               int rows, int k, int n, hipStream_t stream);
// the same with fp16 scale bits and explicit pitches (elements between activation / output rows, bytes between
// weight rows, entries between scale-table rows), and the fused form y = silu(gate . x) * (up . x)
int fp8_f16scale_matvec(const void* x, int x_dtype, size_t x_stride, const uint8_t* w, const uint16_t* scale, size_t weight_stride,
                        int scale_stride, void* y, int y_dtype, size_t y_stride, int rows, int k, int n, hipStream_t stream);
int fp8_bf16scale_matvec(const void* x, int x_dtype, size_t x_stride, const uint8_t* w, const uint16_t* scale, size_t weight_stride,
                         int scale_stride, void* y, int y_dtype, size_t y_stride, int rows, int k, int n, hipStream_t stream);
int fp8_f16scale_swiglu_matvec(const void* x, int x_dtype, size_t x_stride, const uint8_t* gate_w, const uint16_t* gate_scale,
                               const uint8_t* up_w, const uint16_t* up_scale, size_t weight_stride, int scale_stride,
                               void* y, int y_dtype, size_t y_stride, int rows, int k, int n, hipStream_t stream);
int fp8_f16scale_table_to_f32(const uint16_t* scale, int scale_stride, float* out, int n, int k, hipStream_t stream);

}  // namespace pllm
