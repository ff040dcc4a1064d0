// extern "C" surface of libpllm_hip: argument validation and dispatch by type and shape.
#include <mutex>

#include "pllm_internal.h"

namespace {

bool dtype_ok(int d) { return d == PLLM_F32 || d == PLLM_F16 || d == PLLM_BF16; }
bool fits_int(int64_t v) { return v > 0 && v <= 0x7fffffffLL; }

// from this many activation rows on, the tile GEMM replaces one matvec per row
constexpr int64_t kGemmMinRows = 16;

// From how many activation rows on the MFMA tile kernel serves a matmul.  The decode kernels read the matrix once per
// activation row (from cache after the first), the tile kernel decodes it once for up to 64 rows at a fixed cost.  Measured
// crossovers (us, decode kernel against tile kernel): at 17408x5120 Q4_K 5 rows (46.7 / 44), IQ1_M, IQ2_XS and IQ3_XXS 4 rows
// (50 - 56 / 45), Q6_K 5 rows (30.7 at 4 rows in the few-row form of its kernel / 54); at 5120x5120 Q4_K 12 rows (27.0 / 26.1), IQ1_M, IQ2_XS, IQ3_XXS 8 rows
// (27 - 30 / 28.5), Q6_K 5 rows (34.0 / 30.6); FP8 (one matvec per row) 3 rows (34.4 at 2 rows / 42) and 5 rows (22.6 at 4 rows / 24.1).
enum class RowClass { kKQuant, kWave8, kCodebook, kQ6K, kFp8 };
// Q6_K, five to eight rows: the eight-row form of the single-launch kernel while the matrix is this small (5120x5120 23.7 us against 29.4 - 37.6 on
// the tiles; level at 17408x5120, 301 against 256 us at 200064x3072)
constexpr int64_t kQ6KEightRowMaxWeights = int64_t{48} << 20;

static int64_t tile_gemm_min_rows(RowClass cls, int64_t weights) {
    const int size = weights >= (int64_t{64} << 20) ? 2 : (weights >= (int64_t{16} << 20) ? 1 : 0);
    if (size == 0) return kGemmMinRows;
    switch (cls) {
        case RowClass::kKQuant: return size == 2 ? 5 : 12;
        case RowClass::kWave8: return size == 2 ? 9 : 12;   // (up to eight rows: the few-row form of the single-launch kernel, Q4_K 17408x5120 at 5 - 8 float32 rows 34 - 36 us against 50 on the tiles)
        case RowClass::kCodebook: return size == 2 ? 4 : 8;
        case RowClass::kQ6K: return weights <= kQ6KEightRowMaxWeights ? 9 : 5;        // (up to four rows: the single-launch kernel's few-row form, 30.7 us at 17408x5120 and four rows against 54.3 on the tiles)
        case RowClass::kFp8: return size == 2 ? 3 : 5;
    }
    return kGemmMinRows;
}

static bool gguf_uses_tile_gemm(int type_id, int64_t rows, int64_t n, int64_t blocks_per_row) {
    if (!pllm::gemm_f16_supports(type_id)) return false;
    const RowClass cls = type_id == PLLM_TYPE_Q6_K ? RowClass::kQ6K
                         : (type_id == PLLM_TYPE_Q4_K || type_id == PLLM_TYPE_Q5_K || type_id == PLLM_TYPE_IQ4_XS) ? RowClass::kWave8
                         : (type_id == PLLM_TYPE_IQ1_M || type_id == PLLM_TYPE_IQ2_XS || type_id == PLLM_TYPE_IQ3_XXS) ? RowClass::kCodebook
                                                                                                                       : RowClass::kKQuant;
    return rows >= tile_gemm_min_rows(cls, n * blocks_per_row * 256);
}

}  // namespace

namespace pllm {
int compute_units() {
    static int cus = 0;                      // one device kind per process: the count is read once
    if (cus == 0) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
        else cus = 256;
    }
    return cus;
}
}  // namespace pllm

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
        case PLLM_TYPE_IQ2_XS: return 74;
        case PLLM_TYPE_IQ3_XXS: return 98;
        case PLLM_TYPE_IQ4_XS: return 136;
        case PLLM_TYPE_Q6_K: return 210;
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

// Calls of up to this many rows skip the activation pre-pass: the kernels quantize their activation rows themselves (every wave
// the slices of its own blocks, while its weights are in flight).  Q4_K, Q5_K and IQ4_XS take two to four rows through every
// block a wave fetches, one pass over the weights for all of them (Q4_K 17408x5120, float32 rows, us at 3 / 4 rows: 20.7 / 20.8
// against 27.8 / 28.6 with the pre-pass and the kernel that reads prepared images); the other formats run one grid row per row.
constexpr int64_t kInKernelQuantMaxRows = 4;
constexpr int64_t kInKernelQuantMaxRowsWave8 = 8;   // Q4_K, Q5_K, IQ4_XS: up to eight rows through every block a wave fetches

static bool quantizes_in_kernel(int type_id, int64_t rows, int64_t n, int64_t bpr) {
    const bool wave8 = type_id == PLLM_TYPE_Q4_K || type_id == PLLM_TYPE_Q5_K || type_id == PLLM_TYPE_IQ4_XS ||
                       (type_id == PLLM_TYPE_Q6_K && n * bpr * 256 <= kQ6KEightRowMaxWeights);
    if (rows > (wave8 ? kInKernelQuantMaxRowsWave8 : kInKernelQuantMaxRows)) return false;
    return pllm_gguf_block_bytes(type_id) != 0;
}

// Q4_K / Q5_K calls of 17 - 48 rows (up to 64 rows of 16-bit activations the kernel reads as they are: raw16) that the tile kernel
// would otherwise take
static bool uses_rows64(int type_id, int64_t rows, int64_t n, int64_t bpr, const uint8_t* blocks, bool raw16) {
    return gguf_uses_tile_gemm(type_id, rows, n, bpr) && pllm::k45_rows64_supports(type_id, static_cast<int>(rows), static_cast<int>(n), static_cast<int>(bpr), blocks, raw16);
}

}  // extern "C"

namespace pllm {
int superblock_matvec(const ActRows& act, const uint8_t* blocks, int type_id, void* y, int y_dtype,
                      int rows, int n, int bpr, hipStream_t s, WeightRoute route) {
    switch (type_id) {
        case PLLM_TYPE_Q2_K: {
            const int st = groups16_wave_matvec(act, blocks, type_id, y, y_dtype, rows, n, bpr, s, route);
            return st != PLLM_ERR_UNSUPPORTED ? st : dot4_matvec_from_image(act, blocks, type_id, y, y_dtype, rows, n, bpr, s, route);
        }
        case PLLM_TYPE_Q6_K: {
            const int st = groups16_wave_matvec(act, blocks, type_id, y, y_dtype, rows, n, bpr, s, route);
            return st != PLLM_ERR_UNSUPPORTED ? st : iq_mfma_matvec_from_image(act, blocks, type_id, y, y_dtype, rows, n, bpr, s, route);
        }
        case PLLM_TYPE_IQ2_XXS:
        case PLLM_TYPE_IQ1_M:
        case PLLM_TYPE_IQ2_XS:
        case PLLM_TYPE_IQ3_XXS:
            return iq_mfma_matvec_from_image(act, blocks, type_id, y, y_dtype, rows, n, bpr, s, route);
        case PLLM_TYPE_IQ4_XS: {
            const int st = iq4xs_wave_matvec(act, blocks, y, y_dtype, rows, n, bpr, s, route);
            if (st != PLLM_ERR_UNSUPPORTED) return st;
            return iq_mfma_matvec_from_image(act, blocks, type_id, y, y_dtype, rows, n, bpr, s, route);
        }
        case PLLM_TYPE_Q4_K:
        case PLLM_TYPE_Q5_K:
            return kquant_matvec_from_image(act, blocks, type_id, y, y_dtype, rows, n, bpr, s, route);
        default:
            return PLLM_ERR_UNSUPPORTED;
    }
}
}  // namespace pllm
using pllm::superblock_matvec;

extern "C" {

int pllm_gguf_quant_gemm(const void* x, int x_dtype, const uint8_t* blocks, int type_id, void* y, int y_dtype,
                         int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row,
                         void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !blocks || !y || !dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return PLLM_ERR_INVALID_ARGUMENT;
    if (!fits_int(rows) || !fits_int(k) || !fits_int(n) || !fits_int(blocks_per_row)) return PLLM_ERR_INVALID_ARGUMENT;
    if (blocks_per_row * 256 < k) return PLLM_ERR_INVALID_ARGUMENT;
    if (pllm_gguf_block_bytes(type_id) == 0) return PLLM_ERR_UNSUPPORTED;
    if (rows > 65535) return PLLM_ERR_UNSUPPORTED;
    if (!workspace || workspace_bytes < pllm_gguf_quant_gemm_workspace_bytes(type_id, rows, k, n, blocks_per_row)) return PLLM_ERR_WORKSPACE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int bpr = static_cast<int>(blocks_per_row);
    // Q4_K / Q5_K, 3 - 16 rows of 16-bit activations: one pass over the weights, the rows as matrix-core operands (two rows stay with
    // the int8 kernels: 21.1 against 22.7 us at 17408x5120)
    if (rows >= 3 && rows <= 16) {
        const int st16 = pllm::k45_rows16_matvec(x, x_dtype, blocks, type_id, y, y_dtype, static_cast<int>(rows), static_cast<int>(k), static_cast<int>(n), bpr, s);
        if (st16 != PLLM_ERR_UNSUPPORTED) return st16;
    }
    // Q4_K / Q5_K, 17 - 48 rows: every block decoded once in registers and multiplied into all rows
    if (uses_rows64(type_id, rows, n, blocks_per_row, blocks, pllm::k45_rows64_reads_raw(x, x_dtype, static_cast<int>(k), static_cast<int>(n), bpr)))
        return pllm::k45_rows64_gemm(x, x_dtype, blocks, type_id, y, y_dtype, static_cast<int>(rows), static_cast<int>(k), static_cast<int>(n), bpr,
                                     workspace, workspace_bytes, s);
    if (gguf_uses_tile_gemm(type_id, rows, n, blocks_per_row))
        return pllm::gemm_f16(x, x_dtype, blocks, type_id, y, y_dtype, static_cast<int>(rows), static_cast<int>(k), static_cast<int>(n), bpr,
                              workspace, workspace_bytes, s);
    if (quantizes_in_kernel(type_id, rows, n, blocks_per_row))
        return superblock_matvec(pllm::act_rows_raw(x, x_dtype, static_cast<int>(k)), blocks, type_id, y, y_dtype,
                                 static_cast<int>(rows), static_cast<int>(n), bpr, s);
    const int st = pllm::act_image_256(x, x_dtype, static_cast<int>(rows), static_cast<int>(k), bpr, workspace, s);
    if (st != PLLM_OK) return st;
    return superblock_matvec(pllm::act_rows_from_image(static_cast<const unsigned char*>(workspace), pllm::act_image_256_bytes(bpr)), blocks,
                             type_id, y, y_dtype, static_cast<int>(rows), static_cast<int>(n), bpr, s);
}

int pllm_gguf_quant_gemm_accumulate(const void* x, int x_dtype, const uint8_t* blocks, int type_id, void* y, int y_dtype,
                                    int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row,
                                    void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !blocks || !y || !dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return PLLM_ERR_INVALID_ARGUMENT;
    if (!fits_int(rows) || !fits_int(k) || !fits_int(n) || !fits_int(blocks_per_row)) return PLLM_ERR_INVALID_ARGUMENT;
    if (blocks_per_row * 256 < k) return PLLM_ERR_INVALID_ARGUMENT;
    if (pllm_gguf_block_bytes(type_id) == 0) return PLLM_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int bpr = static_cast<int>(blocks_per_row);
    const int into = y_dtype | pllm::kAccumulateInto;
    if (rows >= 3 && rows <= 16) {             // the same kernel as the plain operator takes for these calls
        const int st16 = pllm::k45_rows16_matvec(x, x_dtype, blocks, type_id, y, into, static_cast<int>(rows), static_cast<int>(k), static_cast<int>(n), bpr, s);
        if (st16 != PLLM_ERR_UNSUPPORTED) return st16;
    }
    // the decode kernels only: the row counts the plain operator hands to the tile kernel are not served
    if (rows > 65535 || gguf_uses_tile_gemm(type_id, rows, n, blocks_per_row)) return PLLM_ERR_UNSUPPORTED;
    if (!workspace || workspace_bytes < pllm_gguf_quant_gemm_workspace_bytes(type_id, rows, k, n, blocks_per_row)) return PLLM_ERR_WORKSPACE;
    if (quantizes_in_kernel(type_id, rows, n, blocks_per_row))
        return superblock_matvec(pllm::act_rows_raw(x, x_dtype, static_cast<int>(k)), blocks, type_id, y, into,
                                 static_cast<int>(rows), static_cast<int>(n), bpr, s);
    const int st = pllm::act_image_256(x, x_dtype, static_cast<int>(rows), static_cast<int>(k), bpr, workspace, s);
    if (st != PLLM_OK) return st;
    return superblock_matvec(pllm::act_rows_from_image(static_cast<const unsigned char*>(workspace), pllm::act_image_256_bytes(bpr)), blocks,
                             type_id, y, into, static_cast<int>(rows), static_cast<int>(n), bpr, s);
}

size_t pllm_gguf_quant_gemm_workspace_bytes(int type_id, int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row) {
    (void)k;
    if (!fits_int(rows) || !fits_int(n) || !fits_int(blocks_per_row) || pllm_gguf_block_bytes(type_id) == 0) return 0;
    if (gguf_uses_tile_gemm(type_id, rows, n, blocks_per_row)) {
        // (the weights' alignment is not known here: room for either kernel)
        const size_t tiles = pllm::gemm_f16_workspace_bytes(static_cast<int>(rows), static_cast<int>(n), static_cast<int>(blocks_per_row));
        const size_t rows64 = uses_rows64(type_id, rows, n, blocks_per_row, nullptr, true)
                                  ? pllm::k45_rows64_workspace_bytes(static_cast<int>(rows), static_cast<int>(n), static_cast<int>(blocks_per_row)) : 0;
        return tiles > rows64 ? tiles : rows64;
    }
    return pllm::act_image_256_bytes(static_cast<int>(blocks_per_row)) * static_cast<size_t>(rows);
}

// Q4_K / Q5_K with int8 activation semantics (activations quantized to 32-value int8 blocks, integer dots on the matrix cores)
size_t pllm_gguf_quant_gemm_q8_workspace_bytes(int type_id, int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row) {
    (void)k; (void)n;
    if (!fits_int(rows) || !fits_int(blocks_per_row) || !pllm::gemm_i8_supports(type_id)) return 0;
    return pllm::gemm_i8_workspace_bytes(static_cast<int>(rows), static_cast<int>(blocks_per_row));
}

int pllm_gguf_quant_gemm_q8(const void* x, int x_dtype, const uint8_t* blocks, int type_id, void* y, int y_dtype,
                            int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row,
                            void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !blocks || !y || !dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return PLLM_ERR_INVALID_ARGUMENT;
    if (!fits_int(rows) || !fits_int(k) || !fits_int(n) || !fits_int(blocks_per_row) || rows <= 0 || n <= 0 || k <= 0) return PLLM_ERR_INVALID_ARGUMENT;
    if (blocks_per_row * 256 < k) return PLLM_ERR_INVALID_ARGUMENT;
    if (!pllm::gemm_i8_supports(type_id)) return PLLM_ERR_UNSUPPORTED;
    return pllm::gemm_i8(x, x_dtype, blocks, type_id, y, y_dtype, static_cast<int>(rows), static_cast<int>(k), static_cast<int>(n),
                         static_cast<int>(blocks_per_row), workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

// ---- the entry point that allocates nothing ---------------------------------------------------------------------------
// Device memory for the activation image / the tile kernel's staging lives in a file-scope array instead of a caller's
// workspace.  Every GPU the library runs on holds its own copy of the array at its own address; the address is looked up once
// per device (hipGetSymbolAddress, with that device current) and kept.  Host code never passes the array's name to a kernel.
static __device__ __align__(256) unsigned char scratch[PLLM_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
void* scratch_address[kMaxDevices];

int static_scratch(void** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return PLLM_ERR_LAUNCH;
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_address[dev]) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return PLLM_ERR_LAUNCH;
        scratch_address[dev] = ptr;
    }
    *out = scratch_address[dev];
    return PLLM_OK;
}
}  // namespace

int pllm_gguf_quant_gemm_static_scratch(const void* x, int x_dtype, const uint8_t* blocks, int type_id, void* y, int y_dtype,
                                        int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row, void* stream) {
    if (!fits_int(rows) || !fits_int(k) || !fits_int(n) || !fits_int(blocks_per_row)) return PLLM_ERR_INVALID_ARGUMENT;
    if (pllm_gguf_block_bytes(type_id) == 0) return PLLM_ERR_UNSUPPORTED;
    // sizes beyond the array are refused: "workspace too small" names the limit that was hit
    if (pllm_gguf_quant_gemm_workspace_bytes(type_id, rows, k, n, blocks_per_row) > PLLM_STATIC_SCRATCH_BYTES) return PLLM_ERR_WORKSPACE;
    void* ptr = nullptr;
    const int st = static_scratch(&ptr);
    if (st != PLLM_OK) return st;
    // every kernel behind pllm_gguf_quant_gemm writes what it later reads of the workspace (image, staged rows, partial tiles)
    // within the same call, so nothing has to be cleared between calls
    return pllm_gguf_quant_gemm(x, x_dtype, blocks, type_id, y, y_dtype, rows, k, n, blocks_per_row, ptr, PLLM_STATIC_SCRATCH_BYTES, stream);
}

int pllm_fused_rms_norm(const void* x, int x_dtype, const float* weight, void* y, int y_dtype, int64_t rows, int64_t dim, float eps, void* stream) {
    if (!x || !weight || !y || !dtype_ok(x_dtype) || !dtype_ok(y_dtype) || rows <= 0 || dim <= 0 || !fits_int(rows) || !fits_int(dim))
        return PLLM_ERR_INVALID_ARGUMENT;
    return pllm::rms_norm_rows(x, x_dtype, weight, y, y_dtype, static_cast<int>(rows), static_cast<int>(dim), eps, static_cast<hipStream_t>(stream));
}

size_t pllm_attention_decode_workspace_bytes(int64_t batch, int64_t heads, int64_t pos) {
    if (!fits_int(batch) || !fits_int(heads) || pos < 0 || pos >= 0x7fffffffLL) return 0;
    return pllm::attention_decode_workspace_bytes(static_cast<int>(batch), static_cast<int>(heads), static_cast<int>(pos));
}

int pllm_attention_decode(const void* q, const void* k_new, const void* v_new, int dtype, const float* q_norm_weight, const float* k_norm_weight,
                          float eps, const float* cos_row, const float* sin_row, int64_t rope_dim, void* k_store, void* v_store,
                          int64_t store_batch_stride, int64_t store_head_stride, int64_t batch, int64_t heads, int64_t kv_heads, int64_t head_dim,
                          int64_t pos, void* out, void* workspace, size_t workspace_bytes, void* stream) {
    if (!q || !k_new || !v_new || !k_store || !v_store || !out || (dtype != PLLM_F16 && dtype != PLLM_BF16)) return PLLM_ERR_INVALID_ARGUMENT;
    if (!fits_int(batch) || !fits_int(heads) || !fits_int(kv_heads) || !fits_int(head_dim) || pos < 0 || pos >= 0x7fffffffLL || batch > 65535)
        return PLLM_ERR_INVALID_ARGUMENT;
    if (rope_dim < 0 || rope_dim > head_dim || (rope_dim > 0 && (!cos_row || !sin_row))) return PLLM_ERR_INVALID_ARGUMENT;
    if (store_head_stride < (pos + 1) * head_dim || store_batch_stride < kv_heads * store_head_stride) return PLLM_ERR_INVALID_ARGUMENT;
    if (!pllm::attention_decode_supports(static_cast<int>(heads), static_cast<int>(kv_heads), static_cast<int>(head_dim), static_cast<int>(rope_dim)))
        return PLLM_ERR_UNSUPPORTED;
    const uintptr_t all = reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k_new) | reinterpret_cast<uintptr_t>(v_new) |
                          reinterpret_cast<uintptr_t>(k_store) | reinterpret_cast<uintptr_t>(v_store) | reinterpret_cast<uintptr_t>(out);
    if ((all & 15u) || (store_batch_stride % 8) || (store_head_stride % 8)) return PLLM_ERR_INVALID_ARGUMENT;
    const size_t need = pllm_attention_decode_workspace_bytes(batch, heads, pos);
    if (need > 0 && (!workspace || workspace_bytes < need)) return PLLM_ERR_WORKSPACE;
    return pllm::attention_decode(q, k_new, v_new, dtype, q_norm_weight, k_norm_weight, eps, cos_row, sin_row, static_cast<int>(rope_dim), k_store, v_store,
                                  static_cast<size_t>(store_batch_stride), static_cast<size_t>(store_head_stride), static_cast<int>(batch),
                                  static_cast<int>(heads), static_cast<int>(kv_heads), static_cast<int>(pos), out, workspace,
                                  static_cast<hipStream_t>(stream));
}

// normalized rows (fp16) ahead of the matmul's own workspace when the call has too many rows for the in-kernel form
static size_t rmsnorm_rows_bytes(int64_t rows, int64_t k) {
    return rows <= kInKernelQuantMaxRows ? 0 : (static_cast<size_t>(rows) * static_cast<size_t>(k) * 2 + 255) & ~static_cast<size_t>(255);
}

size_t pllm_gguf_quant_gemm_rmsnorm_workspace_bytes(int type_id, int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row) {
    const size_t inner = pllm_gguf_quant_gemm_workspace_bytes(type_id, rows, k, n, blocks_per_row);
    return inner == 0 ? 0 : inner + rmsnorm_rows_bytes(rows, k);
}

int pllm_gguf_quant_gemm_rmsnorm(const void* x, int x_dtype, const float* norm_weight, float eps, int round_fp16,
                                 const uint8_t* blocks, int type_id, void* y, int y_dtype,
                                 int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row,
                                 void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !norm_weight || !blocks || !y || !dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return PLLM_ERR_INVALID_ARGUMENT;
    if (!fits_int(rows) || !fits_int(k) || !fits_int(n) || !fits_int(blocks_per_row) || rows <= 0 || k <= 0) return PLLM_ERR_INVALID_ARGUMENT;
    if (blocks_per_row * 256 < k) return PLLM_ERR_INVALID_ARGUMENT;
    if (pllm_gguf_block_bytes(type_id) == 0) return PLLM_ERR_UNSUPPORTED;
    if (rows > 65535) return PLLM_ERR_UNSUPPORTED;
    if (!workspace || workspace_bytes < pllm_gguf_quant_gemm_rmsnorm_workspace_bytes(type_id, rows, k, n, blocks_per_row)) return PLLM_ERR_WORKSPACE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (rows <= kInKernelQuantMaxRows)       // every workgroup normalizes and quantizes its activation row itself: one launch
        return superblock_matvec(pllm::act_rows_raw(x, x_dtype, static_cast<int>(k), norm_weight, eps, round_fp16), blocks, type_id, y, y_dtype,
                                 static_cast<int>(rows), static_cast<int>(n), static_cast<int>(blocks_per_row), s);
    // many rows: normalized fp16 rows into the head of the workspace, then the ordinary operator on them
    const size_t head = rmsnorm_rows_bytes(rows, k);
    const int st = pllm::rms_norm_rows(x, x_dtype, norm_weight, workspace, PLLM_F16, static_cast<int>(rows), static_cast<int>(k), eps, s);
    if (st != PLLM_OK) return st;
    return pllm_gguf_quant_gemm(workspace, PLLM_F16, blocks, type_id, y, y_dtype, rows, k, n, blocks_per_row,
                                static_cast<char*>(workspace) + head, workspace_bytes - head, stream);
}

int pllm_gguf_quant_gemm_multi(const void* x, int x_dtype, const float* norm_weight, float eps, int round_fp16,
                               int count, const uint8_t* const* blocks, const int64_t* n, int type_id, void* const* y, int y_dtype,
                               int64_t rows, int64_t k, int64_t blocks_per_row, void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !blocks || !n || !y || !dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return PLLM_ERR_INVALID_ARGUMENT;
    if (count < 1 || count > 4 || !fits_int(rows) || !fits_int(k) || !fits_int(blocks_per_row) || rows <= 0 || k <= 0) return PLLM_ERR_INVALID_ARGUMENT;
    if (blocks_per_row * 256 < k) return PLLM_ERR_INVALID_ARGUMENT;
    int64_t total_n = 0;
    for (int m = 0; m < count; ++m) {
        if (!blocks[m] || !y[m] || n[m] <= 0 || !fits_int(n[m])) return PLLM_ERR_INVALID_ARGUMENT;
        total_n += n[m];
    }
    if (pllm_gguf_block_bytes(type_id) == 0) return PLLM_ERR_UNSUPPORTED;
    // one launch exists in the matrix-core decode kernels; Q2_K (and anything else) is left to one call per matrix
    if (type_id == PLLM_TYPE_Q2_K) return PLLM_ERR_UNSUPPORTED;
    if (rows > 65535 || gguf_uses_tile_gemm(type_id, rows, total_n, blocks_per_row)) return PLLM_ERR_UNSUPPORTED;
    const bool raw = rows <= kInKernelQuantMaxRows && (norm_weight || quantizes_in_kernel(type_id, rows, total_n, blocks_per_row));
    if (norm_weight && !raw) return PLLM_ERR_UNSUPPORTED;                    // the normalisation exists inside the kernel only
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int bpr = static_cast<int>(blocks_per_row);
    if (!norm_weight && rows >= 3 && rows <= 16) {   // the single-matrix operator's kernel for these calls, one launch per matrix
        int m = 0;
        for (; m < count; ++m) {
            const int st = pllm::k45_rows16_matvec(x, x_dtype, blocks[m], type_id, y[m], y_dtype, static_cast<int>(rows), static_cast<int>(k),
                                                   static_cast<int>(n[m]), bpr, s);
            if (st == PLLM_ERR_UNSUPPORTED) break;   // (a matrix it does not take: every output is written again below)
            if (st != PLLM_OK) return st;
        }
        if (m == count) return PLLM_OK;
    }
    pllm::ActRows act = pllm::act_rows_raw(x, x_dtype, static_cast<int>(k), norm_weight, eps, round_fp16);
    if (!raw) {
        if (!workspace || workspace_bytes < pllm_activation_image_bytes(rows, blocks_per_row)) return PLLM_ERR_WORKSPACE;
        const int st = pllm::act_image_256(x, x_dtype, static_cast<int>(rows), static_cast<int>(k), bpr, workspace, s);
        if (st != PLLM_OK) return st;
        act = pllm::act_rows_from_image(static_cast<const unsigned char*>(workspace), pllm::act_image_256_bytes(bpr));
    }
    pllm::WeightRoute all{};
    for (int m = 1; m < count; ++m) {
        all.more_w[m - 1] = blocks[m];
        all.more_y[m - 1] = y[m];
        all.more_n[m - 1] = static_cast<int>(n[m]);
    }
    all.extra = count - 1;
    return superblock_matvec(act, blocks[0], type_id, y[0], y_dtype, static_cast<int>(rows), static_cast<int>(n[0]), bpr, s, all);
}

size_t pllm_activation_image_bytes(int64_t rows, int64_t blocks_per_row) {
    if (!fits_int(rows) || !fits_int(blocks_per_row)) return 0;
    return pllm::act_image_256_bytes(static_cast<int>(blocks_per_row)) * static_cast<size_t>(rows);
}

int pllm_quantize_activations(const void* x, int x_dtype, int64_t rows, int64_t k, int64_t blocks_per_row,
                              void* image, size_t image_bytes, void* stream) {
    if (!x || !image || !dtype_ok(x_dtype) || !fits_int(rows) || !fits_int(k) || !fits_int(blocks_per_row)) return PLLM_ERR_INVALID_ARGUMENT;
    if (blocks_per_row * 256 < k) return PLLM_ERR_INVALID_ARGUMENT;
    if (rows > 65535) return PLLM_ERR_UNSUPPORTED;
    if (image_bytes < pllm_activation_image_bytes(rows, blocks_per_row)) return PLLM_ERR_WORKSPACE;
    return pllm::act_image_256(x, x_dtype, static_cast<int>(rows), static_cast<int>(k), static_cast<int>(blocks_per_row), image,
                               static_cast<hipStream_t>(stream));
}

static int prequantized_matvec(const void* image, const uint8_t* blocks, int type_id, void* y, int y_dtype, int into,
                               int64_t rows, int64_t n, int64_t blocks_per_row, void* stream) {
    if (!image || !blocks || !y || !dtype_ok(y_dtype) || !fits_int(rows) || !fits_int(n) || !fits_int(blocks_per_row)) return PLLM_ERR_INVALID_ARGUMENT;
    if (pllm_gguf_block_bytes(type_id) == 0) return PLLM_ERR_UNSUPPORTED;
    if (rows > 65535) return PLLM_ERR_UNSUPPORTED;
    const int bpr = static_cast<int>(blocks_per_row);
    return superblock_matvec(pllm::act_rows_from_image(static_cast<const unsigned char*>(image), pllm::act_image_256_bytes(bpr)), blocks,
                             type_id, y, y_dtype | into, static_cast<int>(rows), static_cast<int>(n), bpr, static_cast<hipStream_t>(stream));
}

int pllm_gguf_quant_gemm_prequantized(const void* image, const uint8_t* blocks, int type_id, void* y, int y_dtype,
                                      int64_t rows, int64_t n, int64_t blocks_per_row, void* stream) {
    return prequantized_matvec(image, blocks, type_id, y, y_dtype, 0, rows, n, blocks_per_row, stream);
}

int pllm_gguf_quant_gemm_prequantized_accumulate(const void* image, const uint8_t* blocks, int type_id, void* y, int y_dtype,
                                                 int64_t rows, int64_t n, int64_t blocks_per_row, void* stream) {
    return prequantized_matvec(image, blocks, type_id, y, y_dtype, pllm::kAccumulateInto, rows, n, blocks_per_row, stream);
}

int pllm_swiglu_quantize_activations(const void* gate, const void* up, int gu_dtype, int64_t rows, int64_t k, int64_t blocks_per_row,
                                     float swiglu_limit, int round_dtype, void* image, size_t image_bytes, void* stream) {
    if (!gate || !up || !image || !dtype_ok(gu_dtype) || !dtype_ok(round_dtype)) return PLLM_ERR_INVALID_ARGUMENT;
    if (!fits_int(rows) || !fits_int(k) || !fits_int(blocks_per_row) || rows <= 0 || k <= 0) return PLLM_ERR_INVALID_ARGUMENT;
    if (blocks_per_row * 256 < k) return PLLM_ERR_INVALID_ARGUMENT;
    if (rows > 65535) return PLLM_ERR_UNSUPPORTED;
    if (image_bytes < pllm_activation_image_bytes(rows, blocks_per_row)) return PLLM_ERR_WORKSPACE;
    return pllm::swiglu_image_256(gate, up, gu_dtype, swiglu_limit, round_dtype, static_cast<int>(rows), static_cast<int>(k),
                                  static_cast<int>(blocks_per_row), image, static_cast<hipStream_t>(stream));
}

int pllm_gguf_quant_gemm_pair(const void* x, int x_dtype, const uint8_t* blocks0, int type_id0, const uint8_t* blocks1, int type_id1,
                              void* y, int y_dtype, int64_t rows, int64_t k, int64_t n, int64_t blocks_per_row,
                              void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !blocks0 || !blocks1 || !y || !dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return PLLM_ERR_INVALID_ARGUMENT;
    if (!fits_int(rows) || !fits_int(k) || !fits_int(n) || !fits_int(blocks_per_row)) return PLLM_ERR_INVALID_ARGUMENT;
    if (blocks_per_row * 256 < k) return PLLM_ERR_INVALID_ARGUMENT;
    if (pllm_gguf_block_bytes(type_id0) == 0 || pllm_gguf_block_bytes(type_id1) == 0) return PLLM_ERR_UNSUPPORTED;
    if (rows > 65535) return PLLM_ERR_UNSUPPORTED;
    if (!workspace || workspace_bytes < pllm_activation_image_bytes(rows, blocks_per_row)) return PLLM_ERR_WORKSPACE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int bpr = static_cast<int>(blocks_per_row);
    const int R = static_cast<int>(rows), N = static_cast<int>(n);
    const size_t esize = y_dtype == PLLM_F32 ? 4 : 2;
    if (rows >= 3 && rows <= 16) {             // the kernel the single-matrix operator takes for these calls, once per matrix
        const int st0 = pllm::k45_rows16_matvec(x, x_dtype, blocks0, type_id0, y, y_dtype, R, static_cast<int>(k), N, bpr, s);
        if (st0 != PLLM_ERR_UNSUPPORTED) {
            if (st0 != PLLM_OK) return st0;
            void* y1 = static_cast<char*>(y) + static_cast<size_t>(rows) * n * esize;
            const int st1 = pllm::k45_rows16_matvec(x, x_dtype, blocks1, type_id1, y1, y_dtype, R, static_cast<int>(k), N, bpr, s);
            if (st1 != PLLM_ERR_UNSUPPORTED) return st1;
            // (mixed pair: the second matrix on the kernels below, as its own operator call would run)
            if (quantizes_in_kernel(type_id1, rows, n, blocks_per_row))
                return superblock_matvec(pllm::act_rows_raw(x, x_dtype, static_cast<int>(k)), blocks1, type_id1, y1, y_dtype, R, N, bpr, s);
            const int sti = pllm::act_image_256(x, x_dtype, R, static_cast<int>(k), bpr, workspace, s);
            if (sti != PLLM_OK) return sti;
            return superblock_matvec(pllm::act_rows_from_image(static_cast<const unsigned char*>(workspace), pllm::act_image_256_bytes(bpr)), blocks1,
                                     type_id1, y1, y_dtype, R, N, bpr, s);
        }
    }
    const bool k45 = type_id0 == type_id1 && (type_id0 == PLLM_TYPE_Q4_K || type_id0 == PLLM_TYPE_Q5_K);
    const bool raw = k45 ? quantizes_in_kernel(type_id0, rows, 2 * n, blocks_per_row)
                         : quantizes_in_kernel(type_id0, rows, n, blocks_per_row) && quantizes_in_kernel(type_id1, rows, n, blocks_per_row);
    pllm::ActRows act = pllm::act_rows_raw(x, x_dtype, static_cast<int>(k));
    if (!raw) {
        const int st = pllm::act_image_256(x, x_dtype, R, static_cast<int>(k), bpr, workspace, s);
        if (st != PLLM_OK) return st;
        act = pllm::act_rows_from_image(static_cast<const unsigned char*>(workspace), pllm::act_image_256_bytes(bpr));
    }
    if (k45) {                               // one launch over both matrices (grid.z)
        pllm::WeightRoute both{};
        both.more_w[0] = blocks1;
        both.more_y[0] = static_cast<char*>(y) + static_cast<size_t>(rows) * n * esize;
        both.more_n[0] = N;
        both.extra = 1;
        return superblock_matvec(act, blocks0, type_id0, y, y_dtype, R, N, bpr, s, both);
    }
    const int st = superblock_matvec(act, blocks0, type_id0, y, y_dtype, R, N, bpr, s);
    if (st != PLLM_OK) return st;
    return superblock_matvec(act, blocks1, type_id1, static_cast<char*>(y) + static_cast<size_t>(rows) * n * esize, y_dtype, R, N, bpr, s);
}

int pllm_fp8_gemm(const uint8_t* a, const float* a_scale, const uint8_t* weight, const float* scale, void* y, int y_dtype,
                  int64_t rows, int64_t k, int64_t n, void* stream) {
    if (!a || !a_scale || !weight || !scale || !y || !dtype_ok(y_dtype)) return PLLM_ERR_INVALID_ARGUMENT;
    if (!fits_int(rows) || !fits_int(k) || !fits_int(n) || rows <= 0 || n <= 0) return PLLM_ERR_INVALID_ARGUMENT;
    return pllm::fp8_gemm_native(a, a_scale, weight, scale, y, y_dtype, static_cast<int>(rows), static_cast<int>(k), static_cast<int>(n),
                                 nullptr, 0, static_cast<hipStream_t>(stream));
}

size_t pllm_fp8_gemm_workspace_bytes(int64_t rows, int64_t k, int64_t n) {
    if (!fits_int(rows) || !fits_int(k) || !fits_int(n)) return 0;
    return pllm::fp8_gemm_native_workspace_bytes(static_cast<int>(rows), static_cast<int>(k), static_cast<int>(n));
}

int pllm_fp8_gemm_ws(const uint8_t* a, const float* a_scale, const uint8_t* weight, const float* scale, void* y, int y_dtype,
                     int64_t rows, int64_t k, int64_t n, void* workspace, size_t workspace_bytes, void* stream) {
    if (!a || !a_scale || !weight || !scale || !y || !dtype_ok(y_dtype)) return PLLM_ERR_INVALID_ARGUMENT;
    if (!fits_int(rows) || !fits_int(k) || !fits_int(n) || rows <= 0 || n <= 0) return PLLM_ERR_INVALID_ARGUMENT;
    return pllm::fp8_gemm_native(a, a_scale, weight, scale, y, y_dtype, static_cast<int>(rows), static_cast<int>(k), static_cast<int>(n),
                                 workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

// the tile GEMM serves many rows of 256-aligned k; everything else takes the matvec (no workspace)
static bool fp8_uses_gemm(int64_t rows, int64_t k, int64_t n) { return k % 256 == 0 && rows >= tile_gemm_min_rows(RowClass::kFp8, n * k); }
// float32 activations keep the float32 matvec (rel-L2 <= 1e-5 against the float statement of the operator, src/kernels/ops.py:641-648)
// for every row count below 16; from 16 rows on they take the tile kernel like the 16-bit types (operands rounded to fp16, <= 1e-3).
// up to 16 rows of 16-bit activations run the matrix-core form of the matvec (one pass over the weights, exact products)
static bool fp8_uses_gemm_for(int x_dtype, int64_t rows, int64_t k, int64_t n) {
    return fp8_uses_gemm(rows, k, n) && (x_dtype == PLLM_F32 ? rows >= 16 : rows > 16);
}

size_t pllm_fp8_block_gemm_workspace_bytes(int64_t rows, int64_t k, int64_t n) {
    if (!fits_int(rows) || !fits_int(k) || !fits_int(n) || !fp8_uses_gemm(rows, k, n)) return 0;
    return pllm::gemm_f16_workspace_bytes(static_cast<int>(rows), static_cast<int>(n), static_cast<int>(k / 256));
}

int pllm_fp8_block_gemm(const void* x, int x_dtype, const uint8_t* weight, const float* scale, void* y, int y_dtype,
                        int64_t rows, int64_t k, int64_t n, void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !weight || !scale || !y || !dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return PLLM_ERR_INVALID_ARGUMENT;
    if (!fits_int(rows) || !fits_int(k) || !fits_int(n)) return PLLM_ERR_INVALID_ARGUMENT;
    if (fp8_uses_gemm_for(x_dtype, rows, k, n))
        return pllm::gemm_f16_fp8(x, x_dtype, weight, scale, y, y_dtype, static_cast<int>(rows), static_cast<int>(k), static_cast<int>(n),
                                  workspace, workspace_bytes, static_cast<hipStream_t>(stream));
    if (rows > 65535) return PLLM_ERR_UNSUPPORTED;
    return pllm::fp8_matvec(x, x_dtype, weight, scale, y, y_dtype, static_cast<int>(rows), static_cast<int>(k),
                            static_cast<int>(n), static_cast<hipStream_t>(stream));
}

int pllm_fp8_block_gemm_accumulate(const void* x, int x_dtype, const uint8_t* weight, const float* scale, void* y, int y_dtype,
                                   int64_t rows, int64_t k, int64_t n, void* stream) {
    if (!x || !weight || !scale || !y || !dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return PLLM_ERR_INVALID_ARGUMENT;
    if (!fits_int(rows) || !fits_int(k) || !fits_int(n)) return PLLM_ERR_INVALID_ARGUMENT;
    // the matvec only: the row counts pllm_fp8_block_gemm hands to the tile kernel are not served
    if (rows > 65535 || fp8_uses_gemm_for(x_dtype, rows, k, n)) return PLLM_ERR_UNSUPPORTED;
    return pllm::fp8_matvec(x, x_dtype, weight, scale, y, y_dtype | pllm::kAccumulateInto, static_cast<int>(rows), static_cast<int>(k),
                            static_cast<int>(n), static_cast<hipStream_t>(stream));
}

// ---- FP8 with fp16 scales: the raw-pointer operators of the reference's C++ engine -----------------------------------

static bool fp16scale_args_ok(const void* x, const void* w, const void* scale, const void* y, int64_t rows, int64_t cols,
                              int64_t weight_stride, int64_t scale_stride) {
    // cpp_engine/cuda/qwen_fp8_ops.cu:951-955 (valid_common) plus the pitch check every entry point adds
    return x && w && scale && y && rows > 0 && cols > 0 && fits_int(rows) && fits_int(cols) && fits_int(scale_stride) &&
           scale_stride >= (cols + 127) / 128 && weight_stride >= cols;
}

int pllm_fp8_fp16scale_matvec(const void* x, int x_dtype, const uint8_t* weight, const uint16_t* scale_fp16, void* y, int y_dtype,
                              int64_t rows, int64_t cols, int64_t weight_stride, int64_t scale_stride, void* stream) {
    if (!dtype_ok(x_dtype) || !dtype_ok(y_dtype) || !fp16scale_args_ok(x, weight, scale_fp16, y, rows, cols, weight_stride, scale_stride))
        return PLLM_ERR_INVALID_ARGUMENT;
    return pllm::fp8_f16scale_matvec(x, x_dtype, static_cast<size_t>(cols), weight, scale_fp16, static_cast<size_t>(weight_stride),
                                     static_cast<int>(scale_stride), y, y_dtype, static_cast<size_t>(rows), 1, static_cast<int>(cols),
                                     static_cast<int>(rows), static_cast<hipStream_t>(stream));
}

int pllm_fp8_fp16scale_swiglu_matvec(const void* x, int x_dtype, const uint8_t* gate_weight, const uint16_t* gate_scale_fp16,
                                     const uint8_t* up_weight, const uint16_t* up_scale_fp16, void* y, int y_dtype,
                                     int64_t batch, int64_t rows, int64_t cols, int64_t x_stride, int64_t y_stride,
                                     int64_t weight_stride, int64_t scale_stride, void* stream) {
    if (!dtype_ok(x_dtype) || !dtype_ok(y_dtype) || !up_weight || !up_scale_fp16 ||
        !fp16scale_args_ok(x, gate_weight, gate_scale_fp16, y, rows, cols, weight_stride, scale_stride))
        return PLLM_ERR_INVALID_ARGUMENT;
    if (batch <= 0 || x_stride < cols || y_stride < rows) return PLLM_ERR_INVALID_ARGUMENT;
    if (batch > 65535) return PLLM_ERR_UNSUPPORTED;
    return pllm::fp8_f16scale_swiglu_matvec(x, x_dtype, static_cast<size_t>(x_stride), gate_weight, gate_scale_fp16, up_weight, up_scale_fp16,
                                            static_cast<size_t>(weight_stride), static_cast<int>(scale_stride), y, y_dtype,
                                            static_cast<size_t>(y_stride), static_cast<int>(batch), static_cast<int>(cols),
                                            static_cast<int>(rows), static_cast<hipStream_t>(stream));
}

int pllm_fp8_bf16scale_matmul_rows(const void* x, int x_dtype, const uint8_t* weight, const uint16_t* scale_bf16, void* y, int y_dtype,
                                   int64_t batch, int64_t rows, int64_t cols, int64_t x_stride, int64_t y_stride,
                                   int64_t weight_stride, int64_t scale_stride, void* stream) {
    if (!dtype_ok(x_dtype) || !dtype_ok(y_dtype) || !fp16scale_args_ok(x, weight, scale_bf16, y, rows, cols, weight_stride, scale_stride))
        return PLLM_ERR_INVALID_ARGUMENT;
    if (batch <= 0 || x_stride < cols || y_stride < rows) return PLLM_ERR_INVALID_ARGUMENT;
    if (batch > 65535) return PLLM_ERR_UNSUPPORTED;
    return pllm::fp8_bf16scale_matvec(x, x_dtype, static_cast<size_t>(x_stride), weight, scale_bf16, static_cast<size_t>(weight_stride),
                                      static_cast<int>(scale_stride), y, y_dtype, static_cast<size_t>(y_stride), static_cast<int>(batch),
                                      static_cast<int>(cols), static_cast<int>(rows), static_cast<hipStream_t>(stream));
}

// Many rows of 16-bit activations with dense pitches and 256-aligned cols run on the tile kernel (float32 scale table in
// the workspace).  float32 activations stay on the float32 matvec, row by row: the tile kernel rounds its operands to fp16,
// which is inside the bound the reference sets for its fp16-storage variants (2e-2) but not the 2e-4 of its float32 ones.
static bool fp16scale_uses_gemm(int x_dtype, int64_t batch, int64_t rows, int64_t cols, int64_t x_stride, int64_t y_stride, int64_t weight_stride) {
    return x_dtype != PLLM_F32 && batch > 16 && fp8_uses_gemm(batch, cols, rows) && x_stride == cols && y_stride == rows && weight_stride == cols;
}

static size_t fp16scale_table_bytes(int64_t rows, int64_t cols) {
    return (static_cast<size_t>((rows + 127) / 128) * static_cast<size_t>((cols + 127) / 128) * sizeof(float) + 255) & ~static_cast<size_t>(255);
}

size_t pllm_fp8_fp16scale_matmul_rows_workspace_bytes(int64_t batch, int64_t rows, int64_t cols) {
    if (!fits_int(batch) || !fits_int(rows) || !fits_int(cols) || !fp8_uses_gemm(batch, cols, rows)) return 0;
    return fp16scale_table_bytes(rows, cols) + pllm::gemm_f16_workspace_bytes(static_cast<int>(batch), static_cast<int>(rows), static_cast<int>(cols / 256));
}

int pllm_fp8_fp16scale_matmul_rows(const void* x, int x_dtype, const uint8_t* weight, const uint16_t* scale_fp16, void* y, int y_dtype,
                                   int64_t batch, int64_t rows, int64_t cols, int64_t x_stride, int64_t y_stride,
                                   int64_t weight_stride, int64_t scale_stride, void* workspace, size_t workspace_bytes, void* stream) {
    if (!dtype_ok(x_dtype) || !dtype_ok(y_dtype) || !fp16scale_args_ok(x, weight, scale_fp16, y, rows, cols, weight_stride, scale_stride))
        return PLLM_ERR_INVALID_ARGUMENT;
    if (batch <= 0 || !fits_int(batch) || x_stride < cols || y_stride < rows) return PLLM_ERR_INVALID_ARGUMENT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (fp16scale_uses_gemm(x_dtype, batch, rows, cols, x_stride, y_stride, weight_stride) && workspace &&
        workspace_bytes >= pllm_fp8_fp16scale_matmul_rows_workspace_bytes(batch, rows, cols)) {
        float* table = static_cast<float*>(workspace);
        const size_t table_bytes = fp16scale_table_bytes(rows, cols);
        const int st = pllm::fp8_f16scale_table_to_f32(scale_fp16, static_cast<int>(scale_stride), table, static_cast<int>(rows), static_cast<int>(cols), s);
        if (st != PLLM_OK) return st;
        return pllm::gemm_f16_fp8(x, x_dtype, weight, table, y, y_dtype, static_cast<int>(batch), static_cast<int>(cols), static_cast<int>(rows),
                                  static_cast<char*>(workspace) + table_bytes, workspace_bytes - table_bytes, s);
    }
    if (batch > 65535) return PLLM_ERR_UNSUPPORTED;
    return pllm::fp8_f16scale_matvec(x, x_dtype, static_cast<size_t>(x_stride), weight, scale_fp16, static_cast<size_t>(weight_stride),
                                     static_cast<int>(scale_stride), y, y_dtype, static_cast<size_t>(y_stride), static_cast<int>(batch),
                                     static_cast<int>(cols), static_cast<int>(rows), s);
}

}  // extern "C"
