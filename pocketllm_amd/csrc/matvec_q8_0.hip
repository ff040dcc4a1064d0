// Decode matvec over raw Q8_0 blocks (34 B = fp16 scale + 32 int8), bandwidth-bound, wave64.
//
// 34-byte blocks are only 2-byte aligned, but a PAIR of blocks is 68 bytes = 17 dwords and 4-byte
// aligned whenever the row holds an even number of blocks.  A lane owns one pair at a time and pulls
// it in with four 16-byte loads and one 4-byte load (dword alignment is all global_load_dwordx4
// needs); neighbouring lanes sit 68 bytes apart, so a wave's five loads together sweep one
// contiguous span of the row and every fetched cache line is used in full.  The activations sit in
// LDS as an IMAGE OF THE SAME STREAM: per pair two zero bytes where the weight stream has a scale,
// 32 int8 codes, two zeros, 32 codes (padded to 80 bytes so that ds_read_b128 stays aligned).  A
// dword of weights and the image dword at the same offset line up byte for byte, v_dot4_i32_i8 of
// the two is a partial dot of exactly one block (the scale bytes meet zeros): dwords 0..8 belong to
// the even block, 9..16 to the odd one.  TL lanes share a row; their partial sums meet in a
// cross-lane reduction.
#include "pllm_device.h"
#include "pllm_internal.h"
#include <algorithm>

namespace pllm {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;

struct PairRegs { uint4 a, b, c, d; uint32_t e; };

__device__ __forceinline__ void load_pair(PairRegs& r, const uint8_t* p) {
    const uint32_t* q = reinterpret_cast<const uint32_t*>(p);
    r.a = make_uint4(q[0], q[1], q[2], q[3]);
    r.b = make_uint4(q[4], q[5], q[6], q[7]);
    r.c = make_uint4(q[8], q[9], q[10], q[11]);
    r.d = make_uint4(q[12], q[13], q[14], q[15]);
    r.e = q[16];
}

__device__ __forceinline__ void zero_pair(PairRegs& r) {
    r.a = make_uint4(0, 0, 0, 0); r.b = r.a; r.c = r.a; r.d = r.a; r.e = 0;
}

// image: int8 [pairs][80] (hi) | int8 [pairs][80] (lo) | float xs[2 * pairs]
__device__ __forceinline__ float pair_dot(const PairRegs& r, int pair, const unsigned char* img_hi, const unsigned char* img_lo,
                                          const float* xs) {
    const uint4* ih = reinterpret_cast<const uint4*>(img_hi + pair * 80);
    const uint4* il = reinterpret_cast<const uint4*>(img_lo + pair * 80);
    const uint4 h0 = ih[0], h1 = ih[1], h2 = ih[2], h3 = ih[3], h4 = ih[4];
    const uint4 l0 = il[0], l1 = il[1], l2 = il[2], l3 = il[3], l4 = il[4];
    // even block: dwords 0..8
    int ah = dot4(r.a.x, h0.x, 0); ah = dot4(r.a.y, h0.y, ah); ah = dot4(r.a.z, h0.z, ah); ah = dot4(r.a.w, h0.w, ah);
    ah = dot4(r.b.x, h1.x, ah); ah = dot4(r.b.y, h1.y, ah); ah = dot4(r.b.z, h1.z, ah); ah = dot4(r.b.w, h1.w, ah);
    ah = dot4(r.c.x, h2.x, ah);
    int al = dot4(r.a.x, l0.x, 0); al = dot4(r.a.y, l0.y, al); al = dot4(r.a.z, l0.z, al); al = dot4(r.a.w, l0.w, al);
    al = dot4(r.b.x, l1.x, al); al = dot4(r.b.y, l1.y, al); al = dot4(r.b.z, l1.z, al); al = dot4(r.b.w, l1.w, al);
    al = dot4(r.c.x, l2.x, al);
    // odd block: dwords 9..16
    int bh = dot4(r.c.y, h2.y, 0); bh = dot4(r.c.z, h2.z, bh); bh = dot4(r.c.w, h2.w, bh);
    bh = dot4(r.d.x, h3.x, bh); bh = dot4(r.d.y, h3.y, bh); bh = dot4(r.d.z, h3.z, bh); bh = dot4(r.d.w, h3.w, bh);
    bh = dot4(r.e, h4.x, bh);
    int bl = dot4(r.c.y, l2.y, 0); bl = dot4(r.c.z, l2.z, bl); bl = dot4(r.c.w, l2.w, bl);
    bl = dot4(r.d.x, l3.x, bl); bl = dot4(r.d.y, l3.y, bl); bl = dot4(r.d.z, l3.z, bl); bl = dot4(r.d.w, l3.w, bl);
    bl = dot4(r.e, l4.x, bl);
    const float da = f16_bits_to_float(r.a.x & 0xffffu);
    const float db = f16_bits_to_float(r.c.x >> 16);
    const float2 s = *reinterpret_cast<const float2*>(xs + 2 * pair);
    return da * s.x * (static_cast<float>(ah) + static_cast<float>(al) * kLoInv) +
           db * s.y * (static_cast<float>(bh) + static_cast<float>(bl) * kLoInv);
}

// TL = 1 << tl_log2 lanes share a row (4..64); a wave covers 64 / TL rows per pass.
template <int ITERS>
__global__ __launch_bounds__(kThreads) void q8_0_pair_kernel(
    const unsigned char* __restrict__ image, size_t image_stride, const uint8_t* __restrict__ w,
    void* __restrict__ y, int y_dtype, int n, int pairs, int tl_log2) {
    extern __shared__ __align__(16) unsigned char smem[];
    const unsigned char* img_hi = smem;
    const unsigned char* img_lo = smem + static_cast<size_t>(pairs) * 80;
    const float* xs = reinterpret_cast<const float*>(smem + static_cast<size_t>(pairs) * 160);
    const int tl = 1 << tl_log2;
    const int tid = threadIdx.x;
    const int rows_per_wg = kThreads >> tl_log2;
    const int row = blockIdx.x * rows_per_wg + (tid >> tl_log2);
    const int slot = tid & (tl - 1);
    const bool row_ok = row < n;
    const uint8_t* wrow = w + static_cast<size_t>(row_ok ? row : 0) * pairs * 68;

    float acc = 0.0f;
    bool staged = false;
    for (int p0 = slot; p0 < pairs || !staged; p0 += tl * ITERS) {
        PairRegs regs[ITERS];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int p = p0 + it * tl;
            if (row_ok && p < pairs) load_pair(regs[it], wrow + static_cast<size_t>(p) * 68);
            else zero_pair(regs[it]);
        }
        if (!staged) {
            copy_to_lds(smem, image + static_cast<size_t>(blockIdx.y) * image_stride, (pairs * 168 + 15) & ~15);
            __syncthreads();
            staged = true;
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int p = p0 + it * tl;
            if (row_ok && p < pairs) acc += pair_dot(regs[it], p, img_hi, img_lo, xs);
        }
    }
    for (int off = 1; off < tl; off <<= 1) acc += __shfl_xor(acc, off, 64);
    if (row_ok && slot == 0) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + row, acc);
}

// ------------------------------------------------------------------------------------------------
// Streamed form (rows of a multiple of four pairs, 16-byte aligned matrix): one launch per operator call.
//
// The matrix is one contiguous run of 68-byte pairs.  One workgroup of 16 waves per compute unit owns a
// contiguous range of whole rows and walks it in steps of 64 pairs = 4352 contiguous bytes, wave v taking
// steps v, v + 16, ...  A step is loaded the way a stream is read: lane l takes 16 bytes at
// 1024 i + 16 l (five fully coalesced wave instructions, the fifth covering the last 256 bytes four
// lanes to an address), two steps ahead in registers (more waves beat deeper sets: 12 waves x 3 steps and 8 x 4 ran 1 - 2 us slower).  The wave then turns the step by way of an LDS
// buffer of its own (no barrier: written and read by the same wave) so that lane l holds pair l (17
// dwords at 68 l: neighbouring lanes 17 banks apart) and multiplies it as the kernel above does.  A
// step may hold the end of one row and the start of the next: lanes are told apart by row, each row's
// part is reduced over the wave into partial[step][row - first row of the step], and after one barrier
// a thread per row adds the row's parts in step order (deterministic) and stores.
// The workgroup quantizes the activation row itself into the pair image, once per compute unit, from
// loads requested ahead of the first weights.
// ------------------------------------------------------------------------------------------------
constexpr int kStepBytes = 64 * 68;                            // 4352 = 4 x 1024 + 256
constexpr int kStreamWaves = 16;
constexpr int kStreamThreads = 64 * kStreamWaves;
constexpr int kStreamDepth = 2;                                // steps a wave holds in registers (sixteen waves fit 128 registers each)
constexpr int kXBatch = 2;                                     // pieces of the activation row a thread requests ahead of the weights

typedef uint32_t v2u __attribute__((ext_vector_type(2)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));                   // (a native vector: moves of HIP's uint4 struct between address spaces compile to memcpy calls that keep the sets in memory)

__device__ __forceinline__ const uint8_t* not_past(const uint8_t* p, const uint8_t* last16) { return p < last16 ? p : last16; }

__global__ __launch_bounds__(kStreamThreads) void q8_0_stream_kernel(
    const void* __restrict__ x, int x_dtype, const uint8_t* __restrict__ w, void* __restrict__ y, int y_dtype,
    int k, int n, int pairs, uint32_t pairs_magic, int image_bytes, int cols, int rows_each, int rows_left) {
    asm volatile("" : : "s"(x), "s"(x_dtype), "s"(w), "s"(y), "s"(y_dtype), "s"(k), "s"(n), "s"(pairs), "s"(pairs_magic), "s"(image_bytes), "s"(cols),
                 "s"(rows_each), "s"(rows_left));   // the arguments in one batch of scalar loads, one wait
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char* img_hi = smem;
    unsigned char* img_lo = smem + static_cast<size_t>(pairs) * 80;
    float* xs = reinterpret_cast<float*>(smem + static_cast<size_t>(pairs) * 160);
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    unsigned char* turn = smem + image_bytes + wave * kStepBytes;              // this wave's buffer
    float* partial = reinterpret_cast<float*>(smem + image_bytes + kStreamWaves * kStepBytes);   // [step][cols]

    // this workgroup's rows [r0, r1): an even share of the matrix, rows_each = n / grid with one row more for the first
    // rows_left = n % grid workgroups (quotient and remainder come from the host: a 64-bit division here is ~150 dependent
    // instructions, twice, ahead of the kernel's first memory request)
    const int bx = static_cast<int>(blockIdx.x);
    const int r0 = bx * rows_each + min(bx, rows_left);
    const int r1 = r0 + rows_each + (bx < rows_left ? 1 : 0);
    const int count = (r1 - r0) * pairs;
    const int steps = (count + 63) >> 6;
    const uint8_t* base = w + static_cast<size_t>(r0) * pairs * 68;
    const uint8_t* last16 = w + static_cast<size_t>(n) * pairs * 68 - 16;      // loads past the matrix are bent back to here (their lanes are not used)

    // the first pieces of the activation row, requested ahead of the weights (loads return in order) and left as loaded until the
    // weights have been requested too: telling the value types apart before that would wait for the pieces inside each branch
    const size_t xoff = static_cast<size_t>(blockIdx.y) * k;
    constexpr int trip = kStreamThreads * 4;
    v4u raw[kXBatch];
    if (x_dtype == PLLM_F32) {
#pragma unroll
        for (int j = 0; j < kXBatch; ++j)
            raw[j] = *reinterpret_cast<const v4u*>(static_cast<const float*>(x) + xoff + (tid * 4 + j * trip < k ? tid * 4 + j * trip : 0));
    } else {
#pragma unroll
        for (int j = 0; j < kXBatch; ++j) {
            const v2u t = *reinterpret_cast<const v2u*>(static_cast<const uint16_t*>(x) + xoff + (tid * 4 + j * trip < k ? tid * 4 + j * trip : 0));
            raw[j] = v4u{t.x, t.y, 0u, 0u};
        }
    }

    // step s of the workgroup (past its last step: that one again), always five loads
    auto fetch = [&](v4u (&r)[5], int s) __attribute__((always_inline)) {
        const uint8_t* src = base + static_cast<size_t>(min(s, max(steps - 1, 0))) * kStepBytes;
        r[0] = *reinterpret_cast<const v4u*>(not_past(src + lane * 16, last16));
        r[1] = *reinterpret_cast<const v4u*>(not_past(src + 1024 + lane * 16, last16));
        r[2] = *reinterpret_cast<const v4u*>(not_past(src + 2048 + lane * 16, last16));
        r[3] = *reinterpret_cast<const v4u*>(not_past(src + 3072 + lane * 16, last16));
        r[4] = *reinterpret_cast<const v4u*>(not_past(src + 4096 + (lane & 15) * 16, last16));
    };
    v4u regs[kStreamDepth][5];
#pragma unroll
    for (int j = 0; j < kStreamDepth; ++j) fetch(regs[j], wave + j * kStreamWaves);

    float head[kXBatch][4];
    if (x_dtype == PLLM_F32) {
#pragma unroll
        for (int j = 0; j < kXBatch; ++j) {
            head[j][0] = __uint_as_float(raw[j].x); head[j][1] = __uint_as_float(raw[j].y);
            head[j][2] = __uint_as_float(raw[j].z); head[j][3] = __uint_as_float(raw[j].w);
        }
    } else if (x_dtype == PLLM_BF16) {
#pragma unroll
        for (int j = 0; j < kXBatch; ++j) {
            head[j][0] = __uint_as_float(raw[j].x << 16); head[j][1] = __uint_as_float(raw[j].x & 0xffff0000u);
            head[j][2] = __uint_as_float(raw[j].y << 16); head[j][3] = __uint_as_float(raw[j].y & 0xffff0000u);
        }
    } else {
#pragma unroll
        for (int j = 0; j < kXBatch; ++j) {
            head[j][0] = f16_bits_to_float(raw[j].x & 0xffffu); head[j][1] = f16_bits_to_float(raw[j].x >> 16);
            head[j][2] = f16_bits_to_float(raw[j].y & 0xffffu); head[j][3] = f16_bits_to_float(raw[j].y >> 16);
        }
    }
#pragma unroll
    for (int j = 0; j < kXBatch; ++j)
        if (tid * 4 + j * trip < k) quantize4_to_pair_image(head[j], tid * 4 + j * trip, img_hi, img_lo, xs);
    for (int b0 = tid * 4 + kXBatch * trip; b0 < k; b0 += trip) {              // rows longer than one batch
        float v[4];
        load_row4(v, x, x_dtype, xoff, b0, k, true);
        quantize4_to_pair_image(v, b0, img_hi, img_lo, xs);
    }
    __syncthreads();

    // step s from the register set r, which then takes step s + kStreamDepth * kStreamWaves
    auto step = [&](v4u (&r)[5], int s) __attribute__((always_inline)) {
        // turn the step: 16-byte pieces in stream order -> LDS -> this lane's pair
        *reinterpret_cast<v4u*>(turn + lane * 16) = r[0];
        *reinterpret_cast<v4u*>(turn + 1024 + lane * 16) = r[1];
        *reinterpret_cast<v4u*>(turn + 2048 + lane * 16) = r[2];
        *reinterpret_cast<v4u*>(turn + 3072 + lane * 16) = r[3];
        if (lane < 16) *reinterpret_cast<v4u*>(turn + 4096 + lane * 16) = r[4];
        fetch(r, s + kStreamDepth * kStreamWaves);
        if (s >= steps) return;                                                // wave-uniform
        const int pidx = 64 * s + lane;
        const int rowi = static_cast<int>(__umulhi(static_cast<uint32_t>(pidx), pairs_magic));   // row within the workgroup's range
        const int p = pidx - rowi * pairs;
        const uint32_t* q = reinterpret_cast<const uint32_t*>(turn + 68 * lane);
        PairRegs pr;
        pr.a = make_uint4(q[0], q[1], q[2], q[3]);
        pr.b = make_uint4(q[4], q[5], q[6], q[7]);
        pr.c = make_uint4(q[8], q[9], q[10], q[11]);
        pr.d = make_uint4(q[12], q[13], q[14], q[15]);
        pr.e = q[16];
        const float d = pair_dot(pr, p, img_hi, img_lo, xs);
        const float val = pidx < count ? d : 0.0f;
        const int first = static_cast<int>(__umulhi(static_cast<uint32_t>(64 * s), pairs_magic));
        const int last = static_cast<int>(__umulhi(static_cast<uint32_t>(min(64 * s + 63, count - 1)), pairs_magic));
        for (int rr = first; rr <= last; ++rr) {                               // wave-uniform
            const float total = group_sum<64>(rowi == rr ? val : 0.0f);
            if (lane == 0) partial[s * cols + rr - first] = total;
        }
    };
    for (int s = wave; s < steps; s += kStreamDepth * kStreamWaves) {
#pragma unroll
        for (int j = 0; j < kStreamDepth; ++j) step(regs[j], s + j * kStreamWaves);
    }
    __syncthreads();
    for (int i = tid; i < r1 - r0; i += kStreamThreads) {
        const int s_first = (i * pairs) >> 6, s_last = ((i + 1) * pairs - 1) >> 6;
        float total = 0.0f;
        for (int s = s_first; s <= s_last; ++s)
            total += partial[s * cols + i - static_cast<int>(__umulhi(static_cast<uint32_t>(64 * s), pairs_magic))];
        store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + r0 + i, total);
    }
}

struct StreamPlan { int grid_x; int cols; int image_bytes; size_t smem; };

// false when the streamed form does not apply
bool plan_stream(const void* x, int x_dtype, const uint8_t* w, int k, int n, int bpr, StreamPlan& plan) {
    if (bpr % 8 != 0 || k != bpr * 32 || (reinterpret_cast<uintptr_t>(w) & 15u)) return false;
    if (reinterpret_cast<uintptr_t>(x) & (x_dtype == PLLM_F32 ? 15u : 7u)) return false;   // rows are read in vector pieces
    const int pairs = bpr / 2;
    const long long total_steps = (static_cast<long long>(n) * pairs + 63) / 64;
    plan.grid_x = static_cast<int>(std::max<long long>(1, std::min<long long>(compute_units(), (total_steps + kStreamWaves - 1) / kStreamWaves)));
    const long long rows_per_wg = (n + plan.grid_x - 1) / plan.grid_x;
    const long long steps = (rows_per_wg * pairs + 63) / 64;
    // the row index of a pair comes from a multiplication by a rounded-up reciprocal: exact while (pair index) x pairs < 2^32
    if ((steps * 64 + 64) * pairs >= (1ll << 32)) return false;
    plan.cols = (62 + pairs) / pairs + 1;                                      // rows that 64 consecutive pairs can touch
    plan.image_bytes = (pairs * 168 + 15) & ~15;
    plan.smem = static_cast<size_t>(plan.image_bytes) + static_cast<size_t>(kStreamWaves) * kStepBytes + static_cast<size_t>(steps) * plan.cols * sizeof(float);
    return plan.smem <= 160 * 1024;
}

int launch_stream(const void* x, int x_dtype, const uint8_t* w, void* y, int y_dtype, int rows, int k, int n, int pairs, const StreamPlan& plan,
                  hipStream_t stream) {
    auto kern = q8_0_stream_kernel;
    static SmemGrant granted;
    if (!grant_dynamic_smem(reinterpret_cast<const void*>(kern), plan.smem, granted)) return PLLM_ERR_UNSUPPORTED;
    const uint32_t magic = static_cast<uint32_t>(((1ull << 32) + pairs - 1) / pairs);
    hipLaunchKernelGGL(kern, dim3(plan.grid_x, rows), dim3(kStreamThreads), plan.smem, stream, x, x_dtype, w, y, y_dtype, k, n, pairs, magic,
                       plan.image_bytes, plan.cols, n / plan.grid_x, n % plan.grid_x);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

// Any shape, any alignment: one wave per output row, one lane per block, byte loads.  Used when a
// row holds an odd number of blocks or the base pointer is not dword aligned.
__global__ __launch_bounds__(kThreads) void q8_0_generic_kernel(
    const void* __restrict__ x, int x_dtype, const uint8_t* __restrict__ w, void* __restrict__ y, int y_dtype,
    int k, int n, int bpr) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * kWaves + (threadIdx.x >> 6);
    const size_t xoff = static_cast<size_t>(blockIdx.y) * k;
    float acc = 0.0f;
    if (row < n) {
        const uint8_t* wrow = w + static_cast<size_t>(row) * bpr * 34;
        for (int b = lane; b < bpr; b += 64) {
            const uint8_t* blk = wrow + 34 * b;
            const float d = f16_bits_to_float(static_cast<uint32_t>(blk[0]) | (static_cast<uint32_t>(blk[1]) << 8));
            float s = 0.0f;
            for (int i = 0; i < 32; ++i) {
                const int e = 32 * b + i;
                if (e < k) s += load_any(x, x_dtype, xoff + e) * static_cast<float>(static_cast<int8_t>(blk[2 + i]));
            }
            acc += d * s;
        }
    }
    acc = group_sum<64>(acc);
    if (lane == 0 && row < n) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + row, acc);
}

template <int ITERS>
int launch_pair(const unsigned char* image, size_t image_stride, const uint8_t* w, void* y, int y_dtype, int rows, int n,
                int pairs, int tl_log2, hipStream_t stream) {
    const size_t smem = (static_cast<size_t>(pairs) * 168 + 15) & ~static_cast<size_t>(15);
    auto kern = q8_0_pair_kernel<ITERS>;
    if (smem > 64 * 1024) {
        if (smem > 160 * 1024) return PLLM_ERR_UNSUPPORTED;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(smem)) != hipSuccess)
            return PLLM_ERR_UNSUPPORTED;
    }
    const int rows_per_wg = kThreads >> tl_log2;
    dim3 grid((n + rows_per_wg - 1) / rows_per_wg, rows);
    hipLaunchKernelGGL(kern, grid, dim3(kThreads), smem, stream, image, image_stride, w, y, y_dtype, n, pairs, tl_log2);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

}  // namespace

size_t q8_0_matvec_workspace_bytes(int rows, int bpr) {
    return (bpr % 2 == 0) ? act_image_q8pair_bytes(bpr / 2) * static_cast<size_t>(rows) : 0;
}

int q8_0_matvec(const void* x, int x_dtype, const uint8_t* w, void* y, int y_dtype,
                int rows, int k, int n, int bpr, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    StreamPlan plan;
    if (plan_stream(x, x_dtype, w, k, n, bpr, plan)) return launch_stream(x, x_dtype, w, y, y_dtype, rows, k, n, bpr / 2, plan, stream);
    const bool pair_ok = (bpr % 2 == 0) && ((reinterpret_cast<uintptr_t>(w) & 3u) == 0);
    if (!pair_ok) {
        dim3 grid((n + kWaves - 1) / kWaves, rows);
        hipLaunchKernelGGL(q8_0_generic_kernel, grid, dim3(kThreads), 0, stream, x, x_dtype, w, y, y_dtype, k, n, bpr);
        return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
    }
    if (!workspace || workspace_bytes < q8_0_matvec_workspace_bytes(rows, bpr)) return PLLM_ERR_WORKSPACE;
    const int pairs = bpr / 2;
    const int st = act_image_q8pair(x, x_dtype, rows, k, pairs, workspace, stream);
    if (st != PLLM_OK) return st;
    // lanes per row: leave every lane about four pairs
    int tl_log2 = 2;
    while (tl_log2 < 6 && (pairs >> (tl_log2 + 1)) >= 4) ++tl_log2;
    const int tl = 1 << tl_log2;
    const int niter = (pairs + tl - 1) / tl;
    const int passes = (niter + 5) / 6;
    const int iters = (niter + passes - 1) / passes;
    const unsigned char* image = static_cast<const unsigned char*>(workspace);
    const size_t stride = act_image_q8pair_bytes(pairs);
#define PLLM_CASE(I) return launch_pair<I>(image, stride, w, y, y_dtype, rows, n, pairs, tl_log2, stream)
    switch (iters) {
        case 1: PLLM_CASE(1);
        case 2: PLLM_CASE(2);
        case 3: PLLM_CASE(3);
        case 4: PLLM_CASE(4);
        case 5: PLLM_CASE(5);
        default: PLLM_CASE(6);
    }
#undef PLLM_CASE
}

}  // namespace pllm
