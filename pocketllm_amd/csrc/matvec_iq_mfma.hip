// Decode matvec over raw IQ2_XXS / IQ1_M super-blocks with the integer dots on the matrix cores.
//
// Same frame as the Q4_K / Q5_K kernel: a wave owns 16 consecutive output rows, the W waves of a
// workgroup split a row's super-blocks between them and meet in a small LDS reduction, the
// activation image (two int8 terms per value) sits in LDS.  For one super-block index the wave forms
//     C[m][n] = sum_k A[m][k] * B[k][n],     v_mfma_i32_16x16x64_i8, four of them per block,
// with n = output row and m = 2 * group + term (group = 32 weights, term = high / low int8 term of
// the activations).  Lane (n, s) supplies B for the 16-weight slice s of each MFMA; here MFMA t and
// slice s carry half t % 2 of group 2 s + t / 2, so a lane decodes exactly the two groups (64
// weights, one 16-byte piece of the block) whose results it later finds in its own C registers:
// C[4 s .. 4 s + 3][n] = groups 2 s and 2 s + 1, both terms.
//
// The codebook lookups happen once per weight and feed 16 rows x 2 terms of dots each, where the
// v_dot4 form repeats the activation reads and the dots per lane.
#include "block_dot4.h"
#include "pllm_internal.h"

namespace pllm {
namespace {

constexpr int kRowsPerWg = 16;
constexpr int kMaxWaves = 8;

typedef int v4i __attribute__((ext_vector_type(4)));

__device__ __forceinline__ v4i as_v4i(uint32_t x, uint32_t y, uint32_t z, uint32_t w) {
    v4i r;
    r.x = static_cast<int>(x); r.y = static_cast<int>(y); r.z = static_cast<int>(z); r.w = static_cast<int>(w);
    return r;
}

// A operands of one block for this lane: a_off[t] + block * a_step[t] (zeros where the lane's A row
// does not belong to MFMA t's group)
struct AMap { int off[4]; int step[4]; };

// ------------------------------------------------------------------------------------------------
// IQ2_XXS: 66 B = d(2) + 8 sub-blocks of 8 B (four grid ids, then a u32: four 7-bit sign indices and
// a 4-bit scale).  Lane (n, s) holds sub-blocks 2 s and 2 s + 1.  LDS tables as in the v_dot4 form:
// 256 x 8 magnitude bytes, 128 x 8 sign masks; signed codes = (g ^ m) + (m & 0x01010101).
// ------------------------------------------------------------------------------------------------
struct IQ2XXSm {
    static constexpr int kBlockBytes = 66;
    static constexpr int kTableBytes = IQ2XXS::kTableBytes;
    struct Regs { uint4 q; uint32_t d; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int s) {
        r.q = load16_a2(blk + 2 + 16 * s);
        r.d = *reinterpret_cast<const uint16_t*>(blk);
    }
    static __device__ __forceinline__ void stage_tables(unsigned char* lds) { IQ2XXS::stage_tables(lds); }
    static __device__ __forceinline__ uint2 signed8(const uint2* grid, const uint2* sign, uint32_t id, uint32_t s7) {
        const uint2 g = grid[id], m = sign[s7];
        return make_uint2((g.x ^ m.x) + (m.x & 0x01010101u), (g.y ^ m.y) + (m.y & 0x01010101u));
    }
    static __device__ __forceinline__ float block(const Regs& r, int s, int b, const unsigned char* smem, const AMap& am, const StagedX& sx,
                                                  const unsigned char* tables) {
        const uint2* grid = reinterpret_cast<const uint2*>(tables);
        const uint2* sign = grid + 256;
        v4i c = {0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t ids = (t < 2) ? r.q.x : r.q.z, aux = (t < 2) ? r.q.y : r.q.w;
            const int e = 2 * (t & 1);                                         // grid entries e and e + 1 of the sub-block
            const uint2 w0 = signed8(grid, sign, (ids >> (8 * e)) & 0xffu, (aux >> (7 * e)) & 127u);
            const uint2 w1 = signed8(grid, sign, (ids >> (8 * e + 8)) & 0xffu, (aux >> (7 * e + 7)) & 127u);
            const uint4 a = *reinterpret_cast<const uint4*>(smem + am.off[t] + b * am.step[t]);
            c = __builtin_amdgcn_mfma_i32_16x16x64_i8(as_v4i(a.x, a.y, a.z, a.w), as_v4i(w0.x, w0.y, w1.x, w1.y), c, 0, 0, 0);
        }
        const float v0 = static_cast<float>(__mul24(c.x, 254) + c.y);         // group 2 s: 254 * high term + low term
        const float v1 = static_cast<float>(__mul24(c.z, 254) + c.w);         // group 2 s + 1
        const float4 g2 = *reinterpret_cast<const float4*>(sx.gs + b * 8 + 2 * s);   // {xs0 / 254, sum0, xs1 / 254, sum1}
        const float ls0 = static_cast<float>(2 * (r.q.y >> 28) + 1), ls1 = static_cast<float>(2 * (r.q.w >> 28) + 1);
        return 0.125f * f16_bits_to_float(r.d) * (ls0 * g2.x * v0 + ls1 * g2.z * v1);
    }
};

// ------------------------------------------------------------------------------------------------
// IQ1_M: 56 B = qs(32) qh(16) scales(8); w = dl (c - 1 + delta) with c in {0, 1, 2} from the
// codebook, dl = d (2 s3 + 1) per 16 weights, delta = -+1/8 per 8 weights.  Lane (n, s) holds
// entries 8 s .. 8 s + 7.  The 16-weight scale ls = 2 s3 + 1 is folded into the codes (a byte
// permute picks 0, ls or 2 ls <= 30 for every code), so
//     sum w x = d [ dot(c ls, x) - sum_16 ls sum16(x) + sum_8 (+-ls / 8) sum8(x) ]:
// the first term is the MFMA above, the second uses the image's exact 16-value sums, and the third
// is a second set of four MFMAs whose B bytes are +-ls, constant over each entry.
// LDS table: 2048 x u32 of eight nibbles, nibble 2 i = element i, nibble 2 i + 1 = element 4 + i.
// ------------------------------------------------------------------------------------------------
struct IQ1Mm {
    static constexpr int kBlockBytes = 56;
    static constexpr int kTableBytes = IQ1M::kTableBytes;
    struct Regs { uint2 qs; uint32_t qh; uint2 sc; };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* blk, int s) {
        r.qs = *reinterpret_cast<const uint2*>(blk + 8 * s);                   // blocks are 8-byte aligned
        r.qh = *reinterpret_cast<const uint32_t*>(blk + 32 + 4 * s);
        r.sc = *reinterpret_cast<const uint2*>(blk + 48);
    }
    static __device__ __forceinline__ void stage_tables(unsigned char* lds) { IQ1M::stage_tables(lds); }
    static __device__ __forceinline__ float block(const Regs& r, int s, int b, const unsigned char* smem, const AMap& am, const StagedX& sx,
                                                  const unsigned char* tables) {
        const uint32_t* table = reinterpret_cast<const uint32_t*>(tables);
        const uint32_t s01 = r.sc.x, s23 = r.sc.y;
        const uint32_t dbits = ((s01 >> 12) & 0xfu) | ((s01 >> 24) & 0xf0u) | ((s23 >> 4) & 0xf00u) | ((s23 >> 16) & 0xf000u);
        // the lane's four 16-weight scales are the low 12 bits of scale word s
        const uint32_t word = ((s & 2) ? s23 : s01) >> (16 * (s & 1));
        v4i c = {0, 0, 0, 0}, cd = {0, 0, 0, 0};
        float minus = 0.0f;
        const float4 s16 = *reinterpret_cast<const float4*>(sx.sum16 + b * 16 + 4 * s);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t ls = 2 * ((word >> (3 * t)) & 7u) + 1;             // 16-weight group t of the lane = entries 2 t, 2 t + 1
            const uint32_t qw = (t < 2) ? r.qs.x : r.qs.y;
            const uint32_t h0 = (r.qh >> (8 * t)) & 15u, h1 = (r.qh >> (8 * t + 4)) & 15u;
            const uint32_t p0 = table[((qw >> (16 * (t & 1))) & 0xffu) | ((h0 & 7u) << 8)];
            const uint32_t p1 = table[((qw >> (16 * (t & 1) + 8)) & 0xffu) | ((h1 & 7u) << 8)];
            // bytes c in {0, 1, 2} pick byte c of {0, ls, 2 ls}
            const uint32_t lut = ls * 0x020100u;
            const v4i bw = as_v4i(__builtin_amdgcn_perm(0u, lut, p0 & 0x0f0f0f0fu), __builtin_amdgcn_perm(0u, lut, (p0 >> 4) & 0x0f0f0f0fu),
                                  __builtin_amdgcn_perm(0u, lut, p1 & 0x0f0f0f0fu), __builtin_amdgcn_perm(0u, lut, (p1 >> 4) & 0x0f0f0f0fu));
            // +-ls in every byte of the entry: delta = -1/8 where bit 3 of the qh nibble is set
            const uint32_t pos = ls * 0x01010101u, neg = (256u - ls) * 0x01010101u;
            const uint32_t d0 = (h0 & 8u) ? neg : pos, d1 = (h1 & 8u) ? neg : pos;
            const uint4 a = *reinterpret_cast<const uint4*>(smem + am.off[t] + b * am.step[t]);
            const v4i av = as_v4i(a.x, a.y, a.z, a.w);
            c = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bw, c, 0, 0, 0);
            cd = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, as_v4i(d0, d0, d1, d1), cd, 0, 0, 0);
            const float sum = (t == 0) ? s16.x : (t == 1) ? s16.y : (t == 2) ? s16.z : s16.w;
            minus += static_cast<float>(ls) * sum;
        }
        const float4 g2 = *reinterpret_cast<const float4*>(sx.gs + b * 8 + 2 * s);   // {xs0 / 254, sum0, xs1 / 254, sum1}
        const float v0 = static_cast<float>(__mul24(c.x, 254) + c.y) + 0.125f * static_cast<float>(__mul24(cd.x, 254) + cd.y);
        const float v1 = static_cast<float>(__mul24(c.z, 254) + c.w) + 0.125f * static_cast<float>(__mul24(cd.z, 254) + cd.w);
        return f16_bits_to_float(dbits) * (g2.x * v0 + g2.z * v1 - minus);
    }
};

template <typename FMT, int ITERS>
__global__ __launch_bounds__(64 * kMaxWaves) void iq_mfma_matvec_kernel(
    const unsigned char* __restrict__ image, size_t image_stride, const uint8_t* __restrict__ w,
    void* __restrict__ y, int y_dtype, int n, int bpr) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int kpad = bpr * 256;
    const int image_bytes = static_cast<int>(staged_x_bytes(kpad));
    const StagedX sx = carve_staged_x(smem, kpad);
    const int zero_off = image_bytes;                                        // 16 zero bytes
    unsigned char* tables = smem + image_bytes + 16;
    float* partial = reinterpret_cast<float*>(tables + FMT::kTableBytes);   // [waves][16]

    const int tid = threadIdx.x;
    const int waves = blockDim.x >> 6;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int col = lane & 15;        // B/C column = output row within the tile; also A's row index m
    const int ks = lane >> 4;         // k slice of A and B, row quad of C
    const int row = blockIdx.x * kRowsPerWg + col;
    const uint8_t* wrow = w + static_cast<size_t>(row < n ? row : 0) * bpr * FMT::kBlockBytes;

    // A side: this lane supplies row m = col = 2 * group + term of MFMA t, slice ks; it is non-zero
    // only when MFMA t's slice ks belongs to `group`: G(t, ks) = 2 * ks + t / 2, half t % 2
    AMap am;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int g = 2 * ks + (t >> 1);
        const bool active = (col >> 1) == g;
        am.off[t] = active ? ((col & 1) ? kpad : 0) + 32 * g + 16 * (t & 1) : zero_off;
        am.step[t] = active ? 256 : 0;
    }

    float acc = 0.0f;
    bool staged = false;
    for (int b0 = wave; b0 < bpr || !staged; b0 += waves * ITERS) {
        typename FMT::Regs regs[ITERS];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int b = min(b0 + it * waves, bpr - 1);                    // clamped: always a valid address
            FMT::load(regs[it], wrow + static_cast<size_t>(b) * FMT::kBlockBytes, ks);
        }
        if (!staged) {                       // first trip of every thread of the workgroup
            copy_to_lds(smem, image + static_cast<size_t>(blockIdx.y) * image_stride, image_bytes);
            if (tid < 4) reinterpret_cast<uint32_t*>(smem + zero_off)[tid] = 0;
            FMT::stage_tables(tables);
            __syncthreads();
            staged = true;
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int b = b0 + it * waves;
            if (b < bpr) acc += FMT::block(regs[it], ks, b, smem, am, sx, tables);   // wave-uniform guard
        }
    }
    acc += __shfl_xor(acc, 16, 64);
    acc += __shfl_xor(acc, 32, 64);
    if (ks == 0) partial[wave * kRowsPerWg + col] = acc;
    __syncthreads();
    if (tid < kRowsPerWg) {
        float total = 0.0f;
        for (int v = 0; v < waves; ++v) total += partial[v * kRowsPerWg + tid];
        const int out_row = blockIdx.x * kRowsPerWg + tid;
        if (out_row < n) store_any(y, y_dtype, static_cast<size_t>(blockIdx.y) * n + out_row, total);
    }
}

template <typename FMT, int ITERS>
int launch_one(const unsigned char* image, size_t image_stride, const uint8_t* w, void* y, int y_dtype,
               int rows, int n, int bpr, int waves, hipStream_t stream) {
    const size_t smem = staged_x_bytes(bpr * 256) + 16 + FMT::kTableBytes + static_cast<size_t>(waves) * kRowsPerWg * sizeof(float);
    auto kern = iq_mfma_matvec_kernel<FMT, ITERS>;
    if (smem > 64 * 1024) {
        if (smem > 160 * 1024) return PLLM_ERR_UNSUPPORTED;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(smem)) != hipSuccess)
            return PLLM_ERR_UNSUPPORTED;
    }
    dim3 grid((n + kRowsPerWg - 1) / kRowsPerWg, rows);
    hipLaunchKernelGGL(kern, grid, dim3(64 * waves), smem, stream, image, image_stride, w, y, y_dtype, n, bpr);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

template <typename FMT>
int launch_fmt(const unsigned char* image, size_t image_stride, const uint8_t* w, void* y, int y_dtype,
               int rows, int n, int bpr, hipStream_t stream) {
    // waves per workgroup: split a row's blocks so that every wave keeps a handful in flight
    int waves = 1;
    while (waves < kMaxWaves && bpr / (waves * 2) >= 3) waves *= 2;
    const int niter = (bpr + waves - 1) / waves;
    const int passes = (niter + 5) / 6;
    const int iters = (niter + passes - 1) / passes;
#define PLLM_CASE(I) case I: return launch_one<FMT, I>(image, image_stride, w, y, y_dtype, rows, n, bpr, waves, stream)
    switch (iters) {
        PLLM_CASE(1); PLLM_CASE(2); PLLM_CASE(3); PLLM_CASE(4); PLLM_CASE(5);
        default: return launch_one<FMT, 6>(image, image_stride, w, y, y_dtype, rows, n, bpr, waves, stream);
    }
#undef PLLM_CASE
}

}  // namespace

int iq_mfma_matvec_from_image(const unsigned char* image, size_t stride, const uint8_t* w, int type_id, void* y, int y_dtype,
                              int rows, int n, int bpr, hipStream_t stream) {
    switch (type_id) {
        case PLLM_TYPE_IQ2_XXS: return launch_fmt<IQ2XXSm>(image, stride, w, y, y_dtype, rows, n, bpr, stream);
        case PLLM_TYPE_IQ1_M: return launch_fmt<IQ1Mm>(image, stride, w, y, y_dtype, rows, n, bpr, stream);
        default: return PLLM_ERR_UNSUPPORTED;
    }
}

}  // namespace pllm
