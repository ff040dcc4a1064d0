// Prefill matmul of Q4_K / Q5_K weights on the int8 matrix cores, activations quantized to 32-value int8 blocks: the
// semantics of the reference's MMA prefill path (src/csrc/llama_mmq/gguf_mma_wrapper.cu:257-322, the per-group sums of
// mmq.cuh:1374-1378; activation quantizer src/csrc/cuda_kernel_impl.cu:7090-7117):
//     y[t, n] = sum over 32-weight groups g of  xs[t, g] * ( d_n sc_{n,g} * sum_i q_{n,g,i} xq_{t,g,i}  -  dmin_n m_{n,g} * sum_i xq_{t,g,i} )
// with xq = rint(x / xs), xs = amax / 127 per (token, group); d * sc and dmin * m stay float32 (the reference rounds them to fp16).
//
// Two launches.  q8_rows_kernel writes the activation codes int8 [T, kpad] and per (token, group) the pair {xs, xs * sum of codes}.
// gemm_i8_kernel: workgroup tile 128 tokens x 128 rows, four waves as 2 x 2, wave tile 64 x 64 = 2 x 2 accumulator tiles of
// v_mfma_i32_32x32x32_i8, whose K = 32 is exactly one group, so every MFMA result is a pure group dot and takes its two float
// scales in the epilogue: acc += (float(C) * xs_t) * (d sc)_n - (xs S)_t * (dmin m)_n.  The B operand comes straight out of the
// weight bytes: lane (n, half) loads qs[32 p + 16 half, +16) of its row, whose low nibbles are codes [16 half, +16) of group 2p
// and whose high nibbles are the same codes of group 2p + 1 - the K slice that lane owes both MFMAs (Q5_K adds bit 2p / 2p + 1 of
// qh[16 half, +16)).  The A operand (activation codes of the 128 tokens for the two groups of a step) is staged in LDS, rows
// padded to 80 bytes, double buffered; the weight loads of the next step are issued before the current step's matrix work.
// Bound: the float epilogue (4 vector instructions per accumulator element and group against a 16-pass MFMA), not the matrix core.
#include "pllm_device.h"
#include "pllm_internal.h"

namespace pllm {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kBM = 128, kBN = 128, kThreads = 256;
constexpr int kARow = 80;                                    // bytes per token row of a staged step: 64 codes + padding against bank conflicts

__device__ __forceinline__ int group_sum8_int(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, true);      // quad_perm [1,0,3,2]
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, true);      // quad_perm [2,3,0,1]
    v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, true);     // row_half_mirror
    return v;
}

// codes int8 [rows, kpad] (zeros from k on), scales float2 [rows, kpad / 32] = {xs, xs * sum of the group's codes}
__global__ __launch_bounds__(256) void q8_rows_kernel(const void* __restrict__ x, int x_dtype, int8_t* __restrict__ xq, float2* __restrict__ xsc,
                                                      int k, int kpad) {
    const int e0 = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (e0 >= kpad) return;                                   // kpad is a multiple of 256: whole groups leave together
    const size_t row = blockIdx.y;
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = (e0 + i < k) ? load_any(x, x_dtype, row * k + e0 + i) : 0.0f;
    uint32_t hi, lo;
    float scale;
    quantize4(v, hi, lo, scale);
    *reinterpret_cast<uint32_t*>(xq + row * kpad + e0) = hi;
    const int s = group_sum8_int(dot4(hi, 0x01010101u, 0));
    if ((threadIdx.x & 7) == 0) xsc[row * (kpad / 32) + (e0 >> 5)] = make_float2(scale, scale * static_cast<float>(s));
}

struct K4Packed { uint32_t sc_lo, sc_hi, mn_lo, mn_hi; };
__device__ __forceinline__ K4Packed k4_unpack(const uint4& hdr) {
    const uint32_t u0 = hdr.y, u1 = hdr.z, u2 = hdr.w;
    K4Packed r;
    r.sc_lo = u0 & 0x3f3f3f3fu;
    r.mn_lo = u1 & 0x3f3f3f3fu;
    r.sc_hi = (u2 & 0x0f0f0f0fu) | (((u0 >> 6) & 0x03030303u) << 4);
    r.mn_hi = ((u2 >> 4) & 0x0f0f0f0fu) | (((u1 >> 6) & 0x03030303u) << 4);
    return r;
}

struct I8Q4K {
    static constexpr int kBlockBytes = 144, kQs = 16;
    static constexpr bool kFifth = false;
};
struct I8Q5K {
    static constexpr int kBlockBytes = 176, kQs = 48;
    static constexpr bool kFifth = true;
};

// per n-subtile: what a lane holds of its weight row for the current super-block and step
struct BRegs { uint4 hdr; uint4 qh; uint4 qs; };

template <typename FMT>
__global__ __launch_bounds__(kThreads) void gemm_i8_kernel(const int8_t* __restrict__ xq, const float2* __restrict__ xsc, const uint8_t* __restrict__ w,
                                                            void* __restrict__ y, int y_dtype, int rows, int n, int bpr) {
    __shared__ __align__(16) unsigned char a_lds[2][kBM * kARow];
    __shared__ __align__(16) float xs_lds[2][2][2][kBM];      // [buffer][group of the step][0: xs, 1: xs * sum][token]
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int col = lane & 31, half = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;                  // wave tile: tokens 64 wm .. +64, rows 64 wn .. +64
    const int t0 = blockIdx.y * kBM, n0 = blockIdx.x * kBN;
    const int kpad = bpr * 256, groups = bpr * 8;
    const int steps = bpr * 4;                                // one step = one pair of groups (64 weights)

    // B side: the lane's two weight rows
    const uint8_t* wrow[2];
#pragma unroll
    for (int ns = 0; ns < 2; ++ns) {
        const int r = n0 + 64 * wn + 32 * ns + col;
        wrow[ns] = w + static_cast<size_t>(r < n ? r : 0) * bpr * FMT::kBlockBytes;
    }
    // A side: every thread stages two 16-byte pieces per step (token = piece / 4, piece % 4 of the 64 bytes) and one scale pair
    const int a_tok[2] = {tid >> 2, 64 + (tid >> 2)};
    const int a_part = tid & 3;
    const int s_tok = tid >> 1, s_g = tid & 1;
    auto load_a = [&](int step, uint4 (&av)[2], float2& sv) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int t = min(t0 + a_tok[i], rows - 1);
            av[i] = *reinterpret_cast<const uint4*>(xq + static_cast<size_t>(t) * kpad + 64 * step + 16 * a_part);
        }
        sv = xsc[static_cast<size_t>(min(t0 + s_tok, rows - 1)) * groups + 2 * step + s_g];
    };
    auto store_a = [&](int buf, const uint4 (&av)[2], const float2& sv) {
#pragma unroll
        for (int i = 0; i < 2; ++i) *reinterpret_cast<uint4*>(&a_lds[buf][a_tok[i] * kARow + 16 * a_part]) = av[i];
        xs_lds[buf][s_g][0][s_tok] = sv.x;
        xs_lds[buf][s_g][1][s_tok] = sv.y;
    };
    auto load_b = [&](int step, BRegs (&b)[2]) {
        const int blk = step >> 2, p = step & 3;
#pragma unroll
        for (int ns = 0; ns < 2; ++ns) {
            const uint8_t* base = wrow[ns] + static_cast<size_t>(blk) * FMT::kBlockBytes;
            if (p == 0) {
                b[ns].hdr = *reinterpret_cast<const uint4*>(base);
                if constexpr (FMT::kFifth) b[ns].qh = *reinterpret_cast<const uint4*>(base + 16 + 16 * half);
            }
            b[ns].qs = *reinterpret_cast<const uint4*>(base + FMT::kQs + 32 * p + 16 * half);
        }
    };

    float acc[2][2][16];
#pragma unroll
    for (int ms = 0; ms < 2; ++ms)
#pragma unroll
        for (int ns = 0; ns < 2; ++ns)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[ms][ns][i] = 0.0f;

    uint4 av[2];
    float2 sv;
    BRegs b[2], bn[2];
    load_a(0, av, sv);
    load_b(0, b);
    store_a(0, av, sv);
    __syncthreads();
#pragma unroll 1
    for (int step = 0; step < steps; ++step) {
        const int buf = step & 1;
        const int p = step & 3;
        const bool more = step + 1 < steps;
        if (more) {                                           // next step's operands on their way during this step's matrix work
            load_a(step + 1, av, sv);
            bn[0] = b[0]; bn[1] = b[1];                       // header and fifth bits carry over inside a super-block
            load_b(step + 1, bn);
        }
        // float scales of the two groups for the lane's two rows: d * sc, dmin * m
        float dsc[2][2], dmn[2][2];
        uint32_t codes[2][2][4];                              // [n-subtile][group of the step][dword]
#pragma unroll
        for (int ns = 0; ns < 2; ++ns) {
            const K4Packed s4 = k4_unpack(b[ns].hdr);
            const uint32_t scw = ((p & 2) ? s4.sc_hi : s4.sc_lo) >> (16 * (p & 1));
            const uint32_t mnw = ((p & 2) ? s4.mn_hi : s4.mn_lo) >> (16 * (p & 1));
            const float d = f16_bits_to_float(b[ns].hdr.x & 0xffffu), dmin = f16_bits_to_float(b[ns].hdr.x >> 16);
            dsc[ns][0] = d * static_cast<float>(scw & 0xffu);
            dsc[ns][1] = d * static_cast<float>((scw >> 8) & 0xffu);
            dmn[ns][0] = dmin * static_cast<float>(mnw & 0xffu);
            dmn[ns][1] = dmin * static_cast<float>((mnw >> 8) & 0xffu);
            const uint32_t q[4] = {b[ns].qs.x, b[ns].qs.y, b[ns].qs.z, b[ns].qs.w};
            uint32_t h[4] = {0u, 0u, 0u, 0u};
            if constexpr (FMT::kFifth) { h[0] = b[ns].qh.x; h[1] = b[ns].qh.y; h[2] = b[ns].qh.z; h[3] = b[ns].qh.w; }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                uint32_t lo = q[j] & 0x0f0f0f0fu, hi = (q[j] >> 4) & 0x0f0f0f0fu;
                if constexpr (FMT::kFifth) {                  // bit 2p / 2p + 1 of every qh byte to bit 4 of the code
                    lo |= ((h[j] >> (2 * p)) << 4) & 0x10101010u;
                    hi |= ((h[j] >> (2 * p + 1)) << 4) & 0x10101010u;
                }
                codes[ns][0][j] = lo;
                codes[ns][1][j] = hi;
            }
        }
#pragma unroll
        for (int ms = 0; ms < 2; ++ms) {
            const int tok = 64 * wm + 32 * ms;                // first token of the accumulator tile inside the workgroup tile
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                const uint4 a = *reinterpret_cast<const uint4*>(&a_lds[buf][(tok + col) * kARow + 32 * g + 16 * half]);
                const v4i av4 = {static_cast<int>(a.x), static_cast<int>(a.y), static_cast<int>(a.z), static_cast<int>(a.w)};
                v16i c[2];
#pragma unroll
                for (int ns = 0; ns < 2; ++ns) {
                    const v4i bv = {static_cast<int>(codes[ns][g][0]), static_cast<int>(codes[ns][g][1]), static_cast<int>(codes[ns][g][2]),
                                    static_cast<int>(codes[ns][g][3])};
                    const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    c[ns] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av4, bv, zero, 0, 0, 0);
                }
                // the 16 accumulator registers of a lane are tokens 8 (i / 4) + 4 half + i % 4 of the tile
#pragma unroll
                for (int qd = 0; qd < 4; ++qd) {
                    const float4 xsv = *reinterpret_cast<const float4*>(&xs_lds[buf][g][0][tok + 8 * qd + 4 * half]);
                    const float4 xss = *reinterpret_cast<const float4*>(&xs_lds[buf][g][1][tok + 8 * qd + 4 * half]);
                    const float xs4[4] = {xsv.x, xsv.y, xsv.z, xsv.w};
                    const float ss4[4] = {xss.x, xss.y, xss.z, xss.w};
#pragma unroll
                    for (int ns = 0; ns < 2; ++ns) {
                        const float sc = dsc[ns][g], mn = dmn[ns][g];
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const int i = 4 * qd + j;
                            float r = acc[ms][ns][i];
                            r = __builtin_fmaf(static_cast<float>(c[ns][i]) * xs4[j], sc, r);
                            r = __builtin_fmaf(-ss4[j], mn, r);
                            acc[ms][ns][i] = r;
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);            // one pair of MFMA results live at a time
            }
        }
        if (more) {
            store_a(buf ^ 1, av, sv);                         // the other buffer: nobody reads it during this step
            b[0] = bn[0]; b[1] = bn[1];
        }
        __syncthreads();
    }
    // one uniform branch on the output type around the whole store loop
    auto store_all = [&](auto put) {
#pragma unroll
        for (int ms = 0; ms < 2; ++ms)
#pragma unroll
            for (int ns = 0; ns < 2; ++ns) {
                const int r = n0 + 64 * wn + 32 * ns + col;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int t = t0 + 64 * wm + 32 * ms + 8 * (i >> 2) + 4 * half + (i & 3);
                    if (t < rows && r < n) put(static_cast<size_t>(t) * n + r, acc[ms][ns][i]);
                }
            }
    };
    if (y_dtype == PLLM_F32) store_all([&](size_t at, float v) { static_cast<float*>(y)[at] = v; });
    else if (y_dtype == PLLM_BF16) store_all([&](size_t at, float v) { static_cast<bf16_t*>(y)[at] = from_float<bf16_t>(v); });
    else store_all([&](size_t at, float v) { static_cast<f16_t*>(y)[at] = from_float<f16_t>(v); });
}


}  // namespace

bool gemm_i8_supports(int type_id) { return type_id == PLLM_TYPE_Q4_K || type_id == PLLM_TYPE_Q5_K; }

size_t gemm_i8_workspace_bytes(int rows, int bpr) {
    return align256(static_cast<size_t>(rows) * bpr * 256) + align256(static_cast<size_t>(rows) * bpr * 8 * sizeof(float2));
}

int gemm_i8(const void* x, int x_dtype, const uint8_t* w, int type_id, void* y, int y_dtype,
            int rows, int k, int n, int bpr, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    if (!gemm_i8_supports(type_id)) return PLLM_ERR_UNSUPPORTED;
    if (!workspace || workspace_bytes < gemm_i8_workspace_bytes(rows, bpr)) return PLLM_ERR_WORKSPACE;
    if (rows > 65535) return PLLM_ERR_UNSUPPORTED;                          // one grid row of the quantizer per activation row
    const int kpad = bpr * 256;
    int8_t* xq = static_cast<int8_t*>(workspace);
    float2* xsc = reinterpret_cast<float2*>(static_cast<unsigned char*>(workspace) + align256(static_cast<size_t>(rows) * kpad));
    hipLaunchKernelGGL(q8_rows_kernel, dim3((kpad / 4 + 255) / 256, rows), dim3(256), 0, stream, x, x_dtype, xq, xsc, k, kpad);
    if (hipGetLastError() != hipSuccess) return PLLM_ERR_LAUNCH;
    const dim3 grid((n + kBN - 1) / kBN, (rows + kBM - 1) / kBM);
    if (type_id == PLLM_TYPE_Q4_K)
        hipLaunchKernelGGL(gemm_i8_kernel<I8Q4K>, grid, dim3(kThreads), 0, stream, xq, xsc, w, y, y_dtype, rows, n, bpr);
    else
        hipLaunchKernelGGL(gemm_i8_kernel<I8Q5K>, grid, dim3(kThreads), 0, stream, xq, xsc, w, y, y_dtype, rows, n, bpr);
    return hipGetLastError() == hipSuccess ? PLLM_OK : PLLM_ERR_LAUNCH;
}

}  // namespace pllm
