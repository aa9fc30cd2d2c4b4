// W8A8 GEMM: per-token int8 activations x per-channel int8 weights on the gfx950 int8 matrix cores
// (v_mfma_i32_16x16x64_i8), exact int32 accumulation, dequantised to bf16/fp16 in the epilogue:
//   y[m,n] = acc[m,n] * x_scale[m] * w_scale[n] (+ bias[n]) (+ residual[m,n]).
//
// Both operands are K-contiguous ([M,K] and [N,K]), which is exactly the MFMA operand layout
// (lane = row, 16 consecutive k bytes), so tiles go global -> LDS -> registers with 16-byte accesses and no
// transposition.  A workgroup of 4 waves owns a 128 x 128 output tile; each wave a 64 x 64 quadrant
// (4 x 4 MFMA tiles, 64 accumulator registers).  K is walked in 64-byte steps, double-buffered in LDS.
#include "common.h"

namespace {

constexpr int Q_BM = 128, Q_BN = 128, Q_BK = 64;
constexpr int Q_ROW = Q_BK + 16;   // LDS row pitch in bytes (80): 16-byte aligned, spreads rows over banks

template <typename T>
__global__ __launch_bounds__(256, 2) void w8a8_gemm_kernel(uint16_t* __restrict__ y, int32_t* __restrict__ acc_out,
                                                          const int8_t* __restrict__ xq,
                                                          const float* __restrict__ x_scale,
                                                          const int8_t* __restrict__ w,
                                                          const float* __restrict__ w_scale,
                                                          const uint16_t* __restrict__ bias,
                                                          const uint16_t* __restrict__ residual, int M, int N,
                                                          int K) {
    __shared__ __attribute__((aligned(16))) uint8_t sA[2][Q_BM * Q_ROW];
    __shared__ __attribute__((aligned(16))) uint8_t sB[2][Q_BN * Q_ROW];

    const int tid = threadIdx.x;
    const int wv = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int wm = wv >> 1, wn = wv & 1;                      // wave quadrant
    const int m0 = blockIdx.y * Q_BM, n0 = blockIdx.x * Q_BN;

    // cooperative tile load: 128 rows x 64 B = 512 chunks of 16 B per operand, 2 per thread
    const int lrow = tid >> 2, lchunk = tid & 3;              // rows lrow and lrow + 64
    const int8_t* ga[2];
    const int8_t* gb[2];
    bool oka[2], okb[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int am = m0 + lrow + 64 * h, bn = n0 + lrow + 64 * h;
        oka[h] = am < M;
        okb[h] = bn < N;
        ga[h] = xq + (int64_t)(oka[h] ? am : 0) * K + 16 * lchunk;
        gb[h] = w + (int64_t)(okb[h] ? bn : 0) * K + 16 * lchunk;
    }

    i32x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (i32x4){0, 0, 0, 0};

    const int steps = (K + Q_BK - 1) / Q_BK;
    u32x4 ra[2], rb[2];
    auto gload = [&](int s) {
        const int kb = s * Q_BK;
        const bool kok = kb + 16 * lchunk < K;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            ra[h] = (u32x4){0u, 0u, 0u, 0u};
            rb[h] = (u32x4){0u, 0u, 0u, 0u};
            if (kok && oka[h]) ra[h] = *(const u32x4*)(ga[h] + kb);
            if (kok && okb[h]) rb[h] = *(const u32x4*)(gb[h] + kb);
        }
    };
    auto sstore = [&](int buf) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            *(u32x4*)(sA[buf] + (lrow + 64 * h) * Q_ROW + 16 * lchunk) = ra[h];
            *(u32x4*)(sB[buf] + (lrow + 64 * h) * Q_ROW + 16 * lchunk) = rb[h];
        }
    };

    gload(0);
    sstore(0);
    __syncthreads();
    for (int s = 0; s < steps; ++s) {
        const int buf = s & 1;
        if (s + 1 < steps) gload(s + 1);
        i32x4 fa[4], fb[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            fa[i] = *(const i32x4*)(sA[buf] + (wm * 64 + i * 16 + r) * Q_ROW + 16 * g);
#pragma unroll
        for (int j = 0; j < 4; ++j)
            fb[j] = *(const i32x4*)(sB[buf] + (wn * 64 + j * 16 + r) * Q_ROW + 16 * g);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
        if (s + 1 < steps) sstore(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: acc[i][j][e] is row m = 4g + e of tile i, column n = r of tile j
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int m = m0 + wm * 64 + i * 16 + 4 * g + e;
            if (m >= M) continue;
            const float xs = x_scale[m];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = n0 + wn * 64 + j * 16 + r;
                if (n >= N) continue;
                const int a = acc[i][j][e];
                const int64_t o = (int64_t)m * N + n;
                if (acc_out) acc_out[o] = a;
                if (y) {
                    float v = (float)a * xs * w_scale[n];
                    if (bias) v += T::to_float(bias[n]);
                    if (residual) v = T::to_float(T::from_float(v)) + T::to_float(residual[o]);
                    y[o] = T::from_float(v);
                }
            }
        }
}

}  // namespace

extern "C" int mf_w8a8_gemm(void* y, int32_t* acc_out, const int8_t* xq, const float* x_scale, const int8_t* w,
                            const float* w_scale, const void* bias, const void* residual, int m, int n, int k,
                            int dtype, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "w8a8_gemm: dtype must be bf16 or fp16");
    if (m == 0) return 0;
    MF_REQUIRE(xq && w && (y || acc_out), "w8a8_gemm: null argument");
    MF_REQUIRE(!y || (x_scale && w_scale), "w8a8_gemm: scales required for a dequantised output");
    MF_REQUIRE(m >= 0 && n > 0 && k > 0 && k % 16 == 0, "w8a8_gemm: bad sizes m=%d n=%d k=%d (K %% 16 == 0)", m, n, k);
    MF_REQUIRE((((uintptr_t)xq | (uintptr_t)w) & 15) == 0, "w8a8_gemm: xq and w must be 16-byte aligned");
    if (m == 0) return 0;
    dim3 grid((n + Q_BN - 1) / Q_BN, (m + Q_BM - 1) / Q_BM);
    if (dtype == MF_BF16)
        hipLaunchKernelGGL(w8a8_gemm_kernel<BF16>, grid, dim3(256), 0, (hipStream_t)stream, (uint16_t*)y, acc_out, xq,
                           x_scale, w, w_scale, (const uint16_t*)bias, (const uint16_t*)residual, m, n, k);
    else
        hipLaunchKernelGGL(w8a8_gemm_kernel<FP16>, grid, dim3(256), 0, (hipStream_t)stream, (uint16_t*)y, acc_out, xq,
                           x_scale, w, w_scale, (const uint16_t*)bias, (const uint16_t*)residual, m, n, k);
    return MF_LAUNCH_CHECK();
}
