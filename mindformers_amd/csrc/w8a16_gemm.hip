// W8A16 weight-only skinny GEMM for decode (M <= 64 per pass): y = (x . w_i8^T) * scale (+bias) (+residual).
//
// The int8 weight matrix [N, K] is the only large operand: it is streamed from HBM exactly once, each lane
// loading 16 contiguous bytes of one weight row straight into the MFMA A-operand layout (no LDS), converted
// to bf16/fp16 in registers (exact: |w| <= 127) and multiplied on the 16x16x32 matrix cores against the
// activation tile, which every wave re-reads from L2.  A workgroup owns 64 output channels (4 MFMA row tiles) for
// all M rows; its 4 waves interleave the 64-wide k-steps of the workgroup's k-range and are summed through
// LDS at the end.  When N is too small to fill the chip the k-range is additionally split across workgroups
// (fp32 partials + a fused reduce/epilogue kernel).
//
// MFMA roles: A = weights [16 n x 32 k], B = activations [32 k x 16 m], C = y^T tile [16 n x 16 m].
// k-ordering trick: one 16-byte weight load covers 16 k of a row; bytes 0-7 feed the first MFMA of the
// step and bytes 8-15 the second, and the activation operand uses the same (permuted) k order, so no
// shuffling is needed.
#include "common.h"

namespace {

constexpr int GW_WAVES = 4;
constexpr int GW_NT = 4;                    // 16-row weight tiles per wave
constexpr int GW_BN = 16 * GW_NT;           // output channels per workgroup
constexpr int GW_KSTEP = 64;

// 8 int8 (two dwords) -> 8 elements of T, exact.
template <typename T>
__device__ __forceinline__ typename T::vec8 dequant8(uint32_t lo, uint32_t hi);

__device__ __forceinline__ uint32_t i8x2_to_bf16x2(uint32_t w, int shift) {
    const float f0 = (float)(int)(int8_t)(w >> shift);
    const float f1 = (float)(int)(int8_t)(w >> (shift + 8));
    // integers of magnitude <= 128 are exact in bf16: take the high halves
    return __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);
}
template <>
__device__ __forceinline__ bf16x8 dequant8<BF16>(uint32_t lo, uint32_t hi) {
    u32x4 v = {i8x2_to_bf16x2(lo, 0), i8x2_to_bf16x2(lo, 16), i8x2_to_bf16x2(hi, 0), i8x2_to_bf16x2(hi, 16)};
    return bitcast<bf16x8>(v);
}
template <>
__device__ __forceinline__ f16x8 dequant8<FP16>(uint32_t lo, uint32_t hi) {
    f16x8 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[i] = (_Float16)(float)(int)(int8_t)(lo >> (8 * i));
        v[4 + i] = (_Float16)(float)(int)(int8_t)(hi >> (8 * i));
    }
    return v;
}

// Epilogue for 4 consecutive output channels of one row.
template <typename T>
__device__ __forceinline__ void store4(uint16_t* y, const uint16_t* bias, const uint16_t* residual,
                                       const float* scale, int64_t row_off, int n, int N, f32x4 acc) {
    float o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (n + i < N) {
            float v = acc[i] * scale[n + i];
            if (bias) v += T::to_float(bias[n + i]);
            if (residual) v = T::to_float(T::from_float(v)) + T::to_float(residual[row_off + n + i]);
            o[i] = v;
        } else {
            o[i] = 0.f;
        }
    }
    if (n + 3 < N && ((row_off + n) & 3) == 0) {
        *(u32x2*)(y + row_off + n) = (u32x2){pack2<T>(o[0], o[1]), pack2<T>(o[2], o[3])};
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (n + i < N) y[row_off + n + i] = T::from_float(o[i]);
    }
}

// One workgroup tile: 64 output channels [n0, n0+64) x 16*MT rows [m0, ...) x k-steps [s_begin, s_end).
// MT = number of 16-row activation tiles.
template <typename T, int MT>
__device__ __forceinline__ void w8a16_tile(uint16_t* __restrict__ y, float* __restrict__ partial,
                                           const uint16_t* __restrict__ x, const int8_t* __restrict__ w,
                                           const float* __restrict__ scale, const uint16_t* __restrict__ bias,
                                           const uint16_t* __restrict__ residual, int M, int N, int K, int n0,
                                           int m0, int s_begin, int s_end, int split_index) {
    using vec8 = typename T::vec8;
    // red[wave][m][n], 16-byte granules XOR-swizzled by the row so that neither the MFMA-layout writes nor the
    // row-major reads collide on LDS banks (64 KB at MT = 4, the static limit, so no padding)
    __shared__ __attribute__((aligned(16))) float red[GW_WAVES][16 * MT][GW_BN];

    const int wv = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int r = lane & 15;
    const int g = lane >> 4;

    f32x4 acc[GW_NT][MT];
#pragma unroll
    for (int nt = 0; nt < GW_NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // per-lane row pointers (rows beyond N / M read row 0 and are zeroed)
    const int8_t* wrow[GW_NT];
    bool wok[GW_NT];
#pragma unroll
    for (int nt = 0; nt < GW_NT; ++nt) {
        const int n = n0 + nt * 16 + r;
        wok[nt] = n < N;
        wrow[nt] = w + (int64_t)(wok[nt] ? n : 0) * K + 16 * g;
    }
    const uint16_t* xrow[MT];
    bool xok[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = m0 + mt * 16 + r;
        xok[mt] = m < M;
        xrow[mt] = x + (int64_t)(xok[mt] ? m : 0) * K + 16 * g;
    }

    for (int s = s_begin + wv; s < s_end; s += GW_WAVES) {
        const int kb = s * GW_KSTEP;
        const bool kok = kb + 16 * g < K;                     // K is a multiple of 16; the last step may be short
        u32x4 wreg[GW_NT];
#pragma unroll
        for (int nt = 0; nt < GW_NT; ++nt) {
            wreg[nt] = (u32x4){0u, 0u, 0u, 0u};
            if (kok && wok[nt]) wreg[nt] = *(const u32x4*)(wrow[nt] + kb);
        }
        u32x4 xreg[MT][2];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            xreg[mt][0] = (u32x4){0u, 0u, 0u, 0u};
            xreg[mt][1] = (u32x4){0u, 0u, 0u, 0u};
            if (kok && xok[mt]) {
                xreg[mt][0] = *(const u32x4*)(xrow[mt] + kb);
                xreg[mt][1] = *(const u32x4*)(xrow[mt] + kb + 8);
            }
        }
#pragma unroll
        for (int nt = 0; nt < GW_NT; ++nt) {
            const vec8 a0 = dequant8<T>(wreg[nt][0], wreg[nt][1]);
            const vec8 a1 = dequant8<T>(wreg[nt][2], wreg[nt][3]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                acc[nt][mt] = T::mfma16(a0, bitcast<vec8>(xreg[mt][0]), acc[nt][mt]);
                acc[nt][mt] = T::mfma16(a1, bitcast<vec8>(xreg[mt][1]), acc[nt][mt]);
            }
        }
    }

    // ---- sum the 4 waves through LDS: red[wave][m][n]
#pragma unroll
    for (int nt = 0; nt < GW_NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) *(f32x4*)&red[wv][mt * 16 + r][((nt * 4 + g) ^ r) << 2] = acc[nt][mt];
    __syncthreads();

    constexpr int N4 = GW_BN / 4;
    for (int idx = threadIdx.x; idx < 16 * MT * N4; idx += GW_WAVES * 64) {
        const int ml = idx / N4, n4 = idx - ml * N4;
        const int m = m0 + ml, n = n0 + 4 * n4;
        if (m >= M || n >= N) continue;
        const int sw = (n4 ^ (ml & 15)) << 2;
        f32x4 sum = *(const f32x4*)&red[0][ml][sw];
#pragma unroll
        for (int q = 1; q < GW_WAVES; ++q) sum += *(const f32x4*)&red[q][ml][sw];
        if (partial) {
            float* p = partial + ((int64_t)split_index * M + m) * N + n;
            if (n + 3 < N && (N & 3) == 0) {
                *(f32x4*)p = sum;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < N) p[i] = sum[i];
            }
        } else {
            store4<T>(y, bias, residual, scale, (int64_t)m * N, n, N, sum);
        }
    }
}

// Dense: grid = (ceil(N/64), split_k, ceil(M/(16*MT))).
template <typename T, int MT>
__global__ __launch_bounds__(GW_WAVES * 64, 2) void w8a16_gemm_kernel(
    uint16_t* __restrict__ y, float* __restrict__ partial, const uint16_t* __restrict__ x,
    const int8_t* __restrict__ w, const float* __restrict__ scale, const uint16_t* __restrict__ bias,
    const uint16_t* __restrict__ residual, int M, int N, int K, int steps_per_split) {
    const int total_steps = (K + GW_KSTEP - 1) / GW_KSTEP;
    const int s_begin = blockIdx.y * steps_per_split;
    const int s_end = min(total_steps, s_begin + steps_per_split);
    w8a16_tile<T, MT>(y, partial, x, w, scale, bias, residual, M, N, K, blockIdx.x * GW_BN,
                      blockIdx.z * (16 * MT), s_begin, s_end, blockIdx.y);
}

// Grouped (experts): grid = (ceil(N/64), n_experts).  Rows offsets[e] .. offsets[e+1] of x use expert e's
// weights w[e] ([N, K]) and scale[e]; experts with no rows exit at once.  Rows are taken 16 at a time
// (decode batches route a handful of tokens to each expert), re-streaming the expert's weights per pass.
template <typename T>
__global__ __launch_bounds__(GW_WAVES * 64, 2) void w8a16_grouped_kernel(
    uint16_t* __restrict__ y, const uint16_t* __restrict__ x, const int8_t* __restrict__ w,
    const float* __restrict__ scale, const int32_t* __restrict__ offsets, int total_rows, int N, int K) {
    const int e = blockIdx.y;
    int row0 = offsets[e], row1 = offsets[e + 1];
    row0 = max(0, min(row0, total_rows));
    row1 = max(row0, min(row1, total_rows));
    const int rows = row1 - row0;
    if (rows == 0) return;
    const int total_steps = (K + GW_KSTEP - 1) / GW_KSTEP;
    const int8_t* we = w + (int64_t)e * N * K;
    const float* se = scale + (int64_t)e * N;
    for (int m0 = 0; m0 < rows; m0 += 16) {
        w8a16_tile<T, 1>(y + (int64_t)row0 * N, nullptr, x + (int64_t)row0 * K, we, se, nullptr, nullptr, rows, N, K,
                         blockIdx.x * GW_BN, m0, 0, total_steps, 0);
        __syncthreads();                                      // the LDS reduction buffer is reused by the next pass
    }
}

template <typename T>
__global__ void w8a16_splitk_reduce_kernel(uint16_t* __restrict__ y, const float* __restrict__ partial,
                                           const float* __restrict__ scale, const uint16_t* __restrict__ bias,
                                           const uint16_t* __restrict__ residual, int M, int N, int split_k) {
    const int n4cnt = (N + 3) / 4;
    const int64_t total = (int64_t)M * n4cnt;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int m = (int)(idx / n4cnt);
        const int n = (int)(idx - (int64_t)m * n4cnt) * 4;
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int s = 0; s < split_k; ++s) {
            const float* p = partial + ((int64_t)s * M + m) * N + n;
            if (n + 3 < N && (N & 3) == 0) {
                sum += *(const f32x4*)p;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < N) sum[i] += p[i];
            }
        }
        store4<T>(y, bias, residual, scale, (int64_t)m * N, n, N, sum);
    }
}

struct GemmPlan {
    int mt;          // activation tiles per pass (1, 2, 4)
    int m_blocks;
    int n_blocks;
    int split_k;
    int steps_per_split;
};

GemmPlan plan_w8a16(int m, int n, int k) {
    GemmPlan p;
    p.mt = m <= 16 ? 1 : (m <= 32 ? 2 : 4);
    p.m_blocks = (m + 16 * p.mt - 1) / (16 * p.mt);
    p.n_blocks = (n + GW_BN - 1) / GW_BN;
    const int total_steps = (k + GW_KSTEP - 1) / GW_KSTEP;
    // aim at two resident workgroups on each of the 256 CUs; keep at least 8 k-steps per workgroup
    int sk = 512 / (p.n_blocks * p.m_blocks);
    sk = sk < 1 ? 1 : sk;
    const int max_sk = total_steps / 8 < 1 ? 1 : total_steps / 8;
    sk = sk > max_sk ? max_sk : sk;
    sk = sk > 16 ? 16 : sk;
    p.steps_per_split = (total_steps + sk - 1) / sk;
    p.split_k = (total_steps + p.steps_per_split - 1) / p.steps_per_split;
    return p;
}

template <typename T>
int launch_w8a16(void* y, const void* x, const int8_t* w, const float* scale, const void* bias,
                 const void* residual, int m, int n, int k, void* workspace, hipStream_t st) {
    const GemmPlan p = plan_w8a16(m, n, k);
    float* partial = p.split_k > 1 ? (float*)workspace : nullptr;
    dim3 grid(p.n_blocks, p.split_k, p.m_blocks);
    dim3 block(GW_WAVES * 64);
#define GW_LAUNCH(MTV)                                                                                          \
    hipLaunchKernelGGL((w8a16_gemm_kernel<T, MTV>), grid, block, 0, st, (uint16_t*)y, partial, (const uint16_t*)x, \
                       w, scale, (const uint16_t*)bias, (const uint16_t*)residual, m, n, k, p.steps_per_split)
    if (p.mt == 1) GW_LAUNCH(1);
    else if (p.mt == 2) GW_LAUNCH(2);
    else GW_LAUNCH(4);
#undef GW_LAUNCH
    int rc = MF_LAUNCH_CHECK();
    if (rc || !partial) return rc;
    const int64_t total = (int64_t)m * ((n + 3) / 4);
    const int blocks = (int)((total + 255) / 256 > 4096 ? 4096 : (total + 255) / 256);
    hipLaunchKernelGGL((w8a16_splitk_reduce_kernel<T>), dim3(blocks), dim3(256), 0, st, (uint16_t*)y, partial, scale,
                       (const uint16_t*)bias, (const uint16_t*)residual, m, n, p.split_k);
    return MF_LAUNCH_CHECK();
}

}  // namespace

extern "C" size_t mf_w8a16_workspace_bytes(int m, int n, int k) {
    if (m <= 0 || n <= 0 || k <= 0) return 0;
    const GemmPlan p = plan_w8a16(m, n, k);
    return p.split_k > 1 ? (size_t)p.split_k * m * n * sizeof(float) : 0;
}

extern "C" int mf_w8a16_gemm(void* y, const void* x, const int8_t* w, const float* scale, const void* bias,
                             const void* residual, int m, int n, int k, int dtype, void* workspace,
                             size_t workspace_bytes, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "w8a16_gemm: dtype must be bf16 or fp16");
    if (m == 0) return 0;
    MF_REQUIRE(y && x && w && scale, "w8a16_gemm: null argument");
    MF_REQUIRE(m >= 0 && n > 0 && k > 0, "w8a16_gemm: bad sizes m=%d n=%d k=%d", m, n, k);
    MF_REQUIRE(k % 16 == 0, "w8a16_gemm: K (%d) must be a multiple of 16", k);
    MF_REQUIRE((((uintptr_t)x | (uintptr_t)w) & 15) == 0, "w8a16_gemm: x and w must be 16-byte aligned");
    if (m == 0) return 0;
    const size_t need = mf_w8a16_workspace_bytes(m, n, k);
    MF_REQUIRE(need == 0 || (workspace && workspace_bytes >= need && ((uintptr_t)workspace & 15) == 0),
               "w8a16_gemm: 16-byte aligned workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    if (dtype == MF_BF16)
        return launch_w8a16<BF16>(y, x, w, scale, bias, residual, m, n, k, workspace, (hipStream_t)stream);
    return launch_w8a16<FP16>(y, x, w, scale, bias, residual, m, n, k, workspace, (hipStream_t)stream);
}

extern "C" int mf_grouped_w8a16_gemm(void* y, const void* x, const int8_t* w, const float* scale,
                                     const int32_t* offsets, int n_experts, int total_rows, int n, int k, int dtype,
                                     void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "grouped_w8a16_gemm: dtype must be bf16 or fp16");
    if (total_rows == 0) return 0;
    MF_REQUIRE(y && x && w && scale && offsets, "grouped_w8a16_gemm: null argument");
    MF_REQUIRE(n_experts > 0 && n_experts <= 65535 && total_rows >= 0 && n > 0 && k > 0,
               "grouped_w8a16_gemm: bad sizes");
    MF_REQUIRE(k % 16 == 0, "grouped_w8a16_gemm: K (%d) must be a multiple of 16", k);
    MF_REQUIRE((((uintptr_t)x | (uintptr_t)w) & 15) == 0, "grouped_w8a16_gemm: x and w must be 16-byte aligned");
    if (total_rows == 0) return 0;
    dim3 grid((n + GW_BN - 1) / GW_BN, n_experts);
    if (dtype == MF_BF16)
        hipLaunchKernelGGL(w8a16_grouped_kernel<BF16>, grid, dim3(GW_WAVES * 64), 0, (hipStream_t)stream, (uint16_t*)y,
                           (const uint16_t*)x, w, scale, offsets, total_rows, n, k);
    else
        hipLaunchKernelGGL(w8a16_grouped_kernel<FP16>, grid, dim3(GW_WAVES * 64), 0, (hipStream_t)stream, (uint16_t*)y,
                           (const uint16_t*)x, w, scale, offsets, total_rows, n, k);
    return MF_LAUNCH_CHECK();
}
