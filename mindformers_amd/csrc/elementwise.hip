// Row-wise and elementwise kernels of the decode layer: RMSNorm (optionally fused with the preceding
// residual add), SiLU*mul, residual add, per-token dynamic int8 quantisation.
// All are single-pass, HBM-bound, 16-byte lane accesses; one workgroup per row where a row reduction is
// needed (the row is held in registers between the reduction and the scaled write).
#include <algorithm>

#include "common.h"

namespace {

constexpr int ROW_THREADS = 256;   // per-token quantisation: threads per row for narrow rows ...
constexpr int ROW_THREADS_WIDE = 1024;   // ... and for wide ones (one workgroup per row either way: more waves in flight)
constexpr int ROW_MAX_COLS = 24576;
constexpr int NORM_THREADS = 512;  // RMSNorm: the geometry (and summation order) shared with the GEMM-fused norm
constexpr int NORM_MAX_VEC = 4;    // up to 4 x (8 elements) per thread: cols <= 512*4*8 = 16384

__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < (int)(blockDim.x >> 6); ++i) t += red[i];
    __syncthreads();
    return t;
}
template <typename T>
__global__ __launch_bounds__(NORM_THREADS) void rmsnorm_kernel(uint16_t* __restrict__ y,
                                                             uint16_t* __restrict__ sum_out,
                                                             const uint16_t* __restrict__ x,
                                                             const uint16_t* __restrict__ residual,
                                                             const void* __restrict__ gamma, float eps, int cols,
                                                             int gamma_dtype, int64_t x_stride) {
    // x_stride: elements between two rows of x (a column slice of a wider matrix); every other tensor is dense
    __shared__ float red[NORM_THREADS / 64];
    const int64_t row = (int64_t)blockIdx.x * cols;
    const int nvec = cols >> 3;
    float v[NORM_MAX_VEC][8], gm[NORM_MAX_VEC][8];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < NORM_MAX_VEC; ++it) {
        const int c = threadIdx.x + it * NORM_THREADS;
        if (c < nvec) {
            u32x4 raw = *(const u32x4*)(x + (int64_t)blockIdx.x * x_stride + 8 * c);
            u32x4 rraw;
            if (residual) rraw = *(const u32x4*)(residual + row + 8 * c);
            load8_as_float(gamma, 8 * c, gamma_dtype, gm[it]);   // in flight together with the row, used after the sum
            unpack8<T>(raw, v[it]);
            if (residual) {
                float rr[8];
                unpack8<T>(rraw, rr);
                u32x4 s;
#pragma unroll
                for (int i = 0; i < 4; ++i) s[i] = pack2<T>(v[it][2 * i] + rr[2 * i], v[it][2 * i + 1] + rr[2 * i + 1]);
                *(u32x4*)(sum_out + row + 8 * c) = s;
                unpack8<T>(s, v[it]);                          // normalise the rounded sum, as two ops would
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) ss = __fmaf_rn(v[it][i], v[it][i], ss);
        }
    }
    ss = rmsnorm_block_sum<NORM_THREADS>(ss, red);
    const float inv = rsqrtf(ss / (float)cols + eps);
#pragma unroll
    for (int it = 0; it < NORM_MAX_VEC; ++it) {
        const int c = threadIdx.x + it * NORM_THREADS;
        if (c < nvec) {
            u32x4 o;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                o[i] = pack2<T>(v[it][2 * i] * inv * gm[it][2 * i], v[it][2 * i + 1] * inv * gm[it][2 * i + 1]);
            *(u32x4*)(y + row + 8 * c) = o;
        }
    }
}


// layout 0: [gate | up] halves; layout 1: interleaved g,u pairs.  8 outputs per thread.
template <typename T>
__global__ void silu_mul_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ gu, int rows, int cols,
                                int layout) {
    const int64_t nvec = (int64_t)rows * (cols >> 3);
    const int vpr = cols >> 3;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t row = i / vpr;
        const int c = (int)(i - row * vpr) * 8;
        float g[8], u[8];
        const uint16_t* base = gu + row * 2 * cols;
        if (layout == 0) {
            unpack8<T>(*(const u32x4*)(base + c), g);
            unpack8<T>(*(const u32x4*)(base + cols + c), u);
        } else {
            float a[8], b[8];
            unpack8<T>(*(const u32x4*)(base + 2 * c), a);
            unpack8<T>(*(const u32x4*)(base + 2 * c + 8), b);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                g[j] = a[2 * j]; u[j] = a[2 * j + 1];
                g[4 + j] = b[2 * j]; u[4 + j] = b[2 * j + 1];
            }
        }
        u32x4 o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float a0 = T::to_float(T::from_float(silu_f(g[2 * j])));
            const float a1 = T::to_float(T::from_float(silu_f(g[2 * j + 1])));
            o[j] = pack2<T>(a0 * u[2 * j], a1 * u[2 * j + 1]);
        }
        *(u32x4*)(out + row * cols + c) = o;
    }
}

template <typename T>
__global__ void add_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ a,
                           const uint16_t* __restrict__ b, int64_t n) {
    const int64_t nvec = n >> 3;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * blockDim.x) {
        float x[8], y[8];
        unpack8<T>(*(const u32x4*)(a + 8 * i), x);
        unpack8<T>(*(const u32x4*)(b + 8 * i), y);
        u32x4 o;
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = pack2<T>(x[2 * j] + y[2 * j], x[2 * j + 1] + y[2 * j + 1]);
        *(u32x4*)(out + 8 * i) = o;
    }
    // tail (n not a multiple of 8)
    for (int64_t i = (nvec << 3) + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (int64_t)gridDim.x * blockDim.x)
        out[i] = T::from_float(T::to_float(a[i]) + T::to_float(b[i]));
}

// out[m, k] = round_T(float32(x[m, k] * scale[k])): the activation side of an outlier-suppression pair (the multiplier that the
// weights were divided by offline) in front of a weight-only GEMM.  8 elements per thread.
template <typename T>
__global__ void scale_columns_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ x,
                                     const float* __restrict__ scale, int64_t rows, int cols) {
    const int cvec = cols >> 3;
    const int64_t nvec = rows * cvec;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(i % cvec) * 8;
        float v[8];
        unpack8<T>(*(const u32x4*)(x + 8 * i), v);
        const f32x4 s0 = *(const f32x4*)(scale + c), s1 = *(const f32x4*)(scale + c + 4);
        u32x4 o;
        float p[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            p[j] = __fmul_rn(v[j], j < 4 ? s0[j] : s1[j - 4]);
            // the float32 product is the value that is rounded to T: keep the compiler from folding the multiply
            // into a mixed-precision instruction that rounds the exact product once (differs on near-ties)
            asm volatile("" : "+v"(p[j]));
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = pack2<T>(p[2 * j], p[2 * j + 1]);
        *(u32x4*)(out + 8 * i) = o;
    }
}

// Rows grouped by expert (offsets int32 [groups + 1], rows offsets[e] .. offsets[e + 1] - 1 belong to e): the smooth
// multiplier of a row is the row `e` of a [groups, cols] table.  The search is uniform over the workgroup.
struct RowGroups {
    const int32_t* offsets;       // null: one multiplier vector for every row
    int groups;
};
__device__ __forceinline__ const float* smooth_of_row(const float* smooth, RowGroups rg, int row, int cols) {
    if (!smooth || !rg.offsets) return smooth;
    int lo = 0, hi = rg.groups - 1;                           // largest e with offsets[e] <= row
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (rg.offsets[mid] <= row) lo = mid; else hi = mid - 1;
    }
    return smooth + (int64_t)lo * cols;
}

// Per-token dynamic int8: xs = x*smooth; s = max|xs|/127; q = clip(rint(xs/s), -128, 127).
// With static_scale (one float on the device: a calibrated per-tensor activation scale) s is that value for every
// row and no maximum is taken; x_scale still receives s per row, which is what the int8 GEMM's epilogue reads.
template <typename T, int THREADS>
__global__ __launch_bounds__(THREADS) void dynamic_quant_kernel(int8_t* __restrict__ xq, float* __restrict__ x_scale,
                                                               const uint16_t* __restrict__ x,
                                                               const float* __restrict__ smooth_table, int cols,
                                                               int tiled, const float* __restrict__ static_scale,
                                                               RowGroups rg) {
    __shared__ float red[THREADS / 64];
    const float* smooth = smooth_of_row(smooth_table, rg, blockIdx.x, cols);
    const int64_t row = (int64_t)blockIdx.x * cols;
    const int nvec = cols >> 3;
    constexpr int ROW_THREADS = THREADS;
    constexpr int MAXV = ROW_MAX_COLS / 8 / THREADS;
    float v[MAXV][8];
    float amax = 0.f;
#pragma unroll
    for (int it = 0; it < MAXV; ++it) {
        const int c = threadIdx.x + it * ROW_THREADS;
        if (c < nvec) {
            unpack8<T>(*(const u32x4*)(x + row + 8 * c), v[it]);
            amax = fmaxf(amax, smooth_absmax8(v[it], smooth, 8 * c));
        }
    }
    float s;
    if (static_scale) {
        s = static_scale[0];                                  // uniform: no reduction over the row
    } else {
        amax = block_max(amax, red);
        s = __fdiv_rn(amax, 127.0f);
    }
    const float safe = s > 0.f ? s : 1.0f;
    if (threadIdx.x == 0) x_scale[blockIdx.x] = s;
#pragma unroll
    for (int it = 0; it < MAXV; ++it) {
        const int c = threadIdx.x + it * ROW_THREADS;
        if (c < nvec) quant_store8(xq, v[it], safe, blockIdx.x, 8 * c, cols, gridDim.x, tiled);
    }
}

// RMSNorm (optionally with the residual add before it) followed by the per-token quantisation of its output, which
// is not written: the quantised GEMM is its only reader.  Rounding points as the two kernels have them: the sum, and
// the normalised value, are rounded to T before they are used further.
// With PARTIAL the input row is not read but formed from the int32 split-K partial sums of the int8 GEMM before it
// (exact integer sums, then acc * row scale * channel scale (+ bias), rounded to T as that GEMM's own reduce kernel
// rounds what it stores); without a residual that rounded row goes to sum_out when one is given.
struct PartialRow {
    const int32_t* partial;       // [split_k][rows][cols]
    const float* row_scale;       // [rows]: per-token scale of the GEMM's input
    const float* col_scale;       // [cols]: per-channel weight scale
    const uint16_t* bias;         // [cols] or null
    int split_k;
};

template <typename T, bool PARTIAL>
__global__ __launch_bounds__(NORM_THREADS) void rmsnorm_quant_kernel(
    int8_t* __restrict__ xq, float* __restrict__ x_scale, uint16_t* __restrict__ sum_out,
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ residual, const void* __restrict__ gamma,
    const float* __restrict__ smooth, float eps, int cols, int gamma_dtype, int tiled, PartialRow pr) {
    __shared__ float red[NORM_THREADS / 64];
    const int64_t row = (int64_t)blockIdx.x * cols;
    const int nvec = cols >> 3;
    float v[NORM_MAX_VEC][8], gm[NORM_MAX_VEC][8];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < NORM_MAX_VEC; ++it) {
        const int c = threadIdx.x + it * NORM_THREADS;
        if (c < nvec) {
            u32x4 raw;
            if constexpr (PARTIAL) {
                const int32_t* p = pr.partial + row + 8 * c;
                const int64_t stride = (int64_t)gridDim.x * cols;
                i32x4 lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
                for (int s0 = 0; s0 < pr.split_k; s0 += 4) {      // four splits' loads in flight together
                    i32x4 a[4], b[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        if (s0 + q < pr.split_k) {
                            a[q] = *(const i32x4*)(p + (s0 + q) * stride);
                            b[q] = *(const i32x4*)(p + (s0 + q) * stride + 4);
                        }
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        if (s0 + q < pr.split_k) {
                            lo += a[q];
                            hi += b[q];
                        }
                }
                const float xs = pr.row_scale[blockIdx.x];
                const f32x4 w_lo = *(const f32x4*)(pr.col_scale + 8 * c), w_hi = *(const f32x4*)(pr.col_scale + 8 * c + 4);
                float t[8];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    t[i] = (float)lo[i] * xs * w_lo[i];
                    t[4 + i] = (float)hi[i] * xs * w_hi[i];
                }
                if (pr.bias) {
                    float bb[8];
                    unpack8<T>(*(const u32x4*)(pr.bias + 8 * c), bb);
#pragma unroll
                    for (int i = 0; i < 8; ++i) t[i] += bb[i];
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) raw[i] = pack2<T>(t[2 * i], t[2 * i + 1]);
                if (!residual && sum_out) *(u32x4*)(sum_out + row + 8 * c) = raw;
            } else {
                raw = *(const u32x4*)(x + row + 8 * c);
            }
            u32x4 rraw;
            if (residual) rraw = *(const u32x4*)(residual + row + 8 * c);
            load8_as_float(gamma, 8 * c, gamma_dtype, gm[it]);
            unpack8<T>(raw, v[it]);
            if (residual) {
                float rr[8];
                unpack8<T>(rraw, rr);
                u32x4 sm;
#pragma unroll
                for (int i = 0; i < 4; ++i) sm[i] = pack2<T>(v[it][2 * i] + rr[2 * i], v[it][2 * i + 1] + rr[2 * i + 1]);
                *(u32x4*)(sum_out + row + 8 * c) = sm;
                unpack8<T>(sm, v[it]);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) ss = __fmaf_rn(v[it][i], v[it][i], ss);
        }
    }
    ss = rmsnorm_block_sum<NORM_THREADS>(ss, red);
    const float inv = rsqrtf(ss / (float)cols + eps);
    float amax = 0.f;
#pragma unroll
    for (int it = 0; it < NORM_MAX_VEC; ++it) {
        const int c = threadIdx.x + it * NORM_THREADS;
        if (c < nvec) {
            u32x4 o;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                o[i] = pack2<T>(v[it][2 * i] * inv * gm[it][2 * i], v[it][2 * i + 1] * inv * gm[it][2 * i + 1]);
            unpack8<T>(o, v[it]);                              // the rounded norm output, as the next kernel would read it
            amax = fmaxf(amax, smooth_absmax8(v[it], smooth, 8 * c));
        }
    }
    amax = block_max(amax, red);
    const float s = __fdiv_rn(amax, 127.0f);
    const float safe = s > 0.f ? s : 1.0f;
    if (threadIdx.x == 0) x_scale[blockIdx.x] = s;
#pragma unroll
    for (int it = 0; it < NORM_MAX_VEC; ++it) {
        const int c = threadIdx.x + it * NORM_THREADS;
        if (c < nvec) quant_store8(xq, v[it], safe, blockIdx.x, 8 * c, cols, gridDim.x, tiled);
    }
}

// act(gate) * up followed by the per-token quantisation of the product, which is not written.  One workgroup per
// row; rounding points as silu_mul_kernel has them.
template <typename T, int THREADS>
__global__ __launch_bounds__(THREADS) void silu_mul_quant_kernel(int8_t* __restrict__ xq, float* __restrict__ x_scale,
                                                                const uint16_t* __restrict__ gu,
                                                                const float* __restrict__ smooth_table, int cols,
                                                                int layout, int tiled, RowGroups rg) {
    __shared__ float red[THREADS / 64];
    const float* smooth = smooth_of_row(smooth_table, rg, blockIdx.x, cols);
    const int nvec = cols >> 3;
    constexpr int ROW_THREADS = THREADS;
    constexpr int MAXV = ROW_MAX_COLS / 8 / THREADS;
    float v[MAXV][8];
    float amax = 0.f;
    const uint16_t* base = gu + (int64_t)blockIdx.x * 2 * cols;
#pragma unroll
    for (int it = 0; it < MAXV; ++it) {
        const int cv = threadIdx.x + it * ROW_THREADS;
        if (cv < nvec) {
            const int c = 8 * cv;
            float g[8], u[8];
            if (layout == 0) {
                unpack8<T>(*(const u32x4*)(base + c), g);
                unpack8<T>(*(const u32x4*)(base + cols + c), u);
            } else {
                float a[8], b[8];
                unpack8<T>(*(const u32x4*)(base + 2 * c), a);
                unpack8<T>(*(const u32x4*)(base + 2 * c + 8), b);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    g[j] = a[2 * j]; u[j] = a[2 * j + 1];
                    g[4 + j] = b[2 * j]; u[4 + j] = b[2 * j + 1];
                }
            }
            u32x4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float a0 = T::to_float(T::from_float(silu_f(g[2 * j])));
                const float a1 = T::to_float(T::from_float(silu_f(g[2 * j + 1])));
                o[j] = pack2<T>(a0 * u[2 * j], a1 * u[2 * j + 1]);
            }
            unpack8<T>(o, v[it]);                              // the rounded product, as the next kernel would read it
            amax = fmaxf(amax, smooth_absmax8(v[it], smooth, c));
        }
    }
    amax = block_max(amax, red);
    const float s = __fdiv_rn(amax, 127.0f);
    const float safe = s > 0.f ? s : 1.0f;
    if (threadIdx.x == 0) x_scale[blockIdx.x] = s;
#pragma unroll
    for (int it = 0; it < MAXV; ++it) {
        const int cv = threadIdx.x + it * ROW_THREADS;
        if (cv < nvec) quant_store8(xq, v[it], safe, blockIdx.x, 8 * cv, cols, gridDim.x, tiled);
    }
}

}  // namespace

static int rmsnorm_entry(void* y, void* sum_out, const void* x, int64_t x_row_stride, const void* residual,
                         const void* gamma, float eps, int rows, int cols, int dtype, int gamma_dtype, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "rmsnorm: dtype must be bf16 or fp16");
    MF_REQUIRE(gamma_dtype == MF_BF16 || gamma_dtype == MF_FP16 || gamma_dtype == MF_FP32, "rmsnorm: bad gamma dtype");
    if (rows <= 0) return 0;
    MF_REQUIRE(y && x && gamma, "rmsnorm: null argument");
    MF_REQUIRE(!residual || sum_out, "rmsnorm: residual given without sum_out");
    MF_REQUIRE(cols > 0 && cols % 8 == 0 && cols <= NORM_THREADS * NORM_MAX_VEC * 8,
               "rmsnorm: cols (%d) must be a multiple of 8 and at most %d", cols, NORM_THREADS * NORM_MAX_VEC * 8);
    MF_REQUIRE(x_row_stride >= cols && x_row_stride % 8 == 0,
               "rmsnorm: the row stride of x (%lld) must be at least cols and a multiple of 8 elements",
               (long long)x_row_stride);
    MF_REQUIRE((((uintptr_t)y | (uintptr_t)x | (uintptr_t)residual | (uintptr_t)sum_out | (uintptr_t)gamma) & 15) == 0,
               "rmsnorm: pointers must be 16-byte aligned");
    if (dtype == MF_BF16)
        hipLaunchKernelGGL(rmsnorm_kernel<BF16>, dim3(rows), dim3(NORM_THREADS), 0, (hipStream_t)stream, (uint16_t*)y,
                           (uint16_t*)sum_out, (const uint16_t*)x, (const uint16_t*)residual, gamma, eps, cols,
                           gamma_dtype, x_row_stride);
    else
        hipLaunchKernelGGL(rmsnorm_kernel<FP16>, dim3(rows), dim3(NORM_THREADS), 0, (hipStream_t)stream, (uint16_t*)y,
                           (uint16_t*)sum_out, (const uint16_t*)x, (const uint16_t*)residual, gamma, eps, cols,
                           gamma_dtype, x_row_stride);
    return MF_LAUNCH_CHECK();
}

extern "C" int mf_rmsnorm(void* y, void* sum_out, const void* x, const void* residual, const void* gamma,
                          float eps, int rows, int cols, int dtype, int gamma_dtype, void* stream) {
    return rmsnorm_entry(y, sum_out, x, cols, residual, gamma, eps, rows, cols, dtype, gamma_dtype, stream);
}

extern "C" int mf_rmsnorm_strided(void* y, const void* x, int64_t x_row_stride, const void* gamma, float eps, int rows,
                                  int cols, int dtype, int gamma_dtype, void* stream) {
    return rmsnorm_entry(y, nullptr, x, x_row_stride, nullptr, gamma, eps, rows, cols, dtype, gamma_dtype, stream);
}

extern "C" int mf_silu_mul(void* out, const void* gate_up, int rows, int cols, int layout, int dtype,
                           void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "silu_mul: dtype must be bf16 or fp16");
    if (rows <= 0) return 0;
    MF_REQUIRE(out && gate_up, "silu_mul: null argument");
    MF_REQUIRE(layout == 0 || layout == 1, "silu_mul: layout must be 0 (halves) or 1 (interleaved)");
    MF_REQUIRE(cols > 0 && cols % 8 == 0, "silu_mul: cols (%d) must be a multiple of 8", cols);
    MF_REQUIRE((((uintptr_t)out | (uintptr_t)gate_up) & 15) == 0, "silu_mul: pointers must be 16-byte aligned");
    if (rows <= 0) return 0;
    const int64_t nvec = (int64_t)rows * (cols / 8);
    const int blocks = (int)min((int64_t)8192, (nvec + 255) / 256);
    if (dtype == MF_BF16)
        hipLaunchKernelGGL(silu_mul_kernel<BF16>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (uint16_t*)out,
                           (const uint16_t*)gate_up, rows, cols, layout);
    else
        hipLaunchKernelGGL(silu_mul_kernel<FP16>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (uint16_t*)out,
                           (const uint16_t*)gate_up, rows, cols, layout);
    return MF_LAUNCH_CHECK();
}

extern "C" int mf_add(void* out, const void* a, const void* b, int64_t n, int dtype, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "add: dtype must be bf16 or fp16");
    if (n <= 0) return 0;
    MF_REQUIRE(out && a && b, "add: null argument");
    MF_REQUIRE((((uintptr_t)out | (uintptr_t)a | (uintptr_t)b) & 15) == 0, "add: pointers must be 16-byte aligned");
    if (n <= 0) return 0;
    const int blocks = (int)min((int64_t)8192, (n / 8 + 256) / 256);
    if (dtype == MF_BF16)
        hipLaunchKernelGGL(add_kernel<BF16>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (uint16_t*)out,
                           (const uint16_t*)a, (const uint16_t*)b, n);
    else
        hipLaunchKernelGGL(add_kernel<FP16>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (uint16_t*)out,
                           (const uint16_t*)a, (const uint16_t*)b, n);
    return MF_LAUNCH_CHECK();
}

extern "C" int mf_scale_columns(void* out, const void* x, const float* scale, int64_t rows, int cols, int dtype,
                                void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "scale_columns: dtype must be bf16 or fp16");
    MF_REQUIRE(rows >= 0 && cols > 0 && cols % 8 == 0, "scale_columns: cols (%d) must be a positive multiple of 8", cols);
    if (rows == 0) return 0;
    MF_REQUIRE(out && x && scale, "scale_columns: null argument");
    MF_REQUIRE((((uintptr_t)out | (uintptr_t)x | (uintptr_t)scale) & 15) == 0, "scale_columns: 16-byte alignment");
    const int64_t nvec = rows * (cols >> 3);
    const int blocks = (int)std::min<int64_t>((nvec + 255) / 256, 65535);
    if (dtype == MF_BF16)
        hipLaunchKernelGGL(scale_columns_kernel<BF16>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (uint16_t*)out,
                           (const uint16_t*)x, scale, rows, cols);
    else
        hipLaunchKernelGGL(scale_columns_kernel<FP16>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (uint16_t*)out,
                           (const uint16_t*)x, scale, rows, cols);
    return MF_LAUNCH_CHECK();
}

static int quant_rows_entry(int8_t* xq, float* x_scale, const void* x, const float* smooth, const float* static_scale,
                            int m, int k, int dtype, int layout, void* stream, const int32_t* group_offsets = nullptr,
                            int groups = 0);

extern "C" int mf_dynamic_quant_per_token(int8_t* xq, float* x_scale, const void* x, const float* smooth, int m,
                                          int k, int dtype, int layout, void* stream) {
    return quant_rows_entry(xq, x_scale, x, smooth, nullptr, m, k, dtype, layout, stream);
}

extern "C" int mf_static_quant_per_tensor(int8_t* xq, float* x_scale, const void* x, const float* smooth,
                                          const float* act_scale, int m, int k, int dtype, int layout, void* stream) {
    MF_REQUIRE(act_scale != nullptr, "static_quant: null activation scale");
    return quant_rows_entry(xq, x_scale, x, smooth, act_scale, m, k, dtype, layout, stream);
}

static int quant_rows_entry(int8_t* xq, float* x_scale, const void* x, const float* smooth, const float* static_scale,
                            int m, int k, int dtype, int layout, void* stream, const int32_t* group_offsets, int groups) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "dynamic_quant: dtype must be bf16 or fp16");
    MF_REQUIRE(!group_offsets || groups > 0, "dynamic_quant: a group table needs groups > 0");
    const RowGroups rg = {group_offsets, groups};
    MF_REQUIRE(layout == 0 || layout == 1, "dynamic_quant: layout must be 0 (row-major) or 1 (tiled)");
    if (m <= 0) return 0;
    MF_REQUIRE(xq && x_scale && x, "dynamic_quant: null argument");
    MF_REQUIRE(k > 0 && k % 8 == 0 && k <= ROW_MAX_COLS, "dynamic_quant: k (%d) must be a multiple of 8, <= %d", k,
               ROW_MAX_COLS);
    MF_REQUIRE((((uintptr_t)xq & 7) | ((uintptr_t)x & 15) | ((uintptr_t)smooth & 15)) == 0,
               "dynamic_quant: x/smooth must be 16-byte aligned, xq 8-byte aligned");
    if (m <= 0) return 0;
#define DQ_LAUNCH(TT, TH)                                                                                        \
    hipLaunchKernelGGL((dynamic_quant_kernel<TT, TH>), dim3(m), dim3(TH), 0, (hipStream_t)stream, xq, x_scale,    \
                       (const uint16_t*)x, smooth, k, layout, static_scale, rg)
    const bool wide = k > 4096;
    if (dtype == MF_BF16) {
        if (wide) DQ_LAUNCH(BF16, ROW_THREADS_WIDE); else DQ_LAUNCH(BF16, ROW_THREADS);
    } else {
        if (wide) DQ_LAUNCH(FP16, ROW_THREADS_WIDE); else DQ_LAUNCH(FP16, ROW_THREADS);
    }
#undef DQ_LAUNCH
    return MF_LAUNCH_CHECK();
}

extern "C" int mf_rmsnorm_dynamic_quant(int8_t* xq, float* x_scale, void* sum_out, const void* x, const void* residual,
                                        const void* gamma, const float* smooth, float eps, int rows, int cols,
                                        int dtype, int gamma_dtype, int layout, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "rmsnorm_dynamic_quant: dtype must be bf16 or fp16");
    MF_REQUIRE(gamma_dtype == MF_BF16 || gamma_dtype == MF_FP16 || gamma_dtype == MF_FP32,
               "rmsnorm_dynamic_quant: bad gamma dtype");
    MF_REQUIRE(layout == 0 || layout == 1, "rmsnorm_dynamic_quant: layout must be 0 (row-major) or 1 (tiled)");
    if (rows <= 0) return 0;
    MF_REQUIRE(xq && x_scale && x && gamma, "rmsnorm_dynamic_quant: null argument");
    MF_REQUIRE(!residual || sum_out, "rmsnorm_dynamic_quant: residual given without sum_out");
    MF_REQUIRE(cols > 0 && cols % 8 == 0 && cols <= NORM_THREADS * NORM_MAX_VEC * 8,
               "rmsnorm_dynamic_quant: cols (%d) must be a multiple of 8 and at most %d", cols,
               NORM_THREADS * NORM_MAX_VEC * 8);
    MF_REQUIRE((((uintptr_t)x | (uintptr_t)residual | (uintptr_t)sum_out | (uintptr_t)gamma | (uintptr_t)smooth) & 15) == 0 &&
                   ((uintptr_t)xq & 7) == 0,
               "rmsnorm_dynamic_quant: pointers must be 16-byte aligned, xq 8-byte aligned");
    const PartialRow none = {nullptr, nullptr, nullptr, nullptr, 0};
    if (dtype == MF_BF16)
        hipLaunchKernelGGL((rmsnorm_quant_kernel<BF16, false>), dim3(rows), dim3(NORM_THREADS), 0, (hipStream_t)stream, xq,
                           x_scale, (uint16_t*)sum_out, (const uint16_t*)x, (const uint16_t*)residual, gamma, smooth, eps,
                           cols, gamma_dtype, layout, none);
    else
        hipLaunchKernelGGL((rmsnorm_quant_kernel<FP16, false>), dim3(rows), dim3(NORM_THREADS), 0, (hipStream_t)stream, xq,
                           x_scale, (uint16_t*)sum_out, (const uint16_t*)x, (const uint16_t*)residual, gamma, smooth, eps,
                           cols, gamma_dtype, layout, none);
    return MF_LAUNCH_CHECK();
}

// The same kernel fed from the int32 split-K partial sums of an int8 GEMM (called by that GEMM's launcher; arguments
// checked there).
int mf_detail_rmsnorm_quant_from_partial(int8_t* xq, float* x_scale, void* sum_out, const int32_t* partial, int split_k,
                                         const float* row_scale, const float* col_scale, const void* bias,
                                         const void* residual, const void* gamma, const float* smooth, float eps,
                                         int rows, int cols, int dtype, int gamma_dtype, int layout, void* stream) {
    const PartialRow pr = {partial, row_scale, col_scale, (const uint16_t*)bias, split_k};
    if (dtype == MF_BF16)
        hipLaunchKernelGGL((rmsnorm_quant_kernel<BF16, true>), dim3(rows), dim3(NORM_THREADS), 0, (hipStream_t)stream, xq,
                           x_scale, (uint16_t*)sum_out, nullptr, (const uint16_t*)residual, gamma, smooth, eps, cols,
                           gamma_dtype, layout, pr);
    else
        hipLaunchKernelGGL((rmsnorm_quant_kernel<FP16, true>), dim3(rows), dim3(NORM_THREADS), 0, (hipStream_t)stream, xq,
                           x_scale, (uint16_t*)sum_out, nullptr, (const uint16_t*)residual, gamma, smooth, eps, cols,
                           gamma_dtype, layout, pr);
    return MF_LAUNCH_CHECK();
}

static int silu_mul_quant_entry(int8_t* xq, float* x_scale, const void* gate_up, const float* smooth, int rows,
                               int cols, int gate_up_layout, int dtype, int layout, void* stream,
                               const int32_t* group_offsets, int groups) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "silu_mul_dynamic_quant: dtype must be bf16 or fp16");
    MF_REQUIRE(!group_offsets || groups > 0, "silu_mul_dynamic_quant: a group table needs groups > 0");
    const RowGroups rg = {group_offsets, groups};
    MF_REQUIRE(gate_up_layout == 0 || gate_up_layout == 1,
               "silu_mul_dynamic_quant: gate_up_layout must be 0 (halves) or 1 (interleaved)");
    MF_REQUIRE(layout == 0 || layout == 1, "silu_mul_dynamic_quant: layout must be 0 (row-major) or 1 (tiled)");
    if (rows <= 0) return 0;
    MF_REQUIRE(xq && x_scale && gate_up, "silu_mul_dynamic_quant: null argument");
    MF_REQUIRE(cols > 0 && cols % 8 == 0 && cols <= ROW_MAX_COLS,
               "silu_mul_dynamic_quant: cols (%d) must be a multiple of 8, <= %d", cols, ROW_MAX_COLS);
    MF_REQUIRE((((uintptr_t)gate_up | (uintptr_t)smooth) & 15) == 0 && ((uintptr_t)xq & 7) == 0,
               "silu_mul_dynamic_quant: gate_up/smooth must be 16-byte aligned, xq 8-byte aligned");
#define SQ_LAUNCH(TT, TH)                                                                                        \
    hipLaunchKernelGGL((silu_mul_quant_kernel<TT, TH>), dim3(rows), dim3(TH), 0, (hipStream_t)stream, xq, x_scale, \
                       (const uint16_t*)gate_up, smooth, cols, gate_up_layout, layout, rg)
    const bool wide = cols > 4096;
    if (dtype == MF_BF16) {
        if (wide) SQ_LAUNCH(BF16, ROW_THREADS_WIDE); else SQ_LAUNCH(BF16, ROW_THREADS);
    } else {
        if (wide) SQ_LAUNCH(FP16, ROW_THREADS_WIDE); else SQ_LAUNCH(FP16, ROW_THREADS);
    }
#undef SQ_LAUNCH
    return MF_LAUNCH_CHECK();
}

extern "C" int mf_silu_mul_dynamic_quant(int8_t* xq, float* x_scale, const void* gate_up, const float* smooth, int rows,
                                         int cols, int gate_up_layout, int dtype, int layout, void* stream) {
    return silu_mul_quant_entry(xq, x_scale, gate_up, smooth, rows, cols, gate_up_layout, dtype, layout, stream, nullptr, 0);
}

extern "C" int mf_grouped_dynamic_quant_per_token(int8_t* xq, float* x_scale, const void* x, const float* smooth,
                                                  const int32_t* offsets, int n_experts, int m, int k, int dtype,
                                                  int layout, void* stream) {
    MF_REQUIRE(smooth && offsets && n_experts > 0, "grouped_dynamic_quant: smooth [n_experts, k] and offsets are needed");
    return quant_rows_entry(xq, x_scale, x, smooth, nullptr, m, k, dtype, layout, stream, offsets, n_experts);
}

extern "C" int mf_grouped_silu_mul_dynamic_quant(int8_t* xq, float* x_scale, const void* gate_up, const float* smooth,
                                                 const int32_t* offsets, int n_experts, int rows, int cols,
                                                 int gate_up_layout, int dtype, int layout, void* stream) {
    MF_REQUIRE(smooth && offsets && n_experts > 0, "grouped_silu_mul_dynamic_quant: smooth [n_experts, cols] and offsets are needed");
    return silu_mul_quant_entry(xq, x_scale, gate_up, smooth, rows, cols, gate_up_layout, dtype, layout, stream, offsets,
                                n_experts);
}
