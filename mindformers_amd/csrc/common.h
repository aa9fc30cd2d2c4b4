// Shared device helpers for the gfx950 decode kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <utility>
#include <type_traits>

#include "../../include/mf_decode.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(16))) int i32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define MF_WAVE 64
#define MF_MAX_DEVICES 64                 // per-device one-off kernel configuration flags
// The packed int8 operand format shared by both GEMM families (and by mf_w8a16_packed_bytes, which sizes it for
// either): 1 KiB tiles of 16 rows x 64 columns.  Each family names the two constants its own way and asserts them
// against these.
constexpr int MF_PACK_KSTEP = 64;
constexpr int MF_PACK_TILE_BYTES = 16 * MF_PACK_KSTEP;

// Host-side argument error: remember the message, return hipErrorInvalidValue.
void mf_set_error(const char* fmt, ...);
#define MF_REQUIRE(cond, ...)                         \
    do {                                              \
        if (!(cond)) {                                \
            mf_set_error(__VA_ARGS__);                \
            return (int)hipErrorInvalidValue;         \
        }                                             \
    } while (0)

#define MF_LAUNCH_CHECK() ((int)hipGetLastError())

// ---- element types ---------------------------------------------------------------------------------
struct BF16 {
    using vec8 = bf16x8;
    static constexpr int id = MF_BF16;
    static __device__ __forceinline__ float to_float(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }
    static __device__ __forceinline__ uint16_t from_float(float f) {
        return __builtin_bit_cast(uint16_t, (__bf16)f);       // v_cvt_pk_bf16_f32: round to nearest even
    }
    static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    // 32x32x16: twice the work of the 16x16x32 instruction in the same issue time
    static __device__ __forceinline__ f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    // the same with the accumulator held in the accumulation registers (the compiler is not told that this is a
    // matrix instruction: a reader of c other than the next such statement has to wait for its 16 passes itself)
    static __device__ __forceinline__ void mfma32_acc(f32x16& c, vec8 a, vec8 b) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
    // likewise with the accumulator in ordinary registers: c = a b, then c += a b
    static __device__ __forceinline__ void mfma32_first(f32x16& c, vec8 a, vec8 b) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ void mfma32_next(f32x16& c, vec8 a, vec8 b) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
    }
    // c + both halves of a packed pair, in fp32 (one dot-product instruction)
    static __device__ __forceinline__ float sum2(uint32_t pair, float c) {
        typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_v;
        const bf16x2_v one = {(__bf16)1.0f, (__bf16)1.0f};
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_v, pair), one, c, false);
    }
};

struct FP16 {
    using vec8 = f16x8;
    static constexpr int id = MF_FP16;
    static __device__ __forceinline__ float to_float(uint16_t b) {
        union { uint16_t u; _Float16 h; } c; c.u = b; return (float)c.h;
    }
    static __device__ __forceinline__ uint16_t from_float(float f) {
        union { uint16_t u; _Float16 h; } c; c.h = (_Float16)f; return c.u;   // v_cvt_f16_f32: RNE
    }
    static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ void mfma32_acc(f32x16& c, vec8 a, vec8 b) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ void mfma32_first(f32x16& c, vec8 a, vec8 b) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ void mfma32_next(f32x16& c, vec8 a, vec8 b) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ float sum2(uint32_t pair, float c) {
        typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_v;
        const f16x2_v one = {(_Float16)1.0f, (_Float16)1.0f};
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_v, pair), one, c, false);
    }
};

template <typename T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    return (uint32_t)T::from_float(lo) | ((uint32_t)T::from_float(hi) << 16);
}
template <>
__device__ __forceinline__ uint32_t pack2<BF16>(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) float f32x2_t;
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2_t){lo, hi}, bf16x2_t));   // one instruction
}

template <typename T>
__device__ __forceinline__ void unpack8(const u32x4& v, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = T::to_float((uint16_t)(v[i] & 0xffffu));
        f[2 * i + 1] = T::to_float((uint16_t)(v[i] >> 16));
    }
}

// value of a float-like table entry by runtime dtype id (used for cos/sin/gamma that may be fp32)
__device__ __forceinline__ float load_as_float(const void* p, int64_t i, int dt) {
    if (dt == MF_FP32) return ((const float*)p)[i];
    uint16_t b = ((const uint16_t*)p)[i];
    return dt == MF_BF16 ? BF16::to_float(b) : FP16::to_float(b);
}

// 8 consecutive entries of a float-like table (runtime dtype id) as floats; 16-byte aligned
__device__ __forceinline__ void load8_as_float(const void* p, int64_t i, int dt, float* f) {
    if (dt == MF_FP32) {
        const f32x4 a = *(const f32x4*)((const float*)p + i), b = *(const f32x4*)((const float*)p + i + 4);
#pragma unroll
        for (int q = 0; q < 4; ++q) { f[q] = a[q]; f[4 + q] = b[q]; }
    } else {
        const u32x4 v = *(const u32x4*)((const uint16_t*)p + i);
        if (dt == MF_BF16) unpack8<BF16>(v, f); else unpack8<FP16>(v, f);
    }
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Sum over a workgroup of THREADS threads (wave sums, then the waves in order): the one reduction tree that every
// RMSNorm-carrying kernel uses, so that fused and unfused paths agree to the bit.  ``red`` holds THREADS/64 floats.
template <int THREADS>
__device__ __forceinline__ float rmsnorm_block_sum(float v, float* red) {
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < THREADS / 64; ++i) t += red[i];
    return t;
}

// Rotate-half pair (x1 at i, x2 at i + D/2) with separately rounded operations, shared by every kernel that
// applies RoPE so that fused and unfused paths agree to the bit.
__device__ __forceinline__ void rope_pair(float x1, float x2, float c1, float s1, float c2, float s2, float& o1,
                                          float& o2) {
    o1 = __fsub_rn(__fmul_rn(x1, c1), __fmul_rn(x2, s1));
    o2 = __fadd_rn(__fmul_rn(x2, c2), __fmul_rn(x1, s2));
}

// Maximum over the workgroup (red: one float per wave of shared memory); every thread gets the result.
__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float t = red[0];
    for (int i = 1; i < (int)(blockDim.x >> 6); ++i) t = fmaxf(t, red[i]);
    __syncthreads();
    return t;
}


// 8 values of row m, columns k .. k+7, quantised with the row's scale and written in the chosen layout.
// The division is a true IEEE division so that the grid point chosen equals the CPU statement.
__device__ __forceinline__ void quant_store8(int8_t* __restrict__ xq, const float* v, float safe, int m, int k, int cols,
                                             int rows, int tiled) {
    uint32_t o[2] = {0u, 0u};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float qf = rintf(__fdiv_rn(v[i], safe));
        qf = fminf(fmaxf(qf, -128.f), 127.f);
        o[i >> 2] |= ((uint32_t)((int)qf & 0xff)) << (8 * (i & 3));
    }
    if (tiled) {
        // 1 KiB tiles of 16 rows x 64 columns, [column step][row tile], 16 consecutive columns per lane
        // (lane = 16*(column/16 % 4) + row % 16): the operand order of the int8 matrix instructions
        const int64_t tile = (int64_t)(k >> 6) * ((rows + 15) >> 4) + (m >> 4);
        *(u32x2*)(xq + tile * 1024 + ((((k & 63) >> 4) << 4) + (m & 15)) * 16 + (k & 15)) = (u32x2){o[0], o[1]};
    } else {
        *(u32x2*)(xq + (int64_t)m * cols + k) = (u32x2){o[0], o[1]};
    }
}
// x * smooth in place (smooth may be null), returns max |.| of the 8 values
__device__ __forceinline__ float smooth_absmax8(float* v, const float* __restrict__ smooth, int k) {
    if (smooth) {
        const f32x4 s0 = *(const f32x4*)(smooth + k), s1 = *(const f32x4*)(smooth + k + 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[i] = __fmul_rn(v[i], s0[i]);
            v[4 + i] = __fmul_rn(v[4 + i], s1[i]);
        }
    }
    float a = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) a = fmaxf(a, fabsf(v[i]));
    return a;
}

// Launcher shared between source files, not part of the C ABI: the RMSNorm + per-token quantisation kernel fed from
// the int32 split-K partial sums of an int8 GEMM (rows x cols, split_k slabs; row_scale / col_scale / bias
// dequantise the sums; residual, sum_out, gamma, smooth, layout as in mf_rmsnorm_dynamic_quant).
__attribute__((visibility("hidden"))) int mf_detail_rmsnorm_quant_from_partial(
    int8_t* xq, float* x_scale, void* sum_out, const int32_t* partial, int split_k, const float* row_scale,
    const float* col_scale, const void* bias, const void* residual, const void* gamma, const float* smooth, float eps,
    int rows, int cols, int dtype, int gamma_dtype, int layout, void* stream);

// Eight cache elements quantised as the int8 KV scatter defines them: clip(rint(x / scale + offset), -128, 127),
// the quotient in double so that the rounding does not depend on how a float division is lowered; shared by the
// stand-alone scatter kernel's fused counterparts.  v holds values already rounded to the activation type.
__device__ __forceinline__ u32x2 quant8_for_cache(const float* v, const float* __restrict__ sc,
                                                  const float* __restrict__ of) {
    uint32_t w[2] = {0u, 0u};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const double q = (double)v[i] / (double)sc[i] + (of ? (double)of[i] : 0.0);
        const int b = (int)fmin(fmax(rint(q), -128.0), 127.0);
        w[i >> 2] |= (uint32_t)(b & 0xff) << (8 * (i & 3));
    }
    return (u32x2){w[0], w[1]};
}

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + __expf(-x)); }

template <typename V, typename U>
__device__ __forceinline__ V bitcast(const U& u) {
    static_assert(sizeof(V) == sizeof(U), "size mismatch");
    V v;
    __builtin_memcpy(&v, &u, sizeof(V));
    return v;
}

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

// 8 unsigned nibbles holding q + 8 (q in -8 .. 7; nibble i = element i) -> 8 elements of T, exact.
template <typename T>
__device__ __forceinline__ typename T::vec8 dequant8_u4(uint32_t w);

template <>
__device__ __forceinline__ bf16x8 dequant8_u4<BF16>(uint32_t w) {
    const uint32_t even = w & 0x0f0f0f0fu, odd = (w >> 4) & 0x0f0f0f0fu;   // elements 0 2 4 6 / 1 3 5 7 as bytes
    u32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float f0 = (float)((even >> (8 * i)) & 0xffu) - 8.0f;
        const float f1 = (float)((odd >> (8 * i)) & 0xffu) - 8.0f;
        v[i] = __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);   // high halves: exact
    }
    return bitcast<bf16x8>(v);
}
template <>
__device__ __forceinline__ f16x8 dequant8_u4<FP16>(uint32_t w) {
    f16x8 v;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (_Float16)((float)((w >> (4 * i)) & 0xfu) - 8.0f);
    return v;
}

// Transposing 64-bit LDS read (ds_read_b64_tr_b16).  Within every group of 16 lanes, lane j names four consecutive
// 16-bit values M[j][0..3]; lane i receives M[(i >> 2) + 4 e][i & 3] for e = 0..3.
typedef __attribute__((ext_vector_type(4))) short s16x4;
__device__ __forceinline__ s16x4 lds_read_tr16(const uint8_t* p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p);
}

// ---- pieces of hand-scheduled inner loops: LDS reads issued as asm statements (the compiler neither moves them nor
// waits for them), the counted wait that makes the oldest of them valid, and a compile-time loop whose index can
// select immediate offsets
template <int OFF>
__device__ __forceinline__ u32x4 lds_read16_at(uint32_t addr) {
    static_assert(OFF >= 0 && OFF < 65536, "LDS offset field");
    u32x4 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(v) : "v"(addr), "n"(OFF) : "memory");
    return v;
}
template <int OFF>
__device__ __forceinline__ u32x2 lds_read_tr16_at(uint32_t addr) {
    static_assert(OFF >= 0 && OFF < 65536, "LDS offset field");
    u32x2 v;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=&v"(v) : "v"(addr), "n"(OFF) : "memory");
    return v;
}
template <int N>
__device__ __forceinline__ void wait_lds_reads() {
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N) : "memory");
    __builtin_amdgcn_sched_barrier(0);
}
// maximum of a value over the two lanes l and l ^ 32 (the instruction swaps the upper half of its first operand with
// the lower half of its second)
__device__ __forceinline__ float max_xor32(float v) {
    float a = v, b = v;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return fmaxf(a, b);
}
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

