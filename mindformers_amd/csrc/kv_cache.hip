// KV-cache scatter (reshape_and_cache), rotate-half RoPE, and the two fused.
//
// All three are tiny HBM-bound copies: a decode step moves num_tokens * n_kv * head_dim * 2 elements.
// Rows are moved with 16-byte lane accesses, one workgroup per token row.
#include "common.h"

namespace {

// One workgroup per (token, k-or-v).  row_elems = n_kv * head_dim.
template <int VEC_BYTES>
__global__ void reshape_and_cache_kernel(const uint8_t* __restrict__ key, const uint8_t* __restrict__ value,
                                         uint8_t* __restrict__ key_cache, uint8_t* __restrict__ value_cache,
                                         const int32_t* __restrict__ slot_mapping, int row_bytes,
                                         int64_t num_slots, int64_t key_stride_bytes,
                                         int64_t value_stride_bytes) {
    const int t = blockIdx.x;
    const int64_t slot = slot_mapping[t];
    if (slot < 0 || slot >= num_slots) return;  // padding (or a corrupt slot: never write out of bounds)
    const uint8_t* src = blockIdx.y == 0 ? key + (int64_t)t * key_stride_bytes : value + (int64_t)t * value_stride_bytes;
    uint8_t* dst = (blockIdx.y == 0 ? key_cache : value_cache) + slot * (int64_t)row_bytes;
    if (VEC_BYTES == 16) {
        for (int i = threadIdx.x * 16; i < row_bytes; i += blockDim.x * 16)
            *(u32x4*)(dst + i) = *(const u32x4*)(src + i);
    } else {
        for (int i = threadIdx.x * 2; i < row_bytes; i += blockDim.x * 2)
            *(uint16_t*)(dst + i) = *(const uint16_t*)(src + i);
    }
}

// rotate-half on one [heads, D] row; thread p handles the pair (i, i + D/2) of head h.
template <typename T>
__device__ __forceinline__ void rope_row(uint16_t* x, int n_heads, int D, const void* cos, const void* sin,
                                         int64_t table_row, int table_dtype, uint16_t* scatter_dst) {
    const int half = D >> 1;
    for (int p = threadIdx.x; p < n_heads * half; p += blockDim.x) {
        const int h = p / half, i = p - h * half;
        uint16_t* xr = x + h * D;
        const float x1 = T::to_float(xr[i]), x2 = T::to_float(xr[i + half]);
        const float c1 = load_as_float(cos, table_row + i, table_dtype);
        const float s1 = load_as_float(sin, table_row + i, table_dtype);
        const float c2 = load_as_float(cos, table_row + i + half, table_dtype);
        const float s2 = load_as_float(sin, table_row + i + half, table_dtype);
        float r1, r2;
        rope_pair(x1, x2, c1, s1, c2, s2, r1, r2);
        const uint16_t o1 = T::from_float(r1), o2 = T::from_float(r2);
        xr[i] = o1;
        xr[i + half] = o2;
        if (scatter_dst) {
            scatter_dst[h * D + i] = o1;
            scatter_dst[h * D + i + half] = o2;
        }
    }
}

template <typename T>
__global__ void rope_kernel(uint16_t* __restrict__ q, uint16_t* __restrict__ k, const void* __restrict__ cos,
                            const void* __restrict__ sin, int n_heads, int n_kv, int D, int table_dtype,
                            int64_t q_stride, int64_t k_stride) {
    const int t = blockIdx.x;
    const int64_t trow = (int64_t)t * D;
    rope_row<T>(q + (int64_t)t * q_stride, n_heads, D, cos, sin, trow, table_dtype, nullptr);
    if (k) rope_row<T>(k + (int64_t)t * k_stride, n_kv, D, cos, sin, trow, table_dtype, nullptr);
}

template <typename T>
__global__ void rope_and_cache_kernel(uint16_t* __restrict__ q, uint16_t* __restrict__ k,
                                      const uint16_t* __restrict__ v, const void* __restrict__ cos,
                                      const void* __restrict__ sin, uint16_t* __restrict__ key_cache,
                                      uint16_t* __restrict__ value_cache,
                                      const int32_t* __restrict__ slot_mapping, int n_heads, int n_kv, int D,
                                      int64_t num_slots, int table_dtype, int64_t q_stride, int64_t k_stride,
                                      int64_t v_stride, int vec_ok) {
    const int t = blockIdx.x;
    const int64_t trow = (int64_t)t * D;
    const int64_t slot = slot_mapping[t];
    const bool live = slot >= 0 && slot < num_slots;
    const int row = n_kv * D;
    rope_row<T>(q + (int64_t)t * q_stride, n_heads, D, cos, sin, trow, table_dtype, nullptr);
    rope_row<T>(k + (int64_t)t * k_stride, n_kv, D, cos, sin, trow, table_dtype,
                live ? key_cache + slot * row : nullptr);
    if (live) {
        const uint16_t* src = v + (int64_t)t * v_stride;
        uint16_t* dst = value_cache + slot * row;
        if (vec_ok) {
            for (int i = threadIdx.x * 8; i < row; i += blockDim.x * 8)
                *(u32x4*)(dst + i) = *(const u32x4*)(src + i);
        } else {
            for (int i = threadIdx.x; i < row; i += blockDim.x) dst[i] = src[i];
        }
    }
}

// Vector form of the fused rotate-and-scatter for head_dim % 16 == 0: one work item = 8 consecutive elements
// of the first half of a head together with their partners in the second half (16-byte accesses), or one
// 16-byte piece of the value row.  grid = (tokens, ceil(items / 256)).
template <typename T>
__global__ __launch_bounds__(256) void rope_and_cache_vec_kernel(
    uint16_t* __restrict__ q, uint16_t* __restrict__ k, const uint16_t* __restrict__ v, const void* __restrict__ cos,
    const void* __restrict__ sin, uint16_t* __restrict__ key_cache, uint16_t* __restrict__ value_cache,
    const int32_t* __restrict__ slot_mapping, int n_heads, int n_kv, int D, int64_t num_slots, int table_dtype,
    int64_t q_stride, int64_t k_stride, int64_t v_stride) {
    const int t = blockIdx.x;
    const int half = D >> 1;
    const int cph = half >> 3;                                // rotate items per head
    const int rot_items = (n_heads + n_kv) * cph;
    const int v_items = n_kv * D / 8;
    const int item = blockIdx.y * 256 + threadIdx.x;
    if (item >= rot_items + v_items) return;
    const int64_t slot = slot_mapping[t];
    const bool live = slot >= 0 && slot < num_slots;
    const int64_t row = (int64_t)n_kv * D;
    if (item >= rot_items) {
        if (live) {
            const int i = (item - rot_items) * 8;
            *(u32x4*)(value_cache + slot * row + i) = *(const u32x4*)(v + (int64_t)t * v_stride + i);
        }
        return;
    }
    const int h = item / cph, i = (item - h * cph) * 8;
    const bool is_k = h >= n_heads;
    uint16_t* xr = is_k ? k + (int64_t)t * k_stride + (h - n_heads) * D : q + (int64_t)t * q_stride + h * D;
    float x1[8], x2[8], c1[8], s1[8], c2[8], s2[8];
    unpack8<T>(*(const u32x4*)(xr + i), x1);
    unpack8<T>(*(const u32x4*)(xr + i + half), x2);
    const int64_t trow = (int64_t)t * D;
    load8_as_float(cos, trow + i, table_dtype, c1);
    load8_as_float(sin, trow + i, table_dtype, s1);
    load8_as_float(cos, trow + i + half, table_dtype, c2);
    load8_as_float(sin, trow + i + half, table_dtype, s2);
    u32x4 o1, o2;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float a0, b0, a1, b1;
        rope_pair(x1[2 * e], x2[2 * e], c1[2 * e], s1[2 * e], c2[2 * e], s2[2 * e], a0, b0);
        rope_pair(x1[2 * e + 1], x2[2 * e + 1], c1[2 * e + 1], s1[2 * e + 1], c2[2 * e + 1], s2[2 * e + 1], a1, b1);
        o1[e] = pack2<T>(a0, a1);
        o2[e] = pack2<T>(b0, b1);
    }
    *(u32x4*)(xr + i) = o1;
    *(u32x4*)(xr + i + half) = o2;
    if (is_k && live) {
        uint16_t* dst = key_cache + slot * row + (h - n_heads) * D;
        *(u32x4*)(dst + i) = o1;
        *(u32x4*)(dst + i + half) = o2;
    }
}

// Quantize-and-scatter for int8 caches: cache[slot][c] = clip(rint(x[c] / scale[c] + offset[c]), -128, 127), the
// quotient in double so that the rounding does not depend on how a float division is lowered.  One thread per
// element; grid (tokens, 2): y = 0 keys, y = 1 values; scale / offset are [2][row].
template <typename T>
__global__ void quant_reshape_and_cache_kernel(const uint16_t* __restrict__ key, const uint16_t* __restrict__ value,
                                               int8_t* __restrict__ key_cache, int8_t* __restrict__ value_cache,
                                               const int32_t* __restrict__ slot_mapping,
                                               const float* __restrict__ scale, const float* __restrict__ offset,
                                               int row, int64_t num_slots, int64_t k_stride, int64_t v_stride) {
    const int t = blockIdx.x, which = blockIdx.y;
    const int64_t slot = slot_mapping[t];
    if (slot < 0 || slot >= num_slots) return;
    const uint16_t* src = which ? value + (int64_t)t * v_stride : key + (int64_t)t * k_stride;
    int8_t* dst = (which ? value_cache : key_cache) + slot * row;
    const float* sc = scale + which * row;
    const float* of = offset ? offset + which * row : nullptr;
    for (int c = threadIdx.x; c < row; c += blockDim.x) {
        const double q = (double)T::to_float(src[c]) / (double)sc[c] + (of ? (double)of[c] : 0.0);
        dst[c] = (int8_t)fmin(fmax(rint(q), -128.0), 127.0);
    }
}

// Per-token int8 cache write: the row of all kv heads of a token is quantised as the per-token dynamic
// quantisation defines it (s = max|row| / 127 in float32, q = clip(rint(x / s), -128, 127) with a true float32
// division; a zero row gets s = 0 and zeros), the int8 row goes to the token's slot and s to the same slot of the
// scale cache.  grid (tokens, 2): y = 0 keys, y = 1 values.
template <typename T>
__global__ __launch_bounds__(256) void dynamic_quant_reshape_and_cache_kernel(
    const uint16_t* __restrict__ key, const uint16_t* __restrict__ value, int8_t* __restrict__ key_cache,
    int8_t* __restrict__ value_cache, float* __restrict__ key_scale_cache, float* __restrict__ value_scale_cache,
    const int32_t* __restrict__ slot_mapping, int row, int64_t num_slots, int64_t k_stride, int64_t v_stride) {
    __shared__ float red[4];
    const int t = blockIdx.x, which = blockIdx.y;
    const int64_t slot = slot_mapping[t];
    if (slot < 0 || slot >= num_slots) return;                // uniform over the workgroup
    const uint16_t* src = which ? value + (int64_t)t * v_stride : key + (int64_t)t * k_stride;
    int8_t* dst = (which ? value_cache : key_cache) + slot * row;
    float amax = 0.f;
    for (int c = threadIdx.x; c < row; c += blockDim.x) amax = fmaxf(amax, fabsf(T::to_float(src[c])));
    amax = block_max(amax, red);
    const float s = __fdiv_rn(amax, 127.0f);
    const float safe = s > 0.f ? s : 1.0f;
    if (threadIdx.x == 0) (which ? value_scale_cache : key_scale_cache)[slot] = s;
    for (int c = threadIdx.x; c < row; c += blockDim.x) {
        const float q = rintf(__fdiv_rn(T::to_float(src[c]), safe));
        dst[c] = (int8_t)fminf(fmaxf(q, -128.f), 127.f);
    }
}

}  // namespace

extern "C" int mf_quant_reshape_and_cache(const void* key, const void* value, void* key_cache, void* value_cache,
                                          const int32_t* slot_mapping, const float* scale, const float* offset,
                                          int num_tokens, int n_kv_heads, int head_dim, int64_t num_slots,
                                          int64_t key_row_stride, int64_t value_row_stride, int dtype,
                                          void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "quant_reshape_and_cache: dtype must be bf16 or fp16");
    if (num_tokens == 0) return 0;
    MF_REQUIRE(key && value && key_cache && value_cache && slot_mapping && scale,
               "quant_reshape_and_cache: null argument");
    MF_REQUIRE(num_tokens > 0 && n_kv_heads > 0 && head_dim > 0 && num_slots > 0, "quant_reshape_and_cache: bad sizes");
    const int row = n_kv_heads * head_dim;
    if (key_row_stride <= 0) key_row_stride = row;
    if (value_row_stride <= 0) value_row_stride = row;
    MF_REQUIRE(key_row_stride >= row && value_row_stride >= row, "quant_reshape_and_cache: row stride smaller than a row");
    dim3 grid(num_tokens, 2);
    if (dtype == MF_BF16)
        hipLaunchKernelGGL(quant_reshape_and_cache_kernel<BF16>, grid, dim3(256), 0, (hipStream_t)stream,
                           (const uint16_t*)key, (const uint16_t*)value, (int8_t*)key_cache, (int8_t*)value_cache,
                           slot_mapping, scale, offset, row, num_slots, key_row_stride, value_row_stride);
    else
        hipLaunchKernelGGL(quant_reshape_and_cache_kernel<FP16>, grid, dim3(256), 0, (hipStream_t)stream,
                           (const uint16_t*)key, (const uint16_t*)value, (int8_t*)key_cache, (int8_t*)value_cache,
                           slot_mapping, scale, offset, row, num_slots, key_row_stride, value_row_stride);
    return MF_LAUNCH_CHECK();
}

extern "C" int mf_dynamic_quant_reshape_and_cache(const void* key, const void* value, void* key_cache,
                                                  void* value_cache, float* key_scale_cache,
                                                  float* value_scale_cache, const int32_t* slot_mapping,
                                                  int num_tokens, int n_kv_heads, int head_dim, int64_t num_slots,
                                                  int64_t key_row_stride, int64_t value_row_stride, int dtype,
                                                  void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "dynamic_quant_reshape_and_cache: dtype must be bf16 or fp16");
    if (num_tokens == 0) return 0;
    MF_REQUIRE(key && value && key_cache && value_cache && key_scale_cache && value_scale_cache && slot_mapping,
               "dynamic_quant_reshape_and_cache: null argument");
    MF_REQUIRE(num_tokens > 0 && n_kv_heads > 0 && head_dim > 0 && num_slots > 0,
               "dynamic_quant_reshape_and_cache: bad sizes");
    const int row = n_kv_heads * head_dim;
    if (key_row_stride <= 0) key_row_stride = row;
    if (value_row_stride <= 0) value_row_stride = row;
    MF_REQUIRE(key_row_stride >= row && value_row_stride >= row,
               "dynamic_quant_reshape_and_cache: row stride smaller than a row");
    dim3 grid(num_tokens, 2);
    if (dtype == MF_BF16)
        hipLaunchKernelGGL(dynamic_quant_reshape_and_cache_kernel<BF16>, grid, dim3(256), 0, (hipStream_t)stream,
                           (const uint16_t*)key, (const uint16_t*)value, (int8_t*)key_cache, (int8_t*)value_cache,
                           key_scale_cache, value_scale_cache, slot_mapping, row, num_slots, key_row_stride,
                           value_row_stride);
    else
        hipLaunchKernelGGL(dynamic_quant_reshape_and_cache_kernel<FP16>, grid, dim3(256), 0, (hipStream_t)stream,
                           (const uint16_t*)key, (const uint16_t*)value, (int8_t*)key_cache, (int8_t*)value_cache,
                           key_scale_cache, value_scale_cache, slot_mapping, row, num_slots, key_row_stride,
                           value_row_stride);
    return MF_LAUNCH_CHECK();
}

extern "C" int mf_reshape_and_cache(const void* key, const void* value, void* key_cache, void* value_cache,
                                    const int32_t* slot_mapping, int num_tokens, int n_kv_heads, int head_dim,
                                    int64_t num_slots, int64_t key_row_stride, int64_t value_row_stride, int dtype,
                                    void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "reshape_and_cache: dtype must be bf16 or fp16");
    if (num_tokens == 0) return 0;                          // empty step: nothing to check or launch
    MF_REQUIRE(key && key_cache && slot_mapping, "reshape_and_cache: null key / key_cache / slot_mapping");
    MF_REQUIRE((value == nullptr) == (value_cache == nullptr),
               "reshape_and_cache: value and value_cache must both be given or both be null");
    MF_REQUIRE(num_tokens > 0 && n_kv_heads > 0 && head_dim > 0 && num_slots > 0, "reshape_and_cache: bad sizes");
    const int row_bytes = n_kv_heads * head_dim * 2;
    if (key_row_stride <= 0) key_row_stride = (int64_t)n_kv_heads * head_dim;
    if (value_row_stride <= 0) value_row_stride = (int64_t)n_kv_heads * head_dim;
    MF_REQUIRE(key_row_stride >= (int64_t)n_kv_heads * head_dim && value_row_stride >= (int64_t)n_kv_heads * head_dim,
               "reshape_and_cache: row stride smaller than a row");
    const bool vec = (row_bytes % 16 == 0) && (key_row_stride % 8 == 0) && (value_row_stride % 8 == 0) &&
                     (((uintptr_t)key | (uintptr_t)key_cache | (uintptr_t)value | (uintptr_t)value_cache) % 16 == 0);
    dim3 grid(num_tokens, value ? 2 : 1);
    const int threads = vec ? min(256, max(64, row_bytes / 16)) : 256;
    if (vec)
        hipLaunchKernelGGL(reshape_and_cache_kernel<16>, grid, dim3(threads), 0, (hipStream_t)stream,
                           (const uint8_t*)key, (const uint8_t*)value, (uint8_t*)key_cache, (uint8_t*)value_cache,
                           slot_mapping, row_bytes, num_slots, key_row_stride * 2, value_row_stride * 2);
    else
        hipLaunchKernelGGL(reshape_and_cache_kernel<2>, grid, dim3(threads), 0, (hipStream_t)stream,
                           (const uint8_t*)key, (const uint8_t*)value, (uint8_t*)key_cache, (uint8_t*)value_cache,
                           slot_mapping, row_bytes, num_slots, key_row_stride * 2, value_row_stride * 2);
    return MF_LAUNCH_CHECK();
}

extern "C" int mf_rope_half(void* query, void* key, const void* cos, const void* sin, int num_tokens,
                            int n_heads, int n_kv_heads, int head_dim, int64_t q_row_stride, int64_t k_row_stride,
                            int dtype, int table_dtype, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "rope: dtype must be bf16 or fp16");
    MF_REQUIRE(table_dtype == MF_BF16 || table_dtype == MF_FP16 || table_dtype == MF_FP32, "rope: bad table dtype");
    if (num_tokens == 0) return 0;
    MF_REQUIRE(query && cos && sin, "rope: null query / cos / sin");
    MF_REQUIRE(head_dim > 0 && head_dim % 2 == 0, "rope: head_dim must be even");
    if (q_row_stride <= 0) q_row_stride = (int64_t)n_heads * head_dim;
    if (k_row_stride <= 0) k_row_stride = (int64_t)n_kv_heads * head_dim;
    MF_REQUIRE(q_row_stride >= (int64_t)n_heads * head_dim && k_row_stride >= (int64_t)n_kv_heads * head_dim,
               "rope: row stride smaller than a row");
    if (dtype == MF_BF16)
        hipLaunchKernelGGL(rope_kernel<BF16>, dim3(num_tokens), dim3(256), 0, (hipStream_t)stream, (uint16_t*)query,
                           (uint16_t*)key, cos, sin, n_heads, n_kv_heads, head_dim, table_dtype, q_row_stride,
                           k_row_stride);
    else
        hipLaunchKernelGGL(rope_kernel<FP16>, dim3(num_tokens), dim3(256), 0, (hipStream_t)stream, (uint16_t*)query,
                           (uint16_t*)key, cos, sin, n_heads, n_kv_heads, head_dim, table_dtype, q_row_stride,
                           k_row_stride);
    return MF_LAUNCH_CHECK();
}

extern "C" int mf_rope_and_cache(void* query, void* key, const void* value, const void* cos, const void* sin,
                                 void* key_cache, void* value_cache, const int32_t* slot_mapping, int num_tokens,
                                 int n_heads, int n_kv_heads, int head_dim, int64_t num_slots, int64_t q_row_stride,
                                 int64_t k_row_stride, int64_t v_row_stride, int dtype, int table_dtype,
                                 void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "rope_and_cache: dtype must be bf16 or fp16");
    MF_REQUIRE(table_dtype == MF_BF16 || table_dtype == MF_FP16 || table_dtype == MF_FP32,
               "rope_and_cache: bad table dtype");
    if (num_tokens == 0) return 0;
    MF_REQUIRE(query && key && value && cos && sin && key_cache && value_cache && slot_mapping,
               "rope_and_cache: null argument");
    MF_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && num_slots > 0, "rope_and_cache: bad sizes");
    const int64_t kv_row = (int64_t)n_kv_heads * head_dim;
    if (q_row_stride <= 0) q_row_stride = (int64_t)n_heads * head_dim;
    if (k_row_stride <= 0) k_row_stride = kv_row;
    if (v_row_stride <= 0) v_row_stride = kv_row;
    MF_REQUIRE(q_row_stride >= (int64_t)n_heads * head_dim && k_row_stride >= kv_row && v_row_stride >= kv_row,
               "rope_and_cache: row stride smaller than a row");
    const int vec_ok = (kv_row % 8 == 0) && (v_row_stride % 8 == 0) &&
                       (((uintptr_t)value | (uintptr_t)value_cache) % 16 == 0);
    const bool all_vec = vec_ok && head_dim % 16 == 0 && q_row_stride % 8 == 0 && k_row_stride % 8 == 0 &&
                         (((uintptr_t)query | (uintptr_t)key | (uintptr_t)key_cache | (uintptr_t)cos |
                           (uintptr_t)sin) % 16 == 0);
    if (all_vec) {
        const int items = (n_heads + n_kv_heads) * (head_dim / 16) + n_kv_heads * head_dim / 8;
        dim3 grid(num_tokens, (items + 255) / 256);
        if (dtype == MF_BF16)
            hipLaunchKernelGGL(rope_and_cache_vec_kernel<BF16>, grid, dim3(256), 0, (hipStream_t)stream,
                               (uint16_t*)query, (uint16_t*)key, (const uint16_t*)value, cos, sin,
                               (uint16_t*)key_cache, (uint16_t*)value_cache, slot_mapping, n_heads, n_kv_heads,
                               head_dim, num_slots, table_dtype, q_row_stride, k_row_stride, v_row_stride);
        else
            hipLaunchKernelGGL(rope_and_cache_vec_kernel<FP16>, grid, dim3(256), 0, (hipStream_t)stream,
                               (uint16_t*)query, (uint16_t*)key, (const uint16_t*)value, cos, sin,
                               (uint16_t*)key_cache, (uint16_t*)value_cache, slot_mapping, n_heads, n_kv_heads,
                               head_dim, num_slots, table_dtype, q_row_stride, k_row_stride, v_row_stride);
        return MF_LAUNCH_CHECK();
    }
    if (dtype == MF_BF16)
        hipLaunchKernelGGL(rope_and_cache_kernel<BF16>, dim3(num_tokens), dim3(256), 0, (hipStream_t)stream,
                           (uint16_t*)query, (uint16_t*)key, (const uint16_t*)value, cos, sin, (uint16_t*)key_cache,
                           (uint16_t*)value_cache, slot_mapping, n_heads, n_kv_heads, head_dim, num_slots,
                           table_dtype, q_row_stride, k_row_stride, v_row_stride, vec_ok);
    else
        hipLaunchKernelGGL(rope_and_cache_kernel<FP16>, dim3(num_tokens), dim3(256), 0, (hipStream_t)stream,
                           (uint16_t*)query, (uint16_t*)key, (const uint16_t*)value, cos, sin, (uint16_t*)key_cache,
                           (uint16_t*)value_cache, slot_mapping, n_heads, n_kv_heads, head_dim, num_slots,
                           table_dtype, q_row_stride, k_row_stride, v_row_stride, vec_ok);
    return MF_LAUNCH_CHECK();
}

// Host <-> device swap of whole cache blocks.
//
// Scattered blocks: one kernel moves up to SWAP_PAIRS blocks per launch, reading or writing the pinned host cache
// directly over PCIe (a copy call per 256 KiB block costs more in call overhead than in transfer time).  The pair
// list travels in the kernel arguments, so nothing is staged in device memory.  Used when the host cache is mapped
// into the device address space (memory from hipHostMalloc is) and the blocks are 16-byte multiples; otherwise,
// and for long consecutive runs (where one DMA copy is as fast), the blocks go through hipMemcpyAsync.
constexpr int SWAP_PAIRS = 240;
constexpr int SWAP_SPLIT = 16;                                // workgroups per block

struct SwapPairs {
    int64_t src[SWAP_PAIRS];
    int64_t dst[SWAP_PAIRS];
};

__global__ __launch_bounds__(256) void swap_blocks_kernel(uint8_t* __restrict__ dst, const uint8_t* __restrict__ src,
                                                          SwapPairs pairs, int64_t block_bytes) {
    const int p = blockIdx.x;
    const u32x4* s = (const u32x4*)(src + pairs.src[p] * block_bytes);
    u32x4* d = (u32x4*)(dst + pairs.dst[p] * block_bytes);
    const int64_t n16 = block_bytes >> 4;
    const int64_t stride = (int64_t)SWAP_SPLIT * 256;
    int64_t i = (int64_t)blockIdx.y * 256 + threadIdx.x;
    for (; i + 3 * stride < n16; i += 4 * stride) {           // four 16-byte transfers in flight per lane
        const u32x4 a = s[i], b = s[i + stride], c = s[i + 2 * stride], e = s[i + 3 * stride];
        d[i] = a;
        d[i + stride] = b;
        d[i + 2 * stride] = c;
        d[i + 3 * stride] = e;
    }
    for (; i < n16; i += stride) d[i] = s[i];
}

extern "C" int mf_swap_blocks(void* host_cache, void* device_cache, const int64_t* pairs, int64_t n_pairs,
                              int64_t block_bytes, int64_t host_blocks, int64_t device_blocks, int device_to_host,
                              void* stream) {
    MF_REQUIRE(n_pairs >= 0 && block_bytes > 0, "swap_blocks: bad sizes");
    if (n_pairs == 0) return 0;
    MF_REQUIRE(host_cache && device_cache && pairs, "swap_blocks: null argument");
    const int64_t src_blocks = device_to_host ? device_blocks : host_blocks;
    const int64_t dst_blocks = device_to_host ? host_blocks : device_blocks;
    for (int64_t i = 0; i < n_pairs; ++i)
        MF_REQUIRE(pairs[2 * i] >= 0 && pairs[2 * i] < src_blocks && pairs[2 * i + 1] >= 0 &&
                       pairs[2 * i + 1] < dst_blocks,
                   "swap_blocks: pair %lld = (%lld, %lld) outside the caches (%lld source, %lld destination blocks)",
                   (long long)i, (long long)pairs[2 * i], (long long)pairs[2 * i + 1], (long long)src_blocks,
                   (long long)dst_blocks);
    hipStream_t st = (hipStream_t)stream;
    // the device's view of the host cache, if it has one
    void* host_dev = nullptr;
    const bool mapped = hipHostGetDevicePointer(&host_dev, host_cache, 0) == hipSuccess && host_dev != nullptr;
    if (!mapped) (void)hipGetLastError();                      // not an error of this call: the copy path serves it
    const bool by_kernel = mapped && block_bytes % 16 == 0 &&
                           (((uintptr_t)host_dev | (uintptr_t)device_cache) & 15) == 0;
    uint8_t* src = (uint8_t*)(device_to_host ? device_cache : host_cache);
    uint8_t* dst = (uint8_t*)(device_to_host ? host_cache : device_cache);
    uint8_t* ksrc = (uint8_t*)(device_to_host ? device_cache : host_dev);
    uint8_t* kdst = (uint8_t*)(device_to_host ? host_dev : device_cache);
    const hipMemcpyKind kind = device_to_host ? hipMemcpyDeviceToHost : hipMemcpyHostToDevice;
    SwapPairs batch;
    int filled = 0;
    auto flush = [&]() -> int {
        if (filled == 0) return 0;
        hipLaunchKernelGGL(swap_blocks_kernel, dim3(filled, SWAP_SPLIT), dim3(256), 0, st, kdst, ksrc, batch,
                           block_bytes);
        filled = 0;
        return MF_LAUNCH_CHECK();
    };
    int64_t i = 0;
    while (i < n_pairs) {
        int64_t run = 1;
        while (i + run < n_pairs && pairs[2 * (i + run)] == pairs[2 * i] + run &&
               pairs[2 * (i + run) + 1] == pairs[2 * i + 1] + run)
            ++run;
        if (!by_kernel || run * block_bytes >= (int64_t)8 << 20) {        // one DMA copy for a long run
            const hipError_t e = hipMemcpyAsync(dst + pairs[2 * i + 1] * block_bytes, src + pairs[2 * i] * block_bytes,
                                                (size_t)(run * block_bytes), kind, st);
            if (e != hipSuccess) return (int)e;
        } else {
            for (int64_t j = 0; j < run; ++j) {
                batch.src[filled] = pairs[2 * (i + j)];
                batch.dst[filled] = pairs[2 * (i + j) + 1];
                if (++filled == SWAP_PAIRS) {
                    const int rc = flush();
                    if (rc) return rc;
                }
            }
        }
        i += run;
    }
    return flush();
}
