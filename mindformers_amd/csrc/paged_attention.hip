// GQA paged attention for gfx950, decode side: launch rule, entry points and the entry point that allocates
// nothing.  The kernels are in paged_attention_kernels.h.
#include <mutex>

#include "paged_attention_kernels.h"

namespace {

// Partition size rule shared by the workspace query and the launch: 256-token partitions keep the tail of
// the last round of workgroups short; very long contexts use 512 to halve the partial traffic.
static inline int pa_tiles_per_wave(int64_t max_context) { return max_context > 16384 ? 4 : 2; }
// int8 caches halve the bytes per tile, which leaves the fixed cost of a workgroup (work-list scan, query load,
// first tile, merge) exposed: at least 512 tokens per workgroup at every context length (fewer partitions than the
// workspace query, which does not know the cache type, sizes for), more by the rule below.
// 16-bit caches: larger partitions (fewer fp32 partials to write and combine, fewer workgroups that find nothing to
// do when the block table is wider than the contexts are long) where the batch still fills the device with them.
// The lengths are on the device, so the count is taken on the context capacity:
//   512 tokens from 3072 workgroups up (0.7 % off the layer step of the 64-sequence ragged batch, which gains nothing
//   from more: 1024-token partitions leave it 1.8 rounds of workgroups);
//   1024 / 2048 tokens where the sequences alone - one workgroup each per kv head - fill the 768 workgroup slots, so
//   that a ragged batch cannot leave the last round short, or where the capacity is above 16384 tokens
//   (256 sequences of 2048 tokens, 4 kv heads: attention 212.7 us with 256-token partitions, 198.8 with 1024, 186.5
//   with 2048, which is one partition per sequence and no combine at all; 16 sequences of 16-32 k tokens, 8 kv heads:
//   292.1 / 283.0 / 274.5 us with 512 / 1024 / 2048).
static inline int pa_launch_tiles_per_wave(int64_t max_context, int kvq, int64_t batch_kv_groups) {
    auto workgroups = [&](int tpw) {
        return batch_kv_groups * ((max_context + tpw * PA_WAVE_TOKENS - 1) / (tpw * PA_WAVE_TOKENS));
    };
    const bool full = batch_kv_groups >= 768, deep = max_context > 16384;
    if ((full && workgroups(16) >= 1024) || (deep && workgroups(16) >= 2048)) return 16;
    if ((full || deep) && workgroups(8) >= 2048) return 8;
    return (kvq || workgroups(4) >= 3072) ? 4 : pa_tiles_per_wave(max_context);
}

// Per-token quantisation of the output rows requested together with the attention itself.
struct PaQuantArgs {
    int8_t* xq;
    float* x_scale;
    const float* smooth;
    int layout;
};

template <typename T, int D, int KVQ>
int launch_pa(void* out, const void* query, const void* key_cache, const void* value_cache,
              const int32_t* block_tables, const int32_t* context_lens, int batch, int n_heads, int n_kv,
              int block_size, int max_blocks, int num_blocks, float scale, int64_t q_stride, void* workspace,
              hipStream_t st, const float* kv_scale, const float* kv_offset, const PaQuantArgs* qa = nullptr) {
    const int n_rep = n_heads / n_kv;
    const int head_groups = (n_rep + 15) / 16;
    const int64_t max_ctx = (int64_t)max_blocks * block_size;
    const int tpw = pa_launch_tiles_per_wave(max_ctx, KVQ, (int64_t)batch * n_kv * head_groups);
    const int part_tokens = tpw * PA_WAVE_TOKENS;
    const int max_parts = (int)((max_ctx + part_tokens - 1) / part_tokens);
    float* part_out = (float*)workspace;
    float* part_ml = part_out ? part_out + (int64_t)batch * n_heads * max_parts * D : nullptr;
    const float scale_log2 = scale * 1.4426950408889634f;
    dim3 grid((unsigned)((int64_t)batch * max_parts * n_kv * head_groups));
    const bool tib = block_size % PA_TILE == 0;               // a 32-token tile never straddles two blocks
#define PA_LAUNCH(TPWV, TIBV)                                                                                    \
    hipLaunchKernelGGL((paged_attention_kernel<T, D, TPWV, false, KVQ, TIBV>), grid, dim3(PA_WAVES * 64), 0, st,  \
                       (uint16_t*)out, part_out, part_ml, (const uint16_t*)query, (const uint16_t*)key_cache,      \
                       (const uint16_t*)value_cache, block_tables, context_lens, n_heads, n_kv, n_rep, head_groups, \
                       block_size, max_blocks, num_blocks, max_parts, scale_log2, q_stride, batch,                 \
                       (const int32_t*)nullptr, 0, (int64_t)0, 0, kv_scale, kv_offset)
    if (tpw == 16) {
        if (tib) PA_LAUNCH(16, true);
        else PA_LAUNCH(16, false);
    } else if (tpw == 8) {
        if (tib) PA_LAUNCH(8, true);
        else PA_LAUNCH(8, false);
    } else if (tpw == 2) {
        if (tib) PA_LAUNCH(2, true);
        else PA_LAUNCH(2, false);
    } else {
        if (tib) PA_LAUNCH(4, true);
        else PA_LAUNCH(4, false);
    }
#undef PA_LAUNCH
    int rc = MF_LAUNCH_CHECK();
    if (rc) return rc;
    if (qa && max_parts > 1 && max_parts <= 16 && n_heads * D <= PA_RQ_THREADS * 8) {
        // combine of the partitions and quantisation of the row in one kernel
        hipLaunchKernelGGL((paged_attention_reduce_quant_kernel<T, D>), dim3(batch), dim3(PA_RQ_THREADS), 0, st,
                           (uint16_t*)out, qa->xq, qa->x_scale, part_out, part_ml, context_lens, qa->smooth, n_heads,
                           max_parts, part_tokens, qa->layout);
        return MF_LAUNCH_CHECK();
    }
    if (max_parts > 1) {
        hipLaunchKernelGGL((paged_attention_reduce_kernel<T, D, false>), dim3(n_heads, batch),
                           dim3(PA_REDUCE_THREADS<D>), 0, st,
                           (uint16_t*)out, part_out, part_ml, context_lens, n_heads, max_parts, part_tokens,
                           (const int32_t*)nullptr, batch, false, 0);
        rc = MF_LAUNCH_CHECK();
        if (rc) return rc;
    }
    if (qa)
        return mf_dynamic_quant_per_token(qa->xq, qa->x_scale, out, qa->smooth, batch, n_heads * D, T::id, qa->layout, st);
    return rc;
}

}  // namespace
extern "C" size_t mf_paged_attention_workspace_bytes(int batch, int n_heads, int head_dim, int max_context) {
    const int part_tokens = pa_tiles_per_wave(max_context) * PA_WAVE_TOKENS;
    const int64_t max_parts = ((int64_t)max_context + part_tokens - 1) / part_tokens;
    if (max_parts <= 1) return 0;
    return (size_t)batch * n_heads * max_parts * (head_dim + 2) * sizeof(float);
}

static int pa_decode_entry(void* out, const void* query, const void* key_cache, const void* value_cache,
                           const int32_t* block_tables, const int32_t* context_lens, int batch, int n_heads,
                           int n_kv_heads, int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
                           float scale, int64_t q_row_stride, int dtype, void* workspace, size_t workspace_bytes,
                           void* stream, int kvq, const float* kv_scale, const float* kv_offset,
                           const PaQuantArgs* qa = nullptr) {
    // kvq: 0 = 16-bit caches, 1 = int8 with per-channel scale / offset, 2 = int8 with per-token key scales
    // (kv_scale) and value scales (kv_offset), one float per cache slot
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "paged_attention: dtype must be bf16 or fp16");
    MF_REQUIRE(!kvq || kv_scale, "paged_attention: an int8 cache needs its scales");
    MF_REQUIRE(kvq != 2 || (kv_offset && block_size % 4 == 0 && (((uintptr_t)kv_scale | (uintptr_t)kv_offset) & 15) == 0),
               "paged_attention: per-token scales need both 16-byte aligned scale caches and a block size that is a "
               "multiple of 4");
    if (batch == 0) return 0;
    MF_REQUIRE(out && query && key_cache && value_cache && block_tables && context_lens,
               "paged_attention: null argument");
    MF_REQUIRE(batch >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
               "paged_attention: n_heads (%d) must be a positive multiple of n_kv_heads (%d)", n_heads, n_kv_heads);
    MF_REQUIRE(head_dim == 32 || head_dim == 64 || head_dim == 128,
               "paged_attention: head_dim %d not supported (32, 64, 128)", head_dim);
    MF_REQUIRE(block_size > 0 && max_blocks_per_seq > 0 && num_blocks > 0, "paged_attention: bad block geometry");
    MF_REQUIRE((int64_t)block_size * max_blocks_per_seq <= 0x7fffffffLL, "paged_attention: context capacity overflows int");
    if (q_row_stride <= 0) q_row_stride = (int64_t)n_heads * head_dim;
    MF_REQUIRE(q_row_stride >= (int64_t)n_heads * head_dim && q_row_stride % 8 == 0,
               "paged_attention: query row stride must be >= n_heads*head_dim and a multiple of 8 elements");
    MF_REQUIRE((((uintptr_t)out | (uintptr_t)query | (uintptr_t)key_cache | (uintptr_t)value_cache) & 15) == 0,
               "paged_attention: out / query / caches must be 16-byte aligned");
    if (batch == 0) return 0;
    const size_t need = mf_paged_attention_workspace_bytes(batch, n_heads, head_dim, max_blocks_per_seq * block_size);
    MF_REQUIRE(need == 0 || (workspace && workspace_bytes >= need),
               "paged_attention: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    MF_REQUIRE(need == 0 || ((uintptr_t)workspace & 15) == 0, "paged_attention: workspace must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    void* ws = need ? workspace : nullptr;
#define PA_CASE_Q(TT, DD, QQ)                                                                                   \
    return launch_pa<TT, DD, QQ>(out, query, key_cache, value_cache, block_tables, context_lens, batch, n_heads,  \
                                 n_kv_heads, block_size, max_blocks_per_seq, num_blocks, scale, q_row_stride, ws, st, \
                                 kvq ? kv_scale : nullptr, kvq ? kv_offset : nullptr, qa)
#define PA_CASE(TT, DD)                                                                                        \
    {                                                                                                          \
        if (kvq == 2) PA_CASE_Q(TT, DD, 2);                                                                    \
        if (kvq == 1) PA_CASE_Q(TT, DD, 1);                                                                    \
        PA_CASE_Q(TT, DD, 0);                                                                                  \
    }
    if (dtype == MF_BF16) {
        if (head_dim == 32) PA_CASE(BF16, 32);
        if (head_dim == 64) PA_CASE(BF16, 64);
        PA_CASE(BF16, 128);
    } else {
        if (head_dim == 32) PA_CASE(FP16, 32);
        if (head_dim == 64) PA_CASE(FP16, 64);
        PA_CASE(FP16, 128);
    }
#undef PA_CASE
#undef PA_CASE_Q
}

extern "C" int mf_paged_attention_decode(void* out, const void* query, const void* key_cache,
                                         const void* value_cache, const int32_t* block_tables,
                                         const int32_t* context_lens, int batch, int n_heads, int n_kv_heads,
                                         int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
                                         float scale, int64_t q_row_stride, int dtype, void* workspace,
                                         size_t workspace_bytes, void* stream) {
    return pa_decode_entry(out, query, key_cache, value_cache, block_tables, context_lens, batch, n_heads,
                           n_kv_heads, head_dim, block_size, max_blocks_per_seq, num_blocks, scale, q_row_stride,
                           dtype, workspace, workspace_bytes, stream, 0, nullptr, nullptr);
}

extern "C" int mf_paged_attention_decode_dynamic_quant(void* out, int8_t* xq, float* x_scale, const float* smooth,
                                                       int xq_layout, const void* query, const void* key_cache,
                                                       const void* value_cache, const int32_t* block_tables,
                                                       const int32_t* context_lens, int batch, int n_heads,
                                                       int n_kv_heads, int head_dim, int block_size,
                                                       int max_blocks_per_seq, int num_blocks, float scale,
                                                       int64_t q_row_stride, int dtype, void* workspace,
                                                       size_t workspace_bytes, void* stream) {
    if (batch == 0) return 0;
    MF_REQUIRE(xq && x_scale, "paged_attention_decode_dynamic_quant: null argument");
    MF_REQUIRE(xq_layout == 0 || xq_layout == 1,
               "paged_attention_decode_dynamic_quant: xq_layout must be 0 (row-major) or 1 (tiled)");
    MF_REQUIRE(((uintptr_t)xq & 7) == 0 && ((uintptr_t)smooth & 15) == 0,
               "paged_attention_decode_dynamic_quant: xq must be 8-byte aligned, smooth 16-byte aligned");
    const PaQuantArgs qa = {xq, x_scale, smooth, xq_layout};
    return pa_decode_entry(out, query, key_cache, value_cache, block_tables, context_lens, batch, n_heads,
                           n_kv_heads, head_dim, block_size, max_blocks_per_seq, num_blocks, scale, q_row_stride,
                           dtype, workspace, workspace_bytes, stream, 0, nullptr, nullptr, &qa);
}

extern "C" int mf_paged_attention_decode_int8kv(void* out, const void* query, const void* key_cache,
                                                const void* value_cache, const int32_t* block_tables,
                                                const int32_t* context_lens, const float* antiquant_scale,
                                                const float* antiquant_offset, int batch, int n_heads,
                                                int n_kv_heads, int head_dim, int block_size,
                                                int max_blocks_per_seq, int num_blocks, float scale,
                                                int64_t q_row_stride, int dtype, void* workspace,
                                                size_t workspace_bytes, void* stream) {
    return pa_decode_entry(out, query, key_cache, value_cache, block_tables, context_lens, batch, n_heads,
                           n_kv_heads, head_dim, block_size, max_blocks_per_seq, num_blocks, scale, q_row_stride,
                           dtype, workspace, workspace_bytes, stream, 1, antiquant_scale, antiquant_offset);
}

extern "C" int mf_paged_attention_decode_int8kv_per_token(void* out, const void* query, const void* key_cache,
                                                          const void* value_cache, const float* key_scale_cache,
                                                          const float* value_scale_cache, const int32_t* block_tables,
                                                          const int32_t* context_lens, int batch, int n_heads,
                                                          int n_kv_heads, int head_dim, int block_size,
                                                          int max_blocks_per_seq, int num_blocks, float scale,
                                                          int64_t q_row_stride, int dtype, void* workspace,
                                                          size_t workspace_bytes, void* stream) {
    return pa_decode_entry(out, query, key_cache, value_cache, block_tables, context_lens, batch, n_heads,
                           n_kv_heads, head_dim, block_size, max_blocks_per_seq, num_blocks, scale, q_row_stride,
                           dtype, workspace, workspace_bytes, stream, 2, key_scale_cache, value_scale_cache);
}

// ---- decode attention for callers that cannot allocate ----------------------------------------------------------
// The partition partials live in a file-scope device array in place of a caller workspace.  Every GPU the library
// runs on holds its own copy of the array (at its own address) until the process ends; the host-side name of the
// array is not a device address, so the address is asked for once per device and kept.
static __device__ __align__(256) unsigned char scratch[MF_PA_STATIC_SCRATCH_BYTES];

static int pa_static_scratch(void** ptr_out) {
    static std::mutex mu;
    static void* dev_ptr[MF_MAX_DEVICES] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    MF_REQUIRE(dev >= 0 && dev < MF_MAX_DEVICES, "paged_attention_decode_static: device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!dev_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        MF_REQUIRE(p != nullptr, "paged_attention_decode_static: no address for the scratch array");
        dev_ptr[dev] = p;
    }
    *ptr_out = dev_ptr[dev];
    return 0;
}

extern "C" int mf_paged_attention_decode_static(void* out, const void* query, const void* key_cache,
                                                const void* value_cache, const int32_t* block_tables,
                                                const int32_t* context_lens, int batch, int n_heads, int n_kv_heads,
                                                int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
                                                float scale, int64_t q_row_stride, int dtype, void* stream) {
    MF_REQUIRE(batch >= 0 && n_heads > 0 && head_dim > 0 && block_size > 0 && max_blocks_per_seq > 0,
               "paged_attention_decode_static: bad shape");
    MF_REQUIRE((int64_t)block_size * max_blocks_per_seq <= 0x7fffffffLL,
               "paged_attention_decode_static: context capacity overflows int");
    const size_t need = mf_paged_attention_workspace_bytes(batch, n_heads, head_dim, max_blocks_per_seq * block_size);
    MF_REQUIRE(need <= (size_t)MF_PA_STATIC_SCRATCH_BYTES,
               "paged_attention_decode_static: batch %d x %d heads x %d context tokens needs %zu bytes of partition "
               "partials, the built-in scratch holds %zu; use mf_paged_attention_decode with a workspace",
               batch, n_heads, max_blocks_per_seq * block_size, need, (size_t)MF_PA_STATIC_SCRATCH_BYTES);
    void* ws = nullptr;
    const int rc = pa_static_scratch(&ws);
    if (rc) return rc;
    // every partial a row's combine reads is written by this call's attention kernel first: nothing to clear
    return pa_decode_entry(out, query, key_cache, value_cache, block_tables, context_lens, batch, n_heads,
                           n_kv_heads, head_dim, block_size, max_blocks_per_seq, num_blocks, scale, q_row_stride,
                           dtype, ws, (size_t)MF_PA_STATIC_SCRATCH_BYTES, stream, 0, nullptr, nullptr);
}
