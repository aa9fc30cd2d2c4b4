// GQA paged-attention decode for gfx950.
//
// Work decomposition
//   grid = (partitions, n_kv_heads * head_groups, batch); one workgroup of 4 wavefronts owns one
//   512-token partition of one (sequence, kv head) and ALL query heads that share that kv head (up to 16
//   per head group), so every K/V byte is fetched from HBM exactly once.  Workgroups whose partition
//   starts beyond the sequence's context length exit at once; ragged batches therefore cost nothing.
//   The 16 tiles (32 tokens each) of a partition are interleaved over the 4 waves.
//
// Per 32-token tile (one wave)
//   S^T[token, head] = K[token, :] . Q[head, :]      two 16x16 MFMA tiles, k-steps of 32 over head_dim;
//                                                    K rows are loaded from HBM straight into the MFMA
//                                                    A-operand layout (lane = token row, 16 B per k-step)
//   online softmax in fp32 (exp2 domain); the only cross-lane traffic is two xor-shuffles for the row max
//   O^T[d, head] += V^T[d, token] . P^T[token, head] the probabilities sit in exactly the B-operand layout
//                                                    when the 32 tokens are ordered (sub-tile, 4g+i); V is
//                                                    staged through a per-wave LDS tile and read back
//                                                    transposed, two d-rows per 32-bit LDS read
//   The 4 waves are merged through LDS and the workgroup writes either the final rows (single partition)
//   or an fp32 partial (acc, max, sum) that a small second kernel combines.
#include "common.h"

namespace {

constexpr int PA_WAVES = 4;
constexpr int PA_TILE = 32;                                   // tokens per MFMA tile
constexpr int PA_TILES_PER_WAVE = 4;
constexpr int PA_PART = PA_WAVES * PA_TILES_PER_WAVE * PA_TILE;  // 512 tokens per workgroup
constexpr float PA_NEG = -1.0e30f;

template <int D>
struct PaSmem {
    static constexpr int VSTRIDE = D * 2 + 8;                 // bytes per staged V row (+8: bank spread)
    static constexpr int VBYTES = PA_WAVES * PA_TILE * VSTRIDE;
    static constexpr int OBYTES = PA_WAVES * 16 * D * 4;
    static constexpr int BYTES = VBYTES > OBYTES ? VBYTES : OBYTES;
};

template <typename T, int D>
__global__ __launch_bounds__(PA_WAVES * 64, 2) void paged_attention_kernel(
    uint16_t* __restrict__ out, float* __restrict__ part_out, float* __restrict__ part_ml,
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc,
    const int32_t* __restrict__ block_tables, const int32_t* __restrict__ ctx_lens, int n_heads, int n_kv,
    int n_rep, int head_groups, int block_size, int max_blocks, int num_blocks, int max_parts,
    float scale_log2, int64_t q_stride) {
    using vec8 = typename T::vec8;
    constexpr int KS = D / 32;
    constexpr int VSTRIDE = PaSmem<D>::VSTRIDE;

    __shared__ __attribute__((aligned(16))) uint8_t smem[PaSmem<D>::BYTES];
    __shared__ float sm_m[PA_WAVES][16];
    __shared__ float sm_l[PA_WAVES][16];

    const int b = blockIdx.z;
    const int kvh = blockIdx.y / head_groups;
    const int hg = blockIdx.y - kvh * head_groups;
    const int part = blockIdx.x;
    const int L = ctx_lens[b];
    const int part_start = part * PA_PART;
    if (part_start >= L) return;                              // uniform over the workgroup

    const int w = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int r = lane & 15;
    const int g = lane >> 4;

    // ---- Q as MFMA B operand: lane (r, g) holds Q[head r][32j + 8g .. +8]
    const int hh = hg * 16 + r;
    const bool head_ok = hh < n_rep;
    const int head = kvh * n_rep + (head_ok ? hh : 0);
    vec8 qreg[KS];
    {
        const uint16_t* qp = q + (int64_t)b * q_stride + (int64_t)head * D + 8 * g;
#pragma unroll
        for (int j = 0; j < KS; ++j) {
            u32x4 v = {0u, 0u, 0u, 0u};
            if (head_ok) v = *(const u32x4*)(qp + 32 * j);
            qreg[j] = bitcast<vec8>(v);
        }
    }

    f32x4 acc[KS][2];
#pragma unroll
    for (int u = 0; u < KS; ++u) {
        acc[u][0] = (f32x4){0.f, 0.f, 0.f, 0.f};
        acc[u][1] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
    float m_run = PA_NEG, l_run = 0.f;

    uint8_t* vst = smem + w * (PA_TILE * VSTRIDE);
    const int32_t* table = block_tables + (int64_t)b * max_blocks;
    const int64_t row_elems = (int64_t)n_kv * D;

    for (int it = 0; it < PA_TILES_PER_WAVE; ++it) {
        const int tstart = part_start + (it * PA_WAVES + w) * PA_TILE;
        if (tstart >= L) break;                               // uniform over the wave

        // ---- issue K and V loads for the tile (both sub-tiles of 16 tokens)
        u32x4 kreg[2][KS], vreg[2][KS];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            int tok = tstart + s * 16 + r;
            tok = tok < L ? tok : L - 1;                      // rows past the context are masked below
            const int bi = tok / block_size;
            int blk = table[bi];
            blk = (blk < 0 || blk >= num_blocks) ? 0 : blk;   // never leave the cache allocation
            const int64_t off = ((int64_t)blk * block_size + (tok - bi * block_size)) * row_elems +
                                (int64_t)kvh * D + 8 * g;
#pragma unroll
            for (int j = 0; j < KS; ++j) kreg[s][j] = *(const u32x4*)(kc + off + 32 * j);
#pragma unroll
            for (int j = 0; j < KS; ++j) vreg[s][j] = *(const u32x4*)(vc + off + 32 * j);
        }

        // ---- scores: S[s][i] = score of token tstart + 16 s + 4 g + i for head r
        f32x4 sc[2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            sc[s] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < KS; ++j) sc[s] = T::mfma16(bitcast<vec8>(kreg[s][j]), qreg[j], sc[s]);
        }
        float tmax = PA_NEG;
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int tok = tstart + s * 16 + 4 * g + i;
                const float v = tok < L ? sc[s][i] * scale_log2 : PA_NEG;
                sc[s][i] = v;
                tmax = fmaxf(tmax, v);
            }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        float psum = 0.f;
        uint32_t pp[4];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            float p0 = __builtin_amdgcn_exp2f(sc[s][0] - m_new), p1 = __builtin_amdgcn_exp2f(sc[s][1] - m_new);
            float p2 = __builtin_amdgcn_exp2f(sc[s][2] - m_new), p3 = __builtin_amdgcn_exp2f(sc[s][3] - m_new);
            pp[2 * s] = pack2<T>(p0, p1);
            pp[2 * s + 1] = pack2<T>(p2, p3);
            // the denominator sums the probabilities as the PV product sees them (rounded to T)
            psum += T::to_float((uint16_t)(pp[2 * s] & 0xffff)) + T::to_float((uint16_t)(pp[2 * s] >> 16)) +
                    T::to_float((uint16_t)(pp[2 * s + 1] & 0xffff)) + T::to_float((uint16_t)(pp[2 * s + 1] >> 16));
        }
        l_run = l_run * alpha + psum;
#pragma unroll
        for (int u = 0; u < KS; ++u) {
            acc[u][0] *= alpha;
            acc[u][1] *= alpha;
        }
        const vec8 pfrag = bitcast<vec8>((u32x4){pp[0], pp[1], pp[2], pp[3]});

        // ---- stage V (rows = tokens) in this wave's LDS tile
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int j = 0; j < KS; ++j) {
                uint8_t* p = vst + (s * 16 + r) * VSTRIDE + (32 * j + 8 * g) * 2;
                *(u32x2*)p = (u32x2){vreg[s][j][0], vreg[s][j][1]};
                *(u32x2*)(p + 8) = (u32x2){vreg[s][j][2], vreg[s][j][3]};
            }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();

        // ---- O^T += V^T P^T ; lane (r, g) reads d = 32u + 2r, 2r+1 for its 8 tokens (16*(e/4) + 4g + e%4)
#pragma unroll
        for (int u = 0; u < KS; ++u) {
            uint32_t wv[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int tl = 16 * (e >> 2) + 4 * g + (e & 3);
                wv[e] = *(const uint32_t*)(vst + tl * VSTRIDE + (32 * u + 2 * r) * 2);
            }
            u32x4 ev, od;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                ev[e] = __builtin_amdgcn_perm(wv[2 * e + 1], wv[2 * e], 0x05040100u);
                od[e] = __builtin_amdgcn_perm(wv[2 * e + 1], wv[2 * e], 0x07060302u);
            }
            acc[u][0] = T::mfma16(bitcast<vec8>(ev), pfrag, acc[u][0]);
            acc[u][1] = T::mfma16(bitcast<vec8>(od), pfrag, acc[u][1]);
        }
    }

    // ---- merge the 4 waves
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    if (g == 0) {
        sm_m[w][r] = m_run;
        sm_l[w][r] = l_run;
    }
    __syncthreads();                                          // also: every wave is done with its V tile
    float M = sm_m[0][r];
#pragma unroll
    for (int x = 1; x < PA_WAVES; ++x) M = fmaxf(M, sm_m[x][r]);
    const float f = __builtin_amdgcn_exp2f(m_run - M);
    float* obuf = (float*)smem;                               // [wave][head 16][D]
    {
        float* dst = obuf + ((w * 16 + r) * D) + 8 * g;
#pragma unroll
        for (int u = 0; u < KS; ++u) {
            // acc[u][par][i] is d = 32u + 8g + 2i + par
            f32x4 lo = {acc[u][0][0] * f, acc[u][1][0] * f, acc[u][0][1] * f, acc[u][1][1] * f};
            f32x4 hi = {acc[u][0][2] * f, acc[u][1][2] * f, acc[u][0][3] * f, acc[u][1][3] * f};
            *(f32x4*)(dst + 32 * u) = lo;
            *(f32x4*)(dst + 32 * u + 4) = hi;
        }
    }
    __syncthreads();

    constexpr int D4 = D / 4;
    for (int idx = threadIdx.x; idx < 16 * D4; idx += PA_WAVES * 64) {
        const int hr = idx / D4, d4 = idx - hr * D4;
        const int hq = hg * 16 + hr;
        if (hq >= n_rep) continue;
        float Mh = sm_m[0][hr];
#pragma unroll
        for (int x = 1; x < PA_WAVES; ++x) Mh = fmaxf(Mh, sm_m[x][hr]);
        float lt = 0.f;
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int x = 0; x < PA_WAVES; ++x) {
            lt += sm_l[x][hr] * __builtin_amdgcn_exp2f(sm_m[x][hr] - Mh);
            sum += *(const f32x4*)(obuf + (x * 16 + hr) * D + 4 * d4);
        }
        const int64_t gh = (int64_t)b * n_heads + kvh * n_rep + hq;
        if (max_parts == 1) {
            const float inv = 1.0f / lt;
            u32x2 o = {pack2<T>(sum[0] * inv, sum[1] * inv), pack2<T>(sum[2] * inv, sum[3] * inv)};
            *(u32x2*)(out + gh * D + 4 * d4) = o;
        } else {
            const int64_t pi = gh * max_parts + part;
            *(f32x4*)(part_out + pi * D + 4 * d4) = sum;
            if (d4 == 0) {
                part_ml[pi * 2] = Mh;
                part_ml[pi * 2 + 1] = lt;
            }
        }
    }
}

// Combine the partitions of one (sequence, head): out = sum_p 2^(m_p - M) acc_p / sum_p 2^(m_p - M) l_p.
template <typename T, int D>
__global__ void paged_attention_reduce_kernel(uint16_t* __restrict__ out, const float* __restrict__ part_out,
                                              const float* __restrict__ part_ml,
                                              const int32_t* __restrict__ ctx_lens, int n_heads, int max_parts) {
    const int h = blockIdx.x, b = blockIdx.y;
    const int d = threadIdx.x;
    const int L = ctx_lens[b];
    const int64_t gh = (int64_t)b * n_heads + h;
    int np = L <= 0 ? 0 : (L + PA_PART - 1) / PA_PART;
    np = np < max_parts ? np : max_parts;
    if (np == 0) {
        out[gh * D + d] = 0;
        return;
    }
    const float* ml = part_ml + gh * max_parts * 2;
    float M = PA_NEG;
    for (int p = 0; p < np; ++p) M = fmaxf(M, ml[2 * p]);
    float num = 0.f, den = 0.f;
    for (int p = 0; p < np; ++p) {
        const float f = __builtin_amdgcn_exp2f(ml[2 * p] - M);
        den += f * ml[2 * p + 1];
        num += f * part_out[(gh * max_parts + p) * D + d];
    }
    out[gh * D + d] = T::from_float(num / den);
}

template <typename T, int D>
int launch_pa(void* out, const void* query, const void* key_cache, const void* value_cache,
              const int32_t* block_tables, const int32_t* context_lens, int batch, int n_heads, int n_kv,
              int block_size, int max_blocks, int num_blocks, float scale, int64_t q_stride, void* workspace,
              hipStream_t st) {
    const int n_rep = n_heads / n_kv;
    const int head_groups = (n_rep + 15) / 16;
    const int64_t max_ctx = (int64_t)max_blocks * block_size;
    const int max_parts = (int)((max_ctx + PA_PART - 1) / PA_PART);
    float* part_out = (float*)workspace;
    float* part_ml = part_out ? part_out + (int64_t)batch * n_heads * max_parts * D : nullptr;
    const float scale_log2 = scale * 1.4426950408889634f;
    dim3 grid(max_parts, n_kv * head_groups, batch);
    hipLaunchKernelGGL((paged_attention_kernel<T, D>), grid, dim3(PA_WAVES * 64), 0, st, (uint16_t*)out, part_out,
                       part_ml, (const uint16_t*)query, (const uint16_t*)key_cache, (const uint16_t*)value_cache,
                       block_tables, context_lens, n_heads, n_kv, n_rep, head_groups, block_size, max_blocks,
                       num_blocks, max_parts, scale_log2, q_stride);
    int rc = MF_LAUNCH_CHECK();
    if (rc) return rc;
    if (max_parts > 1) {
        hipLaunchKernelGGL((paged_attention_reduce_kernel<T, D>), dim3(n_heads, batch), dim3(D), 0, st,
                           (uint16_t*)out, part_out, part_ml, context_lens, n_heads, max_parts);
        rc = MF_LAUNCH_CHECK();
    }
    return rc;
}

// zero rows of sequences with no context when the single-partition path (which skips them) is used
__global__ void pa_zero_empty_kernel(uint16_t* __restrict__ out, const int32_t* __restrict__ ctx_lens, int row) {
    const int b = blockIdx.x;
    if (ctx_lens[b] > 0) return;
    for (int i = threadIdx.x; i < row; i += blockDim.x) out[(int64_t)b * row + i] = 0;
}

}  // namespace

extern "C" size_t mf_paged_attention_workspace_bytes(int batch, int n_heads, int head_dim, int max_context) {
    const int64_t max_parts = ((int64_t)max_context + PA_PART - 1) / PA_PART;
    if (max_parts <= 1) return 0;
    return (size_t)batch * n_heads * max_parts * (head_dim + 2) * sizeof(float);
}

extern "C" int mf_paged_attention_decode(void* out, const void* query, const void* key_cache,
                                         const void* value_cache, const int32_t* block_tables,
                                         const int32_t* context_lens, int batch, int n_heads, int n_kv_heads,
                                         int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
                                         float scale, int64_t q_row_stride, int dtype, void* workspace,
                                         size_t workspace_bytes,
                                         void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "paged_attention: dtype must be bf16 or fp16");
    if (batch == 0) return 0;
    MF_REQUIRE(out && query && key_cache && value_cache && block_tables && context_lens,
               "paged_attention: null argument");
    MF_REQUIRE(batch >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
               "paged_attention: n_heads (%d) must be a positive multiple of n_kv_heads (%d)", n_heads, n_kv_heads);
    MF_REQUIRE(head_dim == 32 || head_dim == 64 || head_dim == 128,
               "paged_attention: head_dim %d not supported (32, 64, 128)", head_dim);
    MF_REQUIRE(block_size > 0 && max_blocks_per_seq > 0 && num_blocks > 0, "paged_attention: bad block geometry");
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
    if (need == 0) {
        hipLaunchKernelGGL(pa_zero_empty_kernel, dim3(batch), dim3(128), 0, st, (uint16_t*)out, context_lens,
                           n_heads * head_dim);
        int rc = MF_LAUNCH_CHECK();
        if (rc) return rc;
    }
    void* ws = need ? workspace : nullptr;
#define PA_CASE(TT, DD)                                                                                        \
    return launch_pa<TT, DD>(out, query, key_cache, value_cache, block_tables, context_lens, batch, n_heads,   \
                             n_kv_heads, block_size, max_blocks_per_seq, num_blocks, scale, q_row_stride, ws, st)
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
}
