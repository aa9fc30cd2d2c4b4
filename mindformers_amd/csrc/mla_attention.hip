// Multi-latent attention (MLA) decode over the paged latent cache, gfx950.
//
// One cache row per token holds the compressed key/value latent and the rotary key: [kv_lora_rank | rope] =
// 512 + 64 bf16/fp16 values.  Every query head attends with the whole 576-wide row as its key and the first
// 512 values of the same row as its value (the projections that make queries and outputs live in that space are
// absorbed into the caller's GEMMs).  With all heads sharing one row the op is bound by the matrix cores, not by
// HBM: 2 * (576 + 512) flops per (token, head) against 1152 bytes per token.
//
// Work decomposition
//   One workgroup of 8 wavefronts owns one token partition of one sequence and a block of 64 heads.  The cache
//   tile of 32 tokens (36 KB) is fetched once per workgroup with coalesced 16-byte loads, double-buffered in
//   LDS, and shared by all 8 waves: wave w serves heads 16 * (w & 3) .. + 15 and the value columns
//   256 * (w >> 2) .. + 255.  Both waves of a head group compute the scores (they need them for their own half
//   of the output); the PV product, which holds the accumulators, is split between them.
//   S^T[token, head] = C[token, :576] . Q[head, :576]     18 k-steps of mfma_f32_16x16x32 per 16-token sub-tile
//   online softmax in fp32 (exp2 domain), probabilities rounded to the cache dtype
//   O^T[d, head] += C^T[d, token] . P^T[token, head]       the tile is read back through the transposing LDS read
//                                                          (as in the GQA decode kernel)
//   No merge inside the workgroup is needed: every wave owns its (heads, columns).  Partitions of a sequence
//   are combined by the partition-reduce kernel of the GQA path.
#include "common.h"

namespace {

constexpr int MLA_DK = 576;                                   // key width: latent + rotary
constexpr int MLA_DV = 512;                                   // value width: the latent
constexpr int MLA_WAVES = 8;
constexpr int MLA_THREADS = MLA_WAVES * 64;
constexpr int MLA_HEADS = 64;                                 // heads per workgroup
constexpr int MLA_TILE = 32;                                  // tokens per tile
// bytes per staged row: +32 makes the row stride an even, non-multiple-of-4 number of 16-byte slots, which keeps
// both the 16-byte operand reads (served 16 lanes at a time: rows 0-3, 12-15 of one k-chunk with rows 4-11 of the
// next) and the transposed 4-byte reads free of bank conflicts
constexpr int MLA_STRIDE = MLA_DK * 2 + 32;
constexpr int MLA_TILE_BYTES = MLA_TILE * MLA_STRIDE;
constexpr int MLA_SMEM = 2 * MLA_TILE_BYTES;
constexpr int MLA_CPR = MLA_DK * 2 / 16;                      // 16-byte chunks per row
constexpr int MLA_CHUNKS = MLA_TILE * MLA_CPR;
constexpr int MLA_LD = (MLA_CHUNKS + MLA_THREADS - 1) / MLA_THREADS;      // loads per thread per tile
constexpr int MLA_KS = MLA_DK / 32;                           // k-steps of the score product
constexpr int MLA_DB = MLA_DV / 2 / 16;                       // 16-column blocks of one wave's half of the output
constexpr float MLA_NEG = -1.0e30f;

template <typename T>
__global__ __launch_bounds__(MLA_THREADS) void mla_decode_kernel(
    uint16_t* __restrict__ out, float* __restrict__ part_out, float* __restrict__ part_ml,
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ cache, const int32_t* __restrict__ block_tables,
    const int32_t* __restrict__ ctx_lens, int n_heads, int head_blocks, int block_size, int max_blocks,
    int num_blocks, int max_parts, int part_tokens, float scale_log2, int64_t q_stride, int batch) {
    using vec8 = typename T::vec8;
    extern __shared__ __attribute__((aligned(16))) uint8_t mla_smem[];

    // ---- work list: (sequence, partition, head block) triples that exist, from a prefix sum over the lengths
    int b = -1, part = 0, hb = 0, L = 0;
    {
        const int pidx = blockIdx.x;
        const int ln = threadIdx.x & 63;
        int base = 0;
        for (int c0 = 0; c0 < batch; c0 += 64) {
            const int bb = c0 + ln;
            const int len = bb < batch ? min(ctx_lens[bb], max_blocks * block_size) : 0;
            int np = len > 0 ? (len + part_tokens - 1) / part_tokens : 0;
            np = np < max_parts ? np : max_parts;
            const int per_seq = np * head_blocks;
            int incl = per_seq;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const int t = __shfl_up(incl, o, 64);
                if (ln >= o) incl += t;
            }
            const int total = __shfl(incl, 63, 64);
            if (pidx < base + total) {
                const bool hit = pidx >= base + incl - per_seq && pidx < base + incl;
                const int src = __ffsll((unsigned long long)__ballot(hit)) - 1;
                b = c0 + src;
                const int rem = pidx - (base + __shfl(incl - per_seq, src, 64));
                part = rem / head_blocks;
                hb = rem - part * head_blocks;
                L = __shfl(len, src, 64);
                break;
            }
            base += total;
        }
    }
    if (b < 0) return;                                        // uniform over the workgroup
    b = __builtin_amdgcn_readfirstlane(b);
    part = __builtin_amdgcn_readfirstlane(part);
    hb = __builtin_amdgcn_readfirstlane(hb);
    L = __builtin_amdgcn_readfirstlane(L);

    const int tid = threadIdx.x;
    const int w = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int hgw = w & 3, vhalf = w >> 2;
    const int head = hb * MLA_HEADS + hgw * 16 + r;
    const bool head_ok = head < n_heads;

    // ---- Q as MFMA B operand: lane (r, g) holds Q[head r][32 j + 8 g .. + 8]
    vec8 qreg[MLA_KS];
    {
        const uint16_t* qp = q + (int64_t)b * q_stride + (int64_t)(head_ok ? head : 0) * MLA_DK + 8 * g;
#pragma unroll
        for (int j = 0; j < MLA_KS; ++j) {
            u32x4 v = {0u, 0u, 0u, 0u};
            if (head_ok) v = *(const u32x4*)(qp + 32 * j);
            qreg[j] = bitcast<vec8>(v);
        }
    }

    const int part_start = part * part_tokens;
    const int part_end = min(L, part_start + part_tokens);
    const int ntiles = (part_end - part_start + MLA_TILE - 1) / MLA_TILE;
    const int32_t* table = block_tables + (int64_t)b * max_blocks;

    // cooperative tile load: chunk c = row * 72 + col; rows past the context re-read the last valid row
    int lrow[MLA_LD], lcol[MLA_LD];
#pragma unroll
    for (int k = 0; k < MLA_LD; ++k) {
        const int c = tid + k * MLA_THREADS;
        lrow[k] = c / MLA_CPR;
        lcol[k] = c - lrow[k] * MLA_CPR;
    }
    u32x4 lreg[MLA_LD];
    auto load_tile = [&](int tstart) {                        // a tile lies inside one block (host-checked)
        const int bi = tstart / block_size;
        int blk = table[bi];
        blk = (blk < 0 || blk >= num_blocks) ? 0 : blk;       // never leave the cache allocation
        const int64_t slot0 = (int64_t)blk * block_size + (tstart - bi * block_size);
        const uint16_t* base = cache + slot0 * MLA_DK;
        const int last_row = min(MLA_TILE, L - tstart) - 1;
#pragma unroll
        for (int k = 0; k < MLA_LD; ++k)
            if (k + 1 < MLA_LD || tid + k * MLA_THREADS < MLA_CHUNKS)
                lreg[k] = *(const u32x4*)(base + (int64_t)min(lrow[k], last_row) * MLA_DK + 8 * lcol[k]);
    };
    auto store_tile = [&](uint8_t* buf) {
#pragma unroll
        for (int k = 0; k < MLA_LD; ++k)
            if (k + 1 < MLA_LD || tid + k * MLA_THREADS < MLA_CHUNKS)
                *(u32x4*)(buf + lrow[k] * MLA_STRIDE + 16 * lcol[k]) = lreg[k];
    };

    f32x4 acc[MLA_DB];                                        // acc[db][i]: column 16 db + 4 g + i of this wave's half
#pragma unroll
    for (int db = 0; db < MLA_DB; ++db) acc[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m_run = MLA_NEG, l_run = 0.f;

    if (ntiles > 0) {
        load_tile(part_start);
        store_tile(mla_smem);
    }
    __syncthreads();

#pragma unroll 1
    for (int it = 0; it < ntiles; ++it) {
        const int tstart = part_start + it * MLA_TILE;
        const bool more = it + 1 < ntiles;
        const uint8_t* tile = mla_smem + (it & 1) * MLA_TILE_BYTES;
        if (more) load_tile(tstart + MLA_TILE);               // streams in behind this tile's math

        // ---- scores: S[s][i] = score of token tstart + 16 s + 4 g + i for head r
        f32x4 sc[2];
#pragma unroll
        for (int s = 0; s < 2; ++s) sc[s] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < MLA_KS; ++j) {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const u32x4 ka = *(const u32x4*)(tile + (s * 16 + r) * MLA_STRIDE + (32 * j + 8 * g) * 2);
                sc[s] = T::mfma16(bitcast<vec8>(ka), qreg[j], sc[s]);
            }
        }
        float tmax = MLA_NEG;
        if (tstart + MLA_TILE <= L) {
#pragma unroll
            for (int s = 0; s < 2; ++s)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    sc[s][i] *= scale_log2;
                    tmax = fmaxf(tmax, sc[s][i]);
                }
        } else {                                              // last tile of the sequence: mask what lies past it
#pragma unroll
            for (int s = 0; s < 2; ++s)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int tok = tstart + s * 16 + 4 * g + i;
                    const float v = tok < L ? sc[s][i] * scale_log2 : MLA_NEG;
                    sc[s][i] = v;
                    tmax = fmaxf(tmax, v);
                }
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
            const float p0 = __builtin_amdgcn_exp2f(sc[s][0] - m_new), p1 = __builtin_amdgcn_exp2f(sc[s][1] - m_new);
            const float p2 = __builtin_amdgcn_exp2f(sc[s][2] - m_new), p3 = __builtin_amdgcn_exp2f(sc[s][3] - m_new);
            pp[2 * s] = pack2<T>(p0, p1);
            pp[2 * s + 1] = pack2<T>(p2, p3);
            // the denominator sums the probabilities as the PV product sees them (rounded to T)
            psum += T::to_float((uint16_t)(pp[2 * s] & 0xffff)) + T::to_float((uint16_t)(pp[2 * s] >> 16)) +
                    T::to_float((uint16_t)(pp[2 * s + 1] & 0xffff)) + T::to_float((uint16_t)(pp[2 * s + 1] >> 16));
        }
        // when the running maximum moved for no lane of the wave, alpha is exactly 1: skip the rescale
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < MLA_DB; ++db) acc[db] *= alpha;
        }
        l_run += psum;
        const vec8 pfrag = bitcast<vec8>((u32x4){pp[0], pp[1], pp[2], pp[3]});

        // ---- O^T += C^T P^T over this wave's 256 value columns.  The A operand (row d, 8 tokens in the order of the
        // probabilities) comes from the row-major tile through the transposing LDS read: within 16 lanes, lane j
        // names C[token 4g + (j >> 2)][d0 + 4 (j & 3) ..] and lane r receives C[token 4g + e][d0 + r], e = 0..3.
#pragma unroll
        for (int db = 0; db < MLA_DB; ++db) {
            const int d0 = vhalf * (MLA_DV / 2) + 16 * db;
            const uint8_t* p0 = tile + (4 * g + (r >> 2)) * MLA_STRIDE + (d0 + 4 * (r & 3)) * 2;
            const u32x2 l2 = bitcast<u32x2>(lds_read_tr16(p0));
            const u32x2 h2 = bitcast<u32x2>(lds_read_tr16(p0 + 16 * MLA_STRIDE));
            acc[db] = T::mfma16(bitcast<vec8>((u32x4){l2[0], l2[1], h2[0], h2[1]}), pfrag, acc[db]);
        }

        if (more) store_tile(mla_smem + ((it + 1) & 1) * MLA_TILE_BYTES);
        __syncthreads();                                      // next tile staged; this tile's readers are done
    }

    // ---- write this wave's (heads, columns): the final rows (single partition) or an fp32 partial
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    if (!head_ok) return;
    const int64_t gh = (int64_t)b * n_heads + head;
    const float inv = 1.0f / l_run;
#pragma unroll
    for (int db = 0; db < MLA_DB; ++db) {
        const int d = vhalf * (MLA_DV / 2) + 16 * db + 4 * g;
        if (max_parts == 1) {
            const u32x2 o = {pack2<T>(acc[db][0] * inv, acc[db][1] * inv), pack2<T>(acc[db][2] * inv, acc[db][3] * inv)};
            *(u32x2*)(out + gh * MLA_DV + d) = o;
        } else {
            *(f32x4*)(part_out + (gh * max_parts + part) * MLA_DV + d) = acc[db];
        }
    }
    if (max_parts > 1 && g == 0 && vhalf == 0) {
        part_ml[(gh * max_parts + part) * 2] = m_run;
        part_ml[(gh * max_parts + part) * 2 + 1] = l_run;
    }
}

// Combine the partitions of one (sequence, head): out = sum_p 2^(m_p - M) acc_p / sum_p 2^(m_p - M) l_p.
// One workgroup of 512 threads (one per value column) per (head, sequence).
template <typename T>
__global__ __launch_bounds__(MLA_DV) void mla_reduce_kernel(uint16_t* __restrict__ out,
                                                            const float* __restrict__ part_out,
                                                            const float* __restrict__ part_ml,
                                                            const int32_t* __restrict__ ctx_lens, int n_heads,
                                                            int max_parts, int part_tokens, int max_ctx) {
    const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
    const int L = min(ctx_lens[b], max_ctx);
    const int64_t gh = (int64_t)b * n_heads + h;
    int np = L <= 0 ? 0 : (L + part_tokens - 1) / part_tokens;
    np = np < max_parts ? np : max_parts;
    if (np == 0) {
        out[gh * MLA_DV + d] = 0;
        return;
    }
    const float* ml = part_ml + gh * max_parts * 2;
    const float* po = part_out + gh * max_parts * MLA_DV + d;
    float M = MLA_NEG;
    for (int p = 0; p < np; ++p) M = fmaxf(M, ml[2 * p]);     // uniform addresses: broadcast loads
    float num = 0.f, den = 0.f;
    for (int p = 0; p < np; ++p) {
        const float f = __builtin_amdgcn_exp2f(ml[2 * p] - M);
        den += f * ml[2 * p + 1];
        num += f * po[(int64_t)p * MLA_DV];
    }
    out[gh * MLA_DV + d] = T::from_float(num / den);
}

// zero the rows of sequences with no context when a single partition spans the context (the main kernel skips them)
__global__ void mla_zero_empty_kernel(uint16_t* __restrict__ out, const int32_t* __restrict__ ctx_lens, int row) {
    if (ctx_lens[blockIdx.x] > 0) return;
    for (int i = threadIdx.x; i < row; i += blockDim.x) out[(int64_t)blockIdx.x * row + i] = 0;
}

// Partition rule shared by the workspace query and the launch: about two workgroups per compute unit when the
// batch allows it, partitions of whole 256-token multiples (fewer, larger partitions keep the fp32 partials,
// 2 KB per (head, partition), small beside the cache traffic).
struct MlaPlan {
    int part_tokens, max_parts, head_blocks;
};
inline MlaPlan mla_plan(int batch, int n_heads, int64_t max_ctx) {
    MlaPlan p;
    p.head_blocks = (n_heads + MLA_HEADS - 1) / MLA_HEADS;
    const int64_t seq_items = std::max<int64_t>(1, (int64_t)batch * p.head_blocks);
    const int64_t want = std::max<int64_t>(1, (512 + seq_items - 1) / seq_items);
    int64_t pt = (max_ctx + want - 1) / want;
    pt = std::max<int64_t>(256, (pt + 255) / 256 * 256);
    p.part_tokens = (int)pt;
    p.max_parts = (int)std::max<int64_t>(1, (max_ctx + pt - 1) / pt);
    return p;
}

template <typename T>
int launch_mla(void* out, const void* query, const void* cache, const int32_t* block_tables,
               const int32_t* context_lens, int batch, int n_heads, int block_size, int max_blocks, int num_blocks,
               float scale, int64_t q_stride, void* workspace, hipStream_t st) {
    static bool configured[MF_MAX_DEVICES] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MF_MAX_DEVICES) {
        mf_set_error("mla_paged_attention: device index %d outside the supported %d", dev, MF_MAX_DEVICES);
        return (int)hipErrorInvalidValue;
    }
    if (!configured[dev]) {
        e = hipFuncSetAttribute((const void*)mla_decode_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                MLA_SMEM);
        if (e != hipSuccess) return (int)e;
        configured[dev] = true;
    }
    const int64_t max_ctx = (int64_t)max_blocks * block_size;
    const MlaPlan plan = mla_plan(batch, n_heads, max_ctx);
    float* part_out = plan.max_parts > 1 ? (float*)workspace : nullptr;
    float* part_ml = part_out ? part_out + (int64_t)batch * n_heads * plan.max_parts * MLA_DV : nullptr;
    const float scale_log2 = scale * 1.4426950408889634f;
    if (plan.max_parts == 1) {
        hipLaunchKernelGGL(mla_zero_empty_kernel, dim3(batch), dim3(128), 0, st, (uint16_t*)out, context_lens,
                           n_heads * MLA_DV);
        const int rc = MF_LAUNCH_CHECK();
        if (rc) return rc;
    }
    const int64_t wgs = (int64_t)batch * plan.max_parts * plan.head_blocks;
    hipLaunchKernelGGL(mla_decode_kernel<T>, dim3((unsigned)wgs), dim3(MLA_THREADS), MLA_SMEM, st, (uint16_t*)out,
                       part_out, part_ml, (const uint16_t*)query, (const uint16_t*)cache, block_tables, context_lens,
                       n_heads, plan.head_blocks, block_size, max_blocks, num_blocks, plan.max_parts,
                       plan.part_tokens, scale_log2, q_stride, batch);
    int rc = MF_LAUNCH_CHECK();
    if (rc) return rc;
    if (plan.max_parts > 1) {
        hipLaunchKernelGGL(mla_reduce_kernel<T>, dim3(n_heads, batch), dim3(MLA_DV), 0, st, (uint16_t*)out, part_out,
                           part_ml, context_lens, n_heads, plan.max_parts, plan.part_tokens, (int)max_ctx);
        rc = MF_LAUNCH_CHECK();
    }
    return rc;
}

}  // namespace

extern "C" size_t mf_mla_paged_attention_workspace_bytes(int batch, int n_heads, int max_context) {
    if (batch <= 0 || n_heads <= 0 || max_context <= 0) return 0;
    const MlaPlan plan = mla_plan(batch, n_heads, max_context);
    if (plan.max_parts <= 1) return 0;
    return (size_t)batch * n_heads * plan.max_parts * (MLA_DV + 2) * sizeof(float);
}

extern "C" int mf_mla_paged_attention_decode(void* out, const void* query, const void* latent_cache,
                                             const int32_t* block_tables, const int32_t* context_lens, int batch,
                                             int n_heads, int kv_lora_rank, int rope_dim, int block_size,
                                             int max_blocks_per_seq, int num_blocks, float scale,
                                             int64_t q_row_stride, int dtype, void* workspace,
                                             size_t workspace_bytes, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "mla_paged_attention: dtype must be bf16 or fp16");
    MF_REQUIRE(batch >= 0, "mla_paged_attention: negative batch");
    if (batch == 0) return 0;
    MF_REQUIRE(out && query && latent_cache && block_tables && context_lens, "mla_paged_attention: null argument");
    MF_REQUIRE(kv_lora_rank == MLA_DV && rope_dim == MLA_DK - MLA_DV,
               "mla_paged_attention: kv_lora_rank %d / rope dim %d not supported (512 / 64)", kv_lora_rank, rope_dim);
    MF_REQUIRE(n_heads > 0, "mla_paged_attention: n_heads must be positive");
    MF_REQUIRE(block_size > 0 && block_size % MLA_TILE == 0 && max_blocks_per_seq > 0 && num_blocks > 0,
               "mla_paged_attention: block_size (%d) must be a positive multiple of %d", block_size, MLA_TILE);
    MF_REQUIRE((int64_t)block_size * max_blocks_per_seq <= 0x7fffffffLL,
               "mla_paged_attention: context capacity overflows int");
    if (q_row_stride <= 0) q_row_stride = (int64_t)n_heads * MLA_DK;
    MF_REQUIRE(q_row_stride >= (int64_t)n_heads * MLA_DK && q_row_stride % 8 == 0,
               "mla_paged_attention: query row stride must be >= n_heads * 576 and a multiple of 8 elements");
    MF_REQUIRE((((uintptr_t)out | (uintptr_t)query | (uintptr_t)latent_cache) & 15) == 0,
               "mla_paged_attention: out / query / cache must be 16-byte aligned");
    const size_t need = mf_mla_paged_attention_workspace_bytes(batch, n_heads, max_blocks_per_seq * block_size);
    MF_REQUIRE(need == 0 || (workspace && workspace_bytes >= need && ((uintptr_t)workspace & 15) == 0),
               "mla_paged_attention: a 16-byte aligned workspace of %zu bytes is needed, %zu given", need,
               workspace_bytes);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == MF_BF16)
        return launch_mla<BF16>(out, query, latent_cache, block_tables, context_lens, batch, n_heads, block_size,
                                max_blocks_per_seq, num_blocks, scale, q_row_stride, workspace, st);
    return launch_mla<FP16>(out, query, latent_cache, block_tables, context_lens, batch, n_heads, block_size,
                            max_blocks_per_seq, num_blocks, scale, q_row_stride, workspace, st);
}
