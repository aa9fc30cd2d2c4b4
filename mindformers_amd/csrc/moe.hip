// Mixture-of-experts routing kernels: group-limited sigmoid top-k router, counting-sort permute,
// weighted unpermute.  Index work is exact; the heavy parts (row gather / weighted row sum) are plain
// HBM-bound copies with 16-byte lane accesses.
#include "common.h"

namespace {

constexpr int RT_MAX_E = 1024;
constexpr int RT_MAX_K = 32;

// One wavefront per token.
template <typename T>
__global__ __launch_bounds__(64) void moe_route_kernel(uint16_t* __restrict__ weights_out,
                                                      int32_t* __restrict__ index_out,
                                                      const float* __restrict__ logits,
                                                      const float* __restrict__ bias, int E, int k, int n_group,
                                                      int topk_group, float scale, int renorm,
                                                      int biased_weights) {
    __shared__ float s_plain[RT_MAX_E];     // sigmoid(logit)
    __shared__ float s_biased[RT_MAX_E];    // sigmoid(logit) + bias, later masked
    __shared__ float s_gscore[64];
    __shared__ float s_thr;
    const int t = blockIdx.x;
    const int lane = threadIdx.x;
    const float* lg = logits + (int64_t)t * E;

    for (int e = lane; e < E; e += 64) {
        const float s = 1.0f / (1.0f + __expf(-lg[e]));
        s_plain[e] = s;
        s_biased[e] = s + (bias ? bias[e] : 0.f);
    }
    __syncthreads();

    if (n_group > 1 && topk_group < n_group) {
        const int gs = E / n_group;
        float score = -INFINITY;
        if ((n_group & (n_group - 1)) == 0) {
            // 64 / n_group lanes share a group: each scans a strided part, the pairs of largest values merge by
            // shuffles (values only, so the order of the merge does not matter)
            const int lpg = 64 / n_group;
            const int grp = lane / lpg, sub = lane - grp * lpg;
            float a = -INFINITY, b = -INFINITY;               // two largest of the group
            for (int i = sub; i < gs; i += lpg) {
                const float v = s_biased[grp * gs + i];
                if (v > a) { b = a; a = v; } else if (v > b) { b = v; }
            }
            for (int o = 1; o < lpg; o <<= 1) {
                const float oa = __shfl_xor(a, o, 64), ob = __shfl_xor(b, o, 64);
                const float hi = fmaxf(a, oa);
                b = a >= oa ? fmaxf(b, oa) : fmaxf(ob, a);
                a = hi;
            }
            score = gs >= 2 ? a + b : a;
            if (sub == 0) s_gscore[grp] = score;
            __syncthreads();
            score = lane < n_group ? s_gscore[lane] : -INFINITY;
        } else {
            if (lane < n_group) {
                float a = -INFINITY, b = -INFINITY;
                for (int i = 0; i < gs; ++i) {
                    const float v = s_biased[lane * gs + i];
                    if (v > a) { b = a; a = v; } else if (v > b) { b = v; }
                }
                score = gs >= 2 ? a + b : a;
                s_gscore[lane] = score;
            }
            __syncthreads();
        }
        if (lane < n_group) {
            int rank = 0;                                     // groups strictly ahead (ties: lower index first)
            for (int j = 0; j < n_group; ++j) {
                const float o = s_gscore[j];
                rank += (o > score) || (o == score && j < lane);
            }
            if (rank == topk_group - 1) s_thr = score;        // the topk_group-th largest group score
        }
        __syncthreads();
        const float thr = s_thr;
        // keep groups with score >= threshold; experts of dropped groups score 0.0 (masked_fill)
        for (int e = lane; e < E; e += 64)
            if (!(s_gscore[e / gs] >= thr)) s_biased[e] = 0.0f;
        __syncthreads();
    }

    // top-k by repeated wave-wide argmax (larger value first, ties to the lower index); the candidates live in
    // registers, expert e = lane + 64 i in slot i
    __shared__ float s_wsel[RT_MAX_K];
    __shared__ int s_isel[RT_MAX_K];
    constexpr int SLOTS = RT_MAX_E / 64;
    float cand[SLOTS];
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) cand[i] = lane + 64 * i < E ? s_biased[lane + 64 * i] : -INFINITY;
    float wsum = 0.f;
    for (int j = 0; j < k; ++j) {
        float best = -INFINITY;
        int bi = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < SLOTS; ++i) {
            const bool live = lane + 64 * i < E;
            if (live && cand[i] > best) { best = cand[i]; bi = lane + 64 * i; }   // ascending e: first maximum wins
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(best, o, 64);
            const int oi = __shfl_xor(bi, o, 64);
            if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
        }
        if (bi >= E) bi = 0;                                  // all -inf/NaN rows: keep indices in range
        const float wv = biased_weights ? best : s_plain[bi];
        wsum += wv;
#pragma unroll
        for (int i = 0; i < SLOTS; ++i)
            if (bi == lane + 64 * i) cand[i] = -INFINITY;
        if (lane == 0) {
            s_wsel[j] = wv;
            s_isel[j] = bi;
        }
    }
    __syncthreads();
    if (lane == 0) {
        for (int j = 0; j < k; ++j) {
            float wv = s_wsel[j];
            if (renorm && k > 1) wv = wv / wsum;
            wv *= scale;
            weights_out[(int64_t)t * k + j] = T::from_float(wv);
            index_out[(int64_t)t * k + j] = s_isel[j];
        }
    }
}

// Histogram + exclusive scan + stable rank.  One workgroup of 1024 threads; pairs p = t*k + j.
__global__ __launch_bounds__(1024) void moe_sort_kernel(int32_t* __restrict__ row_map, int64_t* __restrict__ counts,
                                                        int32_t* __restrict__ offsets,
                                                        const int32_t* __restrict__ expert_index, int pairs,
                                                        int E) {
    __shared__ int s_cnt[RT_MAX_E];
    __shared__ int s_cur[RT_MAX_E];
    const int tid = threadIdx.x;
    for (int e = tid; e < E; e += blockDim.x) s_cnt[e] = 0;
    __syncthreads();
    for (int p = tid; p < pairs; p += blockDim.x) {
        const int e = expert_index[p];
        if (e >= 0 && e < E) atomicAdd(&s_cnt[e], 1);
    }
    __syncthreads();
    if (tid < 64) {                                           // exclusive scan: a chunk of experts per lane of wave 0
        const int per = (E + 63) / 64;
        const int e0 = tid * per;
        int local = 0;
        for (int i = 0; i < per; ++i)
            if (e0 + i < E) local += s_cnt[e0 + i];
        int incl = local;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int up = __shfl_up(incl, o, 64);
            if (tid >= o) incl += up;
        }
        int run = incl - local;
        for (int i = 0; i < per; ++i) {
            const int e = e0 + i;
            if (e < E) {
                const int c = s_cnt[e];
                s_cur[e] = run;
                offsets[e] = run;
                counts[e] = c;
                run += c;
            }
        }
        if (tid == 63) offsets[E] = incl;
    }
    __syncthreads();
    // stable placement: wave 0 walks the pairs in order, 64 at a time
    if (tid < 64) {
        const int lane = tid;
        for (int base = 0; base < pairs; base += 64) {
            const int p = base + lane;
            const bool live = p < pairs;
            int e = live ? expert_index[p] : -1;
            const bool ok = live && e >= 0 && e < E;
            if (!ok) e = -1;
            // lanes holding the same expert (10 index bits + validity)
            uint64_t same = __ballot(ok);
#pragma unroll
            for (int bit = 0; bit < 10; ++bit) {
                const uint64_t bm = __ballot((e >> bit) & 1);
                same &= ((e >> bit) & 1) ? bm : ~bm;
            }
            if (ok) {
                const uint64_t below = same & ((1ull << lane) - 1ull);
                const int rank = __popcll(below);
                const int dst = s_cur[e] + rank;
                row_map[p] = dst;
            } else if (live) {
                row_map[p] = -1;
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
            if (ok && (same & ((1ull << lane) - 1ull)) == 0) s_cur[e] += __popcll(same);   // group leader
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    }
}

// permuted_x[row_map[p]] = x[p / k]; one workgroup per pair.
__global__ void moe_gather_kernel(uint16_t* __restrict__ permuted, const uint16_t* __restrict__ x,
                                  const int32_t* __restrict__ row_map, int k, int hidden, int pairs) {
    const int p = blockIdx.x;
    const int dst = row_map[p];
    if (dst < 0 || dst >= pairs) return;
    const uint16_t* src = x + (int64_t)(p / k) * hidden;
    uint16_t* d = permuted + (int64_t)dst * hidden;
    for (int i = threadIdx.x * 8; i < hidden; i += blockDim.x * 8) *(u32x4*)(d + i) = *(const u32x4*)(src + i);
}

// out[t] = sum_j probs[t,j] * y[row_map[t*k+j]] (+ shared[t]); grid = (tokens, column chunks of 8 * blockDim.x), one
// 16-byte item per thread.  The k row indices and weights are read first, then the k rows are loaded in batches of
// UNP_BATCH independent loads and summed in choice order (the order fixes the fp32 sum).
constexpr int UNP_BATCH = 8;
template <typename T>
__global__ void moe_unpermute_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ y,
                                     const int32_t* __restrict__ row_map, const uint16_t* __restrict__ probs,
                                     const uint16_t* __restrict__ shared, int k, int hidden, int pairs) {
    const int t = blockIdx.x;
    const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
    if (i >= hidden) return;
    u32x4 sh = {0u, 0u, 0u, 0u};
    if (shared) sh = *(const u32x4*)(shared + (int64_t)t * hidden + i);
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int j0 = 0; j0 < k; j0 += UNP_BATCH) {
        int row[UNP_BATCH];
        float pw[UNP_BATCH];
        u32x4 v[UNP_BATCH];
#pragma unroll
        for (int j = 0; j < UNP_BATCH; ++j) {
            const int jj = j0 + j;
            row[j] = jj < k ? row_map[(int64_t)t * k + jj] : -1;
            pw[j] = jj < k ? T::to_float(probs[(int64_t)t * k + jj]) : 0.f;
        }
#pragma unroll
        for (int j = 0; j < UNP_BATCH; ++j) {
            const bool ok = row[j] >= 0 && row[j] < pairs;
            v[j] = (u32x4){0u, 0u, 0u, 0u};
            if (ok) v[j] = *(const u32x4*)(y + (int64_t)row[j] * hidden + i);
            else row[j] = -1;
        }
#pragma unroll
        for (int j = 0; j < UNP_BATCH; ++j) {
            if (row[j] < 0) continue;                         // a skipped choice adds nothing (not even +0)
            float f[8];
            unpack8<T>(v[j], f);
#pragma unroll
            for (int q = 0; q < 8; ++q) acc[q] += pw[j] * f[q];
        }
    }
    if (shared) {
        // the routed sum is materialised in the activation dtype before the shared-expert add
        float f[8];
        unpack8<T>(sh, f);
#pragma unroll
        for (int q = 0; q < 8; ++q) acc[q] = T::to_float(T::from_float(acc[q])) + f[q];
    }
    u32x4 o;
#pragma unroll
    for (int q = 0; q < 4; ++q) o[q] = pack2<T>(acc[2 * q], acc[2 * q + 1]);
    *(u32x4*)(out + (int64_t)t * hidden + i) = o;
}


// ---- router gate projection -------------------------------------------------------------------------
// logits[t, e] = sum_h x[t, h] * w[e, h], products and sums in fp32 on the fp32 matrix instruction (16 x 16 x 4).
// The weight (E x H, a few MB) is read once: a workgroup owns 16 experts and one slice of H for up to 64 tokens;
// its 4 waves take the slice's 64-column chunks in turn and meet in LDS.  Lane (r = lane & 15, g = lane >> 4) loads
// columns 16 j + 4 g .. + 3 of a chunk for expert r and for token r: the instruction's k index is any bijection as
// long as both operands use the same one.  With more than one slice the workgroups write partial sums
// [slice][token][expert] and router_gate_reduce_kernel adds the slices in order (no atomics: results do not depend
// on scheduling).
struct RG_F32 {};
template <typename WT>
__device__ __forceinline__ f32x4 rg_load4(const void* w, int64_t idx) {
    if constexpr (std::is_same<WT, RG_F32>::value) {
        return *(const f32x4*)((const float*)w + idx);
    } else {
        const u32x2 v = *(const u32x2*)((const uint16_t*)w + idx);
        return (f32x4){WT::to_float((uint16_t)(v[0] & 0xffffu)), WT::to_float((uint16_t)(v[0] >> 16)),
                       WT::to_float((uint16_t)(v[1] & 0xffffu)), WT::to_float((uint16_t)(v[1] >> 16))};
    }
}

template <typename WT>
__device__ __forceinline__ float rg_round(float v) {
    // a 16-bit router computes in its own type: the projection's output is rounded to it before the cast to fp32
    if constexpr (std::is_same<WT, RG_F32>::value) return v;
    else return WT::to_float(WT::from_float(v));
}

constexpr int RG_TT = 4;                                      // token tiles of 16 per workgroup

template <typename T, typename WT>
__global__ __launch_bounds__(256) void router_gate_kernel(float* __restrict__ out, float* __restrict__ partial,
                                                          const uint16_t* __restrict__ x, const void* __restrict__ w,
                                                          int tokens, int E, int H, int k_per_split) {
    __shared__ f32x4 red[4][RG_TT][64];
    const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    const int e0 = blockIdx.x * 16, t0 = blockIdx.z * (16 * RG_TT);
    const int k_begin = blockIdx.y * k_per_split, k_end = min(H, k_begin + k_per_split);
    const int64_t wrow = (int64_t)min(e0 + r, E - 1) * H;     // rows past the matrix re-read the last one, never stored
    int64_t xrow[RG_TT];
#pragma unroll
    for (int tt = 0; tt < RG_TT; ++tt) xrow[tt] = (int64_t)min(t0 + 16 * tt + r, tokens - 1) * H;
    f32x4 acc[RG_TT];
#pragma unroll
    for (int tt = 0; tt < RG_TT; ++tt) acc[tt] = (f32x4){0.f, 0.f, 0.f, 0.f};

    for (int k0 = k_begin + 64 * wv; k0 < k_end; k0 += 256) {
        f32x4 wa[4], xb[RG_TT][4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + 16 * j + 4 * g;
            const bool in = k < k_end;                        // H and the slices are multiples of 4
            const int kc = in ? k : k_begin;
            wa[j] = rg_load4<WT>(w, wrow + kc);
#pragma unroll
            for (int tt = 0; tt < RG_TT; ++tt) xb[tt][j] = rg_load4<T>(x, xrow[tt] + kc);
            if (!in) {
                wa[j] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int tt = 0; tt < RG_TT; ++tt) xb[tt][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int tt = 0; tt < RG_TT; ++tt)
                    acc[tt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wa[j][i], xb[tt][j][i], acc[tt], 0, 0, 0);
    }
#pragma unroll
    for (int tt = 0; tt < RG_TT; ++tt) red[wv][tt][lane] = acc[tt];
    __syncthreads();
    // thread (tt = wave, lane): the sum over the 4 waves, in order.  Lane (r, g) of the instruction's result holds
    // token r, experts 4 g .. 4 g + 3 of the tile.
    const int tt = wv;
    f32x4 v = red[0][tt][lane];
#pragma unroll
    for (int q = 1; q < 4; ++q) {
        const f32x4 u = red[q][tt][lane];
        v = (f32x4){v[0] + u[0], v[1] + u[1], v[2] + u[2], v[3] + u[3]};
    }
    const int t = t0 + 16 * tt + r, e = e0 + 4 * g;
    if (t >= tokens) return;
    float* dst = partial ? partial + ((int64_t)blockIdx.y * tokens + t) * E + e : out + (int64_t)t * E + e;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (e + i < E) dst[i] = partial ? v[i] : rg_round<WT>(v[i]);
}

template <typename WT>
__global__ void router_gate_reduce_kernel(float* __restrict__ out, const float* __restrict__ partial, int64_t n,
                                          int splits) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float v = partial[i];
    for (int s = 1; s < splits; ++s) v += partial[s * n + i];
    out[i] = rg_round<WT>(v);
}

struct GatePlan {
    int splits, k_per_split;
};
GatePlan plan_router_gate(int tokens, int E, int H) {
    const int wgs = ((E + 15) / 16) * ((tokens + 16 * RG_TT - 1) / (16 * RG_TT));
    int s = 512 / wgs;
    const int max_s = H / 256 < 1 ? 1 : H / 256;              // at least one chunk per wave
    s = s < 1 ? 1 : (s > max_s ? max_s : s);
    GatePlan p;
    p.k_per_split = ((H + s - 1) / s + 63) / 64 * 64;
    p.splits = (H + p.k_per_split - 1) / p.k_per_split;
    return p;
}

}  // namespace

extern "C" int mf_moe_route(void* weights_out, int32_t* index_out, const float* logits, const float* bias,
                            int tokens, int n_experts, int k, int n_group, int topk_group, float scale, int renorm,
                            int biased_weights, int dtype, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "moe_route: dtype must be bf16 or fp16");
    if (tokens <= 0) return 0;
    MF_REQUIRE(weights_out && index_out && logits, "moe_route: null argument");
    MF_REQUIRE(n_experts > 0 && n_experts <= RT_MAX_E, "moe_route: n_experts (%d) must be in 1..%d", n_experts, RT_MAX_E);
    MF_REQUIRE(k > 0 && k <= RT_MAX_K && k <= n_experts, "moe_route: k (%d) must be in 1..min(%d, n_experts)", k, RT_MAX_K);
    if (n_group > 1 && topk_group < n_group) {
        MF_REQUIRE(n_group <= 64 && n_experts % n_group == 0 && topk_group >= 1,
                   "moe_route: n_group (%d) must divide n_experts, be <= 64, with 1 <= topk_group (%d)", n_group,
                   topk_group);
    }
    if (tokens <= 0) return 0;
    if (dtype == MF_BF16)
        hipLaunchKernelGGL(moe_route_kernel<BF16>, dim3(tokens), dim3(64), 0, (hipStream_t)stream, (uint16_t*)weights_out,
                           index_out, logits, bias, n_experts, k, n_group, topk_group, scale, renorm, biased_weights);
    else
        hipLaunchKernelGGL(moe_route_kernel<FP16>, dim3(tokens), dim3(64), 0, (hipStream_t)stream, (uint16_t*)weights_out,
                           index_out, logits, bias, n_experts, k, n_group, topk_group, scale, renorm, biased_weights);
    return MF_LAUNCH_CHECK();
}

extern "C" size_t mf_router_gate_workspace_bytes(int tokens, int n_experts, int hidden) {
    if (tokens <= 0 || n_experts <= 0 || hidden <= 0) return 0;
    const GatePlan p = plan_router_gate(tokens, n_experts, hidden);
    return p.splits > 1 ? (size_t)p.splits * tokens * n_experts * sizeof(float) : 0;
}

extern "C" int mf_router_gate_gemm(float* logits, const void* x, const void* w, int tokens, int n_experts, int hidden,
                                   int dtype, int w_dtype, void* workspace, size_t workspace_bytes, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "router_gate_gemm: dtype must be bf16 or fp16");
    MF_REQUIRE(w_dtype == MF_FP32 || w_dtype == dtype, "router_gate_gemm: the weight is fp32 or of the activation type");
    if (tokens <= 0) return 0;
    MF_REQUIRE(logits && x && w, "router_gate_gemm: null argument");
    MF_REQUIRE(n_experts > 0 && hidden > 0 && hidden % 4 == 0, "router_gate_gemm: hidden (%d) must be a multiple of 4", hidden);
    MF_REQUIRE(((uintptr_t)x & 7) == 0 && ((uintptr_t)w & (w_dtype == MF_FP32 ? 15 : 7)) == 0,
               "router_gate_gemm: x must be 8-byte aligned, w 16-byte (fp32) or 8-byte aligned");
    const GatePlan p = plan_router_gate(tokens, n_experts, hidden);
    const size_t need = mf_router_gate_workspace_bytes(tokens, n_experts, hidden);
    MF_REQUIRE(need == 0 || (workspace && workspace_bytes >= need), "router_gate_gemm: workspace of %zu bytes needed, %zu given",
               need, workspace_bytes);
    float* partial = p.splits > 1 ? (float*)workspace : nullptr;
    const dim3 grid((n_experts + 15) / 16, p.splits, (tokens + 16 * RG_TT - 1) / (16 * RG_TT));
    const int64_t n = (int64_t)tokens * n_experts;
    const dim3 rgrid((unsigned)((n + 255) / 256));
#define RG_LAUNCH(TT_, WT_)                                                                                      \
    {                                                                                                            \
        hipLaunchKernelGGL((router_gate_kernel<TT_, WT_>), grid, dim3(256), 0, (hipStream_t)stream, logits, partial, \
                           (const uint16_t*)x, w, tokens, n_experts, hidden, p.k_per_split);                     \
        if (partial) {                                                                                           \
            int rc = MF_LAUNCH_CHECK();                                                                          \
            if (rc) return rc;                                                                                   \
            hipLaunchKernelGGL((router_gate_reduce_kernel<WT_>), rgrid, dim3(256), 0, (hipStream_t)stream, logits, \
                               partial, n, p.splits);                                                            \
        }                                                                                                        \
    }
    if (dtype == MF_BF16) {
        if (w_dtype == MF_FP32) RG_LAUNCH(BF16, RG_F32) else RG_LAUNCH(BF16, BF16)
    } else {
        if (w_dtype == MF_FP32) RG_LAUNCH(FP16, RG_F32) else RG_LAUNCH(FP16, FP16)
    }
#undef RG_LAUNCH
    return MF_LAUNCH_CHECK();
}

extern "C" int mf_moe_permute(void* permuted_x, int32_t* row_map, int64_t* counts, int32_t* offsets, const void* x,
                              const int32_t* expert_index, int tokens, int k, int n_experts, int hidden, int dtype,
                              void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "moe_permute: dtype must be bf16 or fp16");
    MF_REQUIRE(permuted_x && row_map && counts && offsets && x && expert_index, "moe_permute: null argument");
    MF_REQUIRE(n_experts > 0 && n_experts <= RT_MAX_E, "moe_permute: n_experts (%d) must be in 1..%d", n_experts, RT_MAX_E);
    MF_REQUIRE(tokens >= 0 && k > 0 && (int64_t)tokens * k <= 65536, "moe_permute: tokens*k must be <= 65536");
    MF_REQUIRE(hidden > 0 && hidden % 8 == 0, "moe_permute: hidden (%d) must be a multiple of 8", hidden);
    MF_REQUIRE((((uintptr_t)permuted_x | (uintptr_t)x) & 15) == 0, "moe_permute: rows must be 16-byte aligned");
    const int pairs = tokens * k;
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, row_map, counts, offsets,
                       expert_index, pairs, n_experts);
    int rc = MF_LAUNCH_CHECK();
    if (rc || pairs == 0) return rc;
    hipLaunchKernelGGL(moe_gather_kernel, dim3(pairs), dim3(256), 0, (hipStream_t)stream, (uint16_t*)permuted_x,
                       (const uint16_t*)x, row_map, k, hidden, pairs);
    return MF_LAUNCH_CHECK();
}

extern "C" int mf_moe_unpermute(void* out, const void* y, const int32_t* row_map, const void* probs,
                                const void* shared, int tokens, int k, int hidden, int dtype, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "moe_unpermute: dtype must be bf16 or fp16");
    if (tokens <= 0) return 0;
    MF_REQUIRE(out && y && row_map && probs, "moe_unpermute: null argument");
    MF_REQUIRE(k > 0 && hidden > 0 && hidden % 8 == 0, "moe_unpermute: hidden (%d) must be a multiple of 8", hidden);
    MF_REQUIRE((((uintptr_t)out | (uintptr_t)y | (uintptr_t)shared) & 15) == 0,
               "moe_unpermute: rows must be 16-byte aligned");
    if (tokens <= 0) return 0;
    constexpr int UNP_THREADS = 128;
    const dim3 ugrid(tokens, (hidden / 8 + UNP_THREADS - 1) / UNP_THREADS);
    if (dtype == MF_BF16)
        hipLaunchKernelGGL(moe_unpermute_kernel<BF16>, ugrid, dim3(UNP_THREADS), 0, (hipStream_t)stream, (uint16_t*)out,
                           (const uint16_t*)y, row_map, (const uint16_t*)probs, (const uint16_t*)shared, k, hidden,
                           tokens * k);
    else
        hipLaunchKernelGGL(moe_unpermute_kernel<FP16>, ugrid, dim3(UNP_THREADS), 0, (hipStream_t)stream, (uint16_t*)out,
                           (const uint16_t*)y, row_map, (const uint16_t*)probs, (const uint16_t*)shared, k, hidden,
                           tokens * k);
    return MF_LAUNCH_CHECK();
}
