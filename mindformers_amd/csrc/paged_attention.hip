// GQA paged attention for gfx950: the decode kernel (one query row per sequence; also the prefill path of int8
// caches), its partition reduce, and further down the prefill kernel (several causal query rows per sequence).
//
// Decode: work decomposition
//   grid = batch * max_partitions * n_kv_heads * head_groups (1-D); one workgroup of 4 wavefronts owns one
//   256- or 512-token partition of one (sequence, kv head) and ALL query heads that share that kv head (up to 16
//   per head group), so every K/V byte is fetched from HBM exactly once.  Workgroups whose partition
//   starts beyond the sequence's context length exit at once; ragged batches therefore cost nothing.
//   The 16 tiles (32 tokens each) of a partition are interleaved over the 4 waves.
//
// Per 32-token tile (one wave)
//   K and V rows are fetched with fully coalesced 16-byte lane loads (consecutive lanes read consecutive
//   bytes of a token row) and staged through a per-wave LDS tile; the MFMA operand layouts are formed by
//   the LDS reads.  (Loading K straight into the A-operand layout makes every group of lanes touch 16
//   different cache lines per instruction and runs at less than half the bandwidth.)
//   S^T[token, head] = K[token, :] . Q[head, :]      two 16x16 MFMA tiles, k-steps of 32 over head_dim
//   online softmax in fp32 (exp2 domain); the only cross-lane traffic is two xor-shuffles for the row max
//   O^T[d, head] += V^T[d, token] . P^T[token, head] the probabilities sit in exactly the B-operand layout
//                                                    when the 32 tokens are ordered (sub-tile, 4g+i); V is
//                                                    staged through a per-wave LDS tile and read back with
//                                                    the transposing LDS read (ds_read_b64_tr_b16)
//   The 4 waves are merged through LDS and the workgroup writes either the final rows (single partition)
//   or an fp32 partial (acc, max, sum) that a small second kernel combines.
#include <mutex>

#include "common.h"

namespace {

constexpr int PA_WAVES = 4;
constexpr int PA_TILE = 32;                                   // tokens per MFMA tile
constexpr int PA_WAVE_TOKENS = PA_WAVES * PA_TILE;           // tokens one round of the 4 waves covers
constexpr float PA_NEG = -1.0e30f;

template <int D>
struct PaSmem {
    // bytes per staged row: +32 makes the row stride an even, non-multiple-of-4 number of 16-byte slots, which
    // keeps both the 16-byte operand reads (served 16 lanes at a time: rows 0-3, 12-15 of one k-chunk together with
    // rows 4-11 of the next) and the transposed 4-byte reads free of bank conflicts
    static constexpr int VSTRIDE = D * 2 + 32;
    static constexpr int VBYTES = PA_WAVES * PA_TILE * VSTRIDE;
    static constexpr int BYTES = VBYTES;
    static_assert(16 * D * 4 <= PA_TILE * VSTRIDE, "a wave's accumulators must fit its staging tile");
};

// Prefill bookkeeping of sequence s: first query row, number of query rows and context length, made safe
// (never more queries than context; query rows, and with them contiguous keys, never leave the `rows` passed).
__device__ inline void pf_seq(int s, const int32_t* __restrict__ q_starts, const int32_t* __restrict__ ctx_lens,
                              bool contiguous, int rows, int max_ctx, int batch, int& qs, int& ql, int& len) {
    qs = 0, ql = 0, len = 0;
    if (s >= batch) return;
    qs = q_starts[s];
    ql = q_starts[s + 1] - qs;
    if (qs < 0 || ql < 0 || qs + ql > rows) ql = 0;           // never leave the query / output rows
    if (contiguous) {
        len = ql;
    } else {
        len = ctx_lens[s];
        len = len < 0 ? 0 : (len > max_ctx ? max_ctx : len);  // the block table holds no more
        ql = ql < 0 ? 0 : (ql > len ? len : ql);
    }
}

// TPW = tiles per wave: a workgroup covers TPW * 128 tokens.
// PF (prefill / chunked prefill): sequence b brings q_starts[b+1] - q_starts[b] new query rows whose keys and values
// are already in the cache; query i of the sequence sits at position L_b - q_len + i and attends to the cache
// tokens up to and including its own.  The 16 MFMA columns of a workgroup, which in decode are the query heads
// of one kv head, are then 16 consecutive (query, head-of-the-kv-group) pairs, each with its own causal limit.
// PF with block_tables == nullptr: the keys and values are this step's own packed rows (row q_starts[b] + j is
// token j of sequence b, pf_kv_stride elements apart) and the context is q_len.
// KV8: the caches hold int8 (one byte per element, rows of n_kv * D bytes) with per-channel dequantisation
// x = (q - offset[c]) * scale[c]; kv_scale / kv_offset are float [2][n_kv * D] (keys, then values).  The key scale is
// folded into the query, the key offset shifts every score of a column by the same amount and drops out of the
// softmax, the value scale and offset are applied once to the (accumulator, sum) pair; the int8 tiles are widened
// to T (exactly) when they are staged in LDS, so the MFMA path is the same.
template <typename T, int D, int TPW, bool PF, bool KV8, bool TIB>
// Decode over an int8 cache keeps half the prefetch registers of a 16-bit one and fits four workgroups on a compute
// unit (128 registers; measured 6 % faster than with three); the 16-bit kernel needs 166 registers for its two
// prefetched tiles and gained nothing from a one-tile variant that fits four, so it stays at three.
__global__ __launch_bounds__(PA_WAVES * 64, (!PF && KV8 && TIB) ? 4 : 3) void paged_attention_kernel(
    uint16_t* __restrict__ out, float* __restrict__ part_out, float* __restrict__ part_ml,
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc,
    const int32_t* __restrict__ block_tables, const int32_t* __restrict__ ctx_lens, int n_heads, int n_kv,
    int n_rep, int head_groups, int block_size, int max_blocks, int num_blocks, int max_parts,
    float scale_log2, int64_t q_stride, int batch, const int32_t* __restrict__ q_starts, int pf_part_tokens,
    int64_t pf_kv_stride, int pf_rows, const float* __restrict__ kv_scale, const float* __restrict__ kv_offset) {
    using vec8 = typename T::vec8;
    constexpr int KS = D / 32;
    constexpr int VSTRIDE = PaSmem<D>::VSTRIDE;
    // tokens per partition: fixed by TPW in decode, chosen by the host (a multiple of 128) in PF, where the
    // query rows already supply the parallelism and one partition may span the whole context
    const int PART = PF ? pf_part_tokens : TPW * PA_WAVE_TOKENS;
    constexpr int EB = KV8 ? 1 : 2;                           // bytes per cache element
    constexpr int CPR = D * EB / 16;                          // 16-byte chunks per row
    constexpr int RPI = 64 / CPR;                             // rows one wave-wide load covers
    constexpr int NI = PA_TILE / RPI;                         // loads per lane per tile per tensor

    __shared__ __attribute__((aligned(16))) uint8_t smem[PaSmem<D>::BYTES];
    __shared__ float sm_m[PA_WAVES][16];
    __shared__ float sm_l[PA_WAVES][16];
    __shared__ int sm_count;

    // Work list: blockIdx.x enumerates the (sequence, kv head, partition) triples that exist, sequence-major
    // and partition-minor; each wave finds its triple with a prefix sum over ceil(L_b / PART), so a ragged batch
    // leaves no idle workgroups between busy ones (the unused tail of the grid exits here).  The order
    // matters for HBM: walking the kv heads fastest pins each XCD (consecutive workgroup ids go to
    // consecutive XCDs) to one 256-byte lane of every token row and measured 25 % slower.
    const int nkg = n_kv * head_groups;
    int b = -1, part = 0, L = 0, kg = 0;
    int q_len = 1, q_start = 0, col_groups = head_groups;     // PF: per sequence
    {
        const int pidx = blockIdx.x;
        const int ln = threadIdx.x & 63;
        int base = 0;
        for (int c0 = 0; c0 < batch; c0 += 64) {
            const int bb = c0 + ln;
            int len, ql = 1, qs = 0, ncg = head_groups;
            if constexpr (PF) {
                pf_seq(bb, q_starts, ctx_lens, block_tables == nullptr, pf_rows, max_blocks * block_size, batch, qs, ql, len);
                ncg = (ql * n_rep + 15) >> 4;
            } else {
                len = bb < batch ? min(ctx_lens[bb], max_blocks * block_size) : 0;   // the table holds no more
            }
            int np = len > 0 ? (len + PART - 1) / PART : 0;
            np = np < max_parts ? np : max_parts;
            const int per_seq = np * (PF ? n_kv * ncg : nkg);
            int incl = per_seq;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const int t = __shfl_up(incl, o, 64);
                if (ln >= o) incl += t;
            }
            const int total = __shfl(incl, 63, 64);
            if (pidx < base + total) {
                const bool hit = pidx >= base + incl - per_seq && pidx < base + incl;
                const uint64_t m = __ballot(hit);
                const int src = __ffsll((unsigned long long)m) - 1;
                b = c0 + src;
                const int rem = pidx - (base + __shfl(incl - per_seq, src, 64));
                const int npb = __shfl(np, src, 64);
                kg = rem / npb;
                part = rem - kg * npb;
                L = __shfl(len, src, 64);
                if constexpr (PF) {
                    q_len = __shfl(ql, src, 64);
                    q_start = __shfl(qs, src, 64);
                    col_groups = __shfl(ncg, src, 64);
                }
                break;
            }
            base += total;
        }
    }
    kg = __builtin_amdgcn_readfirstlane(kg);
    if (b < 0) return;                                        // uniform over the workgroup
    col_groups = __builtin_amdgcn_readfirstlane(col_groups);
    const int kvh = kg / col_groups;
    const int hg = kg - kvh * col_groups;                     // head group (decode) / column group (PF)
    b = __builtin_amdgcn_readfirstlane(b);
    part = __builtin_amdgcn_readfirstlane(part);
    L = __builtin_amdgcn_readfirstlane(L);
    q_len = __builtin_amdgcn_readfirstlane(q_len);
    q_start = __builtin_amdgcn_readfirstlane(q_start);
    const int part_start = part * PART;
    // PF: the farthest token any column of this group may see; partitions past it have nothing to do (the reduce
    // kernel counts partitions per query row and never reads them)
    const int ctx_before = L - q_len;                         // cache tokens older than this step's queries
    if constexpr (PF) {
        const int last_q = min(q_len, (hg * 16 + 15) / n_rep + 1);
        L = ctx_before + last_q;
        if (part_start >= L) return;
    }
    if (threadIdx.x == 0) sm_count = 0;
    __syncthreads();                                          // the only barrier: all waves are still in step here

    const int w = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int r = lane & 15;
    const int g = lane >> 4;

    // ---- Q as MFMA B operand: lane (r, g) holds Q[head r][32j + 8g .. +8]
    const int hh = hg * 16 + r;
    int qi = 0;                                               // PF: query index of this lane's column
    if constexpr (PF) qi = hh / n_rep;
    const int hcol = PF ? hh - qi * n_rep : hh;               // head within the kv group
    const bool head_ok = PF ? qi < q_len : hh < n_rep;
    const int head = kvh * n_rep + (head_ok ? hcol : 0);
    const int q_row = PF ? q_start + (head_ok ? qi : 0) : b;
    const int Lcol = PF ? (head_ok ? ctx_before + qi + 1 : 0) : L;      // causal limit of this lane's column
    // tiles that end at or before the smallest limit of the group's live columns need no mask (columns past the
    // sequence's queries are never written)
    const int Lmask = PF ? ctx_before + (hg * 16) / n_rep + 1 : L;
    vec8 qreg[KS];
    {
        const uint16_t* qp = q + (int64_t)q_row * q_stride + (int64_t)head * D + 8 * g;
#pragma unroll
        for (int j = 0; j < KS; ++j) {
            u32x4 v = {0u, 0u, 0u, 0u};
            if (head_ok) v = *(const u32x4*)(qp + 32 * j);
            if constexpr (KV8) {                              // fold the per-channel key scale into the query
                float f[8];
                unpack8<T>(v, f);
                const float* ks = kv_scale + kvh * D + 32 * j + 8 * g;
#pragma unroll
                for (int e = 0; e < 8; ++e) f[e] *= ks[e];
                v = (u32x4){pack2<T>(f[0], f[1]), pack2<T>(f[2], f[3]), pack2<T>(f[4], f[5]), pack2<T>(f[6], f[7])};
            }
            qreg[j] = bitcast<vec8>(v);
        }
    }

    constexpr int DB = D / 16;                                // 16-row blocks of O^T
    f32x4 acc[DB];                                            // acc[db][i]: d = 16 db + 4 g + i, head r
#pragma unroll
    for (int db = 0; db < DB; ++db) acc[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
    // PF: a column can find a whole tile masked before it has seen any token; starting the running maximum above
    // the mask value makes those probabilities 2^(-huge) = 0 instead of 2^0
    float m_run = PF ? 0.5f * PA_NEG : PA_NEG, l_run = 0.f;

    uint8_t* vst = smem + w * (PA_TILE * VSTRIDE);
    const bool contiguous = PF && block_tables == nullptr;
    const int32_t* table = block_tables + (int64_t)b * max_blocks;
    const int64_t row_bytes = (PF ? pf_kv_stride : (int64_t)n_kv * D) * EB;

    const int lrow = lane / CPR;                              // coalesced-load coordinates of this lane
    const int lchunk = lane - lrow * CPR;
    constexpr bool tile_in_block = TIB;                       // a tile never straddles two blocks (host-checked)
    const int wu = __builtin_amdgcn_readfirstlane(w);         // wave index as a scalar

    // tiles of this wave: it = 0 .. ntiles-1 start at part_start + (it*4 + wave)*32
    int ntiles = 0;
    {
        const int first = part_start + wu * PA_TILE;
        if (first < L) {
            const int last_tok = min(L, part_start + PART) - 1;
            ntiles = (last_tok - first) / (PA_WAVES * PA_TILE) + 1;
        }
    }
    // slot of a tile's first token when the tile lies inside one block (uniform: a scalar load), looked up
    // two tiles ahead so that no K/V load ever waits on a table load
    auto tile_slot = [&](int ts) -> int64_t {
        if (!tile_in_block || ts >= L) return 0;
        if (contiguous) return (int64_t)q_start + ts;
        const int bi = ts / block_size;
        int blk = table[bi];
        blk = (blk < 0 || blk >= num_blocks) ? 0 : blk;       // never leave the cache allocation
        return (int64_t)blk * block_size + (ts - bi * block_size);
    };
    // byte offset of chunk lchunk of token (tstart + lrow + RPI*i); tokens past the context re-read the last
    // valid row (their scores are masked)
    auto row_offset = [&](int64_t slot0, int tstart, int i) -> int64_t {
        int tok = tstart + lrow + RPI * i;
        tok = tok < L ? tok : L - 1;
        int64_t slot;
        if (tile_in_block) {
            slot = slot0 + (tok - tstart);
        } else {
            const int bi = tok / block_size;
            int blk = table[bi];
            blk = (blk < 0 || blk >= num_blocks) ? 0 : blk;
            slot = (int64_t)blk * block_size + (tok - bi * block_size);
        }
        return slot * row_bytes + (int64_t)kvh * D * EB + 16 * lchunk;
    };

    // A tile that lies inside one block (TIB) is a scalar base (its first slot) plus 32-bit per-lane offsets; rows
    // past the context (last tile of a sequence) re-read the last valid row, whose scores are masked.  Both paths
    // issue the same number of loads on purpose: the compiler counts outstanding loads exactly (and so lets the next
    // tile's loads stay in flight behind this tile's math) only where no paths with different loads join.  Block
    // sizes that tiles straddle (!TIB) need per-lane 64-bit addresses and table lookups.
    const uint32_t lane_col = (uint32_t)(kvh * D * EB + 16 * lchunk);
    const uint32_t lane_off = (uint32_t)(lrow * (int)row_bytes) + lane_col;
    auto load_tile = [&](u32x4* reg, const uint16_t* __restrict__ cache, int64_t slot0, int tstart) {
        if constexpr (TIB) {
            const uint8_t* base = (const uint8_t*)cache + slot0 * row_bytes;       // wave-uniform
            if (tstart + PA_TILE <= L) {                                           // whole tile: constant lane offset
#pragma unroll
                for (int i = 0; i < NI; ++i)
                    reg[i] = *(const u32x4*)(base + (int64_t)(RPI * i) * row_bytes + lane_off);
            } else {                                                               // the same loads, rows clamped
                const int last_row = L - tstart - 1;                               // uniform, >= 0 for a live tile
#pragma unroll
                for (int i = 0; i < NI; ++i)
                    reg[i] = *(const u32x4*)(base + (uint32_t)(min(lrow + RPI * i, last_row) * (int)row_bytes) +
                                             lane_col);
            }
        } else {
#pragma unroll
            for (int i = 0; i < NI; ++i)
                reg[i] = *(const u32x4*)((const uint8_t*)cache + row_offset(slot0, tstart, i));
        }
    };

    // a lane's 16 loaded bytes into its place of the staged row (rows hold T elements)
    auto stage = [&](uint8_t* row, const u32x4& v) {
        if constexpr (KV8) {
            *(vec8*)(row + 32 * lchunk) = dequant8<T>(v[0], v[1]);
            *(vec8*)(row + 32 * lchunk + 16) = dequant8<T>(v[2], v[3]);
        } else {
            *(u32x4*)(row + 16 * lchunk) = v;
        }
    };

    const int tstep = PA_WAVES * PA_TILE;
    const int tfirst = part_start + wu * PA_TILE;
    int64_t slot_cur = tile_slot(tfirst), slot_nxt = tile_slot(tfirst + tstep);
    u32x4 kreg[NI], vreg[NI];
    if (ntiles > 0) {
        load_tile(kreg, kc, slot_cur, tfirst);
        load_tile(vreg, vc, slot_cur, tfirst);
    }
    // the query is complete before the tile loop: a load still pending at the loop head from the entry path only
    // would make the compiler wait for every outstanding load at its first use inside the loop
#pragma unroll
    for (int j = 0; j < KS; ++j) asm volatile("" : "+v"(qreg[j]));

    // One tile.  The last tile of a wave is a copy of the body of its own (more = false at compile time): a branch
    // around the prefetch inside the loop would make the compiler wait for every outstanding load at the join.
    auto tile_body = [&](int it, auto more_c) {
        constexpr bool more = decltype(more_c)::value;
        const int tstart = tfirst + it * tstep;
        const int tnext = tstart + tstep;
        const int64_t slot_nn = more ? tile_slot(tnext + tstep) : 0;

        // ---- stage K row-major in LDS, read it back as MFMA A operands (lane = token row r, 8 d per k-step)
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < NI; ++i) stage(vst + (lrow + RPI * i) * VSTRIDE, kreg[i]);
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if constexpr (more) load_tile(kreg, kc, slot_nxt, tnext);   // streams in behind this tile's math

        // ---- scores: S[s][i] = score of token tstart + 16 s + 4 g + i for head r
        f32x4 sc[2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            sc[s] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < KS; ++j) {
                const u32x4 ka = *(const u32x4*)(vst + (s * 16 + r) * VSTRIDE + (32 * j + 8 * g) * 2);
                sc[s] = T::mfma16(bitcast<vec8>(ka), qreg[j], sc[s]);
            }
        }
        float tmax = PA_NEG;
        if (tstart + PA_TILE <= Lmask) {                      // every token of the tile is visible to every column
#pragma unroll
            for (int s = 0; s < 2; ++s)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    sc[s][i] *= scale_log2;
                    tmax = fmaxf(tmax, sc[s][i]);
                }
        } else {
#pragma unroll
            for (int s = 0; s < 2; ++s)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int tok = tstart + s * 16 + 4 * g + i;
                    const float v = tok < Lcol ? sc[s][i] * scale_log2 : PA_NEG;
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
            float p0 = __builtin_amdgcn_exp2f(sc[s][0] - m_new), p1 = __builtin_amdgcn_exp2f(sc[s][1] - m_new);
            float p2 = __builtin_amdgcn_exp2f(sc[s][2] - m_new), p3 = __builtin_amdgcn_exp2f(sc[s][3] - m_new);
            pp[2 * s] = pack2<T>(p0, p1);
            pp[2 * s + 1] = pack2<T>(p2, p3);
            // the denominator sums the probabilities as the PV product sees them (rounded to T)
            psum += T::to_float((uint16_t)(pp[2 * s] & 0xffff)) + T::to_float((uint16_t)(pp[2 * s] >> 16)) +
                    T::to_float((uint16_t)(pp[2 * s + 1] & 0xffff)) + T::to_float((uint16_t)(pp[2 * s + 1] >> 16));
        }
        // the running maximum of a column rarely moves after the first tiles: when it did not move for any lane of
        // the wave, alpha is exactly 1 everywhere and the rescale is skipped (bit-identical)
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < DB; ++db) acc[db] *= alpha;
        }
        l_run += psum;
        const vec8 pfrag = bitcast<vec8>((u32x4){pp[0], pp[1], pp[2], pp[3]});

        // ---- stage V (rows = tokens) in the same LDS tile
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < NI; ++i) stage(vst + (lrow + RPI * i) * VSTRIDE, vreg[i]);
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if constexpr (more) load_tile(vreg, vc, slot_nxt, tnext);
        slot_cur = slot_nxt;
        slot_nxt = slot_nn;

        // ---- O^T += V^T P^T.  The A operand (row d, 8 tokens in the order of the probabilities: 4g+e, 16+4g+e) comes
        // from the row-major tile through the transposing LDS read: within 16 lanes, lane j names the 4 values
        // V[token 4g + (j >> 2)][16 db + 4 (j & 3) ..] and lane r receives V[token 4g + e][16 db + r], e = 0..3.
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            const uint8_t* p0 = vst + (4 * g + (r >> 2)) * VSTRIDE + (16 * db + 4 * (r & 3)) * 2;
            const s16x4 lo = lds_read_tr16(p0);
            const s16x4 hi = lds_read_tr16(p0 + 16 * VSTRIDE);
            const u32x2 l2 = bitcast<u32x2>(lo), h2 = bitcast<u32x2>(hi);
            acc[db] = T::mfma16(bitcast<vec8>((u32x4){l2[0], l2[1], h2[0], h2[1]}), pfrag, acc[db]);
        }
    };
#pragma unroll 1
    for (int it = 0; it + 1 < ntiles; ++it) tile_body(it, std::true_type{});
    if (ntiles > 0) tile_body(ntiles - 1, std::false_type{});

    // ---- merge the 4 waves without a barrier: every wave parks its (max, sum, acc) in LDS (acc goes into its
    // own, now idle, staging tile), bumps a counter and leaves; the wave that arrives last combines them.
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    if (g == 0) {
        sm_m[w][r] = m_run;
        sm_l[w][r] = l_run;
    }
    {
        float* dst = (float*)vst + r * D + 4 * g;             // [head 16][D] floats: fits the staging tile
#pragma unroll
        for (int db = 0; db < DB; ++db) *(f32x4*)(dst + 16 * db) = acc[db];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    int arrived = 0;
    if (lane == 0) arrived = atomicAdd(&sm_count, 1);
    arrived = __builtin_amdgcn_readfirstlane(arrived);
    if (arrived != PA_WAVES - 1) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");

    constexpr int D4 = D / 4;
    for (int idx = lane; idx < 16 * D4; idx += 64) {
        const int hr = idx / D4, d4 = idx - hr * D4;
        int hq = hg * 16 + hr;
        int row = b;
        if constexpr (PF) {
            const int qe = hq / n_rep;
            if (qe >= q_len) break;                           // columns are ordered: nothing valid follows
            hq -= qe * n_rep;
            row = q_start + qe;
        } else {
            if (hq >= n_rep) break;                           // heads are ordered: nothing valid follows
        }
        float Mh = sm_m[0][hr];
#pragma unroll
        for (int x = 1; x < PA_WAVES; ++x) Mh = fmaxf(Mh, sm_m[x][hr]);
        float lt = 0.f;
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int x = 0; x < PA_WAVES; ++x) {
            const float f = __builtin_amdgcn_exp2f(sm_m[x][hr] - Mh);
            lt += sm_l[x][hr] * f;
            sum += *(const f32x4*)((const float*)(smem + x * (PA_TILE * VSTRIDE)) + hr * D + 4 * d4) * f;
        }
        if constexpr (KV8) {                                  // value dequantisation, linear in (sum, lt)
            const float* vs = kv_scale + n_kv * D + kvh * D + 4 * d4;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float off = kv_offset ? kv_offset[n_kv * D + kvh * D + 4 * d4 + e] : 0.f;
                sum[e] = vs[e] * (sum[e] - off * lt);
            }
        }
        const int64_t gh = (int64_t)row * n_heads + kvh * n_rep + hq;
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

// ---- prefill on the 32x32x16 MFMA ---------------------------------------------------------------------------------
// Prefill has (query, head) columns in abundance.  A workgroup of 4 waves serves 128 consecutive columns of one kv
// head (32 per wave) and walks the keys and values of their causal range once, 32 tokens at a time; every wave
// multiplies its own 32 columns against the shared tile, so each K / V byte is read from L2 once per 128 columns
// (with one tile stream per wave the kernel was bound by L2 bandwidth).  The 32x32x16 instruction does twice the
// work of the 16x16x32 one in the same issue time and halves the LDS reads per column.
//   S^T[token 32, col 32] = K[token, :] . Q[col, :]    D/16 MFMAs; lane (rho, h) holds row rho, k = 8h .. 8h+7
//   accumulator register i of lane (rho, h) is token 8 (i / 4) + 4 h + i % 4 of column rho, so registers
//   8 T .. 8 T + 7 are, in order, exactly the 8 k-values a lane supplies to the B operand of token half T when that
//   half's 16 tokens are taken in the order (4 h + e, 8 + 4 h + e); the V^T operand is read in the same order with
//   the transposing LDS read.
// Tiles go from global memory straight into LDS (no registers in between) through a ring of 3 buffers, two tiles
// ahead, with one barrier per tile.  Such a load writes 64 consecutive 16-byte slots, so rows cannot be padded;
// instead the 16-byte chunks of a row are permuted by the address each lane supplies:
//   K: chunk c of row t sits in slot c ^ key(t): the 16 rows of one chunk that an operand read serves together
//      land on 16 different slots;
//   V: chunk c of row t sits in slot (c + 4 key4(t)) mod chunks-per-row: the 4 tokens x 64 bytes a transposing read
//      serves together land on different slots.
// The LDS reads are asm statements issued a few MFMAs ahead with counted waits (the compiler would wait for each
// read before the next), and the order is pinned with scheduling barriers.  Three workgroups are resident per
// compute unit (48 KB of LDS, at most 168 registers), so a SIMD holds three waves whose matrix and vector phases
// overlap; a version that interleaved the phases of neighbouring tiles inside a wave needed 216 registers and was
// no faster with two.
// A wave owns its columns over the whole partition, so there is no merge: it writes final rows (single partition) or
// fp32 partials for the reduce kernel.
constexpr int PF_COLS = 128;                                  // columns per workgroup
constexpr int PF_TOK = 32;                                    // tokens per staged tile
constexpr int PF_RING = 3;                                    // staged tiles

// A staged K or V tile is one sub-tile of PF_TOK rows of W elements, W a power of two, or, for 192-wide heads (the
// prefill of multi-latent attention: 128 + 64 rope dimensions), a 128-wide sub-tile followed by a 64-wide one: the
// chunk permutations below need a power-of-two number of chunks per row, and the address each lane supplies to a
// direct load is free, so the columns of a row can be split over two regions of the buffer.
template <int W>
struct PfSub {
    static constexpr int ROWB = W * 2;                        // bytes per staged row
    static constexpr int CPR = ROWB / 16;                     // 16-byte chunks per row
    static constexpr int RPB = 16 / CPR;                      // rows per 256 bytes of LDS
    static constexpr int RPI = 64 / CPR;                      // rows one wave-wide load covers
    static constexpr int LOADS = PF_TOK / RPI;                // wave-wide loads per tile per tensor
    static constexpr int LW = LOADS < PA_WAVES ? LOADS : PA_WAVES;   // waves that load
    static constexpr int NI = LOADS / LW;                     // loads per loading wave per tile per tensor
};
template <>
struct PfSub<0> {
    static constexpr int ROWB = 0, CPR = 1, RPB = 1, RPI = 1, LOADS = 0, LW = PA_WAVES, NI = 0;
};

template <int D>
struct PfSmem {
    static constexpr int W0 = D == 192 ? 128 : D;             // widths of the two sub-tiles (the second may be empty)
    static constexpr int W1 = D - W0;
    using Sub0 = PfSub<W0>;
    using Sub1 = PfSub<W1>;
    static constexpr int NI = Sub0::NI + Sub1::NI;            // loads per loading wave per tile per tensor
    static constexpr int KBYTES = PF_TOK * D * 2;
    static constexpr int SUB1 = PF_TOK * W0 * 2;              // byte offset of the second sub-tile within a tile
    static constexpr int BUF = 2 * KBYTES;                    // K tile, then V tile
    static constexpr int BYTES = PF_RING * BUF;
};

// Three workgroups per compute unit; two at 192-wide heads (72 KB of LDS and 96 accumulator registers each).
template <typename T, int D, bool TIB>
__global__ __launch_bounds__(PA_WAVES * 64, D == 192 ? 2 : 3) void prefill_attention_kernel(
    uint16_t* __restrict__ out, float* __restrict__ part_out, float* __restrict__ part_ml,
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc,
    const int32_t* __restrict__ block_tables, const int32_t* __restrict__ ctx_lens, int n_heads, int n_kv,
    int n_rep, int block_size, int max_blocks, int num_blocks, int max_parts, float scale_log2, int64_t q_stride,
    int batch, const int32_t* __restrict__ q_starts, int part_tokens, int64_t kv_stride, int rows) {
    using vec8 = typename T::vec8;
    using S = PfSmem<D>;
    constexpr int KS = D / 16;                                // k-steps of the score product
    constexpr int DB = D / 32;                                // 32-row blocks of O^T
    constexpr int NV = 2 * DB;                                // PV MFMAs per tile
    using S0 = typename S::Sub0;
    using S1 = typename S::Sub1;
    constexpr int NI = S::NI;
    constexpr int KS0 = S::W0 / 16;                           // k-steps served by the first sub-tile
    constexpr int DB0 = S::W0 / 32;                           // 32-row blocks of O^T served by the first sub-tile

    extern __shared__ __attribute__((aligned(16))) uint8_t pf_smem[];

    // work list: see paged_attention_kernel; a sequence has ceil(q_len * n_rep / 128) column groups
    int b = -1, part = 0, L = 0, kg = 0, q_len = 1, q_start = 0, col_groups = 1;
    {
        const int pidx = blockIdx.x;
        const int ln = threadIdx.x & 63;
        int base = 0;
        for (int c0 = 0; c0 < batch; c0 += 64) {
            const int bb = c0 + ln;
            int len, ql, qs;
            pf_seq(bb, q_starts, ctx_lens, block_tables == nullptr, rows, max_blocks * block_size, batch, qs, ql, len);
            const int ncg = (ql * n_rep + PF_COLS - 1) / PF_COLS;
            int np = len > 0 ? (len + part_tokens - 1) / part_tokens : 0;
            np = np < max_parts ? np : max_parts;
            const int per_seq = np * n_kv * ncg;
            int incl = per_seq;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const int t = __shfl_up(incl, o, 64);
                if (ln >= o) incl += t;
            }
            const int total = __shfl(incl, 63, 64);
            if (pidx < base + total) {
                const bool hit = pidx >= base + incl - per_seq && pidx < base + incl;
                const uint64_t m = __ballot(hit);
                const int src = __ffsll((unsigned long long)m) - 1;
                b = c0 + src;
                const int rem = pidx - (base + __shfl(incl - per_seq, src, 64));
                const int npb = __shfl(np, src, 64);
                kg = rem / npb;
                part = rem - kg * npb;
                L = __shfl(len, src, 64);
                q_len = __shfl(ql, src, 64);
                q_start = __shfl(qs, src, 64);
                col_groups = __shfl(ncg, src, 64);
                break;
            }
            base += total;
        }
    }
    if (b < 0) return;                                        // uniform over the workgroup
    kg = __builtin_amdgcn_readfirstlane(kg);
    col_groups = __builtin_amdgcn_readfirstlane(col_groups);
    // kv heads fastest: consecutive workgroups go to consecutive XCDs, so with 8 kv heads each XCD's L2 sees the keys
    // and values of one head only; column groups from the last (longest causal range) to the first, so that the
    // long workgroups start first and the short ones fill the tail
    const int kvh = kg % n_kv;
    const int hg = col_groups - 1 - kg / n_kv;                // column group
    b = __builtin_amdgcn_readfirstlane(b);
    part = __builtin_amdgcn_readfirstlane(part);
    L = __builtin_amdgcn_readfirstlane(L);
    q_len = __builtin_amdgcn_readfirstlane(q_len);
    q_start = __builtin_amdgcn_readfirstlane(q_start);
    const int part_start = part * part_tokens;
    const int ctx_before = L - q_len;                         // cache tokens older than this step's queries
    // the farthest token any column of this group may see; partitions past it have nothing to do (the reduce kernel
    // counts partitions per query row and never reads them)
    const int Lwg = ctx_before + min(q_len, (hg * PF_COLS + PF_COLS - 1) / n_rep + 1);
    if (part_start >= Lwg) return;                            // uniform over the workgroup

    const int tid = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int rho = lane & 31;
    const int h = lane >> 5;

    // ---- this wave's 32 columns; Q as B operand: lane (rho, h) holds Q[column rho][16 j + 8 h .. +8]
    const int c0 = hg * PF_COLS + w * 32;
    const int hh = c0 + rho;
    const int qi = hh / n_rep;                                // query index of this lane's column
    const int hcol = hh - qi * n_rep;                         // head within the kv group
    const bool col_ok = qi < q_len;
    const int Lcol = col_ok ? ctx_before + qi + 1 : 0;        // causal limit of this lane's column
    const int q_first = c0 / n_rep;                           // first query of the wave
    // a wave none of whose columns sees a token of this partition only helps with the loads
    const bool wave_live = q_first < q_len && ctx_before + min(q_len, (c0 + 31) / n_rep + 1) > part_start;
    const int Lmask = ctx_before + q_first + 1;               // tiles that end at or before it need no mask
    vec8 qreg[KS];
    {
        const uint16_t* qp = q + (int64_t)(q_start + (col_ok ? qi : 0)) * q_stride +
                             (int64_t)(kvh * n_rep + (col_ok ? hcol : 0)) * D + 8 * h;
#pragma unroll
        for (int j = 0; j < KS; ++j) {
            u32x4 v = {0u, 0u, 0u, 0u};
            if (col_ok) v = *(const u32x4*)(qp + 16 * j);
            qreg[j] = bitcast<vec8>(v);
        }
    }

    f32x16 acc[DB];                                           // acc[db][i]: d = 32 db + 8 (i / 4) + 4 h + i % 4
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[db][i] = 0.f;

    const bool contiguous = block_tables == nullptr;
    const int32_t* table = block_tables + (int64_t)b * max_blocks;
    const int64_t row_bytes = kv_stride * 2;

    // ---- tile loads: load i of wave w into a sub-tile brings its rows (LW i + w) RPI .. + RPI - 1; lane = (row in
    // the group, LDS slot).  The loads of the first sub-tile come first in the arrays.
    uint32_t kcol[NI], vcol[NI];                              // byte offset of this lane's chunk within a token row
    uint32_t kofs[NI], vofs[NI];
    static_for<NI>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        constexpr bool second = i >= S0::NI;
        using SS = std::conditional_t<second, S1, S0>;
        constexpr int li = i - (second ? S0::NI : 0);
        constexpr int col0 = second ? S::W0 * 2 : 0;          // first byte of the sub-tile's columns within a head
        const int lrow = lane / SS::CPR;
        const int lslot = lane - lrow * SS::CPR;
        const int row = (SS::LW * li + w) * SS::RPI + lrow;
        const int key = (row / SS::RPB) & (SS::CPR - 1);
        const int key4 = (row / SS::RPB) & (SS::CPR / 4 - 1);
        kcol[i] = (uint32_t)(kvh * D * 2 + col0 + 16 * (lslot ^ key));
        vcol[i] = (uint32_t)(kvh * D * 2 + col0 + 16 * ((lslot - 4 * key4) & (SS::CPR - 1)));
        kofs[i] = (uint32_t)(row * (int)(kv_stride * 2)) + kcol[i];      // offsets within a whole tile
        vofs[i] = (uint32_t)(row * (int)(kv_stride * 2)) + vcol[i];
    });
    const int part_end = min(Lwg, part_start + part_tokens);
    const int ntiles = (part_end - part_start + PF_TOK - 1) / PF_TOK;

    // rows past the group's range re-read its last row (their scores are masked)
    auto issue_tile = [&](int t) {
        if (S0::LW < PA_WAVES && w >= S0::LW) return;         // narrow heads: a tile is fewer loads than waves
        const int ts = part_start + t * PF_TOK;
        uint8_t* kdst = pf_smem + (t % PF_RING) * S::BUF;
        int64_t slot0 = 0;
        if constexpr (TIB) {                                  // the tile lies inside one block: one uniform lookup
            if (contiguous) {
                slot0 = (int64_t)q_start + ts;
            } else {
                const int bi = ts / block_size;
                int blk = table[bi];
                blk = (blk < 0 || blk >= num_blocks) ? 0 : blk;   // never leave the cache allocation
                slot0 = (int64_t)blk * block_size + (ts - bi * block_size);
            }
        }
        const int last_row = Lwg - 1 - ts;
        if (TIB && last_row >= PF_TOK - 1) {                  // whole tile inside one block: constant lane offsets
            const uint8_t* kb = (const uint8_t*)kc + slot0 * row_bytes;
            const uint8_t* vb = (const uint8_t*)vc + slot0 * row_bytes;
            static_for<NI>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                constexpr bool second = i >= S0::NI;
                using SS = std::conditional_t<second, S1, S0>;
                constexpr int li = i - (second ? S0::NI : 0);
                uint8_t* dst = kdst + (second ? S::SUB1 : 0) + (SS::LW * li + w) * SS::RPI * SS::ROWB;
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(kb + kofs[i]),
                                                 (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(vb + vofs[i]),
                                                 (__attribute__((address_space(3))) void*)(dst + S::KBYTES), 16, 0, 0);
            });
            return;
        }
        static_for<NI>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            constexpr bool second = i >= S0::NI;
            using SS = std::conditional_t<second, S1, S0>;
            constexpr int li = i - (second ? S0::NI : 0);
            const int r0 = (SS::LW * li + w) * SS::RPI;
            uint8_t* dst = kdst + (second ? S::SUB1 : 0) + r0 * SS::ROWB;
            const int rc = min(r0 + lane / SS::CPR, last_row);
            const uint8_t *kp, *vp;
            if constexpr (TIB) {                              // uniform base, 32-bit lane offset
                const uint32_t lo = (uint32_t)(rc * (int)row_bytes);
                kp = (const uint8_t*)kc + slot0 * row_bytes + (lo + kcol[i]);
                vp = (const uint8_t*)vc + slot0 * row_bytes + (lo + vcol[i]);
            } else {
                const int tok = ts + rc;
                const int bi = tok / block_size;
                int blk = table[bi];
                blk = (blk < 0 || blk >= num_blocks) ? 0 : blk;
                const int64_t off = ((int64_t)blk * block_size + (tok - bi * block_size)) * row_bytes;
                kp = (const uint8_t*)kc + off + kcol[i];
                vp = (const uint8_t*)vc + off + vcol[i];
            }
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)kp,
                                             (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)vp,
                                             (__attribute__((address_space(3))) void*)(dst + S::KBYTES), 16, 0, 0);
        });
    };

    // ---- operand read addresses within a ring buffer (the buffer is a compile-time offset of the read)
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)pf_smem;
    uint32_t klane[KS];                                       // K: row rho, chunk 2 j + h of k-step j, permuted
    static_for<KS>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        constexpr bool second = j >= KS0;
        using SS = std::conditional_t<second, S1, S0>;
        constexpr int lj = j - (second ? KS0 : 0);
        const uint32_t kx = (uint32_t)((16 * h) ^ (16 * ((rho / SS::RPB) & (SS::CPR - 1))));
        klane[j] = lds0 + (second ? S::SUB1 : 0) + rho * SS::ROWB + ((32u * lj) ^ kx);
    });
    const int jj = rho & 15;
    const int tq = jj >> 2;                                   // token of the quad this lane names
    uint32_t vlane[DB];
    static_for<DB>([&](auto dc) {
        constexpr int db = decltype(dc)::value;
        constexpr bool second = db >= DB0;
        using SS = std::conditional_t<second, S1, S0>;
        constexpr int ldb = db - (second ? DB0 : 0);
        const int vkey4 = ((4 * h + tq) / SS::RPB) & (SS::CPR / 4 - 1);
        const int vchunk = (rho & 16) / 8 + ((jj & 3) >> 1) + 4 * vkey4;
        const uint32_t vrow = lds0 + S::KBYTES + (second ? S::SUB1 : 0) + (4 * h + tq) * SS::ROWB + (jj & 1) * 8;
        vlane[db] = vrow + 16 * ((vchunk + 4 * ldb) & (SS::CPR - 1));
    });

    // a column can find a whole tile masked before it has seen any token; starting the running maximum above the
    // mask value makes those probabilities 2^(-huge) = 0 instead of 2^0.  Maxima are kept in raw score units: the
    // (positive) softmax scale is applied inside the exponent.
    // m_run follows the running maximum lazily: it moves only when the maximum exceeds it by more than 2^8 in
    // probability (moving it means rescaling the accumulators); probabilities then lie in (0, 256], which bf16 and
    // fp16 hold with the same relative precision, and the result does not depend on the reference point.
    float m_run = 0.5f * PA_NEG, l_run = 0.f;
    const float lazy = 8.0f / scale_log2;

    // One tile, living in ring buffer R = t mod 3 (a compile-time constant of the step): scores, softmax, PV product,
    // one phase after the other.  A wave does not overlap its own MFMAs with its own vector instructions, so nothing
    // is gained by interleaving the phases of neighbouring tiles inside a wave; the other waves of the SIMD (3
    // workgroups are resident per compute unit) fill the gaps.  The LDS reads run P operands ahead of the MFMAs.
    auto step = [&](int t, auto ring_c) {
        constexpr int R = decltype(ring_c)::value;
        constexpr int OFF = R * S::BUF, P = 4;
        const int ts = part_start + t * PF_TOK;

        // ---- S^T[token, col] = K[token, :] . Q[col, :]
        f32x16 sc;
        {
            u32x4 ka[P];
            auto fetch = [&](auto mc) {
                constexpr int m = decltype(mc)::value;
                if constexpr (m < KS) ka[m % P] = lds_read16_at<OFF>(klane[m]);
            };
            __builtin_amdgcn_sched_barrier(0);
            static_for<(P < KS ? P : KS)>(fetch);
            static_for<KS>([&](auto mc) {
                constexpr int m = decltype(mc)::value;
                constexpr int left = KS - 1 - m;
                wait_lds_reads<(left < P - 1 ? left : P - 1)>();
                if constexpr (m == 0) {
                    f32x16 z;
#pragma unroll
                    for (int e = 0; e < 16; ++e) z[e] = 0.f;
                    sc = T::mfma32(bitcast<vec8>(ka[m % P]), qreg[m], z);
                } else {
                    sc = T::mfma32(bitcast<vec8>(ka[m % P]), qreg[m], sc);
                }
                __builtin_amdgcn_sched_barrier(0);
                fetch(std::integral_constant<int, m + P>{});
            });
        }
        if (ts + PF_TOK > Lmask) {                            // tokens hidden from a column leave its scores
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int tok = ts + 8 * (i >> 2) + 4 * h + (i & 3);
                sc[i] = tok < Lcol ? sc[i] : PA_NEG;
            }
        }
        float tmax = sc[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) tmax = fmaxf(tmax, sc[i]);
        tmax = max_xor32(tmax);
        const float m_new = tmax > m_run + lazy ? tmax : m_run;
        if (__builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {      // the reference point moves: rare
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * scale_log2);
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < DB; ++db) acc[db] *= alpha;
            m_run = m_new;
        }
        const float nm = -m_run * scale_log2;
        // probabilities, rounded to T; the denominator sums them as the PV product sees them
        uint32_t pp[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float p0 = __builtin_amdgcn_exp2f(fmaf(sc[2 * k], scale_log2, nm));
            const float p1 = __builtin_amdgcn_exp2f(fmaf(sc[2 * k + 1], scale_log2, nm));
            pp[k] = pack2<T>(p0, p1);
            l_run = T::sum2(pp[k], l_run);
        }
        const vec8 pf0 = bitcast<vec8>((u32x4){pp[0], pp[1], pp[2], pp[3]});
        const vec8 pf1 = bitcast<vec8>((u32x4){pp[4], pp[5], pp[6], pp[7]});

        // ---- O^T[d, col] += V^T[d, token] . P^T[token, col]: MFMA v = DB th + db (token half th, d block db), two
        // transposing reads each
        {
            u32x2 lo[P], hi[P];
            auto fetch = [&](auto vc_) {
                constexpr int v = decltype(vc_)::value;
                if constexpr (v < NV) {
                    constexpr int th = v / DB, db = v % DB;
                    constexpr int ROWB = db >= DB0 ? S1::ROWB : S0::ROWB;
                    lo[v % P] = lds_read_tr16_at<OFF + 16 * th * ROWB>(vlane[db]);
                    hi[v % P] = lds_read_tr16_at<OFF + (16 * th + 8) * ROWB>(vlane[db]);
                }
            };
            __builtin_amdgcn_sched_barrier(0);
            static_for<(P < NV ? P : NV)>(fetch);
            static_for<NV>([&](auto vc_) {
                constexpr int v = decltype(vc_)::value;
                constexpr int th = v / DB, db = v % DB;
                constexpr int left = NV - 1 - v;
                wait_lds_reads<2 * (left < P - 1 ? left : P - 1)>();
                acc[db] = T::mfma32(bitcast<vec8>((u32x4){lo[v % P][0], lo[v % P][1], hi[v % P][0], hi[v % P][1]}),
                                    th ? pf1 : pf0, acc[db]);
                __builtin_amdgcn_sched_barrier(0);
                fetch(std::integral_constant<int, v + P>{});
            });
        }
    };

    issue_tile(0);
    if (ntiles > 1) issue_tile(1);
#pragma unroll
    for (int j = 0; j < KS; ++j) asm volatile("" : "+v"(qreg[j]));   // the query is complete before the loop
    // tile t has landed for every wave (tile t + 1 may still be on its way), and every wave is done with tile t - 1,
    // whose buffer takes tile t + 2
    auto sync_issue = [&](int t) {
        __builtin_amdgcn_sched_barrier(0);
        if (t + 1 < ntiles) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(2 * NI) : "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        if (t + 2 < ntiles) issue_tile(t + 2);
    };
    constexpr std::integral_constant<int, 0> r0{};
    constexpr std::integral_constant<int, 1> r1{};
    constexpr std::integral_constant<int, 2> r2{};
    int t = 0;
#pragma unroll 1
    for (; t + 2 < ntiles; t += 3) {
        sync_issue(t);
        if (wave_live) step(t, r0);
        sync_issue(t + 1);
        if (wave_live) step(t + 1, r1);
        sync_issue(t + 2);
        if (wave_live) step(t + 2, r2);
    }
    if (t < ntiles) {
        sync_issue(t);
        if (wave_live) step(t, r0);
        if (++t < ntiles) {
            sync_issue(t);
            if (wave_live) step(t, r1);
        }
    }

    // ---- every lane writes its column's values: 4 consecutive d per accumulator quad
    l_run += __shfl_xor(l_run, 32, 64);
    if (!col_ok) return;
    const int64_t gh = (int64_t)(q_start + qi) * n_heads + kvh * n_rep + hcol;
    if (max_parts == 1) {
        const float inv = 1.0f / l_run;
        uint16_t* dst = out + gh * D + 4 * h;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4)
                *(u32x2*)(dst + 32 * db + 8 * q4) =
                    (u32x2){pack2<T>(acc[db][4 * q4] * inv, acc[db][4 * q4 + 1] * inv),
                            pack2<T>(acc[db][4 * q4 + 2] * inv, acc[db][4 * q4 + 3] * inv)};
    } else {
        const int64_t pi = gh * max_parts + part;
        float* dst = part_out + pi * D + 4 * h;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4)
                *(f32x4*)(dst + 32 * db + 8 * q4) =
                    (f32x4){acc[db][4 * q4], acc[db][4 * q4 + 1], acc[db][4 * q4 + 2], acc[db][4 * q4 + 3]};
        if (h == 0) {
            part_ml[pi * 2] = m_run * scale_log2;
            part_ml[pi * 2 + 1] = l_run;
        }
    }
}

// Causal limit (number of cache tokens visible) of query row `row` in a prefill step; 0 for a row that belongs to
// no sequence (before q_starts[0], from q_starts[batch] on, or beyond its sequence's context).
__device__ inline int pf_row_limit(int row, const int32_t* __restrict__ q_starts,
                                   const int32_t* __restrict__ ctx_lens, bool contiguous, int rows, int max_ctx,
                                   int batch) {
    int lo = 0, hi = batch;                                   // last sequence with q_starts[s] <= row
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (q_starts[mid] <= row) lo = mid; else hi = mid;
    }
    int qs, ql, len;
    pf_seq(lo, q_starts, ctx_lens, contiguous, rows, max_ctx, batch, qs, ql, len);
    const int qi = row - qs;
    return (qi >= 0 && qi < ql) ? len - ql + qi + 1 : 0;
}

// Combine the partitions of one (sequence, head): out = sum_p 2^(m_p - M) acc_p / sum_p 2^(m_p - M) l_p.
// One workgroup of D threads per (head, sequence).  The per-partition (max, sum) pairs are read one per lane
// and reduced across the wave; the weighted accumulator sum runs 8 independent loads deep.
// PF: blockIdx.y is a query row; its sequence is found in q_starts and its context is its causal limit.  Rows that
// belong to no sequence (beyond q_starts[batch], or beyond a sequence's context) are written as zeros.
// One output element from up to 16 partitions: (max, sum) pairs mv / lv and the partition accumulators pv of its
// column (entries past the partition count hold PA_NEG, 0, 0 and contribute nothing).
__device__ __forceinline__ float pa_combine16(const float* mv, const float* lv, const float* pv) {
    float M = PA_NEG;
#pragma unroll
    for (int p = 0; p < 16; ++p) M = fmaxf(M, mv[p]);
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int p = 0; p < 16; ++p) {
        const float f = __builtin_amdgcn_exp2f(mv[p] - M);
        den = __fmaf_rn(f, lv[p], den);
        num = __fmaf_rn(f, pv[p], num);
    }
    return __fdiv_rn(num, den);
}

// Threads of the combine kernel: one per output column, and never less than a whole wave (the branch for more than
// 16 partitions spreads the partitions over the 64 lanes of a wave; with head_dim 32 the upper lanes only take
// part in that and own no column).
template <int D>
constexpr int PA_REDUCE_THREADS = D < 64 ? 64 : D;

template <typename T, int D, bool PF>
__global__ __launch_bounds__(PA_REDUCE_THREADS<D>) void paged_attention_reduce_kernel(uint16_t* __restrict__ out,
                                                                  const float* __restrict__ part_out,
                                                                  const float* __restrict__ part_ml,
                                                                  const int32_t* __restrict__ ctx_lens, int n_heads,
                                                                  int max_parts, int part_tokens,
                                                                  const int32_t* __restrict__ q_starts, int batch,
                                                                  bool contiguous, int max_ctx) {
    __shared__ float s_f[64];
    const int h = blockIdx.x, b = blockIdx.y;                 // b: sequence (decode) or query row (PF)
    const bool own = (int)threadIdx.x < D;                    // this thread owns an output column
    const int d = own ? threadIdx.x : 0;
    const int lane = threadIdx.x & 63;
    const int L = PF ? pf_row_limit(b, q_starts, ctx_lens, contiguous, gridDim.y, max_ctx, batch) : ctx_lens[b];
    const int64_t gh = (int64_t)b * n_heads + h;
    int np = L <= 0 ? 0 : (L + part_tokens - 1) / part_tokens;
    np = np < max_parts ? np : max_parts;
    if (np == 0) {
        if (own) out[gh * D + d] = 0;
        return;
    }
    const float* ml = part_ml + gh * max_parts * 2;
    const float* po = part_out + gh * max_parts * D + d;
    if (np <= 16) {
        if (!own) return;
        // common case: every load of the row (the (max, sum) pairs and this thread's accumulator column) is issued
        // at once, one memory round trip instead of three dependent ones
        float mv[16], lv[16], pv[16];
#pragma unroll
        for (int p = 0; p < 16; ++p) {
            const bool on = p < np;
            mv[p] = on ? ml[2 * p] : PA_NEG;
            lv[p] = on ? ml[2 * p + 1] : 0.f;
            pv[p] = on ? po[(int64_t)p * D] : 0.f;
        }
        out[gh * D + d] = T::from_float(pa_combine16(mv, lv, pv));
        return;
    }
    // pass 1: global maximum (every wave computes it for itself)
    float M = PA_NEG;
    for (int p0 = 0; p0 < np; p0 += 64) {
        const int p = p0 + lane;
        M = fmaxf(M, p < np ? ml[2 * p] : PA_NEG);
    }
    M = wave_max(M);
    // pass 2: weights, denominator, weighted sum, 64 partitions at a time
    float num = 0.f, den = 0.f;
    for (int p0 = 0; p0 < np; p0 += 64) {
        const int p = p0 + lane;
        float f = 0.f, l = 0.f;
        if (p < np) {
            f = __builtin_amdgcn_exp2f(ml[2 * p] - M);
            l = ml[2 * p + 1];
        }
        den += wave_sum(f * l);
        __syncthreads();                                      // previous chunk's weights are no longer needed
        if (threadIdx.x < 64) s_f[lane] = f;
        __syncthreads();
        const int cnt = min(64, np - p0);
        int q = 0;
        for (; q + 8 <= cnt; q += 8) {
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = po[(int64_t)(p0 + q + i) * D];
#pragma unroll
            for (int i = 0; i < 8; ++i) num += s_f[q + i] * v[i];
        }
        for (; q < cnt; ++q) num += s_f[q] * po[(int64_t)(p0 + q) * D];
    }
    if (own) out[gh * D + d] = T::from_float(num / den);
}

// The partition combine of a decode step together with the per-token quantisation of the attention output row (all
// heads of a sequence) that a W8A8 output projection wants: one workgroup per sequence, a thread per 8 consecutive
// elements of one head; at most 16 partitions and 512 threads (n_heads * D <= 4096).  out receives the same bits as
// paged_attention_reduce_kernel writes, xq / x_scale what the per-token quantisation kernel makes of that row.
constexpr int PA_RQ_THREADS = 512;
template <typename T, int D>
__global__ __launch_bounds__(PA_RQ_THREADS) void paged_attention_reduce_quant_kernel(
    uint16_t* __restrict__ out, int8_t* __restrict__ xq, float* __restrict__ x_scale,
    const float* __restrict__ part_out, const float* __restrict__ part_ml, const int32_t* __restrict__ ctx_lens,
    const float* __restrict__ smooth, int n_heads, int max_parts, int part_tokens, int tiled) {
    __shared__ float red[PA_RQ_THREADS / 64];
    const int b = blockIdx.x;
    const int cols = n_heads * D;
    const int c = threadIdx.x;                                // 8-element piece of the row
    const bool on_row = c * 8 < cols;
    const int L = ctx_lens[b];
    int np = L <= 0 ? 0 : (L + part_tokens - 1) / part_tokens;
    np = np < max_parts ? np : max_parts;
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = 0.f;
    if (on_row && np > 0) {
        const int h = (c * 8) / D, d = (c * 8) % D;
        const int64_t gh = (int64_t)b * n_heads + h;
        const float* ml = part_ml + gh * max_parts * 2;
        const float* po = part_out + gh * max_parts * D + d;
        float mv[16], lv[16], pv[8][16];
#pragma unroll
        for (int p = 0; p < 16; ++p) {
            const bool on = p < np;
            mv[p] = on ? ml[2 * p] : PA_NEG;
            lv[p] = on ? ml[2 * p + 1] : 0.f;
            f32x4 a = {0.f, 0.f, 0.f, 0.f}, bq = {0.f, 0.f, 0.f, 0.f};
            if (on) {
                a = *(const f32x4*)(po + (int64_t)p * D);
                bq = *(const f32x4*)(po + (int64_t)p * D + 4);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                pv[i][p] = a[i];
                pv[4 + i][p] = bq[i];
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = pa_combine16(mv, lv, pv[i]);
    }
    float amax = 0.f;
    if (on_row) {
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = pack2<T>(v[2 * i], v[2 * i + 1]);
        *(u32x4*)(out + (int64_t)b * cols + c * 8) = o;
        unpack8<T>(o, v);                                     // the rounded row, as the quantisation kernel reads it
        amax = smooth_absmax8(v, smooth, c * 8);
    }
    amax = block_max(amax, red);
    const float s = __fdiv_rn(amax, 127.0f);
    const float safe = s > 0.f ? s : 1.0f;
    if (threadIdx.x == 0) x_scale[b] = s;
    if (on_row) quant_store8(xq, v, safe, b, c * 8, cols, gridDim.x, tiled);
}

// Partition size rule shared by the workspace query and the launch: 256-token partitions keep the tail of
// the last round of workgroups short; very long contexts use 512 to halve the partial traffic.
static inline int pa_tiles_per_wave(int64_t max_context) { return max_context > 16384 ? 4 : 2; }
// int8 caches halve the bytes per tile, which leaves the fixed cost of a workgroup (work-list scan, query load,
// first tile, merge) exposed: twice the tokens per workgroup at every context length (fewer partitions than the
// workspace query, which does not know the cache type, sizes for).
static inline int pa_launch_tiles_per_wave(int64_t max_context, bool kv8) {
    return kv8 ? 4 : pa_tiles_per_wave(max_context);
}

// Per-token quantisation of the output rows requested together with the attention itself.
struct PaQuantArgs {
    int8_t* xq;
    float* x_scale;
    const float* smooth;
    int layout;
};

template <typename T, int D, bool KV8>
int launch_pa(void* out, const void* query, const void* key_cache, const void* value_cache,
              const int32_t* block_tables, const int32_t* context_lens, int batch, int n_heads, int n_kv,
              int block_size, int max_blocks, int num_blocks, float scale, int64_t q_stride, void* workspace,
              hipStream_t st, const float* kv_scale, const float* kv_offset, const PaQuantArgs* qa = nullptr) {
    const int n_rep = n_heads / n_kv;
    const int head_groups = (n_rep + 15) / 16;
    const int64_t max_ctx = (int64_t)max_blocks * block_size;
    const int tpw = pa_launch_tiles_per_wave(max_ctx, KV8);
    const int part_tokens = tpw * PA_WAVE_TOKENS;
    const int max_parts = (int)((max_ctx + part_tokens - 1) / part_tokens);
    float* part_out = (float*)workspace;
    float* part_ml = part_out ? part_out + (int64_t)batch * n_heads * max_parts * D : nullptr;
    const float scale_log2 = scale * 1.4426950408889634f;
    dim3 grid((unsigned)((int64_t)batch * max_parts * n_kv * head_groups));
    const bool tib = block_size % PA_TILE == 0;               // a 32-token tile never straddles two blocks
#define PA_LAUNCH(TPWV, TIBV)                                                                                    \
    hipLaunchKernelGGL((paged_attention_kernel<T, D, TPWV, false, KV8, TIBV>), grid, dim3(PA_WAVES * 64), 0, st,  \
                       (uint16_t*)out, part_out, part_ml, (const uint16_t*)query, (const uint16_t*)key_cache,      \
                       (const uint16_t*)value_cache, block_tables, context_lens, n_heads, n_kv, n_rep, head_groups, \
                       block_size, max_blocks, num_blocks, max_parts, scale_log2, q_stride, batch,                 \
                       (const int32_t*)nullptr, 0, (int64_t)0, 0, kv_scale, kv_offset)
    if (tpw == 2) {
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

// zero rows of sequences with no context when the single-partition path (which skips them) is used
__global__ void pa_zero_empty_kernel(uint16_t* __restrict__ out, const int32_t* __restrict__ ctx_lens, int row) {
    const int b = blockIdx.x;
    if (ctx_lens[b] > 0) return;
    for (int i = threadIdx.x; i < row; i += blockDim.x) out[(int64_t)b * row + i] = 0;
}

// ---- prefill --------------------------------------------------------------------------------------------------
// Partitioning rule shared by the workspace query and the launch.  A workgroup serves 128 (query, head) columns of
// one kv head (16 with an int8 cache); when the query rows alone give the chip enough workgroups one partition spans the
// whole context and no partials are written, otherwise the context is cut so that at least 512 workgroups exist.
struct PfPlan {
    int part_tokens;
    int max_parts;
    int64_t col_groups16, col_groups128;                      // upper bounds over the batch, per column-group width
};

static inline PfPlan pf_plan(int batch, int64_t total_q, int n_heads, int n_kv, int64_t max_ctx) {
    const int n_rep = n_heads / n_kv;
    PfPlan p;
    p.col_groups16 = (total_q * n_rep + 15) / 16 + batch;     // each sequence rounds its own columns up
    p.col_groups128 = (total_q * n_rep + PF_COLS - 1) / PF_COLS + batch;
    // column groups over the batch: at least one per sequence that brings a query
    const int64_t groups = std::max<int64_t>((total_q * n_rep + PF_COLS - 1) / PF_COLS, std::min<int64_t>(batch, total_q));
    const int64_t wgs = std::max<int64_t>(1, groups) * n_kv;
    int64_t want = (512 + wgs - 1) / wgs;                     // 2 workgroups per CU are resident at a time
    const int64_t most = std::max<int64_t>(1, (max_ctx + 255) / 256);
    want = std::min(want, most);
    int64_t pt = (max_ctx + want - 1) / want;
    pt = std::max<int64_t>(PA_WAVE_TOKENS, (pt + PA_WAVE_TOKENS - 1) / PA_WAVE_TOKENS * PA_WAVE_TOKENS);
    p.part_tokens = (int)pt;
    p.max_parts = (int)std::max<int64_t>(1, (max_ctx + pt - 1) / pt);
    return p;
}

// Zero the rows the single-partition prefill path never writes (rows of no sequence): one workgroup per sequence
// takes the rows between the sequence's last query and the next sequence's first (the end of the output for the
// last sequence), the first workgroup also those before the first sequence.  Usually there are none.
__global__ void pf_zero_rows_kernel(uint16_t* __restrict__ out, const int32_t* __restrict__ q_starts,
                                    const int32_t* __restrict__ ctx_lens, bool contiguous, int max_ctx, int batch,
                                    int row, int rows) {
    const int s = blockIdx.x;
    int qs, ql, len;
    pf_seq(s, q_starts, ctx_lens, contiguous, rows, max_ctx, batch, qs, ql, len);
    const int64_t lo = qs < 0 ? 0 : (int64_t)qs + ql;
    int64_t hi = s + 1 < batch ? q_starts[s + 1] : rows;
    hi = hi > rows ? rows : hi;
    const u32x4 z = {0u, 0u, 0u, 0u};
    for (int64_t r = lo; r < hi; ++r)
        for (int i = threadIdx.x * 8; i < row; i += blockDim.x * 8) *(u32x4*)(out + r * row + i) = z;
    if (s == 0) {
        int64_t first = q_starts[0];
        first = first > rows ? rows : first;
        for (int64_t r = 0; r < first; ++r)
            for (int i = threadIdx.x * 8; i < row; i += blockDim.x * 8) *(u32x4*)(out + r * row + i) = z;
    }
}

template <typename T, int D, bool KV8>
int launch_pf(void* out, const void* query, const void* key_cache, const void* value_cache,
              const int32_t* block_tables, const int32_t* context_lens, const int32_t* q_starts, int batch,
              int total_q, int n_heads, int n_kv, int block_size, int max_blocks, int num_blocks, float scale,
              int64_t q_stride, int64_t kv_stride, void* workspace, hipStream_t st, const float* kv_scale,
              const float* kv_offset) {
    const int n_rep = n_heads / n_kv;
    const bool contiguous = block_tables == nullptr;
    const PfPlan plan = pf_plan(batch, total_q, n_heads, n_kv, contiguous ? total_q : (int64_t)max_blocks * block_size);
    float* part_out = plan.max_parts > 1 ? (float*)workspace : nullptr;
    float* part_ml = part_out ? part_out + (int64_t)total_q * n_heads * plan.max_parts * D : nullptr;
    const float scale_log2 = scale * 1.4426950408889634f;
    const int64_t wgs = (KV8 ? plan.col_groups16 : plan.col_groups128) * n_kv * plan.max_parts;
    if (wgs > 0x7fffffffLL) {
        mf_set_error("paged_attention_prefill: %lld workgroups exceed the grid limit", (long long)wgs);
        return 1;
    }
    if (plan.max_parts == 1) {
        hipLaunchKernelGGL(pf_zero_rows_kernel, dim3(batch), dim3(256), 0, st, (uint16_t*)out, q_starts, context_lens,
                           contiguous, max_blocks * block_size, batch, n_heads * D, total_q);
        int rc = MF_LAUNCH_CHECK();
        if (rc) return rc;
    }
    if constexpr (KV8) {
        const bool tib = block_size % PA_TILE == 0;           // a 32-token tile never straddles two blocks
#define PF_LAUNCH(TIBV)                                                                                           \
    hipLaunchKernelGGL((paged_attention_kernel<T, D, 2, true, true, TIBV>), dim3((unsigned)wgs),                   \
                       dim3(PA_WAVES * 64), 0, st, (uint16_t*)out, part_out, part_ml, (const uint16_t*)query,      \
                       (const uint16_t*)key_cache, (const uint16_t*)value_cache, block_tables, context_lens,       \
                       n_heads, n_kv, n_rep, (n_rep + 15) / 16, block_size, max_blocks, num_blocks, plan.max_parts, \
                       scale_log2, q_stride, batch, q_starts, plan.part_tokens, kv_stride, total_q, kv_scale,      \
                       kv_offset)
        if (tib) PF_LAUNCH(true);
        else PF_LAUNCH(false);
#undef PF_LAUNCH
    } else {
        const bool tib = contiguous || block_size % PF_TOK == 0;   // a staged tile never straddles two blocks
        static bool lds_set[2][MF_MAX_DEVICES] = {};          // the tile buffers exceed the default dynamic LDS limit
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return (int)e;
#define PF_LAUNCH(TIBV)                                                                                           \
    {                                                                                                             \
        auto kern = prefill_attention_kernel<T, D, TIBV>;                                                         \
        if (dev < 0 || dev >= MF_MAX_DEVICES || !lds_set[TIBV][dev]) {                                            \
            e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,                \
                                    PfSmem<D>::BYTES);                                                            \
            if (e != hipSuccess) return (int)e;                                                                   \
            if (dev >= 0 && dev < MF_MAX_DEVICES) lds_set[TIBV][dev] = true;                                      \
        }                                                                                                         \
        hipLaunchKernelGGL(kern, dim3((unsigned)wgs), dim3(PA_WAVES * 64), PfSmem<D>::BYTES, st, (uint16_t*)out,  \
                           part_out, part_ml, (const uint16_t*)query, (const uint16_t*)key_cache,                 \
                           (const uint16_t*)value_cache, block_tables, context_lens, n_heads, n_kv, n_rep,        \
                           block_size, max_blocks, num_blocks, plan.max_parts, scale_log2, q_stride, batch,       \
                           q_starts, plan.part_tokens, kv_stride, total_q);                                       \
    }
        if (tib) PF_LAUNCH(true)
        else PF_LAUNCH(false)
#undef PF_LAUNCH
    }
    int rc = MF_LAUNCH_CHECK();
    if (rc) return rc;
    if (plan.max_parts > 1) {
        hipLaunchKernelGGL((paged_attention_reduce_kernel<T, D, true>), dim3(n_heads, total_q),
                           dim3(PA_REDUCE_THREADS<D>), 0, st,
                           (uint16_t*)out, part_out, part_ml, context_lens, n_heads, plan.max_parts,
                           plan.part_tokens, q_starts, batch, contiguous, max_blocks * block_size);
        rc = MF_LAUNCH_CHECK();
    }
    return rc;
}

}  // namespace

extern "C" size_t mf_paged_attention_prefill_workspace_bytes(int batch, int total_q, int n_heads, int n_kv_heads,
                                                             int head_dim, int max_context) {
    if (batch <= 0 || total_q <= 0 || n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads) return 0;
    const PfPlan plan = pf_plan(batch, total_q, n_heads, n_kv_heads, max_context);
    if (plan.max_parts <= 1) return 0;
    return (size_t)total_q * n_heads * plan.max_parts * (head_dim + 2) * sizeof(float);
}

static int pa_prefill_entry(void* out, const void* query, const void* key_cache, const void* value_cache,
                            const int32_t* block_tables, const int32_t* context_lens, const int32_t* q_starts,
                            int batch, int total_q, int n_heads, int n_kv_heads, int head_dim, int block_size,
                            int max_blocks_per_seq, int num_blocks, float scale, int64_t q_row_stride,
                            int64_t kv_row_stride, int dtype, void* workspace, size_t workspace_bytes, void* stream,
                            bool kv8, const float* kv_scale, const float* kv_offset) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "paged_attention_prefill: dtype must be bf16 or fp16");
    MF_REQUIRE(!kv8 || (kv_scale && block_tables), "paged_attention_prefill: an int8 cache needs its scales and a block table");
    MF_REQUIRE(batch >= 0 && total_q >= 0, "paged_attention_prefill: negative batch or row count");
    if (batch == 0 || total_q == 0) return 0;
    MF_REQUIRE(out && query && key_cache && value_cache && q_starts, "paged_attention_prefill: null argument");
    const bool contiguous = block_tables == nullptr;
    MF_REQUIRE(contiguous || context_lens, "paged_attention_prefill: block_tables without context_lens");
    MF_REQUIRE(scale > 0.f, "paged_attention_prefill: the softmax scale must be positive");
    MF_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
               "paged_attention_prefill: n_heads (%d) must be a positive multiple of n_kv_heads (%d)", n_heads,
               n_kv_heads);
    MF_REQUIRE(head_dim == 32 || head_dim == 64 || head_dim == 128 || (head_dim == 192 && !kv8),
               "paged_attention_prefill: head_dim %d not supported (32, 64, 128; 192 with a 16-bit cache)", head_dim);
    MF_REQUIRE(contiguous || (block_size > 0 && max_blocks_per_seq > 0 && num_blocks > 0),
               "paged_attention_prefill: bad block geometry");
    MF_REQUIRE(contiguous || (int64_t)block_size * max_blocks_per_seq <= 0x7fffffffLL,
               "paged_attention_prefill: context capacity overflows int");
    if (kv_row_stride <= 0) kv_row_stride = (int64_t)n_kv_heads * head_dim;
    MF_REQUIRE(kv_row_stride >= (int64_t)n_kv_heads * head_dim && kv_row_stride % 8 == 0,
               "paged_attention_prefill: key/value row stride must be >= n_kv_heads*head_dim and a multiple of 8");
    MF_REQUIRE(contiguous || kv_row_stride == (int64_t)n_kv_heads * head_dim,
               "paged_attention_prefill: a paged cache has dense rows");
    if (q_row_stride <= 0) q_row_stride = (int64_t)n_heads * head_dim;
    MF_REQUIRE(q_row_stride >= (int64_t)n_heads * head_dim && q_row_stride % 8 == 0,
               "paged_attention_prefill: query row stride must be >= n_heads*head_dim and a multiple of 8 elements");
    MF_REQUIRE((((uintptr_t)out | (uintptr_t)query | (uintptr_t)key_cache | (uintptr_t)value_cache) & 15) == 0,
               "paged_attention_prefill: out / query / caches must be 16-byte aligned");
    const size_t need = mf_paged_attention_prefill_workspace_bytes(
        batch, total_q, n_heads, n_kv_heads, head_dim, contiguous ? total_q : max_blocks_per_seq * block_size);
    MF_REQUIRE(need == 0 || (workspace && workspace_bytes >= need),
               "paged_attention_prefill: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    MF_REQUIRE(need == 0 || ((uintptr_t)workspace & 15) == 0,
               "paged_attention_prefill: workspace must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
#define PF_CASE(TT, DD)                                                                                            \
    return kv8 ? launch_pf<TT, DD, true>(out, query, key_cache, value_cache, block_tables, context_lens, q_starts, \
                                         batch, total_q, n_heads, n_kv_heads, block_size, max_blocks_per_seq,      \
                                         num_blocks, scale, q_row_stride, kv_row_stride, workspace, st, kv_scale,  \
                                         kv_offset)                                                                \
               : launch_pf<TT, DD, false>(out, query, key_cache, value_cache, block_tables, context_lens, q_starts, \
                                          batch, total_q, n_heads, n_kv_heads, block_size, max_blocks_per_seq,     \
                                          num_blocks, scale, q_row_stride, kv_row_stride, workspace, st, nullptr,  \
                                          nullptr)
#define PF_CASE192(TT)                                                                                             \
    return launch_pf<TT, 192, false>(out, query, key_cache, value_cache, block_tables, context_lens, q_starts, batch, \
                                     total_q, n_heads, n_kv_heads, block_size, max_blocks_per_seq, num_blocks, scale, \
                                     q_row_stride, kv_row_stride, workspace, st, nullptr, nullptr)
    if (dtype == MF_BF16) {
        if (head_dim == 32) PF_CASE(BF16, 32);
        if (head_dim == 64) PF_CASE(BF16, 64);
        if (head_dim == 192) PF_CASE192(BF16);
        PF_CASE(BF16, 128);
    } else {
        if (head_dim == 32) PF_CASE(FP16, 32);
        if (head_dim == 64) PF_CASE(FP16, 64);
        if (head_dim == 192) PF_CASE192(FP16);
        PF_CASE(FP16, 128);
    }
#undef PF_CASE192
#undef PF_CASE
}

extern "C" int mf_paged_attention_prefill(void* out, const void* query, const void* key_cache,
                                          const void* value_cache, const int32_t* block_tables,
                                          const int32_t* context_lens, const int32_t* q_starts, int batch,
                                          int total_q, int n_heads, int n_kv_heads, int head_dim, int block_size,
                                          int max_blocks_per_seq, int num_blocks, float scale, int64_t q_row_stride,
                                          int64_t kv_row_stride, int dtype, void* workspace,
                                          size_t workspace_bytes, void* stream) {
    return pa_prefill_entry(out, query, key_cache, value_cache, block_tables, context_lens, q_starts, batch, total_q,
                            n_heads, n_kv_heads, head_dim, block_size, max_blocks_per_seq, num_blocks, scale,
                            q_row_stride, kv_row_stride, dtype, workspace, workspace_bytes, stream, false, nullptr,
                            nullptr);
}

extern "C" int mf_paged_attention_prefill_int8kv(void* out, const void* query, const void* key_cache,
                                                 const void* value_cache, const int32_t* block_tables,
                                                 const int32_t* context_lens, const int32_t* q_starts,
                                                 const float* antiquant_scale, const float* antiquant_offset,
                                                 int batch, int total_q, int n_heads, int n_kv_heads, int head_dim,
                                                 int block_size, int max_blocks_per_seq, int num_blocks, float scale,
                                                 int64_t q_row_stride, int dtype, void* workspace,
                                                 size_t workspace_bytes, void* stream) {
    return pa_prefill_entry(out, query, key_cache, value_cache, block_tables, context_lens, q_starts, batch, total_q,
                            n_heads, n_kv_heads, head_dim, block_size, max_blocks_per_seq, num_blocks, scale,
                            q_row_stride, 0, dtype, workspace, workspace_bytes, stream, true, antiquant_scale,
                            antiquant_offset);
}

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
                           void* stream, bool kv8, const float* kv_scale, const float* kv_offset,
                           const PaQuantArgs* qa = nullptr) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "paged_attention: dtype must be bf16 or fp16");
    MF_REQUIRE(!kv8 || kv_scale, "paged_attention: an int8 cache needs its scales");
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
    // with one partition the attention kernel writes the output rows itself and skips sequences without context
    const int64_t launch_part_tokens =
        (int64_t)pa_launch_tiles_per_wave((int64_t)max_blocks_per_seq * block_size, kv8) * PA_WAVE_TOKENS;
    if ((int64_t)max_blocks_per_seq * block_size <= launch_part_tokens) {
        hipLaunchKernelGGL(pa_zero_empty_kernel, dim3(batch), dim3(128), 0, st, (uint16_t*)out, context_lens,
                           n_heads * head_dim);
        int rc = MF_LAUNCH_CHECK();
        if (rc) return rc;
    }
    void* ws = need ? workspace : nullptr;
#define PA_CASE(TT, DD)                                                                                        \
    return kv8 ? launch_pa<TT, DD, true>(out, query, key_cache, value_cache, block_tables, context_lens, batch, \
                                         n_heads, n_kv_heads, block_size, max_blocks_per_seq, num_blocks, scale, \
                                         q_row_stride, ws, st, kv_scale, kv_offset, qa)                        \
               : launch_pa<TT, DD, false>(out, query, key_cache, value_cache, block_tables, context_lens, batch, \
                                          n_heads, n_kv_heads, block_size, max_blocks_per_seq, num_blocks, scale, \
                                          q_row_stride, ws, st, nullptr, nullptr, qa)
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

extern "C" int mf_paged_attention_decode(void* out, const void* query, const void* key_cache,
                                         const void* value_cache, const int32_t* block_tables,
                                         const int32_t* context_lens, int batch, int n_heads, int n_kv_heads,
                                         int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
                                         float scale, int64_t q_row_stride, int dtype, void* workspace,
                                         size_t workspace_bytes, void* stream) {
    return pa_decode_entry(out, query, key_cache, value_cache, block_tables, context_lens, batch, n_heads,
                           n_kv_heads, head_dim, block_size, max_blocks_per_seq, num_blocks, scale, q_row_stride,
                           dtype, workspace, workspace_bytes, stream, false, nullptr, nullptr);
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
                           dtype, workspace, workspace_bytes, stream, false, nullptr, nullptr, &qa);
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
                           dtype, workspace, workspace_bytes, stream, true, antiquant_scale, antiquant_offset);
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
                           dtype, ws, (size_t)MF_PA_STATIC_SCRATCH_BYTES, stream, false, nullptr, nullptr);
}
