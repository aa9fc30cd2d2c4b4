// Kernels shared by the decode and the prefill side of paged attention on gfx950: the 16-column kernel (decode: one
// query row per sequence; also the prefill path of int8 caches) and the partition-combine kernels.  Included by
// paged_attention.hip (decode entry points) and prefill_attention.hip (prefill entry points).
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
#pragma once
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

// K / V rows are read once per launch: the loads carry the non-temporal hint, so that the stream does not push
// what the launch does re-read (the fp32 partial results on their way to the combine kernel, and whatever the kernels
// before and after it keep in the caches) out of L2.  Measured on the 64-sequence ragged batch: attention with its
// combine 119 -> 109 us, and the layer step around it 208.5 -> 185.8 us on the same box.
__device__ __forceinline__ u32x4 pa_stream_load(const uint8_t* p) { return __builtin_nontemporal_load((const u32x4*)p); }

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
// KVQ = 2: int8 caches quantised per token (one scale per cached token row, shared by its heads): kv_scale points at
// the key scales and kv_offset at the value scales, float [num_blocks * block_size] each, indexed by slot.  The score
// of a token is multiplied by its key scale, its probability by its value scale before it is rounded to T for the PV
// product (the denominator sums the unscaled probabilities).  The scales of a tile are loaded one tile ahead, like
// the tile itself.  KVQ = 1 is the per-channel form above, 0 a 16-bit cache.
template <typename T, int D, int TPW, bool PF, int KVQ, bool TIB>
// Decode over an int8 cache keeps half the prefetch registers of a 16-bit one and fits four workgroups on a compute
// unit (128 registers; measured 6 % faster than with three); the 16-bit kernel needs 166 registers for its two
// prefetched tiles and gained nothing from a one-tile variant that fits four, so it stays at three.
__global__ __launch_bounds__(PA_WAVES * 64, (!PF && KVQ == 1 && TIB) ? 4 : 3) void paged_attention_kernel(
    uint16_t* __restrict__ out, float* __restrict__ part_out, float* __restrict__ part_ml,
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc,
    const int32_t* __restrict__ block_tables, const int32_t* __restrict__ ctx_lens, int n_heads, int n_kv,
    int n_rep, int head_groups, int block_size, int max_blocks, int num_blocks, int max_parts,
    float scale_log2, int64_t q_stride, int batch, const int32_t* __restrict__ q_starts, int pf_part_tokens,
    int64_t pf_kv_stride, int pf_rows, const float* __restrict__ kv_scale, const float* __restrict__ kv_offset) {
    using vec8 = typename T::vec8;
    constexpr bool KV8 = KVQ != 0;
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
    int used = 0;                                             // work items that exist (known where none was found)
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
        used = base;
    }
    kg = __builtin_amdgcn_readfirstlane(kg);
    if (b < 0) {                                              // uniform over the workgroup
        // Decode with one partition per sequence writes the output rows itself, and a sequence without context has no
        // workgroup: the nkg workgroups it leaves over write its zeros (left-over workgroup u takes kv group
        // u % nkg of the (u / nkg)-th empty sequence).
        if constexpr (!PF) {
            if (max_parts == 1) {
                const int u = (int)blockIdx.x - used;
                const int rank = u / nkg, kgz = u - rank * nkg;
                const int ln = threadIdx.x & 63;
                int seen = 0, target = -1;
                for (int c0 = 0; c0 < batch; c0 += 64) {
                    const int bb = c0 + ln;
                    const bool empty = bb < batch && min(ctx_lens[bb], max_blocks * block_size) <= 0;
                    const uint64_t m = __ballot(empty);
                    const int cnt = __popcll(m);
                    if (rank < seen + cnt) {
                        const int before = __popcll(m & ((1ull << ln) - 1ull));
                        const uint64_t hm = __ballot(empty && before == rank - seen);
                        target = c0 + __ffsll((unsigned long long)hm) - 1;
                        break;
                    }
                    seen += cnt;
                }
                if (target >= 0 && rank >= 0) {
                    const int kvz = kgz / head_groups, hgz = kgz - kvz * head_groups;
                    const int heads = min(16, n_rep - 16 * hgz);
                    uint16_t* row = out + ((int64_t)target * n_heads + kvz * n_rep + 16 * hgz) * D;
                    for (int i = threadIdx.x; i < heads * D; i += PA_WAVES * 64) row[i] = 0;
                }
            }
        }
        return;
    }
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
            if constexpr (KVQ == 1) {                         // fold the per-channel key scale into the query
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
                    reg[i] = pa_stream_load(base + (int64_t)(RPI * i) * row_bytes + lane_off);
            } else {                                                               // the same loads, rows clamped
                const int last_row = L - tstart - 1;                               // uniform, >= 0 for a live tile
#pragma unroll
                for (int i = 0; i < NI; ++i)
                    reg[i] = pa_stream_load(base + (uint32_t)(min(lrow + RPI * i, last_row) * (int)row_bytes) + lane_col);
            }
        } else {
#pragma unroll
            for (int i = 0; i < NI; ++i) reg[i] = pa_stream_load((const uint8_t*)cache + row_offset(slot0, tstart, i));
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

    // KVQ = 2: the scales of tokens tstart + 16 s + 4 g .. + 3 (the tokens whose scores this lane holds), s = 0, 1.
    // Groups past the context read the scales of the sequence's first tokens: their scores are masked and their
    // value scales replaced by zero where they are used.
    auto load_scales = [&](f32x4* reg, const float* __restrict__ cache, int64_t slot0, int tstart) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            if constexpr (TIB) {
                reg[s2] = *(const f32x4*)(cache + slot0 + 16 * s2 + 4 * g);       // inside the tile's block
            } else {
                int tok = tstart + 16 * s2 + 4 * g;                                // block sizes are multiples of 4
                tok = tok < L ? tok : 0;
                const int bi = tok / block_size;
                int blk = table[bi];
                blk = (blk < 0 || blk >= num_blocks) ? 0 : blk;
                reg[s2] = *(const f32x4*)(cache + (int64_t)blk * block_size + (tok - bi * block_size));
            }
        }
    };

    const int tstep = PA_WAVES * PA_TILE;
    const int tfirst = part_start + wu * PA_TILE;
    int64_t slot_cur = tile_slot(tfirst), slot_nxt = tile_slot(tfirst + tstep);
    u32x4 kreg[NI], vreg[NI];
    [[maybe_unused]] f32x4 ksc[2], vsc[2];                    // KVQ = 2: token scales of the tile in kreg / vreg
    if (ntiles > 0) {
        load_tile(kreg, kc, slot_cur, tfirst);
        load_tile(vreg, vc, slot_cur, tfirst);
        if constexpr (KVQ == 2) {
            load_scales(ksc, kv_scale, slot_cur, tfirst);
            load_scales(vsc, kv_offset, slot_cur, tfirst);
        }
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
        // KVQ = 2: this tile's token scales leave their registers here; the next tile's follow one tile ahead of use
        [[maybe_unused]] f32x4 kts[2], vts[2];
        if constexpr (KVQ == 2) {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                kts[s] = ksc[s] * scale_log2;
                vts[s] = vsc[s];
            }
            if constexpr (more) {
                load_scales(ksc, kv_scale, slot_nxt, tnext);
                load_scales(vsc, kv_offset, slot_nxt, tnext);
            }
        }
        float tmax = PA_NEG;
        if (tstart + PA_TILE <= Lmask) {                      // every token of the tile is visible to every column
#pragma unroll
            for (int s = 0; s < 2; ++s)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if constexpr (KVQ == 2) sc[s][i] *= kts[s][i]; else sc[s][i] *= scale_log2;
                    tmax = fmaxf(tmax, sc[s][i]);
                }
        } else {
#pragma unroll
            for (int s = 0; s < 2; ++s)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int tok = tstart + s * 16 + 4 * g + i;
                    float scaled;
                    if constexpr (KVQ == 2) {
                        scaled = sc[s][i] * kts[s][i];
                        if (tok >= L) vts[s][i] = 0.f;        // whatever the cache holds there
                    } else {
                        scaled = sc[s][i] * scale_log2;
                    }
                    const float v = tok < Lcol ? scaled : PA_NEG;
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
            if constexpr (KVQ == 2) {                         // the value's token scale rides on its probability
                psum += (p0 + p1) + (p2 + p3);
                pp[2 * s] = pack2<T>(p0 * vts[s][0], p1 * vts[s][1]);
                pp[2 * s + 1] = pack2<T>(p2 * vts[s][2], p3 * vts[s][3]);
                continue;
            }
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
        if constexpr (KVQ == 1) {                             // value dequantisation, linear in (sum, lt)
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

}  // namespace
