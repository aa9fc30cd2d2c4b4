// Multi-latent attention (MLA) decode over the paged latent cache, gfx950.
//
// One cache row per token holds the compressed key/value latent and the rotary key: [kv_lora_rank | rope] =
// 512 + 64 bf16/fp16 values.  Every query head attends with the whole 576-wide row as its key and the first
// 512 values of the same row as its value (the projections that make queries and outputs live in that space are
// absorbed into the caller's GEMMs).  With all heads sharing one row the op is bound by the matrix cores, not by
// HBM: 2 * (576 + 512) flops per (token, head) against 1152 bytes per token.
//
// Work decomposition
//   One workgroup of 4 wavefronts, one per SIMD, owns one token partition of one sequence and a block of 128 heads:
//   wave w serves heads 32 w .. + 31 and all 512 value columns.  The cache tile of 32 tokens (36 KB) is fetched once
//   per workgroup and shared by the 4 waves.
//   S^T[token, head] = C[token, :576] . Q[head, :576]     36 k-steps of mfma_f32_32x32x16
//   online softmax in fp32 (exp2 domain), probabilities rounded to the cache dtype
//   O^T[d, head] += C^T[d, token] . P^T[token, head]       the tile is read back through the transposing LDS read
//   No merge inside the workgroup is needed: every wave owns its heads.  Partitions of a sequence are combined by
//   mla_reduce_kernel.
#include "common.h"

namespace {

constexpr int MLA_DK = 576;                                   // key width: latent + rotary
constexpr int MLA_DV = 512;                                   // value width: the latent
constexpr int MLA_TILE = 32;                                  // tokens per tile
constexpr int MLA_CPR = MLA_DK * 2 / 16;                      // 16-byte chunks per row
constexpr float MLA_NEG = -1.0e30f;

// A wave holds 16 accumulator blocks of 32 x 32 (256 registers per lane) in the accumulation registers and its 32
// query rows (144 registers) in the ordinary ones: one wave per SIMD has 512 registers.  No wave computes a score
// twice, and a cache tile is fetched once per 128 heads.  Tiles of 32 tokens (36 KB) go from global memory straight
// into a ring of four LDS buffers, two tiles ahead, one barrier per tile.  Such a load writes 64 consecutive 16-byte
// slots, so the 1152-byte rows cannot be padded; the chunks of a row are permuted within aligned groups of 8 through
// the global address each lane supplies: chunk c of row t sits in slot (c & ~7) | ((c & 7) ^ s(t)),
// s(t) = 4 (t/2 & 1) + (t/4 & 3).  Rows are 72 slots apart (8 mod 16), so the 16 rows of one chunk that an operand
// read serves together, and the 4 tokens x 64 bytes that a transposing read serves together, both fall on 16
// different 16-byte bank groups.
// The reference point of the exponentials follows the running maximum lazily: it moves only when the maximum exceeds
// it by more than 2^8 in probability, because moving it means rescaling 256 accumulator registers per lane;
// probabilities then lie in (0, 256], which bf16 and fp16 hold with the same relative precision, and the result
// does not depend on the reference point.
constexpr int M2_WAVES = 4;
constexpr int M2_HEADS = 32 * M2_WAVES;                       // heads per workgroup
constexpr int M2_ROWB = MLA_DK * 2;                           // bytes per staged row
constexpr int M2_TILE_BYTES = MLA_TILE * M2_ROWB;
constexpr int M2_RING = 4;
constexpr int M2_SMEM = M2_RING * M2_TILE_BYTES;
constexpr int M2_LOADS = M2_TILE_BYTES / 1024 / M2_WAVES;     // wave-wide 1 KB loads per wave per tile
constexpr int M2_KS = MLA_DK / 16;                            // k-steps of the score product
constexpr int M2_DB = MLA_DV / 32;                            // 32-column blocks of the output
constexpr int M2_NV = 2 * M2_DB;                              // PV MFMAs per tile
// cache policy of the latent-row loads (the aux operand of the LDS-direct load; bit 1 = non-temporal): a row is read
// once per launch by the one workgroup that owns its head block, so it need not stay in any cache.  Measured over
// caches that no call has touched just before: attention 79.2 -> 77.9 us, the layer step around it 171.5 -> 168.4 us.
constexpr int M2_AUX = 2;
constexpr float M2_LAZY = 8.0f;                               // log2 of the largest probability before the reference moves
static_assert(M2_TILE_BYTES % (1024 * M2_WAVES) == 0 && M2_SMEM <= 160 * 1024, "tile loads / LDS capacity");

__device__ __forceinline__ int m2_key(int row) { return 4 * ((row >> 1) & 1) + ((row >> 2) & 3); }

// Smallest partition the kernels use: at most 32 partitions per sequence, never less than 256 tokens.
__host__ __device__ inline int mla_min_part(int max_ctx) {
    const int p = ((max_ctx + 31) / 32 + 31) / 32 * 32;
    return p > 256 ? p : 256;
}
// Workgroups the partition rule below can produce at most.
__host__ __device__ inline int mla_free_slots(int batch, int head_blocks, int n_slots) {
    const int f = n_slots - batch * head_blocks;
    return f > n_slots / 4 ? f : n_slots / 4;
}
// Workgroups the launch provides: the partition rule never produces more.
__host__ __device__ inline int mla_grid(int batch, int head_blocks, int n_slots) {
    return mla_free_slots(batch, head_blocks, n_slots) + batch * head_blocks;
}
// The partition rule: the largest number of 32-token tiles a partition may hold, T, chosen from the actual lengths so
// that the workgroups fit the chip's n_slots compute units in one round (one workgroup is resident per unit).
// Sequence b with t_b tiles is cut into ceil(t_b / T) partitions of ceil(t_b / partitions) tiles each (equal up to one
// tile).  T0 = total tiles * head_blocks / (n_slots - batch * head_blocks) always fits, because sum_b ceil(t_b / T) *
// head_blocks <= total * head_blocks / T + batch * head_blocks; that bound charges every sequence a whole extra
// partition, so four smaller candidates T0 - k max(1, T0 / 16) are counted exactly (one packed reduction) and the
// smallest that fits wins: the longest workgroup, which sets the kernel's time, gets that much shorter.  Every wave
// that calls this gets the same value (the main kernel and the reduce kernel both do).  first: this lane's entry of
// the first 64 lengths (0 beyond the batch), which the caller has loaded already.
__device__ inline int mla_tiles_of(int len, int max_ctx) {
    const int l = len < 0 ? 0 : (len > max_ctx ? max_ctx : len);
    return (l + MLA_TILE - 1) / MLA_TILE;
}
__device__ inline int mla_part_tiles(const int32_t* __restrict__ ctx_lens, int batch, int max_ctx, int head_blocks,
                                     int n_slots, int first) {
    const int ln = threadIdx.x & 63;
    const int t_first = mla_tiles_of(first, max_ctx);
    int64_t total = t_first;
    for (int c0 = 64; c0 < batch; c0 += 64) {
        const int bb = c0 + ln;
        total += mla_tiles_of(bb < batch ? ctx_lens[bb] : 0, max_ctx);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) total += __shfl_xor(total, o, 64);
    const int64_t avail = mla_free_slots(batch, head_blocks, n_slots);
    const int lo = mla_min_part(max_ctx) / MLA_TILE;
    const int64_t t0l = (total * head_blocks + avail - 1) / avail;
    const int t0 = __builtin_amdgcn_readfirstlane(t0l < lo ? lo : (int)t0l);
    const int step = t0 / 16 > 1 ? t0 / 16 : 1;
    if (t0 - step < lo) return t0;
    // partitions per candidate, 16 bits each (a chunk of 64 sequences adds at most 64 * 32 to a field)
    int64_t cnt[4] = {0, 0, 0, 0};
    for (int c0 = 0; c0 < batch; c0 += 64) {
        const int bb = c0 + ln;
        const int t = c0 == 0 ? t_first : mla_tiles_of(bb < batch ? ctx_lens[bb] : 0, max_ctx);
        uint64_t packed = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int cand = t0 - (k + 1) * step;
            const int parts = cand >= lo ? (t + cand - 1) / cand : 0;
            packed |= (uint64_t)parts << (16 * k);
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) packed += __shfl_xor(packed, o, 64);
#pragma unroll
        for (int k = 0; k < 4; ++k) cnt[k] += (int64_t)((packed >> (16 * k)) & 0xffff);
    }
    const int64_t grid = mla_grid(batch, head_blocks, n_slots);
    int best = t0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int cand = t0 - (k + 1) * step;
        if (cand >= lo && cnt[k] * head_blocks <= grid) best = cand;      // counts grow with k: the last fit is the smallest
    }
    return __builtin_amdgcn_readfirstlane(best);
}

template <typename T>
__global__ __launch_bounds__(M2_WAVES * 64, 1) void mla_decode_kernel(
    uint16_t* __restrict__ out, float* __restrict__ part_out, float* __restrict__ part_ml,
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ cache, const int32_t* __restrict__ block_tables,
    const int32_t* __restrict__ ctx_lens, int n_heads, int head_blocks, int block_size, int max_blocks,
    int num_blocks, int max_parts, int n_slots, float scale_log2, int64_t q_stride, int batch,
    int32_t* __restrict__ plan_word) {
    using vec8 = typename T::vec8;
    extern __shared__ __attribute__((aligned(16))) uint8_t mla_smem[];
    // the first 64 lengths serve the partition rule and the work list: one trip to memory for both
    const int len_first = (int)(threadIdx.x & 63) < batch ? ctx_lens[threadIdx.x & 63] : 0;
    // (a scalar: it comes out of a cross-lane reduction, and everything derived from it, the tile addresses and the
    // branches on tile positions above all, would otherwise be computed per lane)
    const int max_ctx = max_blocks * block_size;
    const int cap_tiles = __builtin_amdgcn_readfirstlane(
        max_parts == 1 ? (max_ctx + MLA_TILE - 1) / MLA_TILE
                       : mla_part_tiles(ctx_lens, batch, max_ctx, head_blocks, n_slots, len_first));
    if (plan_word && blockIdx.x == 0 && threadIdx.x == 0) *plan_word = cap_tiles;   // for the reduce kernel

    // ---- work list: (sequence, partition, head block) triples that exist, from a prefix sum over the lengths
    int b = -1, part = 0, hb = 0, L = 0, nparts = 1;
    {
        const int pidx = blockIdx.x;
        const int ln = threadIdx.x & 63;
        int base = 0;
        for (int c0 = 0; c0 < batch; c0 += 64) {
            const int bb = c0 + ln;
            const int len = min(c0 == 0 ? len_first : (bb < batch ? ctx_lens[bb] : 0), max_ctx);
            int np = (mla_tiles_of(len, max_ctx) + cap_tiles - 1) / cap_tiles;
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
                nparts = __shfl(np, src, 64);
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
    nparts = __builtin_amdgcn_readfirstlane(nparts);

    const int tid = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int rho = lane & 31, h = lane >> 5;
    const int head = hb * M2_HEADS + w * 32 + rho;
    const bool head_ok = head < n_heads;

    // ---- Q as MFMA B operand: lane (rho, h) holds Q[head rho][16 j + 8 h .. + 8]
    vec8 qreg[M2_KS];
    {
        const uint16_t* qp = q + (int64_t)b * q_stride + (int64_t)(head_ok ? head : 0) * MLA_DK + 8 * h;
#pragma unroll
        for (int j = 0; j < M2_KS; ++j) {
            u32x4 v = {0u, 0u, 0u, 0u};
            if (head_ok) v = *(const u32x4*)(qp + 16 * j);
            qreg[j] = bitcast<vec8>(v);
        }
    }

    // the partitions of a sequence are equal up to one tile
    const int part_tokens = ((L + MLA_TILE - 1) / MLA_TILE + nparts - 1) / nparts * MLA_TILE;
    const int part_start = part * part_tokens;
    const int part_end = min(L, part_start + part_tokens);
    const int ntiles = (part_end - part_start + MLA_TILE - 1) / MLA_TILE;      // >= 1 for a listed partition
    const int32_t* table = block_tables + (int64_t)b * max_blocks;

    // ---- tile loads: load i of wave w fills LDS slots 64 (4 i + w) .. + 63 of the tile; slot = 72 row + position
    uint32_t lofs[M2_LOADS];                                  // byte offset of the lane's chunk within a whole tile
#pragma unroll
    for (int i = 0; i < M2_LOADS; ++i) {
        const int slot = 64 * (M2_WAVES * i + w) + lane;
        const int row = slot / MLA_CPR;
        const int pos = slot - row * MLA_CPR;
        lofs[i] = (uint32_t)(row * M2_ROWB + 16 * ((pos & ~7) | ((pos & 7) ^ m2_key(row))));   // its logical chunk
    }
    // A tile lies inside one block (host-checked).  The table entry of the block being read stays in a scalar
    // register and the next block's entry is fetched when the current one is entered, so that the lookup of a tile's
    // block (a scalar load and its wait) is not on the path of every tile.
    auto lookup = [&](int bi) {
        int blk = bi < max_blocks ? table[bi] : 0;
        return (blk < 0 || blk >= num_blocks) ? 0 : blk;      // never leave the cache allocation
    };
    int bi_cur = part_start / block_size;
    int blk_cur = lookup(bi_cur), blk_nxt = lookup(bi_cur + 1);
    // Where tile t comes from and goes to (tiles are asked for in order).
    struct TileAddr {
        const uint8_t* base;                                  // first row of the tile in the cache
        uint8_t* dst;                                         // its ring buffer
        int last_row;                                         // rows past the context re-read the last valid row
    };
    auto tile_addr = [&](int t) {
        const int ts = part_start + t * MLA_TILE;
        const int bi = ts / block_size;
        if (bi != bi_cur) {                                   // uniform: the tile enters the next block
            bi_cur = bi;
            blk_cur = blk_nxt;
            blk_nxt = lookup(bi + 1);
        }
        TileAddr a;
        a.base = (const uint8_t*)cache + ((int64_t)blk_cur * block_size + (ts - bi * block_size)) * M2_ROWB;
        a.dst = mla_smem + (t & (M2_RING - 1)) * M2_TILE_BYTES;
        a.last_row = L - 1 - ts;
        return a;
    };
    // load i of a whole tile: constant lane offsets
    auto issue_load = [&](const TileAddr& a, auto ic) {
        constexpr int i = decltype(ic)::value;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a.base + lofs[i]),
                                         (__attribute__((address_space(3))) void*)(a.dst + 1024 * (M2_WAVES * i + w)),
                                         16, 0, M2_AUX);
    };
    // all loads of a tile at once (the first tiles of a partition, and the last tile of a sequence, whose rows are
    // clamped)
    auto issue_tile = [&](const TileAddr& a) {
        if (a.last_row >= MLA_TILE - 1) {
            static_for<M2_LOADS>([&](auto ic) { issue_load(a, ic); });
            return;
        }
#pragma unroll
        for (int i = 0; i < M2_LOADS; ++i) {
            const int row = (int)(lofs[i] / M2_ROWB);
            const uint32_t off = lofs[i] - (uint32_t)(max(row - a.last_row, 0) * M2_ROWB);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a.base + off),
                                             (__attribute__((address_space(3))) void*)(a.dst + 1024 * (M2_WAVES * i + w)),
                                             16, 0, M2_AUX);
        }
    };

    // ---- operand read addresses within a ring buffer
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)mla_smem;
    // K: row rho, chunk 2 j + h = 8 (j / 4) + 2 (j % 4) + h: one address per j % 4, 128 (j / 4) is an immediate
    uint32_t klane[2][4];                                     // [half of the ring][j % 4]
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) {
        klane[0][jb] = lds0 + rho * M2_ROWB + ((32u * jb + 16u * h) ^ (16u * m2_key(rho)));
        klane[1][jb] = klane[0][jb] + 2 * M2_TILE_BYTES;
    }
    // V^T: lane j of 16 names token 16 th + 8 e + 4 h + (j >> 2) and the 4 values d = 32 db + rho0 + 4 (j & 3) ..;
    // chunk 4 db + cl: one address per (e, db % 2), the rest is an immediate
    const int jj = rho & 15, tq = jj >> 2;
    const int cl = (rho & 16) / 8 + ((jj & 3) >> 1);
    uint32_t vlane[2][2][2];                                  // [half of the ring][e][db % 2]
#pragma unroll
    for (int e = 0; e < 2; ++e)
#pragma unroll
        for (int pb = 0; pb < 2; ++pb) {
            const int key = 4 * ((tq >> 1) & 1) + ((2 * e + h) & 3);          // m2_key of that token row
            vlane[0][e][pb] = lds0 + (8 * e + 4 * h + tq) * M2_ROWB + 16 * ((4 * pb + cl) ^ key) + 8 * (jj & 1);
            vlane[1][e][pb] = vlane[0][e][pb] + 2 * M2_TILE_BYTES;
        }

    // accumulators: acc[db][i]: d = 32 db + 8 (i / 4) + 4 h + i % 4.  They live in the accumulation registers (the
    // PV MFMAs below are asm statements that name them with the "a" constraint) and leave them only for the rare
    // rescale and for the final store.
    f32x16 acc[M2_DB];
#pragma unroll
    for (int db = 0; db < M2_DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[db][i] = 0.f;
    // m_ref: the reference point of the exponentials in raw score units (the positive softmax scale is applied
    // inside the exponent); it starts above the mask value so that a fully masked tile gives zeros
    float m_ref = 0.5f * MLA_NEG, l_run = 0.f;
    const float lazy = M2_LAZY / scale_log2;

    // One tile: scores, softmax, PV product.  With one wave per SIMD nothing is gained by interleaving the matrix and
    // vector instructions of different tiles (a wave runs its own MFMAs and vector instructions one after the other),
    // so the phases follow each other; the LDS reads run four operands ahead of the MFMAs that use them.
    // The loads of tile t + 2 (its buffer is free: every wave has passed the barrier that ends tile t - 1) go out one
    // at a time between the score MFMAs, each of which waits for its predecessor anyway: issued in a block they cost
    // the wave about 60 cycles apiece.
    auto step = [&](int t, auto ring_c) {
        constexpr int R = decltype(ring_c)::value;
        constexpr int P = 4;
        TileAddr nxt = {nullptr, nullptr, 0};
        bool spread = false;                                  // uniform
        if (t + 2 < ntiles) {
            nxt = tile_addr(t + 2);
            spread = nxt.last_row >= MLA_TILE - 1;
            if (!spread) issue_tile(nxt);
        }
        // ring buffers 2 and 3 lie beyond the 16-bit offset field of an LDS read: a second set of addresses
        constexpr int OFF = (R & 1) * M2_TILE_BYTES, HI = R >> 1;
        const int ts = part_start + t * MLA_TILE;

        // ---- S^T[token, head] = C[token, :576] . Q[head, :576].  These MFMAs are asm statements as well, with the
        // scores in ordinary registers: a compiler-chosen accumulation register tuple for them would have to evict an
        // accumulator block, and the compiler would copy that block without waiting for the asm MFMAs that wrote it.
        f32x16 sc;
        {
            u32x4 ka[P];
            auto fetch = [&](auto mc) {
                constexpr int m = decltype(mc)::value;
                if constexpr (m < M2_KS) ka[m % P] = lds_read16_at<OFF + 128 * (m / 4)>(klane[HI][m % 4]);
            };
            __builtin_amdgcn_sched_barrier(0);
            static_for<P>(fetch);
            static_for<M2_KS>([&](auto mc) {
                constexpr int m = decltype(mc)::value;
                constexpr int left = M2_KS - 1 - m;
                wait_lds_reads<(left < P - 1 ? left : P - 1)>();
                if constexpr (m == 0) T::mfma32_first(sc, bitcast<vec8>(ka[m % P]), qreg[m]);
                else T::mfma32_next(sc, bitcast<vec8>(ka[m % P]), qreg[m]);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (m % 4 == 1 && m / 4 < M2_LOADS) {
                    if (spread) issue_load(nxt, std::integral_constant<int, m / 4>{});
                    __builtin_amdgcn_sched_barrier(0);
                }
                fetch(std::integral_constant<int, m + P>{});
            });
            // the compiler does not know that sc comes from matrix instructions: their 8 passes end here
            asm volatile("s_nop 15\n\ts_nop 15" : "+v"(sc));
        }
        if (ts + MLA_TILE > L) {                              // last tile of the sequence: mask what lies past it
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int tok = ts + 8 * (i >> 2) + 4 * h + (i & 3);
                sc[i] = tok < L ? sc[i] : MLA_NEG;
            }
        }
        float tmax = sc[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) tmax = fmaxf(tmax, sc[i]);
        tmax = max_xor32(tmax);
        const float m_new = tmax > m_ref + lazy ? tmax : m_ref;
        if (__builtin_amdgcn_ballot_w64(m_new != m_ref) != 0) {       // the reference point moves: rare
            const float alpha = __builtin_amdgcn_exp2f((m_ref - m_new) * scale_log2);
            l_run *= alpha;
            if (t != 0) {                                     // (the first tile always moves it, off zero accumulators)
                asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");  // the last PV MFMAs have written their registers
#pragma unroll
                for (int db = 0; db < M2_DB; ++db) {
                    asm volatile("" : "+a"(acc[db]));
                    acc[db] *= alpha;
                    asm volatile("" : "+a"(acc[db]));
                }
                asm volatile("s_nop 7" ::: "memory");
            }
            m_ref = m_new;
        }
        const float nm = -m_ref * scale_log2;
        uint32_t pp[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float p0 = __builtin_amdgcn_exp2f(fmaf(sc[2 * k], scale_log2, nm));
            const float p1 = __builtin_amdgcn_exp2f(fmaf(sc[2 * k + 1], scale_log2, nm));
            pp[k] = pack2<T>(p0, p1);
            l_run = T::sum2(pp[k], l_run);                    // sums the probabilities as the PV product sees them
        }
        const vec8 pf0 = bitcast<vec8>((u32x4){pp[0], pp[1], pp[2], pp[3]});
        const vec8 pf1 = bitcast<vec8>((u32x4){pp[4], pp[5], pp[6], pp[7]});

        // ---- O^T[d, head] += C^T[d, token] . P^T[token, head]: MFMA v = 16 th + db (token half th, column block db)
        {
            u32x2 lo[P], hi[P];
            auto fetch = [&](auto vc) {
                constexpr int v = decltype(vc)::value;
                if constexpr (v < M2_NV) {
                    constexpr int th = v / M2_DB, db = v % M2_DB;
                    lo[v % P] = lds_read_tr16_at<OFF + 16 * th * M2_ROWB + 128 * (db / 2)>(vlane[HI][0][db % 2]);
                    hi[v % P] = lds_read_tr16_at<OFF + 16 * th * M2_ROWB + 128 * (db / 2)>(vlane[HI][1][db % 2]);
                }
            };
            __builtin_amdgcn_sched_barrier(0);
            static_for<P>(fetch);
            static_for<M2_NV>([&](auto vc) {
                constexpr int v = decltype(vc)::value;
                constexpr int th = v / M2_DB, db = v % M2_DB;
                constexpr int left = M2_NV - 1 - v;
                wait_lds_reads<2 * (left < P - 1 ? left : P - 1)>();
                const u32x4 va = {lo[v % P][0], lo[v % P][1], hi[v % P][0], hi[v % P][1]};
                T::mfma32_acc(acc[db], bitcast<vec8>(va), th ? pf1 : pf0);
                __builtin_amdgcn_sched_barrier(0);
                fetch(std::integral_constant<int, v + P>{});
            });
        }
    };

    issue_tile(tile_addr(0));
    if (ntiles > 1) issue_tile(tile_addr(1));
#pragma unroll
    for (int j = 0; j < M2_KS; ++j) asm volatile("" : "+v"(qreg[j]));   // the query is complete before the loop
    // tile t has landed for every wave (tile t + 1 may still be on its way), and every wave is done with tile t - 1:
    // the buffer of tile t - 2 may take tile t + 2 from here on
    auto sync_issue = [&](int t) {
        __builtin_amdgcn_sched_barrier(0);
        if (t + 1 < ntiles) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(M2_LOADS) : "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };
    constexpr std::integral_constant<int, 0> r0{};
    constexpr std::integral_constant<int, 1> r1{};
    constexpr std::integral_constant<int, 2> r2{};
    constexpr std::integral_constant<int, 3> r3{};
    int t = 0;
#pragma unroll 1
    for (; t + 3 < ntiles; t += 4) {
        sync_issue(t);
        step(t, r0);
        sync_issue(t + 1);
        step(t + 1, r1);
        sync_issue(t + 2);
        step(t + 2, r2);
        sync_issue(t + 3);
        step(t + 3, r3);
    }
    if (t < ntiles) {
        sync_issue(t);
        step(t, r0);
        if (++t < ntiles) {
            sync_issue(t);
            step(t, r1);
            if (++t < ntiles) {
                sync_issue(t);
                step(t, r2);
            }
        }
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");              // the last PV MFMAs have written their registers

    // ---- results.  A lane holds 4 consecutive columns per accumulator quad of one head, which would make 8- and
    // 16-byte pieces in global memory; the accumulators go through LDS instead (the ring is idle now: a wave takes a
    // quarter of it, 256 columns of its 32 heads at a time, rows padded by 16 bytes against bank conflicts) and leave
    // as whole rows: 1 KB of fp32 partials, or 512 bytes of final values, per store instruction.
    l_run += __shfl_xor(l_run, 32, 64);
    __syncthreads();                                          // every wave has read its last tile
    constexpr int OROW = 256 * 4 + 16;                        // bytes per staged row of 256 fp32 columns
    static_assert(32 * OROW <= M2_SMEM / M2_WAVES, "a wave's output rows must fit its quarter of the ring");
    uint8_t* stage = mla_smem + w * (M2_SMEM / M2_WAVES);
    const int head0 = hb * M2_HEADS + w * 32;                 // first head of this wave
    const int live = min(32, n_heads - head0);                // heads of this wave that exist (may be <= 0)
    const float inv = nparts == 1 ? 1.0f / l_run : 1.0f;
    if (nparts > 1 && head_ok && h == 0) {
        const int64_t pi = ((int64_t)b * n_heads + head) * max_parts + part;
        part_ml[pi * 2] = m_ref * scale_log2;
        part_ml[pi * 2 + 1] = l_run;
    }
#pragma unroll
    for (int hv = 0; hv < 2; ++hv) {                          // unrolled: the accumulator blocks are named statically
        if (hv) __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int d8 = 0; d8 < M2_DB / 2; ++d8) {
            const int db = hv * (M2_DB / 2) + d8;
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4)
                *(f32x4*)(stage + rho * OROW + (32 * d8 + 8 * q4 + 4 * h) * 4) =
                    (f32x4){acc[db][4 * q4] * inv, acc[db][4 * q4 + 1] * inv, acc[db][4 * q4 + 2] * inv,
                            acc[db][4 * q4 + 3] * inv};
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (nparts == 1) {                                    // the only partition of its sequence: final rows
            // two heads per pass: lanes 0-31 one row, lanes 32-63 the next; 8 columns per lane
            for (int r0 = 0; r0 < live; r0 += 8) {            // 4 pairs of rows at a time
                f32x4 lo[4], hi[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int r = min(r0 + 2 * i + h, 31);
                    lo[i] = *(const f32x4*)(stage + r * OROW + rho * 32);
                    hi[i] = *(const f32x4*)(stage + r * OROW + rho * 32 + 16);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int r = r0 + 2 * i + h;
                    if (r >= live) continue;
                    const u32x4 o = {pack2<T>(lo[i][0], lo[i][1]), pack2<T>(lo[i][2], lo[i][3]),
                                     pack2<T>(hi[i][0], hi[i][1]), pack2<T>(hi[i][2], hi[i][3])};
                    *(u32x4*)(out + ((int64_t)b * n_heads + head0 + r) * MLA_DV + 256 * hv + 8 * rho) = o;
                }
            }
        } else {
            // 8 rows at a time: their LDS reads go out together, then their stores
            float* dst = part_out + (((int64_t)b * n_heads + head0) * max_parts + part) * MLA_DV + 256 * hv + 4 * lane;
            const int64_t rstride = (int64_t)max_parts * MLA_DV;
            for (int r0 = 0; r0 < live; r0 += 8) {
                f32x4 v[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = *(const f32x4*)(stage + min(r0 + i, 31) * OROW + lane * 16);
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (r0 + i < live) *(f32x4*)(dst + (r0 + i) * rstride) = v[i];
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    }
}

// Combine the partitions of (sequence, head) rows: out = sum_p 2^(m_p - M) acc_p / sum_p 2^(m_p - M) l_p.
// One workgroup of 128 threads (4 value columns each) per 4 heads of a sequence.  The partition rule's value comes
// from the word the main kernel left behind the partials, so a row costs one round trip for that word and the
// length and one for everything else: with up to 8 partitions the (max, sum) pairs and the accumulators of all four
// heads are loaded together.
constexpr int MR_THREADS = MLA_DV / 4;
constexpr int MR_HEADS = 4;
template <typename T>
__global__ __launch_bounds__(MR_THREADS) void mla_reduce_kernel(uint16_t* __restrict__ out,
                                                                const float* __restrict__ part_out,
                                                                const float* __restrict__ part_ml,
                                                                const int32_t* __restrict__ ctx_lens,
                                                                const int32_t* __restrict__ plan_word, int n_heads,
                                                                int max_parts, int max_ctx) {
    const int h0 = blockIdx.x * MR_HEADS, b = blockIdx.y, d = 4 * threadIdx.x;
    const int cap_tiles = *plan_word;
    const int L = min(ctx_lens[b], max_ctx);
    int np = (mla_tiles_of(L, max_ctx) + cap_tiles - 1) / cap_tiles;
    np = np < max_parts ? np : max_parts;
    if (np == 1) return;                                      // the main kernel wrote the final rows
    const int live = min(MR_HEADS, n_heads - h0);
    const int64_t gh0 = (int64_t)b * n_heads + h0;
    if (np == 0) {
        for (int hh = 0; hh < live; ++hh) *(u32x2*)(out + (gh0 + hh) * MLA_DV + d) = (u32x2){0u, 0u};
        return;
    }
    if (np <= 8) {
        f32x4 v[MR_HEADS][8];
        float m[MR_HEADS][8], l[MR_HEADS][8];
#pragma unroll
        for (int hh = 0; hh < MR_HEADS; ++hh) {
            const int64_t gh = gh0 + (hh < live ? hh : 0);
            const float* ml = part_ml + gh * max_parts * 2;
            const float* po = part_out + gh * max_parts * MLA_DV + d;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const bool on = i < np;
                v[hh][i] = on ? *(const f32x4*)(po + (int64_t)i * MLA_DV) : (f32x4){0.f, 0.f, 0.f, 0.f};
                m[hh][i] = on ? ml[2 * i] : MLA_NEG;
                l[hh][i] = on ? ml[2 * i + 1] : 0.f;
            }
        }
#pragma unroll
        for (int hh = 0; hh < MR_HEADS; ++hh) {
            if (hh >= live) break;
            float M = MLA_NEG;
#pragma unroll
            for (int i = 0; i < 8; ++i) M = fmaxf(M, m[hh][i]);
            f32x4 num = {0.f, 0.f, 0.f, 0.f};
            float den = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float f = i < np ? __builtin_amdgcn_exp2f(m[hh][i] - M) : 0.f;
                den += f * l[hh][i];
                num += v[hh][i] * f;
            }
            const float inv = 1.0f / den;
            *(u32x2*)(out + (gh0 + hh) * MLA_DV + d) =
                (u32x2){pack2<T>(num[0] * inv, num[1] * inv), pack2<T>(num[2] * inv, num[3] * inv)};
        }
        return;
    }
    for (int hh = 0; hh < live; ++hh) {                       // long contexts: head by head, 8 partitions at a time
        const int64_t gh = gh0 + hh;
        const float* ml = part_ml + gh * max_parts * 2;
        const float* po = part_out + gh * max_parts * MLA_DV + d;
        float M = MLA_NEG;
        for (int p = 0; p < np; ++p) M = fmaxf(M, ml[2 * p]);     // uniform addresses: broadcast loads
        f32x4 num = {0.f, 0.f, 0.f, 0.f};
        float den = 0.f;
        for (int p0 = 0; p0 < np; p0 += 8) {
            f32x4 v[8];
            float f[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const bool on = p0 + i < np;
                v[i] = on ? *(const f32x4*)(po + (int64_t)(p0 + i) * MLA_DV) : (f32x4){0.f, 0.f, 0.f, 0.f};
                f[i] = on ? __builtin_amdgcn_exp2f(ml[2 * (p0 + i)] - M) : 0.f;
                den += on ? f[i] * ml[2 * (p0 + i) + 1] : 0.f;
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) num += v[i] * f[i];
        }
        const float inv = 1.0f / den;
        *(u32x2*)(out + gh * MLA_DV + d) =
            (u32x2){pack2<T>(num[0] * inv, num[1] * inv), pack2<T>(num[2] * inv, num[3] * inv)};
    }
}

// zero the rows of sequences with no context when a single partition spans the context (the main kernel skips them)
__global__ void mla_zero_empty_kernel(uint16_t* __restrict__ out, const int32_t* __restrict__ ctx_lens, int row) {
    if (ctx_lens[blockIdx.x] > 0) return;
    for (int i = threadIdx.x; i < row; i += blockDim.x) out[(int64_t)blockIdx.x * row + i] = 0;
}

// Host side of the partition rule: the worst-case number of partitions per sequence (which sizes the workspace) and
// the number of workgroups the device-side rule can produce at most.
struct MlaPlan {
    int max_parts, head_blocks;
};
inline MlaPlan mla_plan(int n_heads, int64_t max_ctx) {
    MlaPlan p;
    p.head_blocks = (n_heads + M2_HEADS - 1) / M2_HEADS;
    const int lo = mla_min_part((int)max_ctx);
    p.max_parts = (int)std::max<int64_t>(1, (max_ctx + lo - 1) / lo);
    return p;
}

template <typename T>
int launch_mla(void* out, const void* query, const void* cache, const int32_t* block_tables,
               const int32_t* context_lens, int batch, int n_heads, int block_size, int max_blocks, int num_blocks,
               float scale, int64_t q_stride, void* workspace, hipStream_t st) {
    static bool configured[MF_MAX_DEVICES] = {};
    static int cu_count[MF_MAX_DEVICES] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MF_MAX_DEVICES) {
        mf_set_error("mla_paged_attention: device index %d outside the supported %d", dev, MF_MAX_DEVICES);
        return (int)hipErrorInvalidValue;
    }
    if (!configured[dev]) {
        e = hipFuncSetAttribute((const void*)mla_decode_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                M2_SMEM);
        if (e != hipSuccess) return (int)e;
        e = hipDeviceGetAttribute(&cu_count[dev], hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) return (int)e;
        configured[dev] = true;
    }
    const int n_slots = cu_count[dev] > 0 ? cu_count[dev] : 256;
    const int64_t max_ctx = (int64_t)max_blocks * block_size;
    const MlaPlan plan = mla_plan(n_heads, max_ctx);
    float* part_out = plan.max_parts > 1 ? (float*)workspace : nullptr;
    float* part_ml = part_out ? part_out + (int64_t)batch * n_heads * plan.max_parts * MLA_DV : nullptr;
    int32_t* plan_word = part_ml ? (int32_t*)(part_ml + (int64_t)batch * n_heads * plan.max_parts * 2) : nullptr;
    const float scale_log2 = scale * 1.4426950408889634f;
    if (plan.max_parts == 1) {
        hipLaunchKernelGGL(mla_zero_empty_kernel, dim3(batch), dim3(128), 0, st, (uint16_t*)out, context_lens,
                           n_heads * MLA_DV);
        const int rc = MF_LAUNCH_CHECK();
        if (rc) return rc;
    }
    const int64_t wgs = plan.max_parts == 1 ? (int64_t)batch * plan.head_blocks
                                            : (int64_t)mla_grid(batch, plan.head_blocks, n_slots);
    hipLaunchKernelGGL(mla_decode_kernel<T>, dim3((unsigned)wgs), dim3(M2_WAVES * 64), M2_SMEM, st, (uint16_t*)out,
                       part_out, part_ml, (const uint16_t*)query, (const uint16_t*)cache, block_tables, context_lens,
                       n_heads, plan.head_blocks, block_size, max_blocks, num_blocks, plan.max_parts, n_slots,
                       scale_log2, q_stride, batch, plan_word);
    int rc = MF_LAUNCH_CHECK();
    if (rc) return rc;
    if (plan.max_parts > 1) {
        hipLaunchKernelGGL(mla_reduce_kernel<T>, dim3((n_heads + MR_HEADS - 1) / MR_HEADS, batch), dim3(MR_THREADS), 0, st,
                           (uint16_t*)out, part_out, part_ml, context_lens, plan_word, n_heads, plan.max_parts,
                           (int)max_ctx);
        rc = MF_LAUNCH_CHECK();
    }
    return rc;
}


// ---- weight-absorbed per-head projections of a multi-latent attention layer --------------------------------------
// out[t, h, n] = sum_k x[t, h, k] * w[h, n, k]: a batch of `heads` skinny GEMMs with a different [N, K] weight per
// head and the token rows as the small side (decode: the query up-projection folded into the latent space,
// [T, 128] x [128 -> 512] per head, and the value up-projection applied to the attention output, [T, 512] x
// [512 -> 128]).  Weights (2 x 16.8 MB at 128 heads), activations and results should each cross the L2 once.  A
// workgroup of 8 waves owns one head, 128 NT channels of it (all of them at the two decode shapes) and up to 64
// tokens; wave w keeps the weight tiles of its 16 NT channels in registers, already in MFMA operand order (row, 8
// consecutive k per lane: one 16-byte load per k-step), and walks the token tiles; the rows of a token tile are read
// by all 8 waves and meet in the L1, the next tile's rows are in flight while the current one is multiplied.
// Results leave as 16-byte pieces (neighbouring lanes first swap halves so that a lane holds 8 consecutive
// channels).  No LDS, no barriers.
constexpr int AB_WAVES = 8;

template <typename T, int KS, int NT>
__global__ __launch_bounds__(AB_WAVES * 64, 1) void mla_absorb_bmm_kernel(
    uint16_t* __restrict__ out, const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, int tokens, int N,
    int wg_tokens, int64_t xs_t, int64_t xs_h, int64_t os_t, int64_t os_h) {
    using vec8 = typename T::vec8;
    constexpr int K = 32 * KS;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    const int h = blockIdx.y;
    const int nb0 = blockIdx.x * (AB_WAVES * 16 * NT) + wave * (16 * NT);
    if (nb0 >= N) return;                                     // uniform over the wave; there is no barrier below
    const int t_begin = blockIdx.z * wg_tokens;
    const int t_end = min(tokens, t_begin + wg_tokens);
    vec8 wreg[NT][KS];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int n = min(nb0 + 16 * j, N - 16) + r;          // tiles past N (a multiple of 16) repeat the last one
        const uint16_t* wp = w + ((int64_t)h * N + n) * K + 8 * g;
#pragma unroll
        for (int s = 0; s < KS; ++s) wreg[j][s] = *(const vec8*)(wp + 32 * s);
    }
    const uint16_t* xh = x + (int64_t)h * xs_h + 8 * g;
    auto load_x = [&](vec8* xv, int t0) {
        const int t = min(t0 + r, tokens - 1);                // rows past the end repeat the last one, never stored
#pragma unroll
        for (int s = 0; s < KS; ++s) xv[s] = *(const vec8*)(xh + (int64_t)t * xs_t + 32 * s);
    };
    auto tile = [&](const vec8* xv, int t0) {
        u32x2 piece[NT];                                      // channels nb0 + 16 j + 4 g .. + 3 of token t0 + r
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < KS; ++s) acc = T::mfma16(wreg[j][s], xv[s], acc);
            piece[j] = (u32x2){pack2<T>(acc[0], acc[1]), pack2<T>(acc[2], acc[3])};
        }
        const bool row_ok = t0 + r < t_end;
        uint16_t* orow = out + (int64_t)(t0 + r) * os_t + (int64_t)h * os_h + nb0;
        if constexpr (NT == 1) {
            if (row_ok) *(u32x2*)(orow + 4 * g) = piece[0];
        } else {
            // lanes g and g ^ 1 swap one piece per tile pair: the even lane ends up with channels 4 g .. 4 g + 7 of
            // the pair's first tile, the odd lane with channels 4 (g - 1) .. 4 g + 3 of its second
            const bool odd = g & 1;
#pragma unroll
            for (int m = 0; m < NT / 2; ++m) {
                const u32x2 send = odd ? piece[2 * m] : piece[2 * m + 1];
                u32x2 recv;
                recv[0] = __shfl_xor(send[0], 16, 64);
                recv[1] = __shfl_xor(send[1], 16, 64);
                const int j = 2 * m + (odd ? 1 : 0);
                const u32x4 o = odd ? (u32x4){recv[0], recv[1], piece[j][0], piece[j][1]}
                                    : (u32x4){piece[j][0], piece[j][1], recv[0], recv[1]};
                if (row_ok && nb0 + 16 * j < N) *(u32x4*)(orow + 16 * j + 4 * (g & ~1)) = o;
            }
        }
    };
    // two register sets of token rows alternate: the next tile is fetched behind the current one's products
    vec8 xa[KS], xb[KS];
    load_x(xa, t_begin);
    for (int t0 = t_begin; t0 < t_end; t0 += 32) {
        load_x(xb, t0 + 16);
        tile(xa, t0);
        if (t0 + 16 >= t_end) break;
        load_x(xa, t0 + 32);
        tile(xb, t0 + 16);
    }
}

// Long reductions (k = 256, 512: the output side, [T, 512] x [512 -> 128] per head): the token rows are the big
// operand there, and eight waves fetching the same 16 KB tile each would pull it through the L2 eight times.  The
// workgroup loads a token tile once, cooperatively and fully coalesced, into one of two LDS stages (one barrier per
// tile; 16-byte chunk c of row r sits in slot c ^ r, which spreads the 16 rows an operand read touches over all
// banks), and every wave reads its B operands from there.  One 16-channel tile per wave.
template <typename T, int KS>
__global__ __launch_bounds__(AB_WAVES * 64, 1) void mla_absorb_bmm_lds_kernel(
    uint16_t* __restrict__ out, const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, int tokens, int N,
    int wg_tokens, int64_t xs_t, int64_t xs_h, int64_t os_t, int64_t os_h) {
    using vec8 = typename T::vec8;
    constexpr int K = 32 * KS;
    constexpr int CPR = K / 8;                                // 16-byte chunks per token row
    constexpr int STAGE = 16 * K * 2;
    constexpr int XL = 16 * CPR / (AB_WAVES * 64);            // chunks per thread and tile
    static_assert(XL >= 1 && CPR >= 16, "the chunk permutation needs at least 16 chunks per row");
    __shared__ __attribute__((aligned(16))) uint8_t smem[2 * STAGE];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    const int h = blockIdx.y;
    const int nb0 = blockIdx.x * (AB_WAVES * 16) + wave * 16;
    const bool active = nb0 < N;                              // idle waves still stage rows and meet the barriers
    const int t_begin = blockIdx.z * wg_tokens;
    const int t_end = min(tokens, t_begin + wg_tokens);
    vec8 wreg[KS];
    {
        const int n = min(nb0, N - 16) + r;
        const uint16_t* wp = w + ((int64_t)h * N + n) * K + 8 * g;
#pragma unroll
        for (int s = 0; s < KS; ++s) wreg[s] = *(const vec8*)(wp + 32 * s);
    }
    const uint16_t* xh = x + (int64_t)h * xs_h;
    u32x4 stg[XL];
    auto fetch = [&](int t0) {                                // this thread's chunks of tile t0 -> registers
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const int id = threadIdx.x + i * (AB_WAVES * 64);
            const int row = id / CPR, c = id - row * CPR;
            const int t = min(t0 + row, tokens - 1);
            stg[i] = *(const u32x4*)(xh + (int64_t)t * xs_t + 8 * c);
        }
    };
    auto park = [&](int stage) {                              // registers -> LDS stage
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const int id = threadIdx.x + i * (AB_WAVES * 64);
            const int row = id / CPR, c = id - row * CPR;
            *(u32x4*)(smem + stage * STAGE + row * (K * 2) + ((c ^ row) << 4)) = stg[i];
        }
    };
    fetch(t_begin);
    park(0);
    __syncthreads();
    int stage = 0;
    for (int t0 = t_begin; t0 < t_end; t0 += 16, stage ^= 1) {
        const bool more = t0 + 16 < t_end;
        if (more) fetch(t0 + 16);                             // in flight behind this tile's products
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        const uint8_t* row = smem + stage * STAGE + r * (K * 2);
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const u32x4 xb = *(const u32x4*)(row + (((4 * s + g) ^ r) << 4));
            acc = T::mfma16(wreg[s], bitcast<vec8>(xb), acc);
        }
        if (active && t0 + r < t_end)
            *(u32x2*)(out + (int64_t)(t0 + r) * os_t + (int64_t)h * os_h + nb0 + 4 * g) =
                (u32x2){pack2<T>(acc[0], acc[1]), pack2<T>(acc[2], acc[3])};
        if (more) park(stage ^ 1);                            // last read two tiles ago, before the previous barrier
        __syncthreads();
    }
}

template <typename T>
int launch_absorb(void* out, const void* x, const void* w, int tokens, int heads, int n, int k, int64_t xs_t,
                  int64_t xs_h, int64_t os_t, int64_t os_h, hipStream_t st) {
    const int nt = k <= 128 ? 4 : 1;                          // 64 registers of weight tiles per wave (k <= 128)
    const int n_blocks = (n + AB_WAVES * 16 * nt - 1) / (AB_WAVES * 16 * nt);
    // up to 64 tokens per workgroup (the weights are re-read once per token slice, from L2); fewer when the launch
    // would otherwise leave compute units idle
    int wg_tokens = 64;
    while (wg_tokens > 16 && (int64_t)n_blocks * heads * ((tokens + wg_tokens - 1) / wg_tokens) < 256) wg_tokens >>= 1;
    const int tz = (tokens + wg_tokens - 1) / wg_tokens;
    if (tz > 65535) {
        mf_set_error("mla_absorb_bmm: %d tokens exceed the grid limit", tokens);
        return 1;
    }
    const dim3 grid(n_blocks, heads, tz);
#define ABSORB_LAUNCH(KSV, NTV)                                                                                 \
    hipLaunchKernelGGL((mla_absorb_bmm_kernel<T, KSV, NTV>), grid, dim3(AB_WAVES * 64), 0, st, (uint16_t*)out,   \
                       (const uint16_t*)x, (const uint16_t*)w, tokens, n, wg_tokens, xs_t, xs_h, os_t, os_h)
    switch (k) {
        case 64: ABSORB_LAUNCH(2, 4); break;
        case 128: ABSORB_LAUNCH(4, 4); break;
        case 256:
            hipLaunchKernelGGL((mla_absorb_bmm_lds_kernel<T, 8>), grid, dim3(AB_WAVES * 64), 0, st, (uint16_t*)out,
                               (const uint16_t*)x, (const uint16_t*)w, tokens, n, wg_tokens, xs_t, xs_h, os_t, os_h);
            break;
        default:
            hipLaunchKernelGGL((mla_absorb_bmm_lds_kernel<T, 16>), grid, dim3(AB_WAVES * 64), 0, st, (uint16_t*)out,
                               (const uint16_t*)x, (const uint16_t*)w, tokens, n, wg_tokens, xs_t, xs_h, os_t, os_h);
            break;
    }
#undef ABSORB_LAUNCH
    return MF_LAUNCH_CHECK();
}

// ---- the element-wise work between the down projections and the attention, in one launch -------------------------
// Per token: the latent part of the kv down projection is RMS-normalised, the shared rotary key part and the rotary
// part of every head's query are rotated (rotate-half with the token's cos / sin row), the normalised latent row and
// the rotated key part are written to the token's slot of the latent cache, and the rotated query part is stored
// where the caller wants it (behind the absorbed query of a decode step, or back in place for a prefill).  Rounding
// points as the separate kernels have them: the norm output is rounded to T, a rotation's two products and their
// sum are rounded one by one (rope_pair) and the result to T.
// grid (tokens, 1 + query parts): y = 0 handles the kv row (wave 0 the norm, wave 1 the key rotation), y >= 1 a
// share of the heads; a work item is 8 consecutive elements of the first half of a rotary part and their partners.
constexpr int MNR_THREADS = 256;

template <typename T>
__device__ __forceinline__ void mnr_rotate8(const uint16_t* src, uint16_t* dst0, uint16_t* dst1, const void* cos,
                                            const void* sin, int64_t trow, int i0, int half, int table_dtype) {
    float x1[8], x2[8], c1[8], s1[8], c2[8], s2[8];
    unpack8<T>(*(const u32x4*)(src + i0), x1);
    unpack8<T>(*(const u32x4*)(src + half + i0), x2);
    load8_as_float(cos, trow + i0, table_dtype, c1);
    load8_as_float(sin, trow + i0, table_dtype, s1);
    load8_as_float(cos, trow + half + i0, table_dtype, c2);
    load8_as_float(sin, trow + half + i0, table_dtype, s2);
    float o1[8], o2[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) rope_pair(x1[e], x2[e], c1[e], s1[e], c2[e], s2[e], o1[e], o2[e]);
    const u32x4 a = {pack2<T>(o1[0], o1[1]), pack2<T>(o1[2], o1[3]), pack2<T>(o1[4], o1[5]), pack2<T>(o1[6], o1[7])};
    const u32x4 b = {pack2<T>(o2[0], o2[1]), pack2<T>(o2[2], o2[3]), pack2<T>(o2[4], o2[5]), pack2<T>(o2[6], o2[7])};
    *(u32x4*)(dst0 + i0) = a;
    *(u32x4*)(dst0 + half + i0) = b;
    if (dst1) {
        *(u32x4*)(dst1 + i0) = a;
        *(u32x4*)(dst1 + half + i0) = b;
    }
}

template <typename T>
__global__ __launch_bounds__(MNR_THREADS) void mla_norm_rope_cache_kernel(
    uint16_t* __restrict__ q_rope_out, int64_t qo_token_stride, int64_t qo_head_stride, const uint16_t* __restrict__ q,
    int64_t q_token_stride, int64_t q_head_stride, uint16_t* __restrict__ kv_norm_out, uint16_t* __restrict__ k_pe_out,
    const uint16_t* __restrict__ kv, int64_t kv_token_stride, const void* __restrict__ gamma, int gamma_dtype, float eps,
    const void* __restrict__ cos, const void* __restrict__ sin, int table_dtype, uint16_t* __restrict__ cache,
    const int32_t* __restrict__ slot_mapping, int64_t num_slots, int heads, int rank, int rope) {
    const int t = blockIdx.x;
    const int half = rope >> 1;
    const int64_t trow = (int64_t)t * rope;
    const int per_head = half >> 3;                           // work items per rotary part
    if (blockIdx.y > 0) {                                     // the rotary parts of the query heads
        const int items = heads * per_head;
        for (int it = (blockIdx.y - 1) * MNR_THREADS + threadIdx.x; it < items; it += (gridDim.y - 1) * MNR_THREADS) {
            const int h = it / per_head, i0 = 8 * (it - h * per_head);
            mnr_rotate8<T>(q + (int64_t)t * q_token_stride + (int64_t)h * q_head_stride,
                           q_rope_out + (int64_t)t * qo_token_stride + (int64_t)h * qo_head_stride, nullptr, cos, sin,
                           trow, i0, half, table_dtype);
        }
        return;
    }
    int64_t slot = cache ? slot_mapping[t] : -1;
    uint16_t* crow = (slot >= 0 && slot < num_slots) ? cache + slot * (int64_t)(rank + rope) : nullptr;
    const uint16_t* row = kv + (int64_t)t * kv_token_stride;
    const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (wv == 0) {                                            // RMSNorm of the latent part: one wave
        const int nvec = rank >> 3;
        float ss = 0.f;
        for (int c = lane; c < nvec; c += 64) {
            float v[8];
            unpack8<T>(*(const u32x4*)(row + 8 * c), v);
#pragma unroll
            for (int i = 0; i < 8; ++i) ss = __fmaf_rn(v[i], v[i], ss);
        }
        ss = wave_sum(ss);
        const float inv = rsqrtf(ss / (float)rank + eps);
        for (int c = lane; c < nvec; c += 64) {
            float v[8], gm[8];
            unpack8<T>(*(const u32x4*)(row + 8 * c), v);
            load8_as_float(gamma, 8 * c, gamma_dtype, gm);
            u32x4 o;
#pragma unroll
            for (int i = 0; i < 4; ++i) o[i] = pack2<T>(v[2 * i] * inv * gm[2 * i], v[2 * i + 1] * inv * gm[2 * i + 1]);
            if (kv_norm_out) *(u32x4*)(kv_norm_out + (int64_t)t * rank + 8 * c) = o;
            if (crow) *(u32x4*)(crow + 8 * c) = o;
        }
    } else if (wv == 1) {                                     // the rotary key part, shared by the heads
        // destinations: the dense copy when asked for, the cache row when the slot is live; with neither, nothing
        uint16_t* d0 = k_pe_out ? k_pe_out + (int64_t)t * rope : (crow ? crow + rank : nullptr);
        uint16_t* d1 = (k_pe_out && crow) ? crow + rank : nullptr;
        if (d0 && lane < per_head) mnr_rotate8<T>(row + rank, d0, d1, cos, sin, trow, 8 * lane, half, table_dtype);
    }
}

}  // namespace

extern "C" size_t mf_mla_paged_attention_workspace_bytes(int batch, int n_heads, int max_context) {
    if (batch <= 0 || n_heads <= 0 || max_context <= 0) return 0;
    const MlaPlan plan = mla_plan(n_heads, max_context);
    if (plan.max_parts <= 1) return 0;
    // partial accumulators, (max, sum) pairs, and the word that carries the partition rule's value to the reduce kernel
    return (size_t)batch * n_heads * plan.max_parts * (MLA_DV + 2) * sizeof(float) + 16;
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
    MF_REQUIRE(scale > 0.f, "mla_paged_attention: the softmax scale must be positive");
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

extern "C" int mf_mla_absorb_bmm(void* out, const void* x, const void* w, int tokens, int heads, int n, int k,
                                 int64_t x_token_stride, int64_t x_head_stride, int64_t out_token_stride,
                                 int64_t out_head_stride, int dtype, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "mla_absorb_bmm: dtype must be bf16 or fp16");
    MF_REQUIRE(tokens >= 0 && heads >= 0, "mla_absorb_bmm: negative size");
    if (tokens == 0 || heads == 0) return 0;
    MF_REQUIRE(out && x && w, "mla_absorb_bmm: null argument");
    MF_REQUIRE(k == 64 || k == 128 || k == 256 || k == 512, "mla_absorb_bmm: k = %d not supported (64, 128, 256, 512)", k);
    MF_REQUIRE(n > 0 && n % 16 == 0, "mla_absorb_bmm: n (%d) must be a positive multiple of 16", n);
    MF_REQUIRE(heads <= 65535, "mla_absorb_bmm: at most 65535 heads");
    MF_REQUIRE(x_head_stride >= k && x_token_stride >= k && x_head_stride % 8 == 0 && x_token_stride % 8 == 0,
               "mla_absorb_bmm: x strides must be >= k and multiples of 8 elements");
    MF_REQUIRE(out_head_stride >= n && out_token_stride >= n && out_head_stride % 8 == 0 && out_token_stride % 8 == 0,
               "mla_absorb_bmm: out strides must be >= n and multiples of 8 elements");
    MF_REQUIRE((((uintptr_t)x | (uintptr_t)w | (uintptr_t)out) & 15) == 0,
               "mla_absorb_bmm: x / w / out must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    if (dtype == MF_BF16)
        return launch_absorb<BF16>(out, x, w, tokens, heads, n, k, x_token_stride, x_head_stride, out_token_stride,
                                   out_head_stride, st);
    return launch_absorb<FP16>(out, x, w, tokens, heads, n, k, x_token_stride, x_head_stride, out_token_stride,
                               out_head_stride, st);
}

extern "C" int mf_mla_norm_rope_cache(void* q_rope_out, int64_t q_out_token_stride, int64_t q_out_head_stride,
                                      const void* q_rope, int64_t q_token_stride, int64_t q_head_stride,
                                      void* kv_norm_out, void* k_pe_out, const void* kv, int64_t kv_token_stride,
                                      const void* gamma, int gamma_dtype, float eps, const void* cos, const void* sin,
                                      int table_dtype, void* latent_cache, const int32_t* slot_mapping,
                                      int64_t num_slots, int tokens, int heads, int rank, int rope, int dtype,
                                      void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "mla_norm_rope_cache: dtype must be bf16 or fp16");
    MF_REQUIRE(gamma_dtype == MF_BF16 || gamma_dtype == MF_FP16 || gamma_dtype == MF_FP32,
               "mla_norm_rope_cache: bad gamma dtype");
    MF_REQUIRE(table_dtype == MF_BF16 || table_dtype == MF_FP16 || table_dtype == MF_FP32,
               "mla_norm_rope_cache: bad table dtype");
    if (tokens <= 0) return 0;
    MF_REQUIRE(q_rope_out && q_rope && kv && gamma && cos && sin, "mla_norm_rope_cache: null argument");
    MF_REQUIRE(!latent_cache || (slot_mapping && num_slots > 0), "mla_norm_rope_cache: a cache needs slots");
    MF_REQUIRE(heads > 0 && rank > 0 && rank % 8 == 0 && rope > 0 && rope % 16 == 0 && rope <= 1024,
               "mla_norm_rope_cache: rank (%d) must be a multiple of 8, rope (%d) a multiple of 16", rank, rope);
    MF_REQUIRE(q_out_token_stride % 8 == 0 && q_out_head_stride % 8 == 0 && q_token_stride % 8 == 0 &&
                   q_head_stride % 8 == 0 && kv_token_stride % 8 == 0 && kv_token_stride >= rank + rope,
               "mla_norm_rope_cache: strides must be multiples of 8 elements, kv rows at least rank + rope long");
    MF_REQUIRE((((uintptr_t)q_rope_out | (uintptr_t)q_rope | (uintptr_t)kv | (uintptr_t)kv_norm_out |
                 (uintptr_t)k_pe_out | (uintptr_t)latent_cache | (uintptr_t)gamma | (uintptr_t)cos | (uintptr_t)sin) & 15) == 0,
               "mla_norm_rope_cache: pointers must be 16-byte aligned");
    const int items = heads * (rope >> 4);
    const dim3 grid(tokens, 1 + (items + MNR_THREADS - 1) / MNR_THREADS);
#define MNR_LAUNCH(TT)                                                                                            \
    hipLaunchKernelGGL(mla_norm_rope_cache_kernel<TT>, grid, dim3(MNR_THREADS), 0, (hipStream_t)stream,           \
                       (uint16_t*)q_rope_out, q_out_token_stride, q_out_head_stride, (const uint16_t*)q_rope,     \
                       q_token_stride, q_head_stride, (uint16_t*)kv_norm_out, (uint16_t*)k_pe_out,                \
                       (const uint16_t*)kv, kv_token_stride, gamma, gamma_dtype, eps, cos, sin, table_dtype,      \
                       (uint16_t*)latent_cache, slot_mapping, num_slots, heads, rank, rope)
    if (dtype == MF_BF16) MNR_LAUNCH(BF16);
    else MNR_LAUNCH(FP16);
#undef MNR_LAUNCH
    return MF_LAUNCH_CHECK();
}
