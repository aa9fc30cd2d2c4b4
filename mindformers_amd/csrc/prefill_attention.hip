// GQA paged attention for gfx950, prefill side (several causal query rows per sequence): the 32-column kernel,
// its launch rule and entry points.  int8 caches go through the 16-column kernel of paged_attention_kernels.h.
#include "paged_attention_kernels.h"

namespace {

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
// DV: width of a value head and of an output head.  DV < D (the prefill of multi-latent attention: 192-wide queries
// and keys, 128-wide values, packed rows only) loads and multiplies the first sub-tile of the value rows only.
template <typename T, int D, bool TIB, int DV = D>
__global__ __launch_bounds__(PA_WAVES * 64, D == 192 ? 2 : 3) void prefill_attention_kernel(
    uint16_t* __restrict__ out, float* __restrict__ part_out, float* __restrict__ part_ml,
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc,
    const int32_t* __restrict__ block_tables, const int32_t* __restrict__ ctx_lens, int n_heads, int n_kv,
    int n_rep, int block_size, int max_blocks, int num_blocks, int max_parts, float scale_log2, int64_t q_stride,
    int batch, const int32_t* __restrict__ q_starts, int part_tokens, int64_t kv_stride, int rows,
    int64_t v_stride) {
    using vec8 = typename T::vec8;
    using S = PfSmem<D>;
    static_assert(DV == D || DV == S::W0, "value heads as wide as the key heads, or as their first sub-tile");
    constexpr int KS = D / 16;                                // k-steps of the score product
    constexpr int DB = DV / 32;                               // 32-row blocks of O^T
    constexpr int NV = 2 * DB;                                // PV MFMAs per tile
    using S0 = typename S::Sub0;
    using S1 = typename S::Sub1;
    constexpr int NI = S::NI;
    constexpr int NIV = DV == D ? NI : S0::NI;                // value loads per loading wave and tile
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
    const int64_t v_row_bytes = v_stride * 2;

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
        vcol[i] = (uint32_t)(kvh * DV * 2 + col0 + 16 * ((lslot - 4 * key4) & (SS::CPR - 1)));
        kofs[i] = (uint32_t)(row * (int)(kv_stride * 2)) + kcol[i];      // offsets within a whole tile
        vofs[i] = (uint32_t)(row * (int)(v_stride * 2)) + vcol[i];
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
            const uint8_t* vb = (const uint8_t*)vc + slot0 * v_row_bytes;
            static_for<NI>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                constexpr bool second = i >= S0::NI;
                using SS = std::conditional_t<second, S1, S0>;
                constexpr int li = i - (second ? S0::NI : 0);
                uint8_t* dst = kdst + (second ? S::SUB1 : 0) + (SS::LW * li + w) * SS::RPI * SS::ROWB;
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(kb + kofs[i]),
                                                 (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
                if constexpr (i < NIV)
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
                kp = (const uint8_t*)kc + slot0 * row_bytes + ((uint32_t)(rc * (int)row_bytes) + kcol[i]);
                vp = (const uint8_t*)vc + slot0 * v_row_bytes + ((uint32_t)(rc * (int)v_row_bytes) + vcol[i]);
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
            if constexpr (i < NIV)
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
        if (t + 1 < ntiles) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(NI + NIV) : "memory");
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
        uint16_t* dst = out + gh * DV + 4 * h;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4)
                *(u32x2*)(dst + 32 * db + 8 * q4) =
                    (u32x2){pack2<T>(acc[db][4 * q4] * inv, acc[db][4 * q4 + 1] * inv),
                            pack2<T>(acc[db][4 * q4 + 2] * inv, acc[db][4 * q4 + 3] * inv)};
    } else {
        const int64_t pi = gh * max_parts + part;
        float* dst = part_out + pi * DV + 4 * h;
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

template <typename T, int D, int KVQ, int DV = D>
int launch_pf(void* out, const void* query, const void* key_cache, const void* value_cache,
              const int32_t* block_tables, const int32_t* context_lens, const int32_t* q_starts, int batch,
              int total_q, int n_heads, int n_kv, int block_size, int max_blocks, int num_blocks, float scale,
              int64_t q_stride, int64_t kv_stride, void* workspace, hipStream_t st, const float* kv_scale,
              const float* kv_offset, int64_t v_stride = 0) {
    static_assert(DV == D || KVQ == 0, "value heads narrower than the key heads: 16-bit packed rows only");
    if (v_stride <= 0) v_stride = kv_stride;
    const int n_rep = n_heads / n_kv;
    const bool contiguous = block_tables == nullptr;
    const PfPlan plan = pf_plan(batch, total_q, n_heads, n_kv, contiguous ? total_q : (int64_t)max_blocks * block_size);
    float* part_out = plan.max_parts > 1 ? (float*)workspace : nullptr;
    float* part_ml = part_out ? part_out + (int64_t)total_q * n_heads * plan.max_parts * DV : nullptr;
    const float scale_log2 = scale * 1.4426950408889634f;
    constexpr bool KV8 = KVQ != 0;
    const int64_t wgs = (KV8 ? plan.col_groups16 : plan.col_groups128) * n_kv * plan.max_parts;
    if (wgs > 0x7fffffffLL) {
        mf_set_error("paged_attention_prefill: %lld workgroups exceed the grid limit", (long long)wgs);
        return 1;
    }
    if (plan.max_parts == 1) {
        hipLaunchKernelGGL(pf_zero_rows_kernel, dim3(batch), dim3(256), 0, st, (uint16_t*)out, q_starts, context_lens,
                           contiguous, max_blocks * block_size, batch, n_heads * DV, total_q);
        int rc = MF_LAUNCH_CHECK();
        if (rc) return rc;
    }
    if constexpr (KV8) {
        const bool tib = block_size % PA_TILE == 0;           // a 32-token tile never straddles two blocks
#define PF_LAUNCH(TIBV)                                                                                           \
    hipLaunchKernelGGL((paged_attention_kernel<T, D, 2, true, KVQ, TIBV>), dim3((unsigned)wgs),                    \
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
        auto kern = prefill_attention_kernel<T, D, TIBV, DV>;                                                     \
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
                           q_starts, plan.part_tokens, kv_stride, total_q, v_stride);                             \
    }
        if (tib) PF_LAUNCH(true)
        else PF_LAUNCH(false)
#undef PF_LAUNCH
    }
    int rc = MF_LAUNCH_CHECK();
    if (rc) return rc;
    if (plan.max_parts > 1) {
        hipLaunchKernelGGL((paged_attention_reduce_kernel<T, DV, true>), dim3(n_heads, total_q),
                           dim3(PA_REDUCE_THREADS<DV>), 0, st,
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
                            int kvq, const float* kv_scale, const float* kv_offset) {
    // kvq: 0 = 16-bit rows or caches, 1 = int8 caches with per-channel scale / offset, 2 = int8 caches with per-token
    // key scales (kv_scale) and value scales (kv_offset), one float per cache slot
    const bool kv8 = kvq != 0;
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "paged_attention_prefill: dtype must be bf16 or fp16");
    MF_REQUIRE(!kv8 || (kv_scale && block_tables), "paged_attention_prefill: an int8 cache needs its scales and a block table");
    MF_REQUIRE(kvq != 2 || (kv_offset && block_size % 4 == 0 && (((uintptr_t)kv_scale | (uintptr_t)kv_offset) & 15) == 0),
               "paged_attention_prefill: per-token scales need both 16-byte aligned scale caches and a block size that "
               "is a multiple of 4");
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
#define PF_CASE_Q(TT, DD, QQ)                                                                                      \
    return launch_pf<TT, DD, QQ>(out, query, key_cache, value_cache, block_tables, context_lens, q_starts, batch,  \
                                 total_q, n_heads, n_kv_heads, block_size, max_blocks_per_seq, num_blocks, scale,  \
                                 q_row_stride, kv_row_stride, workspace, st, kvq ? kv_scale : nullptr,             \
                                 kvq ? kv_offset : nullptr)
#define PF_CASE(TT, DD)                                                                                            \
    {                                                                                                              \
        if (kvq == 2) PF_CASE_Q(TT, DD, 2);                                                                        \
        if (kvq == 1) PF_CASE_Q(TT, DD, 1);                                                                        \
        PF_CASE_Q(TT, DD, 0);                                                                                      \
    }
#define PF_CASE192(TT)                                                                                             \
    return launch_pf<TT, 192, 0>(out, query, key_cache, value_cache, block_tables, context_lens, q_starts, batch, \
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
#undef PF_CASE_Q
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
                            q_row_stride, kv_row_stride, dtype, workspace, workspace_bytes, stream, 0, nullptr,
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
                            q_row_stride, 0, dtype, workspace, workspace_bytes, stream, 1, antiquant_scale,
                            antiquant_offset);
}

extern "C" int mf_paged_attention_prefill_int8kv_per_token(void* out, const void* query, const void* key_cache,
                                                           const void* value_cache, const float* key_scale_cache,
                                                           const float* value_scale_cache,
                                                           const int32_t* block_tables, const int32_t* context_lens,
                                                           const int32_t* q_starts, int batch, int total_q,
                                                           int n_heads, int n_kv_heads, int head_dim, int block_size,
                                                           int max_blocks_per_seq, int num_blocks, float scale,
                                                           int64_t q_row_stride, int dtype, void* workspace,
                                                           size_t workspace_bytes, void* stream) {
    return pa_prefill_entry(out, query, key_cache, value_cache, block_tables, context_lens, q_starts, batch, total_q,
                            n_heads, n_kv_heads, head_dim, block_size, max_blocks_per_seq, num_blocks, scale,
                            q_row_stride, 0, dtype, workspace, workspace_bytes, stream, 2, key_scale_cache,
                            value_scale_cache);
}

extern "C" int mf_causal_attention_qk192_v128(void* out, const void* query, const void* key, const void* value,
                                              const int32_t* q_starts, int batch, int total_q, int n_heads,
                                              int n_kv_heads, float scale, int64_t q_row_stride,
                                              int64_t k_row_stride, int64_t v_row_stride, int dtype, void* workspace,
                                              size_t workspace_bytes, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "causal_attention_qk192_v128: dtype must be bf16 or fp16");
    MF_REQUIRE(batch >= 0 && total_q >= 0, "causal_attention_qk192_v128: negative batch or row count");
    if (batch == 0 || total_q == 0) return 0;
    MF_REQUIRE(out && query && key && value && q_starts, "causal_attention_qk192_v128: null argument");
    MF_REQUIRE(scale > 0.f, "causal_attention_qk192_v128: the softmax scale must be positive");
    MF_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
               "causal_attention_qk192_v128: n_heads (%d) must be a positive multiple of n_kv_heads (%d)", n_heads,
               n_kv_heads);
    if (q_row_stride <= 0) q_row_stride = (int64_t)n_heads * 192;
    if (k_row_stride <= 0) k_row_stride = (int64_t)n_kv_heads * 192;
    if (v_row_stride <= 0) v_row_stride = (int64_t)n_kv_heads * 128;
    MF_REQUIRE(q_row_stride >= (int64_t)n_heads * 192 && k_row_stride >= (int64_t)n_kv_heads * 192 &&
                   v_row_stride >= (int64_t)n_kv_heads * 128 && q_row_stride % 8 == 0 && k_row_stride % 8 == 0 &&
                   v_row_stride % 8 == 0,
               "causal_attention_qk192_v128: row strides must cover a row and be multiples of 8 elements");
    MF_REQUIRE((((uintptr_t)out | (uintptr_t)query | (uintptr_t)key | (uintptr_t)value) & 15) == 0,
               "causal_attention_qk192_v128: out / query / key / value must be 16-byte aligned");
    const size_t need = mf_paged_attention_prefill_workspace_bytes(batch, total_q, n_heads, n_kv_heads, 128, total_q);
    MF_REQUIRE(need == 0 || (workspace && workspace_bytes >= need && ((uintptr_t)workspace & 15) == 0),
               "causal_attention_qk192_v128: 16-byte aligned workspace of %zu bytes needed, %zu given", need,
               workspace_bytes);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == MF_BF16)
        return launch_pf<BF16, 192, 0, 128>(out, query, key, value, nullptr, nullptr, q_starts, batch, total_q, n_heads,
                                            n_kv_heads, 0, 0, 0, scale, q_row_stride, k_row_stride, workspace, st,
                                            nullptr, nullptr, v_row_stride);
    return launch_pf<FP16, 192, 0, 128>(out, query, key, value, nullptr, nullptr, q_starts, batch, total_q, n_heads,
                                        n_kv_heads, 0, 0, 0, scale, q_row_stride, k_row_stride, workspace, st, nullptr,
                                        nullptr, v_row_stride);
}
