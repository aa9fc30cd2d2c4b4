// W8A16 weight-only skinny GEMM for decode: y = (x . w_i8^T) * scale (+bias) (+residual), dense and grouped.
//
// Weight layout ("packed", produced once at load time by mf_w8a16_pack_weight): the int8 matrix [N, K] is cut
// into tiles of 16 output channels x 64 input channels (1 KiB).  Inside a tile byte (16*g + r)*16 + j holds
// w[16*t + r][64*s + 16*g + j]: exactly the order in which the 64 lanes of a wavefront want their MFMA
// A-operand bytes, so one wave-wide 16-byte load reads one whole tile as 1 KiB of contiguous memory.
// Tiles are ordered [k-step][n-tile] (all output channels of one 64-wide slice of K are contiguous, so at any
// moment the workgroups of a launch read neighbouring memory, spread over all memory channels, instead of
// addresses a whole row of tiles apart); N is padded to 16 and K to 64 with zeros.  (Loading the same bytes
// from the row-major matrix makes every group of lanes touch 16 different cache lines per instruction and
// ran at about a third of the bandwidth.)
//
// Two kernels share the format.  The dense kernel (w8a16_gemm4_kernel, described where it is defined) loads weight
// tiles straight into MFMA operand registers, shares one LDS-staged activation tile among the waves of a workgroup
// and serves the decode layer's projections; its epilogue, or the split-K reduce kernels, carry the fused variants
// (gate/up + SiLU*mul, residual + RMSNorm,
// QKV + RoPE + cache scatter).  The grouped kernel (experts) keeps the earlier register-streaming tile routine
// w8a16_tile: a workgroup of 4 waves owns 64 output channels (4 n-tiles) for up to 64 rows of x; the waves
// interleave the 64-wide k-steps of the workgroup's k-range, each streams its tiles HBM -> registers two steps
// ahead, converts int8 -> bf16/fp16 in registers (exact) and multiplies on the 16x16x32 matrix cores; the
// activation tile of a step is staged through a private, XOR-swizzled LDS tile; the 4 waves are summed through
// LDS at the end.
//
// MFMA roles: A = weights [16 n x 32 k], B = activations [32 k x 16 m], C = y^T tile [16 n x 16 m]; the two
// MFMAs of a k-step take bytes 0-7 and 8-15 of each lane's 16 weight bytes, and the activation operand is
// gathered in the same k order.
#include "common.h"

namespace {

constexpr int GW_WAVES = 4;
constexpr int GW_NT = 4;                    // 16-row weight tiles per wave
constexpr int GW_BN = 16 * GW_NT;           // output channels per workgroup
constexpr int GW_KSTEP = 64;
constexpr int GW_TILE_BYTES = 16 * GW_KSTEP;
static_assert(GW_KSTEP == MF_PACK_KSTEP && GW_TILE_BYTES == MF_PACK_TILE_BYTES, "the packed format is shared with the int8 GEMMs");
constexpr int GW_DEPTH = 2;                 // weight k-steps in flight per wave beyond the current one

// A weight byte is read once per launch.  The non-temporal hint lets the caches drop it first, which keeps the
// activations, the partial sums and what the kernels around this one have left there.  Measured, it pays where many
// expert matrices or a few activation rows are read (the grouped kernel, the 4-wave dense kernel: 2.5 - 3.5 % of the
// layer step) and costs 1 % on the 8-wave dense kernel at 64 rows, which therefore keeps ordinary loads.
template <typename V>
__device__ __forceinline__ V gw_stream_load(const uint8_t* p) { return __builtin_nontemporal_load((const V*)p); }

// acc * scale (+ bias) with separately rounded operations: every epilogue below goes through here, so that the
// fused and the unfused paths give bit-identical values whatever the compiler would contract elsewhere.
template <typename T>
__device__ __forceinline__ float dequant_bias(float acc, float scale, const uint16_t* bias, int n) {
    float v = __fmul_rn(acc, scale);
    if (bias) v = __fadd_rn(v, T::to_float(bias[n]));
    return v;
}

// Epilogue for 4 consecutive output channels of one row.
template <typename T>
__device__ __forceinline__ void store4(uint16_t* y, const uint16_t* bias, const uint16_t* residual,
                                       const float* scale, int64_t row_off, int n, int N, f32x4 acc) {
    float o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (n + i < N) {
            float v = dequant_bias<T>(acc[i], scale ? scale[n + i] : 1.0f, bias, n + i);   // no scale: already applied
            if (residual) v = __fadd_rn(T::to_float(T::from_float(v)), T::to_float(residual[row_off + n + i]));
            o[i] = v;
        } else {
            o[i] = 0.f;
        }
    }
    if (n + 3 < N && ((row_off + n) & 3) == 0) {
        *(u32x2*)(y + row_off + n) = (u32x2){pack2<T>(o[0], o[1]), pack2<T>(o[2], o[3])};
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (n + i < N) y[row_off + n + i] = T::from_float(o[i]);
    }
}

// Gated epilogue for 4 consecutive channels (gate, up, gate, up) of one row: the two activations
// silu(gate) * up go to columns n/2, n/2 + 1 of a [rows, N/2] output.  Rounding points as the unfused sequence has
// them: the projection output, silu(gate), and the product are each rounded to T.
template <typename T>
__device__ __forceinline__ void store_gated(uint16_t* y, const uint16_t* bias, const float* scale, int m, int n,
                                            int N, f32x4 acc) {
    float o[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        float gv = dequant_bias<T>(acc[2 * h], scale ? scale[n + 2 * h] : 1.0f, bias, n + 2 * h);
        float uv = dequant_bias<T>(acc[2 * h + 1], scale ? scale[n + 2 * h + 1] : 1.0f, bias, n + 2 * h + 1);
        gv = T::to_float(T::from_float(gv));
        uv = T::to_float(T::from_float(uv));
        o[h] = T::to_float(T::from_float(silu_f(gv))) * uv;
    }
    const int64_t at = (int64_t)m * (N >> 1) + (n >> 1);
    if (n + 3 < N) *(uint32_t*)(y + at) = pack2<T>(o[0], o[1]);
    else y[at] = T::from_float(o[0]);
}

// One workgroup tile: output channels [n0, n0+64) x 16*MT rows [m0, ...) x k-steps [s_begin, s_end).
// MT = number of 16-row activation tiles; KTAIL = K is not a multiple of 64.  wp = packed weights of this
// matrix, KS = k-steps per n-tile.
template <typename T, int MT, bool KTAIL>
__device__ __forceinline__ void w8a16_tile(uint16_t* __restrict__ y, float* __restrict__ partial,
                                           const uint16_t* __restrict__ x, const uint8_t* __restrict__ wp,
                                           const float* __restrict__ scale, const uint16_t* __restrict__ bias,
                                           const uint16_t* __restrict__ residual, int M, int N, int K, int KS, int n0,
                                           int m0, int s_begin, int s_end, int split_index, uint8_t* smem,
                                           int gated = 0) {
    using vec8 = typename T::vec8;
    constexpr int XROWS = 16 * MT;
    constexpr int XTILE = XROWS * 128;                        // bytes of one staged activation tile
    constexpr int XLD = XROWS / 8;                            // coalesced loads per lane per tile (8 rows each)

    const int wv = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int r = lane & 15;
    const int g = lane >> 4;

    f32x4 acc[GW_NT][MT];
#pragma unroll
    for (int nt = 0; nt < GW_NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // Every load below is unconditional and reads an address that exists (indices are clamped), so the loop body
    // has no divergent branches: tiles beyond N and rows beyond M compute garbage that is never stored, steps
    // beyond s_end are prefetched from a clamped address and never consumed, and only the activation chunks
    // past K (last, short k-step) are replaced by zeros with a select.
    // ---- weights: tile (n-tile t, step s) sits at ((s*n_tiles + t) * 1024) + lane*16
    const int n_tiles_total = (N + 15) >> 4;
    const uint8_t* wbase[GW_NT];
#pragma unroll
    for (int nt = 0; nt < GW_NT; ++nt) {
        const int t = min((n0 >> 4) + nt, n_tiles_total - 1);
        wbase[nt] = wp + (int64_t)t * GW_TILE_BYTES + lane * 16;
    }
    // ---- activations: load i of lane (xr, xc) is the 16-byte chunk xc (8 elements) of row xr + 8*i
    const int xr = lane >> 3, xc = lane & 7;
    const uint16_t* xptr[XLD];
#pragma unroll
    for (int i = 0; i < XLD; ++i) {
        const int m = min(m0 + xr + 8 * i, M - 1);
        xptr[i] = x + (int64_t)m * K + 8 * xc;
    }
    uint8_t* xst = smem + wv * XTILE;                         // this wave's staging tile
    const int s_last = s_end - 1;
    const int k_last_chunk = K - 8;                           // element offset of the last whole 16-byte chunk

    const int first = s_begin + wv;
    u32x4 wreg[GW_DEPTH + 1][GW_NT];
    u32x4 xreg[XLD];
    auto load_w = [&](int slot, int s) {
        const int64_t off = (int64_t)min(s, s_last) * n_tiles_total * GW_TILE_BYTES;
#pragma unroll
        for (int nt = 0; nt < GW_NT; ++nt) wreg[slot][nt] = gw_stream_load<u32x4>(wbase[nt] + off);
    };
    auto load_x = [&](int s) {
        const int kb = min(s, s_last) * GW_KSTEP;
        if (KTAIL) {
            // K is not a multiple of 64: chunks past K (last, short step) read a clamped address and are zeroed
            // with a mask (an AND, so that the load stays unconditional)
            const bool kok = kb + 8 * xc < K;
            const int koff = kok ? kb : k_last_chunk - 8 * xc;
            const uint32_t km = kok ? 0xffffffffu : 0u;
#pragma unroll
            for (int i = 0; i < XLD; ++i) {
                const u32x4 v = *(const u32x4*)(xptr[i] + koff);
                xreg[i] = (u32x4){v[0] & km, v[1] & km, v[2] & km, v[3] & km};
            }
        } else {
#pragma unroll
            for (int i = 0; i < XLD; ++i) xreg[i] = *(const u32x4*)(xptr[i] + kb);
        }
    };
#pragma unroll
    for (int d = 0; d <= GW_DEPTH; ++d) load_w(d, first + d * GW_WAVES);
    load_x(first);

    // the weight registers rotate through GW_DEPTH + 1 slots; the loop body is written once per slot so that
    // every register index is a compile-time constant
    auto step = [&](int slot, int s) {
        // stage this step's activations: physical chunk = logical chunk ^ (row & 7)
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < XLD; ++i) *(u32x4*)(xst + (xr + 8 * i) * 128 + ((xc ^ xr) << 4)) = xreg[i];
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        load_x(s + GW_WAVES);                                 // next step's activations (L2) behind this step's math

        // B operands: lane (r, g), tile mt, half h reads logical chunk 2g + h of row 16*mt + r
        vec8 xb[MT][2];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                xb[mt][h] = bitcast<vec8>(*(const u32x4*)(xst + (16 * mt + r) * 128 + (((2 * g + h) ^ (r & 7)) << 4)));
#pragma unroll
        for (int nt = 0; nt < GW_NT; ++nt) {
            const vec8 a0 = dequant8<T>(wreg[slot][nt][0], wreg[slot][nt][1]);
            const vec8 a1 = dequant8<T>(wreg[slot][nt][2], wreg[slot][nt][3]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                acc[nt][mt] = T::mfma16(a0, xb[mt][0], acc[nt][mt]);
                acc[nt][mt] = T::mfma16(a1, xb[mt][1], acc[nt][mt]);
            }
        }
        load_w(slot, s + (GW_DEPTH + 1) * GW_WAVES);
    };
    for (int s = first; s < s_end; s += (GW_DEPTH + 1) * GW_WAVES) {
#pragma unroll
        for (int slot = 0; slot <= GW_DEPTH; ++slot)
            if (s + slot * GW_WAVES < s_end) step(slot, s + slot * GW_WAVES);
    }

    // ---- sum the 4 waves through LDS: red[wave][m][n], 16-byte granules XOR-swizzled by the row so that
    // neither the MFMA-layout writes nor the row-major reads collide on LDS banks
    __syncthreads();                                          // every wave is done with its staging tile
    float* red = (float*)smem;                                // [GW_WAVES][XROWS][GW_BN]
#pragma unroll
    for (int nt = 0; nt < GW_NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            *(f32x4*)(red + ((wv * XROWS + mt * 16 + r) * GW_BN) + (((nt * 4 + g) ^ r) << 2)) = acc[nt][mt];
    __syncthreads();

    constexpr int N4 = GW_BN / 4;
    for (int idx = threadIdx.x; idx < XROWS * N4; idx += GW_WAVES * 64) {
        const int ml = idx / N4, n4 = idx - ml * N4;
        const int m = m0 + ml, n = n0 + 4 * n4;
        if (m >= M || n >= N) continue;
        const int sw = (n4 ^ (ml & 15)) << 2;
        f32x4 sum = *(const f32x4*)(red + (ml * GW_BN) + sw);
#pragma unroll
        for (int q = 1; q < GW_WAVES; ++q) sum += *(const f32x4*)(red + ((q * XROWS + ml) * GW_BN) + sw);
        if (partial) {
            float* p = partial + ((int64_t)split_index * M + m) * N + n;
            if (n + 3 < N && (N & 3) == 0) {
                *(f32x4*)p = sum;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < N) p[i] = sum[i];
            }
        } else if (gated) {
            store_gated<T>(y, bias, scale, m, n, N, sum);
        } else {
            store4<T>(y, bias, residual, scale, (int64_t)m * N, n, N, sum);
        }
    }
}

template <int MT>
struct GwSmem {
    // activation staging (4 waves x [16*MT, 64] bf16) and the cross-wave reduction ([4][16*MT][64] fp32) alias
    static constexpr int BYTES = GW_WAVES * 16 * MT * GW_BN * 4;
};

// ---- dense kernel: helpers ---------------------------------------------------------------------------
constexpr int G2_WAVES = 4;
constexpr int G2_BN = G2_WAVES * 16;        // output channels of a 4-wave workgroup

// A 16-byte-per-lane LDS read is served 16 lanes per cycle over 64 banks (256 bytes); measured on gfx950, the
// lanes that share a cycle are those of one half of the wave with equal parity of lane bits 2, 3 and 4 - for an
// MFMA operand read (lane = 16*g + r, row r, logical chunk 2g + h) that is rows {0-3, 12-15} of one g together
// with rows {4-11} of the neighbouring g.  Two 128-byte rows span the banks, so with j = (row >> 1) & 7 the key
// j ^ 2*[j in 2..5] sends those 16 lanes to 16 different 16-byte bank groups.
__device__ __forceinline__ int g2_swizzle_key(int row) {
    const int j = (row >> 1) & 7;
    return j ^ ((((j >> 2) ^ (j >> 1)) & 1) << 1);
}
template <int OFFSET>
__device__ __forceinline__ u32x4 g2_lds_read16(uint32_t addr) {
    u32x4 v;
    if constexpr (OFFSET >= 65536) addr += 65536;             // the offset field has 16 bits
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(v) : "v"(addr), "n"(OFFSET & 65535) : "memory");
    return v;
}
template <int LGKM>
__device__ __forceinline__ void g2_wait_lds(u32x4& a, u32x4& b) {
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(LGKM) : "memory");
}
template <int LGKM>
__device__ __forceinline__ void g2_wait_lds(u32x4& a, u32x4& b, u32x4& c) {
    asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(a), "+v"(b), "+v"(c) : "n"(LGKM) : "memory");
}
template <int LGKM>
__device__ __forceinline__ void g2_wait_lds(u32x4& a, u32x4& b, u32x4& c, u32x4& d) {
    asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(LGKM) : "memory");
}
// ---- dense kernel, weights through registers --------------------------------------------------------------
// grid = (ceil(N / (16 * tiles)), split_k, ceil(M / (16*MT))) (or (split_k, n-blocks, m-blocks) when split-major).
// The waves of a workgroup walk the same k-steps and own different 16-channel weight tiles, so one staged activation
// tile ([16*MT rows, 64 k] as 128-byte rows) serves all of them: 4 waves up to 32 rows, 8 waves beyond (one
// activation byte per weight byte instead of two; the L2 -> CU path saturates near 11 TB/s, so the activation
// re-reads are what a skinny GEMM at 64 rows pays most for).  Both operands are fetched by ordinary 16-byte-per-lane
// loads into registers.  (An earlier version used LDS-direct loads for both.  Measured on this part with the GEMM's
// own grid and weight order - 448 workgroups x 64 k-steps x 4 KiB, cold - register loads stream 117 MB at 5.3 TB/s
// and LDS-direct loads at 3.4-3.5 TB/s whatever their number in flight, which is where that version's gate/up launch
// stood.)  A weight tile in registers is already the MFMA operand (after the int8 -> T conversion), so it never
// touches LDS; the activation tile is written to LDS by the lanes that loaded it, its 16-byte chunks XOR-swizzled
// (physical chunk = logical chunk ^ g2_swizzle_key(row), applied on the global-address side) so that the operand
// reads are free of bank conflicts, and read back as B operands by all waves.  A wave keeps DEPTH steps of
// loads in flight in a rotating set of registers (loads complete in issue order: the wait in front of a step's first
// use lets DEPTH-2 steps' worth stay outstanding).  Two LDS stages alternate: the activations of step s+1 are written
// while the operands of step s (read during step s-1) are multiplied.
template <int MT, int WAVES>
struct G4 {
    static constexpr int XROWS = 16 * MT;
    static constexpr int XTILE = XROWS * 128;
    static constexpr int DEPTH = 4;                           // register sets = steps of loads in flight (even)
    static constexpr int BN = 16 * WAVES;                     // output channels per workgroup, one tile per wave
    // activation loads (8 rows each) per wave and step: the 2*MT loads of a tile are dealt over the waves; where there
    // are more waves than loads the surplus waves repeat loads of the others (every wave issues the same number of
    // loads) and do not write them
    static constexpr int XL = 2 * MT > WAVES ? 2 * MT / WAVES : 1;
    static constexpr int XWRITERS = 2 * MT / XL;              // waves that write activations
    static_assert(XL * XWRITERS == 2 * MT && XWRITERS <= WAVES && XL <= 2, "bad split of the activation loads");
};

// W4: the weights are 4-bit (unsigned nibbles holding q + 8, q in -8 .. 7; a 16 x 64 tile is 512 bytes, lane (r, g)
// holds the 16 nibbles of row r, columns 16g .. 16g + 15 in 8 bytes, nibble i = column 16g + i).  GROUP (64 or 128,
// W4 only): one scale per channel and GROUP columns, gscale [K / GROUP][N]: the products of a group are summed in
// fp32 on the exact integer weights and enter the total times the group's scale; the epilogue's per-channel scale is
// then 1.  GROUP = 0: one scale per channel, applied in the epilogue.
template <typename T, int MT, int WAVES, bool KTAIL, bool W4 = false, int GROUP = 0>
__global__ __launch_bounds__(WAVES * 64, WAVES == 4 ? 3 : 1) void w8a16_gemm4_kernel(
    uint16_t* __restrict__ y, float* __restrict__ partial, const uint16_t* __restrict__ x,
    const uint8_t* __restrict__ wp, const float* __restrict__ scale, const uint16_t* __restrict__ bias,
    const uint16_t* __restrict__ residual, int M, int N, int K, int steps_per_split, int gated, int split_major,
    const float* __restrict__ gscale = nullptr) {
    using vec8 = typename T::vec8;
    using C = G4<MT, WAVES>;
    constexpr int D = C::DEPTH;
    static_assert(!W4 || !KTAIL, "4-bit weights: K is a multiple of 64");
    static_assert(GROUP == 0 || (W4 && (GROUP == 64 || GROUP == 128)), "groups of 64 or 128 columns, 4-bit weights");
    constexpr int TB = W4 ? GW_TILE_BYTES / 2 : GW_TILE_BYTES;  // bytes of a weight tile
    using wreg_t = std::conditional_t<W4, u32x2, u32x4>;
    __shared__ __attribute__((aligned(1024))) uint8_t smem[2 * C::XTILE];

    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    const int KS = (K + GW_KSTEP - 1) / GW_KSTEP;
    const int split = split_major ? blockIdx.x : blockIdx.y;
    const int nblock = split_major ? blockIdx.y : blockIdx.x;
    const int s_begin = split * steps_per_split;
    const int s_end = min(KS, s_begin + steps_per_split);
    const int s_last = s_end - 1;
    const int n0 = nblock * C::BN + wv * 16;                  // first output channel of this wave
    const int m0 = blockIdx.z * C::XROWS;

    f32x4 acc[MT], tot[GROUP ? MT : 1];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int mt = 0; mt < (GROUP ? MT : 1); ++mt) tot[mt] = (f32x4){0.f, 0.f, 0.f, 0.f};

    const int n_tiles_total = (N + 15) >> 4;
    const uint8_t* wtile = wp + (int64_t)min(n0 >> 4, n_tiles_total - 1) * TB;               // wave-uniform
    const int64_t wstride = (int64_t)n_tiles_total * TB;
    const uint32_t wlane = lane * (TB / 64);
    // group scales of this lane's 4 output channels (clamped inside the row for channels past N: never stored)
    const float* gsl = GROUP ? gscale + min(n0 + 4 * g, N - 4) : nullptr;
    const uint8_t* xbase = (const uint8_t*)(x + (int64_t)m0 * K);                            // wave-uniform
    uint32_t xlane[C::XL];
    int xchunk8[C::XL];
    uint32_t xdst[C::XL];                                     // LDS byte of the lane's chunk inside a stage
    const bool xwrite = wv < C::XWRITERS;
#pragma unroll
    for (int i = 0; i < C::XL; ++i) {
        const int row0 = 8 * ((wv % C::XWRITERS) * C::XL + i);
        const int row = row0 + (lane >> 3);
        xdst[i] = row0 * 128 + lane * 16;
        xchunk8[i] = 8 * ((lane & 7) ^ g2_swizzle_key(row));
        xlane[i] = (uint32_t)min(row, M - 1 - m0) * (uint32_t)K * 2u + 2u * xchunk8[i];
    }

    // All memory operations below are ordinary loads and stores, so the compiler itself places the counted waits in
    // front of the first use of every register (a hand-written wait cannot stop the register allocator from copying a
    // register whose load is still in flight).  For its count to stay exact, the main loop is free of conditional
    // steps: it runs over whole groups of D steps, the remaining 0 .. D-1 steps follow it.
    wreg_t wreg[D];
    u32x4 xreg[D][C::XL];
    f32x4 greg[GROUP ? D : 1];
    auto issue = [&](auto setc, int s) {
        constexpr int S = decltype(setc)::value;
        const int sc = min(s, s_last);
        if constexpr (WAVES == 4) wreg[S] = gw_stream_load<wreg_t>(wtile + sc * wstride + wlane);
        else wreg[S] = *(const wreg_t*)(wtile + sc * wstride + wlane);
        if constexpr (GROUP != 0) greg[S] = *(const f32x4*)(gsl + (int64_t)(sc * GW_KSTEP / GROUP) * N);
#pragma unroll
        for (int i = 0; i < C::XL; ++i) {
            uint32_t off = xlane[i] + (uint32_t)sc * (GW_KSTEP * 2);
            uint32_t km = 0xffffffffu;
            if (KTAIL) {
                // chunks past K (last, short step) re-read the row's last whole chunk and are zeroed with a mask (an
                // AND, so that the load stays unconditional): the padded weight columns are zero, but an Inf or NaN
                // among the last activations of a row must not meet them
                const int over = sc * GW_KSTEP + xchunk8[i] - (K - 8);
                off -= over > 0 ? 2u * over : 0u;
                km = over > 0 ? 0u : 0xffffffffu;
            }
            const u32x4 v = *(const u32x4*)(xbase + off);
            xreg[S][i] = KTAIL ? (u32x4){v[0] & km, v[1] & km, v[2] & km, v[3] & km} : v;
        }
    };
    auto stage_x = [&](auto setc, int stage) {                // this wave's activation chunks of a set -> LDS stage
        constexpr int S = decltype(setc)::value;
        if (xwrite) {
#pragma unroll
            for (int i = 0; i < C::XL; ++i) *(u32x4*)(smem + stage * C::XTILE + xdst[i]) = xreg[S][i];
        }
    };
    // B operands: lane (r, g), tile mt, half h reads logical chunk 2g + h of row 16*mt + r
    const int xoff0 = r * 128 + (((2 * g) ^ g2_swizzle_key(r)) << 4);
    const int xoff1 = r * 128 + (((2 * g + 1) ^ g2_swizzle_key(r)) << 4);
    u32x4 xb[2][MT][2];
    auto read_operands = [&](auto stagec) {
        constexpr int P = decltype(stagec)::value;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            xb[P][mt][0] = *(const u32x4*)(smem + P * C::XTILE + 2048 * mt + xoff0);
            xb[P][mt][1] = *(const u32x4*)(smem + P * C::XTILE + 2048 * mt + xoff1);
        }
    };

    // prologue: D steps of loads in flight, the first step's activations staged and its operands read
    static_for<D>([&](auto dc) { issue(dc, s_begin + decltype(dc)::value); });
    stage_x(std::integral_constant<int, 0>{}, 0);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    read_operands(std::integral_constant<int, 0>{});

    // step s: register set J holds its weight tile, LDS stage J & 1 held its activations (operands already in
    // xb[J & 1]); set J + 1 (step s + 1) is needed now: its activations go to the other stage
    auto step = [&](auto jc, int s) {
        constexpr int J = decltype(jc)::value;
        constexpr int JN = (J + 1) % D;
        constexpr int P = J & 1;
        __builtin_amdgcn_sched_barrier(0);
        stage_x(std::integral_constant<int, JN>{}, P ^ 1);
        vec8 wa[2];
        f32x4 gs = {1.f, 1.f, 1.f, 1.f};
        if constexpr (W4) {
            wa[0] = dequant8_u4<T>(wreg[J][0]);
            wa[1] = dequant8_u4<T>(wreg[J][1]);
            if constexpr (GROUP != 0) gs = greg[J];
        } else {
            wa[0] = dequant8<T>(wreg[J][0], wreg[J][1]);
            wa[1] = dequant8<T>(wreg[J][2], wreg[J][3]);
        }
        // the conversion happens here, before the set is reloaded (sunk below the reload it would keep the old
        // registers alive next to the new ones, and the sets would no longer rotate in place)
        asm volatile("" : "+v"(wa[0]), "+v"(wa[1]));
        if constexpr (GROUP != 0) asm volatile("" : "+v"(gs));
        __builtin_amdgcn_sched_barrier(0);
        issue(jc, s + D);                                     // set J is free: weights converted, activations staged
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");    // this wave's LDS writes are done
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        read_operands(std::integral_constant<int, P ^ 1>{});  // in flight behind the matrix instructions below
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[mt] = T::mfma16(wa[h], bitcast<vec8>(xb[P][mt][h]), acc[mt]);
        if constexpr (GROUP != 0) {
            if (GROUP == GW_KSTEP || (s & 1)) {               // the group's last step (splits begin on group borders)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) tot[mt][i] = __fmaf_rn(acc[mt][i], gs[i], tot[mt][i]);
                    acc[mt] = (f32x4){0.f, 0.f, 0.f, 0.f};
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    static_assert(D % 2 == 0 && D >= 4, "the two LDS stages alternate with the register sets");
    int s = s_begin;
    for (; s + D <= s_end; s += D) static_for<D>([&](auto jc) { step(jc, s + decltype(jc)::value); });
    static_for<D - 1>([&](auto jc) {
        if (s + decltype(jc)::value < s_end) step(jc, s + decltype(jc)::value);
    });

    // epilogue straight from the accumulator layout: lane (r, g) holds rows m = 16*mt + r, channels 4g .. 4g+3
    const int n = n0 + 4 * g;
    if (n >= N) return;
    const bool vec = n + 3 < N && (N & 3) == 0;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = m0 + 16 * mt + r;
        if (m >= M) continue;
        const f32x4 res = GROUP ? tot[mt] : acc[mt];
        if (partial) {
            float* p = partial + ((int64_t)split * M + m) * N + n;
            if (vec) {
                *(f32x4*)p = res;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < N) p[i] = res[i];
            }
        } else if (gated) {
            store_gated<T>(y, bias, scale, m, n, N, res);
        } else {
            store4<T>(y, bias, residual, scale, (int64_t)m * N, n, N, res);
        }
    }
}

// Grouped (experts): grid = (ceil(N/64), n_experts).  Rows offsets[e] .. offsets[e+1] of x use expert e's
// packed weights and scale[e]; experts with no rows exit at once.  One pass over the expert's weights serves up to
// 64 rows (decode batches route a handful of tokens to each expert: 16 rows per pass there); experts with more rows
// repeat the pass.  gated: the rows of the weight are interleaved gate / up and the epilogue writes
// silu(gate) * up into a [rows, N/2] output, as the dense gated GEMM does.
template <typename T, bool KTAIL>
__global__ __launch_bounds__(GW_WAVES * 64, 2) void w8a16_grouped_kernel(
    uint16_t* __restrict__ y, const uint16_t* __restrict__ x, const uint8_t* __restrict__ wp,
    const float* __restrict__ scale, const int32_t* __restrict__ offsets, int total_rows, int N, int K,
    int64_t expert_bytes, int gated) {
    __shared__ __attribute__((aligned(16))) uint8_t smem[GwSmem<4>::BYTES];
    const int e = blockIdx.y;
    int row0 = offsets[e], row1 = offsets[e + 1];
    row0 = max(0, min(row0, total_rows));
    row1 = max(row0, min(row1, total_rows));
    const int rows = row1 - row0;
    if (rows == 0) return;
    const int KS = (K + GW_KSTEP - 1) / GW_KSTEP;
    const uint8_t* we = wp + (int64_t)e * expert_bytes;
    const float* se = scale + (int64_t)e * N;
    uint16_t* ye = y + (int64_t)row0 * (gated ? N >> 1 : N);
    const uint16_t* xe = x + (int64_t)row0 * K;
    const int n0 = blockIdx.x * GW_BN;
    if (rows <= 16) {
        w8a16_tile<T, 1, KTAIL>(ye, nullptr, xe, we, se, nullptr, nullptr, rows, N, K, KS, n0, 0, 0, KS, 0, smem, gated);
    } else if (rows <= 32) {
        w8a16_tile<T, 2, KTAIL>(ye, nullptr, xe, we, se, nullptr, nullptr, rows, N, K, KS, n0, 0, 0, KS, 0, smem, gated);
    } else {
        for (int m0 = 0; m0 < rows; m0 += 64) {
            w8a16_tile<T, 4, KTAIL>(ye, nullptr, xe, we, se, nullptr, nullptr, rows, N, K, KS, n0, m0, 0, KS, 0, smem,
                                    gated);
            __syncthreads();                                  // the LDS tile is reused by the next pass
        }
    }
}

template <typename T>
__global__ void w8a16_splitk_reduce_kernel(uint16_t* __restrict__ y, const float* __restrict__ partial,
                                           const float* __restrict__ scale, const uint16_t* __restrict__ bias,
                                           const uint16_t* __restrict__ residual, int M, int N, int split_k,
                                           int gated) {
    const int n4cnt = (N + 3) / 4;
    const int64_t total = (int64_t)M * n4cnt;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int m = (int)(idx / n4cnt);
        const int n = (int)(idx - (int64_t)m * n4cnt) * 4;
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        if (n + 3 < N && (N & 3) == 0) {
            // all splits' loads in flight together (at most 16 splits), summed in split order
            const float* p = partial + (int64_t)m * N + n;
            const int64_t stride = (int64_t)M * N;
            f32x4 v[16];
#pragma unroll
            for (int s = 0; s < 16; ++s)
                if (s < split_k) v[s] = *(const f32x4*)(p + s * stride);
#pragma unroll
            for (int s = 0; s < 16; ++s)
                if (s < split_k) sum += v[s];
        } else {
            for (int s = 0; s < split_k; ++s)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < N) sum[i] += partial[((int64_t)s * M + m) * N + n + i];
        }
        if (gated) store_gated<T>(y, bias, scale, m, n, N, sum);
        else store4<T>(y, bias, residual, scale, (int64_t)m * N, n, N, sum);
    }
}

// Split-K reduce fused with the residual add and the RMSNorm that follows a row-parallel projection: one workgroup
// per row sums the splits in split order, forms h = round(round(acc*scale + bias) + residual) (written to h_out)
// and y = h * rsqrt(mean(h^2) + eps) * gamma - the same values, rounding for rounding, as the plain reduce kernel
// followed by the RMSNorm kernel, without the launch and the pass over h in between.
constexpr int RN_THREADS = 512;
constexpr int RN_MAX_VEC = 4;                                 // N <= 512 * 4 * 8 = 16384
constexpr int RN_SPLITS = 8;                                  // splits whose loads are in flight together

// norm_cols: the norm covers the leading norm_cols columns of a row (a multiple of 8; y is dense [M, norm_cols]); the
// other columns are summed and written to h_out only.  residual may be null (no add).
template <typename T>
__global__ __launch_bounds__(RN_THREADS) void w8a16_reduce_add_rmsnorm_kernel(
    uint16_t* __restrict__ y, uint16_t* __restrict__ h_out, const float* __restrict__ partial,
    const float* __restrict__ scale, const uint16_t* __restrict__ bias, const uint16_t* __restrict__ residual,
    const void* __restrict__ gamma, float eps, int M, int N, int split_k, int gamma_dtype, int norm_cols) {
    __shared__ float red[RN_THREADS / 64];
    const int m = blockIdx.x;
    const int nvec = N >> 3;
    const int64_t stride = (int64_t)M * N;
    float v[RN_MAX_VEC][8], gm[RN_MAX_VEC][8];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < RN_MAX_VEC; ++it) {
        const int c = threadIdx.x + it * RN_THREADS;
        if (c < nvec) {
            const int n = 8 * c;
            const bool normed = n < norm_cols;
            const float* p = partial + (int64_t)m * N + n;
            const f32x4 s_lo = *(const f32x4*)(scale + n), s_hi = *(const f32x4*)(scale + n + 4);
            u32x4 rraw = {0u, 0u, 0u, 0u};
            if (residual) rraw = *(const u32x4*)(residual + (int64_t)m * N + n);
            if (normed) load8_as_float(gamma, n, gamma_dtype, gm[it]);
            f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
            for (int s0 = 0; s0 < split_k; s0 += RN_SPLITS) {  // summed in split order
                f32x4 a[RN_SPLITS], b[RN_SPLITS];
#pragma unroll
                for (int q = 0; q < RN_SPLITS; ++q)
                    if (s0 + q < split_k) {
                        a[q] = *(const f32x4*)(p + (s0 + q) * stride);
                        b[q] = *(const f32x4*)(p + (s0 + q) * stride + 4);
                    }
#pragma unroll
                for (int q = 0; q < RN_SPLITS; ++q)
                    if (s0 + q < split_k) {
                        lo += a[q];
                        hi += b[q];
                    }
            }
            float rr[8];
            unpack8<T>(rraw, rr);
            u32x4 hp;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float t0 = dequant_bias<T>(lo[i], s_lo[i], bias, n + i);
                const float t1 = dequant_bias<T>(hi[i], s_hi[i], bias, n + 4 + i);
                const float r0 = T::to_float(T::from_float(t0)), r1 = T::to_float(T::from_float(t1));
                v[it][i] = residual ? __fadd_rn(r0, rr[i]) : r0;
                v[it][4 + i] = residual ? __fadd_rn(r1, rr[4 + i]) : r1;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) hp[i] = pack2<T>(v[it][2 * i], v[it][2 * i + 1]);
            *(u32x4*)(h_out + (int64_t)m * N + n) = hp;
            unpack8<T>(hp, v[it]);                            // the norm sees the rounded h
            if (normed) {
#pragma unroll
                for (int i = 0; i < 8; ++i) ss = __fmaf_rn(v[it][i], v[it][i], ss);
            }
        }
    }
    const float tot = rmsnorm_block_sum<RN_THREADS>(ss, red);
    const float inv = rsqrtf(tot / (float)norm_cols + eps);
#pragma unroll
    for (int it = 0; it < RN_MAX_VEC; ++it) {
        const int c = threadIdx.x + it * RN_THREADS;
        if (c < nvec && 8 * c < norm_cols) {
            u32x4 o;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                o[i] = pack2<T>(v[it][2 * i] * inv * gm[it][2 * i], v[it][2 * i + 1] * inv * gm[it][2 * i + 1]);
            *(u32x4*)(y + (int64_t)m * norm_cols + 8 * c) = o;
        }
    }
}

// Split-K reduce of a fused QKV projection together with what follows it in the attention block: rotate-half RoPE
// on q and k and the scatter of the rotated k and of v into the paged caches.  One work item = 8 consecutive
// elements of the first half of a q/k head with their partners in the second half, or 8 elements of v; grid =
// (tokens, ceil(items / 256)).  q is written (rotated) into its columns of qkv; the k and v columns of qkv are
// not written.  Values and rounding are those of the plain reduce kernel followed by the rope-and-cache kernel.
template <typename T>
__device__ __forceinline__ void qkv_reduce8(const float* __restrict__ p, int64_t stride, int split_k,
                                            const float* __restrict__ scale, const uint16_t* __restrict__ bias,
                                            int n, float* out) {
    f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < split_k; s0 += RN_SPLITS) {
        f32x4 a[RN_SPLITS], b[RN_SPLITS];
#pragma unroll
        for (int q = 0; q < RN_SPLITS; ++q)
            if (s0 + q < split_k) {
                a[q] = *(const f32x4*)(p + (s0 + q) * stride);
                b[q] = *(const f32x4*)(p + (s0 + q) * stride + 4);
            }
#pragma unroll
        for (int q = 0; q < RN_SPLITS; ++q)
            if (s0 + q < split_k) {
                lo += a[q];
                hi += b[q];
            }
    }
    const f32x4 s_lo = *(const f32x4*)(scale + n), s_hi = *(const f32x4*)(scale + n + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        out[i] = T::to_float(T::from_float(dequant_bias<T>(lo[i], s_lo[i], bias, n + i)));
        out[4 + i] = T::to_float(T::from_float(dequant_bias<T>(hi[i], s_hi[i], bias, n + 4 + i)));
    }
}

constexpr int RC_THREADS = 64;            // small workgroups: a 64-row step has only ~450 items per row to spread

// KV8: the caches are int8 and the rows are quantised on the way (kv_scale / kv_offset float32 [2][n_kv * D], keys
// then values), with the values and rounding of the rope kernel followed by the quantising scatter kernel.
template <typename T, bool KV8>
__global__ __launch_bounds__(RC_THREADS) void w8a16_reduce_rope_cache_kernel(
    uint16_t* __restrict__ qkv, const float* __restrict__ partial, const float* __restrict__ scale,
    const uint16_t* __restrict__ bias, const void* __restrict__ cos, const void* __restrict__ sin,
    void* __restrict__ key_cache_, void* __restrict__ value_cache_, const int32_t* __restrict__ slot_mapping,
    int M, int N, int split_k, int n_heads, int n_kv, int D, int64_t num_slots, int table_dtype,
    const float* __restrict__ kv_scale, const float* __restrict__ kv_offset) {
    uint16_t* key_cache = (uint16_t*)key_cache_;
    uint16_t* value_cache = (uint16_t*)value_cache_;
    const int t = blockIdx.x;
    const int half = D >> 1;
    const int cph = half >> 3;
    const int rot_items = (n_heads + n_kv) * cph;
    const int v_items = n_kv * D / 8;
    const int item = blockIdx.y * RC_THREADS + threadIdx.x;
    if (item >= rot_items + v_items) return;
    // the slot is only needed where a row is stored: no load below waits for it
    const int64_t slot = slot_mapping[t];
    const int64_t row = (int64_t)n_kv * D;
    const int64_t stride = (int64_t)M * N;
    const float* prow = partial + (int64_t)t * N;
    if (item >= rot_items) {
        const int i = (item - rot_items) * 8;
        const int col = (n_heads + n_kv) * D + i;
        float v[8];
        qkv_reduce8<T>(prow + col, stride, split_k, scale, bias, col, v);
        if (slot >= 0 && slot < num_slots) {
            if constexpr (KV8) {                              // v already holds values rounded to T
                *(u32x2*)((int8_t*)value_cache_ + slot * row + i) =
                    quant8_for_cache(v, kv_scale + row + i, kv_offset ? kv_offset + row + i : nullptr);
            } else {
                u32x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = pack2<T>(v[2 * e], v[2 * e + 1]);
                *(u32x4*)(value_cache + slot * row + i) = o;
            }
        }
        return;
    }
    const int h = item / cph, i = (item - h * cph) * 8;
    const bool is_k = h >= n_heads;
    const int col = h * D + i;                                // q heads, then k heads, are consecutive columns
    float x1[8], x2[8], c1[8], s1[8], c2[8], s2[8];
    const int64_t trow = (int64_t)t * D;
    load8_as_float(cos, trow + i, table_dtype, c1);
    load8_as_float(sin, trow + i, table_dtype, s1);
    load8_as_float(cos, trow + i + half, table_dtype, c2);
    load8_as_float(sin, trow + i + half, table_dtype, s2);
    qkv_reduce8<T>(prow + col, stride, split_k, scale, bias, col, x1);
    qkv_reduce8<T>(prow + col + half, stride, split_k, scale, bias, col + half, x2);
    u32x4 o1, o2;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float a0, b0, a1, b1;
        rope_pair(x1[2 * e], x2[2 * e], c1[2 * e], s1[2 * e], c2[2 * e], s2[2 * e], a0, b0);
        rope_pair(x1[2 * e + 1], x2[2 * e + 1], c1[2 * e + 1], s1[2 * e + 1], c2[2 * e + 1], s2[2 * e + 1], a1, b1);
        o1[e] = pack2<T>(a0, a1);
        o2[e] = pack2<T>(b0, b1);
    }
    if (is_k) {
        if (slot >= 0 && slot < num_slots) {
            const int kc = (h - n_heads) * D + i;             // column inside the key row
            if constexpr (KV8) {
                float r1[8], r2[8];                           // the rotated key as the rope kernel would store it
                unpack8<T>(o1, r1);
                unpack8<T>(o2, r2);
                int8_t* dst = (int8_t*)key_cache_ + slot * row + kc;
                *(u32x2*)dst = quant8_for_cache(r1, kv_scale + kc, kv_offset ? kv_offset + kc : nullptr);
                *(u32x2*)(dst + half) =
                    quant8_for_cache(r2, kv_scale + kc + half, kv_offset ? kv_offset + kc + half : nullptr);
            } else {
                uint16_t* dst = key_cache + slot * row + kc;
                *(u32x4*)dst = o1;
                *(u32x4*)(dst + half) = o2;
            }
        }
    } else {
        uint16_t* dst = qkv + (int64_t)t * N + col;
        *(u32x4*)dst = o1;
        *(u32x4*)(dst + half) = o2;
    }
}

// [N, K] row-major int8 -> packed tiles.  One thread per 16 packed bytes.
__global__ void w8a16_pack_kernel(uint8_t* __restrict__ dst, const int8_t* __restrict__ src, int N, int K, int KS,
                                  int64_t chunks) {
    for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < chunks; c += (int64_t)gridDim.x * blockDim.x) {
        const int lane = (int)(c & 63);
        const int64_t tile = c >> 6;
        const int n_tiles = (N + 15) >> 4;
        const int t = (int)(tile % n_tiles);
        const int s = (int)(tile / n_tiles);
        const int n = 16 * t + (lane & 15);
        const int k0 = 64 * s + 16 * (lane >> 4);
        uint8_t b[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) b[j] = (n < N && k0 + j < K) ? (uint8_t)src[(int64_t)n * K + k0 + j] : 0;
        u32x4 v;
#pragma unroll
        for (int q = 0; q < 4; ++q)
            v[q] = (uint32_t)b[4 * q] | ((uint32_t)b[4 * q + 1] << 8) | ((uint32_t)b[4 * q + 2] << 16) |
                   ((uint32_t)b[4 * q + 3] << 24);
        *(u32x4*)(dst + c * 16) = v;
    }
}

// [N, K] row-major int8 holding 4-bit values (-8 .. 7) -> packed nibble tiles (q + 8).  One thread per 8 packed bytes.
__global__ void w4a16_pack_kernel(uint8_t* __restrict__ dst, const int8_t* __restrict__ src, int N, int K,
                                  int64_t chunks) {
    for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < chunks; c += (int64_t)gridDim.x * blockDim.x) {
        const int lane = (int)(c & 63);
        const int64_t tile = c >> 6;
        const int n_tiles = (N + 15) >> 4;
        const int t = (int)(tile % n_tiles);
        const int s = (int)(tile / n_tiles);
        const int n = 16 * t + (lane & 15);
        const int k0 = 64 * s + 16 * (lane >> 4);
        uint32_t v[2] = {0u, 0u};
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int q = (n < N && k0 + j < K) ? (int)src[(int64_t)n * K + k0 + j] : 0;
            v[j >> 3] |= (uint32_t)((q + 8) & 15) << (4 * (j & 7));
        }
        *(u32x2*)(dst + c * 8) = (u32x2){v[0], v[1]};
    }
}

struct RopeCacheArgs {
    const void *cos, *sin;
    void *key_cache, *value_cache;
    const int32_t* slot_mapping;
    int n_heads, n_kv, head_dim, table_dtype;
    int64_t num_slots;
    const float *kv_scale, *kv_offset;        // int8 caches: per-channel parameters [2][n_kv * head_dim]; else null
};

struct GemmPlan {
    int waves;       // waves (16-channel tiles) per workgroup
    int mt;          // activation tiles per pass (1, 2, 4)
    int m_blocks;
    int n_blocks;
    int split_k;
    int steps_per_split;
};

GemmPlan plan_w8a16(int m, int n, int k, int step_align = 1) {
    GemmPlan p;
    p.mt = m <= 16 ? 1 : (m <= 32 ? 2 : 4);
    p.m_blocks = (m + 16 * p.mt - 1) / (16 * p.mt);
    // 33+ rows: 8 waves x 16 channels share one staged activation tile (half the activation bytes per weight byte of
    // the 4-wave shape), one workgroup per CU
    p.waves = p.mt == 4 ? 8 : 4;
    const int bn = 16 * p.waves;
    p.n_blocks = (n + bn - 1) / bn;
    const int total_steps = (k + GW_KSTEP - 1) / GW_KSTEP;
    // 4 waves: aim at two resident workgroups on each of the 256 CUs, at least 12 k-steps per workgroup; 8 waves: one
    // workgroup per CU, at least 8 steps
    const int target = p.waves == 8 ? 256 : 512;
    const int min_steps = p.waves == 8 ? 8 : 12;
    int sk = target / (p.n_blocks * p.m_blocks);
    sk = sk < 1 ? 1 : sk;
    const int max_sk = total_steps / min_steps < 1 ? 1 : total_steps / min_steps;
    sk = sk > max_sk ? max_sk : sk;
    sk = sk > 16 ? 16 : sk;
    if (sk > 8) sk = 8 * (sk / 8);                             // multiples of 8 can run split-major
    p.steps_per_split = (total_steps + sk - 1) / sk;
    p.steps_per_split = (p.steps_per_split + step_align - 1) / step_align * step_align;   // splits begin on group borders
    p.split_k = (total_steps + p.steps_per_split - 1) / p.steps_per_split;
    return p;
}

template <typename T>
int launch_w8a16(void* y, const void* x, const uint8_t* wp, const float* scale, const void* bias,
                 const void* residual, int m, int n, int k, int gated, void* workspace, hipStream_t st,
                 void* norm_out = nullptr, const void* gamma = nullptr, float eps = 0.f, int gamma_dtype = MF_FP32,
                 const RopeCacheArgs* rc_args = nullptr, int w4_group = -1, int norm_cols = 0) {
    // norm_cols: columns the norm in norm_out covers (the leading ones; 0 = the whole row)
    if (norm_cols <= 0) norm_cols = n;
    // w4_group >= 0: 4-bit weights; 0 = `scale` holds one value per channel, 64 / 128 = one per channel and group
    // ([K / group][N]), applied inside the kernel (the epilogues then see no scale)
    const GemmPlan p = plan_w8a16(m, n, k, w4_group == 128 ? 2 : 1);
    const float* gscale = w4_group > 0 ? scale : nullptr;
    if (w4_group > 0) scale = nullptr;
    float* partial = p.split_k > 1 ? (float*)workspace : nullptr;
    const int split_major = p.split_k % 8 == 0;
    dim3 grid(split_major ? p.split_k : p.n_blocks, split_major ? p.n_blocks : p.split_k, p.m_blocks);
    const bool ktail = (k % GW_KSTEP) != 0;
#define GW4_LAUNCH(MTV, WV, KT)                                                                                  \
    hipLaunchKernelGGL((w8a16_gemm4_kernel<T, MTV, WV, KT>), grid, dim3(WV * 64), 0, st, (uint16_t*)y, partial,  \
                       (const uint16_t*)x, wp, scale, (const uint16_t*)bias, (const uint16_t*)residual, m, n, k, \
                       p.steps_per_split, gated, split_major)
#define GW4_LAUNCH_W4(MTV, WV, GV)                                                                               \
    hipLaunchKernelGGL((w8a16_gemm4_kernel<T, MTV, WV, false, true, GV>), grid, dim3(WV * 64), 0, st, (uint16_t*)y, \
                       partial, (const uint16_t*)x, wp, scale, (const uint16_t*)bias, (const uint16_t*)residual, m, n, \
                       k, p.steps_per_split, gated, split_major, gscale)
#define GW4_W4_BY_GROUP(MTV, WV)                                                                                 \
    { if (w4_group == 0) GW4_LAUNCH_W4(MTV, WV, 0); else if (w4_group == 64) GW4_LAUNCH_W4(MTV, WV, 64);          \
      else GW4_LAUNCH_W4(MTV, WV, 128); }
    if (w4_group >= 0) {
        if (p.mt == 1) GW4_W4_BY_GROUP(1, 4)
        else if (p.mt == 2) GW4_W4_BY_GROUP(2, 4)
        else GW4_W4_BY_GROUP(4, 8)
    } else
    if (p.mt == 1) { if (ktail) GW4_LAUNCH(1, 4, true); else GW4_LAUNCH(1, 4, false); }
    else if (p.mt == 2) { if (ktail) GW4_LAUNCH(2, 4, true); else GW4_LAUNCH(2, 4, false); }
    else if (p.waves == 8) { if (ktail) GW4_LAUNCH(4, 8, true); else GW4_LAUNCH(4, 8, false); }
    else { if (ktail) GW4_LAUNCH(4, 4, true); else GW4_LAUNCH(4, 4, false); }
#undef GW4_LAUNCH
#undef GW4_LAUNCH_W4
#undef GW4_W4_BY_GROUP
    int rc = MF_LAUNCH_CHECK();
    if (rc) return rc;
    if (rc_args && partial) {                                 // reduce + RoPE + cache scatter in one kernel
        const RopeCacheArgs& a = *rc_args;
        const int items = (a.n_heads + a.n_kv) * (a.head_dim / 16) + a.n_kv * a.head_dim / 8;
        const dim3 rgrid(m, (items + RC_THREADS - 1) / RC_THREADS);
        if (a.kv_scale)
            hipLaunchKernelGGL((w8a16_reduce_rope_cache_kernel<T, true>), rgrid, dim3(RC_THREADS), 0, st, (uint16_t*)y,
                               partial, scale, (const uint16_t*)bias, a.cos, a.sin, a.key_cache, a.value_cache,
                               a.slot_mapping, m, n, p.split_k, a.n_heads, a.n_kv, a.head_dim, a.num_slots,
                               a.table_dtype, a.kv_scale, a.kv_offset);
        else
            hipLaunchKernelGGL((w8a16_reduce_rope_cache_kernel<T, false>), rgrid, dim3(RC_THREADS), 0, st, (uint16_t*)y,
                               partial, scale, (const uint16_t*)bias, a.cos, a.sin, a.key_cache, a.value_cache,
                               a.slot_mapping, m, n, p.split_k, a.n_heads, a.n_kv, a.head_dim, a.num_slots,
                               a.table_dtype, (const float*)nullptr, (const float*)nullptr);
        return MF_LAUNCH_CHECK();
    }
    if (rc_args && rc_args->kv_scale) {                       // no split, int8 caches: rotate, then quantise and scatter
        const RopeCacheArgs& a = *rc_args;
        uint16_t* q = (uint16_t*)y;
        uint16_t* kk = q + (int64_t)a.n_heads * a.head_dim;
        int e = mf_rope_half(q, kk, a.cos, a.sin, m, a.n_heads, a.n_kv, a.head_dim, n, n, T::id, a.table_dtype, st);
        if (e) return e;
        return mf_quant_reshape_and_cache(kk, kk + (int64_t)a.n_kv * a.head_dim, a.key_cache, a.value_cache,
                                          a.slot_mapping, a.kv_scale, a.kv_offset, m, a.n_kv, a.head_dim, a.num_slots, n,
                                          n, T::id, st);
    }
    if (rc_args) {                                            // no split: the GEMM wrote qkv; rotate and scatter
        const RopeCacheArgs& a = *rc_args;
        uint16_t* q = (uint16_t*)y;
        return mf_rope_and_cache(q, q + (int64_t)a.n_heads * a.head_dim, q + (int64_t)(a.n_heads + a.n_kv) * a.head_dim,
                                 a.cos, a.sin, a.key_cache, a.value_cache, a.slot_mapping, m, a.n_heads, a.n_kv,
                                 a.head_dim, a.num_slots, n, n, n, T::id, a.table_dtype, st);
    }
    if (norm_out && partial) {                                // reduce + residual + RMSNorm in one kernel
        hipLaunchKernelGGL((w8a16_reduce_add_rmsnorm_kernel<T>), dim3(m), dim3(RN_THREADS), 0, st, (uint16_t*)norm_out,
                           (uint16_t*)y, partial, scale, (const uint16_t*)bias, (const uint16_t*)residual, gamma, eps, m,
                           n, p.split_k, gamma_dtype, norm_cols);
        return MF_LAUNCH_CHECK();
    }
    if (norm_out)                                             // no split: the GEMM wrote h; normalise it
        return mf_rmsnorm_strided(norm_out, y, n, gamma, eps, m, norm_cols, T::id, gamma_dtype, st);
    if (!partial) return rc;
    const int64_t total = (int64_t)m * ((n + 3) / 4);
    const int blocks = (int)((total + 255) / 256 > 4096 ? 4096 : (total + 255) / 256);
    hipLaunchKernelGGL((w8a16_splitk_reduce_kernel<T>), dim3(blocks), dim3(256), 0, st, (uint16_t*)y, partial, scale,
                       (const uint16_t*)bias, (const uint16_t*)residual, m, n, p.split_k, gated);
    return MF_LAUNCH_CHECK();
}

}  // namespace

extern "C" size_t mf_w8a16_packed_bytes(int n, int k) {
    if (n <= 0 || k <= 0) return 0;
    return (size_t)((n + 15) / 16) * ((k + GW_KSTEP - 1) / GW_KSTEP) * GW_TILE_BYTES;
}

extern "C" int mf_w8a16_pack_weight(void* packed, const int8_t* w, int n, int k, void* stream) {
    MF_REQUIRE(packed && w, "w8a16_pack_weight: null argument");
    MF_REQUIRE(n > 0 && k > 0, "w8a16_pack_weight: bad sizes n=%d k=%d", n, k);
    MF_REQUIRE(((uintptr_t)packed & 15) == 0, "w8a16_pack_weight: packed buffer must be 16-byte aligned");
    const int KS = (k + GW_KSTEP - 1) / GW_KSTEP;
    const int64_t chunks = (int64_t)mf_w8a16_packed_bytes(n, k) / 16;
    const int blocks = (int)((chunks + 255) / 256 > 65535 ? 65535 : (chunks + 255) / 256);
    hipLaunchKernelGGL(w8a16_pack_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (uint8_t*)packed, w, n, k, KS,
                       chunks);
    return MF_LAUNCH_CHECK();
}

extern "C" size_t mf_w8a16_workspace_bytes(int m, int n, int k) {
    if (m <= 0 || n <= 0 || k <= 0) return 0;
    const GemmPlan p = plan_w8a16(m, n, k);
    return p.split_k > 1 ? (size_t)p.split_k * m * n * sizeof(float) : 0;
}

static int w8a16_gemm_entry(const char* who, void* y, const void* x, const void* w_packed, const float* scale,
                            const void* bias, const void* residual, int m, int n, int k, int dtype, int gated,
                            void* workspace, size_t workspace_bytes, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "%s: dtype must be bf16 or fp16", who);
    if (m == 0) return 0;
    MF_REQUIRE(y && x && w_packed && scale, "%s: null argument", who);
    MF_REQUIRE(m >= 0 && n > 0 && k > 0, "%s: bad sizes m=%d n=%d k=%d", who, m, n, k);
    MF_REQUIRE(k % 8 == 0, "%s: K (%d) must be a multiple of 8", who, k);
    MF_REQUIRE(!gated || n % 2 == 0, "%s: N (%d) must be even (gate/up pairs)", who, n);
    MF_REQUIRE((((uintptr_t)x | (uintptr_t)w_packed) & 15) == 0, "%s: x and w_packed must be 16-byte aligned", who);
    const size_t need = mf_w8a16_workspace_bytes(m, n, k);
    MF_REQUIRE(need == 0 || (workspace && workspace_bytes >= need && ((uintptr_t)workspace & 15) == 0),
               "%s: 16-byte aligned workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
    if (dtype == MF_BF16)
        return launch_w8a16<BF16>(y, x, (const uint8_t*)w_packed, scale, bias, residual, m, n, k, gated, workspace,
                                  (hipStream_t)stream);
    return launch_w8a16<FP16>(y, x, (const uint8_t*)w_packed, scale, bias, residual, m, n, k, gated, workspace,
                              (hipStream_t)stream);
}

extern "C" int mf_w8a16_gemm(void* y, const void* x, const void* w_packed, const float* scale, const void* bias,
                             const void* residual, int m, int n, int k, int dtype, void* workspace,
                             size_t workspace_bytes, void* stream) {
    return w8a16_gemm_entry("w8a16_gemm", y, x, w_packed, scale, bias, residual, m, n, k, dtype, 0, workspace,
                            workspace_bytes, stream);
}

extern "C" int mf_w8a16_gemm_add_rmsnorm(void* y_norm, void* h_out, const void* x, const void* w_packed,
                                         const float* scale, const void* bias, const void* residual,
                                         const void* gamma, float eps, int m, int n, int k, int dtype,
                                         int gamma_dtype, void* workspace, size_t workspace_bytes, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "w8a16_gemm_add_rmsnorm: dtype must be bf16 or fp16");
    MF_REQUIRE(gamma_dtype == MF_BF16 || gamma_dtype == MF_FP16 || gamma_dtype == MF_FP32,
               "w8a16_gemm_add_rmsnorm: bad gamma dtype");
    if (m == 0) return 0;
    MF_REQUIRE(y_norm && h_out && x && w_packed && scale && residual && gamma, "w8a16_gemm_add_rmsnorm: null argument");
    MF_REQUIRE(m >= 0 && n > 0 && k > 0 && k % 8 == 0, "w8a16_gemm_add_rmsnorm: bad sizes m=%d n=%d k=%d", m, n, k);
    MF_REQUIRE(n % 8 == 0 && n <= RN_THREADS * RN_MAX_VEC * 8,
               "w8a16_gemm_add_rmsnorm: N (%d) must be a multiple of 8 and at most %d", n, RN_THREADS * RN_MAX_VEC * 8);
    MF_REQUIRE((((uintptr_t)x | (uintptr_t)w_packed | (uintptr_t)y_norm | (uintptr_t)h_out | (uintptr_t)residual |
                 (uintptr_t)gamma | (uintptr_t)scale | (uintptr_t)bias) & 15) == 0,
               "w8a16_gemm_add_rmsnorm: pointers must be 16-byte aligned");
    const size_t need = mf_w8a16_workspace_bytes(m, n, k);
    MF_REQUIRE(need == 0 || (workspace && workspace_bytes >= need && ((uintptr_t)workspace & 15) == 0),
               "w8a16_gemm_add_rmsnorm: 16-byte aligned workspace of %zu bytes needed, %zu given", need,
               workspace_bytes);
    if (dtype == MF_BF16)
        return launch_w8a16<BF16>(h_out, x, (const uint8_t*)w_packed, scale, bias, residual, m, n, k, 0, workspace,
                                  (hipStream_t)stream, y_norm, gamma, eps, gamma_dtype);
    return launch_w8a16<FP16>(h_out, x, (const uint8_t*)w_packed, scale, bias, residual, m, n, k, 0, workspace,
                              (hipStream_t)stream, y_norm, gamma, eps, gamma_dtype);
}

extern "C" int mf_w8a16_gemm_rmsnorm_leading(void* y_norm, void* h_out, const void* x, const void* w_packed,
                                             const float* scale, const void* bias, const void* gamma, float eps, int m,
                                             int n, int k, int norm_cols, int dtype, int gamma_dtype, void* workspace,
                                             size_t workspace_bytes, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "w8a16_gemm_rmsnorm_leading: dtype must be bf16 or fp16");
    MF_REQUIRE(gamma_dtype == MF_BF16 || gamma_dtype == MF_FP16 || gamma_dtype == MF_FP32,
               "w8a16_gemm_rmsnorm_leading: bad gamma dtype");
    if (m == 0) return 0;
    MF_REQUIRE(y_norm && h_out && x && w_packed && scale && gamma, "w8a16_gemm_rmsnorm_leading: null argument");
    MF_REQUIRE(m >= 0 && n > 0 && k > 0 && k % 8 == 0, "w8a16_gemm_rmsnorm_leading: bad sizes m=%d n=%d k=%d", m, n, k);
    MF_REQUIRE(n % 8 == 0 && n <= RN_THREADS * RN_MAX_VEC * 8,
               "w8a16_gemm_rmsnorm_leading: N (%d) must be a multiple of 8 and at most %d", n,
               RN_THREADS * RN_MAX_VEC * 8);
    MF_REQUIRE(norm_cols > 0 && norm_cols <= n && norm_cols % 8 == 0,
               "w8a16_gemm_rmsnorm_leading: norm_cols (%d) must be a multiple of 8 in 8 .. N (%d)", norm_cols, n);
    MF_REQUIRE((((uintptr_t)x | (uintptr_t)w_packed | (uintptr_t)y_norm | (uintptr_t)h_out | (uintptr_t)gamma |
                 (uintptr_t)scale | (uintptr_t)bias) & 15) == 0,
               "w8a16_gemm_rmsnorm_leading: pointers must be 16-byte aligned");
    const size_t need = mf_w8a16_workspace_bytes(m, n, k);
    MF_REQUIRE(need == 0 || (workspace && workspace_bytes >= need && ((uintptr_t)workspace & 15) == 0),
               "w8a16_gemm_rmsnorm_leading: 16-byte aligned workspace of %zu bytes needed, %zu given", need,
               workspace_bytes);
    if (dtype == MF_BF16)
        return launch_w8a16<BF16>(h_out, x, (const uint8_t*)w_packed, scale, bias, nullptr, m, n, k, 0, workspace,
                                  (hipStream_t)stream, y_norm, gamma, eps, gamma_dtype, nullptr, -1, norm_cols);
    return launch_w8a16<FP16>(h_out, x, (const uint8_t*)w_packed, scale, bias, nullptr, m, n, k, 0, workspace,
                              (hipStream_t)stream, y_norm, gamma, eps, gamma_dtype, nullptr, -1, norm_cols);
}

extern "C" int mf_w8a16_qkv_rope_and_cache(void* qkv, const void* x, const void* w_packed, const float* scale,
                                           const void* bias, const void* cos, const void* sin, void* key_cache,
                                           void* value_cache, const int32_t* slot_mapping, int m, int n_heads,
                                           int n_kv_heads, int head_dim, int64_t num_slots, int k, int dtype,
                                           int table_dtype, void* workspace, size_t workspace_bytes, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "w8a16_qkv_rope_and_cache: dtype must be bf16 or fp16");
    MF_REQUIRE(table_dtype == MF_BF16 || table_dtype == MF_FP16 || table_dtype == MF_FP32,
               "w8a16_qkv_rope_and_cache: bad table dtype");
    if (m == 0) return 0;
    MF_REQUIRE(qkv && x && w_packed && scale && cos && sin && key_cache && value_cache && slot_mapping,
               "w8a16_qkv_rope_and_cache: null argument");
    MF_REQUIRE(m >= 0 && n_heads > 0 && n_kv_heads > 0 && k > 0 && k % 8 == 0 && num_slots > 0,
               "w8a16_qkv_rope_and_cache: bad sizes");
    MF_REQUIRE(head_dim > 0 && head_dim % 16 == 0, "w8a16_qkv_rope_and_cache: head_dim (%d) must be a multiple of 16",
               head_dim);
    const int n = (n_heads + 2 * n_kv_heads) * head_dim;
    MF_REQUIRE((((uintptr_t)x | (uintptr_t)w_packed | (uintptr_t)qkv | (uintptr_t)cos | (uintptr_t)sin |
                 (uintptr_t)key_cache | (uintptr_t)value_cache | (uintptr_t)scale | (uintptr_t)bias) & 15) == 0,
               "w8a16_qkv_rope_and_cache: pointers must be 16-byte aligned");
    const size_t need = mf_w8a16_workspace_bytes(m, n, k);
    MF_REQUIRE(need == 0 || (workspace && workspace_bytes >= need && ((uintptr_t)workspace & 15) == 0),
               "w8a16_qkv_rope_and_cache: 16-byte aligned workspace of %zu bytes needed, %zu given", need,
               workspace_bytes);
    const RopeCacheArgs a = {cos, sin, key_cache, value_cache, slot_mapping, n_heads, n_kv_heads, head_dim, table_dtype,
                             num_slots, nullptr, nullptr};
    if (dtype == MF_BF16)
        return launch_w8a16<BF16>(qkv, x, (const uint8_t*)w_packed, scale, bias, nullptr, m, n, k, 0, workspace,
                                  (hipStream_t)stream, nullptr, nullptr, 0.f, MF_FP32, &a);
    return launch_w8a16<FP16>(qkv, x, (const uint8_t*)w_packed, scale, bias, nullptr, m, n, k, 0, workspace,
                              (hipStream_t)stream, nullptr, nullptr, 0.f, MF_FP32, &a);
}

extern "C" int mf_w8a16_qkv_rope_and_quant_cache(void* qkv, const void* x, const void* w_packed, const float* scale,
                                                 const void* bias, const void* cos, const void* sin, void* key_cache,
                                                 void* value_cache, const int32_t* slot_mapping, const float* kv_scale,
                                                 const float* kv_offset, int m, int n_heads, int n_kv_heads,
                                                 int head_dim, int64_t num_slots, int k, int dtype, int table_dtype,
                                                 void* workspace, size_t workspace_bytes, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "w8a16_qkv_rope_and_quant_cache: dtype must be bf16 or fp16");
    MF_REQUIRE(table_dtype == MF_BF16 || table_dtype == MF_FP16 || table_dtype == MF_FP32,
               "w8a16_qkv_rope_and_quant_cache: bad table dtype");
    if (m == 0) return 0;
    MF_REQUIRE(qkv && x && w_packed && scale && cos && sin && key_cache && value_cache && slot_mapping && kv_scale,
               "w8a16_qkv_rope_and_quant_cache: null argument");
    MF_REQUIRE(m >= 0 && n_heads > 0 && n_kv_heads > 0 && k > 0 && k % 8 == 0 && num_slots > 0,
               "w8a16_qkv_rope_and_quant_cache: bad sizes");
    MF_REQUIRE(head_dim > 0 && head_dim % 16 == 0,
               "w8a16_qkv_rope_and_quant_cache: head_dim (%d) must be a multiple of 16", head_dim);
    const int n = (n_heads + 2 * n_kv_heads) * head_dim;
    MF_REQUIRE((((uintptr_t)x | (uintptr_t)w_packed | (uintptr_t)qkv | (uintptr_t)cos | (uintptr_t)sin |
                 (uintptr_t)scale | (uintptr_t)bias) & 15) == 0 &&
                   (((uintptr_t)key_cache | (uintptr_t)value_cache) & 7) == 0,
               "w8a16_qkv_rope_and_quant_cache: pointers must be 16-byte aligned, the caches 8-byte aligned");
    const size_t need = mf_w8a16_workspace_bytes(m, n, k);
    MF_REQUIRE(need == 0 || (workspace && workspace_bytes >= need && ((uintptr_t)workspace & 15) == 0),
               "w8a16_qkv_rope_and_quant_cache: 16-byte aligned workspace of %zu bytes needed, %zu given", need,
               workspace_bytes);
    const RopeCacheArgs a = {cos, sin, key_cache, value_cache, slot_mapping, n_heads, n_kv_heads, head_dim, table_dtype,
                             num_slots, kv_scale, kv_offset};
    if (dtype == MF_BF16)
        return launch_w8a16<BF16>(qkv, x, (const uint8_t*)w_packed, scale, bias, nullptr, m, n, k, 0, workspace,
                                  (hipStream_t)stream, nullptr, nullptr, 0.f, MF_FP32, &a);
    return launch_w8a16<FP16>(qkv, x, (const uint8_t*)w_packed, scale, bias, nullptr, m, n, k, 0, workspace,
                              (hipStream_t)stream, nullptr, nullptr, 0.f, MF_FP32, &a);
}

extern "C" int mf_w8a16_gemm_silu_mul(void* y, const void* x, const void* w_packed, const float* scale,
                                      const void* bias, int m, int n, int k, int dtype, void* workspace,
                                      size_t workspace_bytes, void* stream) {
    return w8a16_gemm_entry("w8a16_gemm_silu_mul", y, x, w_packed, scale, bias, nullptr, m, n, k, dtype, 1, workspace,
                            workspace_bytes, stream);
}

static int grouped_w8a16_entry(const char* who, void* y, const void* x, const void* w_packed, const float* scale,
                               const int32_t* offsets, int n_experts, int total_rows, int n, int k, int dtype, int gated,
                               void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "%s: dtype must be bf16 or fp16", who);
    if (total_rows == 0) return 0;
    MF_REQUIRE(y && x && w_packed && scale && offsets, "%s: null argument", who);
    MF_REQUIRE(n_experts > 0 && n_experts <= 65535 && total_rows >= 0 && n > 0 && k > 0, "%s: bad sizes", who);
    MF_REQUIRE(k % 8 == 0, "%s: K (%d) must be a multiple of 8", who, k);
    MF_REQUIRE(!gated || n % 4 == 0, "%s: N (%d) must be a multiple of 4 (gate / up pairs)", who, n);
    MF_REQUIRE((((uintptr_t)x | (uintptr_t)w_packed) & 15) == 0, "%s: x and w_packed must be 16-byte aligned", who);
    const int64_t expert_bytes = (int64_t)mf_w8a16_packed_bytes(n, k);
    dim3 grid((n + GW_BN - 1) / GW_BN, n_experts);
#define GG_LAUNCH(TT, KT)                                                                                        \
    hipLaunchKernelGGL((w8a16_grouped_kernel<TT, KT>), grid, dim3(GW_WAVES * 64), 0, (hipStream_t)stream,           \
                       (uint16_t*)y, (const uint16_t*)x, (const uint8_t*)w_packed, scale, offsets, total_rows, n, k, \
                       expert_bytes, gated)
    const bool ktail = (k % GW_KSTEP) != 0;
    if (dtype == MF_BF16) { if (ktail) GG_LAUNCH(BF16, true); else GG_LAUNCH(BF16, false); }
    else { if (ktail) GG_LAUNCH(FP16, true); else GG_LAUNCH(FP16, false); }
#undef GG_LAUNCH
    return MF_LAUNCH_CHECK();
}

extern "C" int mf_grouped_w8a16_gemm(void* y, const void* x, const void* w_packed, const float* scale,
                                     const int32_t* offsets, int n_experts, int total_rows, int n, int k, int dtype,
                                     void* stream) {
    return grouped_w8a16_entry("grouped_w8a16_gemm", y, x, w_packed, scale, offsets, n_experts, total_rows, n, k, dtype,
                               0, stream);
}

extern "C" int mf_grouped_w8a16_gemm_silu_mul(void* y, const void* x, const void* w_packed, const float* scale,
                                              const int32_t* offsets, int n_experts, int total_rows, int n, int k,
                                              int dtype, void* stream) {
    return grouped_w8a16_entry("grouped_w8a16_gemm_silu_mul", y, x, w_packed, scale, offsets, n_experts, total_rows, n,
                               k, dtype, 1, stream);
}

// ---- 4-bit weights ---------------------------------------------------------------------------------------------------
extern "C" size_t mf_w4a16_packed_bytes(int n, int k) {
    if (n <= 0 || k <= 0) return 0;
    return (size_t)((n + 15) / 16) * ((k + GW_KSTEP - 1) / GW_KSTEP) * (GW_TILE_BYTES / 2);
}

extern "C" int mf_w4a16_pack_weight(void* packed, const int8_t* w, int n, int k, void* stream) {
    MF_REQUIRE(packed && w && n > 0 && k > 0, "w4a16_pack_weight: bad arguments");
    MF_REQUIRE(((uintptr_t)packed & 15) == 0, "w4a16_pack_weight: packed buffer must be 16-byte aligned");
    const int64_t chunks = (int64_t)mf_w4a16_packed_bytes(n, k) / 8;
    const int blocks = (int)((chunks + 255) / 256 > 65535 ? 65535 : (chunks + 255) / 256);
    hipLaunchKernelGGL(w4a16_pack_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (uint8_t*)packed, w, n, k,
                       chunks);
    return MF_LAUNCH_CHECK();
}

extern "C" size_t mf_w4a16_workspace_bytes(int m, int n, int k, int group_size) {
    if (m <= 0 || n <= 0 || k <= 0) return 0;
    const GemmPlan p = plan_w8a16(m, n, k, group_size == 128 ? 2 : 1);
    return p.split_k > 1 ? (size_t)p.split_k * m * n * sizeof(float) : 0;
}

extern "C" int mf_w4a16_gemm(void* y, const void* x, const void* w_packed, const float* scale, const void* bias,
                             const void* residual, int m, int n, int k, int group_size, int dtype, void* workspace,
                             size_t workspace_bytes, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "w4a16_gemm: dtype must be bf16 or fp16");
    if (m == 0) return 0;
    MF_REQUIRE(y && x && w_packed && scale, "w4a16_gemm: null argument");
    MF_REQUIRE(m >= 0 && n > 0 && k > 0, "w4a16_gemm: bad sizes m=%d n=%d k=%d", m, n, k);
    MF_REQUIRE(group_size == 0 || group_size == 64 || group_size == 128,
               "w4a16_gemm: group_size %d not supported (0 = per channel, 64, 128)", group_size);
    MF_REQUIRE(k % 64 == 0 && (group_size == 0 || k % group_size == 0),
               "w4a16_gemm: K (%d) must be a multiple of 64 and of the group size", k);
    MF_REQUIRE(group_size == 0 || n % 4 == 0, "w4a16_gemm: N (%d) must be a multiple of 4 with per-group scales", n);
    MF_REQUIRE((((uintptr_t)x | (uintptr_t)w_packed | (uintptr_t)scale) & 15) == 0,
               "w4a16_gemm: x, w_packed and scale must be 16-byte aligned");
    const size_t need = mf_w4a16_workspace_bytes(m, n, k, group_size);
    MF_REQUIRE(need == 0 || (workspace && workspace_bytes >= need && ((uintptr_t)workspace & 15) == 0),
               "w4a16_gemm: 16-byte aligned workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    if (dtype == MF_BF16)
        return launch_w8a16<BF16>(y, x, (const uint8_t*)w_packed, scale, bias, residual, m, n, k, 0, workspace,
                                  (hipStream_t)stream, nullptr, nullptr, 0.f, MF_FP32, nullptr, group_size);
    return launch_w8a16<FP16>(y, x, (const uint8_t*)w_packed, scale, bias, residual, m, n, k, 0, workspace,
                              (hipStream_t)stream, nullptr, nullptr, 0.f, MF_FP32, nullptr, group_size);
}
