// W8A8 GEMM: per-token int8 activations x per-channel int8 weights on the gfx950 int8 matrix cores
// (v_mfma_i32_16x16x64_i8), exact int32 accumulation, dequantised to bf16/fp16 in the epilogue:
//   y[m,n] = acc[m,n] * x_scale[m] * w_scale[n] (+ bias[n]) (+ residual[m,n]).
//
// Weights come in the packed tile order of mf_w8a16_pack_weight (1 KiB tiles of 16 output channels x 64 input
// channels, bytes in lane order): 16 consecutive k bytes per lane is the int8 MFMA operand layout as well, so a
// tile is one coalesced wave-wide load and needs no shuffle.  Activations are the row-major int8 [M, K] that
// mf_dynamic_quant_per_token writes.
//
// A workgroup of 4 waves owns BM x BN outputs and walks K in 64-byte steps.  Both operand tiles of a step go
// global -> LDS with LDS-direct loads (no registers in between), two steps ahead of their use, into a ring of
// three stages; one barrier per step.  Every wave issues the same number of loads per step and they complete in
// issue order, so "at most one step's loads outstanding" means this wave's part of the current step has landed.
// The LDS reads and their waits are asm statements (the compiler would wait for every LDS-direct load before any
// LDS read); each wait names the registers it makes valid.
//   M > 64:  waves split the rows (64 each, BM = 256), every wave multiplies its 4 row tiles with all NT weight
//            tiles of the step (BN = 16*NT): 4 + NT operand reads feed 4*NT matrix instructions.
//   M <= 64: one row block, waves split the channels (BN = 64*NT).
// The 64-byte activation rows are XOR-swizzled in LDS (16-byte chunk c of row r sits at chunk c ^ 2*[r & 8]),
// applied on the global-address side, which makes the operand reads bank-conflict free.
// Small N cannot fill the chip with output tiles alone: K is then split across workgroups, which write exact
// int32 partial tiles that a second kernel sums (integer sums do not depend on the order).
// Two more kernels serve the shapes where that one is not the best: a register-streaming kernel for narrow outputs
// at 65+ rows (w8a8_regs_kernel) and, for very wide outputs at 129+ rows, 256 x 192 tiles on 8 waves with the
// full-rate v_mfma_i32_32x32x32_i8 and a coalesced, LDS-turned epilogue (w8a8_wide_kernel).
#include "common.h"

namespace {

constexpr int Q_KSTEP = 64;
constexpr int Q_TILE = 16 * Q_KSTEP;        // bytes of one packed weight tile
static_assert(Q_KSTEP == MF_PACK_KSTEP && Q_TILE == MF_PACK_TILE_BYTES, "the int8 GEMMs read the shared packed format");

// MSPLIT: wave grid of a workgroup.  0: 1 x 4 (64 rows, the waves own different channels); 1: 4 x 1 (256 rows, one
// channel group).
template <int NT, int MSPLIT, int ST>
struct Q2 {
    static constexpr int STAGES = ST;
    static constexpr int WAVES_M = MSPLIT ? 4 : 1;
    static constexpr int WAVES_N = MSPLIT ? 1 : 4;
    static constexpr int WAVES = WAVES_M * WAVES_N;
    static constexpr int BM = 64 * WAVES_M;
    static constexpr int BN = 16 * NT * WAVES_N;
    static constexpr int XTILE = BM * Q_KSTEP;
    static constexpr int WTILES = BN / 16;
    static constexpr int STAGE = XTILE + WTILES * Q_TILE;
    static constexpr int XL = BM / 16 / WAVES;                // activation loads (16 rows each) per wave per stage
    static constexpr int WL = (WTILES + WAVES - 1) / WAVES;   // weight tile loads per wave per stage
    static_assert((BM / 16) % WAVES == 0, "activation tiles must divide over the waves");
    static constexpr int PENDING = (ST - 2) * (XL + WL);      // loads of the ST-2 younger steps may be in flight
    static constexpr int LDS_BYTES = ST * STAGE;
    static_assert(LDS_BYTES <= 160 * 1024 && PENDING < 64, "bad pipeline shape");
};

__device__ __forceinline__ int q2_swizzle_key(int row) { return ((row >> 3) & 1) << 1; }

template <int OFFSET>
__device__ __forceinline__ i32x4 q2_lds_read16(uint32_t addr) {
    i32x4 v;
    if constexpr (OFFSET >= 65536) addr += (OFFSET >> 16) << 16;    // the offset field has 16 bits
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(v) : "v"(addr), "n"(OFFSET & 65535) : "memory");
    return v;
}
__device__ __forceinline__ void q2_lds_direct16(const uint8_t* base_uniform, uint32_t lane_offset,
                                                uint8_t* dst_wave_uniform) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(base_uniform + lane_offset),
                                     (__attribute__((address_space(3))) void*)dst_wave_uniform, 16, 0, 0);
}

// Dequantising store of 4 consecutive channels of one row.
template <typename T>
__device__ __forceinline__ void q2_store4(uint16_t* y, int32_t* acc_out, const float* x_scale, const float* w_scale,
                                          const uint16_t* bias, const uint16_t* residual, int m, int n, int N,
                                          i32x4 a) {
    const int64_t o = (int64_t)m * N + n;
    const bool vec = n + 3 < N && (N & 3) == 0;
    if (acc_out) {
        if (vec) {
            *(i32x4*)(acc_out + o) = a;
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (n + i < N) acc_out[o + i] = a[i];
        }
    }
    if (!y) return;
    const float xs = x_scale[m];
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[i] = 0.f;
        if (n + i < N) {
            float t = (float)a[i] * xs * w_scale[n + i];
            if (bias) t += T::to_float(bias[n + i]);
            if (residual) t = T::to_float(T::from_float(t)) + T::to_float(residual[o + i]);
            v[i] = t;
        }
    }
    if (vec) {
        *(u32x2*)(y + o) = (u32x2){pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3])};
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (n + i < N) y[o + i] = T::from_float(v[i]);
    }
}

// grid = (n_blocks, split_k, m_blocks)
template <typename T, int NT, int MSPLIT, int ST, bool KTAIL, bool XT>
__global__ __launch_bounds__(256, 2) void w8a8_gemm_kernel(
    uint16_t* __restrict__ y, int32_t* __restrict__ acc_out, int32_t* __restrict__ partial,
    const int8_t* __restrict__ xq, const float* __restrict__ x_scale, const uint8_t* __restrict__ wp,
    const float* __restrict__ w_scale, const uint16_t* __restrict__ bias, const uint16_t* __restrict__ residual, int M,
    int N, int K, int steps_per_split) {
    using C = Q2<NT, MSPLIT, ST>;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];       // C::LDS_BYTES, set by the launcher

    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    const int wm = MSPLIT ? wv : 0, wn = MSPLIT ? 0 : wv;
    const int KS = (K + Q_KSTEP - 1) / Q_KSTEP;
    const int s_begin = blockIdx.y * steps_per_split;
    const int s_end = min(KS, s_begin + steps_per_split);
    const int s_last = s_end - 1;
    const int m0 = blockIdx.z * C::BM;
    const int nb = blockIdx.x * C::BN;                        // first channel of the workgroup
    const int nw = nb + wn * 16 * NT;                         // first channel this wave computes

    i32x4 acc[NT][4];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) acc[nt][mt] = (i32x4){0, 0, 0, 0};

    // activation loads: load i of this wave covers rows 16*(wv*XL + i) .. + 15 of the stage.
    //   tiled xq (XT): a 16-row tile of a step is 1 KiB of contiguous memory in operand order, like a weight tile
    //   (tiles ordered [step][row tile]);
    //   row-major xq: 4 lanes per 64-byte row piece; lane -> (row, physical chunk), the global address uses the
    //   logical chunk.  Rows (row tiles) past M re-read the last one; their results are never stored.
    const uint8_t* xbase = (const uint8_t*)xq + (XT ? 0 : (int64_t)m0 * K);
    uint32_t xlane[C::XL];
    int xchunk[C::XL];
    const uint8_t* xtile[C::XL];
    const int m_tiles_total = (M + 15) >> 4;
#pragma unroll
    for (int i = 0; i < C::XL; ++i) {
        const int row = 16 * (wv * C::XL + i) + (lane >> 2);
        xchunk[i] = 16 * ((lane & 3) ^ q2_swizzle_key(row));
        xlane[i] = (uint32_t)min(row, M - 1 - m0) * (uint32_t)K + xchunk[i];
        xtile[i] = xbase + (int64_t)min((m0 >> 4) + wv * C::XL + i, m_tiles_total - 1) * Q_TILE;
    }
    // weight loads: tile j of the stage is n-tile nb/16 + j; this wave loads tiles wv*WL + i (clamped: a wave with
    // fewer tiles re-loads the last one onto itself, so that all waves issue the same number of loads)
    const int n_tiles_total = (N + 15) >> 4;
    const uint8_t* wtile[C::WL];
    int wdst[C::WL];
#pragma unroll
    for (int i = 0; i < C::WL; ++i) {
        const int j = min(wv * C::WL + i, C::WTILES - 1);
        const int t = min((nb >> 4) + j, n_tiles_total - 1);
        wtile[i] = wp + (int64_t)t * Q_TILE;
        wdst[i] = C::XTILE + j * Q_TILE;
    }
    const uint32_t wlane = lane * 16;

    auto issue = [&](int stage, int s) {
        const int sc = min(s, s_last);
        uint8_t* dst = smem + stage * C::STAGE;
#pragma unroll
        for (int i = 0; i < C::XL; ++i) {
            if (XT) {
                q2_lds_direct16(xtile[i] + (int64_t)sc * m_tiles_total * Q_TILE, wlane, dst + 1024 * (wv * C::XL + i));
                continue;
            }
            uint32_t off = xlane[i] + (uint32_t)sc * Q_KSTEP;
            if (KTAIL) {
                // chunks past K (last, short step) re-read the row's last whole chunk; they meet zero weights
                const int over = sc * Q_KSTEP + xchunk[i] - (K - 16);
                off -= over > 0 ? (uint32_t)over : 0u;
            }
            q2_lds_direct16(xbase, off, dst + 1024 * (wv * C::XL + i));
        }
#pragma unroll
        for (int i = 0; i < C::WL; ++i)
            q2_lds_direct16(wtile[i] + (int64_t)sc * n_tiles_total * Q_TILE, wlane, dst + wdst[i]);
    };
#pragma unroll
    for (int p = 0; p < ST - 1; ++p) issue(p, s_begin + p);

    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
    // operand reads: activation tile mt = row 64*wm + 16*mt + r, logical chunk g; weight tile = lane-linear
    const uint32_t xoff = XT ? lds0 + 64 * wm * Q_KSTEP + lane * 16
                             : lds0 + (64 * wm + r) * Q_KSTEP + ((g ^ q2_swizzle_key(r)) << 4);
    const uint32_t woff = lds0 + C::XTILE + wn * NT * Q_TILE + lane * 16;

    auto step = [&](auto jc, int s) {
        constexpr int J = decltype(jc)::value;
        constexpr int SB = J * C::STAGE;
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(C::PENDING) : "memory");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        issue((J + ST - 1) % ST, s + ST - 1);
        i32x4 xb[4], wa[NT];
        xb[0] = q2_lds_read16<SB>(xoff);
        xb[1] = q2_lds_read16<SB + 1024>(xoff);
        xb[2] = q2_lds_read16<SB + 2048>(xoff);
        xb[3] = q2_lds_read16<SB + 3072>(xoff);
        static_for<NT>([&](auto nc) {
            constexpr int nt = decltype(nc)::value;
            wa[nt] = q2_lds_read16<SB + nt * Q_TILE>(woff);
        });
        // the reads return in order: the activation tiles and the first weight tile are enough to start
        asm volatile("s_waitcnt lgkmcnt(%5)"
                     : "+v"(xb[0]), "+v"(xb[1]), "+v"(xb[2]), "+v"(xb[3]), "+v"(wa[0])
                     : "n"(NT - 1)
                     : "memory");
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            if (nt == 1) {                                    // the remaining weight tiles have arrived
                if constexpr (NT == 2) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(wa[1])::"memory");
                if constexpr (NT == 4)
                    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(wa[1]), "+v"(wa[2]), "+v"(wa[3])::"memory");
                if constexpr (NT == 5)
                    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(wa[1]), "+v"(wa[2]), "+v"(wa[3]), "+v"(wa[4])::"memory");
                if constexpr (NT == 8)
                    asm volatile("s_waitcnt lgkmcnt(0)"
                                 : "+v"(wa[1]), "+v"(wa[2]), "+v"(wa[3]), "+v"(wa[4]), "+v"(wa[5]), "+v"(wa[6]), "+v"(wa[7])
                                 :
                                 : "memory");
            }
#pragma unroll
            for (int mt = 0; mt < 4; ++mt)
                acc[nt][mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wa[nt], xb[mt], acc[nt][mt], 0, 0, 0);
        }
    };
    for (int s = s_begin; s < s_end; s += ST) {
        step(std::integral_constant<int, 0>{}, s);
        if (s + 1 < s_end) step(std::integral_constant<int, 1>{}, s + 1);
        if (s + 2 < s_end) step(std::integral_constant<int, 2>{}, s + 2);
        if constexpr (ST > 3)
            if (s + 3 < s_end) step(std::integral_constant<int, 3 % ST>{}, s + 3);
        if constexpr (ST > 4)
            if (s + 4 < s_end) step(std::integral_constant<int, 4 % ST>{}, s + 4);
        if constexpr (ST > 5)
            if (s + 5 < s_end) step(std::integral_constant<int, 5 % ST>{}, s + 5);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");         // loads issued past the end still target the ring

    // epilogue: lane (r, g) holds row m = 16*mt + r, channels 4g .. 4g+3 of each tile
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
        const int m = m0 + 64 * wm + 16 * mt + r;
        if (m >= M) continue;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int n = nw + 16 * nt + 4 * g;
            if (n >= N) continue;
            if (partial) {
                int32_t* p = partial + ((int64_t)blockIdx.y * M + m) * N + n;
                if (n + 3 < N && (N & 3) == 0) {
                    *(i32x4*)p = acc[nt][mt];
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (n + i < N) p[i] = acc[nt][mt][i];
                }
            } else {
                q2_store4<T>(y, acc_out, x_scale, w_scale, bias, residual, m, n, N, acc[nt][mt]);
            }
        }
    }
}

// ---- register-streaming kernel (tiled activations) --------------------------------------------------
// With the activations in tile order too, both operands of the int8 matrix instruction are 1 KiB tiles that a wave
// loads with one coalesced 16-byte-per-lane load straight into operand registers: no LDS, no barriers, no
// shuffles.  The 4 waves of a workgroup form a WM x WN grid; a wave owns MT row tiles x NT channel tiles of the
// output and keeps the operand tiles of the next three k-steps in flight in a rotating set of registers.  Tiles
// that several waves of the workgroup need are fetched by each of them (they meet in the L1/L2 caches); what the
// design buys is memory-level parallelism that does not depend on LDS capacity (4 waves x 3 steps x (MT+NT) KiB in
// flight per workgroup) and a main loop that is nothing but loads and matrix instructions.
constexpr int QR_DEPTH = 3;

// ---- wide outputs at 129+ rows: 256 x 192 tiles on 8 waves with mfma_i32_32x32x32_i8 ----------------------------
// On gfx950 the 16x16x64 int8 instruction issues at half the rate of the 32x32x32 one (measured: 2.4 against
// 4.4 POP/s with independent accumulators), so the kernel that is bound by the matrix cores uses the latter.
// The packed tile format serves it unchanged: rows 32 b .. 32 b + 31 of a k-step are two consecutive 1 KiB
// tiles, and lane (rho = lane & 31, h = lane >> 5) finds row rho, bytes 32 u + 16 h .. + 15 of the step at
// tile (rho >> 4), 16-byte slot 16 (2 u + h) + (rho & 15).  Waves 4 (rows) x 2 (channels): a wave owns 64 rows x 96
// channels = 2 x 3 blocks of 32 x 32.  Both operands go global -> LDS with LDS-direct loads into a ring of stages
// (counted waits, one barrier per step); the operands of step s + 1 are read from LDS into a second register set
// while the matrix cores work on step s.  Activations in tile order only.
struct QW {
    static constexpr int ST = 5;                              // stages: all that fit in 160 KiB of LDS
    static constexpr int WAVES = 8;
    static constexpr int BM = 256, WN = 96, BN = 2 * WN;
    static constexpr int XTILE = BM * Q_KSTEP;                // 16 KiB
    static constexpr int WTILES = BN / 16;                    // 12
    static constexpr int STAGE = XTILE + WTILES * Q_TILE;     // 28 KiB
    static constexpr int XL = BM / 16 / WAVES;                // 2 activation tile loads per wave per stage
    static constexpr int WL = (WTILES + WAVES - 1) / WAVES;   // 2 weight tile loads per wave per stage (clamped)
    static constexpr int L = XL + WL;
    static constexpr int LDS_BYTES = ST * STAGE;
};

template <typename T>
__global__ __launch_bounds__(QW::WAVES * 64, 1) void w8a8_wide_kernel(
    uint16_t* __restrict__ y, int32_t* __restrict__ acc_out, int32_t* __restrict__ partial,
    const int8_t* __restrict__ xq, const float* __restrict__ x_scale, const uint8_t* __restrict__ wp,
    const float* __restrict__ w_scale, const uint16_t* __restrict__ bias, const uint16_t* __restrict__ residual, int M,
    int N, int K, int steps_per_split) {
    using C = QW;
    constexpr int ST = C::ST;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int wm = wv & 3, wn = wv >> 2;
    const int KS = (K + Q_KSTEP - 1) / Q_KSTEP;
    const int s_begin = blockIdx.y * steps_per_split;
    const int s_end = min(KS, s_begin + steps_per_split);
    const int s_last = s_end - 1;
    const int m0 = blockIdx.z * C::BM;
    const int nb0 = blockIdx.x * C::BN;
    const int nw = nb0 + wn * C::WN;

    i32x16 acc[3][2];
#pragma unroll
    for (int nb = 0; nb < 3; ++nb)
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[nb][mb][i] = 0;

    // loads: tiles past the matrix re-read the last one (their results are never stored); every wave issues the same
    // number of loads per stage
    const int m_tiles_total = (M + 15) >> 4, n_tiles_total = (N + 15) >> 4;
    const uint8_t* xtile[C::XL];
    const uint8_t* wtile[C::WL];
    int wdst[C::WL];
#pragma unroll
    for (int i = 0; i < C::XL; ++i)
        xtile[i] = (const uint8_t*)xq + (int64_t)min((m0 >> 4) + wv * C::XL + i, m_tiles_total - 1) * Q_TILE;
#pragma unroll
    for (int i = 0; i < C::WL; ++i) {
        const int j = min(wv * C::WL + i, C::WTILES - 1);
        wtile[i] = wp + (int64_t)min((nb0 >> 4) + j, n_tiles_total - 1) * Q_TILE;
        wdst[i] = C::XTILE + j * Q_TILE;
    }
    const uint32_t wlane = lane * 16;
    auto issue = [&](int stage, int s) {
        const int sc = min(s, s_last);
        uint8_t* dst = smem + stage * C::STAGE;
#pragma unroll
        for (int i = 0; i < C::XL; ++i)
            q2_lds_direct16(xtile[i] + (int64_t)sc * m_tiles_total * Q_TILE, wlane, dst + 1024 * (wv * C::XL + i));
#pragma unroll
        for (int i = 0; i < C::WL; ++i)
            q2_lds_direct16(wtile[i] + (int64_t)sc * n_tiles_total * Q_TILE, wlane, dst + wdst[i]);
    };
#pragma unroll
    for (int p = 0; p < ST - 1; ++p) issue(p, s_begin + p);

    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
    const int rho = lane & 31, h = lane >> 5;
    const uint32_t lane32 = (uint32_t)((rho >> 4) * Q_TILE + (16 * h + (rho & 15)) * 16);
    const uint32_t xoff = lds0 + 4 * wm * Q_TILE + lane32;                 // + 2048 mb + 512 u
    const uint32_t woff = lds0 + C::XTILE + 6 * wn * Q_TILE + lane32;      // + 2048 nb + 512 u

    // operand sets: xb[set][mb][u], wa[set][nb][u]
    i32x4 xb[2][2][2], wa[2][3][2];
    auto read_ops = [&](auto jc, int set) {
        constexpr int SB = decltype(jc)::value * C::STAGE;
        xb[set][0][0] = q2_lds_read16<SB>(xoff);
        xb[set][0][1] = q2_lds_read16<SB + 512>(xoff);
        xb[set][1][0] = q2_lds_read16<SB + 2048>(xoff);
        xb[set][1][1] = q2_lds_read16<SB + 2048 + 512>(xoff);
        wa[set][0][0] = q2_lds_read16<SB>(woff);
        wa[set][0][1] = q2_lds_read16<SB + 512>(woff);
        wa[set][1][0] = q2_lds_read16<SB + 2048>(woff);
        wa[set][1][1] = q2_lds_read16<SB + 2048 + 512>(woff);
        wa[set][2][0] = q2_lds_read16<SB + 4096>(woff);
        wa[set][2][1] = q2_lds_read16<SB + 4096 + 512>(woff);
    };
    auto arrived = [&](int set) {                             // operands read one step ago are in their registers
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(xb[set][0][0]), "+v"(xb[set][0][1]), "+v"(xb[set][1][0]), "+v"(xb[set][1][1]),
                       "+v"(wa[set][0][0]), "+v"(wa[set][0][1]), "+v"(wa[set][1][0]), "+v"(wa[set][1][1]),
                       "+v"(wa[set][2][0]), "+v"(wa[set][2][1])
                     :
                     : "memory");
    };
    // step s_begin's stage has landed when at most the loads of the ST-2 younger steps are in flight
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((ST - 2) * C::L) : "memory");
    __builtin_amdgcn_s_barrier();
    read_ops(std::integral_constant<int, 0>{}, 0);
    auto pstep = [&](auto jc, auto setc, int s) {
        constexpr int J = decltype(jc)::value;                // stage of step s
        constexpr int SET = decltype(setc)::value;            // operand register set of step s (the step's parity)
        __builtin_amdgcn_sched_barrier(0);
        // the next step's stage must have landed, and this step's operands must be in their registers
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((ST - 3) * C::L) : "memory");
        arrived(SET);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        issue((J + ST - 1) % ST, s + ST - 1);
        read_ops(std::integral_constant<int, (J + 1) % ST>{}, SET ^ 1);
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int nb = 0; nb < 3; ++nb)
#pragma unroll
                for (int mb = 0; mb < 2; ++mb)
                    acc[nb][mb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wa[SET][nb][u], xb[SET][mb][u], acc[nb][mb], 0, 0, 0);
    };
    // stages cycle with period ST, register sets with period 2: 2 * ST steps per trip
#define QW_STEP(I)                                                                                              \
    if (s + (I) < s_end) pstep(std::integral_constant<int, (I) % ST>{}, std::integral_constant<int, (I) & 1>{}, s + (I))
    for (int s = s_begin; s < s_end; s += 2 * ST) {
        QW_STEP(0); QW_STEP(1); QW_STEP(2); QW_STEP(3); QW_STEP(4);
        QW_STEP(5); QW_STEP(6); QW_STEP(7); QW_STEP(8); QW_STEP(9);
    }
#undef QW_STEP
    static_assert(ST == 5, "the unrolled trip above covers 2 * ST steps");
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");   // look-ahead loads and reads still target the ring

    // epilogue: lane holds row m = 32 mb + rho and, per block, channels 8 q + 4 h .. + 3 for q = 0..3.  Stored
    // straight from that layout a wave would write 8-byte pieces of 32 different rows per instruction, so the
    // dequantised tile (64 rows x 96 channels per wave) is turned through the wave's share of the now idle ring and
    // written out as whole 16-byte pieces of consecutive rows; the int32 / split-K / ragged cases keep the direct path.
    constexpr int EP_STRIDE = C::WN * 2 + 16;                 // bytes per staged row
    static_assert(C::WAVES * 64 * EP_STRIDE <= C::LDS_BYTES, "the staged output must fit the ring");
    if (y && !acc_out && !partial && (N & 7) == 0 && nw + C::WN <= N) {     // uniform per wave
        __syncthreads();                                      // every wave is done with the ring
        uint8_t* ep = smem + wv * (64 * EP_STRIDE);
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
            const int m = min(m0 + 64 * wm + 32 * mb + rho, M - 1);
            const float xs = x_scale[m];
#pragma unroll
            for (int nb = 0; nb < 3; ++nb)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int nl = 32 * nb + 8 * q + 4 * h;
                    const f32x4 ws4 = *(const f32x4*)(w_scale + nw + nl);
                    float v[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        v[i] = (float)acc[nb][mb][4 * q + i] * xs * ws4[i];
                        if (bias) v[i] += T::to_float(bias[nw + nl + i]);
                    }
                    *(u32x2*)(ep + (32 * mb + rho) * EP_STRIDE + nl * 2) =
                        (u32x2){pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3])};
                }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        constexpr int CPRW = C::WN * 2 / 16;                  // 16-byte pieces per row
#pragma unroll
        for (int it = 0; it < 64 * CPRW / 64; ++it) {
            const int c = it * 64 + lane;
            const int row = c / CPRW, col = c - row * CPRW;
            const int m = m0 + 64 * wm + row;
            u32x4 o = *(const u32x4*)(ep + row * EP_STRIDE + col * 16);
            if (m < M) {
                const int64_t off = (int64_t)m * N + nw + 8 * col;
                if (residual) {
                    float a[8], rsd[8];
                    unpack8<T>(o, a);
                    unpack8<T>(*(const u32x4*)(residual + off), rsd);
                    o = (u32x4){pack2<T>(a[0] + rsd[0], a[1] + rsd[1]), pack2<T>(a[2] + rsd[2], a[3] + rsd[3]),
                                pack2<T>(a[4] + rsd[4], a[5] + rsd[5]), pack2<T>(a[6] + rsd[6], a[7] + rsd[7])};
                }
                *(u32x4*)(y + off) = o;
            }
        }
        return;
    }
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
        const int m = m0 + 64 * wm + 32 * mb + rho;
        if (m >= M) continue;
#pragma unroll
        for (int nb = 0; nb < 3; ++nb)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = nw + 32 * nb + 8 * q + 4 * h;
                if (n >= N) continue;
                const i32x4 a = {acc[nb][mb][4 * q], acc[nb][mb][4 * q + 1], acc[nb][mb][4 * q + 2],
                                 acc[nb][mb][4 * q + 3]};
                if (partial) {
                    int32_t* p = partial + ((int64_t)blockIdx.y * M + m) * N + n;
                    if (n + 3 < N && (N & 3) == 0) {
                        *(i32x4*)p = a;
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            if (n + i < N) p[i] = a[i];
                    }
                } else {
                    q2_store4<T>(y, acc_out, x_scale, w_scale, bias, residual, m, n, N, a);
                }
            }
    }
}

template <typename T, int WM, int MT, int NT>
__global__ __launch_bounds__(256) void w8a8_regs_kernel(
    uint16_t* __restrict__ y, int32_t* __restrict__ acc_out, int32_t* __restrict__ partial,
    const int8_t* __restrict__ xq, const float* __restrict__ x_scale, const uint8_t* __restrict__ wp,
    const float* __restrict__ w_scale, const uint16_t* __restrict__ bias, const uint16_t* __restrict__ residual, int M,
    int N, int K, int steps_per_split) {
    constexpr int WN = 4 / WM;
    constexpr int BM = 16 * MT * WM, BN = 16 * NT * WN;
    constexpr int D = QR_DEPTH;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    const int wm = wv % WM, wn = wv / WM;
    const int KS = (K + Q_KSTEP - 1) / Q_KSTEP;
    const int s_begin = blockIdx.y * steps_per_split;
    const int s_end = min(KS, s_begin + steps_per_split);
    const int s_last = s_end - 1;
    const int m_tiles_total = (M + 15) >> 4, n_tiles_total = (N + 15) >> 4;
    const int mt0 = blockIdx.z * (BM / 16) + wm * MT;         // first row tile of this wave
    const int nt0 = blockIdx.x * (BN / 16) + wn * NT;         // first channel tile of this wave

    // tile (t, step s) of either operand sits at (s * tiles_total + t) * 1024 + lane * 16: a scalar base per step
    // plus a per-lane 32-bit offset that never changes.  Tiles past the matrix are clamped to the last one (their
    // results are never stored).
    uint32_t xoff[MT], woff[NT];
#pragma unroll
    for (int i = 0; i < MT; ++i) xoff[i] = (uint32_t)min(mt0 + i, m_tiles_total - 1) * Q_TILE + lane * 16;
#pragma unroll
    for (int j = 0; j < NT; ++j) woff[j] = (uint32_t)min(nt0 + j, n_tiles_total - 1) * Q_TILE + lane * 16;
    const int64_t xstep = (int64_t)m_tiles_total * Q_TILE, wstep = (int64_t)n_tiles_total * Q_TILE;

    i32x4 acc[NT][MT];
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int i = 0; i < MT; ++i) acc[j][i] = (i32x4){0, 0, 0, 0};

    // The loads and the wait that makes a slot's registers valid are asm statements: the compiler's own counting
    // gives up at the loop back-edge and waits for everything there, which would leave one step in flight, not three.
    i32x4 xr[D][MT], wr[D][NT];
    auto load = [&](int slot, int s) {                        // slot is a compile-time constant at every call
        const int sc = min(s, s_last);                        // past the end: re-read the last step, never used
        const uint8_t* wb = wp + sc * wstep;
        const uint8_t* xb = (const uint8_t*)xq + sc * xstep;
#pragma unroll
        for (int j = 0; j < NT; ++j)
            asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(wr[slot][j]) : "v"(woff[j]), "s"(wb) : "memory");
#pragma unroll
        for (int i = 0; i < MT; ++i)
            asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(xr[slot][i]) : "v"(xoff[i]), "s"(xb) : "memory");
    };
    // loads complete in issue order: once at most (D-1) steps' worth are outstanding, this slot's have arrived
    constexpr int PENDING = (D - 1) * (MT + NT);
    static_assert(PENDING < 64 && (MT == 4 || MT == 8) && (NT == 4 || NT == 5), "the wait below is written for these");
    auto arrived = [&](int slot) {
        i32x4* w = wr[slot];
        i32x4* x = xr[slot];
        if constexpr (NT == 4)
            asm volatile("s_waitcnt vmcnt(%4)" : "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3]) : "n"(PENDING) : "memory");
        else
            asm volatile("s_waitcnt vmcnt(%5)"
                         : "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3]), "+v"(w[4])
                         : "n"(PENDING)
                         : "memory");
        asm volatile("" : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3])::"memory");
        if constexpr (MT == 8) asm volatile("" : "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7])::"memory");
    };
#pragma unroll
    for (int d = 0; d < D; ++d) load(d, s_begin + d);
    auto step = [&](int slot, int s) {
        arrived(slot);
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int i = 0; i < MT; ++i)
                acc[j][i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wr[slot][j], xr[slot][i], acc[j][i], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);                    // the reload must not overtake the slot's last use
        load(slot, s + D);
    };
    for (int s = s_begin; s < s_end; s += D) {
#pragma unroll
        for (int slot = 0; slot < D; ++slot)
            if (s + slot < s_end) step(slot, s + slot);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");         // the reloads of the last steps still target registers

    // epilogue: lane (r, g) holds row m = 16*tile + r, channels 4g .. 4g+3 of each tile
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int m = 16 * (mt0 + i) + r;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const int n = 16 * (nt0 + j) + 4 * g;
            if (n >= N) continue;
            if (partial) {
                int32_t* p = partial + ((int64_t)blockIdx.y * M + m) * N + n;
                if (n + 3 < N && (N & 3) == 0) {
                    *(i32x4*)p = acc[j][i];
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < N) p[e] = acc[j][i][e];
                }
            } else {
                q2_store4<T>(y, acc_out, x_scale, w_scale, bias, residual, m, n, N, acc[j][i]);
            }
        }
    }
}

template <typename T>
__global__ void w8a8_splitk_reduce_kernel(uint16_t* __restrict__ y, int32_t* __restrict__ acc_out,
                                          const int32_t* __restrict__ partial, const float* __restrict__ x_scale,
                                          const float* __restrict__ w_scale, const uint16_t* __restrict__ bias,
                                          const uint16_t* __restrict__ residual, int M, int N, int split_k) {
    const int n4cnt = (N + 3) / 4;
    const int64_t total = (int64_t)M * n4cnt;
    const int64_t stride = (int64_t)M * N;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int m = (int)(idx / n4cnt);
        const int n = (int)(idx - (int64_t)m * n4cnt) * 4;
        const int32_t* p = partial + (int64_t)m * N + n;
        i32x4 sum = {0, 0, 0, 0};
        if (n + 3 < N && (N & 3) == 0) {
            for (int s = 0; s < split_k; ++s) sum += *(const i32x4*)(p + s * stride);
        } else {
            for (int s = 0; s < split_k; ++s)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < N) sum[i] += p[s * stride + i];
        }
        q2_store4<T>(y, acc_out, x_scale, w_scale, bias, residual, m, n, N, sum);
    }
}

// Split-K reduce of a fused QKV projection together with the rotate-half RoPE on q and k and the scatter of the
// rotated k and of v into the paged caches.  One work item = 8 consecutive elements of the first half of a q/k head
// with their partners in the second half, or 8 elements of v; grid = (tokens, ceil(items / 64)).  q is written
// (rotated) into its columns of qkv, the k and v columns are not written.  Values and rounding are those of
// w8a8_splitk_reduce_kernel followed by the rope-and-cache kernel.
template <typename T>
__device__ __forceinline__ void q_reduce8(const int32_t* __restrict__ p, int64_t stride, int split_k, float xs,
                                          const float* __restrict__ w_scale, const uint16_t* __restrict__ bias, int n,
                                          float* out) {
    i32x4 lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
    for (int s0 = 0; s0 < split_k; s0 += 4) {                 // four splits' loads in flight together
        i32x4 a[4], b[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
            if (s0 + q < split_k) {
                a[q] = *(const i32x4*)(p + (s0 + q) * stride);
                b[q] = *(const i32x4*)(p + (s0 + q) * stride + 4);
            }
#pragma unroll
        for (int q = 0; q < 4; ++q)
            if (s0 + q < split_k) {
                lo += a[q];
                hi += b[q];
            }
    }
    const f32x4 w_lo = *(const f32x4*)(w_scale + n), w_hi = *(const f32x4*)(w_scale + n + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float a = (float)lo[i] * xs * w_lo[i], b = (float)hi[i] * xs * w_hi[i];
        if (bias) {
            a += T::to_float(bias[n + i]);
            b += T::to_float(bias[n + 4 + i]);
        }
        out[i] = T::to_float(T::from_float(a));
        out[4 + i] = T::to_float(T::from_float(b));
    }
}

constexpr int QRC_THREADS = 64;

template <typename T>
__global__ __launch_bounds__(QRC_THREADS) void w8a8_reduce_rope_cache_kernel(
    uint16_t* __restrict__ qkv, const int32_t* __restrict__ partial, const float* __restrict__ x_scale,
    const float* __restrict__ w_scale, const uint16_t* __restrict__ bias, const void* __restrict__ cos,
    const void* __restrict__ sin, uint16_t* __restrict__ key_cache, uint16_t* __restrict__ value_cache,
    const int32_t* __restrict__ slot_mapping, int M, int N, int split_k, int n_heads, int n_kv, int D,
    int64_t num_slots, int table_dtype) {
    const int t = blockIdx.x;
    const int half = D >> 1;
    const int cph = half >> 3;
    const int rot_items = (n_heads + n_kv) * cph;
    const int v_items = n_kv * D / 8;
    const int item = blockIdx.y * QRC_THREADS + threadIdx.x;
    if (item >= rot_items + v_items) return;
    const int64_t slot = slot_mapping[t];
    const float xs = x_scale[t];
    const int64_t row = (int64_t)n_kv * D;
    const int64_t stride = (int64_t)M * N;
    const int32_t* prow = partial + (int64_t)t * N;
    if (item >= rot_items) {
        const int i = (item - rot_items) * 8;
        const int col = (n_heads + n_kv) * D + i;
        float v[8];
        q_reduce8<T>(prow + col, stride, split_k, xs, w_scale, bias, col, v);
        u32x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = pack2<T>(v[2 * e], v[2 * e + 1]);
        if (slot >= 0 && slot < num_slots) *(u32x4*)(value_cache + slot * row + i) = o;
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
    q_reduce8<T>(prow + col, stride, split_k, xs, w_scale, bias, col, x1);
    q_reduce8<T>(prow + col + half, stride, split_k, xs, w_scale, bias, col + half, x2);
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
            uint16_t* dst = key_cache + slot * row + (h - n_heads) * D;
            *(u32x4*)(dst + i) = o1;
            *(u32x4*)(dst + i + half) = o2;
        }
    } else {
        uint16_t* dst = qkv + (int64_t)t * N + col;
        *(u32x4*)dst = o1;
        *(u32x4*)(dst + half) = o2;
    }
}

// ---- grouped (experts): rows offsets[e] .. offsets[e+1] of the quantised activations use expert e's weights --------
// grid = (ceil(N / 64), n_experts); a workgroup of 4 waves owns 64 output channels of one expert for all of its
// rows.  Decode batches route a handful of tokens to each expert, so the kernel is a weight stream: the waves
// interleave the 64-wide k-steps, each loads its four 1 KiB weight tiles of a step straight into operand registers
// (two steps ahead) and the 16 bytes per lane of each 16-row activation tile from the row-major int8 rows (a few KiB
// per expert, served by L2), and the four waves' exact int32 sums meet in LDS at the end.  Up to 64 rows go through
// one pass over the weights (16 / 32 / 64 by the expert's row count, as in the W8A16 grouped kernel); experts with
// more rows repeat the pass.  Two builds of the kernel: passes of up to 32 rows (138 registers, three workgroups per
// compute unit: the decode-sized case, a pure weight stream) and of up to 64 rows (197 registers, two per compute unit),
// which the launch picks when the groups average more than 16 rows.
constexpr int QG_WAVES = 4;
constexpr int QG_NT = 4;                                      // 16-channel weight tiles per wave and step
constexpr int QG_BN = 16 * QG_NT;
template <int MTMAX>
constexpr int QG_SMEM = QG_WAVES * 16 * MTMAX * QG_BN * 4;    // MTMAX 16-row activation tiles per pass

template <typename T, int MT>
__device__ __forceinline__ void w8a8_group_pass(uint16_t* __restrict__ y, int32_t* __restrict__ acc_out,
                                                const int8_t* __restrict__ x, const float* __restrict__ xs,
                                                const uint8_t* __restrict__ wp, const float* __restrict__ ws, int rows,
                                                int N, int K, int n0, int m0, int32_t* red) {
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    const int KS = (K + Q_KSTEP - 1) / Q_KSTEP;
    const int n_tiles_total = (N + 15) >> 4;
    // operands: every load reads an address that exists (tiles past N, rows past the group and k past K are
    // clamped; what they contribute is never stored, or meets the zero padding of the packed weights)
    uint32_t woff[QG_NT];
#pragma unroll
    for (int j = 0; j < QG_NT; ++j) woff[j] = (uint32_t)min((n0 >> 4) + j, n_tiles_total - 1) * Q_TILE + lane * 16;
    const int8_t* xrow[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) xrow[i] = x + (int64_t)min(m0 + 16 * i + r, rows - 1) * K;
    const int64_t wstep = (int64_t)n_tiles_total * Q_TILE;
    const int k_last = K - 16;                                // byte offset of the last whole 16-byte chunk of a row

    i32x4 acc[QG_NT][MT];
#pragma unroll
    for (int j = 0; j < QG_NT; ++j)
#pragma unroll
        for (int i = 0; i < MT; ++i) acc[j][i] = (i32x4){0, 0, 0, 0};

    constexpr int D = 2;                                      // steps in flight beyond the current one
    i32x4 wr[D + 1][QG_NT], xr[D + 1][MT];
    auto load = [&](int slot, int s) {
        const int sc = min(s, KS - 1);
        const uint8_t* wb = wp + sc * wstep;
        const int kb = min(sc * Q_KSTEP + 16 * g, k_last);    // chunks past K meet zero weights
#pragma unroll
        for (int j = 0; j < QG_NT; ++j) wr[slot][j] = *(const i32x4*)(wb + woff[j]);
#pragma unroll
        for (int i = 0; i < MT; ++i) xr[slot][i] = *(const i32x4*)(xrow[i] + kb);
    };
    const int first = wv;
#pragma unroll
    for (int d = 0; d <= D; ++d) load(d, first + d * QG_WAVES);
    auto step = [&](int slot, int s) {
#pragma unroll
        for (int j = 0; j < QG_NT; ++j)
#pragma unroll
            for (int i = 0; i < MT; ++i)
                acc[j][i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wr[slot][j], xr[slot][i], acc[j][i], 0, 0, 0);
        load(slot, s + (D + 1) * QG_WAVES);
    };
    for (int s = first; s < KS; s += (D + 1) * QG_WAVES) {
#pragma unroll
        for (int slot = 0; slot <= D; ++slot)
            if (s + slot * QG_WAVES < KS) step(slot, s + slot * QG_WAVES);
    }

    // sum of the four waves through LDS: red[wave][row][channel], 16-byte granules XOR-swizzled by the row
    constexpr int XROWS = 16 * MT;
    __syncthreads();                                          // the previous pass has been read out
#pragma unroll
    for (int j = 0; j < QG_NT; ++j)
#pragma unroll
        for (int i = 0; i < MT; ++i)
            *(i32x4*)(red + ((wv * XROWS + 16 * i + r) * QG_BN) + (((4 * j + g) ^ r) << 2)) = acc[j][i];
    __syncthreads();
    constexpr int N4 = QG_BN / 4;
    for (int idx = threadIdx.x; idx < XROWS * N4; idx += QG_WAVES * 64) {
        const int ml = idx / N4, n4 = idx - ml * N4;
        const int m = m0 + ml, n = n0 + 4 * n4;
        if (m >= rows || n >= N) continue;
        const int sw = (n4 ^ (ml & 15)) << 2;
        i32x4 sum = *(const i32x4*)(red + ml * QG_BN + sw);
#pragma unroll
        for (int q = 1; q < QG_WAVES; ++q) sum += *(const i32x4*)(red + (q * XROWS + ml) * QG_BN + sw);
        q2_store4<T>(y, acc_out, xs, ws, nullptr, nullptr, m, n, N, sum);
    }
}

template <typename T, int MTMAX>
__global__ __launch_bounds__(QG_WAVES * 64, 2) void w8a8_grouped_kernel(
    uint16_t* __restrict__ y, int32_t* __restrict__ acc_out, const int8_t* __restrict__ xq,
    const float* __restrict__ x_scale, const uint8_t* __restrict__ wp, const float* __restrict__ w_scale,
    const int32_t* __restrict__ offsets, int total_rows, int N, int K, int64_t expert_bytes) {
    __shared__ __attribute__((aligned(16))) int32_t red[QG_SMEM<MTMAX> / 4];
    const int e = blockIdx.y;
    int row0 = offsets[e], row1 = offsets[e + 1];
    row0 = max(0, min(row0, total_rows));
    row1 = max(row0, min(row1, total_rows));
    const int rows = row1 - row0;
    if (rows == 0) return;
    const uint8_t* we = wp + (int64_t)e * expert_bytes;
    const float* se = w_scale + (int64_t)e * N;
    uint16_t* ye = y ? y + (int64_t)row0 * N : nullptr;
    int32_t* ae = acc_out ? acc_out + (int64_t)row0 * N : nullptr;
    const int8_t* xe = xq + (int64_t)row0 * K;
    const float* xse = x_scale + row0;
    const int n0 = blockIdx.x * QG_BN;
    if (rows <= 16) {
        w8a8_group_pass<T, 1>(ye, ae, xe, xse, we, se, rows, N, K, n0, 0, red);
    } else if (rows <= 32 || MTMAX == 2) {
        for (int m0 = 0; m0 < rows; m0 += 32)
            w8a8_group_pass<T, 2>(ye, ae, xe, xse, we, se, rows, N, K, n0, m0, red);
    } else {
        for (int m0 = 0; m0 < rows; m0 += 16 * MTMAX)
            w8a8_group_pass<T, MTMAX>(ye, ae, xe, xse, we, se, rows, N, K, n0, m0, red);
    }
}

// What may follow the GEMM in the same call, fused with the split-K reduce where K is split.
struct QNormQuantArgs {           // residual add (through `residual`) + RMSNorm + per-token quantisation
    int8_t* xq_out;
    float* x_scale_out;
    const void* gamma;
    const float* smooth;
    float eps;
    int gamma_dtype, out_layout;
};
struct QRopeCacheArgs {           // RoPE on q and k + cache scatter of k and v
    const void *cos, *sin;
    void *key_cache, *value_cache;
    const int32_t* slot_mapping;
    int n_heads, n_kv, head_dim, table_dtype;
    int64_t num_slots;
};

struct QPlan {
    int regs;        // 0: LDS-staged kernel; 1: register-streaming kernel, 4x1 waves of 64 x 64
    bool msplit;
    bool wide;       // w8a8_wide_kernel: 8 waves, 256 x 192 tiles
    int nt;
    int n_blocks, m_blocks, split_k, steps_per_split;
};

QPlan plan_w8a8(int m, int n, int k, bool x_tiled) {
    QPlan p;
    p.msplit = m > 64;
    p.wide = false;
    p.regs = 0;
    const int steps = (k + Q_KSTEP - 1) / Q_KSTEP;
    if (x_tiled && m > 64 && n < 8192) {
        // narrow outputs: the register-streaming kernel on 256 x 64 tiles (measured faster than the LDS-staged one
        // there; on wide outputs it re-fetches the activation tiles too often and the LDS-staged kernel wins)
        p.regs = 1;
        p.nt = 4;                                             // channel tiles per workgroup
        p.m_blocks = (m + 255) / 256;
    } else if (p.msplit) {
        // 80-channel tiles, two workgroups per CU: close to 512 tiles balance best; wide N only
        p.nt = n >= 16384 ? 5 : 4;
        // very wide outputs: 256 x 192 tiles on 8 waves, one workgroup per CU (one staged activation tile serves
        // more channels, and the 32 x 32 x 32 instruction runs at twice the rate of the 16 x 16 x 64 one)
        p.wide = x_tiled && n >= 16384 && m > 128;
        p.m_blocks = (m + 255) / 256;
    } else {
        p.nt = 2;
        p.m_blocks = 1;
    }
    const int bn = p.wide ? QW::BN : 16 * p.nt * (p.regs || p.msplit ? 1 : 4);
    p.n_blocks = (n + bn - 1) / bn;
    // split K only as far as needed to give every CU a workgroup, and keep at least 16 steps per split: every
    // split writes (and the reduce kernel reads back) an int32 copy of the output
    const int tiles = p.n_blocks * p.m_blocks;
    // (the 8-wave tiles hold a whole CU each: from half the CUs up, splitting K would only add partial traffic)
    int sk = tiles >= (p.wide ? 128 : 200) ? 1 : (224 + tiles - 1) / tiles;
    const int max_sk = steps / 16 < 1 ? 1 : steps / 16;
    sk = sk > max_sk ? max_sk : sk;
    sk = sk > 32 ? 32 : sk;
    p.steps_per_split = (steps + sk - 1) / sk;
    p.split_k = (steps + p.steps_per_split - 1) / p.steps_per_split;
    return p;
}

template <typename T>
int launch_w8a8(void* y, int32_t* acc_out, const int8_t* xq, const float* x_scale, const uint8_t* wp,
                const float* w_scale, const void* bias, const void* residual, int m, int n, int k, bool x_tiled,
                void* workspace, hipStream_t st, const QNormQuantArgs* nq = nullptr,
                const QRopeCacheArgs* rc = nullptr) {
    const QPlan p = plan_w8a8(m, n, k, x_tiled);
    int32_t* partial = p.split_k > 1 ? (int32_t*)workspace : nullptr;
    dim3 grid(p.n_blocks, p.split_k, p.m_blocks);
    const bool ktail = (k % Q_KSTEP) != 0;
#define Q_LAUNCH(NTV, MS, STV, KT, XTV)                                                                                \
    do {                                                                                                         \
        auto kern = w8a8_gemm_kernel<T, NTV, MS, STV, KT, XTV>;                                                        \
        constexpr int lds = Q2<NTV, MS, STV>::LDS_BYTES;                                                          \
        static bool configured[MF_MAX_DEVICES] = {};                                                              \
        int dev = 0;                                                                                             \
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MF_MAX_DEVICES)                                \
            return (int)hipErrorInvalidDevice;                                                                   \
        if (!configured[dev]) {                                                                                  \
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds); \
            if (e != hipSuccess) return (int)e;                                                                  \
            configured[dev] = true;                                                                              \
        }                                                                                                        \
        hipLaunchKernelGGL(kern, grid, dim3(Q2<NTV, MS, STV>::WAVES * 64), lds, st, (uint16_t*)y, acc_out, partial, xq,  \
                           x_scale, wp, w_scale,                                                                  \
                           (const uint16_t*)bias, (const uint16_t*)residual, m, n, k, p.steps_per_split);         \
    } while (0)
#define Q_LAUNCH_KT(NTV, MS, STV)                                                                                 \
    do {                                                                                                         \
        if (x_tiled) Q_LAUNCH(NTV, MS, STV, false, true);                                                        \
        else if (ktail) Q_LAUNCH(NTV, MS, STV, true, false);                                                     \
        else Q_LAUNCH(NTV, MS, STV, false, false);                                                               \
    } while (0)
#define QR_LAUNCH(WMV, MTV, NTV)                                                                                  \
    hipLaunchKernelGGL((w8a8_regs_kernel<T, WMV, MTV, NTV>), grid, dim3(256), 0, st, (uint16_t*)y, acc_out, partial, \
                       xq, x_scale, wp, w_scale, (const uint16_t*)bias, (const uint16_t*)residual, m, n, k,          \
                       p.steps_per_split)
    if (p.regs == 1) QR_LAUNCH(4, 4, 4);
    else if (!p.msplit) Q_LAUNCH_KT(2, 0, 4);
    else if (p.wide) {
        static bool configured[MF_MAX_DEVICES] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MF_MAX_DEVICES) return (int)hipErrorInvalidDevice;
        if (!configured[dev]) {
            hipError_t e = hipFuncSetAttribute((const void*)w8a8_wide_kernel<T>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, QW::LDS_BYTES);
            if (e != hipSuccess) return (int)e;
            configured[dev] = true;
        }
        hipLaunchKernelGGL(w8a8_wide_kernel<T>, grid, dim3(QW::WAVES * 64), QW::LDS_BYTES, st, (uint16_t*)y, acc_out,
                           partial, xq, x_scale, wp, w_scale, (const uint16_t*)bias, (const uint16_t*)residual, m, n, k,
                           p.steps_per_split);
    }
    else if (p.nt == 5) Q_LAUNCH_KT(5, 1, 3);
    else Q_LAUNCH_KT(4, 1, 3);
#undef QR_LAUNCH
#undef Q_LAUNCH_KT
#undef Q_LAUNCH
    int err = MF_LAUNCH_CHECK();
    if (err) return err;
    if (nq) {
        if (partial)                                          // sum of the splits + residual + norm + quantisation
            return mf_detail_rmsnorm_quant_from_partial(nq->xq_out, nq->x_scale_out, y, partial, p.split_k, x_scale,
                                                        w_scale, bias, residual, nq->gamma, nq->smooth, nq->eps, m, n,
                                                        T::id, nq->gamma_dtype, nq->out_layout, st);
        return mf_rmsnorm_dynamic_quant(nq->xq_out, nq->x_scale_out, nullptr, y, nullptr, nq->gamma, nq->smooth, nq->eps,
                                        m, n, T::id, nq->gamma_dtype, nq->out_layout, st);   // the GEMM wrote h
    }
    if (rc && partial) {
        const int items = (rc->n_heads + rc->n_kv) * (rc->head_dim / 16) + rc->n_kv * rc->head_dim / 8;
        hipLaunchKernelGGL((w8a8_reduce_rope_cache_kernel<T>), dim3(m, (items + QRC_THREADS - 1) / QRC_THREADS),
                           dim3(QRC_THREADS), 0, st, (uint16_t*)y, partial, x_scale, w_scale, (const uint16_t*)bias,
                           rc->cos, rc->sin, (uint16_t*)rc->key_cache, (uint16_t*)rc->value_cache, rc->slot_mapping, m, n,
                           p.split_k, rc->n_heads, rc->n_kv, rc->head_dim, rc->num_slots, rc->table_dtype);
        return MF_LAUNCH_CHECK();
    }
    if (rc) {                                                 // no split: the GEMM wrote qkv; rotate and scatter
        uint16_t* q = (uint16_t*)y;
        return mf_rope_and_cache(q, q + (int64_t)rc->n_heads * rc->head_dim,
                                 q + (int64_t)(rc->n_heads + rc->n_kv) * rc->head_dim, rc->cos, rc->sin, rc->key_cache,
                                 rc->value_cache, rc->slot_mapping, m, rc->n_heads, rc->n_kv, rc->head_dim, rc->num_slots,
                                 n, n, n, T::id, rc->table_dtype, st);
    }
    if (!partial) return 0;
    const int64_t total = (int64_t)m * ((n + 3) / 4);
    const int blocks = (int)((total + 255) / 256 > 4096 ? 4096 : (total + 255) / 256);
    hipLaunchKernelGGL((w8a8_splitk_reduce_kernel<T>), dim3(blocks), dim3(256), 0, st, (uint16_t*)y, acc_out, partial,
                       x_scale, w_scale, (const uint16_t*)bias, (const uint16_t*)residual, m, n, p.split_k);
    return MF_LAUNCH_CHECK();
}

}  // namespace

extern "C" size_t mf_w8a8_workspace_bytes(int m, int n, int k) {
    if (m <= 0 || n <= 0 || k <= 0) return 0;
    size_t need = 0;                                          // enough for either activation layout
    for (int tiled = 0; tiled < 2; ++tiled) {
        const QPlan p = plan_w8a8(m, n, k, tiled != 0);
        const size_t b = p.split_k > 1 ? (size_t)p.split_k * m * n * sizeof(int32_t) : 0;
        need = b > need ? b : need;
    }
    return need;
}

extern "C" int mf_w8a8_gemm(void* y, int32_t* acc_out, const int8_t* xq, const float* x_scale, const void* w_packed,
                            const float* w_scale, const void* bias, const void* residual, int m, int n, int k,
                            int dtype, int x_layout, void* workspace, size_t workspace_bytes, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "w8a8_gemm: dtype must be bf16 or fp16");
    if (m == 0) return 0;
    MF_REQUIRE(xq && w_packed && (y || acc_out), "w8a8_gemm: null argument");
    MF_REQUIRE(x_layout == 0 || x_layout == 1, "w8a8_gemm: x_layout must be 0 (row-major) or 1 (tiled)");
    MF_REQUIRE(!y || (x_scale && w_scale), "w8a8_gemm: scales required for a dequantised output");
    MF_REQUIRE(m >= 0 && n > 0 && k > 0 && k % 16 == 0, "w8a8_gemm: bad sizes m=%d n=%d k=%d (K %% 16 == 0)", m, n, k);
    MF_REQUIRE((((uintptr_t)xq | (uintptr_t)w_packed) & 15) == 0, "w8a8_gemm: xq and w_packed must be 16-byte aligned");
    const size_t need = mf_w8a8_workspace_bytes(m, n, k);
    MF_REQUIRE(need == 0 || (workspace && workspace_bytes >= need && ((uintptr_t)workspace & 15) == 0),
               "w8a8_gemm: 16-byte aligned workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    if (dtype == MF_BF16)
        return launch_w8a8<BF16>(y, acc_out, xq, x_scale, (const uint8_t*)w_packed, w_scale, bias, residual, m, n, k,
                                 x_layout == 1, workspace, (hipStream_t)stream);
    return launch_w8a8<FP16>(y, acc_out, xq, x_scale, (const uint8_t*)w_packed, w_scale, bias, residual, m, n, k,
                             x_layout == 1, workspace, (hipStream_t)stream);
}

extern "C" int mf_w8a8_gemm_add_rmsnorm_quant(int8_t* xq_out, float* x_scale_out, void* h_out, const int8_t* xq,
                                              const float* x_scale, const void* w_packed, const float* w_scale,
                                              const void* bias, const void* residual, const void* gamma,
                                              const float* smooth, float eps, int m, int n, int k, int dtype,
                                              int gamma_dtype, int x_layout, int out_layout, void* workspace,
                                              size_t workspace_bytes, void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "w8a8_gemm_add_rmsnorm_quant: dtype must be bf16 or fp16");
    MF_REQUIRE(gamma_dtype == MF_BF16 || gamma_dtype == MF_FP16 || gamma_dtype == MF_FP32,
               "w8a8_gemm_add_rmsnorm_quant: bad gamma dtype");
    MF_REQUIRE((x_layout == 0 || x_layout == 1) && (out_layout == 0 || out_layout == 1),
               "w8a8_gemm_add_rmsnorm_quant: layouts must be 0 (row-major) or 1 (tiled)");
    if (m == 0) return 0;
    MF_REQUIRE(xq_out && x_scale_out && h_out && xq && x_scale && w_packed && w_scale && gamma,
               "w8a8_gemm_add_rmsnorm_quant: null argument");
    MF_REQUIRE(m >= 0 && n > 0 && k > 0 && k % 16 == 0, "w8a8_gemm_add_rmsnorm_quant: bad sizes m=%d n=%d k=%d (K %% 16 == 0)",
               m, n, k);
    MF_REQUIRE(n % 8 == 0 && n <= 16384, "w8a8_gemm_add_rmsnorm_quant: N (%d) must be a multiple of 8, at most 16384", n);
    MF_REQUIRE((((uintptr_t)xq | (uintptr_t)w_packed | (uintptr_t)h_out | (uintptr_t)residual | (uintptr_t)gamma |
                 (uintptr_t)smooth | (uintptr_t)bias | (uintptr_t)w_scale) & 15) == 0 && ((uintptr_t)xq_out & 7) == 0,
               "w8a8_gemm_add_rmsnorm_quant: pointers must be 16-byte aligned, xq_out 8-byte aligned");
    const size_t need = mf_w8a8_workspace_bytes(m, n, k);
    MF_REQUIRE(need == 0 || (workspace && workspace_bytes >= need && ((uintptr_t)workspace & 15) == 0),
               "w8a8_gemm_add_rmsnorm_quant: 16-byte aligned workspace of %zu bytes needed, %zu given", need,
               workspace_bytes);
    const QNormQuantArgs nq = {xq_out, x_scale_out, gamma, smooth, eps, gamma_dtype, out_layout};
    if (dtype == MF_BF16)
        return launch_w8a8<BF16>(h_out, nullptr, xq, x_scale, (const uint8_t*)w_packed, w_scale, bias, residual, m, n, k,
                                 x_layout == 1, workspace, (hipStream_t)stream, &nq);
    return launch_w8a8<FP16>(h_out, nullptr, xq, x_scale, (const uint8_t*)w_packed, w_scale, bias, residual, m, n, k,
                             x_layout == 1, workspace, (hipStream_t)stream, &nq);
}

extern "C" int mf_w8a8_qkv_rope_and_cache(void* qkv, const int8_t* xq, const float* x_scale, const void* w_packed,
                                          const float* w_scale, const void* bias, const void* cos, const void* sin,
                                          void* key_cache, void* value_cache, const int32_t* slot_mapping, int m,
                                          int n_heads, int n_kv_heads, int head_dim, int64_t num_slots, int k, int dtype,
                                          int table_dtype, int x_layout, void* workspace, size_t workspace_bytes,
                                          void* stream) {
    MF_REQUIRE(dtype == MF_BF16 || dtype == MF_FP16, "w8a8_qkv_rope_and_cache: dtype must be bf16 or fp16");
    MF_REQUIRE(table_dtype == MF_BF16 || table_dtype == MF_FP16 || table_dtype == MF_FP32,
               "w8a8_qkv_rope_and_cache: bad cos/sin dtype");
    MF_REQUIRE(x_layout == 0 || x_layout == 1, "w8a8_qkv_rope_and_cache: x_layout must be 0 (row-major) or 1 (tiled)");
    if (m == 0) return 0;
    MF_REQUIRE(qkv && xq && x_scale && w_packed && w_scale && cos && sin && key_cache && value_cache && slot_mapping,
               "w8a8_qkv_rope_and_cache: null argument");
    MF_REQUIRE(m >= 0 && n_heads > 0 && n_kv_heads > 0 && k > 0 && k % 16 == 0 && num_slots > 0,
               "w8a8_qkv_rope_and_cache: bad sizes m=%d heads=%d/%d k=%d slots=%lld", m, n_heads, n_kv_heads, k,
               (long long)num_slots);
    MF_REQUIRE(head_dim > 0 && head_dim % 16 == 0, "w8a8_qkv_rope_and_cache: head_dim (%d) must be a multiple of 16",
               head_dim);
    const int n = (n_heads + 2 * n_kv_heads) * head_dim;
    MF_REQUIRE((((uintptr_t)xq | (uintptr_t)w_packed | (uintptr_t)qkv | (uintptr_t)cos | (uintptr_t)sin |
                 (uintptr_t)key_cache | (uintptr_t)value_cache | (uintptr_t)bias | (uintptr_t)w_scale) & 15) == 0,
               "w8a8_qkv_rope_and_cache: pointers must be 16-byte aligned");
    const size_t need = mf_w8a8_workspace_bytes(m, n, k);
    MF_REQUIRE(need == 0 || (workspace && workspace_bytes >= need && ((uintptr_t)workspace & 15) == 0),
               "w8a8_qkv_rope_and_cache: 16-byte aligned workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    const QRopeCacheArgs rc = {cos, sin, key_cache, value_cache, slot_mapping, n_heads, n_kv_heads, head_dim, table_dtype,
                               num_slots};
    if (dtype == MF_BF16)
        return launch_w8a8<BF16>(qkv, nullptr, xq, x_scale, (const uint8_t*)w_packed, w_scale, bias, nullptr, m, n, k,
                                 x_layout == 1, workspace, (hipStream_t)stream, nullptr, &rc);
    return launch_w8a8<FP16>(qkv, nullptr, xq, x_scale, (const uint8_t*)w_packed, w_scale, bias, nullptr, m, n, k,
                             x_layout == 1, workspace, (hipStream_t)stream, nullptr, &rc);
}

extern "C" int mf_grouped_w8a8_gemm(void* y, int32_t* acc_out, const int8_t* xq, const float* x_scale,
                                    const void* w_packed, const float* w_scale, const int32_t* offsets, int n_experts,
                                    int total_rows, int n, int k, int out_dtype, void* stream) {
    MF_REQUIRE(out_dtype == MF_BF16 || out_dtype == MF_FP16, "grouped_w8a8_gemm: out_dtype must be bf16 or fp16");
    if (total_rows == 0) return 0;
    MF_REQUIRE((y || acc_out) && xq && x_scale && w_packed && w_scale && offsets, "grouped_w8a8_gemm: null argument");
    MF_REQUIRE(n_experts > 0 && n_experts <= 65535 && total_rows >= 0 && n > 0 && k > 0, "grouped_w8a8_gemm: bad sizes");
    MF_REQUIRE(k % 16 == 0, "grouped_w8a8_gemm: K (%d) must be a multiple of 16", k);
    MF_REQUIRE((((uintptr_t)xq | (uintptr_t)w_packed) & 15) == 0,
               "grouped_w8a8_gemm: xq and w_packed must be 16-byte aligned");
    const int64_t expert_bytes = (int64_t)mf_w8a16_packed_bytes(n, k);
    dim3 grid((n + QG_BN - 1) / QG_BN, n_experts);
    // groups that average more than 16 rows (prefill-sized) take the 64-row passes; both builds serve any row count
    const bool big = (int64_t)total_rows > 16 * (int64_t)n_experts;
#define QG_LAUNCH(TT, MTV)                                                                                      \
    hipLaunchKernelGGL((w8a8_grouped_kernel<TT, MTV>), grid, dim3(QG_WAVES * 64), 0, (hipStream_t)stream,        \
                       (uint16_t*)y, acc_out, xq, x_scale, (const uint8_t*)w_packed, w_scale, offsets, total_rows, n, \
                       k, expert_bytes)
    if (out_dtype == MF_BF16) {
        if (big) QG_LAUNCH(BF16, 4);
        else QG_LAUNCH(BF16, 2);
    } else {
        if (big) QG_LAUNCH(FP16, 4);
        else QG_LAUNCH(FP16, 2);
    }
#undef QG_LAUNCH
    return MF_LAUNCH_CHECK();
}
