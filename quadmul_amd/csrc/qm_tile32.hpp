// Software-pipelined int4 GEMM tile kernel for compute-bound shapes (gfx950).
//
// Takes the place of the reference's igemm<Config> main loop (kernel.cu:186-260)
// for large tiles.  Differences in kind, not in degree:
//   * contraction by v_mfma_i32_32x32x32_i8 on nibbles widened to 16*s4 after the
//     LDS read (LDS holds the packed bytes, so LDS traffic is half of an int8 tile);
//     one 32x32x32 MFMA keeps the matrix pipe busy for 32 cycles but the issue port
//     only 8, which leaves room for the widening VALU work between MFMAs;
//   * a 3-deep LDS ring with one barrier per K-step: while tile t is contracted,
//     fragments of tile t+1 are already being read and tile t+2 is being written;
//   * fragment reads run two sub-steps ahead of their MFMAs and the widening one
//     sub-step ahead, interleaved with the MFMAs by scheduling-group hints.
#pragma once
#include "qm_common.hpp"

namespace qm {

typedef int v16i __attribute__((ext_vector_type(16)));

// D(32x32) += S0(32x32) * S1(32x32).  Lane l supplies row l%32 of S0 / column l%32
// of S1 for the 16 k-values of half l/32, and owns D[8*(r/4) + 4*(l/32) + r%4][l%32]
// in register r.
__device__ __forceinline__ v16i mfma32(const v4i s0, const v4i s1, const v16i acc)
{
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(s0, s1, acc, 0, 0, 0);
}

template <int BM_, int BN_, int WGM_, int WGN_>
struct Tile32Cfg {
    static constexpr int BM = BM_, BN = BN_, BK = 128, WGM = WGM_, WGN = WGN_;
    static constexpr int WAVES = WGM * WGN, THREADS = 64 * WAVES;
    static constexpr int WM = BM / WGM, WN = BN / WGN;
    static constexpr int FM = WM / 32, FN = WN / 32;  // 32x32 accumulator blocks per wave
    static constexpr int PITCH = 64;                  // packed bytes per row per K-step
    static constexpr int A_BYTES = BM * PITCH, B_BYTES = BN * PITCH;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int STAGES = 3;
    static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
    static constexpr int ROWS_PER_PASS = THREADS / 4;
    static constexpr int A_LOADS = BM / ROWS_PER_PASS, B_LOADS = BN / ROWS_PER_PASS;
    static constexpr int SUBSTEPS = 2 * FM;  // per K-step: two 64-nibble halves x FM A-fragments
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile is a multiple of 32x32");
    static_assert(BM % ROWS_PER_PASS == 0 && BN % ROWS_PER_PASS == 0, "loader must tile the block evenly");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU");
    static_assert(FM >= 2 && FN >= 1, "pipeline needs at least two A fragments per wave");
};

template <class Cfg>
__global__ void __launch_bounds__(Cfg::THREADS)
gemm_tile32_kernel(const GemmArgs p, const int tiles_m, const int tiles_n, const int group_m_in)
{
    const int group_m = group_m_in & 63;
    const bool dbg_same = group_m_in & 64;  // TEMP experiment: every workgroup loads tile (0,0)
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, FM = Cfg::FM, FN = Cfg::FN;
    constexpr int PITCH = Cfg::PITCH, STAGE = Cfg::STAGE_BYTES;
    constexpr int A_LOADS = Cfg::A_LOADS, B_LOADS = Cfg::B_LOADS, RPP = Cfg::ROWS_PER_PASS;

    extern __shared__ __align__(16) uint8_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / Cfg::WGN, wn = wave % Cfg::WGN;
    const int r32 = lane & 31, half = lane >> 5;

    const int pid = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int width = group_m * tiles_n;
    const int first_m = (pid / width) * group_m;
    const int gsz = min(tiles_m - first_m, group_m);
    const int m0 = (first_m + (pid % width) % gsz) * BM;
    const int n0 = ((pid % width) / gsz) * BN;

    const int Kb = p.K >> 1;
    const int KT = (p.K + BK - 1) / BK;

    // ---- global -> LDS staging: thread -> (row, 16-byte chunk), 4 chunks per row ----
    const int ld_ch = tid & 3, ld_row = tid >> 2;
    uint32_t a_off[A_LOADS], b_off[B_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i)
        a_off[i] = (uint32_t)min((dbg_same ? 0 : m0) + ld_row + i * RPP, p.M - 1) * (uint32_t)Kb + ld_ch * 16;
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i)
        b_off[i] = (uint32_t)min((dbg_same ? 0 : n0) + ld_row + i * RPP, p.N - 1) * (uint32_t)Kb + ld_ch * 16;
    // chunk swizzle: physical chunk = chunk ^ ((row >> 2) & 3) -- measured conflict-free
    // for 32-row x 2-chunk fragment reads at a 64-byte pitch; RPP is a multiple of 16
    // so the XOR term is the same for every pass of this thread
    const int st_off = ld_row * PITCH + ((ld_ch ^ ((ld_row >> 2) & 3)) << 4);

    v4i g_a[A_LOADS], g_b[B_LOADS];
    // K is a multiple of 128 here, so every chunk of every tile is whole; tiles past
    // the end are re-reads of the last one and never reach an MFMA.  No branch: the
    // K loop must stay one basic block for the scheduling hints to hold.
    auto load_global = [&](int kt) {
        const int kofs = min(kt, KT - 1) * (BK / 2);
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) g_a[i] = *reinterpret_cast<const v4i *>(p.A + a_off[i] + kofs);
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) g_b[i] = *reinterpret_cast<const v4i *>(p.B + b_off[i] + kofs);
    };
    auto store_lds = [&](int stage_byte) {
        uint8_t *As = smem + stage_byte + st_off;
        uint8_t *Bs = As + Cfg::A_BYTES;
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) *reinterpret_cast<v4i *>(As + i * RPP * PITCH) = g_a[i];
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) *reinterpret_cast<v4i *>(Bs + i * RPP * PITCH) = g_b[i];
    };
    // One staging piece (a 16-byte chunk per thread): write the copy of tile kt+2 held in
    // registers to LDS, then refill the same registers from tile kt+3.  Pieces are
    // spread over the sub-steps so that neither LDS writes nor loads come in bursts.
    auto restage_piece = [&](int piece, int stage_byte, int kt_next) {
        const int kofs = min(kt_next, KT - 1) * (BK / 2);
        if (piece < A_LOADS) {
            *reinterpret_cast<v4i *>(smem + stage_byte + st_off + piece * RPP * PITCH) = g_a[piece];
            g_a[piece] = *reinterpret_cast<const v4i *>(p.A + a_off[piece] + kofs);
        } else {
            const int b = piece - A_LOADS;
            *reinterpret_cast<v4i *>(smem + stage_byte + Cfg::A_BYTES + st_off + b * RPP * PITCH) = g_b[b];
            g_b[b] = *reinterpret_cast<const v4i *>(p.B + b_off[b] + kofs);
        }
    };

    // ---- fragment reads: lane -> row r32 of a 32-row fragment, chunk 2*q + half ----
    // (rows of consecutive fragments differ by 32, which leaves (row >> 2) & 3 unchanged)
    const int a_row = wm * Cfg::WM + r32, b_row = wn * Cfg::WN + r32;
    const int a_rd0 = a_row * PITCH + (((0 + half) ^ ((a_row >> 2) & 3)) << 4);
    const int a_rd1 = a_row * PITCH + (((2 + half) ^ ((a_row >> 2) & 3)) << 4);
    const int b_rd0 = Cfg::A_BYTES + b_row * PITCH + (((0 + half) ^ ((b_row >> 2) & 3)) << 4);
    const int b_rd1 = Cfg::A_BYTES + b_row * PITCH + (((2 + half) ^ ((b_row >> 2) & 3)) << 4);

    auto read_a = [&](int stage_byte, int q, int i) -> v4i {
        return *reinterpret_cast<const v4i *>(smem + stage_byte + (q ? a_rd1 : a_rd0) + i * 32 * PITCH);
    };
    auto read_b = [&](int stage_byte, int q, int j) -> v4i {
        return *reinterpret_cast<const v4i *>(smem + stage_byte + (q ? b_rd1 : b_rd0) + j * 32 * PITCH);
    };

    v16i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    // ---- prologue: tiles 0 and 1 into stages 0 and 1, tile 2 in flight ----
    load_global(0);
    store_lds(0);
    load_global(1);
    store_lds(STAGE);
    load_global(2);
    __syncthreads();

    // B fragments: two register sets, one per 64-nibble half q; A: ping-pong per sub-step
    v4i b_ev[2][FN], b_od[2][FN], b_pk[FN];
    v4i a_ev[2], a_od[2], a_pk[2];
#pragma unroll
    for (int j = 0; j < FN; ++j) x16_expand(read_b(0, 0, j), b_ev[0][j], b_od[0][j]);
    x16_expand(read_a(0, 0, 0), a_ev[0], a_od[0]);
    a_pk[1] = read_a(0, 0, 1);

    int cur = 0, nxt = STAGE, wr = 2 * STAGE;  // byte offsets of the ring stages

    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
        for (int q = 0; q < 2; ++q) {
#pragma unroll
            for (int i = 0; i < FM; ++i) {
                constexpr int S = 0;  // scheduling group id
                constexpr int NPS = (A_LOADS + B_LOADS + 2 * FM - 1) / (2 * FM);  // staging pieces per sub-step (upper bound)
                const int u = q * FM + i;  // sub-step within the K-step
                const int pa = u & 1;      // A register set used by this sub-step
                // -- LDS reads issued now, consumed one / two sub-steps later --
                {
                    // A fragment for sub-step u + 2
                    const int u2 = u + 2;
                    const int q2 = (u2 / FM) & 1, i2 = u2 % FM;
                    const int st2 = u2 >= 2 * FM ? nxt : cur;
                    a_pk[pa] = read_a(st2, q2, i2);
                }
                if (i == 0) {
                    // all B fragments of the next half (next tile when q == 1)
#pragma unroll
                    for (int j = 0; j < FN; ++j) b_pk[j] = read_b(q ? nxt : cur, q ^ 1, j);
                }
                // -- global staging traffic, spread over the sub-steps --
                constexpr int NP = A_LOADS + B_LOADS, SS = 2 * FM;
#pragma unroll
                for (int pc = 0; pc < NP; ++pc)
                    if (pc * SS / NP == u) restage_piece(pc, wr, kt + 3);
                // -- widen A for the next sub-step --
                x16_expand(a_pk[pa ^ 1], a_ev[pa ^ 1], a_od[pa ^ 1]);
                // -- widen this sub-step's share of the next half's B fragments --
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    if (j * FM / FN == i && (FN >= FM || j < FN)) x16_expand(b_pk[j], b_ev[q ^ 1][j], b_od[q ^ 1][j]);
                // -- contraction for this sub-step --
#pragma unroll
                for (int j = 0; j < FN; ++j) acc[i][j] = mfma32(b_ev[q][j], a_ev[pa], acc[i][j]);
#pragma unroll
                for (int j = 0; j < FN; ++j) acc[i][j] = mfma32(b_od[q][j], a_od[pa], acc[i][j]);
                // -- ask the scheduler for: the A read first, then MFMAs with everything
                //    else (B reads, staging traffic, widening VALU) in their shadow --
                __builtin_amdgcn_sched_group_barrier(0x100, 1, S);
#pragma unroll
                for (int j = 0; j < 2 * FN; ++j) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, S);  // one MFMA
                    if (i == 0 && j < FN) __builtin_amdgcn_sched_group_barrier(0x100, 1, S);  // a B read
                    if (j == 1) __builtin_amdgcn_sched_group_barrier(0x200, NPS, S);  // staging writes of this sub-step
                    if (j == 2) __builtin_amdgcn_sched_group_barrier(0x020, NPS, S);  // staging loads of this sub-step
                    __builtin_amdgcn_sched_group_barrier(0x002, 4, S);  // widening VALU
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // all waves are done reading stage `cur` and writing stage `wr`
        // (LDS counter only: the global prefetch of tile kt + 3 stays in flight)
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        const int t = cur;
        cur = nxt;
        nxt = wr;
        wr = t;
    }

    // ---- epilogue: drop the factor 256, guarded 16-byte stores ----
    const bool vec_ok = (p.N & 3) == 0 && ((uintptr_t)p.C & 15) == 0;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
        const int m = m0 + wm * Cfg::WM + i * 32 + r32;
        if (m >= p.M) continue;
        int32_t *crow = p.C + (size_t)m * p.N;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + wn * Cfg::WN + j * 32 + g * 8 + half * 4;
                v4i v = {acc[i][j][4 * g] >> 8, acc[i][j][4 * g + 1] >> 8, acc[i][j][4 * g + 2] >> 8, acc[i][j][4 * g + 3] >> 8};
                if (vec_ok && n + 3 < p.N) {
                    *reinterpret_cast<v4i *>(crow + n) = v;
                } else {
                    if (n < p.N) crow[n] = v.x;
                    if (n + 1 < p.N) crow[n + 1] = v.y;
                    if (n + 2 < p.N) crow[n + 2] = v.z;
                    if (n + 3 < p.N) crow[n + 3] = v.w;
                }
            }
        }
    }
}

}  // namespace qm
