// Wave-level split-K int4 GEMM for skinny, HBM-bound M, operands streamed global -> LDS.
//
// The reference has no such path (smallest tile 32 rows, configs.cu; shapes outside its
// table skipped, kernel.cu:340-385).  Same decomposition as gemm_skinny_kernel
// (qm_skinny.hpp): a workgroup owns 16*FN rows of B (columns of C) and all of M (padded to
// 16*FM); its NW waves split K between them.  What differs is how a fragment reaches the
// matrix core.  The MFMA wants lane r + 16 g to hold 16 bytes of row r, which as a load has
// consecutive lanes in different rows; the memory pipeline wants consecutive lanes in one
// row.  There the lanes load runs of rows into registers and a lane permutation on the LDS
// crossbar (ds_bpermute) sorts them out afterwards -- measured, that crossbar is where the
// time goes (bank-conflict cycles on 83 % of the cycles with an LDS instruction active at
// M = 16).  Here every load is a direct global -> LDS load (global_load_lds_dwordx4, as in
// the pipelined tile kernel): the lanes fetch whole 128-byte lines, 8 lanes per row, 8 rows
// per instruction; the hardware drops lane l's 16 bytes at LDS offset 16 l; and one
// ds_read_b128 per fragment picks them up in MFMA order.  No staging registers, no
// permutes, no ds_write, and all of a wave's loads are in flight within a few dozen cycles
// of its start.
//
// LDS layout.  One load instruction fills 1 KiB = 8 rows x 128 bytes (a "run": two
// 128-nibble chunks of K side by side).  A fragment block of 16 rows is two such loads
// (rows 0..7, rows 8..15).  Within a row the eight 16-byte pieces are stored permuted:
// logical piece p of row r sits at position p ^ ((r >> 1) & 7).  The 16 lanes r = 0..15 of a
// fragment read (k-group g, chunk j -> logical piece 4 j + g) then fall into 16 different
// 16-byte bank groups.  The permutation is applied on the global side (a lane chooses which
// piece of its line it fetches), so the 8 lanes of a row still cover one whole line.  K is
// contracted in that permuted order for A and B alike, which a sum over K cannot see.
//
// Every wave owns its ring slots (its own runs of K): no barrier between loading and
// contracting, only the wave's own s_waitcnt.  The waves' partial blocks are added up in
// the LDS with integer atomics; after one barrier the waves read the sums and store C, one
// 16 x 16 block per wave, 16 bytes per lane.  One launch, no workspace, no global atomics, C
// overwritten.
//
// Rows beyond 16 FM: the grid's second dimension walks over blocks of 16 FM rows of A
// (blockIdx.y), so a workgroup owns 16 FM rows x 16 FN columns.  Every workgroup pulls the
// rows of A and of B it owns through its CU's L1 once, over all of K: with four fragment
// blocks a square 2 x 2 moves 4 runs per 128 bytes of K where 4 x 1 moves 5, and its ring
// slot is 8 KiB instead of 10, so that two runs per wave -- all of K = 4096 on eight waves --
// are in flight at once within the 160 KiB of LDS.  The workgroups of one column block lie
// gridDim.x apart in launch order, on the same XCD when gridDim.x is a multiple of 8: the
// second reader of B's lines finds them in that XCD's L2.
#pragma once
#include <type_traits>

#include "qm_common.hpp"

namespace qm {

template <int FM_, int FN_, int NW_, int D_>
struct SkinnyDmaCfg {
    static constexpr int FM = FM_, FN = FN_, NW = NW_, D = D_;  // D: runs in flight per wave (ring depth)
    static constexpr int THREADS = 64 * NW;
    static constexpr int MAX_M = 16 * FM, BN = 16 * FN;
    static constexpr int BLOCKS = FM + FN;             // 16-row fragment blocks per run: A's first, then B's
    static constexpr int SLOT_BYTES = BLOCKS * 2048;   // one run of every block: 2 loads of 1 KiB each
    static constexpr int RING_BYTES = NW * D * SLOT_BYTES;
    static constexpr int RED_BYTES = FM * FN * 1024;   // the sum of the waves' blocks: [block][register][lane]
    static constexpr int LDS_BYTES = RING_BYTES + RED_BYTES;
    static constexpr int LOADS_PER_RUN = 2 * BLOCKS;
    static_assert(D >= 1 && D <= 4, "ring depth");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU");
    static_assert(LOADS_PER_RUN * D <= 63, "the memory counter counts to 63");
};

template <class Cfg>
__global__ void __launch_bounds__(Cfg::THREADS)
gemm_skinny_dma_kernel(const uint8_t *A, const uint8_t *B, int32_t *C, const int M, const int N, const int K, const int ldc, const int out,
                       const float *row_scale, const float *col_scale)
{
    // (scalar arguments: preloaded into SGPRs before the first wave starts, see gemm_skinny_stream_dma_kernel)
    GemmArgs p{A, B, C, M, N, K};
    p.row_scale = row_scale;
    p.col_scale = col_scale;
    p.out = out;
    p.ldc = ldc;
    constexpr int FM = Cfg::FM, FN = Cfg::FN, NW = Cfg::NW, D = Cfg::D, LPR = Cfg::LOADS_PER_RUN;
    extern __shared__ __align__(16) uint8_t smem[];
    int32_t *const red = reinterpret_cast<int32_t *>(smem + Cfg::RING_BYTES);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * Cfg::BN, m0 = blockIdx.y * Cfg::MAX_M;
    const bool b_read_once = M <= Cfg::MAX_M;  // one block of rows (gridDim.y == 1, without fetching the grid's size)
    const int Kb = p.K >> 1;             // bytes per row; a multiple of 16
    const int nruns = (Kb + 127) >> 7;   // 128-byte runs per row, the last one possibly short
    // this wave's runs: wave, wave + NW, ...
    const int cnt = wave < nruns ? (nruns - wave + NW - 1) / NW : 0;

    // ---- global side of a load: lane -> row l / 8 of the 8 rows, position l % 8 in the line.
    // Half h of a block holds its rows 8 h .. 8 h + 7; the piece fetched is the logical one
    // that belongs at this position.  A piece past the end of a short last run is fetched
    // from the last 16 bytes of the row instead (in bounds; the reader masks it away).
    const int row8 = lane >> 3, pos = lane & 7;
    uint32_t row_off[Cfg::BLOCKS][2], piece_off[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int r16 = 8 * h + row8;
        piece_off[h] = (uint32_t)((pos ^ ((r16 >> 1) & 7)) * 16);
#pragma unroll
        for (int i = 0; i < FM; ++i) row_off[i][h] = row_bytes24(min(m0 + i * 16 + r16, p.M - 1), Kb);
#pragma unroll
        for (int j = 0; j < FN; ++j) row_off[FM + j][h] = row_bytes24(min(n0 + j * 16 + r16, p.N - 1), Kb);
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const uint32_t wave_lds = __builtin_amdgcn_readfirstlane(lds0 + wave * D * Cfg::SLOT_BYTES);
    const uint32_t last16 = (uint32_t)(Kb - 16);
    auto issue_run = [&](const int run, const int slot) __attribute__((always_inline)) {
#pragma unroll
        for (int b = 0; b < Cfg::BLOCKS; ++b)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t dst = wave_lds + slot * Cfg::SLOT_BYTES + (2 * b + h) * 1024;
                const uint32_t goff = row_off[b][h] + min((uint32_t)run * 128u + piece_off[h], last16);
                // (a B that is read once and streams from HBM is marked non-temporal: it does not
                // push A out of the L2s -- measured 5-10 % on shapes whose B exceeds them; with
                // several row blocks the later readers want its lines kept)
                if (b < FM) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(goff), "s"(p.A) : "memory", "m0");
                else if (b_read_once) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(dst), "v"(goff), "s"(p.B) : "memory", "m0");
                else asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(goff), "s"(p.B) : "memory", "m0");
            }
    };

    // ---- all loads the ring holds go out first ----
#pragma unroll
    for (int d = 0; d < D; ++d)
        if (d < cnt) issue_run(wave + d * NW, d);

    // (the sums start from zero; cleared while the loads are in flight, and the barrier comes
    // while every wave is still waiting for its data anyway)
    for (int idx = tid; idx < FM * FN * 256; idx += Cfg::THREADS) red[idx] = 0;
    __syncthreads();

    // ---- reader side: lane (r, g) of a fragment, chunk j of the run -> logical piece 4 j + g ----
    const int rd_row = (r >> 3) * 1024 + (r & 7) * 128, rd_sw = (r >> 1) & 7;
    const int rd_at[2] = {rd_row + ((g ^ rd_sw) << 4), rd_row + (((4 + g) ^ rd_sw) << 4)};

    v4i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = v4i{0, 0, 0, 0};

    // Wait until at most `n` of this wave's loads are still in flight (n a compile-time value:
    // the counter's limit is an immediate operand).
    auto wait_loads = [&](const int younger, auto extra_) __attribute__((always_inline)) {
        constexpr int extra = decltype(extra_)::value;
        if (younger == 0) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(extra) : "memory");
        else if (younger == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LPR + extra > 63 ? 63 : LPR + extra) : "memory");
        else if (younger == 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * LPR + extra > 63 ? 63 : 2 * LPR + extra) : "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * LPR + extra > 63 ? 63 : 3 * LPR + extra) : "memory");
    };
    for (int it = 0; it < cnt; ++it) {
        const int run = wave + it * NW, slot = it % D;
        const uint8_t *const at = smem + wave * D * Cfg::SLOT_BYTES + slot * Cfg::SLOT_BYTES;
        // the loads of this run have landed when at most those of the younger runs are in
        // flight.  A's were issued first and come from the L2s: its fragments are read and
        // widened while B's are still on their way from HBM.
        const int younger = min(D - 1, cnt - 1 - it);
        wait_loads(younger, std::integral_constant<int, 2 * FN>{});
        v4i aev[FM][2], aod[FM][2];
        {
            v4i apk[FM][2];
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) apk[i][j] = *reinterpret_cast<const v4i *>(at + i * 2048 + rd_at[j]);
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) x16_expand_pairs(apk[i][j], aev[i][j], aod[i][j]);
        }
        wait_loads(younger, std::integral_constant<int, 0>{});
        v4i bpk[FN][2];
#pragma unroll
        for (int b = 0; b < FN; ++b)
#pragma unroll
            for (int j = 0; j < 2; ++j) bpk[b][j] = *reinterpret_cast<const v4i *>(at + (FM + b) * 2048 + rd_at[j]);
        if (it + D < cnt) {
            // the slot is free once its fragments are in registers: refill it
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            issue_run(run + D * NW, slot);
        }
        // a short last run: pieces past the end of K hold bytes that belong to other pieces
        if (run == nruns - 1 && (Kb & 127) != 0) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const bool valid = run * 128 + (4 * j + g) * 16 < Kb;
#pragma unroll
                for (int b = 0; b < FN; ++b) bpk[b][j] = valid ? bpk[b][j] : v4i{0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            v4i bev[FN], bod[FN];
#pragma unroll
            for (int b = 0; b < FN; ++b) x16_expand_pairs(bpk[b][j], bev[b], bod[b]);
#pragma unroll
            for (int i = 0; i < FM; ++i) {
#pragma unroll
                for (int b = 0; b < FN; ++b) acc[i][b] = mfma16(bev[b], aev[i][j], acc[i][b]);
#pragma unroll
                for (int b = 0; b < FN; ++b) acc[i][b] = mfma16(bod[b], aod[i][j], acc[i][b]);
            }
        }
    }

    // ---- add the NW partial sums up in the LDS (integer atomics: any order) ----
    if (cnt > 0) {
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    __hip_atomic_fetch_add(&red[((i * FN + j) * 4 + e) * 64 + lane], acc[i][j][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    // Every wave's adds are complete at the barrier; block bb is then stored by wave bb % NW.
    __syncthreads();

    // lane (r, g) of block (i, j) holds C[m0 + 16 i + r][n0 + 16 j + 4 g .. + 3]
    const bool vec_ok = (c_stride(p) & 3) == 0 && ((uintptr_t)p.C & (p.out == OUT_I32 ? 15 : 7)) == 0;
    for (int bb = wave; bb < FM * FN; bb += NW) {
        const int i = bb / FN, j = bb % FN;
        v4i s;
#pragma unroll
        for (int e = 0; e < 4; ++e) s[e] = red[(bb * 4 + e) * 64 + lane] >> 8;
        const int m = m0 + i * 16 + r, n = n0 + j * 16 + 4 * g;
        if (m >= p.M || n >= p.N) continue;
        const size_t at = (size_t)m * c_stride(p) + n;
        if (p.out == OUT_I32) {
            if (vec_ok) {
                *reinterpret_cast<v4i *>(p.C + at) = s;  // n % 4 == 0 and N % 4 == 0 (with a row stride: N is that stride or differs from it by a multiple of 256): all four inside
            } else if (n + 3 < p.N) {
                *reinterpret_cast<v4i_elem_aligned *>(p.C + at) = s;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < p.N) p.C[at + e] = s[e];
            }
        } else {
            uint16_t *const d = reinterpret_cast<uint16_t *>(p.C) + at;
            const float rs = scale_at(p.row_scale, m, p.M);
            uint16_t h[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int c = s[e];
                h[e] = round16(scaled(c, rs, scale_at(p.col_scale, n + e, p.N)), p.out);
            }
            if (vec_ok) {
                *reinterpret_cast<v2i *>(d) = v2i{(int)(h[0] | ((uint32_t)h[1] << 16)), (int)(h[2] | ((uint32_t)h[3] << 16))};
            } else if (n + 3 < p.N) {
                *reinterpret_cast<v2i_half_aligned *>(d) = v2i{(int)(h[0] | ((uint32_t)h[1] << 16)), (int)(h[2] | ((uint32_t)h[3] << 16))};
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < p.N) d[e] = h[e];
            }
        }
    }
}

}  // namespace qm

namespace qm {

// --------------------------------------------------------------------------
// The same for many column blocks per workgroup: a persistent grid (as many workgroups as
// the device holds at once) whose workgroups walk over column blocks blockIdx.x,
// + gridDim.x, ...  A wave's runs of K are the same for every block (K <= 256 NW R nibbles:
// at most R runs per wave), so its fragments of A are loaded, read and widened once and stay
// in registers; only B streams, through a ring of D (block, run) units per wave that runs
// ahead across block boundaries -- the loads of the next blocks are in flight while the
// current one is multiplied and added up.  The sums of consecutive blocks meet in
// alternating halves of the LDS array, one barrier per block (a half is cleared by the
// threads that stored it, two barriers before it is added into again).
// --------------------------------------------------------------------------
template <int FM_, int FN_, int NW_, int D_, int R_>
struct SkinnyStreamCfg {
    static constexpr int FM = FM_, FN = FN_, NW = NW_, D = D_, R = R_;
    static constexpr int THREADS = 64 * NW;
    static constexpr int MAX_M = 16 * FM, BN = 16 * FN;
    static constexpr int MAX_K = 256 * NW * R;            // nibbles
    static constexpr int UNIT_BYTES = FN * 2048;           // one run of B's blocks
    static constexpr int RING_BYTES = NW * D * UNIT_BYTES;
    static constexpr int A_BYTES = NW * R * FM * 2048;     // staging of A's fragments on their way into registers
    static constexpr int RED_BYTES = 2 * FM * FN * 1024;
    static constexpr int LDS_BYTES = RING_BYTES + A_BYTES + RED_BYTES;
    static constexpr int LOADS_PER_UNIT = 2 * FN;
    static_assert(D >= 1 && D <= 4 && R >= 1 && R <= 4, "ring depth, runs per wave");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU");
    static_assert(LOADS_PER_UNIT * D <= 63, "the memory counter counts to 63");
    static_assert(R * FM * 16 <= 64, "A's widened fragments live in registers");
};

// (The arguments are scalars, not a GemmArgs by value: scalar kernel arguments are preloaded
// into SGPRs before the first wave starts -- the library is built with
// -amdgpu-kernarg-preload-count=16 -- where a structure is fetched by the waves themselves;
// measured 1.5 % at M = 16, N = K = 4096 with B from HBM.)
template <class Cfg>
__global__ void __launch_bounds__(Cfg::THREADS)
gemm_skinny_stream_dma_kernel(const uint8_t *A, const uint8_t *B, int32_t *C, const int M, const int N, const int K, const int ldc,
                              const int out_and_grid, const int nblocks, const float *row_scale, const float *col_scale)  // 16 dwords: all preloaded
{
    // (out_and_grid: the output form in bits 0..7, the number of workgroups above.  gridDim.x
    // is a hidden kernel argument beyond the preloaded ones: read from there it is a scalar
    // load that every wave waits for before it can issue its first load.)
    GemmArgs p{A, B, C, M, N, K};
    p.row_scale = row_scale;
    p.col_scale = col_scale;
    p.out = out_and_grid & 0xFF;
    p.ldc = ldc;
    constexpr int FM = Cfg::FM, FN = Cfg::FN, NW = Cfg::NW, D = Cfg::D, R = Cfg::R, LPU = Cfg::LOADS_PER_UNIT;
    extern __shared__ __align__(16) uint8_t smem[];
    uint8_t *const a_stage = smem + Cfg::RING_BYTES;
    int32_t *const red = reinterpret_cast<int32_t *>(smem + Cfg::RING_BYTES + Cfg::A_BYTES);  // [2][block][register][lane]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int Kb = p.K >> 1;
    const int nruns = (Kb + 127) >> 7;
    const int cnt = wave < nruns ? (nruns - wave + NW - 1) / NW : 0;  // this wave's runs: wave, wave + NW, ... (at most R)
    // (set after A's loads are on their way: the number of blocks takes a division)
    int G, my_blocks, units;

    const int row8 = lane >> 3, pos = lane & 7;
    uint32_t piece_off[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) piece_off[h] = (uint32_t)((pos ^ (((8 * h + row8) >> 1) & 7)) * 16);
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const uint32_t last16 = (uint32_t)(Kb - 16);

    // ---- B: unit u -> block blockIdx.x + (u / cnt) G, run wave + (u % cnt) NW, ring slot u % D.
    // The cursor (u_blk, u_run) runs ahead of the unit being multiplied.
    const uint32_t ring_lds = __builtin_amdgcn_readfirstlane(lds0 + wave * D * Cfg::UNIT_BYTES);
    int ld_u = 0, ld_blk = blockIdx.x, ld_run = 0;
    auto issue_unit = [&]() __attribute__((always_inline)) {
        const int slot = ld_u % D, run = wave + ld_run * NW, n0 = ld_blk * Cfg::BN;
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t dst = ring_lds + slot * Cfg::UNIT_BYTES + (2 * j + h) * 1024;
                const uint32_t goff = row_bytes24(min(n0 + j * 16 + 8 * h + row8, p.N - 1), Kb) + min((uint32_t)run * 128u + piece_off[h], last16);
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(dst), "v"(goff), "s"(p.B) : "memory", "m0");
            }
        ++ld_u;
        if (++ld_run == cnt) { ld_run = 0; ld_blk += G; }
    };

    // ---- A first (it comes from the L2s and is needed by every block), then the ring ----
    const uint32_t a_lds = __builtin_amdgcn_readfirstlane(lds0 + Cfg::RING_BYTES + wave * R * FM * 2048);
    // (issued the other way round -- B first, its requests out before A's pass through the L1 --
    // the kernel is 10-15 % slower with B from HBM: every wave then waits for all of its loads
    // before it can widen A)
#pragma unroll
    for (int q = 0; q < R; ++q)
        if (q < cnt) {
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const uint32_t dst = a_lds + (q * FM + i) * 2048 + h * 1024;
                    const uint32_t goff = row_bytes24(min(i * 16 + 8 * h + row8, p.M - 1), Kb) + min((uint32_t)(wave + q * NW) * 128u + piece_off[h], last16);
                    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(goff), "s"(p.A) : "memory", "m0");
                }
        }
    {
        // (the asm keeps the compiler from starting on the division before A's loads above)
        int grid = out_and_grid >> 8;
        asm volatile("" : "+s"(grid));
        G = grid;
        // one block per workgroup whenever the device holds them all at once: no division then
        my_blocks = (int)blockIdx.x >= nblocks ? 0 : (G >= nblocks ? 1 : (nblocks - (int)blockIdx.x + G - 1) / G);
        units = my_blocks * cnt;  // (block, run) pairs of this wave, block-major
    }
    const int ahead = min(D, units);
    for (int d = 0; d < ahead; ++d) issue_unit();

    for (int idx = tid; idx < 2 * FM * FN * 256; idx += Cfg::THREADS) red[idx] = 0;
    __syncthreads();

    const int rd_row = (r >> 3) * 1024 + (r & 7) * 128, rd_sw = (r >> 1) & 7;
    const int rd_at[2] = {rd_row + ((g ^ rd_sw) << 4), rd_row + (((4 + g) ^ rd_sw) << 4)};

    // A's fragments -> registers, widened: everything issued after them may stay in flight
    auto wait_b = [&](const int younger) __attribute__((always_inline)) {
        if (younger <= 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        else if (younger == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LPU) : "memory");
        else if (younger == 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * LPU > 63 ? 63 : 2 * LPU) : "memory");
        else if (younger == 3) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * LPU > 63 ? 63 : 3 * LPU) : "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(4 * LPU > 63 ? 63 : 4 * LPU) : "memory");
    };
    wait_b(ahead);
    v4i aev[R][FM][2], aod[R][FM][2];
#pragma unroll
    for (int q = 0; q < R; ++q)
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                // (a run this wave does not have reads whatever the staging area holds; it is never multiplied)
                const v4i pk = *reinterpret_cast<const v4i *>(a_stage + (wave * R + q) * FM * 2048 + i * 2048 + rd_at[j]);
                x16_expand_pairs(pk, aev[q][i][j], aod[q][i][j]);
            }

    int u = 0;
    for (int b = 0, half = 0; b < my_blocks; ++b, half ^= 1) {
        const int blk = blockIdx.x + b * G;
        v4i acc[FM][FN];
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) acc[i][j] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int q = 0; q < R; ++q) {
            if (q < cnt) {
                const int slot = u % D, run = wave + q * NW;
                wait_b(min(D - 1, units - 1 - u));
                const uint8_t *const at = smem + (wave * D + slot) * Cfg::UNIT_BYTES;
                v4i bpk[FN][2];
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int c = 0; c < 2; ++c) bpk[j][c] = *reinterpret_cast<const v4i *>(at + j * 2048 + rd_at[c]);
                if (u + D < units) {
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    issue_unit();
                }
                ++u;
                if (run == nruns - 1 && (Kb & 127) != 0) {
#pragma unroll
                    for (int c = 0; c < 2; ++c) {
                        const bool valid = run * 128 + (4 * c + g) * 16 < Kb;
#pragma unroll
                        for (int j = 0; j < FN; ++j) bpk[j][c] = valid ? bpk[j][c] : v4i{0, 0, 0, 0};
                    }
                }
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    v4i bev[FN], bod[FN];
#pragma unroll
                    for (int j = 0; j < FN; ++j) x16_expand_pairs(bpk[j][c], bev[j], bod[j]);
#pragma unroll
                    for (int i = 0; i < FM; ++i) {
#pragma unroll
                        for (int j = 0; j < FN; ++j) acc[i][j] = mfma16(bev[j], aev[q][i][c], acc[i][j]);
#pragma unroll
                        for (int j = 0; j < FN; ++j) acc[i][j] = mfma16(bod[j], aod[q][i][c], acc[i][j]);
                    }
                }
            }
        }
        int32_t *const rh = red + half * (FM * FN * 256);
        if (cnt > 0) {
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        __hip_atomic_fetch_add(&rh[((i * FN + j) * 4 + e) * 64 + lane], acc[i][j][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
        __syncthreads();
        // Block bb is stored (and its sums cleared for the block after next) by wave bb % NW:
        // lane (r, g) holds C[16 i + r][n0 + 16 j + 4 g .. + 3] in register order, four reads of
        // 64 consecutive words each, 16 bytes per lane to C.
        const int n0 = blk * Cfg::BN;
        const bool vec_ok = (c_stride(p) & 3) == 0 && ((uintptr_t)p.C & (p.out == OUT_I32 ? 15 : 7)) == 0;
        for (int bb = wave; bb < FM * FN; bb += NW) {
            v4i s;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                int32_t *const at_red = &rh[(bb * 4 + e) * 64 + lane];
                s[e] = *at_red >> 8;
                *at_red = 0;
            }
            const int m = (bb / FN) * 16 + r, n = n0 + (bb % FN) * 16 + 4 * g;
            if (m >= p.M || n >= p.N) continue;
            const size_t at = (size_t)m * c_stride(p) + n;
            if (p.out == OUT_I32) {
                if (vec_ok) {
                    *reinterpret_cast<v4i *>(p.C + at) = s;
                } else if (n + 3 < p.N) {
                    *reinterpret_cast<v4i_elem_aligned *>(p.C + at) = s;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < p.N) p.C[at + e] = s[e];
                }
            } else {
                uint16_t *const d = reinterpret_cast<uint16_t *>(p.C) + at;
                const float rs = scale_at(p.row_scale, m, p.M);
                uint16_t h[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int c = s[e];
                    h[e] = round16(scaled(c, rs, scale_at(p.col_scale, n + e, p.N)), p.out);
                }
                if (vec_ok) {
                    *reinterpret_cast<v2i *>(d) = v2i{(int)(h[0] | ((uint32_t)h[1] << 16)), (int)(h[2] | ((uint32_t)h[3] << 16))};
                } else if (n + 3 < p.N) {
                    *reinterpret_cast<v2i_half_aligned *>(d) = v2i{(int)(h[0] | ((uint32_t)h[1] << 16)), (int)(h[2] | ((uint32_t)h[3] << 16))};
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < p.N) d[e] = h[e];
                }
            }
        }
    }
}

}  // namespace qm
