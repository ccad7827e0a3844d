// Wave-level split-K int4 GEMM for skinny, HBM-bound M (decode-style shapes).
//
// The reference has no such path: its smallest tile is 32 rows (configs.cu) and
// shapes outside its table are skipped (kernel.cu:340-385).  Here a workgroup
// owns 16*FN rows of B (columns of C) and all of M (padded to 16*FM <= 128); its
// NW waves split K between them in 128-nibble chunks, each wave streaming its
// share of B straight from HBM into registers, and the partial 16x16 blocks are
// added up in the LDS with integer atomics.  One launch, no workspace, no global atomics,
// C overwritten.
//
// The MFMA wants lane r + 16 g to hold 16 bytes of row r (k-group g), which as a
// load has consecutive lanes in different rows: the memory pipeline then handles
// every lane's 16 bytes separately.  Lanes therefore load runs of contiguous bytes
// of a row and a lane permutation through the LDS crossbar (ds_bpermute, no LDS
// memory involved) puts the fragments into MFMA order afterwards.  With an even
// number of chunks per wave and turn the runs are whole 128-byte lines -- 8 lanes per
// row, two chunks side by side, 8 rows per load (measured with B from HBM: 15-19 %
// faster than 64-byte runs; 256-byte runs add nothing) -- and the two loads that hold
// the upper and lower 8 rows are merged into one register per chunk with a DPP move
// before the permutation; with an odd number the runs are 64 bytes, 4 lanes per row.
#pragma once
#include "qm_common.hpp"

namespace qm {

// Lane l of `q` moves to the lane whose byte address table entry `from_byte` names it.
__device__ __forceinline__ v4i lane_gather(const v4i q, const int from_byte)
{
    v4i o;
    o.x = __builtin_amdgcn_ds_bpermute(from_byte, q.x);
    o.y = __builtin_amdgcn_ds_bpermute(from_byte, q.y);
    o.z = __builtin_amdgcn_ds_bpermute(from_byte, q.z);
    o.w = __builtin_amdgcn_ds_bpermute(from_byte, q.w);
    return o;
}

// 128-byte runs: lane l of a load holds row l / 8 of its 8 rows, bytes 16 * (l % 8) ..
// of the pair of chunks (l % 8 < 4: chunk c, else chunk c + 1).  `lo` holds rows 0..7,
// `hi` rows 8..15.  c0 gets chunk c of all 16 rows: where lo has chunk c + 1 (lanes
// 4..7 of every 8) the chunk c of hi, which sits 4 lanes lower, is moved in (DPP row
// shift right by 4, banks 1 and 3 written); c1 likewise gets chunk c + 1 (shift left by
// 4, banks 0 and 2).  Afterwards row r, k-group g of chunk c is in lane
// 8 * (r % 8) + 4 * (r / 8) + g of c0, and of chunk c + 1 in lane
// 8 * (r % 8) + 4 * (1 - r / 8) + g of c1.
__device__ __forceinline__ void chunks_from_halves(const v4i lo, const v4i hi, v4i &c0, v4i &c1)
{
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        c0[e] = __builtin_amdgcn_update_dpp(lo[e], hi[e], 0x114, 0xF, 0xA, false);
        c1[e] = __builtin_amdgcn_update_dpp(lo[e], hi[e], 0x104, 0xF, 0x5, false);
    }
}

template <int FM_, int FN_, int NW_, int U_>
struct SkinnyCfg {
    static constexpr int FM = FM_, FN = FN_, NW = NW_, U = U_;
    static constexpr int THREADS = 64 * NW;
    static constexpr int MAX_M = 16 * FM, BN = 16 * FN;
    static constexpr int LDS_BYTES = FM * FN * 64 * 16;  // one block set: the waves add into it
    static_assert(LDS_BYTES <= 64 * 1024, "static LDS");
};

template <class Cfg>
__global__ void __launch_bounds__(Cfg::THREADS)
gemm_skinny_kernel(const GemmArgs p)
{
    constexpr int FM = Cfg::FM, FN = Cfg::FN, NW = Cfg::NW, U = Cfg::U;
    // the sum of the waves' partial blocks: [block][register e][lane], so that the 64 lanes
    // of an LDS atomic fall into 64 consecutive words
    __shared__ int32_t red[FM * FN][4][64];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * Cfg::BN;
    const int Kb = p.K >> 1;
    const int nchunks = (p.K + 127) >> 7;  // 64 packed bytes per row per chunk

    // Rows past the edge are clamped to a valid row; their products are dropped
    // by the store guards.
    v4i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = v4i{0, 0, 0, 0};
    // (cleared now, while the waves are still starting up; the barrier costs nothing yet)
    for (int idx = tid; idx < FM * FN * 256; idx += Cfg::THREADS) (&red[0][0][0])[idx] = 0;
    __syncthreads();

    // chunk c belongs to wave (c / U) % NW: each wave takes U consecutive chunks
    // per round so that its U*(FN+FM) loads are all in flight before the first MFMA.
    auto contract = [&](const int from, const v4i (&bq)[FN], const v4i (&aq)[FM]) __attribute__((always_inline)) {
        v4i bev[FN], bod[FN];
#pragma unroll
        for (int j = 0; j < FN; ++j) x16_expand(lane_gather(bq[j], from), bev[j], bod[j]);
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            v4i aev, aod;
            x16_expand(lane_gather(aq[i], from), aev, aod);
#pragma unroll
            for (int j = 0; j < FN; ++j) acc[i][j] = mfma16(bev[j], aev, acc[i][j]);
#pragma unroll
            for (int j = 0; j < FN; ++j) acc[i][j] = mfma16(bod[j], aod, acc[i][j]);
        }
    };
    if constexpr (U % 2 == 0) {
        // pairs of chunks, 128-byte runs: 8 rows per load, lower and upper half of a fragment's rows
        const int ld8_row = lane >> 3, ld8_ch = lane & 7;
        const int from_c0 = (8 * (r & 7) + 4 * (r >> 3) + g) * 4, from_c1 = (8 * (r & 7) + 4 * (1 - (r >> 3)) + g) * 4;
        uint32_t b8_off[FN][2], a8_off[FM][2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int j = 0; j < FN; ++j) b8_off[j][h] = row_bytes24(min(n0 + j * 16 + 8 * h + ld8_row, p.N - 1), Kb) + ld8_ch * 16;
#pragma unroll
            for (int i = 0; i < FM; ++i) a8_off[i][h] = row_bytes24(min(i * 16 + 8 * h + ld8_row, p.M - 1), Kb) + ld8_ch * 16;
        }
        for (int c0 = wave * U; c0 < nchunks; c0 += NW * U) {
            v4i bl[U / 2][FN][2], al[U / 2][FM][2];
#pragma unroll
            for (int pu = 0; pu < U / 2; ++pu) {
                const int kofs = (c0 + 2 * pu) * 64;
                const bool ok = kofs + ld8_ch * 16 < Kb;  // also false for chunks past the last
#pragma unroll
                for (int h = 0; h < 2; ++h) {
#pragma unroll
                    for (int j = 0; j < FN; ++j)
                        bl[pu][j][h] = ok ? __builtin_nontemporal_load(reinterpret_cast<const v4i *>(p.B + b8_off[j][h] + kofs)) : v4i{0, 0, 0, 0};
#pragma unroll
                    for (int i = 0; i < FM; ++i)
                        al[pu][i][h] = ok ? *reinterpret_cast<const v4i *>(p.A + a8_off[i][h] + kofs) : v4i{0, 0, 0, 0};
                }
            }
#pragma unroll
            for (int pu = 0; pu < U / 2; ++pu) {
                v4i bq0[FN], bq1[FN], aq0[FM], aq1[FM];
#pragma unroll
                for (int j = 0; j < FN; ++j) chunks_from_halves(bl[pu][j][0], bl[pu][j][1], bq0[j], bq1[j]);
#pragma unroll
                for (int i = 0; i < FM; ++i) chunks_from_halves(al[pu][i][0], al[pu][i][1], aq0[i], aq1[i]);
                contract(from_c0, bq0, aq0);
                contract(from_c1, bq1, aq1);
            }
        }
    } else {
        // single chunks, 64-byte runs: row lane / 4, 16-byte piece lane % 4
        const int ld_row = lane >> 2, ld_ch = lane & 3;
        const int from_lane = (4 * r + g) * 4;  // where MFMA lane (r, g) finds its fragment (byte address of a lane)
        uint32_t b_off[FN], a_off[FM];
#pragma unroll
        for (int j = 0; j < FN; ++j) b_off[j] = row_bytes24(min(n0 + j * 16 + ld_row, p.N - 1), Kb) + ld_ch * 16;
#pragma unroll
        for (int i = 0; i < FM; ++i) a_off[i] = row_bytes24(min(i * 16 + ld_row, p.M - 1), Kb) + ld_ch * 16;
        for (int c0 = wave * U; c0 < nchunks; c0 += NW * U) {
            v4i bq[U][FN], aq[U][FM];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int kofs = (c0 + u) * 64;
                const bool ok = kofs + ld_ch * 16 < Kb;  // also false for c0+u >= nchunks
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    bq[u][j] = ok ? __builtin_nontemporal_load(reinterpret_cast<const v4i *>(p.B + b_off[j] + kofs)) : v4i{0, 0, 0, 0};
#pragma unroll
                for (int i = 0; i < FM; ++i)
                    aq[u][i] = ok ? *reinterpret_cast<const v4i *>(p.A + a_off[i] + kofs) : v4i{0, 0, 0, 0};
            }
#pragma unroll
            for (int u = 0; u < U; ++u) contract(from_lane, bq[u], aq[u]);
        }
    }

    // ---- add the NW partial sums up in the LDS (integer atomics: any order) ----
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                __hip_atomic_fetch_add(&red[i * FN + j][e][lane], acc[i][j][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    __syncthreads();

    // One output element per thread and pass: element (m, n) of block blk sits in register
    // n % 4 of lane m + 16 * (n / 4); 16 consecutive threads write 64 contiguous bytes of a
    // row of C.
    for (int idx = tid; idx < FM * FN * 256; idx += Cfg::THREADS) {
        const int blk = idx >> 8, ml = (idx >> 4) & 15, nl = idx & 15;
        const int32_t s = red[blk][nl & 3][ml + 16 * (nl >> 2)];
        const int m = (blk / FN) * 16 + ml, n = n0 + (blk % FN) * 16 + nl;
        if (m < p.M && n < p.N) {
            const size_t at = (size_t)m * c_stride(p) + n;
            if (p.out == OUT_I32) p.C[at] = s >> 8;
            else reinterpret_cast<uint16_t *>(p.C)[at] = round16(scaled(s >> 8, scale_at(p.row_scale, m, p.M), scale_at(p.col_scale, n, p.N)), p.out);
        }
    }
}

// --------------------------------------------------------------------------
// The same for many column blocks per workgroup (N well beyond 16 * FN * 2 workgroups per
// CU) when every wave's share of K is one turn of U chunks (K <= 128 * NW * U): the
// workgroup walks over column blocks blockIdx.x, + gridDim.x, ...  A wave's fragments of A
// are the same for every block, so they are loaded, permuted and widened once; the B
// fragments of the next block are on their way while the current one is multiplied; and
// the sums of consecutive blocks meet in alternating halves of the LDS array, which takes
// one barrier per block (a half is cleared by the threads that stored it, two barriers
// before it is added into again).
// --------------------------------------------------------------------------
template <class Cfg>
__global__ void __launch_bounds__(Cfg::THREADS)
gemm_skinny_stream_kernel(const GemmArgs p, const int nblocks)
{
    constexpr int FM = Cfg::FM, FN = Cfg::FN, U = Cfg::U, PAIRS = U / 2;
    static_assert(U % 2 == 0, "pairs of chunks (128-byte runs)");
    __shared__ int32_t red[2][FM * FN][4][64];
    static_assert(2 * Cfg::LDS_BYTES <= 64 * 1024, "static LDS");

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int Kb = p.K >> 1;
    const int ld8_row = lane >> 3, ld8_ch = lane & 7;
    const int from_c0 = (8 * (r & 7) + 4 * (r >> 3) + g) * 4, from_c1 = (8 * (r & 7) + 4 * (1 - (r >> 3)) + g) * 4;
    // this wave's chunks: wave * U + 0 .. U-1, in pairs; a pair (or the lane's piece of it) past K reads as zero
    bool ok[PAIRS];
    uint32_t kofs[PAIRS];
#pragma unroll
    for (int pu = 0; pu < PAIRS; ++pu) {
        kofs[pu] = (uint32_t)(wave * U + 2 * pu) * 64 + ld8_ch * 16;
        ok[pu] = (int)kofs[pu] < Kb;
    }
    auto load_b = [&](int blk, v4i (&bl)[PAIRS][FN][2]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t row = row_bytes24(min(blk * Cfg::BN + j * 16 + 8 * h + ld8_row, p.N - 1), Kb);
#pragma unroll
                for (int pu = 0; pu < PAIRS; ++pu)
                    bl[pu][j][h] = ok[pu] ? __builtin_nontemporal_load(reinterpret_cast<const v4i *>(p.B + row + kofs[pu])) : v4i{0, 0, 0, 0};
            }
    };
    int blk = blockIdx.x;
    v4i bl[PAIRS][FN][2], bl_next[PAIRS][FN][2];
    load_b(blk, bl);

    v4i aev[U][FM], aod[U][FM];
#pragma unroll
    for (int i = 0; i < FM; ++i) {
        v4i al[PAIRS][2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t row = row_bytes24(min(i * 16 + 8 * h + ld8_row, p.M - 1), Kb);
#pragma unroll
            for (int pu = 0; pu < PAIRS; ++pu)
                al[pu][h] = ok[pu] ? *reinterpret_cast<const v4i *>(p.A + row + kofs[pu]) : v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int pu = 0; pu < PAIRS; ++pu) {
            v4i q0, q1;
            chunks_from_halves(al[pu][0], al[pu][1], q0, q1);
            x16_expand(lane_gather(q0, from_c0), aev[2 * pu][i], aod[2 * pu][i]);
            x16_expand(lane_gather(q1, from_c1), aev[2 * pu + 1][i], aod[2 * pu + 1][i]);
        }
    }
    for (int idx = tid; idx < 2 * FM * FN * 256; idx += Cfg::THREADS) (&red[0][0][0][0])[idx] = 0;
    __syncthreads();

    for (int half = 0; blk < nblocks; blk += gridDim.x, half ^= 1) {
        const int next = blk + (int)gridDim.x;
        if (next < nblocks) load_b(next, bl_next);
        v4i acc[FM][FN];
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) acc[i][j] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int pu = 0; pu < PAIRS; ++pu) {
            v4i bev[2][FN], bod[2][FN];
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                v4i q0, q1;
                chunks_from_halves(bl[pu][j][0], bl[pu][j][1], q0, q1);
                x16_expand(lane_gather(q0, from_c0), bev[0][j], bod[0][j]);
                x16_expand(lane_gather(q1, from_c1), bev[1][j], bod[1][j]);
            }
#pragma unroll
            for (int c = 0; c < 2; ++c)
#pragma unroll
                for (int i = 0; i < FM; ++i) {
#pragma unroll
                    for (int j = 0; j < FN; ++j) acc[i][j] = mfma16(bev[c][j], aev[2 * pu + c][i], acc[i][j]);
#pragma unroll
                    for (int j = 0; j < FN; ++j) acc[i][j] = mfma16(bod[c][j], aod[2 * pu + c][i], acc[i][j]);
                }
        }
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    __hip_atomic_fetch_add(&red[half][i * FN + j][e][lane], acc[i][j][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        __syncthreads();
        const int n0 = blk * Cfg::BN;
        for (int idx = tid; idx < FM * FN * 256; idx += Cfg::THREADS) {
            const int b = idx >> 8, ml = (idx >> 4) & 15, nl = idx & 15;
            int32_t *at_red = &red[half][b][nl & 3][ml + 16 * (nl >> 2)];
            const int32_t s = *at_red;
            *at_red = 0;
            const int m = (b / FN) * 16 + ml, n = n0 + (b % FN) * 16 + nl;
            if (m < p.M && n < p.N) {
                const size_t at = (size_t)m * c_stride(p) + n;
                if (p.out == OUT_I32) p.C[at] = s >> 8;
                else reinterpret_cast<uint16_t *>(p.C)[at] = round16(scaled(s >> 8, scale_at(p.row_scale, m, p.M), scale_at(p.col_scale, n, p.N)), p.out);
            }
        }
#pragma unroll
        for (int pu = 0; pu < PAIRS; ++pu)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int h = 0; h < 2; ++h) bl[pu][j][h] = bl_next[pu][j][h];
    }
}

// --------------------------------------------------------------------------
// One or two rows of A (GEMV-like shapes): no matrix core.  v_dot8_i32_i4 multiplies eight
// signed nibbles of one dword with the eight of another and adds them up -- the packed
// format as it is, no widening, no lane permutation, no factor to shift away.  A workgroup
// owns 16 * FN rows of B and all of M; its NW waves split K in 128-nibble chunks as above;
// a lane loads 16 bytes of row lane / 8 of B (eight lanes = one 128-byte line, two chunks
// side by side) and the matching 16 bytes of every row of A (the same 128 bytes for all
// eight rows of the load: one cache line), and the eight lanes of a row add their sums up
// at the end.  Measured against the matrix-core
// kernel at N = K = 4096: 2.3 us against 3.0 us for one row, 2.5 against 3.0 for two, even
// from three rows on (the dot instructions then take as long as the lane permutations).
// --------------------------------------------------------------------------
template <int MR_, int FN_, int NW_, int U_>
struct DotCfg {
    static constexpr int MR = MR_, FN = FN_, NW = NW_, U = U_;
    static constexpr int THREADS = 64 * NW;
    static constexpr int MAX_M = MR, BN = 16 * FN;
};

template <class Cfg>
__global__ void __launch_bounds__(Cfg::THREADS)
gemm_dot_kernel(const uint8_t *A, const uint8_t *B, int32_t *C, const int M, const int N, const int K, const int ldc, const int out,
                       const float *row_scale, const float *col_scale)
{
    // (scalar arguments: preloaded into SGPRs before the first wave starts, see gemm_skinny_stream_dma_kernel)
    GemmArgs p{A, B, C, M, N, K};
    p.row_scale = row_scale;
    p.col_scale = col_scale;
    p.out = out;
    p.ldc = ldc;
    constexpr int MR = Cfg::MR, FN = Cfg::FN, NW = Cfg::NW, U = Cfg::U;
    __shared__ int32_t red[NW][MR][FN * 16];  // every wave's sums, added up after one barrier (nothing to clear, no barrier in front of the loads)

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n0 = blockIdx.x * Cfg::BN;
    const int Kb = p.K >> 1;
    const int nchunks = (p.K + 127) >> 7;
    static_assert(U % 2 == 0, "pairs of chunks (128-byte runs)");
    // 8 lanes per row: 128 contiguous bytes (two chunks side by side), 8 rows per load;
    // h = 0, 1: the lower and upper 8 of a block's 16 rows
    const int ld_row = lane >> 3, ld_ch = lane & 7;
    uint32_t b_off[FN][2], a_off[MR];
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int h = 0; h < 2; ++h) b_off[j][h] = row_bytes24(min(n0 + j * 16 + 8 * h + ld_row, p.N - 1), Kb) + ld_ch * 16;
#pragma unroll
    for (int i = 0; i < MR; ++i) a_off[i] = row_bytes24(min(i, p.M - 1), Kb) + ld_ch * 16;

    int32_t acc[MR][FN][2];
#pragma unroll
    for (int i = 0; i < MR; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j][0] = acc[i][j][1] = 0;
    for (int c0 = wave * U; c0 < nchunks; c0 += NW * U) {
        v4i bq[U / 2][FN][2], aq[U / 2][MR];
#pragma unroll
        for (int pu = 0; pu < U / 2; ++pu) {
            const int kofs = (c0 + 2 * pu) * 64;
            const bool ok = kofs + ld_ch * 16 < Kb;  // also false for chunks past the last; zeros add nothing
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int h = 0; h < 2; ++h)
                    bq[pu][j][h] = ok ? __builtin_nontemporal_load(reinterpret_cast<const v4i *>(p.B + b_off[j][h] + kofs)) : v4i{0, 0, 0, 0};
#pragma unroll
            for (int i = 0; i < MR; ++i)
                aq[pu][i] = ok ? *reinterpret_cast<const v4i *>(p.A + a_off[i] + kofs) : v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int pu = 0; pu < U / 2; ++pu)
#pragma unroll
            for (int i = 0; i < MR; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int h = 0; h < 2; ++h)
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[i][j][h] = __builtin_amdgcn_sdot8(aq[pu][i][e], bq[pu][j][h][e], acc[i][j][h], false);
    }

    // the eight lanes of a row hold the eight 32-nibble pieces of a pair of chunks: add them
    // up (within the quads, then the two quads through the mirror image of the eight), then
    // the waves' sums through the LDS
#pragma unroll
    for (int i = 0; i < MR; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                int32_t v = acc[i][j][h];
                v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]
                v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
                v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true);  // row_half_mirror: lane i <-> 7 - i
                if (ld_ch == 0) red[wave][i][j * 16 + 8 * h + ld_row] = v;
            }
    __syncthreads();
    for (int idx = tid; idx < MR * FN * 16; idx += Cfg::THREADS) {
        const int m = idx / (FN * 16), n = n0 + idx % (FN * 16);
        if (m < p.M && n < p.N) {
            int32_t s = 0;
#pragma unroll
            for (int w = 0; w < NW; ++w) s += (&red[w][0][0])[idx];
            const size_t at = (size_t)m * c_stride(p) + n;
            if (p.out == OUT_I32) p.C[at] = s;
            else reinterpret_cast<uint16_t *>(p.C)[at] = round16(scaled(s, scale_at(p.row_scale, m, p.M), scale_at(p.col_scale, n, p.N)), p.out);
        }
    }
}

}  // namespace qm
