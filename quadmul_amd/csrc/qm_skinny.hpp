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
// every lane's 16 bytes separately.  Lanes therefore load row lane/4, chunk lane%4
// (4 consecutive lanes = 64 contiguous bytes) and a lane permutation through the
// LDS crossbar (ds_bpermute, no LDS memory involved) puts the fragments into MFMA
// order afterwards.
#pragma once
#include "qm_common.hpp"

namespace qm {

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
    const int ld_row = lane >> 2, ld_ch = lane & 3;  // what this lane loads: row, 16-byte chunk
    const int from_lane = (4 * r + g) * 4;           // where MFMA lane (r, g) finds its fragment (byte address of a lane)
    uint32_t b_off[FN], a_off[FM];
#pragma unroll
    for (int j = 0; j < FN; ++j) b_off[j] = (uint32_t)min(n0 + j * 16 + ld_row, p.N - 1) * (uint32_t)Kb + ld_ch * 16;
#pragma unroll
    for (int i = 0; i < FM; ++i) a_off[i] = (uint32_t)min(i * 16 + ld_row, p.M - 1) * (uint32_t)Kb + ld_ch * 16;
    auto to_mfma_order = [&](const v4i q) -> v4i {
        v4i o;
        o.x = __builtin_amdgcn_ds_bpermute(from_lane, q.x);
        o.y = __builtin_amdgcn_ds_bpermute(from_lane, q.y);
        o.z = __builtin_amdgcn_ds_bpermute(from_lane, q.z);
        o.w = __builtin_amdgcn_ds_bpermute(from_lane, q.w);
        return o;
    };

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
    auto contract = [&](const v4i (&bq)[FN], const v4i (&aq)[FM]) __attribute__((always_inline)) {
        v4i bev[FN], bod[FN];
#pragma unroll
        for (int j = 0; j < FN; ++j) x16_expand(to_mfma_order(bq[j]), bev[j], bod[j]);
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            v4i aev, aod;
            x16_expand(to_mfma_order(aq[i]), aev, aod);
#pragma unroll
            for (int j = 0; j < FN; ++j) acc[i][j] = mfma16(bev[j], aev, acc[i][j]);
#pragma unroll
            for (int j = 0; j < FN; ++j) acc[i][j] = mfma16(bod[j], aod, acc[i][j]);
        }
    };
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
        for (int u = 0; u < U; ++u) contract(bq[u], aq[u]);
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
            const size_t at = (size_t)m * p.N + n;
            if (p.out == OUT_I32) p.C[at] = s >> 8;
            else reinterpret_cast<uint16_t *>(p.C)[at] = round16(scaled(s >> 8, scale_at(p.row_scale, m, p.M), scale_at(p.col_scale, n, p.N)), p.out);
        }
    }
}

// --------------------------------------------------------------------------
// One or two rows of A (GEMV-like shapes): no matrix core.  v_dot8_i32_i4 multiplies eight
// signed nibbles of one dword with the eight of another and adds them up -- the packed
// format as it is, no widening, no lane permutation, no factor to shift away.  A workgroup
// owns 16 * FN rows of B and all of M; its NW waves split K in 128-nibble chunks as above;
// a lane loads 16 bytes of row lane / 4 of B (coalesced quads) and the matching 16 bytes
// of every row of A (the same 64 bytes for all 16 quads of the wave: one cache line),
// and the four lanes of a quad add their sums up at the end.  Measured against the matrix-core
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
gemm_dot_kernel(const GemmArgs p)
{
    constexpr int MR = Cfg::MR, FN = Cfg::FN, NW = Cfg::NW, U = Cfg::U;
    __shared__ int32_t red[MR][FN * 16];  // the sum over the waves

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n0 = blockIdx.x * Cfg::BN;
    const int Kb = p.K >> 1;
    const int nchunks = (p.K + 127) >> 7;
    const int ld_row = lane >> 2, ld_ch = lane & 3;
    uint32_t b_off[FN], a_off[MR];
#pragma unroll
    for (int j = 0; j < FN; ++j) b_off[j] = (uint32_t)min(n0 + j * 16 + ld_row, p.N - 1) * (uint32_t)Kb + ld_ch * 16;
#pragma unroll
    for (int i = 0; i < MR; ++i) a_off[i] = (uint32_t)min(i, p.M - 1) * (uint32_t)Kb + ld_ch * 16;

    int32_t acc[MR][FN];
#pragma unroll
    for (int i = 0; i < MR; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = 0;
    for (int idx = tid; idx < MR * FN * 16; idx += Cfg::THREADS) (&red[0][0])[idx] = 0;
    __syncthreads();

    for (int c0 = wave * U; c0 < nchunks; c0 += NW * U) {
        v4i bq[U][FN], aq[U][MR];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int kofs = (c0 + u) * 64;
            const bool ok = kofs + ld_ch * 16 < Kb;  // also false for c0+u >= nchunks; zeros add nothing
#pragma unroll
            for (int j = 0; j < FN; ++j)
                bq[u][j] = ok ? __builtin_nontemporal_load(reinterpret_cast<const v4i *>(p.B + b_off[j] + kofs)) : v4i{0, 0, 0, 0};
#pragma unroll
            for (int i = 0; i < MR; ++i)
                aq[u][i] = ok ? *reinterpret_cast<const v4i *>(p.A + a_off[i] + kofs) : v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int i = 0; i < MR; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[i][j] = __builtin_amdgcn_sdot8(aq[u][i][e], bq[u][j][e], acc[i][j], false);
    }

    // the four lanes of a quad hold the four 32-nibble pieces of a chunk: add them up, then
    // the waves' sums in the LDS
#pragma unroll
    for (int i = 0; i < MR; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            int32_t v = acc[i][j];
            v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
            v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
            if (ld_ch == 0) __hip_atomic_fetch_add(&red[i][j * 16 + ld_row], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
    __syncthreads();
    for (int idx = tid; idx < MR * FN * 16; idx += Cfg::THREADS) {
        const int m = idx / (FN * 16), n = n0 + idx % (FN * 16);
        if (m < p.M && n < p.N) {
            const int32_t s = (&red[0][0])[idx];
            const size_t at = (size_t)m * p.N + n;
            if (p.out == OUT_I32) p.C[at] = s;
            else reinterpret_cast<uint16_t *>(p.C)[at] = round16(scaled(s, scale_at(p.row_scale, m, p.M), scale_at(p.col_scale, n, p.N)), p.out);
        }
    }
}

}  // namespace qm
