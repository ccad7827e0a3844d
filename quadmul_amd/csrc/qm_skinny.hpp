// Wave-level split-K int4 GEMM for skinny, HBM-bound M (decode-style shapes).
//
// The reference has no such path: its smallest tile is 32 rows (configs.cu) and
// shapes outside its table are skipped (kernel.cu:340-385).  Here a workgroup
// owns 16*FN rows of B (columns of C) and all of M (padded to 16*FM <= 64); its
// NW waves split K between them in 128-nibble chunks, each wave streaming its
// share of B straight from HBM into MFMA operand registers (16-byte loads, 64
// contiguous bytes per row, no LDS on the way in), and the partial 16x16 blocks
// are summed through LDS.  One launch, no workspace, no atomics, C overwritten.
#pragma once
#include "qm_common.hpp"

namespace qm {

template <int FM_, int FN_, int NW_, int U_>
struct SkinnyCfg {
    static constexpr int FM = FM_, FN = FN_, NW = NW_, U = U_;
    static constexpr int THREADS = 64 * NW;
    static constexpr int MAX_M = 16 * FM, BN = 16 * FN;
    static constexpr int LDS_BYTES = NW * FM * FN * 64 * 16;
    static_assert(LDS_BYTES <= 64 * 1024, "static LDS");
};

template <class Cfg>
__global__ void __launch_bounds__(Cfg::THREADS)
gemm_skinny_kernel(const GemmArgs p)
{
    constexpr int FM = Cfg::FM, FN = Cfg::FN, NW = Cfg::NW, U = Cfg::U;
    __shared__ v4i red[NW][FM * FN][64];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * Cfg::BN;
    const int Kb = p.K >> 1;
    const int nchunks = (p.K + 127) >> 7;  // 64 packed bytes per row per chunk

    // Rows past the edge are clamped to a valid row; their products are dropped
    // by the store guards.
    uint32_t b_off[FN], a_off[FM];
#pragma unroll
    for (int j = 0; j < FN; ++j) b_off[j] = (uint32_t)min(n0 + j * 16 + r, p.N - 1) * (uint32_t)Kb + g * 16;
#pragma unroll
    for (int i = 0; i < FM; ++i) a_off[i] = (uint32_t)min(i * 16 + r, p.M - 1) * (uint32_t)Kb + g * 16;

    v4i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = v4i{0, 0, 0, 0};

    // chunk c belongs to wave (c / U) % NW: each wave takes U consecutive chunks
    // per round so that its U*(FN+FM) loads are all in flight before the first MFMA.
    for (int c0 = wave * U; c0 < nchunks; c0 += NW * U) {
        v4i bq[U][FN], aq[U][FM];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int kofs = (c0 + u) * 64;
            const bool ok = kofs + g * 16 < Kb;  // also false for c0+u >= nchunks
#pragma unroll
            for (int j = 0; j < FN; ++j)
                bq[u][j] = ok ? __builtin_nontemporal_load(reinterpret_cast<const v4i *>(p.B + b_off[j] + kofs)) : v4i{0, 0, 0, 0};
#pragma unroll
            for (int i = 0; i < FM; ++i)
                aq[u][i] = ok ? *reinterpret_cast<const v4i *>(p.A + a_off[i] + kofs) : v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            v4i bev[FN], bod[FN];
#pragma unroll
            for (int j = 0; j < FN; ++j) x16_expand(bq[u][j], bev[j], bod[j]);
#pragma unroll
            for (int i = 0; i < FM; ++i) {
                v4i aev, aod;
                x16_expand(aq[u][i], aev, aod);
#pragma unroll
                for (int j = 0; j < FN; ++j) acc[i][j] = mfma16(bev[j], aev, acc[i][j]);
#pragma unroll
                for (int j = 0; j < FN; ++j) acc[i][j] = mfma16(bod[j], aod, acc[i][j]);
            }
        }
    }

    // ---- reduce the NW partial sums through LDS ----
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) red[wave][i * FN + j][lane] = acc[i][j];
    __syncthreads();

    const bool vec_ok = (p.N & 3) == 0 && ((uintptr_t)p.C & 15) == 0;
    for (int item = tid; item < FM * FN * 64; item += Cfg::THREADS) {
        const int blk = item >> 6, l = item & 63;
        v4i s = red[0][blk][l];
#pragma unroll
        for (int w = 1; w < NW; ++w) {
            const v4i t = red[w][blk][l];
            s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
        }
        s.x >>= 8; s.y >>= 8; s.z >>= 8; s.w >>= 8;
        const int m = (blk / FN) * 16 + (l & 15);
        const int n = n0 + (blk % FN) * 16 + (l >> 4) * 4;
        if (m >= p.M) continue;
        int32_t *crow = p.C + (size_t)m * p.N;
        if (vec_ok && n + 3 < p.N) {
            *reinterpret_cast<v4i *>(crow + n) = s;
        } else {
            if (n < p.N) crow[n] = s.x;
            if (n + 1 < p.N) crow[n + 1] = s.y;
            if (n + 2 < p.N) crow[n + 2] = s.z;
            if (n + 3 < p.N) crow[n + 3] = s.w;
        }
    }
}

}  // namespace qm
