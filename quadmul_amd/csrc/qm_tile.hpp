// LDS-tiled int4 GEMM kernel for compute-bound shapes (gfx950, wave64, int8 MFMA).
//
// Takes the place of the reference's igemm<Config> (kernel.cu:62-266): its
// cp.async loaders (kernel.cu:118-152), two-stage pipeline (kernel.cu:186-260),
// WMMA s4 contraction (kernel.cu:246) and fragment stores (kernel.cu:155-184).
// Nothing of its structure is kept: the contraction is v_mfma_i32_16x16x64_i8 on
// nibbles widened to 16*s4 (see qm_common.hpp), tiles are up to 256x256 with one
// wave per SIMD, and LDS rows are XOR-swizzled in 16-byte chunks.
#pragma once
#include "qm_common.hpp"

namespace qm {

// MODE 0: LDS holds the packed bytes; every wave widens its fragments after ds_read.
// MODE 1: nibbles are widened while staging global -> LDS; LDS holds int8.
template <int BM_, int BN_, int BK_, int WGM_, int WGN_, int MODE_>
struct TileCfg {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WGM = WGM_, WGN = WGN_, MODE = MODE_;
    static constexpr int WAVES = WGM * WGN, THREADS = 64 * WAVES;
    static constexpr int WM = BM / WGM, WN = BN / WGN;  // per-wave tile
    static constexpr int FM = WM / 16, FN = WN / 16;    // 16x16 accumulator blocks per wave
    static constexpr int PCH = BK / 32;                 // packed 16-byte chunks per row per K-step
    static constexpr int PITCH = MODE == 0 ? BK / 2 : BK;  // LDS bytes per row
    static constexpr int CPR = PITCH / 16;                 // LDS 16-byte chunks per row
    static constexpr int A_BYTES = BM * PITCH, B_BYTES = BN * PITCH;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
    static constexpr int ROWS_PER_PASS = THREADS / PCH;  // rows covered by one load per thread
    static constexpr int A_LOADS = BM / ROWS_PER_PASS, B_LOADS = BN / ROWS_PER_PASS;
    static_assert(BK == 128 || BK == 256, "BK is 128 or 256 nibbles");
    static_assert(WM % 16 == 0 && WN % 16 == 0, "wave tile is a multiple of 16x16");
    static_assert(BM % ROWS_PER_PASS == 0 && BN % ROWS_PER_PASS == 0, "loader must tile the block evenly");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU");
};

// Chunk swizzle: lanes 0..15 of a fragment read touch 16 consecutive rows at the
// same logical chunk; XOR-ing the chunk index with low row bits spreads them over
// all banks.  With 4 chunks per row two rows share a 128-byte bank line.
template <int CPR>
__device__ __forceinline__ int swz(int row)
{
    if constexpr (CPR >= 8) return row & 7;
    else return (row >> 1) & (CPR - 1);
}

template <class Cfg>
__global__ void __launch_bounds__(Cfg::THREADS)
gemm_tile_kernel(const GemmArgs p, const int tiles_m, const int tiles_n, const int group_m)
{
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, MODE = Cfg::MODE;
    constexpr int FM = Cfg::FM, FN = Cfg::FN, PCH = Cfg::PCH, PITCH = Cfg::PITCH, CPR = Cfg::CPR;
    constexpr int A_LOADS = Cfg::A_LOADS, B_LOADS = Cfg::B_LOADS, RPP = Cfg::ROWS_PER_PASS;

    extern __shared__ __align__(16) uint8_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / Cfg::WGN, wn = wave % Cfg::WGN;
    const int r = lane & 15, g = lane >> 4;

    // ---- which tile: XCD-contiguous id, then columns of group_m tiles ----
    const int pid = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int width = group_m * tiles_n;
    const int first_m = (pid / width) * group_m;
    const int gsz = min(tiles_m - first_m, group_m);
    const int m0 = (first_m + (pid % width) % gsz) * BM;
    const int n0 = ((pid % width) / gsz) * BN;

    const int Kb = p.K >> 1;  // bytes per packed row
    const int KT = (p.K + BK - 1) / BK;

    // ---- loader geometry: thread -> (row, chunk) of the packed tile ----
    const int ld_ch = tid % PCH, ld_row = tid / PCH;
    uint32_t a_off[A_LOADS], b_off[B_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i)
        a_off[i] = (uint32_t)min(m0 + ld_row + i * RPP, p.M - 1) * (uint32_t)Kb + ld_ch * 16;
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i)
        b_off[i] = (uint32_t)min(n0 + ld_row + i * RPP, p.N - 1) * (uint32_t)Kb + ld_ch * 16;

    v4i a_reg[A_LOADS], b_reg[B_LOADS];

    auto load_global = [&](int kt) {
        const int kofs = kt * (BK / 2);
        const bool ok = kofs + ld_ch * 16 < Kb;  // whole chunks only: K % 32 == 0
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i)
            a_reg[i] = ok ? *reinterpret_cast<const v4i *>(p.A + a_off[i] + kofs) : v4i{0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i)
            b_reg[i] = ok ? *reinterpret_cast<const v4i *>(p.B + b_off[i] + kofs) : v4i{0, 0, 0, 0};
    };

    auto store_lds = [&](int stage) {
        uint8_t *As = smem + stage * Cfg::STAGE_BYTES;
        uint8_t *Bs = As + Cfg::A_BYTES;
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            const int row = ld_row + i * RPP;
            if constexpr (MODE == 0) {
                *reinterpret_cast<v4i *>(As + row * PITCH + ((ld_ch ^ swz<CPR>(row)) << 4)) = a_reg[i];
            } else {
                v4i ev, od;
                x16_expand(a_reg[i], ev, od);
                *reinterpret_cast<v4i *>(As + row * PITCH + (((2 * ld_ch) ^ swz<CPR>(row)) << 4)) = ev;
                *reinterpret_cast<v4i *>(As + row * PITCH + (((2 * ld_ch + 1) ^ swz<CPR>(row)) << 4)) = od;
            }
        }
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) {
            const int row = ld_row + i * RPP;
            if constexpr (MODE == 0) {
                *reinterpret_cast<v4i *>(Bs + row * PITCH + ((ld_ch ^ swz<CPR>(row)) << 4)) = b_reg[i];
            } else {
                v4i ev, od;
                x16_expand(b_reg[i], ev, od);
                *reinterpret_cast<v4i *>(Bs + row * PITCH + (((2 * ld_ch) ^ swz<CPR>(row)) << 4)) = ev;
                *reinterpret_cast<v4i *>(Bs + row * PITCH + (((2 * ld_ch + 1) ^ swz<CPR>(row)) << 4)) = od;
            }
        }
    };

    // acc[fm][fn]: B rows feed MFMA source 0 and A rows source 1, so a lane ends up
    // with 4 consecutive n for one m -- one 16-byte store into row-major C.
    v4i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = v4i{0, 0, 0, 0};

    const int a_row0 = wm * Cfg::WM + r, b_row0 = wn * Cfg::WN + r;

    auto compute = [&](int stage) {
        const uint8_t *As = smem + stage * Cfg::STAGE_BYTES;
        const uint8_t *Bs = As + Cfg::A_BYTES;
        if constexpr (MODE == 0) {
            // one packed 16-byte chunk per lane = 32 nibbles = two MFMA K-slices
#pragma unroll
            for (int kc = 0; kc < PCH / 4; ++kc) {
                v4i bev[FN], bod[FN];
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    const int row = b_row0 + j * 16;
                    const v4i q = *reinterpret_cast<const v4i *>(Bs + row * PITCH + (((kc * 4 + g) ^ swz<CPR>(row)) << 4));
                    x16_expand(q, bev[j], bod[j]);
                }
#pragma unroll
                for (int i = 0; i < FM; ++i) {
                    const int row = a_row0 + i * 16;
                    const v4i q = *reinterpret_cast<const v4i *>(As + row * PITCH + (((kc * 4 + g) ^ swz<CPR>(row)) << 4));
                    v4i aev, aod;
                    x16_expand(q, aev, aod);
#pragma unroll
                    for (int j = 0; j < FN; ++j) acc[i][j] = mfma16(bev[j], aev, acc[i][j]);
#pragma unroll
                    for (int j = 0; j < FN; ++j) acc[i][j] = mfma16(bod[j], aod, acc[i][j]);
                }
            }
        } else {
#pragma unroll
            for (int ks = 0; ks < BK / 64; ++ks) {
                v4i bf[FN];
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    const int row = b_row0 + j * 16;
                    bf[j] = *reinterpret_cast<const v4i *>(Bs + row * PITCH + (((ks * 4 + g) ^ swz<CPR>(row)) << 4));
                }
#pragma unroll
                for (int i = 0; i < FM; ++i) {
                    const int row = a_row0 + i * 16;
                    const v4i af = *reinterpret_cast<const v4i *>(As + row * PITCH + (((ks * 4 + g) ^ swz<CPR>(row)) << 4));
#pragma unroll
                    for (int j = 0; j < FN; ++j) acc[i][j] = mfma16(bf[j], af, acc[i][j]);
                }
            }
        }
    };

    // ---- main loop: register-staged double buffer, one barrier per K-step ----
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const int stage = kt & 1;
        if (kt + 1 < KT) load_global(kt + 1);
        compute(stage);
        if (kt + 1 < KT) store_lds(stage ^ 1);
        __syncthreads();
    }

    // ---- epilogue: drop the factor 256, guarded store ----
    const bool vec_ok = (p.N & 3) == 0 && ((uintptr_t)p.C & 15) == 0;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
        const int m = m0 + wm * Cfg::WM + i * 16 + r;
        if (m >= p.M) continue;
        int32_t *crow = p.C + (size_t)m * p.N;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const int n = n0 + wn * Cfg::WN + j * 16 + g * 4;
            v4i v = acc[i][j];
            v.x >>= 8; v.y >>= 8; v.z >>= 8; v.w >>= 8;
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

}  // namespace qm
