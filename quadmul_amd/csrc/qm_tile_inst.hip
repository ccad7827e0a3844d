// Instantiates the tile kernels assigned to translation unit QM_TU (see
// qm_configs.inc); compiled once per unit so the build runs in parallel.
#include "qm_launch.hpp"
#include "qm_tile.hpp"

#ifndef QM_TU
#error "compile with -DQM_TU=<n>"
#endif

namespace qm {

template <class Cfg>
static hipError_t launch_tile(const GemmArgs &p, hipStream_t stream, int group_m)
{
    static bool lds_ok[QM_MAX_DEVICES] = {};
    hipError_t e = ensure_dynamic_lds(&gemm_tile_kernel<Cfg>, Cfg::LDS_BYTES, lds_ok);
    if (e != hipSuccess) return e;
    const int tiles_m = (p.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (p.N + Cfg::BN - 1) / Cfg::BN;
    if (group_m < 1) group_m = 1;
    if (group_m > tiles_m) group_m = tiles_m;
    gemm_tile_kernel<Cfg><<<dim3(tiles_m * tiles_n), dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream>>>(p, tiles_m, tiles_n, group_m);
    return hipGetLastError();
}

#define QM_TILE_DEF(BM, BN, BK, WGM, WGN, MODE)                                                        \
    hipError_t QM_TILE_FN(BM, BN, BK, WGM, WGN, MODE)(const GemmArgs &p, hipStream_t s, int gm)            \
    {                                                                                                      \
        return launch_tile<TileCfg<BM, BN, BK, WGM, WGN, MODE>>(p, s, gm);                                 \
    }
#define QM_TILE_SKIP(...)
#define QM_TILE_IF_0(...) QM_TILE_SKIP(__VA_ARGS__)
#define QM_TILE_IF_1(...) QM_TILE_SKIP(__VA_ARGS__)
#define QM_TILE_IF_2(...) QM_TILE_SKIP(__VA_ARGS__)
#define QM_TILE_IF_3(...) QM_TILE_SKIP(__VA_ARGS__)
#define QM_TILE_IF_4(...) QM_TILE_SKIP(__VA_ARGS__)
#define QM_TILE_IF_5(...) QM_TILE_SKIP(__VA_ARGS__)
#define QM_TILE_IF_6(...) QM_TILE_SKIP(__VA_ARGS__)
#define QM_TILE_IF_7(...) QM_TILE_SKIP(__VA_ARGS__)
#if QM_TU == 0
#undef QM_TILE_IF_0
#define QM_TILE_IF_0(...) QM_TILE_DEF(__VA_ARGS__)
#elif QM_TU == 1
#undef QM_TILE_IF_1
#define QM_TILE_IF_1(...) QM_TILE_DEF(__VA_ARGS__)
#elif QM_TU == 2
#undef QM_TILE_IF_2
#define QM_TILE_IF_2(...) QM_TILE_DEF(__VA_ARGS__)
#elif QM_TU == 3
#undef QM_TILE_IF_3
#define QM_TILE_IF_3(...) QM_TILE_DEF(__VA_ARGS__)
#elif QM_TU == 4
#undef QM_TILE_IF_4
#define QM_TILE_IF_4(...) QM_TILE_DEF(__VA_ARGS__)
#elif QM_TU == 5
#undef QM_TILE_IF_5
#define QM_TILE_IF_5(...) QM_TILE_DEF(__VA_ARGS__)
#elif QM_TU == 6
#undef QM_TILE_IF_6
#define QM_TILE_IF_6(...) QM_TILE_DEF(__VA_ARGS__)
#elif QM_TU == 7
#undef QM_TILE_IF_7
#define QM_TILE_IF_7(...) QM_TILE_DEF(__VA_ARGS__)
#else
#error "QM_TU out of range"
#endif
#define QM_TILE(tu, ...) QM_TILE_IF_##tu(__VA_ARGS__)
#include "qm_configs.inc"

}  // namespace qm
