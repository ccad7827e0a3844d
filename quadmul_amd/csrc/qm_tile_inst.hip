// Instantiates the tile kernels assigned to translation unit QM_TU (see
// qm_configs.inc); compiled once per unit so the build runs in parallel.
#include "qm_launch.hpp"
#include "qm_tile16.hpp"

#ifndef QM_TU
#error "compile with -DQM_TU=<n>"
#endif

namespace qm {

// opt: tile raster group height in bits 0..7, the K split in bits 8..15 (the caller has
// zero-filled C, or given the kernel a workspace, when it is above 1), in bit 16 "one
// work item per workgroup", and in bit 17 "prepare only" (qm_init: the kernel's one-off
// set-up on this device, no launch).  By
// default the grid is persistent: as many workgroups as the device holds at once, each
// running several (K split, tile) items back to back.
// (OUT is a template parameter so that every kernel gets launcher statics of its own.)
// (... and TAIL: the kernel for K % 128 != 0 is another kernel with statics of its own)
template <class Cfg, int OUT, bool TAIL, class Kernel>
static hipError_t launch_tiled_persistent(Kernel kernel, const GemmArgs &p, hipStream_t stream, int opt)
{
    static std::atomic<bool> lds_ok[QM_MAX_DEVICES] = {};
    static std::atomic<int> resident[QM_MAX_DEVICES] = {};  // workgroups the device holds at once (0: not asked yet)
    hipError_t e = ensure_dynamic_lds(kernel, Cfg::LDS_BYTES, lds_ok);
    if (e != hipSuccess) return e;
    int dev = 0;
    e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= QM_MAX_DEVICES) return hipErrorInvalidDevice;
    int held = resident[dev].load(std::memory_order_acquire);
    if (held == 0) {
        int per_cu = 0, cus = 0;
        e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, Cfg::THREADS, Cfg::LDS_BYTES);
        if (e != hipSuccess) return e;
        e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) return e;
        if (per_cu < 1) per_cu = 1;
        // a multiple of 8, so that an item index modulo 8 names the XCD it runs on
        int g = per_cu * cus / 8 * 8;
        held = g < 8 ? 8 : g;
        resident[dev].store(held, std::memory_order_release);
    }
    if (opt & QM_OPT_PREPARE) return hipSuccess;  // the one-off set-up above was all that was asked for
    const int tiles_m = (p.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (p.N + Cfg::BN - 1) / Cfg::BN;
    int group_m = opt & 0xFF, ksplit = (opt >> 8) & 0xFF;
    if (group_m < 1) group_m = 1;
    if (group_m > tiles_m) group_m = tiles_m;
    ksplit = normalised_ksplit(p.K, ksplit);
    const long long items = (long long)tiles_m * tiles_n * ksplit;
    if (items > 0x7FFFFFFF) return hipErrorInvalidValue;
    int grid = (int)items;
    if (!(opt & 0x10000) && grid > held) grid = held;
    kernel<<<dim3(grid), dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream>>>(p, tiles_m, tiles_n, group_m, ksplit);
    return hipGetLastError();
}

}  // namespace qm

#define QM_TILE16_DEF(BM, BN, WGM, WGN, ST, OCC)                                                 \
    namespace qm {                                                                               \
    hipError_t QM_TILE16_FN(BM, BN, WGM, WGN, ST, OCC)(const GemmArgs &p, hipStream_t s, int gm) \
    {                                                                                            \
        using Cfg = Tile16Cfg<BM, BN, WGM, WGN, ST, OCC>;                                        \
        if (p.K % 128) return launch_tiled_persistent<Cfg, OUT_I32, true>(&gemm_tile16_kernel<Cfg, OUT_I32, true>, p, s, gm); \
        return launch_tiled_persistent<Cfg, OUT_I32, false>(&gemm_tile16_kernel<Cfg, OUT_I32, false>, p, s, gm);  \
    }                                                                                            \
    }
// the same configuration with the scaled 16-bit float outputs
#define QM_TILE16S_DEF(BM, BN, WGM, WGN, ST, OCC)                                                 \
    namespace qm {                                                                                \
    hipError_t QM_TILE16S_FN(BM, BN, WGM, WGN, ST, OCC)(const GemmArgs &p, hipStream_t s, int gm) \
    {                                                                                             \
        using Cfg = Tile16Cfg<BM, BN, WGM, WGN, ST, OCC>;                                         \
        if (p.K % 128) {                                                                            \
            if (p.out == OUT_F16) return launch_tiled_persistent<Cfg, OUT_F16, true>(&gemm_tile16_kernel<Cfg, OUT_F16, true>, p, s, gm); \
            return launch_tiled_persistent<Cfg, OUT_BF16, true>(&gemm_tile16_kernel<Cfg, OUT_BF16, true>, p, s, gm); \
        }                                                                                           \
        if (p.out == OUT_F16) return launch_tiled_persistent<Cfg, OUT_F16, false>(&gemm_tile16_kernel<Cfg, OUT_F16, false>, p, s, gm); \
        return launch_tiled_persistent<Cfg, OUT_BF16, false>(&gemm_tile16_kernel<Cfg, OUT_BF16, false>, p, s, gm); \
    }                                                                                             \
    }

// An entry of qm_configs.inc is compiled here only when its unit number equals QM_TU:
// QM_PICK*_<n> expands to nothing except for n == QM_TU.
#define QM_PICK16_0(...)
#define QM_PICK16_1(...)
#define QM_PICK16_2(...)
#define QM_PICK16_3(...)
#define QM_PICK16_4(...)
#define QM_PICK16_5(...)
#define QM_PICK16_6(...)
#define QM_PICK16_7(...)
#define QM_PICK16_8(...)
#define QM_PICK16_9(...)
#define QM_PICK16_10(...)
#define QM_PICK16_11(...)
#define QM_PICK16_12(...)
#define QM_PICK16_13(...)
#define QM_PICK16S_0(...)
#define QM_PICK16S_1(...)
#define QM_PICK16S_2(...)
#define QM_PICK16S_3(...)
#define QM_PICK16S_4(...)
#define QM_PICK16S_5(...)
#define QM_PICK16S_6(...)
#define QM_PICK16S_7(...)
#define QM_PICK16S_8(...)
#define QM_PICK16S_9(...)
#define QM_PICK16S_10(...)
#define QM_PICK16S_11(...)
#define QM_PICK16S_12(...)
#define QM_PICK16S_13(...)
#if QM_TU == 0
#undef QM_PICK16_0
#define QM_PICK16_0(...) QM_TILE16_DEF(__VA_ARGS__)
#undef QM_PICK16S_0
#define QM_PICK16S_0(...) QM_TILE16S_DEF(__VA_ARGS__)
#elif QM_TU == 1
#undef QM_PICK16_1
#define QM_PICK16_1(...) QM_TILE16_DEF(__VA_ARGS__)
#undef QM_PICK16S_1
#define QM_PICK16S_1(...) QM_TILE16S_DEF(__VA_ARGS__)
#elif QM_TU == 2
#undef QM_PICK16_2
#define QM_PICK16_2(...) QM_TILE16_DEF(__VA_ARGS__)
#undef QM_PICK16S_2
#define QM_PICK16S_2(...) QM_TILE16S_DEF(__VA_ARGS__)
#elif QM_TU == 3
#undef QM_PICK16_3
#define QM_PICK16_3(...) QM_TILE16_DEF(__VA_ARGS__)
#undef QM_PICK16S_3
#define QM_PICK16S_3(...) QM_TILE16S_DEF(__VA_ARGS__)
#elif QM_TU == 4
#undef QM_PICK16_4
#define QM_PICK16_4(...) QM_TILE16_DEF(__VA_ARGS__)
#undef QM_PICK16S_4
#define QM_PICK16S_4(...) QM_TILE16S_DEF(__VA_ARGS__)
#elif QM_TU == 5
#undef QM_PICK16_5
#define QM_PICK16_5(...) QM_TILE16_DEF(__VA_ARGS__)
#undef QM_PICK16S_5
#define QM_PICK16S_5(...) QM_TILE16S_DEF(__VA_ARGS__)
#elif QM_TU == 6
#undef QM_PICK16_6
#define QM_PICK16_6(...) QM_TILE16_DEF(__VA_ARGS__)
#undef QM_PICK16S_6
#define QM_PICK16S_6(...) QM_TILE16S_DEF(__VA_ARGS__)
#elif QM_TU == 7
#undef QM_PICK16_7
#define QM_PICK16_7(...) QM_TILE16_DEF(__VA_ARGS__)
#undef QM_PICK16S_7
#define QM_PICK16S_7(...) QM_TILE16S_DEF(__VA_ARGS__)
#elif QM_TU == 8
#undef QM_PICK16_8
#define QM_PICK16_8(...) QM_TILE16_DEF(__VA_ARGS__)
#undef QM_PICK16S_8
#define QM_PICK16S_8(...) QM_TILE16S_DEF(__VA_ARGS__)
#elif QM_TU == 9
#undef QM_PICK16_9
#define QM_PICK16_9(...) QM_TILE16_DEF(__VA_ARGS__)
#undef QM_PICK16S_9
#define QM_PICK16S_9(...) QM_TILE16S_DEF(__VA_ARGS__)
#elif QM_TU == 10
#undef QM_PICK16_10
#define QM_PICK16_10(...) QM_TILE16_DEF(__VA_ARGS__)
#undef QM_PICK16S_10
#define QM_PICK16S_10(...) QM_TILE16S_DEF(__VA_ARGS__)
#elif QM_TU == 11
#undef QM_PICK16_11
#define QM_PICK16_11(...) QM_TILE16_DEF(__VA_ARGS__)
#undef QM_PICK16S_11
#define QM_PICK16S_11(...) QM_TILE16S_DEF(__VA_ARGS__)
#elif QM_TU == 12
#undef QM_PICK16_12
#define QM_PICK16_12(...) QM_TILE16_DEF(__VA_ARGS__)
#undef QM_PICK16S_12
#define QM_PICK16S_12(...) QM_TILE16S_DEF(__VA_ARGS__)
#elif QM_TU == 13
#undef QM_PICK16_13
#define QM_PICK16_13(...) QM_TILE16_DEF(__VA_ARGS__)
#undef QM_PICK16S_13
#define QM_PICK16S_13(...) QM_TILE16S_DEF(__VA_ARGS__)
#else
#error "QM_TU out of range"
#endif

#define QM_TILE16(tu, ...) QM_PICK16_##tu(__VA_ARGS__)
#define QM_TILE16S(tu, ...) QM_PICK16S_##tu(__VA_ARGS__)
#include "qm_configs.inc"
