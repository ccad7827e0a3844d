// Configuration registry and the choice of a configuration for a shape: the measured
// per-shape table (qm_tile_table.inc, written by the autotuner) and, for every other shape,
// a cost model.  Takes the place of the reference's exact-(m, n, k) dispatch over its
// KernelConfig table (kernel.cu:321-385, configs.cu:19-689), which skips unknown shapes.
// Included by qm_dispatch.hip only, after the launchers of the skinny and dot kernels.
#pragma once
#include <cstring>

#include "qm_launch.hpp"

namespace qm {

// --------------------------------------------------------------------------
// Configuration registry
// --------------------------------------------------------------------------
enum Kind { KIND_GENERIC = 0, KIND_SKINNY = 2, KIND_TILE16 = 3 };

struct ConfigDesc {
    const char *name;
    int kind;
    int bm, bn, bk;  // tile: block shape; skinny: bm = rows, bn = columns per workgroup (bm is the most M takes, without row_blocks)
    int waves, mode;
    LaunchFn launch;
    int wgm = 0, wgn = 0;  // pipelined kernel: waves down and across the tile
    int max_k = 0;         // skinny kernels whose waves hold A in registers: the K they hold (0: any)
    bool row_blocks = false;  // skinny kernels whose grid walks over blocks of bm rows: any M
};

#define QM_STR2(x) #x
#define QM_STR(x) QM_STR2(x)
static const ConfigDesc g_configs[] = {
    {"generic", KIND_GENERIC, 16, 16, 128, 4, 0, &launch_generic},
#define QM_TILE16(tu, BM, BN, WGM, WGN, ST, OCC)                                                              \
    {"q" QM_STR(BM) "x" QM_STR(BN) "_w" QM_STR(WGM) "x" QM_STR(WGN) "_s" QM_STR(ST) "o" QM_STR(OCC), KIND_TILE16, BM, BN, 128, \
     (WGM) * (WGN), 0, &QM_TILE16_FN(BM, BN, WGM, WGN, ST, OCC), WGM, WGN},
#define QM_SKINNY(FM, FN, NW, U)                                                     \
    {"s" QM_STR(FM) "x" QM_STR(FN) "_w" QM_STR(NW) "_u" QM_STR(U), KIND_SKINNY, 16 * (FM), 16 * (FN), 128, NW, 0, \
     &QM_SKINNY_FN(FM, FN, NW, U)},
#define QM_SKINNYD(FM, FN, NW, D)                                                    \
    {"d" QM_STR(FM) "x" QM_STR(FN) "_w" QM_STR(NW) "_r" QM_STR(D), KIND_SKINNY, 16 * (FM), 16 * (FN), 128, NW, 0, \
     &QM_SKINNYD_FN(FM, FN, NW, D), 0, 0, 0, true},
#define QM_SKINNYP(FM, FN, NW, D, R)                                                 \
    {"p" QM_STR(FM) "x" QM_STR(FN) "_w" QM_STR(NW) "_r" QM_STR(D) "k" QM_STR(R), KIND_SKINNY, 16 * (FM), 16 * (FN), 128, NW, 0, \
     &QM_SKINNYP_FN(FM, FN, NW, D, R), 0, 0, 256 * (NW) * (R)},
#define QM_DOT(MR, FN, NW, U)                                                     \
    {"v" QM_STR(MR) "x" QM_STR(FN) "_w" QM_STR(NW) "_u" QM_STR(U), KIND_SKINNY, MR, 16 * (FN), 128, NW, 0, \
     &QM_DOT_FN(MR, FN, NW, U)},
#include "qm_configs.inc"
};
static constexpr int g_num_configs = (int)(sizeof(g_configs) / sizeof(g_configs[0]));

// Pipelined configurations that also exist with the scaled 16-bit float output
static const struct { const char *name; LaunchFn launch; } g_scaled_tile16[] = {
#define QM_TILE16S(tu, BM, BN, WGM, WGN, ST, OCC) \
    {"q" QM_STR(BM) "x" QM_STR(BN) "_w" QM_STR(WGM) "x" QM_STR(WGN) "_s" QM_STR(ST) "o" QM_STR(OCC), &QM_TILE16S_FN(BM, BN, WGM, WGN, ST, OCC)},
#include "qm_configs.inc"
};

// The launcher of configuration cfg for the scaled output, or null: the generic and the
// skinny kernels take the output form at run time, the pipelined ones as separate kernels
// (not every configuration has them).
static LaunchFn scaled_launcher(int cfg)
{
    const ConfigDesc &c = g_configs[cfg];
    if (c.kind == KIND_GENERIC || c.kind == KIND_SKINNY) return c.launch;
    if (c.kind == KIND_TILE16)
        for (const auto &e : g_scaled_tile16)
            if (std::strcmp(e.name, c.name) == 0) return e.launch;
    return nullptr;
}

static int find_config(const char *name)
{
    for (int i = 0; i < g_num_configs; ++i)
        if (std::strcmp(g_configs[i].name, name) == 0) return i;
    return -1;
}

// The 16-byte-load kernels need whole, aligned chunks and 32-bit row offsets,
// and the x16 widening bounds K.
static bool fast_path_ok(int m, int n, int k, int ptr_align)
{
    if (k % 32 != 0 || k > QM_MAX_K_X16 || ptr_align < 16) return false;
    const long long kb = k / 2;
    return (long long)m * kb < 0x7fffffffLL && (long long)n * kb < 0x7fffffffLL;
}

static bool config_supports(int cfg, int m, int n, int k, int ptr_align)
{
    if (cfg < 0 || cfg >= g_num_configs || m < 1 || n < 1 || k < 2 || (k & 1)) return false;
    const ConfigDesc &c = g_configs[cfg];
    if (c.kind == KIND_GENERIC) return true;
    if (!fast_path_ok(m, n, k, ptr_align)) return false;
    // (the skinny kernels address rows through 24-bit multiplies: rows and bytes per row below 2^24)
    if (c.kind == KIND_SKINNY)
        return (m <= c.bm || (c.row_blocks && m <= 65535 * c.bm)) && (c.max_k == 0 || k <= c.max_k) && m < (1 << 24) && n < (1 << 24) && k / 2 < (1 << 24);
    if (c.kind == KIND_TILE16) return k % 128 == 0 || k > 128;  // a short last K-step needs a step before it
    return true;
}

// --------------------------------------------------------------------------
// Shape table (autotuned on MI355X; regenerated by quadmul_amd/autotune.py) with
// a cost-model fallback -- the reference instead skips unknown shapes.
// --------------------------------------------------------------------------
struct TableEntry {
    int m, n, k;
    const char *config;
    int group_m, ksplit;
    int spread;  // 1: one work item per workgroup instead of a persistent grid (pipelined kernel)
    // rows whose choice splits K through a workspace: the measured choice for calls that have
    // none (the bare seven-argument entry point), never split
    const char *nows_config = nullptr;
    int nows_group_m = 0;
};
static const TableEntry g_table[] = {
#include "qm_tile_table.inc"
    {0, 0, 0, nullptr, 0, 0},
};

struct Choice {
    int cfg, group_m, ksplit;
    int spread = 0;
};

static Choice heuristic(int m, int n, int k, int ptr_align, bool has_ws)
{
    if (!fast_path_ok(m, n, k, ptr_align)) return {0, 1, 1};
    // Up to 64 rows: chosen on measurements with B streamed from HBM (launches rotating over
    // copies of B), M = 1 .. 64, N = 2048 .. 28672, K = 2048 .. 14336.
    const auto pick = [](const char *name) { const int id = find_config(name); return Choice{id >= 0 ? id : 0, 1, 1}; };
    const bool skinny_ok = m < (1 << 24) && n < (1 << 24);  // (their 24-bit row arithmetic, see config_supports)
    if (!skinny_ok) goto tiles;
    if (m <= 2) {
        // no matrix core: v_dot8_i32_i4 on the packed bytes as they are
        if (m == 1) return pick(k <= 2048 ? "v1x1_w8_u4" : (k <= 4096 ? "v1x1_w4_u8" : "v1x1_w16_u2"));
        return pick(k <= 4096 ? "v2x1_w8_u4" : "v2x1_w16_u2");
    }
    if (m <= 16) {
        // operands streamed global -> LDS; with A resident in registers and a persistent grid
        // while the waves hold all of K
        if (k <= 4096) return pick(k > 2048 || n >= 8192 ? "p1x1_w8_r2k2" : "d1x1_w16_r1");
        if (k <= 8192 && n >= 8192) return pick("p1x1_w16_r2k2");
        return pick("d1x1_w16_r1");
    }
    if (m <= 32) {
        if (k <= 2048) return pick("p2x1_w16_r2k1");
        // few column blocks and a long K: two blocks of 16 rows each double the workgroups
        if (n <= 2048) return pick("d1x1_w16_r1");
        if (k <= 4096) return pick("p2x1_w8_r2k2");
        // a long K: every workgroup re-reads the rows of A it owns over all of K; 32 columns
        // per workgroup halve that against 16
        return pick(n <= 4096 ? "d2x1_w16_r1" : "d2x2_w8_r1");
    }
    if (m > 32 && m <= 1024 && k >= 1024 && k <= 32768) {
        // From 33 to a thousand rows on few columns: blocks of 64 x 64 or 64 x 32 of the same
        // kernel when that makes one round of workgroups that fills most of the device (eight
        // waves, one workgroup per CU), or up to two rounds of 64 x 64 blocks on four waves,
        // two workgroups to a CU -- a workgroup pulls (rows + columns) x K / 2 bytes through its
        // L1 for rows x columns x K multiply-adds, so the larger block moves half as much per
        // product.  Measured with B from HBM, M = 40 .. 1024, N = 1024 .. 32768, K = 1024 .. 28672,
        // against the tiles and the 32 x 32 blocks: 128 x 8192 x 8192 15.4 us (64 x 64 tiles:
        // 19.1), 256 x 4096 x 8192 14.5 (18.8), 512 x 2048 x 4096 8.7 (11.3), 128 x 4096 x 8192
        // 9.6 on 64 x 32 (32 x 32: 11.1), 64 x 8192 x 4096 6.5 on 64 x 32 (32 x 32: 7.5); in two
        // rounds 256 x 8192 x 8192 23.1 (128 x 64 tiles: 25.3), 512 x 4096 x 4096 13.5 (15.1).
        // Beyond two rounds the tiles win, and on a K this long they win with a workspace to
        // split it through.
        const long long r64 = (m + 63) / 64, c64 = (n + 63) / 64, c32 = (n + 31) / 32, r32 = (m + 31) / 32;
        if (r64 * c64 >= 140 && r64 * c64 <= 256) return pick("d4x4_w8_r1");
        if (r64 * c64 > 256 && r64 * c64 <= 512 && (k <= 16384 || !has_ws)) return pick("d4x4_w4_r1");
        if (r64 * c32 >= 140 && r64 * c32 <= 256) return pick("d4x2_w8_r1");
        if (r32 * c64 >= 140 && r32 * c64 <= 256) return pick("d2x4_w8_r1");
    }
    if (m <= 64) {
        // blocks of 32 rows: 32 x 16 per workgroup while that leaves one workgroup per CU,
        // 32 x 32 (two to a CU) up to about three rounds of them, tiles beyond
        if (n <= 2048) return pick("d2x1_w16_r1");
        if (n <= 12288) return pick("d2x2_w8_r1");
        if (n <= 16384 && config_supports(find_config("q64x64_w2x2_s8o2"), m, n, k, ptr_align)) return pick("q64x64_w2x2_s8o2");
    }
    if (k < 128) {
        // A K of one short step (32, 64 or 96) is nothing for the pipelined kernel: it has no
        // earlier step to overlap that one with.  The 32 x 32 blocks take any number of rows;
        // one wave per workgroup when there are thousands of them (only one wave has a run of
        // K to work on).  Measured: 2048 x 4096 x 96 13.0 us (eight waves: 27.7; the generic
        // kernel: 114; on zero-padded copies in a workspace: 11.9), 8192 x 8192 x 96 66 us (875; 56).
        const long long wgs = (long long)((m + 31) / 32) * ((n + 31) / 32);
        return pick(wgs > 1024 ? "d2x2_w1_r1" : "d2x2_w8_r1");
    }
    if (m <= 256 && k <= 16384) {
        // The same 32 x 32 blocks on a few hundred rows (measured with B from HBM, M = 65 .. 256,
        // N = 2048 .. 11008, K = 2048 .. 8192): ahead of the tiles -- no ring to fill, one
        // workgroup per 32 x 32 block of C over all of K -- up to about three rounds of
        // workgroups (two to a CU), e.g. 128 x 4096 x 8192 11.4 us against 17.3, 192 x 4096 x 4096
        // 9.7 against 11.1; level with the 64 x 64 tiles at four rounds, behind them beyond.
        const long long wgs = (long long)((m + 31) / 32) * ((n + 31) / 32);
        if (wgs <= 800 || (wgs <= 1040 && m <= 96)) return pick("d2x2_w8_r1");
    }
tiles:
    // Tiles: minimise (rounds of 256 workgroups) x (tile area / relative efficiency),
    // over the configurations that can run this K.  Efficiencies are measured ratios.
    // eff: throughput per tile area relative to the 256 x 256 tile with the GPU full (measured)
    static const struct { const char *name; double eff; } cands[] = {
        {"q256x256_w2x2_s9o1", 1.00}, {"q256x128_w2x2_s9o1", 0.82}, {"q128x256_w2x2_s9o1", 0.82}, {"q128x128_w2x2_s9o1", 0.60},
        {"q128x64_w2x2_s6o2", 0.46},  {"q64x128_w2x2_s6o2", 0.44},  {"q64x64_w2x2_s8o2", 0.37},
    };
    int best = 0, best_ks = 1;
    double best_cost = 1e300;
    for (const auto &c : cands) {
        const int id = find_config(c.name);
        if (id < 0 || !config_supports(id, m, n, k, ptr_align)) continue;
        const ConfigDesc &d = g_configs[id];
        const long long tiles = (long long)((m + d.bm - 1) / d.bm) * ((n + d.bn - 1) / d.bn);
        // Few tiles and a long K: the pipelined kernel can split K over several workgroups
        // per tile.  With a workspace the partial sums cost a second kernel (about 8 us all
        // told, measured); without one they meet in C through 4-byte atomics, which are slow
        // enough that splitting only pays when each split keeps a long K of its own
        // (measured: wins at K = 28672, loses at K = 8192).
        // Cost in units of 16.5 ps (one K-step of the 256 x 256 tile = 65536): K-steps per
        // item x tile area / efficiency, plus 4 us per round of workgroups for filling the
        // ring and writing out, plus the split's own cost.
        const int kt = (k + 127) / 128;
        auto cost_of = [&](int ks_) {
            const double rounds = (double)((tiles * ks_ + 255) / 256);
            return rounds * ((double)((kt + ks_ - 1) / ks_) * d.bm * d.bn / c.eff + 240000.0) + (ks_ > 1 ? 480000.0 + 0.04 * ks_ * tiles * d.bm * d.bn : 0.0);  // (+ the partial tiles, written and read back at about 6 TB/s)
        };
        int ks = 1;
        double cost = cost_of(1);
        if (d.kind == KIND_TILE16 && has_ws) {
            for (int t = 2; t <= 16 && tiles * t <= 256 && kt / t >= 4; ++t)
                if (cost_of(t) < cost) { cost = cost_of(t); ks = t; }
        } else if (d.kind == KIND_TILE16) {
            // (no workspace: the split is kept only where it is priced below the unsplit launch)
            int t = 1;
            while (t < 4 && tiles * t * 2 <= 256 && (k / 128) / (t * 2) >= 48) t *= 2;
            if (t > 1) {
                // (+ one 4-byte atomic per element and split at about 10 ps each, 0.6 units --
                // measured: 512 x 8192 x 28672 in four splits 253 us, 170 of them the atomics)
                const double split_cost = (double)d.bm * d.bn / c.eff * ((kt + t - 1) / t) * 1.25 + 180000.0 + 0.6 * (double)m * (double)n * t;
                if (split_cost < cost) { cost = split_cost; ks = t; }
            }
        }
        if (cost < best_cost) { best_cost = cost; best = id; best_ks = ks; }
    }
    if (m <= 128 && skinny_ok) {
        // The wave-level split-K kernel has no ring to fill and no second kernel, and wins
        // while N x K is small.  Measured, in the units above: about 2 us plus, per million
        // elements of B, 0.24 us with four row blocks (33..64 rows, B from HBM) and 0.38 us
        // with eight (65..128 rows).
        const char *name = m > 64 ? "s8x1_w8_u1" : (n >= 8192 ? (k >= 8192 ? "s4x1_w8_u2" : "s4x1_w16_u2") : (k >= 8192 ? "s4x1_w16_u2" : "s4x1_w16_u1"));
        const int id = find_config(name);
        const double cost_s = (2.0 + (double)n * (double)k / (m > 64 ? 2.6e6 : 4.2e6)) / 1.65e-5;
        if (id >= 0 && cost_s < best_cost) return {id, 1, 1};
    }
    const int ksplit = best_ks;
    return {best, 4, ksplit};
}

static Choice select_config(int m, int n, int k, int ptr_align, bool has_ws)
{
    static int resolved[sizeof(g_table) / sizeof(g_table[0])], resolved_nows[sizeof(g_table) / sizeof(g_table[0])];
    static std::once_flag once;
    std::call_once(once, [] {
        for (size_t i = 0; g_table[i].config; ++i) {
            resolved[i] = find_config(g_table[i].config);
            resolved_nows[i] = g_table[i].nows_config ? find_config(g_table[i].nows_config) : -1;
        }
    });
    for (size_t i = 0; g_table[i].config; ++i)
        if (g_table[i].m == m && g_table[i].n == n && g_table[i].k == k && resolved[i] >= 0 &&
            config_supports(resolved[i], m, n, k, ptr_align)) {
            // The table's K splits were measured through the workspace (partial tiles, then the
            // kernel that adds them up).  Without one the row's second choice runs, measured
            // without a workspace; where a row has none, the cost model decides.
            if (g_table[i].ksplit > 1 && !has_ws) {
                if (resolved_nows[i] >= 0 && config_supports(resolved_nows[i], m, n, k, ptr_align))
                    return {resolved_nows[i], g_table[i].nows_group_m > 0 ? g_table[i].nows_group_m : 4, 1, 0};
                break;
            }
            return {resolved[i], g_table[i].group_m, g_table[i].ksplit > 0 ? g_table[i].ksplit : 1, g_table[i].spread};
        }
    return heuristic(m, n, k, ptr_align, has_ws);
}

// The scaled output has fewer kernels to choose from: the table's choice when that
// configuration has the output form, else the best pipelined one that has it, else what the
// heuristic says for skinny shapes, else the generic kernel.
static Choice select_scaled(int m, int n, int k, int ptr_align, bool has_ws)
{
    const Choice ch = select_config(m, n, k, ptr_align, has_ws);
    if (ch.ksplit <= 1 && scaled_launcher(ch.cfg)) return ch;
    // K split: the int32 kernel of any pipelined configuration leaves partial sums in the
    // workspace, and the kernel that adds them up scales and rounds
    if (ch.ksplit > 1 && has_ws && g_configs[ch.cfg].kind == KIND_TILE16) return ch;
    if (fast_path_ok(m, n, k, ptr_align)) {
        int best = -1;
        double best_cost = 1e300;
        for (const auto &e : g_scaled_tile16) {
            const int id = find_config(e.name);
            if (id < 0 || !config_supports(id, m, n, k, ptr_align)) continue;
            const ConfigDesc &d = g_configs[id];
            const long long tiles = (long long)((m + d.bm - 1) / d.bm) * ((n + d.bn - 1) / d.bn);
            const int area = d.bm * d.bn;
            const double eff = area >= 256 * 256 ? 1.0 : (area >= 256 * 128 ? 0.82 : (area >= 128 * 128 ? 0.60 : (area >= 128 * 64 ? 0.45 : 0.37)));
            const double cost = (double)((tiles + 255) / 256) * ((double)((k + 127) / 128) * area / eff + 240000.0);  // as in heuristic()
            if (cost < best_cost) { best_cost = cost; best = id; }
        }
        if (best >= 0) return {best, 4, 1};
    }
    const Choice h = heuristic(m, n, k, ptr_align, false);
    if (h.ksplit <= 1 && scaled_launcher(h.cfg)) return h;
    return {0, 1, 1};
}

}  // namespace qm
