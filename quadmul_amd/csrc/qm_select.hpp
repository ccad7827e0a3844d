// Configuration registry and the choice of a configuration for a shape: the measured
// per-shape table (qm_tile_table.inc, written by the autotuner) and, for every other shape,
// a cost model.  Takes the place of the reference's exact-(m, n, k) dispatch over its
// KernelConfig table (kernel.cu:321-385, configs.cu:19-689), which skips unknown shapes.
// Included by qm_dispatch.hip only, after the launchers of the skinny and dot kernels.
#pragma once
#include <cmath>
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

// --------------------------------------------------------------------------
// Fitted cost model (qm_cost_model.inc, written by quadmul_amd/cost_model.py from timings of
// every candidate on a few hundred random shapes).  A configuration works on items of bm x bn
// elements of C -- tiles of the pipelined kernel, blocks of the wave-level one -- `slots` of
// them at a time:
//     items  = ceil(M / bm) * ceil(N / bn) * ksplit
//     rounds = blend * ceil(items / slots) + (1 - blend) * max(1, items / slots)
//     fill   = min(1, items / slots),  ksteps = ceil(ceil(K / 128) / ksplit)
//     us     = ksteps * (rounds * step_us + fill * busy_us) + rounds * round_us + launch_us
//              + (K % 256 != 0:  ksteps * rounds * skew_us)
//              + (N % 4 != 0, ksplit == 1:  rounds * odd_us)
//              + (pipelined kernel, N % 4 == 0, ksplit == 1:  max(1, items sticking out of C / slots) * ragged_us)
//              + (wave-level kernel, N * K / 2 > 32 MB, items > slots:  (ceil(M / bm) - 1) * N * K / 2e6 * reread_us)
//              + (ksplit > 1:  split_us + split_us_per_melem * ksplit * M * N / 1e6)
// blend = 1: a partly filled last round costs as much as a full one (one workgroup per CU);
// towards 0: in proportion (several small workgroups per CU: the ones left speed up).
// busy_us: what a K-step slows down by as the device fills up (shared L2s, fabric, power).
// odd_us: rows of C that are not 16-byte aligned -- the pipelined kernel then writes every
// tile after its last K-step.  ragged_us: tiles that stick out of C are written through
// guarded stores.  reread_us: per megabyte of B that the second and later blocks of rows of
// the wave-level kernel read again after the L2s (32 MB between them) have lost it.
// skew_us: rows of A and B that are not whole 128-byte lines -- every 128-byte run of a row
// then lies across two cache lines.
// --------------------------------------------------------------------------
struct CostFit {
    const char *name;
    int slots;
    float blend, step_us, busy_us, round_us, odd_us, ragged_us, reread_us, skew_us, launch_us;
};
static const CostFit g_cost_fits[] = {
#define QM_COST(name, slots, blend, step, busy, round, odd, ragged, reread, skew, launch) {name, slots, blend, step, busy, round, odd, ragged, reread, skew, launch},
#define QM_COST_SPLIT(fixed, per_melem)
#include "qm_cost_model.inc"
#undef QM_COST
#undef QM_COST_SPLIT
};
static const float g_cost_split[2] = {
#define QM_COST(name, slots, blend, step, busy, round, odd, ragged, reread, skew, launch)
#define QM_COST_SPLIT(fixed, per_melem) fixed, per_melem
#include "qm_cost_model.inc"
#undef QM_COST
#undef QM_COST_SPLIT
};

static double modelled_us(const CostFit &f, const ConfigDesc &d, int m, int n, int k, int ks)
{
    const long long rows = (m + d.bm - 1) / d.bm, cols = (n + d.bn - 1) / d.bn;
    const double items = (double)rows * (double)cols * ks;
    const double share = items / f.slots;
    const double rounds = f.blend * std::ceil(share) + (1.0 - f.blend) * (share > 1.0 ? share : 1.0);
    const double ksteps = (double)(((k + 127) / 128 + ks - 1) / ks);
    double us = ksteps * (rounds * f.step_us + (share < 1.0 ? share : 1.0) * f.busy_us) + rounds * f.round_us + f.launch_us;
    if (k & 255) us += ksteps * rounds * f.skew_us;
    if (ks == 1 && (n & 3)) us += rounds * f.odd_us;
    if (ks == 1 && !(n & 3) && d.kind == KIND_TILE16) {
        const double sticking_out = (double)(rows * cols - (long long)(m / d.bm) * (n / d.bn));
        if (sticking_out > 0) us += (sticking_out > f.slots ? sticking_out / f.slots : 1.0) * f.ragged_us;
    }
    if (d.kind == KIND_SKINNY && (double)n * k / 2 > 32e6 && items > f.slots) us += (double)(rows - 1) * n * k / 2e6 * f.reread_us;
    if (ks > 1) us += g_cost_split[0] + g_cost_split[1] * 1e-6 * ks * (double)m * (double)n;
    return us;
}

// The cheapest candidate by the model.  `scaled`: the 16-bit float output, which not every
// pipelined configuration has a kernel for (a K split through the workspace always does: the
// kernel that adds the partial sums up scales and rounds).
static Choice modelled_choice(int m, int n, int k, int ptr_align, bool has_ws, bool scaled)
{
    Choice best{0, 1, 1};
    double best_us = 1e300;
    const int kt = (k + 127) / 128;
    for (const CostFit &f : g_cost_fits) {
        const int id = find_config(f.name);
        if (id < 0 || !config_supports(id, m, n, k, ptr_align)) continue;
        const ConfigDesc &d = g_configs[id];
        const bool tile = d.kind == KIND_TILE16;
        const auto offer = [&](double us, int ks) {
            if (us < best_us) { best_us = us; best = Choice{id, tile ? 4 : 1, ks}; }
        };
        if (!scaled || scaled_launcher(id)) offer(modelled_us(f, d, m, n, k, 1), 1);
        if (!tile) continue;
        // Few tiles and a long K: the pipelined kernel can split K over several workgroups per
        // tile (the splits the autotuner times).
        const long long tiles = (long long)((m + d.bm - 1) / d.bm) * ((n + d.bn - 1) / d.bn);
        if (has_ws) {
            static const int splits[] = {2, 3, 4, 6, 8, 12, 16};
            for (int ks : splits)
                if (tiles <= 256 && tiles * ks <= 1024 && kt / ks >= 4) offer(modelled_us(f, d, m, n, k, ks), ks);
        } else if (!scaled) {
            // No workspace: the partial sums meet in C through 4-byte atomics, which are slow
            // enough that splitting only pays when each split keeps a long K of its own
            // (measured: wins at K = 28672, loses at K = 8192): + a quarter on the K-steps, 3 us
            // and about 10 ps per element and split (512 x 8192 x 28672 in four splits 253 us,
            // 170 of them the atomics).
            int t = 1;
            while (t < 4 && tiles * t * 2 <= 256 && (k / 128) / (t * 2) >= 48) t *= 2;
            if (t > 1) offer((double)((kt + t - 1) / t) * (f.step_us + f.busy_us) * 1.25 + f.round_us + f.launch_us + 3.0 + 9.9e-6 * (double)m * (double)n * t, t);
        }
    }
    return best;
}

static Choice heuristic(int m, int n, int k, int ptr_align, bool has_ws)
{
    if (!fast_path_ok(m, n, k, ptr_align)) return {0, 1, 1};
    // Up to 64 rows: chosen on measurements with B streamed from HBM (launches rotating over
    // copies of B), M = 1 .. 64, N = 2048 .. 57344, K = 2048 .. 28672.
    const auto pick = [](const char *name) { const int id = find_config(name); return Choice{id >= 0 ? id : 0, 1, 1}; };
    const bool skinny_ok = m < (1 << 24) && n < (1 << 24);  // (their 24-bit row arithmetic, see config_supports)
    if (!skinny_ok) goto tiles;
    if (m <= 2) {
        // The persistent kernel of the rows above, sixteen waves holding a K of 8192 between
        // them, is ahead of the dot kernel on that K and many columns even with one row
        // (1 x 8192 x 8192 7.0 us against 7.8, 1 x 10240 x 8192 8.3 against 9.2, 1 x 57344 x 8192 36.2
        // against 37.5).
        if (k > 4096 && k <= 8192 && n >= 8192) return pick("p1x1_w16_r2k2");
        // no matrix core: v_dot8_i32_i4 on the packed bytes as they are (four waves of eight
        // chunk pairs again on a very long K: 1 x 8192 x 28672 17.9 us against 19.1)
        if (m == 1) return pick(k <= 2048 ? "v1x1_w8_u4" : (k <= 4096 || k > 16384 ? "v1x1_w4_u8" : "v1x1_w16_u2"));
        return pick(k <= 4096 ? "v2x1_w8_u4" : "v2x1_w16_u2");
    }
    if (m <= 16) {
        // operands streamed global -> LDS; with A resident in registers and a persistent grid
        // while the waves hold all of K
        if (k <= 4096) return pick(k > 2048 || n >= 8192 ? "p1x1_w8_r2k2" : "d1x1_w16_r1");
        if (k <= 8192 && n >= 8192) return pick("p1x1_w16_r2k2");
        // a very long K: every workgroup re-reads A over all of it; 32 columns per workgroup
        // halve that (16 x 8192 x 28672 19.1 us against 21.7)
        if (k > 16384) return pick("d1x2_w8_r2");
        return pick("d1x1_w16_r1");
    }
    if (m <= 32) {
        // tens of thousands of columns on a long K: one wave per workgroup, thousands of them
        // (32 x 57344 x 8192 39.9 us against 49.2 on eight waves)
        if (k > 4096 && n >= 32768) return pick("d2x2_w1_r1");
        if (k <= 2048) return pick("p2x1_w16_r2k1");
        // few column blocks and a long K: two blocks of 16 rows each double the workgroups
        if (n <= 2048) return pick("d1x1_w16_r1");
        if (k <= 4096) return pick("p2x1_w8_r2k2");
        // a long K: every workgroup re-reads the rows of A it owns over all of K; 32 columns
        // per workgroup halve that against 16
        return pick(n <= 4096 ? "d2x1_w16_r1" : "d2x2_w8_r1");
    }
    if (m <= 64 && k >= 1024) {
        // 33 to 64 rows (measured with B from HBM, M = 40 and 64, N = 1024 .. 32768, K = 1024 ..
        // 28672): blocks of 64 x 64 or 64 x 32 of the same kernel when that makes one round of
        // workgroups that fills most of the device (eight waves, one workgroup per CU) -- a
        // workgroup pulls (rows + columns) x K / 2 bytes through its L1 for rows x columns x K
        // multiply-adds, so the larger block moves half as much per product: 64 x 8192 x 4096
        // 6.5 us on 64 x 32 (32 x 32: 7.5) -- else blocks of 32 rows: 32 x 16 per workgroup while
        // that leaves one workgroup per CU, 32 x 32 (two to a CU) up to about three rounds.
        const long long c64 = (n + 63) / 64, c32 = (n + 31) / 32;
        if (k <= 32768) {
            if (c64 >= 140 && c64 <= 256) return pick("d4x4_w8_r1");
            if (c64 > 256 && c64 <= 512 && (k <= 16384 || !has_ws)) return pick("d4x4_w4_r1");
            if (c32 >= 140 && c32 <= 256) return pick("d4x2_w8_r1");
            if (2 * c64 >= 140 && 2 * c64 <= 256) return pick("d2x4_w8_r1");   // (two blocks of 32 rows)
        }
        if (n <= 2048) return pick("d2x1_w16_r1");
        if (n <= 12288) return pick("d2x2_w8_r1");
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
tiles:
    // Everything else -- from 65 rows, and 33 to 64 rows on a short K or very many columns:
    // the fitted cost model over the tiles of the pipelined kernel and the blocks of the
    // wave-level one.
    return modelled_choice(m, n, k, ptr_align, has_ws, false);
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
        const Choice c = modelled_choice(m, n, k, ptr_align, has_ws, true);
        if (c.cfg > 0) return c;
    }
    const Choice h = heuristic(m, n, k, ptr_align, false);
    if (h.ksplit <= 1 && scaled_launcher(h.cfg)) return h;
    return {0, 1, 1};
}

}  // namespace qm
