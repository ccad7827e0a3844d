// C ABI of libqm_hip.so (include/qm_abi.h): argument checks, configuration
// choice and launches.  Takes the place of the reference's host side:
// wrapper (kernel.cu:334-385), LAUNCH_KERNEL_IF_CONDITION (kernel.cu:321-332)
// and launch_igemm (kernel.cu:268-289).
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <mutex>

#include "../../include/qm_abi.h"
#include "qm_launch.hpp"
#include "qm_skinny.hpp"
#include "qm_skinny_dma.hpp"
#include "qm_aux.hpp"

#define QM_EXPORT extern "C" __attribute__((visibility("default")))

namespace qm {

// --------------------------------------------------------------------------
// Launchers of the skinny and dot kernels
// --------------------------------------------------------------------------
template <class Cfg>
static hipError_t launch_skinny(const GemmArgs &p, hipStream_t stream, int opt)
{
    if (opt & QM_OPT_PREPARE) return hipSuccess;  // static LDS, nothing to set up
    const int blocks = (p.N + Cfg::BN - 1) / Cfg::BN;
    // More column blocks than two workgroups per CU can hold at once, and K within one turn
    // of the waves: workgroups that walk over several blocks each, evenly.
    constexpr int resident = 2 * 256;
    if constexpr (Cfg::U % 2 == 0) {
        if (blocks > resident && (p.K + 127) / 128 <= Cfg::NW * Cfg::U) {
            const int turns = (blocks + resident - 1) / resident;
            gemm_skinny_stream_kernel<Cfg><<<dim3((blocks + turns - 1) / turns), dim3(Cfg::THREADS), 0, stream>>>(p, blocks);
            return hipGetLastError();
        }
    }
    gemm_skinny_kernel<Cfg><<<dim3(blocks), dim3(Cfg::THREADS), 0, stream>>>(p);
    return hipGetLastError();
}
#define QM_SKINNY(FM, FN, NW, U) \
    hipError_t QM_SKINNY_FN(FM, FN, NW, U)(const GemmArgs &p, hipStream_t s, int gm) { return launch_skinny<SkinnyCfg<FM, FN, NW, U>>(p, s, gm); }
template <class Cfg>
static hipError_t launch_dot(const GemmArgs &p, hipStream_t stream, int opt)
{
    if (opt & QM_OPT_PREPARE) return hipSuccess;
    const int blocks = (p.N + Cfg::BN - 1) / Cfg::BN;
    gemm_dot_kernel<Cfg><<<dim3(blocks), dim3(Cfg::THREADS), 0, stream>>>(p.A, p.B, p.C, p.M, p.N, p.K, p.ldc, p.out, p.row_scale, p.col_scale);
    return hipGetLastError();
}
#define QM_DOT(MR, FN, NW, U) \
    hipError_t QM_DOT_FN(MR, FN, NW, U)(const GemmArgs &p, hipStream_t s, int gm) { return launch_dot<DotCfg<MR, FN, NW, U>>(p, s, gm); }
template <class Cfg>
static hipError_t launch_skinny_dma(const GemmArgs &p, hipStream_t stream, int opt)
{
    static std::atomic<bool> lds_ok[QM_MAX_DEVICES] = {};
    const hipError_t e = ensure_dynamic_lds(&gemm_skinny_dma_kernel<Cfg>, Cfg::LDS_BYTES, lds_ok);
    if (e != hipSuccess) return e;
    if (opt & QM_OPT_PREPARE) return hipSuccess;
    const int blocks = (p.N + Cfg::BN - 1) / Cfg::BN, row_blocks = (p.M + Cfg::MAX_M - 1) / Cfg::MAX_M;
    if (row_blocks > 65535) return hipErrorInvalidValue;
    gemm_skinny_dma_kernel<Cfg><<<dim3(blocks, row_blocks), dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream>>>(p.A, p.B, p.C, p.M, p.N, p.K, p.ldc, p.out, p.row_scale, p.col_scale);
    return hipGetLastError();
}
// Compute units of the current device (asked once per device).
static hipError_t device_cus(int *cus)
{
    static std::atomic<int> cached[QM_MAX_DEVICES] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= QM_MAX_DEVICES) return hipErrorInvalidDevice;
    int n = cached[dev].load(std::memory_order_acquire);
    if (n == 0) {
        e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) return e;
        if (n < 1) n = 1;
        cached[dev].store(n, std::memory_order_release);
    }
    *cus = n;
    return hipSuccess;
}
template <class Cfg>
static hipError_t launch_skinny_stream_dma(const GemmArgs &p, hipStream_t stream, int opt)
{
    static std::atomic<bool> lds_ok[QM_MAX_DEVICES] = {};
    hipError_t e = ensure_dynamic_lds(&gemm_skinny_stream_dma_kernel<Cfg>, Cfg::LDS_BYTES, lds_ok);
    if (e != hipSuccess) return e;
    int cus = 0;
    e = device_cus(&cus);
    if (e != hipSuccess) return e;
    if (opt & QM_OPT_PREPARE) return hipSuccess;
    const int blocks = (p.N + Cfg::BN - 1) / Cfg::BN;
    const int resident = cus * (160 * 1024 / Cfg::LDS_BYTES);  // workgroups the device holds at once (the LDS decides)
    const int grid = blocks < resident ? blocks : resident;
    gemm_skinny_stream_dma_kernel<Cfg><<<dim3(grid), dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream>>>(
        p.A, p.B, p.C, p.M, p.N, p.K, p.ldc, p.out | (grid << 8), blocks, p.row_scale, p.col_scale);
    return hipGetLastError();
}
#define QM_SKINNYP(FM, FN, NW, D, R) \
    hipError_t QM_SKINNYP_FN(FM, FN, NW, D, R)(const GemmArgs &p, hipStream_t s, int gm) { return launch_skinny_stream_dma<SkinnyStreamCfg<FM, FN, NW, D, R>>(p, s, gm); }
#define QM_SKINNYD(FM, FN, NW, D) \
    hipError_t QM_SKINNYD_FN(FM, FN, NW, D)(const GemmArgs &p, hipStream_t s, int gm) { return launch_skinny_dma<SkinnyDmaCfg<FM, FN, NW, D>>(p, s, gm); }
#include "qm_configs.inc"

}  // namespace qm

#include "qm_select.hpp"

namespace qm {

static thread_local int g_last_hip_error = 0;

static int ptr_alignment(const void *a, const void *b)
{
    const uintptr_t x = (uintptr_t)a | (uintptr_t)b;
    if (x == 0) return 4096;
    const uintptr_t low = x & (~x + 1);
    return low > 4096 ? 4096 : (int)low;
}

static int check_gemm_args(const void *A, const void *B, void *C, int m, int n, int k)
{
    if (m < 0 || n < 0 || k < 0 || (k & 1)) return QM_ERR_SHAPE;
    if (m == 0 || n == 0) return QM_OK;
    if (!C) return QM_ERR_NULL;
    if ((uintptr_t)C & 3) return QM_ERR_ALIGN;
    if (k > 0 && (!A || !B)) return QM_ERR_NULL;
    return QM_OK;
}

static int fail_launch(hipError_t e)
{
    g_last_hip_error = (int)e;
    return QM_ERR_LAUNCH;
}

// The splits of K that have work (with kps K-steps per split only ceil(kt / kps) have any)
// and the workspace they fill: one padded tile of int32 per (split, tile).
static int effective_ksplit(const ConfigDesc &d, int k, int ksplit)
{
    if (d.kind != KIND_TILE16 || ksplit <= 1) return 1;
    return normalised_ksplit(k, ksplit);
}

static size_t split_workspace_bytes(const ConfigDesc &d, int m, int n, int ksplit)
{
    const size_t tiles = (size_t)((m + d.bm - 1) / d.bm) * (size_t)((n + d.bn - 1) / d.bn);
    return tiles * (size_t)ksplit * (size_t)d.bm * (size_t)d.bn * sizeof(int32_t);
}

static bool workspace_fits(const ConfigDesc &d, int m, int n, int ksplit, const void *ws, size_t ws_bytes)
{
    return ws != nullptr && ((uintptr_t)ws & 15) == 0 && ws_bytes >= split_workspace_bytes(d, m, n, ksplit);
}

// Automatic choice only: K padded to a multiple of 128 (operands copied into the workspace) so
// that the pipelined kernel can run instead of the generic one.  Worth it when the shape is
// large -- the copy is (M + N) K / 2 bytes twice over.  `direct` is the choice without padding.
struct PadPlan {
    bool on = false;
    int kp = 0;
    Choice ch{};
    size_t a_bytes = 0, b_bytes = 0;
    size_t bytes() const { return a_bytes + b_bytes; }
};

static PadPlan plan_padded_k(int m, int n, int k, int ptr_align, const Choice &direct)
{
    PadPlan pl;
    const int kind = g_configs[direct.cfg].kind;
    if (kind == KIND_TILE16 || kind == KIND_SKINNY) return pl;
    const int kp = (k + 127) / 128 * 128;
    if (kp > QM_MAX_K_X16 || !fast_path_ok(m, n, kp, 256)) return pl;
    const long long outs = (long long)m * n;
    if (outs * kp < (1LL << 27)) return pl;  // (kp: a K below one K-step counts as the step it is padded to)
    (void)ptr_align;
    Choice ch = heuristic(m, n, kp, 256, false);
    if (g_configs[ch.cfg].kind == KIND_GENERIC) return pl;
    ch.ksplit = 1;
    pl.on = true;
    pl.kp = kp;
    pl.ch = ch;
    pl.a_bytes = ((size_t)m * (kp / 2) + 255) / 256 * 256;
    pl.b_bytes = ((size_t)n * (kp / 2) + 255) / 256 * 256;
    return pl;
}

// The padded copies of A and B in the workspace, and the arguments of the GEMM on them.
static hipError_t launch_padded(GemmArgs &p, const PadPlan &pl, void *ws, hipStream_t s)
{
    uint8_t *a_p = static_cast<uint8_t *>(ws), *b_p = a_p + pl.a_bytes;
    const PadRowsArgs q{p.A, p.B, reinterpret_cast<uint32_t *>(a_p), reinterpret_cast<uint32_t *>(b_p), p.M, p.N, p.K / 2, pl.kp / 8};
    const long long rows = (long long)p.M + p.N;
    pad_rows_kernel<<<dim3((unsigned)std::min<long long>((rows + 3) / 4, 256 * 32)), dim3(256), 0, s>>>(q);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    p.A = a_p;
    p.B = b_p;
    p.K = pl.kp;
    return hipSuccess;
}

static Choice choice_from_code(int cfg)
{
    Choice ch;
    ch.cfg = cfg & 0xFFFF;
    ch.group_m = (cfg >> 16) & 0xFF;
    ch.ksplit = (cfg >> 24) & 0x3F;
    ch.spread = (cfg >> 30) & 1;
    if (ch.group_m == 0) ch.group_m = 4;
    if (ch.ksplit == 0) ch.ksplit = 1;
    return ch;
}

// GEMM with K split into ch.ksplit (> 1, normalised) through the workspace, then the sum of
// the splits into C in the output form p.out.
static hipError_t launch_split_with_workspace(GemmArgs p, const Choice &ch, void *ws, hipStream_t s)
{
    const ConfigDesc &d = g_configs[ch.cfg];
    SplitReduceArgs q;
    q.ws = static_cast<const v4i *>(ws);
    q.C = p.C;
    q.M = p.M;
    q.N = p.N;
    q.tiles_m = (p.M + d.bm - 1) / d.bm;
    q.tiles_n = (p.N + d.bn - 1) / d.bn;
    q.group_m = ch.group_m < 1 ? 1 : (ch.group_m > q.tiles_m ? q.tiles_m : ch.group_m);  // as the launcher clamps it
    q.ksplit = ch.ksplit;
    q.BM = d.bm;
    q.BN = d.bn;
    q.WGN = d.wgn;
    q.FM = d.bm / d.wgm / 16;
    q.FN = d.bn / d.wgn / 16;
    q.waves = d.waves;
    q.row_scale = p.row_scale;
    q.col_scale = p.col_scale;
    q.out = p.out;
    p.out = OUT_I32;
    p.row_scale = p.col_scale = nullptr;
    p.ws = static_cast<int32_t *>(ws);
    hipError_t e = d.launch(p, s, ch.group_m | (ch.ksplit << 8) | (ch.spread << 16));
    if (e != hipSuccess) return e;
    const size_t pieces = (size_t)q.tiles_m * q.tiles_n * (size_t)(d.bm * d.bn / 4);
    if (pieces > 0x7fffff00ULL) return hipErrorInvalidValue;
    splitk_reduce_kernel<<<dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, s>>>(q);
    return hipGetLastError();
}

// Operands of this many bytes or more are cut into blocks (below).  2^31 - 1 in production: what
// the kernels' 32-bit row offsets reach.  qm_debug_set_operand_limit lowers it so that tests
// can drive the block paths -- C written through a row stride, blocks of rows then of columns --
// on small shapes.
static std::atomic<long long> g_operand_limit{0x7fffffffLL};

// An A of 2 GiB or more is beyond the 32-bit row offsets of the fast kernels; its row blocks
// are independent (block r0.. of A gives rows r0.. of C), so the call is cut into blocks
// of rows that fit, one after the other on the stream (they share the workspace).  Returns
// the rows per block, 0 when the call needs no cutting or cutting does not help (B too large
// as well, or a shape the fast kernels do not take anyway).
static int row_block_for_large_a(int m, int n, int k, int ptr_align)
{
    (void)n;
    if (k < 32 || k % 32 != 0 || k > QM_MAX_K_X16 || ptr_align < 16) return 0;
    const long long kb = k / 2, limit = g_operand_limit.load(std::memory_order_relaxed);
    if ((long long)m * kb < limit) return 0;
    const long long rows = ((limit - 1) / kb) & ~255LL;
    return rows >= 256 ? (int)rows : 0;
}

// The same for a B of 2 GiB or more (and an A that fits, or a row block of one): blocks of
// rows of B are blocks of columns of C, which the kernels write through a row stride.
static int col_block_for_large_b(int m, int n, int k, int ptr_align)
{
    if (k < 32 || k % 32 != 0 || k > QM_MAX_K_X16 || ptr_align < 16) return 0;
    const long long kb = k / 2, limit = g_operand_limit.load(std::memory_order_relaxed);
    if ((long long)n * kb < limit || (long long)m * kb >= limit) return 0;
    const long long cols = ((limit - 1) / kb) & ~255LL;
    return cols >= 256 ? (int)cols : 0;
}

// One GEMM call, arguments already checked (m, n >= 1, k even).  `out` is OUT_I32 with C in
// `dst`, or OUT_F16 / OUT_BF16 with the scaled and rounded D there.  The two differ in one
// place: a K split whose partial sums have no workspace to meet in falls back to atomic adds
// into a zero-filled C for int32, and is not taken at all for a rounded output.
static int run_gemm(const void *A, const void *B, void *dst, int m, int n, int k, const float *row_scale,
                    const float *col_scale, int out, hipStream_t s, int cfg, void *workspace, size_t workspace_bytes, int ldc = 0)
{
    const bool scaled = out != OUT_I32;
    const size_t cnt = (size_t)m * (size_t)n;
    const int row_stride = ldc != 0 ? ldc : n;   // of the output, in elements
    const bool strided = row_stride != n;        // a block of columns of a wider output
    if (k == 0) {
        if (scaled) fill_zero16_kernel<<<dim3(flat_grid(cnt, 256)), dim3(256), 0, s>>>(static_cast<uint16_t *>(dst), cnt);
        else fill_zero_kernel<<<dim3(flat_grid(cnt, 256)), dim3(256), 0, s>>>(static_cast<int32_t *>(dst), cnt);
        const hipError_t e = hipGetLastError();
        return e == hipSuccess ? QM_OK : fail_launch(e);
    }
    const int align = ptr_alignment(A, B);
    if (const int rb = cfg == QM_CFG_AUTO ? row_block_for_large_a(m, n, k, align) : 0) {
        for (int r0 = 0; r0 < m; r0 += rb) {
            const int st = run_gemm(static_cast<const uint8_t *>(A) + (size_t)r0 * (size_t)(k / 2), B,
                                    static_cast<uint8_t *>(dst) + (size_t)r0 * (size_t)row_stride * (scaled ? 2 : 4), m - r0 < rb ? m - r0 : rb,
                                    n, k, row_scale ? row_scale + r0 : nullptr, col_scale, out, s, cfg, workspace, workspace_bytes, ldc);
            if (st != QM_OK) return st;
        }
        return QM_OK;
    }
    if (const int cb = cfg == QM_CFG_AUTO ? col_block_for_large_b(m, n, k, align) : 0) {
        for (int c0 = 0; c0 < n; c0 += cb) {
            const int st = run_gemm(A, static_cast<const uint8_t *>(B) + (size_t)c0 * (size_t)(k / 2),
                                    static_cast<uint8_t *>(dst) + (size_t)c0 * (scaled ? 2 : 4), m, n - c0 < cb ? n - c0 : cb, k, row_scale,
                                    col_scale ? col_scale + c0 : nullptr, out, s, cfg, workspace, workspace_bytes, row_stride);
            if (st != QM_OK) return st;
        }
        return QM_OK;
    }
    const bool has_ws = workspace != nullptr && workspace_bytes > 0;
    GemmArgs p{static_cast<const uint8_t *>(A), static_cast<const uint8_t *>(B), static_cast<int32_t *>(dst), m, n, k};
    p.row_scale = row_scale;
    p.col_scale = col_scale;
    p.out = out;
    p.ldc = strided ? row_stride : 0;
    if (strided && cfg != QM_CFG_AUTO) return QM_ERR_CONFIG;
    const auto launcher = [&](int id) { return scaled ? scaled_launcher(id) : g_configs[id].launch; };
    Choice ch;
    if (strided) {
        // one launch straight into the wider output: no K split (its partial sums are added up
        // into a contiguous C) and no padded copies
        ch = scaled ? select_scaled(m, n, k, align, false) : select_config(m, n, k, align, false);
        ch.ksplit = 1;
        const LaunchFn launch = launcher(ch.cfg);
        if (!launch) return QM_ERR_CONFIG;
        const hipError_t e = launch(p, s, ch.group_m | (1 << 8) | (ch.spread << 16));
        return e == hipSuccess ? QM_OK : fail_launch(e);
    }
    if (cfg == QM_CFG_AUTO) {
        ch = scaled ? select_scaled(m, n, k, align, has_ws) : select_config(m, n, k, align, has_ws);
    } else {
        ch = choice_from_code(cfg);
        if (!config_supports(ch.cfg, m, n, k, align)) return QM_ERR_CONFIG;
        if (ch.ksplit > 1 && g_configs[ch.cfg].kind != KIND_TILE16) return QM_ERR_CONFIG;
    }
    ch.ksplit = effective_ksplit(g_configs[ch.cfg], k, ch.ksplit);
    if (ch.ksplit > 1 && workspace_fits(g_configs[ch.cfg], m, n, ch.ksplit, workspace, workspace_bytes)) {
        const hipError_t e = launch_split_with_workspace(p, ch, workspace, s);
        return e == hipSuccess ? QM_OK : fail_launch(e);
    }
    if (ch.ksplit > 1 && scaled) {
        // partial sums cannot meet in a rounded output: without the workspace, no split
        if (cfg != QM_CFG_AUTO) return QM_ERR_CONFIG;
        ch = select_scaled(m, n, k, align, false);
        ch.ksplit = 1;
    }
    if (cfg == QM_CFG_AUTO && has_ws) {
        PadPlan pl = plan_padded_k(m, n, k, align, ch);
        if (pl.on && !launcher(pl.ch.cfg)) {
            // a pipelined configuration that has the scaled output, if the shape is one for those
            const int id = find_config("q256x256_w2x2_s9o1");
            if (id >= 0 && launcher(id)) pl.ch.cfg = id; else pl.on = false;
        }
        if (pl.on && ((uintptr_t)workspace & 15) == 0 && workspace_bytes >= pl.bytes()) {
            hipError_t e = launch_padded(p, pl, workspace, s);
            if (e == hipSuccess) e = launcher(pl.ch.cfg)(p, s, pl.ch.group_m | (1 << 8) | (pl.ch.spread << 16));
            return e == hipSuccess ? QM_OK : fail_launch(e);
        }
    }
    if (ch.ksplit > 1) {
        // int32, no workspace: the partial sums meet in C by integer atomic adds, C starts from zero
        fill_zero_kernel<<<dim3(flat_grid(cnt, 256)), dim3(256), 0, s>>>(static_cast<int32_t *>(dst), cnt);
        const hipError_t ez = hipGetLastError();
        if (ez != hipSuccess) return fail_launch(ez);
    }
    const LaunchFn launch = launcher(ch.cfg);
    if (!launch) return QM_ERR_CONFIG;
    const hipError_t e = launch(p, s, ch.group_m | (ch.ksplit << 8) | (ch.spread << 16));
    return e == hipSuccess ? QM_OK : fail_launch(e);
}

}  // namespace qm

using namespace qm;

QM_EXPORT int qm_gemm_i4_ws(const void *A, const void *B, void *C, int m, int n, int k, void *stream, int cfg,
                            void *workspace, size_t workspace_bytes)
{
    const int st = check_gemm_args(A, B, C, m, n, k);
    if (st != QM_OK) return st;
    if (m == 0 || n == 0) return QM_OK;
    return run_gemm(A, B, C, m, n, k, nullptr, nullptr, OUT_I32, reinterpret_cast<hipStream_t>(stream), cfg, workspace, workspace_bytes);
}

// Every one-off set-up a first launch on the current device would otherwise do.
QM_EXPORT int qm_init(void)
{
    GemmArgs p{nullptr, nullptr, nullptr, 256, 256, 256};
    for (int id = 0; id < g_num_configs; ++id) {
        if (g_configs[id].kind == KIND_GENERIC) continue;
        for (const int k : {256, 256 + 32}) {   // the kernel for whole K-steps and the one with a short last step
            p.K = k;
            for (const int out : {(int)OUT_I32, (int)OUT_F16, (int)OUT_BF16}) {
                const LaunchFn fn = out == OUT_I32 ? g_configs[id].launch : scaled_launcher(id);
                if (!fn || (out != OUT_I32 && g_configs[id].kind != KIND_TILE16)) continue;
                p.out = out;
                const hipError_t e = fn(p, nullptr, QM_OPT_PREPARE);
                if (e != hipSuccess) return fail_launch(e);
            }
        }
    }
    void *ws = nullptr;
    const hipError_t e = static_scratch(&ws);
    return e == hipSuccess ? QM_OK : fail_launch(e);
}

QM_EXPORT int qm_gemm_i4_static(const void *A, const void *B, void *C, int m, int n, int k, void *stream)
{
    const int st = check_gemm_args(A, B, C, m, n, k);
    if (st != QM_OK) return st;
    if (m == 0 || n == 0) return QM_OK;
    const size_t need = qm_gemm_workspace_bytes(m, n, k, ptr_alignment(A, B), QM_CFG_AUTO, 0);
    if (need > (size_t)QM_STATIC_SCRATCH_BYTES) return QM_ERR_SCRATCH;
    void *ws = nullptr;
    if (need > 0) {
        const hipError_t e = static_scratch(&ws);
        if (e != hipSuccess) return fail_launch(e);
    }
    return run_gemm(A, B, C, m, n, k, nullptr, nullptr, OUT_I32, reinterpret_cast<hipStream_t>(stream), QM_CFG_AUTO, ws,
                    ws ? (size_t)QM_STATIC_SCRATCH_BYTES : 0);
}

QM_EXPORT int qm_gemm_i4_cfg(const void *A, const void *B, void *C, int m, int n, int k, void *stream, int cfg)
{
    return qm_gemm_i4_ws(A, B, C, m, n, k, stream, cfg, nullptr, 0);
}

QM_EXPORT int qm_gemm_i4_scaled_ws(const void *A, const void *B, void *D, int m, int n, int k, const float *row_scale,
                                   const float *col_scale, int out_dtype, void *stream, int cfg, void *workspace,
                                   size_t workspace_bytes)
{
    if (out_dtype != QM_OUT_F16 && out_dtype != QM_OUT_BF16) return QM_ERR_DTYPE;
    if (m < 0 || n < 0 || k < 0 || (k & 1)) return QM_ERR_SHAPE;
    if (m == 0 || n == 0) return QM_OK;
    if (!D) return QM_ERR_NULL;
    if ((uintptr_t)D & 1) return QM_ERR_ALIGN;
    if (k > 0 && (!A || !B)) return QM_ERR_NULL;
    return run_gemm(A, B, D, m, n, k, row_scale, col_scale, out_dtype == QM_OUT_F16 ? OUT_F16 : OUT_BF16,
                    reinterpret_cast<hipStream_t>(stream), cfg, workspace, workspace_bytes);
}

QM_EXPORT int qm_gemm_i4_scaled_cfg(const void *A, const void *B, void *D, int m, int n, int k, const float *row_scale,
                                    const float *col_scale, int out_dtype, void *stream, int cfg)
{
    return qm_gemm_i4_scaled_ws(A, B, D, m, n, k, row_scale, col_scale, out_dtype, stream, cfg, nullptr, 0);
}

QM_EXPORT int qm_gemm_i4_scaled(const void *A, const void *B, void *D, int m, int n, int k, const float *row_scale,
                                const float *col_scale, int out_dtype, void *stream)
{
    return qm_gemm_i4_scaled_ws(A, B, D, m, n, k, row_scale, col_scale, out_dtype, stream, QM_CFG_AUTO, nullptr, 0);
}

QM_EXPORT size_t qm_gemm_workspace_bytes(int m, int n, int k, int ptr_align, int cfg, int scaled)
{
    if (m < 1 || n < 1 || k < 2 || (k & 1)) return 0;
    if (const int rb = cfg == QM_CFG_AUTO ? row_block_for_large_a(m, n, k, ptr_align) : 0) {
        // the blocks run one after the other: the largest need of the two block sizes
        const size_t whole = qm_gemm_workspace_bytes(rb, n, k, ptr_align, cfg, scaled);
        const size_t rest = m % rb ? qm_gemm_workspace_bytes(m % rb, n, k, ptr_align, cfg, scaled) : 0;
        return whole > rest ? whole : rest;
    }
    if (cfg == QM_CFG_AUTO && col_block_for_large_b(m, n, k, ptr_align)) return 0;  // blocks of columns: one launch each, no workspace
    Choice ch;
    if (cfg == QM_CFG_AUTO) {
        ch = scaled ? select_scaled(m, n, k, ptr_align, true) : select_config(m, n, k, ptr_align, true);
    } else {
        ch = choice_from_code(cfg);
        if (!config_supports(ch.cfg, m, n, k, ptr_align)) return 0;
    }
    const int ks = effective_ksplit(g_configs[ch.cfg], k, ch.ksplit);
    if (ks > 1) return split_workspace_bytes(g_configs[ch.cfg], m, n, ks);
    if (cfg == QM_CFG_AUTO) {
        const PadPlan pl = plan_padded_k(m, n, k, ptr_align, ch);
        if (pl.on) return pl.bytes();
    }
    return 0;
}

QM_EXPORT int qm_config_has_scaled(int cfg)
{
    cfg &= 0xFFFF;
    return (cfg >= 0 && cfg < g_num_configs && scaled_launcher(cfg)) ? 1 : 0;
}

QM_EXPORT int qm_gemm_i4(const void *A, const void *B, void *C, int m, int n, int k, void *stream)
{
    return qm_gemm_i4_cfg(A, B, C, m, n, k, stream, QM_CFG_AUTO);
}

QM_EXPORT int qm_select_config(int m, int n, int k, int ptr_align)
{
    if (m < 1 || n < 1 || k < 2 || (k & 1)) return QM_ERR_SHAPE;
    const Choice ch = select_config(m, n, k, ptr_align, true);
    return ch.cfg | (ch.group_m << 16) | (ch.ksplit << 24) | (ch.spread << 30);
}

QM_EXPORT int qm_select_config_ex(int m, int n, int k, int ptr_align, int has_workspace, int scaled)
{
    if (m < 1 || n < 1 || k < 2 || (k & 1)) return QM_ERR_SHAPE;
    Choice ch = scaled ? select_scaled(m, n, k, ptr_align, has_workspace != 0) : select_config(m, n, k, ptr_align, has_workspace != 0);
    if (scaled && ch.ksplit > 1 && !has_workspace) {
        // as run_gemm: partial sums cannot meet in a rounded output
        ch = select_scaled(m, n, k, ptr_align, false);
        ch.ksplit = 1;
    }
    return ch.cfg | (ch.group_m << 16) | (ch.ksplit << 24) | (ch.spread << 30);
}

QM_EXPORT int qm_num_configs(void) { return g_num_configs; }

QM_EXPORT const char *qm_config_name(int cfg)
{
    cfg &= 0xFFFF;
    return (cfg >= 0 && cfg < g_num_configs) ? g_configs[cfg].name : nullptr;
}

QM_EXPORT int qm_config_supports(int cfg, int m, int n, int k, int ptr_align)
{
    return config_supports(cfg & 0xFFFF, m, n, k, ptr_align) ? 1 : 0;
}

QM_EXPORT int qm_pack_i4(const void *src_i8, void *dst_packed, int rows, int k, void *stream)
{
    if (rows < 0 || k < 0 || (k & 1)) return QM_ERR_SHAPE;
    const size_t nbytes = (size_t)rows * (size_t)(k / 2);
    if (nbytes == 0) return QM_OK;
    if (!src_i8 || !dst_packed) return QM_ERR_NULL;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (nbytes % 8 == 0 && ((uintptr_t)src_i8 & 15) == 0 && ((uintptr_t)dst_packed & 7) == 0)
        pack_i4_vec_kernel<<<dim3(flat_grid(nbytes / 8, 256)), dim3(256), 0, s>>>(static_cast<const v4i *>(src_i8), static_cast<v2i *>(dst_packed), nbytes / 8);
    else
        pack_i4_byte_kernel<<<dim3(flat_grid(nbytes, 256)), dim3(256), 0, s>>>(static_cast<const uint8_t *>(src_i8), static_cast<uint8_t *>(dst_packed), nbytes);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? QM_OK : fail_launch(e);
}

QM_EXPORT int qm_quantize_pack_i4(const void *x, int in_dtype, void *dst_packed, float *scales, int rows, int k, void *stream)
{
    if (in_dtype != QM_IN_F16 && in_dtype != QM_IN_BF16 && in_dtype != QM_IN_F32) return QM_ERR_DTYPE;
    if (rows < 0 || k < 0 || (k & 1)) return QM_ERR_SHAPE;
    if (rows == 0) return QM_OK;
    if (!scales || (k > 0 && (!x || !dst_packed))) return QM_ERR_NULL;
    if (((uintptr_t)x & (in_dtype == QM_IN_F32 ? 3 : 1)) || ((uintptr_t)scales & 3)) return QM_ERR_ALIGN;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    hipError_t e;
    if (in_dtype == QM_IN_F16) e = launch_quantize_pack<QM_IN_F16>(x, dst_packed, scales, rows, k, s);
    else if (in_dtype == QM_IN_BF16) e = launch_quantize_pack<QM_IN_BF16>(x, dst_packed, scales, rows, k, s);
    else e = launch_quantize_pack<QM_IN_F32>(x, dst_packed, scales, rows, k, s);
    return e == hipSuccess ? QM_OK : fail_launch(e);
}

QM_EXPORT int qm_unpack_i4(const void *src_packed, void *dst_i8, int rows, int k, void *stream)
{
    if (rows < 0 || k < 0 || (k & 1)) return QM_ERR_SHAPE;
    const size_t nbytes = (size_t)rows * (size_t)(k / 2);
    if (nbytes == 0) return QM_OK;
    if (!src_packed || !dst_i8) return QM_ERR_NULL;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (nbytes % 4 == 0 && ((uintptr_t)src_packed & 3) == 0 && ((uintptr_t)dst_i8 & 7) == 0)
        unpack_i4_vec_kernel<<<dim3(flat_grid(nbytes / 4, 256)), dim3(256), 0, s>>>(static_cast<const uint32_t *>(src_packed), static_cast<v2i *>(dst_i8), nbytes / 4);
    else
        unpack_i4_byte_kernel<<<dim3(flat_grid(nbytes, 256)), dim3(256), 0, s>>>(static_cast<const uint8_t *>(src_packed), static_cast<int8_t *>(dst_i8), nbytes);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? QM_OK : fail_launch(e);
}

QM_EXPORT const char *qm_status_string(int status)
{
    switch (status) {
    case QM_OK: return "ok";
    case QM_ERR_NULL: return "null pointer";
    case QM_ERR_SHAPE: return "bad shape (m, n, k must be >= 0 and k even)";
    case QM_ERR_CONFIG: return "unknown kernel configuration, or it cannot run this shape";
    case QM_ERR_LAUNCH: return "HIP launch failed";
    case QM_ERR_ALIGN: return "C must be 4-byte aligned (a 16-bit output 2-byte aligned)";
    case QM_ERR_DTYPE: return "unknown output type";
    case QM_ERR_SCRATCH: return "the call needs more scratch memory than the library's static array (QM_STATIC_SCRATCH_BYTES) holds";
    default: return "unknown status";
    }
}

QM_EXPORT int qm_last_hip_error(void) { return g_last_hip_error; }

QM_EXPORT long long qm_debug_set_operand_limit(long long bytes)
{
    const long long full = 0x7fffffffLL;
    return g_operand_limit.exchange(bytes <= 0 || bytes > full ? full : bytes, std::memory_order_relaxed);
}

#ifndef QM_COMPILER_VERSION
#define QM_COMPILER_VERSION "unknown compiler"
#endif
QM_EXPORT const char *qm_version(void) { return "quadmul-amd 0.3 (gfx950; built with " QM_COMPILER_VERSION ")"; }
