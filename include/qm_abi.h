/*
 * C ABI of the MI355X (gfx950) packed-int4 GEMM library, libqm_hip.so.
 *
 *   C[M,N] (int32, row-major) = A[M,K] (s4) * B[N,K]^T (s4)
 *
 * A and B are packed two nibbles per byte along K: byte j of a row holds element
 * 2j in bits 0..3 and element 2j+1 in bits 4..7, two's complement (reference:
 * pack_b, test.py:6-15; unpack_int4_matrix, kernel.cu:389-408).  A is [M, K/2]
 * bytes, B is [N, K/2] bytes ("B is transposed", kernel.cu:78), C is fully
 * overwritten (kernel.cu:99-114,173).
 *
 * Plain pointers and sizes only; every pointer is a DEVICE pointer borrowed for
 * the duration of the enqueued work; `stream` is a hipStream_t passed as void*
 * (NULL = the default stream).  Every call is asynchronous, allocates nothing,
 * never synchronises and is therefore safe under HIP graph capture, as the
 * reference's harness requires (test.py:78-81).
 *
 * Every function returning int returns QM_OK (0) or a negative QM_ERR_* code;
 * qm_status_string() names it.  The reference has no error reporting at all
 * (extension.cpp:11-15 commented out, kernel.cu:282-288 commented out, unknown
 * shapes silently skipped at kernel.cu:340-385); returning a status is a
 * deliberate strengthening.
 */
#ifndef QM_ABI_H
#define QM_ABI_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QM_OK                 0
#define QM_ERR_NULL          -1 /* a required pointer is NULL                               */
#define QM_ERR_SHAPE         -2 /* m, n or k negative, k odd, or a size overflows int32     */
#define QM_ERR_CONFIG        -3 /* cfg id unknown, or that config cannot run this shape     */
#define QM_ERR_LAUNCH        -4 /* the HIP runtime refused the launch (see qm_last_hip_error) */
#define QM_ERR_ALIGN         -5 /* C is not 4-byte aligned (a 16-bit output: 2-byte)         */
#define QM_ERR_DTYPE         -6 /* out_dtype is none of the QM_OUT_* values                 */
#define QM_ERR_SCRATCH       -7 /* qm_gemm_i4_static: the call needs more scratch memory than
                                   QM_STATIC_SCRATCH_BYTES                                   */

#define QM_CFG_AUTO          -1 /* let the shape table / heuristic choose                   */

/*
 * The hot path.  Replaces
 *   void wrapper(void *A, void *B, void *C, const int m, const int n, const int k,
 *                cudaStream_t stream)                 (kernel.cu:334, declared extension.cpp:6)
 * with the same seven arguments in the same order plus a status.  Unlike the
 * reference, every shape with m,n >= 0 and even k >= 0 is computed (m or n == 0
 * is a no-op, k == 0 zero-fills C).
 *
 * Seven arguments leave no room for a workspace.  On every shape whose best schedule needs
 * none -- 40 of the 42 shapes of the reference's table (kernel.cu:343-384), every BASELINE
 * shape, K below one 128-nibble step -- this entry point runs exactly what qm_gemm_i4_ws
 * runs.  It is slower than qm_gemm_i4_ws / qm_gemm_i4_static (measured, MI355X, both columns
 * of benchmarks/mi355x.md's second table) in two cases:
 *   - few output tiles and a long K, which those entry points split over several workgroups
 *     per tile through the workspace: here the best unsplit configuration runs instead.
 *     Two shapes of the reference's table are left that split K: 256 x 8192 x 28672, 59.3 us
 *     against 55.8 (1.06x), and 512 x 8192 x 28672, 96-105 us against 92-95 (1.04-1.11x);
 *   - K % 32 != 0, or A or B not 16-byte aligned: no 16-byte loads, the one-thread-per-element
 *     kernel runs (2048 x 4096 x 4100: 3.3 ms, against 44 us on zero-padded copies in a
 *     workspace).  Weight matrices of the reference's table all have K % 32 == 0.
 * A caller that can lend device memory should bind qm_gemm_i4_ws; one that cannot allocate,
 * qm_gemm_i4_static.
 */
int qm_gemm_i4(const void *A, const void *B, void *C, int m, int n, int k, void *stream);

/*
 * Same, with an explicit kernel configuration.  Replaces the compile-time choice
 * made by LAUNCH_KERNEL_IF_CONDITION / IGemmConfig (kernel.cu:321-332, 23-50)
 * from the constexpr table in configs.cu:19-689; used by the autotuner that
 * regenerates this library's per-shape table.  cfg = QM_CFG_AUTO behaves as
 * qm_gemm_i4.  Otherwise: configuration id in bits 0..15, tile raster group
 * height in bits 16..23 (0 = default), K split in bits 24..29 (0 or 1 = none;
 * above 1 only for the pipelined "q" configurations: C is zero-filled by a first
 * kernel and the partial sums are added into it with integer atomics, still
 * exact, still one enqueue on the caller's stream).  Bit 30, "q" configurations
 * only: launch one workgroup per (K split, tile) instead of the default persistent
 * grid whose workgroups each run several tiles back to back.
 */
int qm_gemm_i4_cfg(const void *A, const void *B, void *C, int m, int n, int k, void *stream, int cfg);

/*
 * The GEMM with a dequantising epilogue fused in:
 *   D[m][n] = round16( ((float)C[m][n] * row_scale[m]) * col_scale[n] )
 * where C is the exact int32 product above, both multiplications are IEEE single
 * precision in this order, and round16 rounds to nearest even into fp16 (QM_OUT_F16) or
 * bfloat16 (QM_OUT_BF16).  D is [M, N] 16-bit, row-major; row_scale is [M], col_scale is
 * [N], device pointers, either may be NULL for all ones.  No counterpart in the
 * reference's code: its README.md:7 names fused epilogues as what the kernel is for
 * (per-token activation scales x per-channel weight scales of an int4 linear layer);
 * C (4 bytes per element, most of the traffic of the int32 form) is never written.
 * Same calling rules as qm_gemm_i4.  The _cfg form takes a configuration as
 * qm_gemm_i4_cfg does (no K split; QM_ERR_CONFIG when that configuration has no scaled
 * output, see qm_config_has_scaled).
 */
#define QM_OUT_F16  1
#define QM_OUT_BF16 2
int qm_gemm_i4_scaled(const void *A, const void *B, void *D, int m, int n, int k, const float *row_scale,
                      const float *col_scale, int out_dtype, void *stream);
int qm_gemm_i4_scaled_cfg(const void *A, const void *B, void *D, int m, int n, int k, const float *row_scale,
                          const float *col_scale, int out_dtype, void *stream, int cfg);
int qm_config_has_scaled(int cfg); /* 1 / 0 */

/*
 * The two GEMMs with a caller-provided workspace (the counterpart of the workspace
 * argument of vendor GEMM libraries; the reference's wrapper, kernel.cu:334, has none
 * because its kernels never split K).  Shapes with few output tiles and a long K run
 * faster with K split over several workgroups per tile; with a workspace each split
 * stores its partial tile there with plain 16-byte stores and a second kernel adds the
 * splits up (scaling and rounding, for the scaled form), instead of 4-byte atomics into
 * C.  The second use (cfg = QM_CFG_AUTO only): large shapes whose K is not a multiple of
 * 32, or whose operands are not 16-byte aligned, get copies of A and B in the workspace
 * with every row padded with zeros to whole 128-nibble steps, and run on the pipelined
 * kernel instead of the generic one.  Results are identical to the forms without a
 * workspace.
 *   workspace        device memory, 16-byte aligned, or NULL; used by the kernels of this
 *                    call only (in stream order): calls that may overlap on the GPU need
 *                    a workspace each, calls on one stream can share one
 *   workspace_bytes  its size; qm_gemm_workspace_bytes says how much this call can use.
 *                    A smaller (or no) workspace is not an error: the call then runs as
 *                    the form without one (except that an explicit cfg with a K split
 *                    and the scaled output returns QM_ERR_CONFIG).
 * cfg as for qm_gemm_i4_cfg (QM_CFG_AUTO included); with a workspace the scaled form also
 * takes K splits, on every "q" configuration.
 * qm_gemm_workspace_bytes: what the call with these arguments uses at most (0 when it
 * needs none); scaled = 1 for the scaled form.
 */
int qm_gemm_i4_ws(const void *A, const void *B, void *C, int m, int n, int k, void *stream, int cfg,
                  void *workspace, size_t workspace_bytes);
int qm_gemm_i4_scaled_ws(const void *A, const void *B, void *D, int m, int n, int k, const float *row_scale,
                         const float *col_scale, int out_dtype, void *stream, int cfg, void *workspace,
                         size_t workspace_bytes);
size_t qm_gemm_workspace_bytes(int m, int n, int k, int ptr_align, int cfg, int scaled);

/*
 * qm_gemm_i4 for callers that cannot allocate and have no workspace to lend: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in
 * the reference (its wrapper, kernel.cu:334, never needs scratch memory because it never
 * splits K and skips the shapes it has no table row for).  Runs exactly what
 * qm_gemm_i4_ws(..., QM_CFG_AUTO, workspace, bytes) runs when it is lent a workspace of
 * qm_gemm_workspace_bytes(m, n, k, align, QM_CFG_AUTO, 0) bytes -- same kernels, same result
 * bit for bit -- but the partial tiles of a K split and the zero-padded operand copies live
 * in an array of QM_STATIC_SCRATCH_BYTES that is part of the library's device code: every
 * GPU the library runs on holds one copy of it from the first kernel launch until the
 * process ends.  The call makes no hipMalloc / hipFree and no other allocating call.
 *   - A call that would use more than QM_STATIC_SCRATCH_BYTES returns QM_ERR_SCRATCH and
 *     enqueues nothing (use qm_gemm_i4_ws with a workspace of your own, or qm_gemm_i4).
 *   - All calls on one GPU share that GPU's array: calls on ONE stream are ordered and
 *     safe; calls that may overlap on the GPU (different streams, no dependency) race on
 *     it and must not both use this entry point.  Nothing in the array has to start from
 *     zero (every byte a kernel reads was written by an earlier kernel of the same call).
 *   - The first call on a device looks the array's address up (hipGetSymbolAddress); make
 *     one call per device before capturing this entry point into a graph.
 */
#define QM_STATIC_SCRATCH_BYTES (64u << 20)
int qm_gemm_i4_static(const void *A, const void *B, void *C, int m, int n, int k, void *stream);

/* The configuration qm_gemm_i4_ws picks for this shape when it is given a workspace
 * (the table lookup the reference does at kernel.cu:340-385, here with a heuristic
 * fallback instead of a silent no-op); without a workspace the K split may be lower.  ptr_align is the smallest alignment in bytes shared by A and
 * B (pass 16 or more when they come from a device allocator). */
int qm_select_config(int m, int n, int k, int ptr_align);
/* The same for every form of the call: has_workspace = 0 gives what qm_gemm_i4 / qm_gemm_i4_cfg
 * (QM_CFG_AUTO) run, which never split K through a workspace; scaled = 1 the choice of the
 * qm_gemm_i4_scaled* forms. */
int qm_select_config_ex(int m, int n, int k, int ptr_align, int has_workspace, int scaled);

/* Introspection of the compiled-in configurations (the counterpart of the
 * KernelConfig instances, configs.cu:1-17). */
int         qm_num_configs(void);
const char *qm_config_name(int cfg);                       /* NULL when cfg is out of range */
int         qm_config_supports(int cfg, int m, int n, int k, int ptr_align); /* 1 / 0      */

/*
 * Device-side packing and unpacking, the steps on either side of the GEMM:
 *   qm_pack_i4   replaces pack_b (test.py:6-15):             [rows,K] int8 -> [rows,K/2] bytes
 *   qm_unpack_i4 replaces unpack_int4_matrix (kernel.cu:389-408): the inverse
 * Values outside [-8,7] are truncated to their low nibble when packing.
 */
int qm_pack_i4(const void *src_i8, void *dst_packed, int rows, int k, void *stream);
int qm_unpack_i4(const void *src_packed, void *dst_i8, int rows, int k, void *stream);

/*
 * Quantise and pack in one pass: the step before the GEMM when the activations of an int4
 * linear layer arrive as floats.  Per row r of x ([rows, k], row-major, fp16 / bf16 / fp32):
 *   amax = max_j |x[r][j]|,  scales[r] = amax / 7,
 *   q[j] = clamp(rint(x[r][j] * (7 / amax)), -7, 7)        (all zero when amax == 0)
 * in IEEE single precision with round-half-to-even, packed as qm_pack_i4 packs (the
 * packing half is pack_b, test.py:6-15; the reference has no quantiser: its test draws
 * int4 values directly, test.py:22-23).  scales is [rows] float32 and is what
 * qm_gemm_i4_scaled takes as row_scale.  x must be finite.  Each row is read from HBM once.
 */
#define QM_IN_F16  1
#define QM_IN_BF16 2
#define QM_IN_F32  3
int qm_quantize_pack_i4(const void *x, int in_dtype, void *dst_packed, float *scales, int rows, int k, void *stream);

/*
 * Optional: everything a first launch on the current device would otherwise do once -- the
 * LDS size attribute and the residency query of every kernel, the address of the library's
 * scratch array -- without launching anything.  No counterpart in the reference (its
 * launch_igemm, kernel.cu:268-289, needs no set-up: 32 KB of shared memory at most).  First
 * launches do this by themselves, under HIP graph capture too; a caller that wants no
 * runtime queries inside a capture or a latency-critical first call makes this call first,
 * once per device, with that device current.
 */
int qm_init(void);

/*
 * Testing aid, not for production callers.  Operands of 2 GiB and more are cut by the library
 * into blocks its kernels' 32-bit row offsets reach: blocks of rows of A, and blocks of rows
 * of B, which are blocks of columns of C written through a row stride.  This call lowers that
 * limit (bytes; <= 0 restores 2^31 - 1) so that the block paths can be driven on small
 * shapes; it returns the previous limit.  Process-wide, not synchronised with calls in
 * flight on other threads.  No counterpart in the reference (its kernels take no operand
 * beyond their table's shapes, kernel.cu:340-385).
 */
long long qm_debug_set_operand_limit(long long bytes);

/* Diagnostics.  qm_version names the compiler the library was built with: the kernels
 * manage matrix-core hazards by hand, so a result is validated for that compiler. */
const char *qm_status_string(int status);
int         qm_last_hip_error(void);      /* hipError_t of the last failed launch on this thread */
const char *qm_version(void);

#ifdef __cplusplus
}
#endif
#endif /* QM_ABI_H */
