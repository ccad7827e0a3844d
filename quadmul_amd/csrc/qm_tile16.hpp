// Software-pipelined int4 GEMM tile kernel on v_mfma_i32_16x16x64_i8 (gfx950).
//
// Takes the place of the reference's igemm<Config> (kernel.cu:62-266) for large
// tiles: its cp.async loaders (kernel.cu:118-152) become direct global->LDS loads,
// its two-stage pipeline (kernel.cu:186-260) a four-stage LDS ring, its WMMA s4
// contraction (kernel.cu:246) int8 MFMAs on nibbles widened to 16*s4.
//
// What shapes it (all measured on MI355X):
//   * The part runs this workload at its package power limit, so energy spent
//     outside the MFMAs costs throughput directly.  Under the power cap the
//     16x16x64 int8 MFMA sustains a clearly higher rate than the 32x32x32 one, and
//     operands of the form 16*s4 (low nibble zero) are cheaper than sign-extended.
//   * LDS holds the packed bytes (half the LDS traffic of an int8 tile); each wave
//     widens its own fragments after ds_read: 10 VALU instructions per 16 bytes.
//   * Tiles travel global -> LDS without touching registers (global_load_lds, 16
//     bytes per lane): no staging registers, no ds_write.  Ring of 3 to 5 stages
//     (4 by default): while step s is contracted, B fragments of step s+1 are read
//     and widened, step s+2 has landed and step s+3 is in flight; one barrier per
//     K-step.
//   * The compiler's scheduler, left alone, puts the two MFMAs that update one
//     accumulator back to back and bunches the VALU work, which stalls the matrix
//     pipe.  The K-step is therefore written slot by slot -- one MFMA plus its share
//     of reads / widening / DMA -- with a scheduling barrier after every slot.
//   * The grid is persistent: a workgroup runs its tiles as one stream of K-steps,
//     the loads running ahead through tile boundaries, and the write-out of a whole
//     tile rides in the MFMA slots of its last K-step, through a per-wave LDS
//     transpose where there is room, so that stores cover contiguous row segments.
//   * Outputs: the exact int32 product, or (template parameter OUT) the product
//     scaled per row and per column in fp32 and rounded to fp16 / bf16.
//
// Rules the code keeps, each learnt from a wrong result or a slow kernel:
//   * the accumulators are read, written and cleared through asm statements only,
//     by one set of statements on every path (else the register allocator copies
//     all of them around);
//   * no per-lane branch inside the slot code of a K-step (selects instead);
//   * every lambda is always_inline (an outlined one takes all state to memory);
//   * values an asm statement writes into registers that a 16-byte store or
//     ds_write just before may still be reading get two wait states first (the
//     compiler pads that hazard only for instructions it can see).
#pragma once
#include <type_traits>

#include "qm_common.hpp"

namespace qm {

template <int B, int E, class F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

// acc += S0 * S1 with the accumulator pinned in AGPRs and tied in place.  Written as
// an asm statement for two reasons: the register allocator otherwise shuffles the 256
// accumulator registers around at the loop back-edge (hundreds of v_accvgpr moves per
// iteration), and volatile asm statements keep their program order, which is the issue
// order this kernel is built around.  The compiler cannot see the MFMA inside, so the
// kernel keeps every producer of S0/S1 and every other user of `acc` several
// instructions away (no MFMA hazard wait states are needed at those distances).
__device__ __forceinline__ void mfma16_acc(v4i &acc, const v4i &s0, const v4i &s1)
{
    asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(acc) : "v"(s0), "v"(s1));
}

// Wait states between the last MFMA into `acc` and its first ordinary reader.
__device__ __forceinline__ void mfma16_settle(v4i &acc)
{
    asm volatile("s_nop 15\n\ts_nop 15" : "+a"(acc));
}

// the 64-bit value (hi:lo) << 4, as one instruction (it issues faster than two
// 32-bit shifts).
__device__ __forceinline__ v2i shl4_pair(const int lo, const int hi)
{
    v2i in = {lo, hi}, out;
    asm("v_lshlrev_b64 %0, 4, %1" : "=v"(out) : "v"(in));
    return out;
}

// A use of `x` that generates no code: the value has to exist at this point of the program.
__device__ __forceinline__ void keep_here(const v4i &x) { asm volatile("" ::"v"(x)); }

__device__ __forceinline__ void keep_here_f(const float &x) { asm volatile("" ::"v"(x)); }

// One accumulator register -> ordinary register.  Inside the loop the accumulators are
// touched by asm statements only: an ordinary read there makes the register allocator
// treat them as general values, and it starts moving and spilling them.
__device__ __forceinline__ int acc_read(const int acc_elem)
{
    int dst;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(dst) : "a"(acc_elem));
    return dst;
}
// The same with two wait states in front, for the first read of a block: the destination
// registers may be the data of a 16-byte store or ds_write issued just before, which the
// hardware is still reading; the compiler pads that hazard for its own instructions but
// does not look inside asm statements.
__device__ __forceinline__ int acc_read_first(const int acc_elem)
{
    int dst;
    asm volatile("s_nop 1\n\tv_accvgpr_read_b32 %0, %1" : "=v"(dst) : "a"(acc_elem));
    return dst;
}

// acc = 0, as an MFMA on zero operands with a zero addend.  The accumulators are only
// ever redefined by asm statements that tie them in place; an ordinary assignment here
// would give the register allocator a second, unrelated definition to merge at the loop
// head, which it does by copying all of them.
__device__ __forceinline__ void mfma16_zero(v4i &acc, const v4i &zero)
{
    asm volatile("s_nop 1\n\tv_mfma_i32_16x16x64_i8 %0, %1, %1, 0" : "+a"(acc) : "v"(zero));
}

template <int BM_, int BN_, int WGM_, int WGN_, int STAGES_ = 4, int OCC_ = 1>
struct Tile16Cfg {
    static constexpr int OCC = OCC_;  // workgroups meant to share a CU (sets the register budget)
    static constexpr int BM = BM_, BN = BN_, BK = 128, WGM = WGM_, WGN = WGN_;
    static constexpr int WAVES = WGM * WGN, THREADS = 64 * WAVES;
    static constexpr int WM = BM / WGM, WN = BN / WGN;
    static constexpr int FM = WM / 16, FN = WN / 16;  // 16x16 accumulator blocks per wave
    static constexpr int W_OPS = 10;                  // VALU instructions that widen one packed fragment
    static constexpr int PITCH = 64;                  // packed bytes per row per K-step
    static constexpr int A_BYTES = BM * PITCH, B_BYTES = BN * PITCH;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int STAGES = STAGES_;  // LDS ring depth: 4 or 5 on the large tiles; 6 to 8 on the small ones, whose K-steps are short against the latency of HBM
    // STAGES = 9 is the paired ring: five stages of A and four of B, each operand in a ring of
    // its own, filled two K-steps at a time.  A K-step takes 64 bytes of every row, half a
    // 128-byte cache line; loading the halves of a line a K-step apart fetches the line twice
    // (64 KiB of other lines pass through the 32 KiB L1 of the CU in between).  The paired ring
    // issues the loads of steps 2n and 2n+1 of the same rows back to back, in every other
    // step.  Both target stages must be free then and the data is needed one step before its
    // MFMAs: A's stage frees when its step ends (5 stages), B's when its step begins (its
    // fragments are read and widened a step ahead: 4 stages).
    static constexpr bool PAIR = STAGES_ == 9;
    static constexpr int A_STAGES = PAIR ? 5 : STAGES_, B_STAGES = PAIR ? 4 : STAGES_;
    static constexpr int RING_BYTES = A_STAGES * A_BYTES + B_STAGES * B_BYTES;
    // Per-wave LDS area through which finished accumulator blocks are turned into row-major
    // order before they are stored: 16 rows x 64 int32, rows padded by 16 bytes so that the
    // 16 lanes of a ds_write_b128 (one row each) fall into different banks.  Used when it
    // fits beside the ring of every co-resident workgroup.
    static constexpr int XPOSE_PITCH = 64 * 4 + 16, XPOSE_BYTES = 16 * XPOSE_PITCH;
    static constexpr bool XPOSE = FN % 4 == 0 && OCC * (RING_BYTES + WAVES * XPOSE_BYTES) <= 160 * 1024;
    // Where that does not fit: half the area, 16 rows x 32 int32 without padding -- the 16-byte
    // chunk c of row r sits at chunk c ^ (r & 7), which keeps eight consecutive lanes of a
    // write (one row each) and of a read (the eight chunks of a row) in different banks.
    // (Measured on the tiles built for two workgroups per CU: 2-4 % on 256x128, nothing to
    // -1.5 % on the 64- and 128-row tiles, whose blocks keep going out as they are.)
    static constexpr int XHALF_BYTES = 16 * 128;
    static constexpr bool XHALF = !XPOSE && FN % 2 == 0 && BM * BN >= 256 * 128 && OCC * (RING_BYTES + WAVES * XHALF_BYTES) <= 160 * 1024;
    static constexpr int LDS_BYTES = RING_BYTES + (XPOSE ? WAVES * XPOSE_BYTES : XHALF ? WAVES * XHALF_BYTES : 0);
    // one DMA piece = one wave-wide 16-byte-per-lane load = 16 rows x 64 bytes
    static constexpr int A_PIECES = BM / 16 / WAVES, B_PIECES = BN / 16 / WAVES;
    static_assert(WM % 16 == 0 && WN % 16 == 0, "wave tile is a multiple of 16x16");
    static_assert(BM % (16 * WAVES) == 0 && BN % (16 * WAVES) == 0, "DMA pieces must divide evenly among the waves");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU");
    static_assert(STAGES >= 3 && STAGES <= 9, "ring depth");
    static_assert(OCC * LDS_BYTES <= 160 * 1024, "co-resident workgroups must fit the LDS together");
    static_assert(FM >= 2 && FM % 2 == 0 && FN >= 1, "pipeline needs an even number (>= 2) of A fragments per wave");
    static_assert((W_OPS * FN) % FM == 0, "B widening must split evenly over the sub-steps");
    static_assert(FN <= 2 * FM, "at most two B fragments are read per sub-step (two packed registers)");
    static_assert(FN <= 2 * FM, "at most two B fragments are read per sub-step (two packed registers)");
};

// TAIL: K % 128 may be 32, 64 or 96 (a short last K-step); the instantiation without it is
// the same kernel with that code left out.
template <class Cfg, int OUT = OUT_I32, bool TAIL = false>
__global__ void __launch_bounds__(Cfg::THREADS, Cfg::OCC * Cfg::THREADS / 256)
gemm_tile16_kernel(const GemmArgs p, const int tiles_m, const int tiles_n, const int group_m, const int ksplit)
{
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, FM = Cfg::FM, FN = Cfg::FN;
    constexpr int PITCH = Cfg::PITCH, STAGE = Cfg::STAGE_BYTES, WAVES = Cfg::WAVES;
    constexpr int A_PIECES = Cfg::A_PIECES, B_PIECES = Cfg::B_PIECES, NP = A_PIECES + B_PIECES;
    constexpr int ESZ = OUT == OUT_I32 ? 4 : 2;  // bytes per element of the output

    // (Every lambda below is marked always_inline: the state they share -- accumulators,
    // ring, load cursor -- lives in registers only as long as nothing is outlined.)
    extern __shared__ __align__(16) uint8_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / Cfg::WGN, wn = wave % Cfg::WGN;
    const int r = lane & 15, g = lane >> 4;

    // ---- work items ----
    // An item is one (K split, output tile) pair.  The grid is persistent: workgroup w runs
    // items w, w + G, w + 2G, ... (G = gridDim.x, at most the number of items) as ONE
    // continuous stream of K-steps, so the loads of the next item's first tiles are already
    // in flight while the current item finishes and its result is stored.  G is a multiple
    // of 8 whenever a workgroup gets more than one item, so an item's index modulo 8 is the
    // XCD it runs on and the XCD-contiguous renumbering applies to items as it would to
    // workgroups of a one-item-per-workgroup launch.
    const int G = gridDim.x;
    const int ntiles = tiles_m * tiles_n;
    const int nitems = ntiles * ksplit;
    const int Kb = p.K >> 1;
    // K is a multiple of 128, or with TAIL of 32.  A last K-step of fewer than 128 nibbles
    // (K % 128 = 32, 64 or 96) is loaded as the last 128 nibbles of the row -- in bounds,
    // 16-byte aligned -- and the part of it that the step before already covered is masked
    // away in the widening of B.
    const int kt_all = TAIL ? (p.K + BK - 1) / BK : p.K / BK;
    const int k_tail = TAIL ? (p.K & (BK - 1)) >> 5 : 0;  // valid 32-nibble chunks of that step, 0: none short
    const int kps = (kt_all + ksplit - 1) / ksplit;

    // item -> tile origin and K-step range [kt0, kt0 + KT); KT >= 1 (the launcher never
    // creates an empty split).  Tiles are numbered in columns of group_m.
    // (readfirstlane: the quotients are computed on the vector ALU; everything derived from
    // them is wave-uniform and belongs in scalar registers)
    //
    // When C takes plain 16-byte stores and K is not split, a tile's write-out is folded into
    // its last K-step.  The items are then numbered in two ranges: [0, nwhole) the tiles that
    // lie wholly inside the matrix, [nwhole, nitems) the ragged right column and bottom row of
    // tiles, whose stores are under the condition that their rows and columns exist.  A
    // workgroup's items ascend, so it runs its whole tiles first.  Otherwise (nwhole is 0: K
    // split, odd N, unaligned C) every item is written out by the guarded code after its last
    // K-step.
    const int ldc = c_stride(p);  // row stride of C in elements (N, unless this call computes a block of columns of a wider C)
    const bool vec_ok = (ldc & 3) == 0 && ((uintptr_t)p.C & (4 * ESZ - 1)) == 0;  // 4 elements per store
    const bool plain_c = vec_ok && ksplit == 1 && ldc < (1 << 21);
    const int full_m = p.M / BM, full_n = p.N / BN;
    const int nwhole = __builtin_amdgcn_readfirstlane(plain_c ? full_m * full_n : 0);
    auto locate = [&](const int item, int &m0, int &n0, int &kt0, int &KT) __attribute__((always_inline)) {
        // (both numberings are evaluated and one is picked: a branch here, with quotients
        // from the vector ALU on one side only, costs the scalar registers of everything
        // computed after it)
        const int rows = nwhole ? full_m : tiles_m, cols = nwhole ? full_n : tiles_n;
        const int gid = xcd_contiguous_id(nwhole ? min(item, nwhole - 1) : item, nwhole ? nwhole : nitems);
        const int ks = __builtin_amdgcn_readfirstlane(gid / ntiles);  // 0 unless K is split (then nwhole is 0)
        const int pid = gid - ks * ntiles;
        const int width = group_m * cols;
        const int first_m = (pid / width) * group_m;
        const int gsz = min(rows - first_m, group_m);
        const int tm_a = __builtin_amdgcn_readfirstlane(first_m + (pid % width) % gsz);
        const int tn_a = __builtin_amdgcn_readfirstlane((pid % width) / gsz);
        // Ragged tiles: the right column top to bottom (if N is ragged) and the bottom row left to
        // right, merged into one list in proportion (position q of nr holds right-column tile
        // floor(q right / nr) where that quotient steps, a bottom-row tile otherwise), and the
        // ragged items of one XCD (item % 8) take neighbouring positions of it, XCD 0 the head.
        // An XCD's ragged tiles then lie beside the whole tiles it runs last -- the whole tiles
        // are numbered top to bottom in the same XCD order -- and share panels with them and
        // with each other in its L2, instead of every ragged tile fetching two panels of its own.
        const bool ragged = nwhole != 0 && item >= nwhole;
        const int nr = max(nitems - nwhole, 1), right = tiles_n > full_n ? tiles_m : 0;
        const int e8 = max(item - nwhole, 0) + (nwhole & 7), x8 = e8 & 7, s8 = nwhole & 7;
        // positions before this XCD's: ragged items on lower XCDs, F(t) = integers in [0, t) with residue < x8
        const int f_hi = ((s8 + nr) >> 3) * x8 + min((s8 + nr) & 7, x8), f_lo = min(s8, x8);
        const int q = __builtin_amdgcn_readfirstlane(min(f_hi - f_lo + (e8 >> 3) - (x8 < s8 ? 1 : 0), nr - 1));
        const int r0 = __builtin_amdgcn_readfirstlane(q * right / nr), r1 = __builtin_amdgcn_readfirstlane((q + 1) * right / nr);
        const int tm_b = r1 > r0 ? r0 : full_m, tn_b = r1 > r0 ? full_n : q - r0;
        m0 = (ragged ? tm_b : tm_a) * BM;
        n0 = (ragged ? tn_b : tn_a) * BN;
        kt0 = __builtin_amdgcn_readfirstlane(min(ks * kps, kt_all - 1));
        KT = __builtin_amdgcn_readfirstlane(max(min(kps, kt_all - ks * kps), 1));
    };

    // ---- global -> LDS: piece q of this wave covers tile rows (q*WAVES + wave)*16 .. +15.
    // The hardware puts lane l's 16 bytes at (wave-uniform LDS base) + 16*l, i.e. row l/4,
    // physical chunk l%4 of the piece; the lane therefore fetches the logical chunk that
    // the swizzle (chunk ^ ((row >> 1) & 3)) maps there.  Rows past the edge of the matrix
    // are clamped (their products are never stored).
    //
    // The loads run AHEAD K-steps in front of the MFMAs, through item boundaries, so they
    // have a cursor of their own: (item, K-step within the item) and the per-lane row
    // offsets of that item's tile.  Every item is padded to an even number of K-steps (the
    // padding step re-reads the last real tile; its products are masked to zero).
    const int dma_row = lane >> 2;
    const int dma_ch = (lane & 3) ^ ((dma_row >> 1) & 3);
    uint32_t a_goff[A_PIECES], b_goff[B_PIECES];
    int d_item = blockIdx.x, d_kt = 0, d_kt0, d_KT;
    // (scalar part first: only dma_base stays live in a vector register between items)
    const int dma_base = wave * 16 + dma_row;
    const uint32_t dma_col = dma_ch * 16;
    auto cursor_load = [&]() __attribute__((always_inline)) {
        int m0, n0;
        locate(d_item, m0, n0, d_kt0, d_KT);
#pragma unroll
        for (int q = 0; q < A_PIECES; ++q)
            a_goff[q] = (uint32_t)min((m0 + q * WAVES * 16) + dma_base, p.M - 1) * (uint32_t)Kb + dma_col;
#pragma unroll
        for (int q = 0; q < B_PIECES; ++q)
            b_goff[q] = (uint32_t)min((n0 + q * WAVES * 16) + dma_base, p.N - 1) * (uint32_t)Kb + dma_col;
    };
    const uint8_t *a_src, *b_src;  // operand base + K offset of the step the cursor points at
    const uint8_t *a_src2 = nullptr, *b_src2 = nullptr;  // paired ring: the same for the step after it
    auto cursor_point = [&]() __attribute__((always_inline)) {
        const int step = d_kt0 + min(d_kt, d_KT - 1);
        const int kofs = (TAIL && k_tail != 0 && step == kt_all - 1) ? Kb - BK / 2 : step * (BK / 2);
        a_src = p.A + kofs;
        b_src = p.B + kofs;
        if constexpr (Cfg::PAIR) {
            const int step2 = d_kt0 + min(d_kt + 1, d_KT - 1);
            const int kofs2 = (TAIL && k_tail != 0 && step2 == kt_all - 1) ? Kb - BK / 2 : step2 * (BK / 2);
            a_src2 = p.A + kofs2;
            b_src2 = p.B + kofs2;
        }
    };
    // Past the last item the cursor stays on the last step: those loads land in stages
    // nobody reads any more.
    auto cursor_advance = [&]() __attribute__((always_inline)) {
        d_kt += Cfg::PAIR ? 2 : 1;  // (an item's steps come in pairs: two steps on never pass the item's end)
        if (d_kt >= d_KT + (d_KT & 1)) {
            if (d_item + G < nitems) {
                d_item += G;
                d_kt = 0;
                cursor_load();
            } else {
                d_kt = d_KT - 1;
            }
        }
        cursor_point();
    };
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const uint32_t dma_lds = __builtin_amdgcn_readfirstlane(lds0 + wave * 16 * PITCH);

    // piece index -> (operand, piece): one wave-wide load of the cursor's step into `stage_byte`
    auto dma_piece = [&](int piece, int stage_byte) __attribute__((always_inline)) {
        if (piece < A_PIECES) {
            const uint32_t dst = dma_lds + stage_byte + piece * WAVES * 16 * PITCH;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(a_goff[piece]), "s"(a_src) : "memory", "m0");
        } else {
            const int b = piece - A_PIECES;
            const uint32_t dst = dma_lds + stage_byte + Cfg::A_BYTES + b * WAVES * 16 * PITCH;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(b_goff[b]), "s"(b_src) : "memory", "m0");
        }
    };

    // The same in two halves, two MFMA slots apart, for the K loop: the LDS address goes into
    // M0 first (the slots in between are the wait state the load needs after a write of M0),
    // the load itself follows alone -- five instructions in one slot are more than the shadow
    // of that slot's MFMA hides.  Nothing else in this kernel uses M0.
    // (These statements read the operand's base pointer from scalar registers.  If the
    // compiler fetched it into them with a vector instruction just before -- v_readlane, when
    // it keeps scalar registers in the lanes of a vector one -- the load would have to wait
    // five wait states, which the compiler sees to for its own memory instructions only: the
    // build scans the generated code for that and fails if it finds it.)
    auto dma_setup = [&](int piece, int stage_byte) __attribute__((always_inline)) {
        const uint32_t dst = dma_lds + stage_byte +
                             (piece < A_PIECES ? piece * WAVES * 16 * PITCH : Cfg::A_BYTES + (piece - A_PIECES) * WAVES * 16 * PITCH);
        asm volatile("s_mov_b32 m0, %0" ::"s"(dst) : "memory", "m0");
    };
    auto dma_issue = [&](int piece) __attribute__((always_inline)) {
        if (piece < A_PIECES) asm volatile("global_load_lds_dwordx4 %0, %1" ::"v"(a_goff[piece]), "s"(a_src) : "memory");
        else asm volatile("global_load_lds_dwordx4 %0, %1" ::"v"(b_goff[piece - A_PIECES]), "s"(b_src) : "memory");
    };

    // Paired ring: piece q of the cursor's step (second = false) or of the step after it, into
    // the stage at byte offset `at` of that operand's ring.
    auto pair_setup = [&](int piece, int at) __attribute__((always_inline)) {
        const uint32_t dst = dma_lds + at + (piece < A_PIECES ? piece : piece - A_PIECES) * WAVES * 16 * PITCH;
        asm volatile("s_mov_b32 m0, %0" ::"s"(dst) : "memory", "m0");
    };
    auto pair_issue = [&](int piece, bool second) __attribute__((always_inline)) {
        if (piece < A_PIECES) asm volatile("global_load_lds_dwordx4 %0, %1" ::"v"(a_goff[piece]), "s"(second ? a_src2 : a_src) : "memory");
        else asm volatile("global_load_lds_dwordx4 %0, %1" ::"v"(b_goff[piece - A_PIECES]), "s"(second ? b_src2 : b_src) : "memory");
    };
    auto pair_piece = [&](int piece, int at, bool second) __attribute__((always_inline)) {
        const uint32_t dst = dma_lds + at + (piece < A_PIECES ? piece : piece - A_PIECES) * WAVES * 16 * PITCH;
        if (piece < A_PIECES)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(a_goff[piece]), "s"(second ? a_src2 : a_src) : "memory", "m0");
        else
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(b_goff[piece - A_PIECES]), "s"(second ? b_src2 : b_src) : "memory", "m0");
    };

    // ---- fragment reads: lane -> row r of a 16-row fragment, chunk g (32 nibbles) ----
    // (rows of consecutive fragments differ by 16, which leaves (row >> 1) & 3 unchanged)
    const int a_row = wm * Cfg::WM + r, b_row = wn * Cfg::WN + r;
    const int a_rd = a_row * PITCH + ((g ^ ((a_row >> 1) & 3)) << 4);
    const int b_rd = (Cfg::PAIR ? 0 : Cfg::A_BYTES) + b_row * PITCH + ((g ^ ((b_row >> 1) & 3)) << 4);  // (paired ring: the B stages have offsets of their own)
    auto read_a = [&](int stage_byte, int i) -> v4i {
        return *reinterpret_cast<const v4i *>(smem + stage_byte + a_rd + i * 16 * PITCH);
    };
    auto read_b = [&](int stage_byte, int j) -> v4i {
        return *reinterpret_cast<const v4i *>(smem + stage_byte + b_rd + j * 16 * PITCH);
    };

    // acc[i][j]: B rows feed MFMA source 0 and A rows source 1, so a lane ends up with
    // 4 consecutive n for one m -- one 16-byte store into row-major C.
    v4i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = v4i{0, 0, 0, 0};

    // ---- prologue: steps 0 .. STAGES-2 of the stream on their way into stages 0 .. STAGES-2;
    // wait for 0 and 1 ----
    constexpr int STAGES = Cfg::PAIR ? 4 : Cfg::STAGES, AHEAD = STAGES - 1;  // step s+AHEAD is issued during step s (paired ring: steps s+3 and s+4 during every odd step s)
    constexpr int B_BASE = Cfg::A_STAGES * Cfg::A_BYTES;  // paired ring: where the B stages begin
    cursor_load();
    cursor_point();
    if constexpr (Cfg::PAIR) {
        // steps 0..3 into stages 0..3 of both rings; wait for 0 and 1
#pragma unroll
        for (int t = 0; t < 4; t += 2) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int q = 0; q < NP; ++q) pair_piece(q, q < A_PIECES ? (t + h) * Cfg::A_BYTES : B_BASE + (t + h) * Cfg::B_BYTES, h == 1);
            cursor_advance();
        }
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NP) : "memory");
    } else {
#pragma unroll
        for (int t = 0; t < AHEAD; ++t) {
#pragma unroll
            for (int q = 0; q < NP; ++q) dma_piece(q, t * STAGE);
            cursor_advance();
        }
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((AHEAD - 2) * NP) : "memory");
    }
    __syncthreads();

    // B fragments of the current step (widened) and of the next (being widened); the two
    // sets swap roles every K-step, so the K loop is unrolled by two.  A: ping-pong per
    // sub-step (FM is even, so the parity carries over K-steps).
    v4i b_ev[2][FN], b_od[2][FN], b_pk[2];
    v4i a_ev[2], a_od[2], a_pk[2];
#pragma unroll
    for (int j = 0; j < FN; ++j) x16_expand(read_b(Cfg::PAIR ? B_BASE : 0, j), b_ev[0][j], b_od[0][j]);
    x16_expand(read_a(0, 0), a_ev[0], a_od[0]);
    a_pk[1] = read_a(0, 1);

    // byte offsets of the ring stages: step s, s+1, ..., and the one being (re)filled
    int ring[STAGES];
#pragma unroll
    for (int t = 0; t < STAGES; ++t) ring[t] = t * STAGE;
    // Paired ring, during step s: a_ring[t] holds (or waits for) A of step s+t, t = 0..4;
    // b_ring[t] B of step s+t, t = 1..3, and b_ring[0] is free (B of step s went into
    // registers during step s-1).
    int a_ring[Cfg::PAIR ? 5 : 1], b_ring[Cfg::PAIR ? 4 : 1];
    if constexpr (Cfg::PAIR) {
#pragma unroll
        for (int t = 0; t < 5; ++t) a_ring[t] = t * Cfg::A_BYTES;
#pragma unroll
        for (int t = 0; t < 4; ++t) b_ring[t] = B_BASE + t * Cfg::B_BYTES;
    }

    // Widening op k (0..W-1) of a packed fragment, W = 10: for each half (dwords 2h, 2h+1) one
    // 64-bit shift of the pair (the nibble that crosses into the upper dword is masked away
    // with the rest), then a mask each for the even and the odd nibbles of both dwords.
    auto widen_op = [&](auto k_, const v4i &pk, v4i &ev, v4i &od, const uint32_t mask) __attribute__((always_inline)) {
        constexpr int k = decltype(k_)::value, h = k / 5, part = k % 5, d = 2 * h + (part - 1) / 2;
        if constexpr (part == 0) {
            const v2i t = shl4_pair(pk[2 * h], pk[2 * h + 1]);
            ev[2 * h] = t.x;
            ev[2 * h + 1] = t.y;
        }
        else if constexpr (part % 2 == 1) ev[d] = (int)((uint32_t)ev[d] & mask);
        else od[d] = (int)((uint32_t)pk[d] & mask);
    };

    // The nibble mask lives in an SGPR (opaque to the compiler): a VALU instruction with
    // an SGPR operand is half the size of one with a 32-bit literal.
    uint32_t amask;
    asm volatile("s_mov_b32 %0, 0xf0f0f0f0" : "=s"(amask));
    // TAIL: B's mask is a vector register: all nibbles, none (an item's padding step), or per
    // lane for a short last step -- lane (r, g) holds chunk g of the step, and of the 128
    // nibbles loaded for that step the first 4 - k_tail chunks belong to the step before.
    uint32_t vmask_full = 0, vmask_tail = 0;
    if constexpr (TAIL) {
        asm volatile("v_mov_b32 %0, 0xf0f0f0f0" : "=v"(vmask_full));
        vmask_tail = (k_tail == 0 || g >= 4 - k_tail) ? vmask_full : 0u;
    }

    // ---- writing a finished tile ----
    // A 16x16 block leaves the MFMA with lane (r, g) holding row r, columns 4g..4g+3: a
    // wave-wide 16-byte store of it touches 16 rows, and consecutive lanes sit in different
    // rows.  The memory pipeline of a CU takes such stores more than three times slower
    // than stores in which every 4 consecutive lanes cover 64 contiguous bytes (measured:
    // 6.4 us against 2.1 us for the 256 KiB of one tile).  Where the LDS has room, four
    // blocks that are neighbours along n (16 rows x 64 columns) therefore pass through a
    // per-wave LDS area: written as they come, read back with 16 consecutive lanes per row
    // (4 rows x 256 bytes per store).  The accumulators are only touched through asm
    // statements: an ordinary read or write inside the loop makes the register allocator
    // treat them as general values and copy them around.
    int c_item = blockIdx.x, c_kt = 0, c_m0, c_n0, c_kt0, c_KT;  // the item being contracted
    char *tile_c = nullptr;  // its corner in C (wave-uniform)
    v4i *split_ws = nullptr;  // this lane's place in the item's workspace slot (K split with a workspace)
    // scaled output: this lane's scales for the item, as the MFMA leaves a block (row r of
    // every block row, columns 4g..4g+3 of every block column)
    typedef float v4f __attribute__((ext_vector_type(4)));
    float rs_reg[OUT != OUT_I32 ? FM : 1];
    v4f cs_reg[OUT != OUT_I32 ? FN : 1];
    v4i zero4;
    asm volatile("v_mov_b32 %0, 0" : "=v"(zero4.x));  // (opaque, so the MFMA operand is a plain register tuple)
    zero4.y = zero4.z = zero4.w = zero4.x;
    // accumulator block -> registers, cleared behind the read, factor 256 dropped
    auto take_block = [&](auto ib_, auto j_) __attribute__((always_inline)) -> v4i {
        constexpr int ib = decltype(ib_)::value, j = decltype(j_)::value;
        v4i v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = e == 0 ? acc_read_first(acc[ib][j][e]) : acc_read(acc[ib][j][e]);
        mfma16_zero(acc[ib][j], zero4);
        v.x >>= 8; v.y >>= 8; v.z >>= 8; v.w >>= 8;
        if constexpr (OUT != OUT_I32) {
            // scaled output: from here on the four registers hold fp32 bit patterns
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = __builtin_bit_cast(int, scaled(v[e], rs_reg[ib], cs_reg[j][e]));
        }
        return v;
    };
    // four fp32 bit patterns -> four 16-bit floats in two registers
    auto pack16 = [&](const v4i v) __attribute__((always_inline)) -> v2i {
        uint32_t h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int bits = v[e];  // (by value: a bit cast applied to the vector element itself reads element 0)
            h[e] = round16<OUT == OUT_I32 ? OUT_F16 : OUT>(__builtin_bit_cast(float, bits));
        }
        return v2i{(int)(h[0] | (h[1] << 16)), (int)(h[2] | (h[3] << 16))};
    };
    // byte offsets of this lane from the tile's corner (32 bits are enough for the rows of one
    // tile when N is below 2^21): as the MFMA leaves a block, and as the LDS area is read back
    const uint32_t lane_blk = ((uint32_t)(wm * Cfg::WM + r) * (uint32_t)ldc + (uint32_t)(wn * Cfg::WN + g * 4)) * (uint32_t)ESZ;
    const uint32_t lane_row = ((uint32_t)(wm * Cfg::WM + (lane >> 4)) * (uint32_t)ldc + (uint32_t)(wn * Cfg::WN + (lane & 15) * 4)) * (uint32_t)ESZ;
    uint8_t *const xp = smem + Cfg::RING_BYTES + wave * Cfg::XPOSE_BYTES;
    const int xp_wr = r * Cfg::XPOSE_PITCH + g * 16, xp_rd = (lane >> 4) * Cfg::XPOSE_PITCH + (lane & 15) * 16;
    const uint32_t xp_wr_lds = lds0 + Cfg::RING_BYTES + wave * Cfg::XPOSE_BYTES + xp_wr;  // the same as an LDS address
    v4i xr[4];
    // A tile that sticks out of C is written the same way as a whole one, every store with the
    // lanes switched off whose row or columns do not exist.  The store is issued under a lane
    // mask set and restored around it, not under a branch: the write-out stays one basic block
    // (with branches between the MFMA slots the register allocator spills), and the address
    // stays base register + 32-bit lane offset.  rows_left / cols_left are what the matrix has
    // from this lane's first row and column of the tile on, in the order the stores below use
    // (set per item; N % 4 == 0, so a lane's four columns are inside or outside together).
    // A store whose lanes are all off may or may not count as issued, so the last K-step of
    // such a tile allows for none of its stores in its wait.  Whole tiles keep their plain
    // stores (the conditions cost ten instructions a store: 1 to 10 % on whole-tile shapes
    // when every tile went this way), so the kernel has the K loop three times: whole tiles,
    // tiles that stick out (`edge`), and the guarded write-out after the last K-step.
    int rows_left = 0, cols_left = 0;
    // (The two comparisons sit inside the statement as well: written in C++, the compiler
    // works all the lane masks of a tile out ahead -- 64 register pairs -- and runs out of scalar
    // registers.  s_nop 4: the compiler may have produced the base register pair with a vector
    // instruction just before this statement -- v_readlane, when it keeps scalar registers in
    // the lanes of a vector one -- and a memory instruction must not read such a register
    // within five wait states; the compiler sees to that for its own instructions and cannot
    // for the store in here.)
    auto store_lanes = [&](char *const base, const uint32_t lane_off, const auto v, auto row_, auto col_) __attribute__((always_inline)) {
        constexpr int row = decltype(row_)::value, col = decltype(col_)::value;
        const int rl = rows_left, cl = cols_left;   // (an asm operand cannot name a captured variable)
        uint64_t saved, on;
        if constexpr (sizeof(v) == 16)
            asm volatile("s_nop 4\n\tv_cmp_lt_i32_e32 vcc, %7, %5\n\ts_mov_b64 %1, vcc\n\tv_cmp_lt_i32_e32 vcc, %8, %6\n\ts_and_b64 %1, %1, vcc\n\t"
                         "s_mov_b64 %0, exec\n\ts_mov_b64 exec, %1\n\tglobal_store_dwordx4 %2, %3, %4\n\ts_mov_b64 exec, %0"
                         : "=&s"(saved), "=&s"(on) : "v"(lane_off), "v"(v), "s"(base), "v"(rl), "v"(cl), "n"(row), "n"(col) : "memory", "vcc");
        else
            asm volatile("s_nop 4\n\tv_cmp_lt_i32_e32 vcc, %7, %5\n\ts_mov_b64 %1, vcc\n\tv_cmp_lt_i32_e32 vcc, %8, %6\n\ts_and_b64 %1, %1, vcc\n\t"
                         "s_mov_b64 %0, exec\n\ts_mov_b64 exec, %1\n\tglobal_store_dwordx2 %2, %3, %4\n\ts_mov_b64 exec, %0"
                         : "=&s"(saved), "=&s"(on) : "v"(lane_off), "v"(v), "s"(base), "v"(rl), "v"(cl), "n"(row), "n"(col) : "memory", "vcc");
    };
    // Whole tile, through the LDS: part t = 0..7 of blocks (ib, 4*grp .. 4*grp+3), one part per
    // MFMA slot.  Parts 0..3 write one block each; the read-back of row quartet k and its
    // store are two parts apart, so the store does not wait for the LDS.
    auto write_group = [&](auto ib_, auto grp_, auto t_, auto edge_) __attribute__((always_inline)) {
        constexpr int ib = decltype(ib_)::value, grp = decltype(grp_)::value, t = decltype(t_)::value;
        constexpr bool edge = decltype(edge_)::value;
        auto read_back = [&](auto k_) __attribute__((always_inline)) {
            constexpr int k = decltype(k_)::value;
            xr[k] = *reinterpret_cast<const v4i *>(xp + xp_rd + 4 * k * Cfg::XPOSE_PITCH);
        };
        auto store_rows = [&](auto k_) __attribute__((always_inline)) {
            constexpr int k = decltype(k_)::value;
            char *const at = tile_c + ((size_t)(ib * 16 + 4 * k) * ldc + grp * 64) * ESZ;  // wave-uniform
            if constexpr (OUT == OUT_I32) {
                v4i v = xr[k];
                v.x >>= 8; v.y >>= 8; v.z >>= 8; v.w >>= 8;
                if constexpr (edge) store_lanes(at, lane_row, v, std::integral_constant<int, ib * 16 + 4 * k>{}, std::integral_constant<int, grp * 64>{});
                else *reinterpret_cast<v4i *>(at + lane_row) = v;
            } else {
                if constexpr (edge) store_lanes(at, lane_row, pack16(xr[k]), std::integral_constant<int, ib * 16 + 4 * k>{}, std::integral_constant<int, grp * 64>{});
                else *reinterpret_cast<v2i *>(at + lane_row) = pack16(xr[k]);
            }
        };
        if constexpr (t < 4) {
            if constexpr (OUT == OUT_I32) {
                // int32: the block goes to the LDS area as it is -- 256 x the result, straight
                // from its accumulator registers (a DS instruction takes them as data) -- and is
                // cleared behind; the factor is dropped after the read-back, in row order
                asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(xp_wr_lds), "a"(acc[ib][4 * grp + t]), "n"(64 * t) : "memory");
                mfma16_zero(acc[ib][4 * grp + t], zero4);
            } else {
                *reinterpret_cast<v4i *>(xp + xp_wr + 64 * t) = take_block(ib_, std::integral_constant<int, 4 * grp + t>{});
            }
        }
        if constexpr (t == 3) read_back(std::integral_constant<int, 0>{});
        if constexpr (t == 4) read_back(std::integral_constant<int, 1>{});
        if constexpr (t == 5) { read_back(std::integral_constant<int, 2>{}); store_rows(std::integral_constant<int, 0>{}); }
        if constexpr (t == 6) { read_back(std::integral_constant<int, 3>{}); store_rows(std::integral_constant<int, 1>{}); }
        if constexpr (t == 7) { store_rows(std::integral_constant<int, 2>{}); store_rows(std::integral_constant<int, 3>{}); }
    };
    // Whole tile through the half-size area: part t = 0..3 of blocks (ib, 2*h) and (ib, 2*h + 1).
    // Parts 0 and 1 write a block each -- and store the two row octets (8 rows x 128 bytes, eight
    // consecutive lanes per row) that the half group before this one read back in its parts 2
    // and 3; the last half group of a tile leaves its two for flush_half().
    const uint32_t lane_half = ((uint32_t)(wm * Cfg::WM + (lane >> 3)) * (uint32_t)ldc + (uint32_t)(wn * Cfg::WN + (lane & 7) * 4)) * (uint32_t)ESZ;
    uint8_t *const xh = smem + Cfg::RING_BYTES + wave * Cfg::XHALF_BYTES;
    const int xh_wr = r * 128 + ((g ^ (r & 7)) << 4);                             // block 2h; block 2h + 1 is 64 bytes (chunk bit 2) away
    const int xh_rd = (lane >> 3) * 128 + (((lane & 7) ^ (lane >> 3)) << 4);      // rows 0..7; rows 8..15: + 1024
    auto store_half = [&](auto ib_, auto h_, auto k_, auto edge_) __attribute__((always_inline)) {
        constexpr bool edge = decltype(edge_)::value;
        constexpr int ib = decltype(ib_)::value, h = decltype(h_)::value, k = decltype(k_)::value;
        char *const at = tile_c + ((size_t)(ib * 16 + 8 * k) * ldc + h * 32) * ESZ;  // wave-uniform
        if constexpr (OUT == OUT_I32) {
            v4i v = xr[k];
            v.x >>= 8; v.y >>= 8; v.z >>= 8; v.w >>= 8;
            if constexpr (edge) store_lanes(at, lane_half, v, std::integral_constant<int, ib * 16 + 8 * k>{}, std::integral_constant<int, h * 32>{});
            else *reinterpret_cast<v4i *>(at + lane_half) = v;
        } else {
            if constexpr (edge) store_lanes(at, lane_half, pack16(xr[k]), std::integral_constant<int, ib * 16 + 8 * k>{}, std::integral_constant<int, h * 32>{});
            else *reinterpret_cast<v2i *>(at + lane_half) = pack16(xr[k]);
        }
    };
    auto write_half = [&](auto ib_, auto h_, auto t_, auto edge_) __attribute__((always_inline)) {
        constexpr int ib = decltype(ib_)::value, h = decltype(h_)::value, t = decltype(t_)::value;
        constexpr int pib = h > 0 ? ib : ib - 1, ph = h > 0 ? h - 1 : FN / 2 - 1;  // the half group before this one
        if constexpr (t < 2) {
            const int at = t == 0 ? xh_wr : xh_wr ^ 64;
            if constexpr (OUT == OUT_I32) {
                const uint32_t at_lds = lds0 + Cfg::RING_BYTES + wave * Cfg::XHALF_BYTES + at;
                asm volatile("ds_write_b128 %0, %1" ::"v"(at_lds), "a"(acc[ib][2 * h + t]) : "memory");
                mfma16_zero(acc[ib][2 * h + t], zero4);
            } else {
                *reinterpret_cast<v4i *>(xh + at) = take_block(ib_, std::integral_constant<int, 2 * h + t>{});
            }
            if constexpr (pib >= 0) store_half(std::integral_constant<int, pib>{}, std::integral_constant<int, ph>{}, t_, edge_);
        }
        if constexpr (t == 2) xr[0] = *reinterpret_cast<const v4i *>(xh + xh_rd);
        if constexpr (t == 3) xr[1] = *reinterpret_cast<const v4i *>(xh + xh_rd + 1024);
    };
    auto flush_half = [&](auto edge_) __attribute__((always_inline)) {
        store_half(std::integral_constant<int, FM - 1>{}, std::integral_constant<int, FN / 2 - 1>{}, std::integral_constant<int, 0>{}, edge_);
        store_half(std::integral_constant<int, FM - 1>{}, std::integral_constant<int, FN / 2 - 1>{}, std::integral_constant<int, 1>{}, edge_);
    };
    // Whole tile, no room in the LDS: block (ib, j) stored as it is, in two parts.
    auto write_block = [&](auto ib_, auto j_, auto t_, auto edge_) __attribute__((always_inline)) {
        constexpr int ib = decltype(ib_)::value, j = decltype(j_)::value, t = decltype(t_)::value;
        if constexpr (t == 0) {
            xr[0] = take_block(ib_, j_);
        } else {
            char *const at = tile_c + ((size_t)(ib * 16) * ldc + j * 16) * ESZ;  // wave-uniform
            if constexpr (decltype(edge_)::value) {
                if constexpr (OUT == OUT_I32) store_lanes(at, lane_blk, xr[0], std::integral_constant<int, ib * 16>{}, std::integral_constant<int, j * 16>{});
                else store_lanes(at, lane_blk, pack16(xr[0]), std::integral_constant<int, ib * 16>{}, std::integral_constant<int, j * 16>{});
            } else {
                if constexpr (OUT == OUT_I32) *reinterpret_cast<v4i *>(at + lane_blk) = xr[0];
                else *reinterpret_cast<v2i *>(at + lane_blk) = pack16(xr[0]);
            }
        }
    };
    // Slot s of 2*FN for the blocks of row ib of a whole tile
    auto write_whole = [&](auto ib_, auto s_, auto edge_) __attribute__((always_inline)) {
        constexpr int s = decltype(s_)::value;
        if constexpr (Cfg::XPOSE) write_group(ib_, std::integral_constant<int, s / 8>{}, std::integral_constant<int, s % 8>{}, edge_);
        else if constexpr (Cfg::XHALF) write_half(ib_, std::integral_constant<int, s / 4>{}, std::integral_constant<int, s % 4>{}, edge_);
        else write_block(ib_, std::integral_constant<int, s / 2>{}, std::integral_constant<int, s % 2>{}, edge_);
    };
    // Any tile: guarded stores (ragged edges, odd N or unaligned C, K-split partial sums)
    auto write_guarded = [&](auto ib_, auto j_) __attribute__((always_inline)) {
        constexpr int ib = decltype(ib_)::value, j = decltype(j_)::value;
        const v4i v = take_block(ib_, j_);
        if constexpr (OUT == OUT_I32) {
            if (split_ws != nullptr) {
                // K-split partial sums with a workspace: the block as it is, 16 bytes per lane
                // (whole 1 KiB lines per wave; the padding of a ragged tile has room there)
                split_ws[(ib * FN + j) * 64] = v;
                return;
            }
        }
        const int m = (c_m0 + ib * 16) + (wm * Cfg::WM + r), n = (c_n0 + j * 16) + (wn * Cfg::WN + g * 4);
        if constexpr (OUT != OUT_I32) {
            if (m < p.M) {
                uint16_t *drow = reinterpret_cast<uint16_t *>(p.C) + (size_t)m * ldc;
                const v2i o = pack16(v);
                if (vec_ok && n + 3 < p.N) {
                    *reinterpret_cast<v2i *>(drow + n) = o;
                } else if (n + 3 < p.N) {
                    *reinterpret_cast<v2i_half_aligned *>(drow + n) = o;
                } else {
                    if (n < p.N) drow[n] = (uint16_t)o.x;
                    if (n + 1 < p.N) drow[n + 1] = (uint16_t)((uint32_t)o.x >> 16);
                    if (n + 2 < p.N) drow[n + 2] = (uint16_t)o.y;
                    if (n + 3 < p.N) drow[n + 3] = (uint16_t)((uint32_t)o.y >> 16);
                }
            }
        } else if (m < p.M) {
            int32_t *crow = p.C + (size_t)m * ldc;
            if (ksplit > 1) {
                // every partial accumulator is a multiple of 256, so the shifted partials add
                // up to the shifted total; integer atomics make the order irrelevant
                // (this branch only runs without a workspace: see below)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < p.N) __hip_atomic_fetch_add(crow + n + e, v[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else if (vec_ok && n + 3 < p.N) {
                *reinterpret_cast<v4i *>(crow + n) = v;
            } else if (n + 3 < p.N) {
                *reinterpret_cast<v4i_elem_aligned *>(crow + n) = v;
            } else {
                if (n < p.N) crow[n] = v.x;
                if (n + 1 < p.N) crow[n + 1] = v.y;
                if (n + 2 < p.N) crow[n + 2] = v.z;
                if (n + 3 < p.N) crow[n + 3] = v.w;
            }
        }
    };

    // One K-step: contracts the step in ring[0] (its B fragments sit widened in register set
    // bs), reads and widens the B fragments of the step in ring[1] with `bmask` (zero when
    // that step is an item's padding), and issues the cursor's loads into the last stage.
    // In the last step of a whole tile, row i-1 of the accumulator blocks is final once
    // sub-step i begins: its write-out rides in the slots of sub-step i instead of stalling
    // the matrix cores afterwards (row FM-1 is left to the caller).
    auto k_step = [&](const uint32_t bmask, auto bs_tag, auto last_tag) __attribute__((always_inline)) {
        constexpr int bs = decltype(bs_tag)::value;
        constexpr bool last = decltype(last_tag)::value != 0;  // 1: the last step of a whole tile, 2: of one that sticks out of C (`edge`)
        constexpr bool edge = decltype(last_tag)::value == 2;
        constexpr int SLOTS = 2 * FN;                // MFMAs per sub-step
        constexpr int W = Cfg::W_OPS;
        constexpr int BSHARE = W * FN / FM;          // B widening ops per sub-step
        constexpr int NOPS = W + BSHARE;             // VALU ops per sub-step, spread over slots 1..SLOTS-1
        static_for<0, FM>([&](auto i_) {
            constexpr int i = decltype(i_)::value;
            constexpr int pa = i & 1;
            static_for<0, SLOTS>([&](auto s_) {
                constexpr int s = decltype(s_)::value;
                // -- the MFMA of this slot: even-nibble K-slice for all j, then the odd one --
                if constexpr (s < FN) mfma16_acc(acc[i][s], b_ev[bs][s], a_ev[pa]);
                else mfma16_acc(acc[i][s - FN], b_od[bs][s - FN], a_od[pa]);
                if constexpr (s == 0) {
                    // -- LDS reads: B fragments of the next step whose widening starts in this
                    //    sub-step, and the A fragment two sub-steps ahead --
                    static_for<0, FN>([&](auto j_) {
                        constexpr int j = decltype(j_)::value;
                        if constexpr ((W * j) / BSHARE == i) b_pk[j & 1] = read_b(Cfg::PAIR ? b_ring[1] : ring[1], j);
                    });
                    constexpr int i2 = i + 2;
                    if constexpr (Cfg::PAIR) a_pk[pa] = read_a(i2 >= FM ? a_ring[1] : a_ring[0], i2 % FM);
                    else a_pk[pa] = read_a(i2 >= FM ? ring[1] : ring[0], i2 % FM);
                } else {
                    // -- this slot's share of the widening work: ops [lo, hi) of the sub-step's
                    //    list: W ops for the next A fragment, then BSHARE ops of the next B --
                    constexpr int lo = (s - 1) * NOPS / (SLOTS - 1), hi = s * NOPS / (SLOTS - 1);
                    static_for<lo, hi>([&](auto o_) {
                        constexpr int o = decltype(o_)::value;
                        if constexpr (o < W) {
                            widen_op(std::integral_constant<int, o>{}, a_pk[pa ^ 1], a_ev[pa ^ 1], a_od[pa ^ 1], amask);
                        } else {
                            constexpr int gop = i * BSHARE + (o - W);  // index into the K-step's B op list
                            constexpr int j = gop / W;
                            widen_op(std::integral_constant<int, gop % W>{}, b_pk[j & 1], b_ev[bs ^ 1][j], b_od[bs ^ 1][j], bmask);
                        }
                    });
                }
                // -- write-out of the accumulator row finished one sub-step ago --
                if constexpr (last && i >= 1) write_whole(std::integral_constant<int, i - 1>{}, s_, std::integral_constant<bool, edge>{});
                // -- DMA pieces of the step AHEAD of this one, one sub-step apart --
                // (With a ring of three stages the loads issued in a step must have landed
                // at its end.  In a last step they all go out in sub-step 0, ahead of the
                // first store, so that "all but the stores" can be waited for.)
                constexpr bool bunched = !Cfg::PAIR && last && AHEAD == 2;
                constexpr bool split = !Cfg::PAIR && !bunched && NP <= FM && SLOTS >= 4;  // at most one piece per sub-step
                if constexpr (Cfg::PAIR && bs == 1) {
                    // paired ring, odd steps: piece i of step s+3 in the first half of the sub-step,
                    // the same rows of step s+4 (the other half of their cache lines) in the second
                    static_for<0, NP>([&](auto q_) {
                        constexpr int q = decltype(q_)::value;
                        if constexpr (q * FM / NP == i) {
                            // the pieces of this sub-step are q = first .. first + cnt - 1; each gets two loads,
                            // `spacing` slots apart, M0 written two slots ahead of each
                            constexpr int first = (i * NP + FM - 1) / FM, last1 = ((i + 1) * NP + FM - 1) / FM, cnt = last1 > first ? last1 - first : 1;
                            constexpr int spacing = SLOTS / (2 * cnt), at1 = 2 * (q - first) * spacing + spacing - 1, at2 = at1 + spacing;
                            static_assert(spacing >= 4, "too many pieces per sub-step for the slots it has");
                            if constexpr (s == at1 - 2) pair_setup(q, q < A_PIECES ? a_ring[3] : b_ring[3]);
                            if constexpr (s == at1) pair_issue(q, false);
                            if constexpr (s == at2 - 2) pair_setup(q, q < A_PIECES ? a_ring[4] : b_ring[0]);
                            if constexpr (s == at2) pair_issue(q, true);
                        }
                    });
                }
                if constexpr (split && s == SLOTS - 3) {
                    static_for<0, NP>([&](auto q_) {
                        constexpr int q = decltype(q_)::value;
                        if constexpr (q * FM / NP == i) dma_setup(q, ring[STAGES - 1]);
                    });
                }
                if constexpr (!Cfg::PAIR && s == SLOTS - 1) {
                    static_for<0, NP>([&](auto q_) {
                        constexpr int q = decltype(q_)::value;
                        if constexpr (split) {
                            if constexpr (q * FM / NP == i) dma_issue(q);
                        } else if constexpr (bunched ? i == 0 : q * FM / NP == i) {
                            dma_piece(q, ring[STAGES - 1]);
                        }
                    });
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        });
        // (The fragments widened for the next step are only used after the branches of the
        // load cursor below; without a use here the compiler sinks their widening out of
        // the MFMA slots to the far side of those branches.)
        static_for<0, FN>([&](auto j_) {
            constexpr int j = decltype(j_)::value;
            keep_here(b_ev[bs ^ 1][j]);
            keep_here(b_od[bs ^ 1][j]);
        });
        keep_here(a_ev[0]);
        keep_here(a_od[0]);
        keep_here(a_pk[1]);
        // The step two ahead must have landed, and every wave must be done reading this
        // step's stage, before the roles rotate; the younger steps stay in flight.  The
        // counter counts loads and stores alike, in order of issue: the stores of a last
        // step are all younger than the loads that must have landed, and are allowed to stay
        // in flight as well (the counter cannot express more than 63).
        // (through the half-size area the last two stores of row FM-2 go out with row FM-1, after this step)
        // (paired ring: an odd step has issued the loads of two steps, all younger than what must
        // have landed; after an even step, which issues none, the youngest load belongs to step
        // s+3 and the one before it to s+2, which must be there)
        // (a tile that sticks out of C: none of its stores is allowed for, see store_lanes)
        constexpr int pending = (Cfg::PAIR ? (bs == 1 ? 2 * NP : 1) : (AHEAD - 2) * NP) + (last && !edge ? (FM - 1) * FN - (Cfg::XHALF ? 2 : 0) : 0);
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(pending > 63 ? 63 : pending) : "memory");
        if constexpr (Cfg::PAIR) {
            const int ta = a_ring[0], tb = b_ring[0];
#pragma unroll
            for (int u = 0; u < 4; ++u) a_ring[u] = a_ring[u + 1];
            a_ring[4] = ta;
#pragma unroll
            for (int u = 0; u < 3; ++u) b_ring[u] = b_ring[u + 1];
            b_ring[3] = tb;
            if constexpr (bs == 1) cursor_advance();
        } else {
            const int t = ring[0];
#pragma unroll
            for (int u = 0; u + 1 < STAGES; ++u) ring[u] = ring[u + 1];
            ring[STAGES - 1] = t;
            cursor_advance();
        }
    };

    // One item: K-steps in pairs; when the item has an odd number of them, the second of the
    // last pair is the padding step and its B operand is widened to zero.
    auto run_item = [&](auto mode_) __attribute__((always_inline)) {
        // mode 1: a whole tile, written out with plain stores inside its last K-step; 2: a tile
        // that sticks out of C, the same with every store under its lanes' conditions;
        // 0: guarded stores after the last K-step (K split, or a C that does not take plain
        // 16-byte stores)
        constexpr int mode = decltype(mode_)::value;
        constexpr bool whole = mode != 0, edge = mode == 2;
        locate(c_item, c_m0, c_n0, c_kt0, c_KT);
        if constexpr (edge) {
            const int mrem = p.M - c_m0, nrem = p.N - c_n0;
            if constexpr (Cfg::XPOSE) { rows_left = mrem - wm * Cfg::WM - (lane >> 4); cols_left = nrem - wn * Cfg::WN - (lane & 15) * 4; }
            else if constexpr (Cfg::XHALF) { rows_left = mrem - wm * Cfg::WM - (lane >> 3); cols_left = nrem - wn * Cfg::WN - (lane & 7) * 4; }
            else { rows_left = mrem - wm * Cfg::WM - r; cols_left = nrem - wn * Cfg::WN - g * 4; }
        }
        if constexpr (OUT != OUT_I32) {
            // The item's scales, loaded now and waited for now: the compiler cannot see the
            // asm loads of the ring in the memory counter, so a wait it placed at the first
            // use -- inside the last K-step -- would drain the whole ring there.
#pragma unroll
            for (int ib = 0; ib < FM; ++ib) rs_reg[ib] = scale_at(p.row_scale, c_m0 + wm * Cfg::WM + ib * 16 + r, p.M);
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e) cs_reg[j][e] = scale_at(p.col_scale, c_n0 + wn * Cfg::WN + j * 16 + g * 4 + e, p.N);
#pragma unroll
            for (int ib = 0; ib < FM; ++ib) keep_here_f(rs_reg[ib]);
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e) keep_here_f(cs_reg[j][e]);
        }
        // (the masks are made opaque: knowing one to be all-ones-per-nibble or zero, the
        // compiler would hoist the whole widening of B out of the MFMA slots into a branch)
        uint32_t bmask, full;
        if constexpr (TAIL) {
            // the step of this item that is the short last step of K, or -1 (the launcher sees to
            // it that such an item has at least two steps: its B is widened inside the item)
            const int tail_at = (k_tail != 0 && c_kt0 + c_KT == kt_all) ? c_KT - 1 : -1;
            for (c_kt = 0; c_kt + 2 < c_KT; c_kt += 2) {
                k_step(vmask_full, std::integral_constant<int, 0>{}, std::false_type{});
                uint32_t m2 = c_kt + 2 == tail_at ? vmask_tail : vmask_full;
                asm volatile("" : "+v"(m2));
                k_step(m2, std::integral_constant<int, 1>{}, std::false_type{});
            }
            bmask = c_kt + 1 < c_KT ? (c_kt + 1 == tail_at ? vmask_tail : vmask_full) : 0u;
            asm volatile("" : "+v"(bmask));
            full = vmask_full;
        } else {
            for (c_kt = 0; c_kt + 2 < c_KT; c_kt += 2) {
                k_step(amask, std::integral_constant<int, 0>{}, std::false_type{});
                k_step(amask, std::integral_constant<int, 1>{}, std::false_type{});
            }
            bmask = c_kt + 1 < c_KT ? amask : 0u;
            asm volatile("" : "+s"(bmask));
            full = amask;
        }
        tile_c = reinterpret_cast<char *>(p.C) + ((size_t)c_m0 * ldc + c_n0) * ESZ;
        if constexpr (OUT == OUT_I32 && !whole) {
            // workspace slot of a K-split item: (split, tile) in the order locate() numbers them
            if (p.ws != nullptr && ksplit > 1)
                split_ws = reinterpret_cast<v4i *>(p.ws) +
                           ((size_t)xcd_contiguous_id(c_item, nitems) * WAVES + wave) * (FM * FN * 64) + lane;
        }
        k_step(bmask, std::integral_constant<int, 0>{}, std::false_type{});
        k_step(full, std::integral_constant<int, 1>{}, std::integral_constant<int, mode>{});
        // Let the last MFMAs retire before their accumulators are read (the compiler does not
        // know the asm statements were MFMAs, so the wait is tied to the accumulators written
        // last and cannot be scheduled around); then the rows not written out yet.
        static_for<(FN > 4 ? FN - 4 : 0), FN>([&](auto j_) {
            mfma16_settle(acc[FM - 1][decltype(j_)::value]);
        });
        if constexpr (whole) {
            static_for<0, 2 * FN>([&](auto s_) {
                write_whole(std::integral_constant<int, FM - 1>{}, s_, std::integral_constant<bool, edge>{});
                __builtin_amdgcn_sched_barrier(0);
            });
            if constexpr (Cfg::XHALF) flush_half(std::integral_constant<bool, edge>{});
        } else {
            static_for<0, FM>([&](auto ib_) {
                static_for<0, FN>([&](auto j_) {
                    write_guarded(ib_, j_);
                    // one block at a time: the widened fragments of the next step stay live
                    // across this code, so there are few registers to stage results in
                    __builtin_amdgcn_sched_barrier(0);
                });
            });
        }
        // The clearing MFMAs issued last must have retired before anything else touches the
        // accumulators: between the two loops below the register allocator may move
        // accumulators to other registers with instructions of its own, and it does not know
        // that asm statements are still writing them.
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    };
    // (three loops one after the other, each of which may run nothing: with loops in the arms
    // of a branch instead, the register allocator spills)
    const int nfolded = __builtin_amdgcn_readfirstlane(plain_c ? nitems : 0);
    for (; c_item < nwhole; c_item += G) run_item(std::integral_constant<int, 1>{});
    for (; c_item < nfolded; c_item += G) run_item(std::integral_constant<int, 2>{});
    for (; c_item < nitems; c_item += G) run_item(std::integral_constant<int, 0>{});
    // drain the DMA before the LDS is released
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

}  // namespace qm
