// Shared device helpers for the gfx950 packed-int4 GEMM kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace qm {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
// The same at the alignment of one element: what a row of C has when N % 4 != 0 (or C itself
// is not 16-byte aligned).  A store through these is still one global_store_dwordx4 / x2 --
// the device takes them at any alignment -- where four element-wise stores per lane, 16 bytes
// apart from the next lane's, ran at a third of the speed (1444 x 31702 x 128: 104 us).
typedef v4i v4i_elem_aligned __attribute__((aligned(4)));
typedef v2i v2i_half_aligned __attribute__((aligned(2)));

// Output forms: the exact int32 product, or the product scaled per row and per column in
// fp32 and rounded to a 16-bit float (the "dequantise on the way out" use the reference's
// README.md:7 has in mind; no code of the reference does it).
enum OutKind { OUT_I32 = 0, OUT_F16 = 1, OUT_BF16 = 2 };

struct GemmArgs {
    const uint8_t *A;  // [M, K/2] packed s4
    const uint8_t *B;  // [N, K/2] packed s4
    int32_t *C;        // [M, N] int32; or [M, N] 16-bit floats when `out` says so
    int M, N, K;
    // scaled output only: D[m][n] = round16(((float)C[m][n] * row_scale[m]) * col_scale[n]),
    // a null pointer standing for all ones
    const float *row_scale = nullptr;  // [M]
    const float *col_scale = nullptr;  // [N]
    int out = OUT_I32;
    // K split over several work items per tile (pipelined kernel): where the partial sums go.
    // Null: they meet in C by atomic adds (C zero-filled beforehand).  Otherwise item i of the
    // launch stores its tile here, 16 bytes per lane in the order the MFMA leaves them, and a
    // second kernel adds the splits up.
    int32_t *ws = nullptr;
    // Row stride of C in elements, 0 standing for N: set when the call computes a block of
    // columns of a wider C (a B beyond the kernels' 32-bit offsets is cut along N).
    int ldc = 0;
};

__device__ __forceinline__ int c_stride(const GemmArgs &p) { return p.ldc != 0 ? p.ldc : p.N; }

__device__ __forceinline__ float scale_at(const float *s, int i, int n) { return (s != nullptr && i < n) ? s[i] : 1.0f; }

// fp32 -> 16-bit float, round to nearest even (NaN stays NaN).  Contraction is switched
// off in these helpers: fused, the compiler turns "multiply, then round to fp16" into one
// instruction with a single rounding, which is not the value defined above.
template <int OUT>
__device__ __forceinline__ uint16_t round16(float x)
{
#pragma clang fp contract(off)
    if constexpr (OUT == OUT_F16) {
        // (the empty asm hides where x came from: instruction selection otherwise merges a
        // preceding fp32 multiply and this conversion into v_fma_mixlo_f16, which rounds the
        // exact product once, straight to fp16 -- not the twice-rounded value defined above)
        asm("" : "+v"(x));
        const _Float16 h = (_Float16)x;
        return __builtin_bit_cast(uint16_t, h);
    } else {
        // (both candidates computed and one selected: no per-lane branch in the callers' code)
        const uint32_t u = __builtin_bit_cast(uint32_t, x);
        const uint32_t rounded = (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16, quiet = (u >> 16) | 0x0040u;
        return (uint16_t)(((u & 0x7FFFFFFFu) > 0x7F800000u) ? quiet : rounded);
    }
}
__device__ __forceinline__ uint16_t round16(float x, int out) { return out == OUT_F16 ? round16<OUT_F16>(x) : round16<OUT_BF16>(x); }

// the scaled value of one element, in the one order of operations everything here uses
__device__ __forceinline__ float scaled(int c, float rs, float cs)
{
#pragma clang fp contract(off)
    const float t = (float)c * rs;
    return t * cs;
}

// gfx950 has no int4 MFMA, so nibbles are widened to int8 -- but scaled by 16,
// which needs no per-byte sign fix-up.  For a dword w holding nibbles k0..k7
// (k0 in bits 0..3), read as four int8 lanes:
//     (w << 4) & 0xF0F0F0F0  ==  16 * s4(k0), 16 * s4(k2), 16 * s4(k4), 16 * s4(k6)
//      w       & 0xF0F0F0F0  ==  16 * s4(k1), 16 * s4(k3), 16 * s4(k5), 16 * s4(k7)
// because a nibble n placed in the high half of a byte is the int8 value 16*s4(n).
// Both operands get the same treatment, so every int8 product carries a factor
// 256 and the int32 accumulator holds exactly 256 * C; the epilogue shifts it out.
// |C| <= 64 K, hence exact while 256 * 64 * K < 2^31, i.e. K <= QM_MAX_K_X16.
// The even/odd split permutes K inside a dword; the contraction runs over K and
// A and B are permuted identically, so the sum is unchanged.
constexpr int QM_MAX_K_X16 = 131071;

__device__ __forceinline__ int x16_even(int w) { return (int)(((uint32_t)w << 4) & 0xF0F0F0F0u); }
__device__ __forceinline__ int x16_odd(int w) { return (int)((uint32_t)w & 0xF0F0F0F0u); }

__device__ __forceinline__ void x16_expand(const v4i q, v4i &even, v4i &odd)
{
    even.x = x16_even(q.x); even.y = x16_even(q.y); even.z = x16_even(q.z); even.w = x16_even(q.w);
    odd.x = x16_odd(q.x);   odd.y = x16_odd(q.y);   odd.z = x16_odd(q.z);   odd.w = x16_odd(q.w);
}

// The same in 10 instructions instead of 12: one 64-bit shift per pair of dwords (the nibble
// that crosses into the upper dword lands in a low nibble and is masked away with the rest).
__device__ __forceinline__ void x16_expand_pairs(const v4i q, v4i &even, v4i &odd)
{
    const v2i lo = {q.x, q.y}, hi = {q.z, q.w};
    v2i slo, shi;
    asm("v_lshlrev_b64 %0, 4, %1" : "=v"(slo) : "v"(lo));
    asm("v_lshlrev_b64 %0, 4, %1" : "=v"(shi) : "v"(hi));
    even.x = (int)((uint32_t)slo.x & 0xF0F0F0F0u); even.y = (int)((uint32_t)slo.y & 0xF0F0F0F0u);
    even.z = (int)((uint32_t)shi.x & 0xF0F0F0F0u); even.w = (int)((uint32_t)shi.y & 0xF0F0F0F0u);
    odd.x = x16_odd(q.x); odd.y = x16_odd(q.y); odd.z = x16_odd(q.z); odd.w = x16_odd(q.w);
}

// D(16x16) += S0(16x64) * S1(64x16), int8 in, int32 out.  Lane l supplies row
// l%16 of S0 / column l%16 of S1 for the 16 k-values of group l/16, and owns
// D[4*(l/16) + r][l%16] in register r.
__device__ __forceinline__ v4i mfma16(const v4i s0, const v4i s1, const v4i acc)
{
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(s0, s1, acc, 0, 0, 0);
}

// Byte offset of row `row` of a packed operand with Kb bytes per row, for the skinny
// kernels: both factors are below 2^24 there (the host side sees to it), so the full-rate
// 24-bit multiply does (the 32-bit one issues at a quarter of the rate, and these products
// sit in front of a wave's first load).
__device__ __forceinline__ uint32_t row_bytes24(int row, int Kb) { return __umul24((uint32_t)row, (uint32_t)Kb); }

// Workgroups are dealt round-robin to the 8 XCDs (id % 8), each with a private
// L2.  Renumber so that every XCD owns one contiguous range of tile ids.
__device__ __forceinline__ int xcd_contiguous_id(int bid, int nblocks)
{
    constexpr int XCDS = 8;
    const int xcd = bid % XCDS, local = bid / XCDS;
    const int per = (nblocks + XCDS - 1) / XCDS;  // size of the larger shares
    const int tall = nblocks % XCDS;              // how many XCDs get a larger share (0: all equal)
    if (tall == 0 || xcd < tall) return xcd * per + local;
    return tall * per + (xcd - tall) * (per - 1) + local;
}

}  // namespace qm
