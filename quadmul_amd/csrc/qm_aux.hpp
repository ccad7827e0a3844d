// Kernels beside the MFMA ones, and their launchers: the generic GEMM (any even K, any
// alignment), zero fill, zero-padded operand copies, the kernel that adds up a K split out
// of a workspace, pack / unpack (reference: test.py:6-15, kernel.cu:387-408) and the fused
// quantise + pack.  Included by qm_dispatch.hip only.
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/qm_abi.h"
#include "qm_common.hpp"

namespace qm {

// --------------------------------------------------------------------------
// Fallback kernel: any M, N, even K, any alignment, no limit on K.  One thread
// per element of C over LDS-staged 16x16x(128 nibble) tiles, plain byte loads.
// --------------------------------------------------------------------------
__device__ __forceinline__ int s4_lo(uint32_t b) { return (int)(int8_t)(b << 4) >> 4; }
__device__ __forceinline__ int s4_hi(uint32_t b) { return (int)(int8_t)b >> 4; }

__global__ void __launch_bounds__(256) gemm_generic_kernel(const GemmArgs p, const int tiles_n)
{
    __shared__ uint8_t As[16][64 + 4];
    __shared__ uint8_t Bs[16][64 + 4];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int m0 = (blockIdx.x / tiles_n) * 16, n0 = (blockIdx.x % tiles_n) * 16;
    const size_t Kb = (size_t)(p.K >> 1);
    int32_t sum = 0;
    for (size_t k0 = 0; k0 < Kb; k0 += 64) {
        // 16 rows x 64 bytes per operand = 1024 bytes each, 4 bytes per thread
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int idx = threadIdx.x + t * 256, row = idx >> 6, col = idx & 63;
            const bool kin = k0 + col < Kb;
            As[row][col] = (kin && m0 + row < p.M) ? p.A[(size_t)(m0 + row) * Kb + k0 + col] : (uint8_t)0;
            Bs[row][col] = (kin && n0 + row < p.N) ? p.B[(size_t)(n0 + row) * Kb + k0 + col] : (uint8_t)0;
        }
        __syncthreads();
#pragma unroll 16
        for (int j = 0; j < 64; ++j) {
            const uint32_t a = As[ty][j], b = Bs[tx][j];
            sum += s4_lo(a) * s4_lo(b) + s4_hi(a) * s4_hi(b);
        }
        __syncthreads();
    }
    const int m = m0 + ty, n = n0 + tx;
    if (m < p.M && n < p.N) {
        const size_t at = (size_t)m * c_stride(p) + n;
        if (p.out == OUT_I32) p.C[at] = sum;
        else reinterpret_cast<uint16_t *>(p.C)[at] = round16(scaled(sum, scale_at(p.row_scale, m, p.M), scale_at(p.col_scale, n, p.N)), p.out);
    }
}

static hipError_t launch_generic(const GemmArgs &p, hipStream_t stream, int)
{
    const long long tiles_m = (p.M + 15) / 16, tiles_n = (p.N + 15) / 16;
    if (tiles_m * tiles_n > 0x7fffffffLL) return hipErrorInvalidValue;
    gemm_generic_kernel<<<dim3((unsigned)(tiles_m * tiles_n)), dim3(256), 0, stream>>>(p, (int)tiles_n);
    return hipGetLastError();
}

// --------------------------------------------------------------------------
// Zero fill (k == 0) and pack / unpack, flat over the whole array: K is even so
// a byte never straddles two rows.
// --------------------------------------------------------------------------
__global__ void fill_zero16_kernel(uint16_t *dst, size_t n)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) dst[i] = 0;
}

__global__ void fill_zero_kernel(int32_t *dst, size_t n)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) dst[i] = 0;
}

// --------------------------------------------------------------------------
// Operand copies with every row padded with zeros to a whole number of 128-nibble K-steps
// (zero nibbles add nothing to a product): what lets the pipelined kernel run shapes whose
// K is not a multiple of 32, or whose operands are not 16-byte aligned, out of a
// caller-provided workspace.  Both operands in one launch (a second dependent launch costs
// more than the copy of a small operand): rows 0 .. rows_a-1 are A's, the rest B's.
// Source rows may start at any byte: one wave per row, one 32-bit word of the copy per
// lane and turn, put together from the two aligned source words that hold its bytes
// (consecutive lanes read consecutive words), the bytes past the end of the row zeroed.  An
// aligned word that holds at least one byte of a matrix lies in the same page as that byte,
// so reading it whole is safe; a word wholly past the end of the matrix is not read.
// kb: bytes per source row; kbp4: 32-bit words per row of the copy.
// --------------------------------------------------------------------------
struct PadRowsArgs {
    const uint8_t *src_a, *src_b;
    uint32_t *dst_a, *dst_b;
    int rows_a, rows_b, kb, kbp4;
};

__global__ void __launch_bounds__(256) pad_rows_kernel(const PadRowsArgs q)
{
    const int lane = threadIdx.x & 63;
    for (int r = blockIdx.x * 4 + (threadIdx.x >> 6); r < q.rows_a + q.rows_b; r += gridDim.x * 4) {
        const bool is_a = r < q.rows_a;
        const uint8_t *src = is_a ? q.src_a : q.src_b;
        const int row = is_a ? r : r - q.rows_a;
        const uintptr_t end = (uintptr_t)src + (size_t)(is_a ? q.rows_a : q.rows_b) * q.kb;
        const uintptr_t at = (uintptr_t)src + (size_t)row * q.kb;
        const uint32_t *w = reinterpret_cast<const uint32_t *>(at & ~(uintptr_t)3);
        const uint32_t shift = (uint32_t)(at & 3);
        uint32_t *out = (is_a ? q.dst_a : q.dst_b) + (size_t)row * q.kbp4;
        for (int i = lane; i < q.kbp4; i += 64) {
            const int keep = q.kb - 4 * i;  // bytes of the row from this word on
            uint32_t v = 0;
            if (keep > 0) {
                const uint32_t x0 = w[i];
                const uint32_t x1 = (uintptr_t)(w + i + 1) < end ? w[i + 1] : 0u;
                v = __builtin_amdgcn_alignbyte(x1, x0, shift) & (keep >= 4 ? 0xffffffffu : (1u << (8 * keep)) - 1u);
            }
            out[i] = v;
        }
    }
}

// --------------------------------------------------------------------------
// K split with a workspace (pipelined kernel): item (split s, tile t) of the GEMM launch
// left its BM x BN partial sums in slot s * ntiles + t, wave by wave, block by block, 16
// bytes per lane in the order the MFMA leaves a block (lane l: row l % 16, columns
// 4 * (l / 16) .. + 3).  One thread here adds up the splits of one such 16-byte piece and
// stores the four sums -- as int32, or scaled and rounded to a 16-bit float -- with the
// guards of the matrix edge.  Tiles are numbered as the GEMM kernel numbers them (columns of
// group_m tiles).
// --------------------------------------------------------------------------
struct SplitReduceArgs {
    const v4i *ws;
    void *C;
    int M, N;
    int tiles_m, tiles_n, group_m, ksplit;
    int BM, BN, WGN, FM, FN, waves;
    const float *row_scale, *col_scale;
    int out;
};

__global__ __launch_bounds__(256) void splitk_reduce_kernel(const SplitReduceArgs q)
{
    const int blocks = q.FM * q.FN;
    const size_t per_tile = (size_t)q.waves * blocks * 64;  // 16-byte pieces per slot
    const size_t ntiles = (size_t)q.tiles_m * q.tiles_n;
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;  // (the launcher keeps the count below 2^31)
    if (t >= ntiles * per_tile) return;
    const v4i *src = q.ws + t;
    const size_t stride = ntiles * per_tile;
    v4i sum = {0, 0, 0, 0};
    // four splits at a time, so that their loads are in flight together (splits past the
    // last re-read it and count for nothing)
    for (int s = 0; s < q.ksplit; s += 4) {
        v4i v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = __builtin_nontemporal_load(src + (size_t)min(s + i, q.ksplit - 1) * stride);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int on = s + i < q.ksplit ? -1 : 0;
            sum.x += v[i].x & on; sum.y += v[i].y & on; sum.z += v[i].z & on; sum.w += v[i].w & on;
        }
    }
    const int lane = (int)(t & 63);
    uint32_t u = t >> 6;
    const int blk = (int)(u % (uint32_t)blocks);
    u /= (uint32_t)blocks;
    const int wave = (int)(u % (uint32_t)q.waves);
    const int pid = (int)(u / (uint32_t)q.waves);
    const int width = q.group_m * q.tiles_n;
    const int first_m = (pid / width) * q.group_m;
    const int gsz = min(q.tiles_m - first_m, q.group_m);
    const int tm = first_m + (pid % width) % gsz, tn = (pid % width) / gsz;
    const int m = tm * q.BM + (wave / q.WGN) * q.FM * 16 + (blk / q.FN) * 16 + (lane & 15);
    const int n = tn * q.BN + (wave % q.WGN) * q.FN * 16 + (blk % q.FN) * 16 + (lane >> 4) * 4;
    if (m >= q.M || n >= q.N) return;
    if (q.out == OUT_I32) {
        int32_t *crow = static_cast<int32_t *>(q.C) + (size_t)m * q.N;
        if ((q.N & 3) == 0 && ((uintptr_t)q.C & 15) == 0) {
            *reinterpret_cast<v4i *>(crow + n) = sum;  // n % 4 == 0 and N % 4 == 0: all four inside
        } else if (n + 3 < q.N) {
            *reinterpret_cast<v4i_elem_aligned *>(crow + n) = sum;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (n + e < q.N) crow[n + e] = sum[e];
        }
    } else {
        uint16_t *drow = static_cast<uint16_t *>(q.C) + (size_t)m * q.N;
        const float rs = scale_at(q.row_scale, m, q.M);
        uint16_t h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int c = sum[e];
            h[e] = round16(scaled(c, rs, scale_at(q.col_scale, n + e, q.N)), q.out);
        }
        if ((q.N & 3) == 0 && ((uintptr_t)q.C & 7) == 0) {
            *reinterpret_cast<v2i *>(drow + n) = v2i{(int)(h[0] | ((uint32_t)h[1] << 16)), (int)(h[2] | ((uint32_t)h[3] << 16))};
        } else if (n + 3 < q.N) {
            *reinterpret_cast<v2i_half_aligned *>(drow + n) = v2i{(int)(h[0] | ((uint32_t)h[1] << 16)), (int)(h[2] | ((uint32_t)h[3] << 16))};
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (n + e < q.N) drow[n + e] = h[e];
        }
    }
}

// 16 int8 in -> 8 packed bytes out per thread when aligned, else one byte per thread.
__device__ __forceinline__ uint32_t pack4(uint32_t w)  // 4 int8 -> 2 packed bytes in bits 0..15
{
    uint32_t t = w & 0x0F0F0F0Fu;
    t |= t >> 4;  // byte0 = n0 | n1<<4, byte2 = n2 | n3<<4
    return (t & 0xFFu) | ((t >> 8) & 0xFF00u);
}

__global__ void pack_i4_vec_kernel(const v4i *__restrict__ src, v2i *__restrict__ dst, size_t nvec)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += (size_t)gridDim.x * blockDim.x) {
        const v4i v = src[i];
        v2i o;
        o.x = (int)(pack4((uint32_t)v.x) | (pack4((uint32_t)v.y) << 16));
        o.y = (int)(pack4((uint32_t)v.z) | (pack4((uint32_t)v.w) << 16));
        dst[i] = o;
    }
}

__global__ void pack_i4_byte_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, size_t nbytes)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nbytes; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = (uint8_t)((src[2 * i] & 0x0Fu) | ((src[2 * i + 1] & 0x0Fu) << 4));
}

// 4 packed bytes -> 8 int8: widen nibbles to bytes, sign-extend (bit 3 set => OR 0xF0),
// interleave even/odd elements back into K order.
__device__ __forceinline__ uint32_t sext_nibbles(uint32_t x)  // x = 0x0n0n0n0n
{
    const uint32_t t = x & 0x08080808u;
    return x | ((t << 5) - (t << 1));  // 0x08 -> 0xF0 in each byte (the top byte wraps mod 2^32)
}

__global__ void unpack_i4_vec_kernel(const uint32_t *__restrict__ src, v2i *__restrict__ dst, size_t nwords)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nwords; i += (size_t)gridDim.x * blockDim.x) {
        const uint32_t w = src[i];
        const uint32_t ev = sext_nibbles(w & 0x0F0F0F0Fu), od = sext_nibbles((w >> 4) & 0x0F0F0F0Fu);
        v2i o;  // bytes: ev0 od0 ev1 od1 | ev2 od2 ev3 od3
        o.x = (int)__builtin_amdgcn_perm(od, ev, 0x05010400u);
        o.y = (int)__builtin_amdgcn_perm(od, ev, 0x07030602u);
        dst[i] = o;
    }
}

__global__ void unpack_i4_byte_kernel(const uint8_t *__restrict__ src, int8_t *__restrict__ dst, size_t nbytes)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nbytes; i += (size_t)gridDim.x * blockDim.x) {
        const uint32_t b = src[i];
        dst[2 * i] = (int8_t)s4_lo(b);
        dst[2 * i + 1] = (int8_t)s4_hi(b);
    }
}

// --------------------------------------------------------------------------
// Per-row symmetric quantisation to int4 fused with the packing: one workgroup per row,
// the row held in registers between the two passes over it (maximum, then quantise), so
// HBM is read once.  x is fp16, bf16 or fp32; 8 elements (4 packed bytes) per thread-chunk.
// --------------------------------------------------------------------------
template <int IN> struct QuantIn;
template <> struct QuantIn<QM_IN_F16> {
    static constexpr int BYTES = 2;
    static __device__ __forceinline__ float widen(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
};
template <> struct QuantIn<QM_IN_BF16> {
    static constexpr int BYTES = 2;
    static __device__ __forceinline__ float widen(uint16_t h) { return __builtin_bit_cast(float, (uint32_t)h << 16); }
};
template <> struct QuantIn<QM_IN_F32> {
    static constexpr int BYTES = 4;
};

template <int IN>
__device__ __forceinline__ void load8(const uint8_t *src, float (&v)[8])
{
    if constexpr (IN == QM_IN_F32) {
        const v4i lo = *reinterpret_cast<const v4i *>(src), hi = *reinterpret_cast<const v4i *>(src + 16);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int a = lo[e], b = hi[e];
            v[e] = __builtin_bit_cast(float, a);
            v[4 + e] = __builtin_bit_cast(float, b);
        }
    } else {
        const v4i w = *reinterpret_cast<const v4i *>(src);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t d = (uint32_t)w[e];
            v[2 * e] = QuantIn<IN>::widen((uint16_t)(d & 0xFFFFu));
            v[2 * e + 1] = QuantIn<IN>::widen((uint16_t)(d >> 16));
        }
    }
}

__device__ __forceinline__ uint32_t quant8(const float (&v)[8], float inv)
{
#pragma clang fp contract(off)
    uint32_t out = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float r = __builtin_rintf(v[e] * inv);  // round half to even
        r = fminf(fmaxf(r, -7.0f), 7.0f);
        out |= ((uint32_t)(int)r & 0xFu) << (4 * e);  // element e -> nibble e: low nibble = even k (test.py:8,14)
    }
    return out;
}

// workgroup-wide maximum of non-negative floats
__device__ __forceinline__ float block_max(float x, float *lds)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) x = fmaxf(x, __shfl_xor(x, off));
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) lds[wave] = x;
    __syncthreads();
    float m = lds[0];
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w) m = fmaxf(m, lds[w]);
    __syncthreads();
    return m;
}

// NC: chunks of 8 elements a thread keeps in registers (k <= 2048 * NC); NC == 0: any k that is
// a multiple of 8, the row read twice (the second time out of the L2)
template <int IN, int NC>
__global__ void __launch_bounds__(256) quantize_pack_kernel(const uint8_t *__restrict__ x, uint8_t *__restrict__ dst, float *__restrict__ scales, int k)
{
    __shared__ float red[4];
    const int row = blockIdx.x, tid = threadIdx.x, nchunks = k >> 3;
    const uint8_t *xr = x + (size_t)row * k * QuantIn<IN>::BYTES;
    uint32_t *out = reinterpret_cast<uint32_t *>(dst + (size_t)row * (k >> 1));
    float amax = 0.0f;
    if constexpr (NC > 0) {
        float v[NC][8];
#pragma unroll
        for (int i = 0; i < NC; ++i) {
            const int c = tid + i * 256;
            if (c < nchunks) {
                load8<IN>(xr + (size_t)c * 8 * QuantIn<IN>::BYTES, v[i]);
#pragma unroll
                for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(v[i][e]));
            }
        }
        amax = block_max(amax, red);
        const float inv = amax > 0.0f ? 7.0f / amax : 0.0f;
        if (tid == 0) scales[row] = amax / 7.0f;
#pragma unroll
        for (int i = 0; i < NC; ++i) {
            const int c = tid + i * 256;
            if (c < nchunks) out[c] = quant8(v[i], inv);
        }
    } else {
        float v[8];
        for (int c = tid; c < nchunks; c += 256) {
            load8<IN>(xr + (size_t)c * 8 * QuantIn<IN>::BYTES, v);
#pragma unroll
            for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(v[e]));
        }
        amax = block_max(amax, red);
        const float inv = amax > 0.0f ? 7.0f / amax : 0.0f;
        if (tid == 0) scales[row] = amax / 7.0f;
        for (int c = tid; c < nchunks; c += 256) {
            load8<IN>(xr + (size_t)c * 8 * QuantIn<IN>::BYTES, v);
            out[c] = quant8(v, inv);
        }
    }
}

// any even k, any alignment: one pair of elements per thread and pass
template <int IN>
__global__ void __launch_bounds__(256) quantize_pack_scalar_kernel(const uint8_t *__restrict__ x, uint8_t *__restrict__ dst, float *__restrict__ scales, int k)
{
#pragma clang fp contract(off)
    __shared__ float red[4];
    const int row = blockIdx.x, tid = threadIdx.x;
    auto at = [&](int j) -> float {
        if constexpr (IN == QM_IN_F32) {
            return reinterpret_cast<const float *>(x)[(size_t)row * k + j];
        } else {
            return QuantIn<IN>::widen(reinterpret_cast<const uint16_t *>(x)[(size_t)row * k + j]);
        }
    };
    float amax = 0.0f;
    for (int j = tid; j < k; j += 256) amax = fmaxf(amax, fabsf(at(j)));
    amax = block_max(amax, red);
    const float inv = amax > 0.0f ? 7.0f / amax : 0.0f;
    if (tid == 0) scales[row] = amax / 7.0f;
    for (int j = 2 * tid; j < k; j += 512) {
        const float r0 = fminf(fmaxf(__builtin_rintf(at(j) * inv), -7.0f), 7.0f), r1 = fminf(fmaxf(__builtin_rintf(at(j + 1) * inv), -7.0f), 7.0f);
        dst[(size_t)row * (k >> 1) + (j >> 1)] = (uint8_t)(((int)r0 & 0xF) | (((int)r1 & 0xF) << 4));
    }
}

template <int IN>
static hipError_t launch_quantize_pack(const void *x, void *dst, float *scales, int rows, int k, hipStream_t s)
{
    const uint8_t *xb = static_cast<const uint8_t *>(x);
    uint8_t *db = static_cast<uint8_t *>(dst);
    const bool vec = k % 8 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)dst & 3) == 0;
    if (!vec) quantize_pack_scalar_kernel<IN><<<dim3(rows), dim3(256), 0, s>>>(xb, db, scales, k);
    else if (k <= 2048 * 2) quantize_pack_kernel<IN, 2><<<dim3(rows), dim3(256), 0, s>>>(xb, db, scales, k);
    else if (k <= 2048 * 8) quantize_pack_kernel<IN, 8><<<dim3(rows), dim3(256), 0, s>>>(xb, db, scales, k);
    else quantize_pack_kernel<IN, 0><<<dim3(rows), dim3(256), 0, s>>>(xb, db, scales, k);
    return hipGetLastError();
}

static unsigned flat_grid(size_t items, unsigned block)
{
    size_t g = (items + block - 1) / block;
    if (g < 1) g = 1;
    if (g > 256u * 32u) g = 256u * 32u;
    return (unsigned)g;
}

}  // namespace qm
