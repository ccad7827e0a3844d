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

#define QM_EXPORT extern "C" __attribute__((visibility("default")))

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
        const size_t at = (size_t)m * p.N + n;
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
// Operand copy with every row padded with zeros to a whole number of 128-nibble K-steps
// (zero nibbles add nothing to a product): what lets the pipelined kernel run shapes whose
// K is not a multiple of 128, or whose operands are not 16-byte aligned, out of a
// caller-provided workspace.  kb / kbp: bytes per row of the source / of the copy.
// --------------------------------------------------------------------------
__global__ void pad_rows_vec_kernel(const v4i *__restrict__ src, v4i *__restrict__ dst, int rows, int kb16, int kbp16)
{
    const size_t total = (size_t)rows * kbp16;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / kbp16;
        const int c = (int)(i - r * kbp16);
        dst[i] = c < kb16 ? src[r * kb16 + c] : v4i{0, 0, 0, 0};
    }
}

__global__ void pad_rows_byte_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int rows, int kb, int kbp)
{
    const size_t total = (size_t)rows * kbp;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / kbp;
        const int c = (int)(i - r * kbp);
        dst[i] = c < kb ? src[r * kb + c] : (uint8_t)0;
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

// --------------------------------------------------------------------------
// Skinny launchers
// --------------------------------------------------------------------------
template <class Cfg>
static hipError_t launch_skinny(const GemmArgs &p, hipStream_t stream, int)
{
    const int blocks = (p.N + Cfg::BN - 1) / Cfg::BN;
    gemm_skinny_kernel<Cfg><<<dim3(blocks), dim3(Cfg::THREADS), 0, stream>>>(p);
    return hipGetLastError();
}
#define QM_SKINNY(FM, FN, NW, U) \
    hipError_t QM_SKINNY_FN(FM, FN, NW, U)(const GemmArgs &p, hipStream_t s, int gm) { return launch_skinny<SkinnyCfg<FM, FN, NW, U>>(p, s, gm); }
template <class Cfg>
static hipError_t launch_dot(const GemmArgs &p, hipStream_t stream, int)
{
    const int blocks = (p.N + Cfg::BN - 1) / Cfg::BN;
    gemm_dot_kernel<Cfg><<<dim3(blocks), dim3(Cfg::THREADS), 0, stream>>>(p);
    return hipGetLastError();
}
#define QM_DOT(MR, FN, NW, U) \
    hipError_t QM_DOT_FN(MR, FN, NW, U)(const GemmArgs &p, hipStream_t s, int gm) { return launch_dot<DotCfg<MR, FN, NW, U>>(p, s, gm); }
#include "qm_configs.inc"

// --------------------------------------------------------------------------
// Configuration registry
// --------------------------------------------------------------------------
enum Kind { KIND_GENERIC = 0, KIND_SKINNY = 2, KIND_TILE16 = 3 };

struct ConfigDesc {
    const char *name;
    int kind;
    int bm, bn, bk;  // tile: block shape; skinny: bm = max M, bn = columns per workgroup
    int waves, mode;
    LaunchFn launch;
    int wgm = 0, wgn = 0;  // pipelined kernel: waves down and across the tile
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
    if (c.kind == KIND_SKINNY) return m <= c.bm;
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
    if (m <= 2) {
        const int id = find_config(m == 1 ? "v1x1_w8_u4" : "v2x1_w16_u2");
        if (id >= 0) return {id, 1, 1};
    }
    if (m <= 64) {
        const int fm = m <= 16 ? 1 : (m <= 32 ? 2 : 4);
        const char *name = fm == 1 ? "s1x1_w8_u4" : (fm == 2 ? "s2x1_w8_u4" : "s4x1_w16_u1");
        const int id = find_config(name);
        if (id >= 0) return {id, 1, 1};
    }
    // Tiles: minimise (rounds of 256 workgroups) x (tile area / relative efficiency),
    // over the configurations that can run this K.  Efficiencies are measured ratios.
    // eff: throughput per tile area relative to the 256 x 256 tile with the GPU full (measured)
    static const struct { const char *name; double eff; } cands[] = {
        {"q256x256_w2x2_s4o1", 1.00}, {"q256x128_w2x2_s4o1", 0.82}, {"q128x256_w2x2_s4o1", 0.82}, {"q128x128_w2x2_s4o1", 0.60},
        {"q128x64_w2x2_s4o2", 0.46},  {"q64x128_w2x2_s4o2", 0.44},  {"q64x64_w2x2_s4o2", 0.37},
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
            while (ks < 4 && tiles * ks * 2 <= 256 && (k / 128) / (ks * 2) >= 48) ks *= 2;
            if (ks > 1) cost = (double)d.bm * d.bn / c.eff * ((kt + ks - 1) / ks) * 1.25 + 180000.0;
        }
        if (cost < best_cost) { best_cost = cost; best = id; best_ks = ks; }
    }
    if (m <= 128) {
        // 65..128 rows: the wave-level split-K kernel with eight row blocks has no ring to
        // fill and no second kernel, and wins while N x K is small (measured: about 2 us
        // plus 0.38 us per million elements of B, in the units above)
        const int id = find_config("s8x1_w8_u1");
        const double cost_s = (2.0 + (double)n * (double)k / 2.6e6) / 1.65e-5;
        if (id >= 0 && cost_s < best_cost) return {id, 1, 1};
    }
    const int ksplit = best_ks;
    return {best, 4, ksplit};
}

static Choice select_config(int m, int n, int k, int ptr_align, bool has_ws)
{
    static int resolved[sizeof(g_table) / sizeof(g_table[0])];
    static std::once_flag once;
    std::call_once(once, [] {
        for (size_t i = 0; g_table[i].config; ++i) resolved[i] = find_config(g_table[i].config);
    });
    for (size_t i = 0; g_table[i].config; ++i)
        if (g_table[i].m == m && g_table[i].n == n && g_table[i].k == k && resolved[i] >= 0 &&
            config_supports(resolved[i], m, n, k, ptr_align))
            return {resolved[i], g_table[i].group_m, g_table[i].ksplit > 0 ? g_table[i].ksplit : 1, g_table[i].spread};
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
    if (fast_path_ok(m, n, k, ptr_align) && k % 128 == 0) {
        int best = -1;
        double best_cost = 1e300;
        for (const auto &e : g_scaled_tile16) {
            const int id = find_config(e.name);
            if (id < 0) continue;
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
    if (outs * k < (1LL << 27)) return pl;
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

static hipError_t launch_pad_rows(const void *src, void *dst, int rows, int k, int kp, hipStream_t s)
{
    const int kb = k / 2, kbp = kp / 2;
    if (kb % 16 == 0 && ((uintptr_t)src & 15) == 0) {
        const size_t total = (size_t)rows * (kbp / 16);
        pad_rows_vec_kernel<<<dim3(flat_grid(total, 256)), dim3(256), 0, s>>>(static_cast<const v4i *>(src), static_cast<v4i *>(dst), rows, kb / 16, kbp / 16);
    } else {
        const size_t total = (size_t)rows * kbp;
        pad_rows_byte_kernel<<<dim3(flat_grid(total, 256)), dim3(256), 0, s>>>(static_cast<const uint8_t *>(src), static_cast<uint8_t *>(dst), rows, kb, kbp);
    }
    return hipGetLastError();
}

// The padded copies of A and B in the workspace, and the arguments of the GEMM on them.
static hipError_t launch_padded(GemmArgs &p, const PadPlan &pl, void *ws, hipStream_t s)
{
    uint8_t *a_p = static_cast<uint8_t *>(ws), *b_p = a_p + pl.a_bytes;
    hipError_t e = launch_pad_rows(p.A, a_p, p.M, p.K, pl.kp, s);
    if (e != hipSuccess) return e;
    e = launch_pad_rows(p.B, b_p, p.N, p.K, pl.kp, s);
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

// An A of 2 GiB or more is beyond the 32-bit row offsets of the fast kernels; its row blocks
// are independent (block r0.. of A gives rows r0.. of C), so the call is cut into blocks
// of rows that fit, one after the other on the stream (they share the workspace).  Returns
// the rows per block, 0 when the call needs no cutting or cutting does not help (B too large
// as well, or a shape the fast kernels do not take anyway).
static int row_block_for_large_a(int m, int n, int k, int ptr_align)
{
    if (k < 32 || k % 32 != 0 || k > QM_MAX_K_X16 || ptr_align < 16) return 0;
    const long long kb = k / 2;
    if ((long long)m * kb < 0x7fffffffLL || (long long)n * kb >= 0x7fffffffLL) return 0;
    const long long rows = ((0x7fffffffLL - 1) / kb) & ~255LL;
    return rows >= 256 ? (int)rows : 0;
}

}  // namespace qm

using namespace qm;

QM_EXPORT int qm_gemm_i4_ws(const void *A, const void *B, void *C, int m, int n, int k, void *stream, int cfg,
                            void *workspace, size_t workspace_bytes)
{
    const int st = check_gemm_args(A, B, C, m, n, k);
    if (st != QM_OK) return st;
    if (m == 0 || n == 0) return QM_OK;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (k == 0) {
        const size_t cnt = (size_t)m * (size_t)n;
        fill_zero_kernel<<<dim3(flat_grid(cnt, 256)), dim3(256), 0, s>>>(static_cast<int32_t *>(C), cnt);
        const hipError_t e = hipGetLastError();
        return e == hipSuccess ? QM_OK : fail_launch(e);
    }
    const int align = ptr_alignment(A, B);
    if (const int rb = cfg == QM_CFG_AUTO ? row_block_for_large_a(m, n, k, align) : 0) {
        for (int r0 = 0; r0 < m; r0 += rb) {
            const int st_b = qm_gemm_i4_ws(static_cast<const uint8_t *>(A) + (size_t)r0 * (size_t)(k / 2), B,
                                           static_cast<int32_t *>(C) + (size_t)r0 * (size_t)n, m - r0 < rb ? m - r0 : rb, n, k,
                                           stream, cfg, workspace, workspace_bytes);
            if (st_b != QM_OK) return st_b;
        }
        return QM_OK;
    }
    const bool has_ws = workspace != nullptr && workspace_bytes > 0;
    Choice ch;
    if (cfg == QM_CFG_AUTO) {
        ch = select_config(m, n, k, align, has_ws);
    } else {
        ch = choice_from_code(cfg);
        if (!config_supports(ch.cfg, m, n, k, align)) return QM_ERR_CONFIG;
        if (ch.ksplit > 1 && g_configs[ch.cfg].kind != KIND_TILE16) return QM_ERR_CONFIG;
    }
    ch.ksplit = effective_ksplit(g_configs[ch.cfg], k, ch.ksplit);
    GemmArgs p{static_cast<const uint8_t *>(A), static_cast<const uint8_t *>(B), static_cast<int32_t *>(C), m, n, k};
    if (cfg == QM_CFG_AUTO && has_ws) {
        const PadPlan pl = plan_padded_k(m, n, k, align, ch);
        if (pl.on && ((uintptr_t)workspace & 15) == 0 && workspace_bytes >= pl.bytes()) {
            hipError_t e = launch_padded(p, pl, workspace, s);
            if (e == hipSuccess) e = g_configs[pl.ch.cfg].launch(p, s, pl.ch.group_m | (1 << 8) | (pl.ch.spread << 16));
            return e == hipSuccess ? QM_OK : fail_launch(e);
        }
    }
    if (ch.ksplit > 1 && workspace_fits(g_configs[ch.cfg], m, n, ch.ksplit, workspace, workspace_bytes)) {
        const hipError_t e = launch_split_with_workspace(p, ch, workspace, s);
        return e == hipSuccess ? QM_OK : fail_launch(e);
    }
    if (ch.ksplit > 1) {
        // no workspace: split-K partial sums meet in C by integer atomic adds, C starts from zero
        const size_t cnt = (size_t)m * (size_t)n;
        fill_zero_kernel<<<dim3(flat_grid(cnt, 256)), dim3(256), 0, s>>>(static_cast<int32_t *>(C), cnt);
        const hipError_t ez = hipGetLastError();
        if (ez != hipSuccess) return fail_launch(ez);
    }
    const hipError_t e = g_configs[ch.cfg].launch(p, s, ch.group_m | (ch.ksplit << 8) | (ch.spread << 16));
    return e == hipSuccess ? QM_OK : fail_launch(e);
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
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (k == 0) {
        const size_t cnt = (size_t)m * (size_t)n;
        fill_zero16_kernel<<<dim3(flat_grid(cnt, 256)), dim3(256), 0, s>>>(static_cast<uint16_t *>(D), cnt);
        const hipError_t e = hipGetLastError();
        return e == hipSuccess ? QM_OK : fail_launch(e);
    }
    const int align = ptr_alignment(A, B);
    if (const int rb = cfg == QM_CFG_AUTO ? row_block_for_large_a(m, n, k, align) : 0) {
        for (int r0 = 0; r0 < m; r0 += rb) {
            const int st_b = qm_gemm_i4_scaled_ws(static_cast<const uint8_t *>(A) + (size_t)r0 * (size_t)(k / 2), B,
                                                  static_cast<uint16_t *>(D) + (size_t)r0 * (size_t)n, m - r0 < rb ? m - r0 : rb, n,
                                                  k, row_scale ? row_scale + r0 : nullptr, col_scale, out_dtype, stream, cfg,
                                                  workspace, workspace_bytes);
            if (st_b != QM_OK) return st_b;
        }
        return QM_OK;
    }
    const bool has_ws = workspace != nullptr && workspace_bytes > 0;
    GemmArgs p{static_cast<const uint8_t *>(A), static_cast<const uint8_t *>(B), static_cast<int32_t *>(D), m, n, k};
    p.row_scale = row_scale;
    p.col_scale = col_scale;
    p.out = out_dtype == QM_OUT_F16 ? OUT_F16 : OUT_BF16;
    Choice ch;
    if (cfg == QM_CFG_AUTO) {
        ch = select_scaled(m, n, k, align, has_ws);
        ch.ksplit = effective_ksplit(g_configs[ch.cfg], k, ch.ksplit);
        if (ch.ksplit > 1 && !workspace_fits(g_configs[ch.cfg], m, n, ch.ksplit, workspace, workspace_bytes)) {
            ch = select_scaled(m, n, k, align, false);  // too small a workspace: as without one
            ch.ksplit = 1;
        }
    } else {
        ch = choice_from_code(cfg);
        if (!config_supports(ch.cfg, m, n, k, align)) return QM_ERR_CONFIG;
        if (ch.ksplit > 1 && g_configs[ch.cfg].kind != KIND_TILE16) return QM_ERR_CONFIG;
        ch.ksplit = effective_ksplit(g_configs[ch.cfg], k, ch.ksplit);
        // partial sums cannot meet in a rounded output: a K split needs the workspace
        if (ch.ksplit > 1 && !workspace_fits(g_configs[ch.cfg], m, n, ch.ksplit, workspace, workspace_bytes)) return QM_ERR_CONFIG;
    }
    if (ch.ksplit > 1) {
        const hipError_t e = launch_split_with_workspace(p, ch, workspace, s);
        return e == hipSuccess ? QM_OK : fail_launch(e);
    }
    if (cfg == QM_CFG_AUTO && has_ws) {
        PadPlan pl = plan_padded_k(m, n, k, align, ch);
        if (pl.on && !scaled_launcher(pl.ch.cfg)) {
            // a pipelined configuration that has the scaled output, if the shape is one for those
            const int id = find_config(g_configs[pl.ch.cfg].kind == KIND_TILE16 ? "q256x256_w2x2_s4o1" : "q128x128_w2x2_s4o1");
            if (id >= 0) pl.ch.cfg = id; else pl.on = false;
        }
        if (pl.on && ((uintptr_t)workspace & 15) == 0 && workspace_bytes >= pl.bytes()) {
            hipError_t e = launch_padded(p, pl, workspace, s);
            if (e == hipSuccess) e = scaled_launcher(pl.ch.cfg)(p, s, pl.ch.group_m | (1 << 8) | (pl.ch.spread << 16));
            return e == hipSuccess ? QM_OK : fail_launch(e);
        }
    }
    const LaunchFn launch = scaled_launcher(ch.cfg);
    if (!launch) return QM_ERR_CONFIG;
    const hipError_t e = launch(p, s, ch.group_m | (1 << 8) | (ch.spread << 16));
    return e == hipSuccess ? QM_OK : fail_launch(e);
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
    default: return "unknown status";
    }
}

QM_EXPORT int qm_last_hip_error(void) { return g_last_hip_error; }

QM_EXPORT const char *qm_version(void) { return "quadmul-amd 0.1 (gfx950)"; }
