// Measurement probes for bench.py (libqm_probe.so): what the part itself sustains, to set
// beside the nominal peaks the roofline fractions are quoted against.  Not part of the GEMM
// library and not linked into it.  The timing method follows the reference's own harness
// (kernel.cu:468-497: warm-ups, then launches between two events), with the kernels below
// in place of the GEMM.
//
//   qm_probe_mfma_issue   a loop of independent v_mfma_i32_16x16x64_i8 on operands of the
//                         form 16 * s4 (low nibble zero), the instruction and the operand
//                         form of the GEMM kernels, with nothing else in the loop: the
//                         issue peak of the matrix cores at the clock the part sustains,
//                         with every MFMA on the same operand registers or rotating over
//                         four pairs of them
//   qm_probe_empty        a kernel that does nothing: the launch floor
//   qm_probe_read         a kernel that only reads `bytes` (16 bytes per lane, whole lines)
//                         and keeps a checksum: the floor of "launch + one pass over B"
#include <hip/hip_runtime.h>
#include <stdint.h>

#define QM_PROBE_EXPORT extern "C" __attribute__((visibility("default")))

typedef int v4i __attribute__((ext_vector_type(4)));

namespace {

constexpr int MFMA_PER_ITER = 16;   // independent accumulators: 16 x 4 AGPRs
constexpr int MFMA_OPS = 2 * 16 * 16 * 64;

// One workgroup of four waves (one per SIMD) per launch slot; `iters` trips of 16 MFMAs.
// PAIRS: distinct operand register pairs the MFMAs of a trip rotate over (1: every MFMA reads
// the same two registers, so the operand buses never toggle -- an upper bound under a power
// cap; 4: consecutive MFMAs read different pseudo-random operands, as the GEMM's do).
// out[2 * block], out[2 * block + 1]: what the two counters of the core (s_memtime) and of
// the constant 100 MHz reference (s_memrealtime) advanced by around the loop, from wave 0.
template <int PAIRS>
__global__ void __launch_bounds__(256) mfma_issue_kernel(uint64_t *out, int iters, uint32_t seed)
{
    // pseudo-random nibbles in the high half of every byte: the matrix cores draw power by
    // the bits that toggle, so all-zero operands would flatter the result
    uint32_t h = (threadIdx.x + 1) * 2654435761u + blockIdx.x * 40503u + seed;
    v4i s0[PAIRS], s1[PAIRS];
#pragma unroll
    for (int q = 0; q < PAIRS; ++q)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            h ^= h << 13; h ^= h >> 17; h ^= h << 5;
            s0[q][i] = (int)(h & 0xF0F0F0F0u);
            h ^= h << 13; h ^= h >> 17; h ^= h << 5;
            s1[q][i] = (int)(h & 0xF0F0F0F0u);
        }
    v4i acc[MFMA_PER_ITER];
#pragma unroll
    for (int i = 0; i < MFMA_PER_ITER; ++i) acc[i] = v4i{0, 0, 0, 0};
    const uint64_t t0 = __builtin_readcyclecounter(), r0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < MFMA_PER_ITER; ++i)
            asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(acc[i]) : "v"(s0[i % PAIRS]), "v"(s1[i % PAIRS]));
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    const uint64_t t1 = __builtin_readcyclecounter(), r1 = wall_clock64();
    int sum = 0;
#pragma unroll
    for (int i = 0; i < MFMA_PER_ITER; ++i) sum += acc[i].x ^ acc[i].y ^ acc[i].z ^ acc[i].w;
    if (threadIdx.x == 0) {
        out[2 * blockIdx.x] = t1 - t0;
        out[2 * blockIdx.x + 1] = r1 - r0;
    }
    if (sum == 0x7fffffff && iters < 0) out[0] = (uint64_t)sum;  // keeps the accumulators alive
}

__global__ void empty_kernel() {}

// (launched with 256 or 1024 threads per workgroup and any amount of dynamic LDS, which it
// does not touch: the launch shape is part of what is measured)
__global__ void __launch_bounds__(1024) read_kernel(const v4i *src, size_t n16, int *sink)
{
    extern __shared__ __align__(16) uint8_t unused_lds[];
    v4i acc = {0, 0, 0, 0};
    const size_t per = (size_t)blockDim.x * 4, stride = (size_t)gridDim.x * per;
    for (size_t i = (size_t)blockIdx.x * per + threadIdx.x; i < n16; i += stride) {
        v4i v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = i + u * blockDim.x < n16 ? __builtin_nontemporal_load(src + i + u * blockDim.x) : v4i{0, 0, 0, 0};
#pragma unroll
        for (int u = 0; u < 4; ++u) acc ^= v[u];
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x5A5A5A5B) *sink = 1 + (int)(uintptr_t)unused_lds;  // (practically never: keeps the loads)
}

}  // namespace

// Enqueues one launch of `blocks` workgroups x 4 waves x iters x 16 MFMAs.  out: device
// memory for 2 * blocks uint64.  operand_pairs: 1 or 4 (see the kernel).  Returns the integer
// operations of the launch (2 * 16 * 16 * 64 per MFMA per wave) as a double, or a negative
// hipError_t.
QM_PROBE_EXPORT double qm_probe_mfma_issue(void *out, int blocks, int iters, int operand_pairs, void *stream)
{
    if (!out || blocks < 1 || iters < 1 || (operand_pairs != 1 && operand_pairs != 4)) return -1.0;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (operand_pairs == 1) mfma_issue_kernel<1><<<dim3(blocks), dim3(256), 0, s>>>(static_cast<uint64_t *>(out), iters, 12345u);
    else mfma_issue_kernel<4><<<dim3(blocks), dim3(256), 0, s>>>(static_cast<uint64_t *>(out), iters, 12345u);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return -(double)(int)e;
    return (double)blocks * 4.0 * (double)iters * MFMA_PER_ITER * (double)MFMA_OPS;
}

QM_PROBE_EXPORT int qm_probe_empty(void *stream)
{
    empty_kernel<<<dim3(1), dim3(64), 0, reinterpret_cast<hipStream_t>(stream)>>>();
    return (int)hipGetLastError();
}

// `src`: 16-byte aligned device memory of `bytes` bytes (a multiple of 16); `sink`: one int.
// `threads` per workgroup: 64 .. 1024; `lds_bytes` of dynamic LDS per workgroup (untouched).
QM_PROBE_EXPORT int qm_probe_read(const void *src, size_t bytes, void *sink, int blocks, int threads, int lds_bytes, void *stream)
{
    if (!src || !sink || (bytes & 15) || ((uintptr_t)src & 15) || blocks < 1 || threads < 64 || threads > 1024 || (threads & 63) || lds_bytes < 0 ||
        lds_bytes > 160 * 1024)
        return -1;
    if (lds_bytes > 64 * 1024) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&read_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return (int)e;
    }
    read_kernel<<<dim3(blocks), dim3(threads), lds_bytes, reinterpret_cast<hipStream_t>(stream)>>>(static_cast<const v4i *>(src), bytes / 16, static_cast<int *>(sink));
    return (int)hipGetLastError();
}
