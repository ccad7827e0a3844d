// Host-side launch plumbing shared by the translation units of libqm_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>
#include "qm_common.hpp"

namespace qm {

// Launchers return hipSuccess or the error of the failed runtime call.
typedef hipError_t (*LaunchFn)(const GemmArgs &, hipStream_t, int group_m);

constexpr int QM_MAX_DEVICES = 64;
// bit of a launcher's third argument: do the kernel's one-off set-up on the current device
// (LDS size attribute, residency query) and return without launching
constexpr int QM_OPT_PREPARE = 1 << 17;

// K split of the pipelined kernel, normalised: kt K-steps of 128 nibbles (the last one may
// be short); with kps steps per split only ceil(kt / kps) splits have work; and a split
// that holds a short last step keeps at least two steps (the kernel widens that step's B
// operand during the step before it, inside the same work item).
inline int normalised_ksplit(int K, int ksplit)
{
    const int kt = (K + 127) / 128;
    if (ksplit < 1) ksplit = 1;
    for (;;) {
        const int kps = (kt + ksplit - 1) / ksplit;
        ksplit = (kt + kps - 1) / kps;
        if (ksplit == 1 || (K & 127) == 0 || kt - (ksplit - 1) * kps >= 2) return ksplit;
        --ksplit;
    }
}

// Kernels that want more than 64 KiB of dynamic LDS must say so once per device.  (The
// flags are atomics: several host threads may launch at once; setting the attribute twice
// is harmless.)
template <class KernelPtr>
inline hipError_t ensure_dynamic_lds(KernelPtr kernel, int bytes, std::atomic<bool> *done_per_device)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= QM_MAX_DEVICES) return hipErrorInvalidDevice;
    if (!done_per_device[dev].load(std::memory_order_acquire)) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (e != hipSuccess) return e;
        done_per_device[dev].store(true, std::memory_order_release);
    }
    return hipSuccess;
}

// The address, on the current device, of the library's own scratch array (qm_scratch.hip).
hipError_t static_scratch(void **out);

#define QM_SKINNY_FN(FM, FN, NW, U) qm_launch_skinny_##FM##_##FN##_##NW##_##U
#define QM_DOT_FN(MR, FN, NW, U) qm_launch_dot_##MR##_##FN##_##NW##_##U
#define QM_SKINNYD_FN(FM, FN, NW, D) qm_launch_skinnyd_##FM##_##FN##_##NW##_##D
#define QM_SKINNYP_FN(FM, FN, NW, D, R) qm_launch_skinnyp_##FM##_##FN##_##NW##_##D##_##R
#define QM_TILE16_FN(BM, BN, WGM, WGN, ST, OCC) qm_launch_tile16_##BM##_##BN##_##WGM##_##WGN##_##ST##_##OCC
#define QM_TILE16S_FN(BM, BN, WGM, WGN, ST, OCC) qm_launch_tile16s_##BM##_##BN##_##WGM##_##WGN##_##ST##_##OCC

#define QM_TILE16(tu, BM, BN, WGM, WGN, ST, OCC) hipError_t QM_TILE16_FN(BM, BN, WGM, WGN, ST, OCC)(const GemmArgs &, hipStream_t, int);
#define QM_TILE16S(tu, BM, BN, WGM, WGN, ST, OCC) hipError_t QM_TILE16S_FN(BM, BN, WGM, WGN, ST, OCC)(const GemmArgs &, hipStream_t, int);
#define QM_SKINNY(FM, FN, NW, U) hipError_t QM_SKINNY_FN(FM, FN, NW, U)(const GemmArgs &, hipStream_t, int);
#define QM_DOT(MR, FN, NW, U) hipError_t QM_DOT_FN(MR, FN, NW, U)(const GemmArgs &, hipStream_t, int);
#define QM_SKINNYD(FM, FN, NW, D) hipError_t QM_SKINNYD_FN(FM, FN, NW, D)(const GemmArgs &, hipStream_t, int);
#define QM_SKINNYP(FM, FN, NW, D, R) hipError_t QM_SKINNYP_FN(FM, FN, NW, D, R)(const GemmArgs &, hipStream_t, int);
#include "qm_configs.inc"

}  // namespace qm
