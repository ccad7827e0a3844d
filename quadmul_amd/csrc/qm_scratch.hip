// Library-owned scratch memory for qm_gemm_i4_static (include/qm_abi.h), in a translation
// unit of its own with no kernels in it: the code object that holds the array -- and with it
// the array's QM_STATIC_SCRATCH_BYTES of device memory on every GPU the process uses -- is
// loaded by the first qm_gemm_i4_static or qm_init call, not by the first launch of any GEMM
// kernel.  The reference has no scratch memory (its wrapper, kernel.cu:334, never splits K).
//
// In host code the array's name is only a handle for hipGetSymbolAddress: every device has
// its own copy at its own address, looked up once per device (with that device current) and
// kept; kernels and every other use take that pointer.
#include <atomic>

#include "../../include/qm_abi.h"
#include "qm_launch.hpp"

static __device__ __align__(256) unsigned char scratch[QM_STATIC_SCRATCH_BYTES];

namespace qm {

static std::atomic<void *> g_scratch_ptr[QM_MAX_DEVICES] = {};

hipError_t static_scratch(void **out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= QM_MAX_DEVICES) return hipErrorInvalidDevice;
    void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (ptr == nullptr || ((uintptr_t)ptr & 255) != 0) return hipErrorInvalidSymbol;
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return hipSuccess;
}

}  // namespace qm
