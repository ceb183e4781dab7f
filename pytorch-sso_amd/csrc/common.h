// Host-side helpers shared by the C-ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/kfac_hip.h"

namespace kfac {

inline int cdiv(int a, int b) { return (a + b - 1) / b; }

// Kernels built on the 2x2 tile engine stage 72 KiB in LDS, above the 64 KiB
// that a kernel may use without opting in; the opt-in is done once per kernel.
bool enable_large_lds(const void* kernel, int bytes);

#define KFAC_LAUNCH_TILE2(kernel, grid, stream, ...)                                         \
  do {                                                                                       \
    constexpr int lds_bytes_ = kfac::Cfg<2, 2>::SMEM_FLOATS * (int)sizeof(float);            \
    if (kfac::enable_large_lds((const void*)(kernel), lds_bytes_))                           \
      hipLaunchKernelGGL((kernel), (grid), dim3(kfac::NTHREADS), lds_bytes_, (stream),       \
                         __VA_ARGS__);                                                       \
  } while (0)

inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? KFAC_OK : KFAC_ERR_LAUNCH;
}

}  // namespace kfac
