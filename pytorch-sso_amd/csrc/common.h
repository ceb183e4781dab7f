// Host-side helpers shared by the C-ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/kfac_hip.h"

namespace kfac {

inline int cdiv(int a, int b) { return (a + b - 1) / b; }

inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? KFAC_OK : KFAC_ERR_LAUNCH;
}

}  // namespace kfac
