// Host-side helpers shared by the C-ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/kfac_hip.h"

namespace kfac {

// Number of workgroups that fill the chip about twice (256 CUs, 2 resident
// workgroups of this engine per CU); used to choose k-splits.
constexpr int TARGET_BLOCKS = 1024;

inline int cdiv(int a, int b) { return (a + b - 1) / b; }

inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? KFAC_OK : KFAC_ERR_LAUNCH;
}

// k-split heuristic for a symmetric d x d product with reduction length K.
// Returns the number of splits; *chunks_per_split is in units of 16 k.
int choose_splits(int ntiles, long K, int* chunks_per_split);

}  // namespace kfac
