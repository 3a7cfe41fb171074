// Constants every kernel of the convolution path shares.
#pragma once
#include "common.h"

namespace {
constexpr int R = SPH_TILE_ROWS; // stationary rows per tile
constexpr int kWave = 64;        // lanes per wavefront

#ifdef __HIPCC__
// Barrier for data exchanged through LDS only.  __syncthreads() also waits for every global load and store of
// the thread that is still in flight (a full memory round trip each time one is pending); the rule kernels
// share nothing through global memory inside a workgroup, so their barriers order LDS accesses alone.
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}
#endif
} // namespace
