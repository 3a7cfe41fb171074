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
// Inclusive sum over the wave's 64 lanes through the data-parallel-primitive lane shifts of the vector ALU
// (four shifts inside a row of 16 lanes, then lane 15 and lane 31 broadcast into the rows behind them):
// no LDS round trip per step as a shuffle has.
__device__ __forceinline__ int wave_inclusive_sum(int x)
{
    x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xf, 0xf, false); // row_shr:1
    x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xf, 0xf, false); // row_shr:2
    x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xf, 0xf, false); // row_shr:4
    x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xf, 0xf, false); // row_shr:8
    x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xa, 0xf, false); // row_bcast:15 into rows 1 and 3
    x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xc, 0xf, false); // row_bcast:31 into rows 2 and 3
    return x;
}

#endif
} // namespace
