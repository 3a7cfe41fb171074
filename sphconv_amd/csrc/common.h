// Internal helpers shared by the HIP translation units of libsphconv_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/sphconv_hip.h"

#define SPH_EXPORT extern "C" __attribute__((visibility("default")))

void sph_set_error(const char *fmt, ...);

#define SPH_REQUIRE(cond, code, ...)      \
    do {                                  \
        if (!(cond)) {                    \
            sph_set_error(__VA_ARGS__);   \
            return (code);                \
        }                                 \
    } while (0)

// Called after every launch: turns a launch failure into a status code.
static inline int sph_check_launch(const char *what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        sph_set_error("%s: %s", what, hipGetErrorString(e));
        return SPH_ERR_LAUNCH;
    }
    return SPH_OK;
}

static inline int sph_div_up(int a, int b) { return (a + b - 1) / b; }

static inline int sph_geom_ok(const sph_geom *g)
{
    if (!g || g->B <= 0) return 0;
    for (int d = 0; d < 3; d++)
        if (g->S[d] <= 0 || g->O[d] <= 0 || g->K[d] <= 0 || g->stride[d] <= 0 || g->pad[d] < 0)
            return 0;
    long kv = (long)g->K[0] * g->K[1] * g->K[2];
    if (kv > SPH_MAX_KV) return 0;
    long icol = (long)g->B * g->S[0] * g->S[1], ocol = (long)g->B * g->O[0] * g->O[1];
    if (icol > 0x7fffffffL || ocol > 0x7fffffffL) return 0;
    return 1;
}

// Workgroups are handed to the 8 XCDs of an MI355X round robin (workgroup i runs on
// XCD i % 8) and every XCD has its own L2.  Neighbouring tiles share feature rows and
// index ranges, so each XCD is given one contiguous run of tiles: launch
// sph_xcd_grid(ntiles) workgroups and map blockIdx.x with sph_xcd_tile(); a result
// >= ntiles means "no tile, exit".
#define SPH_NUM_XCD 8
static inline int sph_xcd_grid(int ntiles) { return sph_div_up(ntiles, SPH_NUM_XCD) * SPH_NUM_XCD; }
#ifdef __HIPCC__
__device__ __forceinline__ int sph_xcd_tile(int block, int ntiles)
{
    const int per_xcd = (ntiles + SPH_NUM_XCD - 1) / SPH_NUM_XCD;
    return (block % SPH_NUM_XCD) * per_xcd + block / SPH_NUM_XCD;
}
#endif
