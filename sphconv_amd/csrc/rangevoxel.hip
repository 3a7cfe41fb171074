// Point cloud -> range voxels (one voxel per range-image pixel), replacing the numpy
// code of xyz2RangeVoxel (sphconv/data.py:75-128, whose own note says "CUDA accelerate
// this").  Arithmetic follows the reference operation by operation in float32, each
// product and sum rounded on its own (no fused multiply-add), truncation toward zero,
// then clamping into the grid:
//   r = sqrt(x*x + y*y + z*z); theta = acos(z / r); phi = asin(y / sqrt(x*x + y*y))
//   theta_idx = int((theta - v0) / dtheta), phi_idx = int((phi - h0) / dphi)
//   depth = (log(r) - log(d0)) / dr   or   (r - d0) / dr, clamped as a float, then int
// Points that land on the same pixel: the reference's indexed assignment lets the later
// point win; here a first kernel keeps the largest point index per pixel (atomicMax), a
// second one writes the winners -- the same result, deterministic.
#include "common.h"

namespace {

struct RangeParams {
    int v_res, h_res, d_res;
    float v0, h0, dtheta, dphi;   // radians
    float d0, dr;                 // log(d_range[0]) and log step if use_log, else d_range[0] and linear step
    int use_log;
};

__device__ __forceinline__ void range_index(const float *p, const RangeParams &q, int &ti, int &pi, int &di)
{
    const float x = p[0], y = p[1], z = p[2];
    const float x2y2 = __fadd_rn(__fmul_rn(x, x), __fmul_rn(y, y));
    const float r = __fsqrt_rn(__fadd_rn(x2y2, __fmul_rn(z, z)));
    const float theta = acosf(__fdiv_rn(z, r));
    const float phi = asinf(__fdiv_rn(y, __fsqrt_rn(x2y2)));
    const float tf = __fdiv_rn(__fsub_rn(theta, q.v0), q.dtheta);
    const float pf = __fdiv_rn(__fsub_rn(phi, q.h0), q.dphi);
    float df = q.use_log ? __fdiv_rn(__fsub_rn(logf(r), q.d0), q.dr) : __fdiv_rn(__fsub_rn(r, q.d0), q.dr);
    // float -> int truncates toward zero; NaN (a point on the z axis) becomes 0 like every
    // value below the range
    ti = (tf == tf) ? (int)fminf(fmaxf(tf, -1.f), (float)q.v_res) : 0;
    pi = (pf == pf) ? (int)fminf(fmaxf(pf, -1.f), (float)q.h_res) : 0;
    ti = min(max(ti, 0), q.v_res - 1);
    pi = min(max(pi, 0), q.h_res - 1);
    // the depth index is clamped as a float first (data.py:103-104), then truncated
    if (!(df == df) || df < 0.f) df = 0.f;
    if (df >= (float)q.d_res) df = (float)(q.d_res - 1);
    di = (int)df;
}

__global__ void range_winner_kernel(const float *points, int m, int ndim, RangeParams q, int32_t *winner, int32_t *idx_out)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= m) return;
    int ti, pi, di;
    range_index(points + (long)i * ndim, q, ti, pi, di);
    if (idx_out) {
        idx_out[3 * (long)i] = ti;
        idx_out[3 * (long)i + 1] = pi;
        idx_out[3 * (long)i + 2] = di;
    }
    atomicMax(&winner[ti * q.h_res + pi], i);
}

__global__ void range_fill_kernel(int32_t *winner, int npix)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < npix) winner[i] = -1;
}

// one thread per pixel: feature [C][V*H], depth [V*H], thick [V*H]
__global__ void range_write_kernel(const float *points, int m, int ndim, RangeParams q, const int32_t *winner,
                                   float *feature, int32_t *depth, int32_t *thick)
{
    const int pix = blockIdx.x * blockDim.x + threadIdx.x;
    const int npix = q.v_res * q.h_res;
    if (pix >= npix) return;
    const int w = winner[pix];
    if ((unsigned)w >= (unsigned)m) {
        for (int c = 0; c < ndim; c++) feature[(long)c * npix + pix] = 0.f;
        depth[pix] = 0;
        thick[pix] = 0;
        return;
    }
    const float *p = points + (long)w * ndim;
    int ti, pi, di;
    range_index(p, q, ti, pi, di);
    for (int c = 0; c < ndim; c++) feature[(long)c * npix + pix] = p[c];
    depth[pix] = di;
    thick[pix] = 1;
}

} // namespace

SPH_EXPORT int sph_xyz_to_rangevoxel(const float *points, int m, int ndim, int v_res, int h_res, int d_res,
                                     float v0_rad, float h0_rad, float dtheta, float dphi, float d0, float dr,
                                     int use_log, int32_t *winner, float *feature, int32_t *depth, int32_t *thick,
                                     int32_t *idx_out, void *stream)
{
    SPH_REQUIRE(m >= 0 && ndim >= 3 && v_res > 0 && h_res > 0 && d_res > 0, SPH_ERR_ARG,
                "sph_xyz_to_rangevoxel: bad sizes (points need at least x, y, z)");
    SPH_REQUIRE((double)v_res * h_res < 2147483648.0, SPH_ERR_UNSUPPORTED, "sph_xyz_to_rangevoxel: image too large");
    SPH_REQUIRE(winner && feature && depth && thick && (m == 0 || points), SPH_ERR_ARG,
                "sph_xyz_to_rangevoxel: null pointer");
    SPH_REQUIRE(dtheta != 0.f && dphi != 0.f && dr != 0.f, SPH_ERR_ARG, "sph_xyz_to_rangevoxel: empty range");
    RangeParams q;
    q.v_res = v_res; q.h_res = h_res; q.d_res = d_res;
    q.v0 = v0_rad; q.h0 = h0_rad; q.dtheta = dtheta; q.dphi = dphi; q.d0 = d0; q.dr = dr; q.use_log = use_log;
    hipStream_t st = (hipStream_t)stream;
    const int npix = v_res * h_res;
    hipLaunchKernelGGL(range_fill_kernel, dim3((npix + 255) / 256), dim3(256), 0, st, winner, npix);
    if (m > 0)
        hipLaunchKernelGGL(range_winner_kernel, dim3((m + 255) / 256), dim3(256), 0, st, points, m, ndim, q, winner,
                           idx_out);
    hipLaunchKernelGGL(range_write_kernel, dim3((npix + 255) / 256), dim3(256), 0, st, points, m, ndim, q,
                       (const int32_t *)winner, feature, depth, thick);
    return sph_check_launch("sph_xyz_to_rangevoxel");
}
