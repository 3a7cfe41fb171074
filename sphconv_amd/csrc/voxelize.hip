// Point cloud -> voxels with up to max_points points each, replacing the sequential CPU loop of
// points_to_voxel_3d (include/point2voxel.h:412-512, called from sphconv/utils/voxelize.py:126-214)
// and the coordinate transforms of sphconv/utils/coord_transform.py:8-118.
//
// The reference walks the points in order: a point outside the grid is skipped; a point in a
// new cell opens the next voxel, unless max_voxels are open already -- then the whole loop
// stops; a voxel keeps its first max_points points.  The same result without the sequential
// loop:
//   1. vox_cell_kernel   system coordinates (float32, operation by operation as numpy does it)
//                        and the cell of every point; points outside get the largest key
//   2. stable radix sort of (cell, point index): a cell's points become one segment, in point
//                        order, so a segment's head is the point that opens the voxel
//   3. vox_head_kernel   marks the heads in point order and in sorted order
//   4. scans             exclusive sum of the marks in point order = voxel number of each head;
//                        running maximum of the head positions = each entry's segment start
//   5. vox_stop_kernel   the point that would open voxel number max_voxels is where the
//                        reference's loop stops: every later point is dropped
//   6. vox_write_kernel  entry j of a segment is the voxel's (j - start)-th point
// Nothing is allocated; keys, marks and the library scratch live in the caller's workspace.
#include "common.h"

#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

#include "scan.h"

namespace {

enum { SYS_SPHERICAL = 0, SYS_LSPHERICAL, SYS_CYLINDER, SYS_LCYLINDER, SYS_HYBRID, SYS_LHYBRID, SYS_COUNT };

struct VoxParams {
    int system, nfeat, append_mode, max_points, max_voxels;
    float lo[3], vs[3];   // lower bound and voxel size per system coordinate
    int grid[3];
    unsigned long long cells;
};

// (c0, c1, c2) of a point in the chosen system; every operation rounded to float32 on its own
__device__ __forceinline__ void system_coords(const float *p, int system, float (&c)[3])
{
    const float x = p[0], y = p[1], z = p[2];
    const float x2y2 = __fadd_rn(__fmul_rn(x, x), __fmul_rn(y, y));
    const float d = __fsqrt_rn(x2y2);
    const float phi = asinf(__fdiv_rn(y, d));
    c[1] = phi;
    if (system == SYS_CYLINDER || system == SYS_LCYLINDER) {
        c[0] = system == SYS_CYLINDER ? d : logf(d);
        c[2] = z;
        return;
    }
    const float r = __fsqrt_rn(__fadd_rn(x2y2, __fmul_rn(z, z)));
    c[2] = acosf(__fdiv_rn(z, r));
    switch (system) {
    case SYS_SPHERICAL: c[0] = r; break;
    case SYS_LSPHERICAL: c[0] = logf(r); break;
    case SYS_HYBRID: c[0] = d; break;
    default: c[0] = logf(d); break;
    }
}

// bins (idx of c0, c1, c2) or false if the point is outside the grid (point2voxel.h:447-457)
__device__ __forceinline__ bool cell_of(const float (&c)[3], const VoxParams &q, int (&bin)[3])
{
    bool ok = true;
#pragma unroll
    for (int i = 0; i < 3; i++) {
        const float f = floorf(__fdiv_rn(__fsub_rn(c[i], q.lo[i]), q.vs[i]));
        ok = ok && f >= 0.f && f < (float)q.grid[i]; // false for NaN
        bin[i] = ok ? (int)f : 0;
    }
    return ok;
}

__global__ void vox_cell_kernel(const float *points, int n, VoxParams q, const long long *cell_in, uint64_t *keys,
                                int32_t *vals, long long *cell_out)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    uint64_t key = q.cells; // outside: sorts behind every cell
    if (cell_in) {
        const long long c = cell_in[i];
        if (c >= 0 && (unsigned long long)c < q.cells) key = (uint64_t)c;
    } else {
        float c[3];
        int bin[3];
        system_coords(points + (long)i * q.nfeat, q.system, c);
        // the reference indexes its map [c2 bin][c1 bin][c0 bin]
        if (cell_of(c, q, bin)) key = ((uint64_t)bin[2] * q.grid[1] + bin[1]) * q.grid[0] + bin[0];
    }
    keys[i] = key;
    vals[i] = i;
    if (cell_out) cell_out[i] = key == q.cells ? -1 : (long long)key;
}

__global__ void vox_fill_kernel(int32_t *p, long n, int32_t v)
{
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

__global__ void vox_head_kernel(const uint64_t *keys, const int32_t *vals, int n, uint64_t cells, int32_t *mark_pt,
                                int32_t *start_in)
{
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= n) return;
    const uint64_t k = keys[j];
    const bool head = k != cells && (j == 0 || keys[j - 1] != k);
    start_in[j] = head ? j : 0;
    if (head) mark_pt[vals[j]] = 1;
}

__global__ void vox_stop_kernel(const int32_t *mark_pt, const int32_t *vid_pt, int n, int max_voxels, int32_t *stop,
                                int32_t *voxel_num)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    if (mark_pt[i] && vid_pt[i] == max_voxels) *stop = i;          // exactly one such point, if any
    if (i == n - 1) *voxel_num = min(vid_pt[i] + mark_pt[i], max_voxels);
}

__global__ void vox_write_kernel(const float *points, int n, VoxParams q, const uint64_t *keys, const int32_t *vals,
                                 const int32_t *start, const int32_t *vid_pt, const int32_t *stop, float *voxels,
                                 float *mask, int32_t *coors, int32_t *num_points)
{
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= n) return;
    const uint64_t key = keys[j];
    if (key == q.cells) return;
    const int h = start[j];
    const int vid = vid_pt[vals[h]];
    const int i = vals[j];
    if (vid >= q.max_voxels || i >= *stop) return;
    if (j == h) {
        const int b0 = (int)(key % q.grid[0]);
        const uint64_t t = key / q.grid[0];
        coors[3 * (long)vid] = (int)(t / q.grid[1]);       // c2 bin
        coors[3 * (long)vid + 1] = (int)(t % q.grid[1]);   // c1 bin
        coors[3 * (long)vid + 2] = b0;                     // c0 bin
    }
    const int rank = j - h;
    if (rank >= q.max_points) return;
    const int width = q.append_mode == 1 ? q.nfeat + 3 : q.nfeat;
    float *dst = voxels + ((long)vid * q.max_points + rank) * width;
    const float *p = points + (long)i * q.nfeat;
    if (q.append_mode == 2) {
        float c[3];
        system_coords(p, q.system, c);
        dst[0] = c[0]; dst[1] = c[1]; dst[2] = c[2]; dst[3] = p[3];
    } else {
        for (int f = 0; f < q.nfeat; f++) dst[f] = p[f];
        if (q.append_mode == 1) {
            float c[3];
            system_coords(p, q.system, c);
            dst[q.nfeat] = c[0]; dst[q.nfeat + 1] = c[1]; dst[q.nfeat + 2] = c[2];
        }
    }
    mask[(long)vid * q.max_points + rank] = 1.f;
    atomicMax(&num_points[vid], rank + 1);
}

struct VoxLayout {
    size_t keys_in, keys_out, vals_in, vals_out, mark, vid, start_in, start, stop, temp, temp_bytes, total;
};

inline size_t al256(size_t x) { return (x + 255) & ~(size_t)255; }
inline int bits_for(unsigned long long v)
{
    int b = 1;
    while (b < 64 && (1ULL << b) <= v) b++;
    return b;
}

inline VoxLayout vox_layout(int n, unsigned long long cells)
{
    VoxLayout l;
    const size_t nn = (size_t)(n > 0 ? n : 1);
    size_t o = 0;
    l.keys_in = o; o += al256(nn * 8);
    l.keys_out = o; o += al256(nn * 8);
    l.vals_in = o; o += al256(nn * 4);
    l.vals_out = o; o += al256(nn * 4);
    l.mark = o; o += al256(nn * 4);
    l.vid = o; o += al256(nn * 4);
    l.start_in = o; o += al256(nn * 4);
    l.start = o; o += al256(nn * 4);
    l.stop = o; o += 256;
    l.temp = o;
    // the sort's temporary storage (what rocPRIM asks for) and the scans' state share one area
    size_t sort_b = 0;
    hipError_t e = rocprim::radix_sort_pairs(nullptr, sort_b, (const uint64_t *)nullptr, (uint64_t *)nullptr,
                                             (const int32_t *)nullptr, (int32_t *)nullptr, nn, 0, bits_for(cells),
                                             (hipStream_t)0);
    const size_t scan_b = sph_scan::state_bytes((long)nn);
    const size_t t = sort_b > scan_b ? sort_b : scan_b;
    l.temp_bytes = e == hipSuccess ? t + 256 : 0;
    l.total = l.temp_bytes ? o + al256(l.temp_bytes) : 0;
    return l;
}

inline unsigned blocks(long n) { return (unsigned)((n + 255) / 256); }

} // namespace

SPH_EXPORT size_t sph_points_to_voxel_workspace(int n, int g0, int g1, int g2)
{
    if (n < 0 || g0 <= 0 || g1 <= 0 || g2 <= 0) return 0;
    return vox_layout(n, (unsigned long long)g0 * g1 * g2).total;
}

SPH_EXPORT int sph_points_to_voxel(const float *points, int n, int nfeat, int system, float lo0, float lo1, float lo2,
                                   float vs0, float vs1, float vs2, int g0, int g1, int g2, int max_points,
                                   int max_voxels, int append_mode, float *voxels, float *mask, int32_t *coors,
                                   int32_t *num_points, int32_t *voxel_num, const long long *cell_in,
                                   long long *cell_out, void *workspace, size_t workspace_bytes, void *stream)
{
    SPH_REQUIRE(n >= 0 && nfeat >= 4 && max_points > 0 && max_voxels > 0 && g0 > 0 && g1 > 0 && g2 > 0, SPH_ERR_ARG,
                "sph_points_to_voxel: bad sizes (points need x, y, z, intensity)");
    SPH_REQUIRE(system >= 0 && system < SYS_COUNT && append_mode >= 0 && append_mode <= 2, SPH_ERR_ARG,
                "sph_points_to_voxel: unknown coordinate system %d or append mode %d", system, append_mode);
    SPH_REQUIRE(vs0 != 0.f && vs1 != 0.f && vs2 != 0.f, SPH_ERR_ARG, "sph_points_to_voxel: empty range");
    SPH_REQUIRE(voxels && mask && coors && num_points && voxel_num && workspace && (n == 0 || points), SPH_ERR_ARG,
                "sph_points_to_voxel: null pointer");
    SPH_REQUIRE((uintptr_t)workspace % 256 == 0, SPH_ERR_ARG, "sph_points_to_voxel: workspace must be 256-byte aligned");
    VoxParams q;
    q.system = system; q.nfeat = nfeat; q.append_mode = append_mode; q.max_points = max_points; q.max_voxels = max_voxels;
    q.lo[0] = lo0; q.lo[1] = lo1; q.lo[2] = lo2; q.vs[0] = vs0; q.vs[1] = vs1; q.vs[2] = vs2;
    q.grid[0] = g0; q.grid[1] = g1; q.grid[2] = g2;
    q.cells = (unsigned long long)g0 * g1 * g2;
    const VoxLayout l = vox_layout(n, q.cells);
    SPH_REQUIRE(l.total != 0, SPH_ERR_LAUNCH, "sph_points_to_voxel: temporary storage query failed");
    SPH_REQUIRE(workspace_bytes >= l.total, SPH_ERR_ARG, "sph_points_to_voxel: workspace of %zu bytes, %zu needed",
                workspace_bytes, l.total);
    hipStream_t st = (hipStream_t)stream;
    char *ws = (char *)workspace;
    uint64_t *keys_in = (uint64_t *)(ws + l.keys_in), *keys_out = (uint64_t *)(ws + l.keys_out);
    int32_t *vals_in = (int32_t *)(ws + l.vals_in), *vals_out = (int32_t *)(ws + l.vals_out);
    int32_t *mark = (int32_t *)(ws + l.mark), *vid = (int32_t *)(ws + l.vid);
    int32_t *start_in = (int32_t *)(ws + l.start_in), *start = (int32_t *)(ws + l.start), *stop = (int32_t *)(ws + l.stop);

    const int width = append_mode == 1 ? nfeat + 3 : nfeat;
    const long nv = (long)max_voxels * max_points;
    hipLaunchKernelGGL(vox_fill_kernel, dim3(blocks(nv * width)), dim3(256), 0, st, (int32_t *)voxels, nv * width, 0);
    hipLaunchKernelGGL(vox_fill_kernel, dim3(blocks(nv)), dim3(256), 0, st, (int32_t *)mask, nv, 0);
    hipLaunchKernelGGL(vox_fill_kernel, dim3(blocks(3L * max_voxels)), dim3(256), 0, st, coors, 3L * max_voxels, 0);
    hipLaunchKernelGGL(vox_fill_kernel, dim3(blocks(max_voxels)), dim3(256), 0, st, num_points, (long)max_voxels, 0);
    hipLaunchKernelGGL(vox_fill_kernel, dim3(1), dim3(256), 0, st, voxel_num, 1L, 0);
    int rc = sph_check_launch("sph_points_to_voxel(fill)");
    if (rc || n == 0) return rc;
    hipLaunchKernelGGL(vox_fill_kernel, dim3(blocks(n)), dim3(256), 0, st, mark, (long)n, 0);
    hipLaunchKernelGGL(vox_fill_kernel, dim3(1), dim3(256), 0, st, stop, 1L, n);
    hipLaunchKernelGGL(vox_cell_kernel, dim3(blocks(n)), dim3(256), 0, st, points, n, q, cell_in, keys_in, vals_in, cell_out);
    rc = sph_check_launch("sph_points_to_voxel(cells)");
    if (rc) return rc;
    size_t tb = l.temp_bytes;
    hipError_t e = rocprim::radix_sort_pairs(ws + l.temp, tb, (const uint64_t *)keys_in, keys_out, (const int32_t *)vals_in,
                                             vals_out, (size_t)n, 0, bits_for(q.cells), st);
    if (e == hipSuccess) {
        hipLaunchKernelGGL(vox_head_kernel, dim3(blocks(n)), dim3(256), 0, st, (const uint64_t *)keys_out,
                           (const int32_t *)vals_out, n, (uint64_t)q.cells, mark, start_in);
        e = sph_scan::launch<sph_scan::Plus, false>(mark, vid, n, ws + l.temp, 0, st);
    }
    if (e == hipSuccess) e = sph_scan::launch<sph_scan::Max, true>(start_in, start, n, ws + l.temp, 0, st);
    if (e != hipSuccess) {
        sph_set_error("sph_points_to_voxel: sort/scan: %s", hipGetErrorString(e));
        return SPH_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(vox_stop_kernel, dim3(blocks(n)), dim3(256), 0, st, (const int32_t *)mark, (const int32_t *)vid, n,
                       max_voxels, stop, voxel_num);
    hipLaunchKernelGGL(vox_write_kernel, dim3(blocks(n)), dim3(256), 0, st, points, n, q, (const uint64_t *)keys_out,
                       (const int32_t *)vals_out, (const int32_t *)start, (const int32_t *)vid, (const int32_t *)stop,
                       voxels, mask, coors, num_points);
    return sph_check_launch("sph_points_to_voxel");
}
