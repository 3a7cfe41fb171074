// Point cloud -> voxels with up to max_points points each, replacing the sequential CPU loop of
// points_to_voxel_3d (include/point2voxel.h:412-512, called from sphconv/utils/voxelize.py:126-214)
// and the coordinate transforms of sphconv/utils/coord_transform.py:8-118.
//
// The reference walks the points in order: a point outside the grid is skipped; a point in a
// new cell opens the next voxel, unless max_voxels are open already -- then the whole loop
// stops; a voxel keeps its first max_points points.  The same result without the sequential
// loop:
//   1. vox_clear_kernel    zeroes the outputs and resets the workspace (one launch)
//   2. vox_insert_kernel   system coordinates (float32, operation by operation as numpy does it) and
//                          the cell of every point; a point inside the grid enters its cell into a hash
//                          table (open addressing, at most half full), counts itself there and offers
//                          its index as the cell's first point (atomic minimum)
//   3. vox_mark_kernel     marks the points that open a cell, in point order, behind the cells' counts
//   4. one exclusive sum   over [counts of the table's slots | marks of the points]: a slot's segment
//                          of the point list, and (minus the points inside) every mark's voxel number
//   5. vox_scatter_kernel  writes every point into its cell's segment (in any order); the point
//                          that would open voxel number max_voxels is where the reference's loop
//                          stops: every later point is dropped
//   6. vox_write_kernel    a point's place in its voxel = the number of smaller point indices in its
//                          segment (counted until max_points are found: such a point is dropped);
//                          segments of more than 256 points are walked by the whole wave, 64 entries at a time
// Which slot a cell gets, and the order inside a segment, depend on the order the atomics land in;
// no output does.  Nothing is allocated; table, segments and the scan's state live in the caller's workspace.
#include "common.h"

#include <cstring>

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

// cell of point i as the table's key, or `cells` for a point that is skipped
__device__ __forceinline__ uint64_t point_cell(const float *points, int i, const VoxParams &q, const long long *cell_in)
{
    if (cell_in) {
        const long long c = cell_in[i];
        return c >= 0 && (unsigned long long)c < q.cells ? (uint64_t)c : (uint64_t)q.cells;
    }
    float c[3];
    int bin[3];
    system_coords(points + (long)i * q.nfeat, q.system, c);
    // the reference indexes its map [c2 bin][c1 bin][c0 bin]
    if (cell_of(c, q, bin)) return ((uint64_t)bin[2] * q.grid[1] + bin[1]) * q.grid[0] + bin[0];
    return q.cells;
}

constexpr uint64_t kEmptyKey = ~0ull;
constexpr int kFills = 10;
constexpr int kFillBlocks = 128;  // workgroups per range
constexpr int kLongSegment = 256; // longer segments are walked by the wave together

// up to kFills ranges of 32-bit words, each set to its value: blockIdx.y = range
struct VoxFills {
    int32_t *p[kFills];
    long words[kFills];
    int32_t value[kFills];
};

__global__ __launch_bounds__(256) void vox_clear_kernel(VoxFills f)
{
    int32_t *p = f.p[blockIdx.y];
    const long n = f.words[blockIdx.y];
    const int32_t v = f.value[blockIdx.y];
    const long t = (long)blockIdx.x * 256 + threadIdx.x, step = (long)gridDim.x * 256;
    if (((uintptr_t)p & 15) == 0) {
        const int4 v4 = make_int4(v, v, v, v);
        for (long i = t; i < n / 4; i += step) ((int4 *)p)[i] = v4;
        if (t < (n & 3)) p[(n & ~3L) + t] = v;
    } else {
        for (long i = t; i < n; i += step) p[i] = v;
    }
}

// tbits = log2 of the table's slots
__global__ __launch_bounds__(256) void vox_insert_kernel(const float *points, int n, VoxParams q, const long long *cell_in,
                                                         int tbits, unsigned long long *keys, int32_t *first,
                                                         int32_t *count, int32_t *slot_of, long long *cell_out)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const uint64_t key = point_cell(points, i, q, cell_in);
    if (cell_out) cell_out[i] = key == q.cells ? -1 : (long long)key;
    if (key == q.cells) {
        slot_of[i] = -1;
        return;
    }
    const unsigned mask = (1u << tbits) - 1u;
    unsigned slot = (unsigned)((key * 0x9E3779B97F4A7C15ull) >> (64 - tbits));
    // the table has at least twice as many slots as there are points: a free one is always met
    for (;;) {
        const unsigned long long seen = atomicCAS(&keys[slot], (unsigned long long)kEmptyKey, (unsigned long long)key);
        if (seen == kEmptyKey || seen == key) break;
        slot = (slot + 1) & mask;
    }
    atomicAdd(&count[slot], 1);
    atomicMin(&first[slot], i);
    slot_of[i] = (int32_t)slot;
}

__global__ __launch_bounds__(256) void vox_mark_kernel(const int32_t *slot_of, const int32_t *first, int n, int32_t *mark)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int s = slot_of[i];
    mark[i] = s >= 0 && first[s] == i;
}

// sum[0..T): first place of every slot's segment; sum[T + i] - sum[T]: marks in front of point i; *total: all of it
__global__ __launch_bounds__(256) void vox_scatter_kernel(const int32_t *slot_of, const int32_t *sum, const int32_t *mark,
                                                          const int32_t *total, int n, long T, int max_voxels,
                                                          int32_t *count, int32_t *seg, int32_t *stop, int32_t *voxel_num)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int s = slot_of[i];
    if (s >= 0) seg[sum[s] + atomicSub(&count[s], 1) - 1] = i;
    const int inside = sum[T];
    if (mark[i] && sum[T + i] - inside == max_voxels) *stop = i; // exactly one such point, if any
    if (i == 0) *voxel_num = min(*total - inside, max_voxels);
}

__global__ __launch_bounds__(256) void vox_write_kernel(const float *points, int n, VoxParams q, const unsigned long long *keys,
                                                        const int32_t *first, const int32_t *slot_of, const int32_t *sum,
                                                        const int32_t *seg, long T, const int32_t *stop, float *voxels,
                                                        float *mask, int32_t *coors, int32_t *num_points)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    const int lane = threadIdx.x & 63;
    const int s = i < n ? slot_of[i] : -1;
    int vid = 0, h = 0, s0 = 0, s1 = 0;
    bool live = s >= 0;
    if (live) {
        h = first[s];
        vid = sum[T + h] - sum[T];
        live = vid < q.max_voxels && i < *stop;
        s0 = sum[s];
        s1 = sum[s + 1]; // slot T - 1 ends where the marks begin: sum[T] = points inside
    }
    // place among the cell's points = smaller indices in the segment
    int rank = 0;
    const bool wide = live && s1 - s0 > kLongSegment;
    if (live && !wide)
        for (int p = s0; p < s1 && rank < q.max_points; p++) rank += seg[p] < i;
    for (unsigned long long todo = __ballot(wide); todo; todo &= todo - 1) {
        const int l = __ffsll((long long)todo) - 1;
        const int ti = __shfl(i, l, 64), t1 = __shfl(s1, l, 64);
        int r = 0;
        for (int p = __shfl(s0, l, 64); p < t1 && r < q.max_points; p += 64)
            r += __popcll(__ballot(p + lane < t1 && seg[p + lane] < ti));
        if (lane == l) rank = r;
    }
    if (!live || rank >= q.max_points) return;
    if (i == h) {
        const uint64_t key = keys[s];
        const uint64_t t = key / q.grid[0];
        coors[3 * (long)vid] = (int)(t / q.grid[1]);       // c2 bin
        coors[3 * (long)vid + 1] = (int)(t % q.grid[1]);   // c1 bin
        coors[3 * (long)vid + 2] = (int)(key % q.grid[0]); // c0 bin
    }
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
    int tbits;
    long T; // slots of the table: a power of two, at least twice the points
    size_t keys, first, count, sum, slot_of, seg, stop, state, state_words, total;
};

inline size_t al256(size_t x) { return (x + 255) & ~(size_t)255; }

inline VoxLayout vox_layout(int n)
{
    VoxLayout l;
    const size_t nn = (size_t)(n > 0 ? n : 1);
    l.tbits = 10;
    while ((1ull << l.tbits) < 2 * nn) l.tbits++;
    l.T = 1L << l.tbits;
    size_t o = 0;
    l.keys = o; o += al256((size_t)l.T * 8);
    l.first = o; o += al256((size_t)l.T * 4);
    l.count = o; o += al256(((size_t)l.T + nn) * 4); // the slots' counts, then the points' marks
    l.sum = o; o += al256(((size_t)l.T + nn) * 4);
    l.slot_of = o; o += al256(nn * 4);
    l.seg = o; o += al256(nn * 4);
    l.stop = o; o += 256;                            // stop, total
    l.state = o;
    l.state_words = (size_t)sph_scan::state_ints(l.T + (long)nn);
    o += al256(sph_scan::state_bytes(l.T + (long)nn));
    l.total = o;
    return l;
}

inline unsigned blocks(long n) { return (unsigned)((n + 255) / 256); }

} // namespace

SPH_EXPORT size_t sph_points_to_voxel_workspace(int n, int g0, int g1, int g2)
{
    if (n < 0 || n > (1 << 29) || g0 <= 0 || g1 <= 0 || g2 <= 0) return 0;
    return vox_layout(n).total;
}

SPH_EXPORT int sph_points_to_voxel(const float *points, int n, int nfeat, int system, float lo0, float lo1, float lo2,
                                   float vs0, float vs1, float vs2, int g0, int g1, int g2, int max_points,
                                   int max_voxels, int append_mode, float *voxels, float *mask, int32_t *coors,
                                   int32_t *num_points, int32_t *voxel_num, const long long *cell_in,
                                   long long *cell_out, void *workspace, size_t workspace_bytes, void *stream)
{
    SPH_REQUIRE(n >= 0 && n <= (1 << 29) && nfeat >= 4 && max_points > 0 && max_voxels > 0 && g0 > 0 && g1 > 0 && g2 > 0,
                SPH_ERR_ARG, "sph_points_to_voxel: bad sizes (points need x, y, z, intensity; at most 2^29 points)");
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
    SPH_REQUIRE(q.cells / g0 / g1 == (unsigned long long)g2 && q.cells < (1ull << 63), SPH_ERR_ARG,
                "sph_points_to_voxel: grid %d x %d x %d has too many cells", g0, g1, g2);
    const VoxLayout l = vox_layout(n);
    SPH_REQUIRE(workspace_bytes >= l.total, SPH_ERR_ARG, "sph_points_to_voxel: workspace of %zu bytes, %zu needed",
                workspace_bytes, l.total);
    hipStream_t st = (hipStream_t)stream;
    char *ws = (char *)workspace;
    unsigned long long *keys = (unsigned long long *)(ws + l.keys);
    int32_t *first = (int32_t *)(ws + l.first), *count = (int32_t *)(ws + l.count), *sum = (int32_t *)(ws + l.sum);
    int32_t *slot_of = (int32_t *)(ws + l.slot_of), *seg = (int32_t *)(ws + l.seg), *stop = (int32_t *)(ws + l.stop);
    int32_t *total = stop + 1, *mark = count + l.T;

    const int width = append_mode == 1 ? nfeat + 3 : nfeat;
    const long nv = (long)max_voxels * max_points;
    VoxFills f;
    int nf = 0;
    auto fill = [&](void *p, long words, int32_t v) {
        f.p[nf] = (int32_t *)p; f.words[nf] = words; f.value[nf] = v;
        nf++;
    };
    fill(voxels, nv * width, 0);
    fill(mask, nv, 0);
    fill(coors, 3L * max_voxels, 0);
    fill(num_points, (long)max_voxels, 0);
    fill(voxel_num, 1L, 0);
    if (n > 0) {
        fill(keys, 2 * l.T, -1);
        fill(first, l.T, INT_MAX);
        fill(count, l.T, 0);
        fill(stop, 1L, n);
        fill(ws + l.state, (long)l.state_words, 0);
    }
    hipLaunchKernelGGL(vox_clear_kernel, dim3(kFillBlocks, nf), dim3(256), 0, st, f);
    int rc = sph_check_launch("sph_points_to_voxel(clear)");
    if (rc || n == 0) return rc;
    hipLaunchKernelGGL(vox_insert_kernel, dim3(blocks(n)), dim3(256), 0, st, points, n, q, cell_in, l.tbits, keys, first,
                       count, slot_of, cell_out);
    hipLaunchKernelGGL(vox_mark_kernel, dim3(blocks(n)), dim3(256), 0, st, (const int32_t *)slot_of, (const int32_t *)first,
                       n, mark);
    rc = sph_check_launch("sph_points_to_voxel(cells)");
    if (rc) return rc;
    const hipError_t e = sph_scan::launch<sph_scan::Plus, false>(count, sum, l.T + n, ws + l.state, 0, st, total, false);
    if (e != hipSuccess) {
        sph_set_error("sph_points_to_voxel: scan: %s", hipGetErrorString(e));
        return SPH_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(vox_scatter_kernel, dim3(blocks(n)), dim3(256), 0, st, (const int32_t *)slot_of, (const int32_t *)sum,
                       (const int32_t *)mark, (const int32_t *)total, n, l.T, max_voxels, count, seg, stop, voxel_num);
    hipLaunchKernelGGL(vox_write_kernel, dim3(blocks(n)), dim3(256), 0, st, points, n, q, (const unsigned long long *)keys,
                       (const int32_t *)first, (const int32_t *)slot_of, (const int32_t *)sum, (const int32_t *)seg, l.T,
                       (const int32_t *)stop, voxels, mask, coors, num_points);
    return sph_check_launch("sph_points_to_voxel");
}
