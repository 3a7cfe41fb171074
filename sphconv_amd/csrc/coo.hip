// COO -> per-column compressed layout (sph_init_tensor), replacing the dense
// occupancy grid + per-fiber atomics of init_tensor (src/sphconv/tensor.cu:78-127,
// fillGridKernel 21-36, reorderFeatureKernel 39-76): rows are sorted by their linear
// cell index (b, s0, s1, s2), which orders fibers by column and, inside a fiber, by
// ascending S2 -- one legal, deterministic serialisation of the reference's output
// (its order inside a fiber is the order in which atomics happen to land).
//
//   1. coo_key_kernel      key = ((b*S0 + s0)*S1 + s1)*S2 + s2, value = row; coordinates
//                          outside the grid are counted in status[0]
//   2. rocprim radix sort  (key, row) pairs, only the bits the grid needs
//   3. coo_finish_kernel   z_idx = key % S2; permutation[row] = sorted position; equal
//                          neighbours counted in status[1]; the last row of a column
//                          writes its position+1 into z_ptr[column]
//   4. rocprim max-scan    z_ptr is an inclusive count, so empty columns inherit the
//                          value of the last non-empty one before them
// That is the path for deep grids (S2 > 128).  For S2 <= 128, the usual case, no sort is
// needed: fibers are short, so
//   1. coo_count_kernel    slot = atomicAdd(count[column]) per row (arrival order, only used
//                          to park the row inside its column's segment)
//   2. rocprim sum-scan    counts -> z_ptr (inclusive)
//   3. coo_scatter_kernel  (s2, row) -> segment position start + slot
//   4. coo_rank_kernel     every row counts the entries of its column with a smaller s2:
//                          that rank is its final position, whatever the arrival order was
// six launches instead of the eighteen of the merge-sort path rocPRIM takes at 100k keys.
// The feature rows are then moved with sph_permute_rows.  No memory is allocated:
// keys, values and the library scratch live in the caller's workspace.
#include "common.h"

#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

#include "scan.h"

namespace {

struct CooLayout {
    size_t keys_in, keys_out, vals_in, vals_out, temp, temp_bytes, total;
};

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

inline int key_bits(long cells)
{
    int b = 1;
    while (b < 63 && (1L << b) < cells) b++;
    return b;
}

// temporary storage of the sort of n pairs (what rocPRIM asks for) and of the scan of ncol ints, which share
// one area; 0 on error
inline size_t library_temp_bytes(int n, int ncol, long cells)
{
    size_t sort_bytes = 0;
    hipError_t e = rocprim::radix_sort_pairs(nullptr, sort_bytes, (const uint64_t *)nullptr, (uint64_t *)nullptr,
                                             (const int32_t *)nullptr, (int32_t *)nullptr, (size_t)(n > 0 ? n : 1), 0,
                                             key_bits(cells), (hipStream_t)0);
    if (e != hipSuccess) return 0;
    const size_t scan_bytes = sph_scan::state_bytes(ncol);
    return (sort_bytes > scan_bytes ? sort_bytes : scan_bytes) + 256;
}

constexpr int kRankMaxDepth = 128; // S2 up to which rows are ranked inside their column instead of sorted

inline size_t sum_scan_bytes(int ncol) { return sph_scan::state_bytes(ncol); }

struct RankLayout {
    size_t slot, seg_z, seg_row, temp, temp_bytes, total;
};

inline RankLayout rank_layout(int n, int ncol)
{
    RankLayout l;
    const size_t nn = (size_t)(n > 0 ? n : 1);
    size_t o = 0;
    l.slot = o; o += align256(nn * 4);
    l.seg_z = o; o += align256(nn * 4);
    l.seg_row = o; o += align256(nn * 4);
    l.temp = o;
    l.temp_bytes = sum_scan_bytes(ncol);
    l.total = l.temp_bytes ? o + align256(l.temp_bytes) : 0;
    return l;
}

inline CooLayout layout(int n, int ncol, long cells)
{
    CooLayout l;
    const size_t nn = (size_t)(n > 0 ? n : 1);
    size_t o = 0;
    l.keys_in = o; o += align256(nn * 8);
    l.keys_out = o; o += align256(nn * 8);
    l.vals_in = o; o += align256(nn * 4);
    l.vals_out = o; o += align256(nn * 4);
    l.temp = o;
    l.temp_bytes = library_temp_bytes(n, ncol, cells);
    l.total = l.temp_bytes ? o + align256(l.temp_bytes) : 0;
    return l;
}

__global__ void coo_key_kernel(const int32_t *idx, int n, int B, int S0, int S1, int S2, uint64_t *keys, int32_t *vals,
                               int32_t *status)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int4 c = ((const int4 *)idx)[i]; // (b, s0, s1, s2)
    const bool ok = (unsigned)c.x < (unsigned)B && (unsigned)c.y < (unsigned)S0 && (unsigned)c.z < (unsigned)S1 &&
                    (unsigned)c.w < (unsigned)S2;
    if (!ok) atomicAdd(&status[0], 1);
    // rows outside the grid sort to the end (largest key of the sorted bit range)
    const uint64_t cells = (uint64_t)B * S0 * S1 * S2;
    keys[i] = ok ? (((uint64_t)c.x * S0 + c.y) * S1 + c.z) * S2 + c.w : cells - 1;
    vals[i] = i;
}

__global__ void fill_zero_kernel(int32_t *p, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

__global__ void coo_finish_kernel(const uint64_t *keys, const int32_t *vals, int n, int S2, int ncol, int32_t *z_idx,
                                  int32_t *z_ptr, int32_t *permutation, int32_t *status)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const uint64_t k = keys[i];
    const uint64_t col = k / (uint64_t)S2;
    z_idx[i] = (int32_t)(k - col * (uint64_t)S2);
    const int row = vals[i];
    if ((unsigned)row < (unsigned)n) permutation[row] = i;
    if (i + 1 < n) {
        const uint64_t kn = keys[i + 1];
        if (kn == k) atomicAdd(&status[1], 1);
        if (kn / (uint64_t)S2 != col && col < (uint64_t)ncol) z_ptr[col] = i + 1;
    } else if (col < (uint64_t)ncol) {
        z_ptr[col] = n;
    }
}

__global__ void coo_count_kernel(const int32_t *idx, int n, int B, int S0, int S1, int S2, int32_t *counts, int32_t *slot,
                                 int32_t *status)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int4 c = ((const int4 *)idx)[i]; // (b, s0, s1, s2)
    const bool ok = (unsigned)c.x < (unsigned)B && (unsigned)c.y < (unsigned)S0 && (unsigned)c.z < (unsigned)S1 &&
                    (unsigned)c.w < (unsigned)S2;
    int sl = -1;
    if (ok) sl = atomicAdd(&counts[(c.x * S0 + c.y) * S1 + c.z], 1);
    else atomicAdd(&status[0], 1);
    slot[i] = sl;
}

__global__ void coo_scatter_kernel(const int32_t *idx, int n, int S0, int S1, const int32_t *z_ptr, const int32_t *slot,
                                   int32_t *seg_z, int32_t *seg_row)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int sl = slot[i];
    if (sl < 0) return;
    const int4 c = ((const int4 *)idx)[i];
    const int col = (c.x * S0 + c.y) * S1 + c.z;
    const int pos = (col ? z_ptr[col - 1] : 0) + sl;
    if ((unsigned)pos >= (unsigned)n) return;
    seg_z[pos] = c.w;
    seg_row[pos] = i;
}

__global__ void coo_rank_kernel(const int32_t *idx, int n, int S0, int S1, int S2, const int32_t *z_ptr, const int32_t *slot,
                                const int32_t *seg_z, const int32_t *seg_row, int32_t *z_idx, int32_t *permutation,
                                int32_t *status)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    if (slot[i] < 0) return;
    const int4 c = ((const int4 *)idx)[i];
    const int col = (c.x * S0 + c.y) * S1 + c.z;
    const int start = col ? z_ptr[col - 1] : 0;
    int end = min(z_ptr[col], n);
    int rank = 0, dup = 0;
    if (end - start > S2) { // more rows than bins: duplicates for sure; keep the walk bounded
        dup = 1;
        end = start + S2;
    }
    for (int j = start; j < end; j++) {
        const int z = seg_z[j];
        rank += z < c.w;
        dup += (z == c.w && seg_row[j] < i);
    }
    if (dup) atomicAdd(&status[1], dup);
    const int pos = start + rank;
    if ((unsigned)pos < (unsigned)n) {
        z_idx[pos] = c.w;
        permutation[i] = pos;
    }
}

} // namespace

SPH_EXPORT size_t sph_init_tensor_workspace(int n, int B, int S0, int S1, int S2)
{
    if (n < 0 || B <= 0 || S0 <= 0 || S1 <= 0 || S2 <= 0) return 0;
    if ((double)B * S0 * S1 >= 2147483648.0) return 0;
    if (S2 <= kRankMaxDepth) return rank_layout(n, B * S0 * S1).total;
    return layout(n, B * S0 * S1, (long)B * S0 * S1 * S2).total;
}

// S2 <= kRankMaxDepth: count, scan, scatter, rank
static int init_tensor_by_rank(const int32_t *indices, int n, int B, int S0, int S1, int S2, int32_t *z_idx, int32_t *z_ptr,
                               int32_t *permutation, int32_t *status, void *workspace, size_t workspace_bytes,
                               hipStream_t st)
{
    const int ncol = B * S0 * S1;
    const RankLayout l = rank_layout(n, ncol);
    SPH_REQUIRE(l.total != 0, SPH_ERR_LAUNCH, "sph_init_tensor: temporary storage query failed");
    SPH_REQUIRE(workspace_bytes >= l.total, SPH_ERR_ARG, "sph_init_tensor: workspace of %zu bytes, %zu needed",
                workspace_bytes, l.total);
    char *ws = (char *)workspace;
    int32_t *slot = (int32_t *)(ws + l.slot), *seg_z = (int32_t *)(ws + l.seg_z), *seg_row = (int32_t *)(ws + l.seg_row);
    hipLaunchKernelGGL(fill_zero_kernel, dim3((ncol + 255) / 256), dim3(256), 0, st, z_ptr, ncol);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(64), 0, st, status, 2);
    int rc = sph_check_launch("sph_init_tensor(fill)");
    if (rc || n == 0) return rc;
    const dim3 grid((n + 255) / 256), block(256);
    hipLaunchKernelGGL(coo_count_kernel, grid, block, 0, st, indices, n, B, S0, S1, S2, z_ptr, slot, status);
    rc = sph_check_launch("sph_init_tensor(count)");
    if (rc) return rc;
    hipError_t e = sph_scan::launch<sph_scan::Plus, true>(z_ptr, z_ptr, ncol, ws + l.temp, 0, st);
    if (e != hipSuccess) {
        sph_set_error("sph_init_tensor: scan: %s", hipGetErrorString(e));
        return SPH_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(coo_scatter_kernel, grid, block, 0, st, indices, n, S0, S1, (const int32_t *)z_ptr,
                       (const int32_t *)slot, seg_z, seg_row);
    hipLaunchKernelGGL(coo_rank_kernel, grid, block, 0, st, indices, n, S0, S1, S2, (const int32_t *)z_ptr, (const int32_t *)slot,
                       (const int32_t *)seg_z, (const int32_t *)seg_row, z_idx, permutation, status);
    return sph_check_launch("sph_init_tensor(rank)");
}

SPH_EXPORT int sph_init_tensor(const int32_t *indices, int n, int B, int S0, int S1, int S2, int32_t *z_idx,
                               int32_t *z_ptr, int32_t *permutation, int32_t *status, void *workspace,
                               size_t workspace_bytes, void *stream)
{
    SPH_REQUIRE(n >= 0 && B > 0 && S0 > 0 && S1 > 0 && S2 > 0, SPH_ERR_ARG, "sph_init_tensor: bad sizes");
    SPH_REQUIRE((double)B * S0 * S1 < 2147483648.0, SPH_ERR_UNSUPPORTED, "sph_init_tensor: more than 2^31 columns");
    SPH_REQUIRE(z_ptr && status && workspace && (n == 0 || (indices && z_idx && permutation)), SPH_ERR_ARG,
                "sph_init_tensor: null pointer");
    SPH_REQUIRE((uintptr_t)indices % 16 == 0 && (uintptr_t)workspace % 256 == 0, SPH_ERR_ARG,
                "sph_init_tensor: indices must be 16-byte aligned, the workspace 256-byte aligned");
    if (S2 <= kRankMaxDepth)
        return init_tensor_by_rank(indices, n, B, S0, S1, S2, z_idx, z_ptr, permutation, status, workspace, workspace_bytes,
                                   (hipStream_t)stream);
    const int ncol = B * S0 * S1;
    const long cells = (long)ncol * S2;
    const CooLayout l = layout(n, ncol, cells);
    SPH_REQUIRE(l.total != 0, SPH_ERR_LAUNCH, "sph_init_tensor: temporary storage query failed");
    SPH_REQUIRE(workspace_bytes >= l.total, SPH_ERR_ARG, "sph_init_tensor: workspace of %zu bytes, %zu needed",
                workspace_bytes, l.total);
    hipStream_t st = (hipStream_t)stream;
    char *ws = (char *)workspace;
    uint64_t *keys_in = (uint64_t *)(ws + l.keys_in), *keys_out = (uint64_t *)(ws + l.keys_out);
    int32_t *vals_in = (int32_t *)(ws + l.vals_in), *vals_out = (int32_t *)(ws + l.vals_out);

    hipLaunchKernelGGL(fill_zero_kernel, dim3((ncol + 255) / 256), dim3(256), 0, st, z_ptr, ncol);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(64), 0, st, status, 2);
    int rc = sph_check_launch("sph_init_tensor(fill)");
    if (rc || n == 0) return rc;
    hipLaunchKernelGGL(coo_key_kernel, dim3((n + 255) / 256), dim3(256), 0, st, indices, n, B, S0, S1, S2, keys_in,
                       vals_in, status);
    rc = sph_check_launch("sph_init_tensor(keys)");
    if (rc) return rc;
    size_t temp_bytes = l.temp_bytes;
    hipError_t e = rocprim::radix_sort_pairs(ws + l.temp, temp_bytes, (const uint64_t *)keys_in, keys_out,
                                             (const int32_t *)vals_in, vals_out, (size_t)n, 0, key_bits(cells), st);
    if (e != hipSuccess) {
        sph_set_error("sph_init_tensor: radix sort: %s", hipGetErrorString(e));
        return SPH_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(coo_finish_kernel, dim3((n + 255) / 256), dim3(256), 0, st, (const uint64_t *)keys_out,
                       (const int32_t *)vals_out, n, S2, ncol, z_idx, z_ptr, permutation, status);
    rc = sph_check_launch("sph_init_tensor(finish)");
    if (rc) return rc;
    e = sph_scan::launch<sph_scan::Max, true>(z_ptr, z_ptr, ncol, ws + l.temp, 0, st);
    if (e != hipSuccess) {
        sph_set_error("sph_init_tensor: scan: %s", hipGetErrorString(e));
        return SPH_ERR_LAUNCH;
    }
    return SPH_OK;
}
