// COO -> per-column compressed layout (sph_init_tensor), replacing the dense
// occupancy grid + per-fiber atomics of init_tensor (src/sphconv/tensor.cu:78-127,
// fillGridKernel 21-36, reorderFeatureKernel 39-76): rows are sorted by their linear
// cell index (b, s0, s1, s2), which orders fibers by column and, inside a fiber, by
// ascending S2 -- one legal, deterministic serialisation of the reference's output
// (its order inside a fiber is the order in which atomics happen to land).
//
// No sort: a row's place is the start of its column (a scan of per-column counts) plus its rank
// inside the column, and the rank needs no order of arrival.
// Shallow grids (S2 <= 128, the usual case):
//   1. coo_count_kernel    slot = atomicAdd(count[column]) per row (arrival order, only used
//                          to park the row inside its column's segment)
//   2. sum-scan (scan.h)   counts -> z_ptr (inclusive)
//   3. coo_scatter_kernel  (s2, row) -> segment position start + slot
//   4. coo_rank_kernel     every row counts the entries of its column with a smaller s2:
//                          that rank is its final position, whatever the arrival order was
// Deep grids (S2 > 128), where a full column would make that walk long: one bit per cell instead,
//   1. coo_mark_kernel     count[column]++ and the cell's bit set in the column's bitmap (a bit
//                          that was set already is a duplicate coordinate: status[1])
//   2. sum-scan            counts -> z_ptr
//   3. coo_place_kernel    rank = set bits of the column below s2 (popcounts of up to S2/64 words)
// (the reference keeps four bytes per cell for the same purpose, tensor.cu:21-36; a bitmap of more
// than 1 GiB -- 8.6e9 cells -- falls back to the walk, which needs memory by rows only).
// Four to six launches, none from a library.
// The feature rows are then moved with sph_permute_rows.  No memory is allocated:
// segments, bitmaps and the scan's state live in the caller's workspace.
#include "common.h"

#include <cstring>

#include "scan.h"

namespace {

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

constexpr int kRankMaxDepth = 128; // S2 up to which a row's rank is found by walking its column's segment

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

constexpr size_t kBitmapMaxBytes = (size_t)1 << 30; // deep grids whose bitmap would be larger are ranked by the walk

struct BitLayout {
    size_t bits, bits_bytes, temp, temp_bytes, total;
    int words; // 64-bit words per column
};

inline BitLayout bit_layout(int ncol, int S2)
{
    BitLayout l;
    l.words = (S2 + 63) / 64;
    l.bits = 0;
    l.bits_bytes = (size_t)ncol * l.words * sizeof(unsigned long long);
    l.temp = align256(l.bits_bytes);
    l.temp_bytes = sum_scan_bytes(ncol);
    l.total = l.temp_bytes ? l.temp + align256(l.temp_bytes) : 0;
    return l;
}

inline bool by_bitmap(int ncol, int S2)
{
    return S2 > kRankMaxDepth && (double)ncol * ((S2 + 63) / 64) * 8.0 <= (double)kBitmapMaxBytes;
}

__global__ void fill_zero_kernel(int32_t *p, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

// Deep grids, step 1: the row is counted in its column and marks its cell.
__global__ void coo_mark_kernel(const int32_t *idx, int n, int B, int S0, int S1, int S2, int words, int32_t *counts,
                                unsigned long long *bits, int32_t *status)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int4 c = ((const int4 *)idx)[i]; // (b, s0, s1, s2)
    const bool ok = (unsigned)c.x < (unsigned)B && (unsigned)c.y < (unsigned)S0 && (unsigned)c.z < (unsigned)S1 &&
                    (unsigned)c.w < (unsigned)S2;
    if (!ok) {
        atomicAdd(&status[0], 1);
        return;
    }
    const int col = (c.x * S0 + c.y) * S1 + c.z;
    atomicAdd(&counts[col], 1);
    const unsigned long long bit = 1ull << (c.w & 63);
    const unsigned long long old = atomicOr(&bits[(size_t)col * words + (c.w >> 6)], bit);
    if (old & bit) atomicAdd(&status[1], 1);
}

// Deep grids, step 3: place = start of the column + number of its cells below the row's.
__global__ void coo_place_kernel(const int32_t *idx, int n, int B, int S0, int S1, int S2, int words, const int32_t *z_ptr,
                                 const unsigned long long *bits, int32_t *z_idx, int32_t *permutation)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int4 c = ((const int4 *)idx)[i];
    const bool ok = (unsigned)c.x < (unsigned)B && (unsigned)c.y < (unsigned)S0 && (unsigned)c.z < (unsigned)S1 &&
                    (unsigned)c.w < (unsigned)S2;
    if (!ok) return;
    const int col = (c.x * S0 + c.y) * S1 + c.z;
    const unsigned long long *cb = bits + (size_t)col * words;
    const int wz = c.w >> 6;
    int rank = __popcll(cb[wz] & ((1ull << (c.w & 63)) - 1ull));
    for (int w = 0; w < wz; w++) rank += __popcll(cb[w]);
    const int pos = (col ? z_ptr[col - 1] : 0) + rank;
    if ((unsigned)pos < (unsigned)n) {
        z_idx[pos] = c.w;
        permutation[i] = pos;
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
    if (by_bitmap(B * S0 * S1, S2)) return bit_layout(B * S0 * S1, S2).total;
    return rank_layout(n, B * S0 * S1).total;
}

// count, scan, scatter, rank by a walk of the column's segment (shallow grids; deep ones whose bitmap would not fit)
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
    const int ncol = B * S0 * S1;
    if (!by_bitmap(ncol, S2))
        return init_tensor_by_rank(indices, n, B, S0, S1, S2, z_idx, z_ptr, permutation, status, workspace, workspace_bytes,
                                   (hipStream_t)stream);
    const BitLayout l = bit_layout(ncol, S2);
    SPH_REQUIRE(l.total != 0, SPH_ERR_LAUNCH, "sph_init_tensor: temporary storage query failed");
    SPH_REQUIRE(workspace_bytes >= l.total, SPH_ERR_ARG, "sph_init_tensor: workspace of %zu bytes, %zu needed",
                workspace_bytes, l.total);
    hipStream_t st = (hipStream_t)stream;
    char *ws = (char *)workspace;
    unsigned long long *bits = (unsigned long long *)(ws + l.bits);
    const int bit_ints = (int)(l.bits_bytes / sizeof(int32_t)); // at most 2^28
    hipLaunchKernelGGL(fill_zero_kernel, dim3((ncol + 255) / 256), dim3(256), 0, st, z_ptr, ncol);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(64), 0, st, status, 2);
    hipLaunchKernelGGL(fill_zero_kernel, dim3((bit_ints + 255) / 256), dim3(256), 0, st, (int32_t *)bits, bit_ints);
    int rc = sph_check_launch("sph_init_tensor(fill)");
    if (rc || n == 0) return rc;
    const dim3 grid((n + 255) / 256), block(256);
    hipLaunchKernelGGL(coo_mark_kernel, grid, block, 0, st, indices, n, B, S0, S1, S2, l.words, z_ptr, bits, status);
    rc = sph_check_launch("sph_init_tensor(mark)");
    if (rc) return rc;
    hipError_t e = sph_scan::launch<sph_scan::Plus, true>(z_ptr, z_ptr, ncol, ws + l.temp, 0, st);
    if (e != hipSuccess) {
        sph_set_error("sph_init_tensor: scan: %s", hipGetErrorString(e));
        return SPH_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(coo_place_kernel, grid, block, 0, st, indices, n, B, S0, S1, S2, l.words, (const int32_t *)z_ptr,
                       (const unsigned long long *)bits, z_idx, permutation);
    rc = sph_check_launch("sph_init_tensor(place)");
    if (rc) return rc;
    return SPH_OK;
}
