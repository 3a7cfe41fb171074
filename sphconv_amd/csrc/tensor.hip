// Row permutation and densify kernels (HBM-bound copies), replacing
// reorderFeatureKernel / toDenseKernel and their backward twins
// (src/sphconv/tensor.cu:39-76, 130-145, 165-220).  A row is copied in units of
// the widest power-of-two granule (16/8/4/2/1 bytes) that divides the row size
// and the base addresses; consecutive lanes take consecutive granules of a row.
#include "common.h"

namespace {

template <int G> struct Gran;
template <> struct Gran<16> { typedef uint4 type; };
template <> struct Gran<8> { typedef uint2 type; };
template <> struct Gran<4> { typedef uint32_t type; };
template <> struct Gran<2> { typedef uint16_t type; };
template <> struct Gran<1> { typedef uint8_t type; };

inline int pick_granule(int row_bytes, const void *a, const void *b)
{
    uintptr_t m = (uintptr_t)row_bytes | (uintptr_t)a | (uintptr_t)b;
    for (int g = 16; g > 1; g >>= 1)
        if (m % g == 0) return g;
    return 1;
}

// gather == 0: out[index[n]] = src[n];  gather != 0: out[n] = src[index[n]]
template <int G>
__global__ void permute_rows_kernel(const char *src, const int32_t *index, int rows, int gpr, int gather, char *out)
{
    typedef typename Gran<G>::type T;
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (long)rows * gpr) return;
    int n = (int)(i / gpr), c = (int)(i - (long)n * gpr);
    int m = index ? index[n] : n;
    if ((unsigned)m >= (unsigned)rows) return;
    long s = gather ? m : n, d = gather ? n : m;
    ((T *)out)[d * gpr + c] = ((const T *)src)[s * gpr + c];
}

// One thread per (row, granule): the row's column comes from a binary search in
// z_ptr (inclusive scan), the cell from z_idx.
__device__ __forceinline__ int column_of_row(const int32_t *z_ptr, int ncol, int row)
{
    int lo = 0, hi = ncol; // first c with z_ptr[c] > row
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if (z_ptr[mid] > row) hi = mid; else lo = mid + 1;
    }
    return lo;
}

template <int G, bool BACKWARD>
__global__ void dense_kernel(const char *sparse_in, char *sparse_out, const char *dense_in, char *dense_out,
                             const int32_t *z_idx, const int32_t *z_ptr, int rows, int ncol, int S2, int gpr)
{
    typedef typename Gran<G>::type T;
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (long)rows * gpr) return;
    int n = (int)(i / gpr), c = (int)(i - (long)n * gpr);
    int col = column_of_row(z_ptr, ncol, n);
    int z = z_idx[n];
    if (col >= ncol || (unsigned)z >= (unsigned)S2) return;
    long cell = (long)col * S2 + z;
    if (!BACKWARD)
        ((T *)dense_out)[cell * gpr + c] = ((const T *)sparse_in)[(long)n * gpr + c];
    else
        ((T *)sparse_out)[(long)n * gpr + c] = ((const T *)dense_in)[cell * gpr + c];
}

#define DISPATCH_GRANULE(g, CALL) \
    switch (g) {                  \
    case 16: CALL(16); break;     \
    case 8: CALL(8); break;       \
    case 4: CALL(4); break;       \
    case 2: CALL(2); break;       \
    default: CALL(1); break;      \
    }

} // namespace

SPH_EXPORT int sph_permute_rows(const void *src, const int32_t *index, int rows, int row_bytes,
                                int gather, void *out, void *stream)
{
    SPH_REQUIRE(rows >= 0 && row_bytes > 0, SPH_ERR_ARG, "sph_permute_rows: bad size");
    if (rows == 0) return SPH_OK;
    SPH_REQUIRE(src && out, SPH_ERR_ARG, "sph_permute_rows: null pointer");
    int g = pick_granule(row_bytes, src, out);
    int gpr = row_bytes / g;
    long total = (long)rows * gpr;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    hipStream_t st = (hipStream_t)stream;
#define CALL(G) hipLaunchKernelGGL(permute_rows_kernel<G>, grid, block, 0, st, (const char *)src, index, rows, gpr, gather, (char *)out)
    DISPATCH_GRANULE(g, CALL)
#undef CALL
    return sph_check_launch("sph_permute_rows");
}

SPH_EXPORT int sph_to_dense(const void *feature, const int32_t *z_idx, const int32_t *z_ptr, int rows,
                            int ncol, int S2, int row_bytes, void *dense, void *stream)
{
    SPH_REQUIRE(rows >= 0 && ncol > 0 && S2 > 0 && row_bytes > 0, SPH_ERR_ARG, "sph_to_dense: bad size");
    if (rows == 0) return SPH_OK;
    SPH_REQUIRE(feature && z_idx && z_ptr && dense, SPH_ERR_ARG, "sph_to_dense: null pointer");
    int g = pick_granule(row_bytes, feature, dense);
    int gpr = row_bytes / g;
    long total = (long)rows * gpr;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    hipStream_t st = (hipStream_t)stream;
#define CALL(G) hipLaunchKernelGGL((dense_kernel<G, false>), grid, block, 0, st, (const char *)feature, (char *)nullptr, (const char *)nullptr, (char *)dense, z_idx, z_ptr, rows, ncol, S2, gpr)
    DISPATCH_GRANULE(g, CALL)
#undef CALL
    return sph_check_launch("sph_to_dense");
}

SPH_EXPORT int sph_to_dense_backward(const void *d_dense, const int32_t *z_idx, const int32_t *z_ptr,
                                     int rows, int ncol, int S2, int row_bytes, void *d_feature, void *stream)
{
    SPH_REQUIRE(rows >= 0 && ncol > 0 && S2 > 0 && row_bytes > 0, SPH_ERR_ARG, "sph_to_dense_backward: bad size");
    if (rows == 0) return SPH_OK;
    SPH_REQUIRE(d_dense && z_idx && z_ptr && d_feature, SPH_ERR_ARG, "sph_to_dense_backward: null pointer");
    int g = pick_granule(row_bytes, d_dense, d_feature);
    int gpr = row_bytes / g;
    long total = (long)rows * gpr;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    hipStream_t st = (hipStream_t)stream;
#define CALL(G) hipLaunchKernelGGL((dense_kernel<G, true>), grid, block, 0, st, (const char *)nullptr, (char *)d_feature, (const char *)d_dense, (char *)nullptr, z_idx, z_ptr, rows, ncol, S2, gpr)
    DISPATCH_GRANULE(g, CALL)
#undef CALL
    return sph_check_launch("sph_to_dense_backward");
}
