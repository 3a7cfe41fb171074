/*
 * sphconv_hip.h -- C ABI of libsphconv_hip.so (gfx950 / MI355X).
 *
 * Drop-in boundary for the sparse-convolution hot path of reveriel/sphconv:
 * the entry points below are what a binding of the reference's extension module
 * `sphconv.sphconv_cuda` (src/sphconv/all.cpp:14-38) calls instead of the CUDA
 * kernels.  Every pointer is a DEVICE pointer unless the comment says "host".
 * The library never allocates, frees or synchronises: the caller provides all
 * outputs and scratch, and every call only enqueues kernels on `stream`.
 *
 * Every function returns 0 on success or a negative sph_status; the message of
 * the last failure on the calling thread is returned by sph_last_error().
 *
 * Data layout (same as the reference, tensor.py:33-102 / tensor.cu:78-127):
 *   feature [rows, C]  row-major, element type given by sph_dtype
 *   z_idx   [rows]     int32, S2 coordinate of each row
 *   z_ptr   [B*S0*S1]  int32, INCLUSIVE prefix sum of per-column row counts in
 *                      flattened (b,s0,s1) order
 * Kernel offset index k = (k0*K1 + k1)*K2 + k2 (rules.cu:124-126); weight is
 * [KV, iC, oC].  Input x pairs with output o_d = (x_d + pad_d - k_d) / stride_d
 * iff divisible and 0 <= o_d < O_d (rules.cu:36-45); dilation is accepted and
 * ignored exactly as the reference does (rules.cu:39-40).
 *
 * Rule book (this library's compact replacement of the reference's padded
 * `rules [NTile,KV,2,tile_n_max]` tensor, rules.cu:364-366): the rows of the
 * stationary side are cut into tiles of SPH_TILE_ROWS consecutive rows; the
 * pairs of a tile are stored per kernel offset k, in ascending row order, in
 * groups of SPH_GROUP slots padded with -1:
 *   tile_ngrp [NT]              groups used by each tile
 *   tile_koff [NT, KV+1] u16    first group of offset k inside the tile
 *   grp_k     [NT*cap]          kernel offset of each group
 *   grp_gather[NT*cap*16]       row on the gathered side (or -1)
 *   grp_owner [NT*cap*16]       row on the stationary side (or -1)
 * with NT = sph_book_tiles(rows) and cap = sph_book_cap(KV) groups per tile.
 * A forward book is stationary on OUTPUT rows (gather = input row), a
 * transposed book on INPUT rows (gather = output row; used by dgrad).
 */
#ifndef SPHCONV_HIP_H
#define SPHCONV_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SPH_TILE_ROWS 128
#define SPH_GROUP 16
#define SPH_MAX_KV 128
#define SPH_MAX_CHANNELS 256

typedef enum sph_status {
    SPH_OK = 0,
    SPH_ERR_ARG = -1,         /* null pointer, bad size, bad enum                */
    SPH_ERR_UNSUPPORTED = -2, /* channel count / kernel volume out of range      */
    SPH_ERR_LAUNCH = -3       /* HIP reported an error at launch                 */
} sph_status;

typedef enum sph_dtype {
    SPH_F32 = 0,  /* fp32 storage, fp32 accumulate                     */
    SPH_F16 = 1,  /* fp16 storage, fp32 accumulate                     */
    SPH_BF16 = 2, /* bf16 storage, fp32 accumulate                     */
    SPH_I8 = 3    /* int8 storage, int32 accumulate, requantised store */
} sph_dtype;

/* Geometry of one convolution; argument meaning follows get_rules[_subm]
 * (include/sphconv/rules.h:8-32): spatialShape, outSpatialShape, kernelSize,
 * stride, padding, dilation, each ordered (S0,S1,S2). */
typedef struct sph_geom {
    int32_t B;
    int32_t S[3];
    int32_t O[3];
    int32_t K[3];
    int32_t stride[3];
    int32_t pad[3];
    int32_t dil[3];
} sph_geom;

typedef struct sph_book {
    int32_t *tile_ngrp;
    uint16_t *tile_koff;
    int32_t *grp_k;
    int32_t *grp_gather;
    int32_t *grp_owner;
    int32_t rows; /* rows on the stationary side */
    int32_t KV;
    /* Optional second form of the same pairs, by stationary row: [NT][KV][SPH_TILE_ROWS],
     * gathered row of (tile, offset, row of the tile) or -1.  When not null, sph_rules_build*
     * and sph_rules_from_padded fill it too, and sph_conv_apply walks it instead of the groups
     * (every offset of every block of 16 rows costs one step, whatever it holds: the faster
     * way from about ten pairs per row upwards).  Null: not kept.
     * A book that keeps this table may leave grp_k, grp_gather and grp_owner null (all three):
     * the rule kernel then writes only the table (tile_ngrp and tile_koff stay as they were), sph_conv_apply serves the calls
     * it can walk by rows (rows of 16-byte multiples up to 128 bytes) and refuses the others,
     * sph_conv_wgrad and sph_rules_to_padded_count refuse the book. */
    int32_t *tile_nbr;
    /* Set by the caller, read by sph_conv_apply: not 0 = the middle offset KV/2 holds a run of full groups in most
     * tiles, as in a submanifold layer, where it pairs every row with itself (and in that layer's transposed book).
     * The grouped kernel then gives that run to helper waves, which load its weight fragments once.  0 (also what
     * a zero-initialised struct says): no assumption; results are the same either way, up to the order of summation. */
    int32_t middle_run;
} sph_book;

const char *sph_last_error(void);
int sph_abi_version(void);

/* Sizing helpers (host arithmetic only). */
int sph_book_tiles(int rows);          /* NT = ceil(rows / SPH_TILE_ROWS)            */
int sph_book_cap(int KV);              /* groups per tile = KV * SPH_TILE_ROWS / 16  */
/* closed forms of the reference: rules.cu:21-34, conv.py:32-38 */
int sph_tile_n_max(const sph_geom *g, int T0, int T1, int nnz);
int sph_num_tiles(const sph_geom *g, int T0, int T1);

/* ---- rule generation --------------------------------------------------- */

/* Replaces get_rules_subm (rules.cu:326-390) and the pair half of get_rules
 * (rules.cu:445-485): builds the rule book of one convolution.
 *   transposed == 0: stationary side = output rows (oz_idx/oz_ptr over the O
 *                    grid), gathered side = input rows (z_idx/z_ptr over S).
 *   transposed == 1: stationary side = input rows, gathered side = output rows.
 * For a submanifold convolution pass the input arrays as the output arrays and
 * O == S.  `book.rows` must equal the stationary side's row count.
 * row_cols (may be null): the column (flattened (b,s0,s1) index into the stationary side's pointer
 * array) of every stationary row, as sph_row_columns, sph_init_tensor and sph_outcoords_fill write it.
 * The reference gets a row's column for free from its launch geometry (one thread per column,
 * rules.cu:256-259); here the tile workgroups otherwise search the pointer array for it.  Every
 * entry is checked against the pointer array before it is believed: a wrong table costs time and
 * cannot change the result. */
int sph_rules_build(const int32_t *z_idx, const int32_t *z_ptr, int in_rows,
                    const int32_t *oz_idx, const int32_t *oz_ptr, int out_rows,
                    const sph_geom *g, int transposed, const sph_book *book,
                    const int32_t *row_cols, void *stream);
/* row_cols[r] = column of row r, from the inclusive pointer array z_ptr [ncol] (the expansion the
 * reference's one-thread-per-column kernels never need, rules.cu:256-259). */
int sph_row_columns(const int32_t *z_ptr, int ncol, int rows, int32_t *row_cols, void *stream);
/* sph_rules_build with a weight pack (sph_weight_pack, same arguments) riding along as extra
 * workgroups of the same launch: for a layer whose rules are not cached yet, the forward pass
 * then is two launches (rules + pack, convolution) instead of three.  No reference counterpart
 * beyond get_rules* (rules.cu:326-486) and the weight argument of rule_conv (rule_conv.cu:286). */
int sph_rules_build_pack(const int32_t *z_idx, const int32_t *z_ptr, int in_rows,
                         const int32_t *oz_idx, const int32_t *oz_ptr, int out_rows,
                         const sph_geom *g, int transposed, const sph_book *book,
                         const int32_t *row_cols,
                         sph_dtype dt, const void *w, int KV, int kdim, int ndim, long stride_k,
                         long stride_kk, long stride_n, void *packed, void *stream);

/* Replaces the output-coordinate half of get_rules (rules.cu:417-443, 461-462: prepareGridKernel, two
 * cumsums, roll/index_put/add and the device->host read), in two steps because the caller must size oz_idx:
 *  1. sph_outcoords_count: counts every output column's active bins into oz_ptr and scans them in place
 *     (inclusive; one pass over the counts: tiles of 2048 columns look back over their predecessors'
 *     sums), and writes the number of output rows to *total_dev (null: not written; it is also the
 *     last element of oz_ptr).  total_dev is any address the GPU can write: device memory, or pinned host
 *     memory (hipHostMalloc) that the host reads after synchronising the stream, without a copy.
 *     `scratch`: 8-byte aligned device memory of sph_outcoords_scratch_ints(g) int32, contents arbitrary;
 *     its first sph_outcoords_state_ints(g) entries hold the state of the scan across workgroups, which
 *     the count kernel clears for the scan behind it (calls that overlap on one scratch race).
 *     Behind the state, when O[2] <= 512 and the masks of all columns take at most 128 MB, each column's
 *     64-bit masks of active bins (one per 64 bins) are kept for step 2; deeper or larger grids keep none
 *     and step 2 walks the fibers again.
 *  2. once the caller knows the total: sph_outcoords_fill, given the same scratch and oz_ptr, writes
 *     oz_idx (ascending within a column) and, when row_cols is not null, every output row's column
 *     (out_rows entries: the table sph_rules_build* takes for a layer that is stationary on these rows).
 * sph_outcoords_blocks(g) = ceil(columns / 256), the grid of the fill kernel. */
int sph_outcoords_blocks(const sph_geom *g);
int sph_outcoords_scratch_ints(const sph_geom *g);
int sph_outcoords_state_ints(const sph_geom *g);
int sph_outcoords_count(const int32_t *z_idx, const int32_t *z_ptr, int in_rows,
                        const sph_geom *g, int32_t *oz_ptr, int32_t *scratch,
                        int32_t *total_dev, void *stream);
int sph_outcoords_fill(const int32_t *z_idx, const int32_t *z_ptr, int in_rows,
                       const sph_geom *g, const int32_t *scratch, int32_t *oz_ptr,
                       int32_t *oz_idx, int out_rows, int32_t *row_cols, void *stream);

/* sph_outcoords_count for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * kernels and results as sph_outcoords_count, but the scratch is an array of the library's own
 * (8.0 MiB of static device memory on each GPU the library runs on, held until the process ends),
 * so the call allocates and frees nothing.  It serves grids of up to SPH_STATIC_MAX_COLUMNS output
 * columns (B * O[0] * O[1]; with 64 < O[2] <= 512 a column counts ceil(O[2] / 64) times, once per mask
 * it keeps) and refuses larger ones with SPH_ERR_UNSUPPORTED.  *scratch_out (may be
 * null) receives the array's device address on the current GPU: pass it as `scratch` to
 * sph_outcoords_fill.  Every call on a GPU shares that GPU's array, which keeps the last call's
 * contents (the call clears the part that must start at zero): calls that overlap on one GPU race,
 * and a second call overwrites the bin masks a pending sph_outcoords_fill of the first would read. */
#define SPH_STATIC_MAX_COLUMNS 1048576
int sph_outcoords_count_static(const int32_t *z_idx, const int32_t *z_ptr, int in_rows,
                               const sph_geom *g, int32_t *oz_ptr, int32_t *total_dev,
                               const int32_t **scratch_out, void *stream);

/* Conversions between the rule book and the reference's padded tensors
 * `rules [NTile,KV,2,tile_n_max]`, `rule_size [NTile,KV]` (rules.cu:364-369).
 * nbr is scratch of out_rows*KV int32 (forward) / in_rows*KV (transposed). */
int sph_rules_to_padded_count(const sph_book *fwd_book, const int32_t *oz_ptr,
                              const sph_geom *g, int T0, int T1, int32_t *nbr,
                              int32_t *rule_size, void *stream);
int sph_rules_to_padded_fill(const int32_t *oz_ptr, const sph_geom *g, int T0, int T1,
                             const int32_t *nbr, int out_rows, int KV, int tile_n_max,
                             int32_t *rules, void *stream);
int sph_rules_from_padded(const int32_t *rules, const int32_t *rule_size, int ntile, int KV,
                          int tile_n_max, int in_rows, int out_rows, int transposed,
                          int32_t *nbr, const sph_book *book, void *stream);

/* ---- convolution ------------------------------------------------------- */

/* Bytes of the packed (MFMA fragment order) copy of a [KV, kdim, ndim] weight. */
size_t sph_weight_packed_bytes(sph_dtype dt, int KV, int kdim, int ndim);
/* Packs weight for the contraction  out[., n] += sum_kk in[., kk] * B[k][kk][n]
 * where B[k][kk][n] = w[k*stride_k + kk*stride_kk + n*stride_n] (element strides). */
int sph_weight_pack(sph_dtype dt, const void *w, int KV, int kdim, int ndim,
                    long stride_k, long stride_kk, long stride_n, void *packed, void *stream);

/* Optional epilogue applied to the accumulator before the store:
 *   y = acc * scale[c] + shift[c]   (each pointer may be null: 1 / 0)
 *   y = max(y, 0) if relu
 * For SPH_I8, scale is required and the store is
 *   q = clamp(rint((float)acc * scale[c]), -128, 127)      (shift, relu unused). */
typedef struct sph_epilogue {
    const float *scale;
    const float *shift;
    int32_t relu;
} sph_epilogue;

/* Replaces rule_conv (rule_conv.cu:286-336) and, with a transposed book and a
 * weight packed from W[k]^T, rule_conv_d_feature (rule_conv.cu:520-575):
 *   out[owner, :] = sum over the owner's pairs (k, gather) of
 *                   feature[gather, :kdim] @ B[k]          (rows with no pair: 0)
 * out has book->rows rows of ndim elements and is fully overwritten. */
int sph_conv_apply(sph_dtype dt, const void *feature, int feature_rows, int kdim,
                   const void *packed_w, int ndim, const sph_book *book,
                   const sph_epilogue *epi, void *out, void *stream);

/* get_rules_subm / get_rules' pair half (rules.cu:326-390, 445-485) and rule_conv (rule_conv.cu:286-336) of ONE
 * layer in ONE launch: every workgroup builds its tile's pairs in LDS as sph_rules_build does and convolves them
 * at once as sph_conv_apply does; `out` [out_rows, ndim] is fully overwritten.  Arguments as for sph_rules_build
 * (transposed == 0) and sph_conv_apply.  `book` must provide all group arrays: with SPH_FUSED_WRITE_BOOK in
 * `flags` the book is filled as sph_rules_build fills it (for layers that share it through an indice_key, or for
 * a backward pass); without it only tiles whose groups do not fit the workgroup's LDS (more than 64 groups) use
 * their part of it, and its contents are unspecified afterwards.  SPH_FUSED_IN_FLIGHT says that the caller keeps
 * several scans in flight on streams of their own: the launch then uses two-wave workgroups, four of which fit a
 * CU where three four-wave ones do -- a lone scan takes about a tenth longer, a stream of scans a tenth less.  Returns SPH_ERR_UNSUPPORTED (nothing launched) for
 * shapes the fused kernel does not take -- rows that are not 16-byte multiples of up to 128 bytes, more than 64
 * output channels, more than 32 kernel offsets: call sph_rules_build + sph_conv_apply then. */
enum { SPH_FUSED_WRITE_BOOK = 1, SPH_FUSED_IN_FLIGHT = 2 };
int sph_rules_conv(const int32_t *z_idx, const int32_t *z_ptr, int in_rows, const int32_t *oz_idx,
                   const int32_t *oz_ptr, int out_rows, const sph_geom *g, const sph_book *book, int flags,
                   const int32_t *row_cols, sph_dtype dt, const void *feature, int kdim, const void *packed_w,
                   int ndim, const sph_epilogue *epi, void *out, void *stream);

/* Replaces rule_conv_d_weight (rule_conv.cu:469-518):
 *   d_weight[k, ci, co] = sum over pairs (k, in, out) feature[in, ci] * d_out[out, co]
 * from a FORWARD book.  partial is fp32 scratch of
 * sph_wgrad_partial_elems(KV, iC, oC, rows) elements; the reduction over it is
 * done in fp32 in a fixed order.  d_weight [KV, iC, oC] has the element type dt, or is fp32
 * when d_weight_f32 != 0 (16-bit features with an fp32 master weight: the sums over 1e5
 * pairs need not be rounded to, or overflow, a 16-bit type). */
size_t sph_wgrad_partial_elems(int KV, int iC, int oC, int out_rows);
int sph_conv_wgrad(sph_dtype dt, const void *feature, int in_rows, int iC, const void *d_out,
                   int oC, const sph_book *fwd_book, float *partial, void *d_weight,
                   int d_weight_f32, void *stream);

/* ---- tensor construction / densify (tensor.cu) ------------------------- */

/* out[dst_row[n], :] = src[n, :] (dst_row null: identity) or, with gather != 0,
 * out[n, :] = src[dst_row[n], :].  Rows of row_bytes bytes.  Replaces
 * reorderFeatureKernel / reorderFeatureBackwardKernel (tensor.cu:39-76,130-145). */
int sph_permute_rows(const void *src, const int32_t *index, int rows, int row_bytes,
                     int gather, void *out, void *stream);
/* Replaces init_tensor's index work (src/sphconv/tensor.cu:78-127 with fillGridKernel 21-36
 * and the index half of reorderFeatureKernel 39-76): COO coordinates `indices` [n,4] int32
 * (b, s0, s1, s2) -> z_idx [n], z_ptr [B*S0*S1] (inclusive counts) and permutation [n]
 * (input row r becomes row permutation[r]; move the features with sph_permute_rows,
 * gather = 0).  Fibers come out in ascending S2 order.  status [2] int32 (device) receives
 * the number of coordinates outside the grid and the number of duplicated coordinates;
 * the outputs are only meaningful when both are 0.  `workspace` is device memory of at
 * least sph_init_tensor_workspace(...) bytes, 256-byte aligned; nothing is allocated. */
size_t sph_init_tensor_workspace(int n, int B, int S0, int S1, int S2);
int sph_init_tensor(const int32_t *indices, int n, int B, int S0, int S1, int S2, int32_t *z_idx,
                    int32_t *z_ptr, int32_t *permutation, int32_t *status, void *workspace,
                    size_t workspace_bytes, void *stream);
/* Replaces to_dense / to_dense_backward (tensor.cu:222-309): dense is
 * [B,S0,S1,S2,C]; only active cells are written (forward) / read (backward). */
int sph_to_dense(const void *feature, const int32_t *z_idx, const int32_t *z_ptr, int rows,
                 int ncol, int S2, int row_bytes, void *dense, void *stream);
int sph_to_dense_backward(const void *d_dense, const int32_t *z_idx, const int32_t *z_ptr,
                          int rows, int ncol, int S2, int row_bytes, void *d_feature,
                          void *stream);

/* Replaces the numpy body of xyz2RangeVoxel (sphconv/data.py:75-128): `points` [m,ndim] float32
 * on the device (x, y, z first) -> one voxel per pixel of a v_res x h_res range image:
 * feature [ndim, v_res, h_res] (the winning point's values, 0 elsewhere), depth [v_res, h_res]
 * (depth bin), thick [v_res, h_res] (1 where a point landed).  Angles in radians:
 * v0 / h0 = lower bounds of the polar / azimuth range, dtheta / dphi = bin sizes; depth bin =
 * (log(r) - d0) / dr with d0 = log(d_range[0]) if use_log, else (r - d0) / dr.  Among points
 * that share a pixel the one with the largest index wins (the reference's "later points
 * overwrite earlier ones", data.py:106-108).  `winner` is scratch of v_res*h_res int32;
 * idx_out (optional, [m,3] int32) receives each point's (theta, phi, depth) bins. */
int sph_xyz_to_rangevoxel(const float *points, int m, int ndim, int v_res, int h_res, int d_res,
                          float v0_rad, float h0_rad, float dtheta, float dphi, float d0, float dr,
                          int use_log, int32_t *winner, float *feature, int32_t *depth, int32_t *thick,
                          int32_t *idx_out, void *stream);

/* Replaces points_to_voxel_3d (include/point2voxel.h:412-512) together with the coordinate
 * transforms of sphconv/utils/coord_transform.py:8-118: `points` [n,nfeat] float32 on the device
 * (x, y, z, intensity first) are mapped to system coordinates (c0, c1, c2) --
 *   system 0 spherical (r, phi, theta)   1 l-spherical (log r, phi, theta)
 *          2 cylinder  (d, phi, z)       3 l-cylinder  (log d, phi, z)
 *          4 hybrid    (d, phi, theta)   5 l-hybrid    (log d, phi, theta)
 * -- and binned: bin_i = floor((c_i - lo_i) / vs_i), points with a bin outside [0, g_i) are skipped.
 * Voxels are numbered in order of first appearance in the point list, keep their first max_points
 * points, and every point from the one that would open voxel number max_voxels on is dropped, as
 * in the reference's loop.  Outputs (all zero where unused): voxels [max_voxels, max_points, W]
 * (append_mode 0: the point's nfeat values, W = nfeat; 1: those plus (c0, c1, c2), W = nfeat + 3;
 * 2: (c0, c1, c2, intensity), W = nfeat), mask [max_voxels, max_points] (1.0 where a point sits),
 * coors [max_voxels, 3] = (bin of c2, of c1, of c0), num_points [max_voxels], voxel_num [1] (device).
 * cell_in (optional, [n] int64): take these cells ((bin2*g1 + bin1)*g0 + bin0, negative = skip)
 * instead of computing them; cell_out (optional): receives the cells.  `workspace`: device memory
 * of sph_points_to_voxel_workspace(n, g0, g1, g2) bytes, 256-byte aligned; nothing is allocated. */
size_t sph_points_to_voxel_workspace(int n, int g0, int g1, int g2);
int sph_points_to_voxel(const float *points, int n, int nfeat, int system, float lo0, float lo1, float lo2,
                        float vs0, float vs1, float vs2, int g0, int g1, int g2, int max_points,
                        int max_voxels, int append_mode, float *voxels, float *mask, int32_t *coors,
                        int32_t *num_points, int32_t *voxel_num, const long long *cell_in,
                        long long *cell_out, void *workspace, size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SPHCONV_HIP_H */
