/*
 * sphconv_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C, CPU restatement of the reference's sparse-convolution hot path
 * (reveriel/sphconv).  The reference implements this path only as CUDA
 * kernels; there is no reference CPU path.  Each function below follows the
 * loop structure and arithmetic of the reference kernel it cites, with the
 * parallel thread grid replaced by (optionally OpenMP) loops.
 *
 * Only tests, the smoke check and the benchmark's cpu_baseline leg may load
 * this library -- as the checker / reported baseline, never as a fallback for
 * the HIP library.
 *
 * Parity status of each function (what independently pins it) is listed in
 * oracle/README.md; functions that restate behaviour defined by this
 * repository rather than by the reference (int8 requantisation) say so.
 *
 * Layout restated from the reference (tensor.py:33-102, tensor.cu:78-127):
 *   feature [NNZ,C] row-major; z_idx [NNZ] = S2 coordinate of each row;
 *   z_ptr [B,S0,S1] = INCLUSIVE prefix sum of per-column voxel counts over the
 *   flattened (b,s0,s1) order; column c owns rows [z_ptr[c-1] (0 if c==0), z_ptr[c]).
 *   rules [NTile,KV,2,tile_n_max] filled with -1; rule_size [NTile,KV].
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define EXPORT __attribute__((visibility("default")))

/* debug_utils.h:17-20 */
static inline int div_up(int x, int y) { return (x + y - 1) / y; }

/* debug_utils.h:37-42 */
static inline int linear_tile_idx(int T0, int T1, int x, int y, int tile_grid_w)
{
    return (x / T0) * tile_grid_w + (y / T1);
}

/* rules.cu:36-45 -- dilation is accepted and ignored, as in the reference. */
static inline int out_spatial1(int k, int x, int s, int d, int pad)
{
    (void)d;
    if ((x + pad - k) % s == 0)
        return (x + pad - k) / s;
    return -1;
}

EXPORT int orc_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

EXPORT void orc_set_num_threads(int n)
{
#ifdef _OPENMP
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* rules.cu:30-34 */
EXPORT int orc_in_tile_size(int out_tile, int stride, int kernel)
{
    return stride * (out_tile - 1) + kernel;
}

/* rules.cu:21-28 (`& (-1 << 4)` == clear the low four bits) */
EXPORT int orc_tile_n_max(int in_t0, int in_t1, int B, int S0, int S1, int S2, int nnz)
{
    double sparsity = (double)nnz / ((double)B * S0 * S1 * S2);
    double size = (double)B * in_t0 * in_t1 * S2 * sparsity * 2;
    return (int)(size + 64) & ~15;
}

/* utils/__init__.py:27-44 (floor of the PyTorch output-size formula) */
EXPORT int orc_out_spatial_dim(int in, int k, int s, int pad, int dil)
{
    return (int)floor((double)(in + 2 * pad - dil * (k - 1) - 1) / s + 1);
}

/* ---------------------------------------------------------------------------
 * init_tensor: COO -> per-column compressed form.  tensor.cu:78-127.
 * The reference orders rows inside a fiber by atomic race; this restatement
 * emits the canonical order (ascending S2), one legal serialisation.
 * indices rows are (b, s0, s1, s2) (tensor.cu:30-33).
 * Returns 0, or -1 on an out-of-range coordinate, -2 on a duplicate.
 * ------------------------------------------------------------------------- */
EXPORT int orc_init_tensor(const float *feature, const int32_t *indices, int nnz, int C,
                           int B, int S0, int S1, int S2,
                           float *out_feature, int32_t *z_idx, int32_t *z_ptr,
                           int32_t *permutation)
{
    size_t ncol = (size_t)B * S0 * S1;
    size_t ncell = ncol * S2;
    int32_t *grid = (int32_t *)malloc(ncell * sizeof(int32_t));
    if (!grid) return -3;
    /* fillGridKernel (tensor.cu:21-36): mark occupied cells; here the cell keeps
       the COO row (+1) so the reorder below can be done in S2 order. */
    memset(grid, 0, ncell * sizeof(int32_t));
    for (int n = 0; n < nnz; n++) {
        int b = indices[4 * n + 0], x = indices[4 * n + 1];
        int y = indices[4 * n + 2], z = indices[4 * n + 3];
        if (b < 0 || b >= B || x < 0 || x >= S0 || y < 0 || y >= S1 || z < 0 || z >= S2) {
            free(grid);
            return -1;
        }
        size_t cell = (((size_t)b * S0 + x) * S1 + y) * S2 + z;
        if (grid[cell]) { free(grid); return -2; }
        grid[cell] = n + 1;
    }
    /* fiberSize = sum over S2; zPtr = inclusive cumsum (tensor.cu:106-109) */
    int32_t run = 0;
    for (size_t c = 0; c < ncol; c++) {
        int32_t start = run;
        for (int z = 0; z < S2; z++) {
            int32_t src = grid[c * S2 + z];
            if (src) {
                int n = src - 1;
                /* reorderFeatureKernel (tensor.cu:39-76) */
                memcpy(out_feature + (size_t)run * C, feature + (size_t)n * C, C * sizeof(float));
                z_idx[run] = z;
                permutation[n] = run;
                run++;
            }
        }
        (void)start;
        z_ptr[c] = run;
    }
    free(grid);
    return 0;
}

/* tensor.cu:130-162 */
EXPORT void orc_init_tensor_backward(const float *d_out, const int32_t *permutation,
                                     int nnz, int C, float *d_feature)
{
    for (int n = 0; n < nnz; n++)
        memcpy(d_feature + (size_t)n * C, d_out + (size_t)permutation[n] * C, C * sizeof(float));
}

/* tensor.cu:165-192, 222-264: out is [B,S0,S1,S2,C]; only active cells are written. */
EXPORT void orc_to_dense(const float *feature, const int32_t *z_idx, const int32_t *z_ptr,
                         int B, int S0, int S1, int S2, int C, float *out)
{
    size_t ncol = (size_t)B * S0 * S1;
    for (size_t c = 0; c < ncol; c++) {
        int zs = c ? z_ptr[c - 1] : 0, ze = z_ptr[c];
        for (int pos = zs; pos < ze; pos++)
            memcpy(out + (c * S2 + z_idx[pos]) * C, feature + (size_t)pos * C, C * sizeof(float));
    }
}

/* tensor.cu:194-220, 266-309 */
EXPORT void orc_to_dense_backward(const float *d_out, const int32_t *z_idx, const int32_t *z_ptr,
                                  int B, int S0, int S1, int S2, int C, float *d_feature)
{
    size_t ncol = (size_t)B * S0 * S1;
    for (size_t c = 0; c < ncol; c++) {
        int zs = c ? z_ptr[c - 1] : 0, ze = z_ptr[c];
        for (int pos = zs; pos < ze; pos++)
            memcpy(d_feature + (size_t)pos * C, d_out + (c * S2 + z_idx[pos]) * C, C * sizeof(float));
    }
}

/* ---------------------------------------------------------------------------
 * Rule generation.
 * ------------------------------------------------------------------------- */
typedef struct {
    int B, S0, S1, S2;      /* input grid                    */
    int O0, O1, O2;         /* output grid                   */
    int K0, K1, K2;
    int s0, s1, s2;
    int p0, p1, p2;
    int d0, d1, d2;         /* accepted, ignored (rules.cu:39-40) */
    int T0, T1;             /* output tile size              */
} orc_geom;

static int cmp_pair(const void *a, const void *b)
{
    const int32_t *x = (const int32_t *)a, *y = (const int32_t *)b;
    if (x[0] != y[0]) return x[0] < y[0] ? -1 : 1;
    return (x[1] > y[1]) - (x[1] < y[1]);
}

/* Put every (tile,k) list into canonical order (ascending input row).  The
   reference's order inside a list is the order in which atomicAdd handed out
   slots (rules.cu:215,299), i.e. unspecified; sorting picks one legal order. */
EXPORT void orc_rules_canonicalize(int32_t *rules, const int32_t *rule_size,
                                   int ntile, int KV, int tile_n_max)
{
#pragma omp parallel
    {
        int32_t *tmp = (int32_t *)malloc((size_t)tile_n_max * 2 * sizeof(int32_t));
#pragma omp for schedule(dynamic, 64)
        for (int tk = 0; tk < ntile * KV; tk++) {
            int n = rule_size[tk];
            if (n > tile_n_max) n = tile_n_max;
            if (n < 2) continue;
            int32_t *in = rules + (size_t)tk * 2 * tile_n_max, *out = in + tile_n_max;
            for (int v = 0; v < n; v++) { tmp[2 * v] = in[v]; tmp[2 * v + 1] = out[v]; }
            qsort(tmp, n, 2 * sizeof(int32_t), cmp_pair);
            for (int v = 0; v < n; v++) { in[v] = tmp[2 * v]; out[v] = tmp[2 * v + 1]; }
        }
        free(tmp);
    }
}

/* get_rules_subm: rules.cu:326-390 with prepareSubMGridKernel (55-82) and
 * getSubMRulesKernel (234-311).  grid is caller-provided scratch of
 * B*O0*O1*O2 int32.  rules must hold NTile*KV*2*tile_n_max, rule_size NTile*KV.
 * Returns the number of pairs dropped by overflow (the reference printf's and
 * drops them, rules.cu:301-308; rule_size still counts them). */
EXPORT int orc_rules_subm(const int32_t *z_idx, const int32_t *z_ptr, const orc_geom *g,
                          int tile_n_max, int32_t *grid, int32_t *rules, int32_t *rule_size)
{
    const int B = g->B, H = g->S0, W = g->S1;
    const int oH = g->O0, oW = g->O1, oD = g->O2;
    const int KV = g->K0 * g->K1 * g->K2;
    const int tile_grid_w = div_up(oW, g->T1);
    const int ntile = div_up(oH, g->T0) * tile_grid_w;
    size_t ncell = (size_t)B * oH * oW * oD;
    size_t nrules = (size_t)ntile * KV * 2 * tile_n_max;
    int dropped = 0;

    /* torch::full(grid,-1), torch::full(rules,-1), zeros(ruleSize): rules.cu:339,364,368 */
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < ncell; i++) grid[i] = -1;
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < nrules; i++) rules[i] = -1;
    memset(rule_size, 0, (size_t)ntile * KV * sizeof(int32_t));

    /* prepareSubMGridKernel */
#pragma omp parallel for collapse(2) schedule(static)
    for (int x = 0; x < H; x++)
        for (int y = 0; y < W; y++)
            for (int b = 0; b < B; b++) {
                size_t c = ((size_t)b * H + x) * W + y;
                int zs = c ? z_ptr[c - 1] : 0, ze = z_ptr[c];
                for (int pos = zs; pos < ze; pos++)
                    grid[c * oD + z_idx[pos]] = pos; /* subm: input grid == output grid */
            }

    /* getSubMRulesKernel: one logical thread per (x, y, k) */
#pragma omp parallel for collapse(2) schedule(static) reduction(+ : dropped)
    for (int x = 0; x < H; x++)
        for (int y = 0; y < W; y++)
            for (int k = 0; k < KV; k++) {
                int k_H = k / (g->K1 * g->K2);
                int k_W = (k / g->K2) % g->K1;
                int k_D = k % g->K2;
                int oX = out_spatial1(k_H, x, g->s0, g->d0, g->p0);
                if (oX < 0 || oX >= oH) continue;
                int oY = out_spatial1(k_W, y, g->s1, g->d1, g->p1);
                if (oY < 0 || oY >= oW) continue;
                int tile = linear_tile_idx(g->T0, g->T1, oX, oY, tile_grid_w);
                for (int b = 0; b < B; b++) {
                    size_t c = ((size_t)b * H + x) * W + y;
                    int zs = c ? z_ptr[c - 1] : 0, ze = z_ptr[c];
                    for (int gi = zs; gi < ze; gi++) {
                        int z = z_idx[gi];
                        int oZ = out_spatial1(k_D, z, g->s2, g->d2, g->p2);
                        if (oZ < 0 || oZ >= oD) continue;
                        int go = grid[(((size_t)b * oH + oX) * oW + oY) * oD + oZ];
                        if (go < 0) continue;
                        int counter;
#pragma omp atomic capture
                        counter = rule_size[tile * KV + k]++;
                        if (counter < tile_n_max) {
                            int32_t *r = rules + ((size_t)tile * KV + k) * 2 * tile_n_max;
                            r[counter] = gi;
                            r[tile_n_max + counter] = go;
                        } else {
                            dropped++;
                        }
                    }
                }
            }
    return dropped;
}

/* get_rules, first half: rules.cu:417-443.  prepareGridKernel (98-150) marks every
 * reachable output cell, then cumsum along S2, cumsum of the column totals
 * (= oz_ptr, inclusive), and grid += exclusive column scan so that
 * grid[cell] - 1 is the global output row of an active cell.
 * Returns outNNZ (rules.cu:461). */
EXPORT int orc_rules_std_outgrid(const int32_t *z_idx, const int32_t *z_ptr, const orc_geom *g,
                                 int32_t *grid, int32_t *oz_ptr)
{
    const int B = g->B, H = g->S0, W = g->S1;
    const int oH = g->O0, oW = g->O1, oD = g->O2;
    const int KV = g->K0 * g->K1 * g->K2;
    size_t ocol = (size_t)B * oH * oW;
    memset(grid, 0, ocol * oD * sizeof(int32_t));

#pragma omp parallel for collapse(2) schedule(static)
    for (int x = 0; x < H; x++)
        for (int y = 0; y < W; y++)
            for (int k = 0; k < KV; k++) {
                int k_H = k / (g->K1 * g->K2);
                int k_W = (k / g->K2) % g->K1;
                int k_D = k % g->K2;
                int oX = out_spatial1(k_H, x, g->s0, g->d0, g->p0);
                if (oX < 0 || oX >= oH) continue;
                int oY = out_spatial1(k_W, y, g->s1, g->d1, g->p1);
                if (oY < 0 || oY >= oW) continue;
                for (int b = 0; b < B; b++) {
                    size_t c = ((size_t)b * H + x) * W + y;
                    int zs = c ? z_ptr[c - 1] : 0, ze = z_ptr[c];
                    for (int pos = zs; pos < ze; pos++) {
                        int oZ = out_spatial1(k_D, z_idx[pos], g->s2, g->d2, g->p2);
                        if (oZ < 0 || oZ >= oD) continue;
                        /* benign race: every writer stores 1 */
                        grid[(((size_t)b * oH + oX) * oW + oY) * oD + oZ] = 1;
                    }
                }
            }

    /* cumsum over S2 (rules.cu:434), column totals -> inclusive scan (436-437) */
#pragma omp parallel for schedule(static)
    for (size_t c = 0; c < ocol; c++) {
        int32_t run = 0;
        for (int z = 0; z < oD; z++) { run += grid[c * oD + z]; grid[c * oD + z] = run; }
    }
    int32_t total = 0;
    for (size_t c = 0; c < ocol; c++) { total += grid[c * oD + oD - 1]; oz_ptr[c] = total; }
    /* exclusive scan broadcast onto the grid (439-441) */
#pragma omp parallel for schedule(static)
    for (size_t c = 0; c < ocol; c++) {
        int32_t excl = c ? oz_ptr[c - 1] : 0;
        for (int z = 0; z < oD; z++) grid[c * oD + z] += excl;
    }
    return total;
}

/* get_rules, second half: rules.cu:445-485 with getOzIndicesAndRulesKernel (156-228).
 * `grid` is the array produced by orc_rules_std_outgrid.  Returns dropped pairs. */
EXPORT int orc_rules_std_fill(const int32_t *z_idx, const int32_t *z_ptr, const orc_geom *g,
                              int tile_n_max, const int32_t *grid, int32_t *oz_idx,
                              int32_t *rules, int32_t *rule_size)
{
    const int B = g->B, H = g->S0, W = g->S1;
    const int oH = g->O0, oW = g->O1, oD = g->O2;
    const int KV = g->K0 * g->K1 * g->K2;
    const int tile_grid_w = div_up(oW, g->T1);
    const int ntile = div_up(oH, g->T0) * tile_grid_w;
    size_t nrules = (size_t)ntile * KV * 2 * tile_n_max;
    int dropped = 0;

#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < nrules; i++) rules[i] = -1;
    memset(rule_size, 0, (size_t)ntile * KV * sizeof(int32_t));

#pragma omp parallel for collapse(2) schedule(static) reduction(+ : dropped)
    for (int x = 0; x < H; x++)
        for (int y = 0; y < W; y++)
            for (int k = 0; k < KV; k++) {
                int k_H = k / (g->K1 * g->K2);
                int k_W = (k / g->K2) % g->K1;
                int k_D = k % g->K2;
                int oX = out_spatial1(k_H, x, g->s0, g->d0, g->p0);
                if (oX < 0 || oX >= oH) continue;
                int oY = out_spatial1(k_W, y, g->s1, g->d1, g->p1);
                if (oY < 0 || oY >= oW) continue;
                int tile = linear_tile_idx(g->T0, g->T1, oX, oY, tile_grid_w);
                for (int b = 0; b < B; b++) {
                    size_t c = ((size_t)b * H + x) * W + y;
                    int zs = c ? z_ptr[c - 1] : 0, ze = z_ptr[c];
                    for (int gi = zs; gi < ze; gi++) {
                        int oZ = out_spatial1(k_D, z_idx[gi], g->s2, g->d2, g->p2);
                        if (oZ < 0 || oZ >= oD) continue;
                        int go = grid[(((size_t)b * oH + oX) * oW + oY) * oD + oZ] - 1;
                        int counter;
#pragma omp atomic capture
                        counter = rule_size[tile * KV + k]++;
                        if (counter < tile_n_max) {
                            int32_t *r = rules + ((size_t)tile * KV + k) * 2 * tile_n_max;
                            r[counter] = gi;
                            r[tile_n_max + counter] = go;
                        } else {
                            dropped++;
                        }
                        oz_idx[go] = oZ; /* same value from every writer */
                    }
                }
            }
    return dropped;
}

/* ---------------------------------------------------------------------------
 * Convolution, fp32.
 * ------------------------------------------------------------------------- */
#define VBLOCK 8 /* rule_conv.cu:308-323: every instance uses VBLOCK = 8 */

/* rule_conv (rule_conv.cu:286-336) + kernel::Conv::tile_rule_conv
 * (rule_conv_kernel.cu.h:91-153): out is zero-initialised, then for every
 * tile, k and block of 8 pairs:  D = 1*(A*W[k]) + 1*C  with C = D = out rows.
 * One tile per logical thread block; tiles own disjoint output rows. */
EXPORT void orc_rule_conv_f32(const float *feature, const float *weight,
                              const int32_t *rules, const int32_t *rule_size,
                              int ntile, int KV, int tile_n_max, int iC, int oC,
                              int out_nnz, float *out)
{
    memset(out, 0, (size_t)out_nnz * oC * sizeof(float));
#pragma omp parallel
    {
        float *acc = (float *)malloc((size_t)VBLOCK * oC * sizeof(float));
#pragma omp for schedule(dynamic, 32)
        for (int t = 0; t < ntile; t++) {
            for (int k = 0; k < KV; k++) {
                int n = rule_size[t * KV + k];
                if (n == 0) continue;
                if (n > tile_n_max) n = tile_n_max;
                const int32_t *rin = rules + ((size_t)t * KV + k) * 2 * tile_n_max;
                const int32_t *rout = rin + tile_n_max;
                const float *Wk = weight + (size_t)k * iC * oC;
                for (int vb = 0; vb < n; vb += VBLOCK) {
                    int nv = n - vb < VBLOCK ? n - vb : VBLOCK;
                    memset(acc, 0, (size_t)VBLOCK * oC * sizeof(float));
                    for (int v = 0; v < nv; v++) {
                        const float *a = feature + (size_t)rin[vb + v] * iC;
                        float *d = acc + (size_t)v * oC;
                        for (int c = 0; c < iC; c++) {
                            float av = a[c];
                            const float *w = Wk + (size_t)c * oC;
                            for (int o = 0; o < oC; o++) d[o] = fmaf(av, w[o], d[o]);
                        }
                    }
                    for (int v = 0; v < nv; v++) {
                        float *dst = out + (size_t)rout[vb + v] * oC;
                        const float *d = acc + (size_t)v * oC;
                        for (int o = 0; o < oC; o++) dst[o] = d[o] + dst[o];
                    }
                }
            }
        }
        free(acc);
    }
}

/* rule_conv_d_feature (rule_conv.cu:520-575): the forward kernel with the two
 * rule columns swapped and the weight pre-permuted by the caller to [KV,oC,iC]
 * (functional.py:73).  Overlapping input halos of neighbouring tiles are kept
 * race free by nine serial phases, phase i covering tiles (3*bx + i/3, 3*by + i%3)
 * (rule_conv.cu:271-276, threadblock_swizzle.h:113-173). */
EXPORT void orc_rule_conv_dfeature_f32(const float *d_out, const float *weight_oc_ic,
                                       const int32_t *rules, const int32_t *rule_size,
                                       int tile_grid_h, int tile_grid_w, int KV, int tile_n_max,
                                       int iC, int oC, int nnz, float *d_feature)
{
    memset(d_feature, 0, (size_t)nnz * iC * sizeof(float));
    for (int phase = 0; phase < 9; phase++) {
        int ph = phase / 3, pw = phase % 3;
        int nbh = div_up(tile_grid_h, 3), nbw = div_up(tile_grid_w, 3);
#pragma omp parallel
        {
            float *acc = (float *)malloc((size_t)VBLOCK * iC * sizeof(float));
#pragma omp for collapse(2) schedule(dynamic, 8)
            for (int bx = 0; bx < nbh; bx++)
                for (int by = 0; by < nbw; by++) {
                    int th = 3 * bx + ph, tw = 3 * by + pw;
                    if (th >= tile_grid_h || tw >= tile_grid_w) continue;
                    int t = th * tile_grid_w + tw;
                    for (int k = 0; k < KV; k++) {
                        int n = rule_size[t * KV + k];
                        if (n == 0) continue;
                        if (n > tile_n_max) n = tile_n_max;
                        const int32_t *rin = rules + ((size_t)t * KV + k) * 2 * tile_n_max;
                        const int32_t *rout = rin + tile_n_max;
                        const float *Wk = weight_oc_ic + (size_t)k * oC * iC;
                        for (int vb = 0; vb < n; vb += VBLOCK) {
                            int nv = n - vb < VBLOCK ? n - vb : VBLOCK;
                            memset(acc, 0, (size_t)VBLOCK * iC * sizeof(float));
                            for (int v = 0; v < nv; v++) {
                                const float *a = d_out + (size_t)rout[vb + v] * oC;
                                float *d = acc + (size_t)v * iC;
                                for (int o = 0; o < oC; o++) {
                                    float av = a[o];
                                    const float *w = Wk + (size_t)o * iC;
                                    for (int c = 0; c < iC; c++) d[c] = fmaf(av, w[c], d[c]);
                                }
                            }
                            for (int v = 0; v < nv; v++) {
                                float *dst = d_feature + (size_t)rin[vb + v] * iC;
                                const float *d = acc + (size_t)v * iC;
                                for (int c = 0; c < iC; c++) dst[c] = d[c] + dst[c];
                            }
                        }
                    }
                }
            free(acc);
        }
    }
}

/* rule_conv_d_weight (rule_conv.cu:469-518) + kernel::ConvDW
 * (rule_conv_kernel.cu.h:381-450): per tile and k a partial
 * dW[tile][k] = sum_v feature[in_v]^T (x) d_out[out_v], then torch::sum over
 * tiles (rule_conv.cu:517).  The reference materialises [NTile,KV,iC,oC]
 * (gigabytes at the benchmark shapes); here each thread keeps one [KV,iC,oC]
 * partial, summed over threads at the end -- the same sum, other association. */
EXPORT void orc_rule_conv_dweight_f32(const float *feature, const float *d_out,
                                      const int32_t *rules, const int32_t *rule_size,
                                      int ntile, int KV, int tile_n_max, int iC, int oC,
                                      float *d_weight)
{
    size_t wsz = (size_t)KV * iC * oC;
    memset(d_weight, 0, wsz * sizeof(float));
#pragma omp parallel
    {
        float *part = (float *)calloc(wsz, sizeof(float));
#pragma omp for schedule(dynamic, 32)
        for (int t = 0; t < ntile; t++)
            for (int k = 0; k < KV; k++) {
                int n = rule_size[t * KV + k];
                if (n > tile_n_max) n = tile_n_max;
                const int32_t *rin = rules + ((size_t)t * KV + k) * 2 * tile_n_max;
                const int32_t *rout = rin + tile_n_max;
                float *Wk = part + (size_t)k * iC * oC;
                for (int v = 0; v < n; v++) {
                    const float *a = feature + (size_t)rin[v] * iC;
                    const float *g = d_out + (size_t)rout[v] * oC;
                    for (int c = 0; c < iC; c++) {
                        float av = a[c];
                        float *w = Wk + (size_t)c * oC;
                        for (int o = 0; o < oC; o++) w[o] = fmaf(av, g[o], w[o]);
                    }
                }
            }
#pragma omp critical
        for (size_t i = 0; i < wsz; i++) d_weight[i] += part[i];
        free(part);
    }
}

/* ---------------------------------------------------------------------------
 * Quantised forward (int8 x int8 -> int32 accumulate -> int8).  The reference
 * has no integer path; the pair-sum is the reference's (rule_conv_kernel.cu.h:
 * 91-153) evaluated in exact integer arithmetic and the requantisation rule is
 * defined by this repository:
 *     q = clamp(rint((float)acc * scale[oc]), -128, 127)
 * with the int32->float conversion and the product rounded to nearest-even in
 * IEEE binary32 and rint() rounding half to even.  acc32 (optional) receives
 * the raw accumulators.
 * ------------------------------------------------------------------------- */
EXPORT void orc_rule_conv_i8(const int8_t *feature, const int8_t *weight, const float *scale,
                             const int32_t *rules, const int32_t *rule_size,
                             int ntile, int KV, int tile_n_max, int iC, int oC,
                             int out_nnz, int32_t *acc32, int8_t *out)
{
    int32_t *acc = acc32 ? acc32 : (int32_t *)malloc((size_t)out_nnz * oC * sizeof(int32_t));
    memset(acc, 0, (size_t)out_nnz * oC * sizeof(int32_t));
#pragma omp parallel for schedule(dynamic, 32)
    for (int t = 0; t < ntile; t++)
        for (int k = 0; k < KV; k++) {
            int n = rule_size[t * KV + k];
            if (n > tile_n_max) n = tile_n_max;
            const int32_t *rin = rules + ((size_t)t * KV + k) * 2 * tile_n_max;
            const int32_t *rout = rin + tile_n_max;
            const int8_t *Wk = weight + (size_t)k * iC * oC;
            for (int v = 0; v < n; v++) {
                const int8_t *a = feature + (size_t)rin[v] * iC;
                int32_t *d = acc + (size_t)rout[v] * oC;
                for (int c = 0; c < iC; c++) {
                    int32_t av = a[c];
                    const int8_t *w = Wk + (size_t)c * oC;
                    for (int o = 0; o < oC; o++) d[o] += av * (int32_t)w[o];
                }
            }
        }
#pragma omp parallel for schedule(static)
    for (int j = 0; j < out_nnz; j++)
        for (int o = 0; o < oC; o++) {
            volatile float prod = (float)acc[(size_t)j * oC + o] * scale[o];
            float r = rintf(prod);
            if (r < -128.f) r = -128.f;
            if (r > 127.f) r = 127.f;
            out[(size_t)j * oC + o] = (int8_t)r;
        }
    if (!acc32) free(acc);
}
