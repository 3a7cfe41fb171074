// Rule (indice) generation for gfx950: output coordinates of a strided
// convolution and the rule book of (kernel offset, gathered row, owner row)
// triples, replacing the reference's dense [B,S0,S1,S2] position grid and
// atomic counters (src/sphconv/rules.cu) by fiber joins, wave ballots and
// prefix popcounts; the per-column output counts are scanned by a second kernel
// (scan.h: one pass over the counts, decoupled look-back between workgroups).
// All kernels are integer and HBM/latency bound.
#include "common.h"
#include "pack.h"
#include "scan.h"

#include <cstring>
#include <mutex>

#include "rules_tile.h"

namespace {

// Book builder: one workgroup per tile of R stationary rows (tile_table, then emit_groups); workgroups behind
// the tiles' pack a weight.
template <bool TRANSPOSED>
__global__ __launch_bounds__(kThreads) void build_book_kernel(BuildArgs a)
{
    extern __shared__ __attribute__((aligned(16))) int32_t s_nbr[]; // [R * KV], emit scratch, masks of the mask join
    const int tid = threadIdx.x;
    if ((int)blockIdx.x >= a.tile_blocks) {
        // a weight rides along with the rule generation: the copy needs a launch of its own
        // otherwise, which costs more than the copy
        sph_pack_element(a.pack, (long)(blockIdx.x - a.tile_blocks) * kThreads + tid);
        return;
    }
    const int tile = sph_xcd_tile(blockIdx.x, (a.q_rows + R - 1) / R);
    const int KV = a.cv.K0 * a.cv.K1 * a.cv.K2;
    const int r0 = tile * R;
    if (r0 >= a.q_rows) return; // grid is padded to a multiple of the XCD count
    tile_table<TRANSPOSED, true, kThreads>(a, tile, s_nbr, (char *)(s_nbr + R * KV) + emit_scratch_bytes(KV));
    emit_groups<kThreads>(s_nbr, min(R, a.q_rows - r0), r0, KV, tile, a.cap, emit_scratch_at(s_nbr + R * KV, KV), a.book);
}

// Book builder from a global neighbour table nbr[rows, KV] (used when the rules
// arrive in the reference's padded format).
__global__ __launch_bounds__(kThreads) void book_from_nbr_kernel(const int32_t *nbr, int rows, int KV,
                                                                 int cap, sph_book book)
{
    extern __shared__ __attribute__((aligned(16))) int32_t s_nbr[];
    const int tile = blockIdx.x;
    const int r0 = tile * R;
    const int nrows = min(R, rows - r0);
    for (int i = threadIdx.x; i < R * KV; i += kThreads) s_nbr[i] = i < nrows * KV ? nbr[(long)r0 * KV + i] : -1;
    lds_barrier();
    emit_groups<kThreads>(s_nbr, nrows, r0, KV, tile, cap, emit_scratch_at(s_nbr + R * KV, KV), book);
}

// Kernel volumes above 96 need more than 48 KB of dynamic LDS for the neighbour table.
template <typename K>
static int allow_lds(K kernel, size_t bytes, const char *who)
{
    if (bytes <= 48 * 1024) return SPH_OK;
    hipError_t e = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) {
        sph_set_error("%s: hipFuncSetAttribute(%zu bytes of LDS): %s", who, bytes, hipGetErrorString(e));
        return SPH_ERR_LAUNCH;
    }
    return SPH_OK;
}

// ---------------------------------------------------------------------------
// Output coordinates of a strided convolution.  One thread per output column:
// the set of active S2 bins of the column is the union, over the K0*K1 input
// columns that reach it, of the bins (z + p2 - k2)/s2.  Bins are collected as
// 64-bit masks, 64 bins per pass (one pass when O2 <= 64).
// ---------------------------------------------------------------------------
struct OutArgs {
    const int32_t *z_idx, *z_ptr;
    int in_rows;
    int B;
    Grid3 S, O;
    ConvParams cv;
};

// Bins of output column (b, o0, o1) inside chunk `chunk` that the input columns k01 = part,
// part + step, ... reach.
__device__ unsigned long long column_mask(const OutArgs &a, int b, int o0, int o1, int chunk, int part, int step)
{
    unsigned long long mask = 0;
    const int K01 = a.cv.K0 * a.cv.K1;
    const bool pow2 = (a.cv.s2 & (a.cv.s2 - 1)) == 0;
    const int sh2 = __ffs(a.cv.s2) - 1;
    for (int k01 = part; k01 < K01; k01 += step) {
        const int k0 = k01 / a.cv.K1, k1 = k01 - k0 * a.cv.K1;
        int x0 = o0 * a.cv.s0 - a.cv.p0 + k0;
        int x1 = o1 * a.cv.s1 - a.cv.p1 + k1;
        if (x0 < 0 || x0 >= a.S.n0 || x1 < 0 || x1 >= a.S.n1) continue;
        int pc = (b * a.S.n0 + x0) * a.S.n1 + x1;
        int ps, pe;
        fiber_range(a.z_ptr, pc, a.in_rows, ps, pe);
        // four entries of the fiber per round, their loads in flight together
        for (int e0 = ps; e0 < pe; e0 += 4) {
            int z[4];
#pragma unroll
            for (int q = 0; q < 4; q++) z[q] = a.z_idx[min(e0 + q, pe - 1)];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                if (e0 + q >= pe) continue;
                for (int k2 = 0; k2 < a.cv.K2; k2++) {
                    int t = z[q] + a.cv.p2 - k2;
                    int o2;
                    if (pow2) { // uniform: strides 1, 2, 4, ... need no division
                        if (t < 0 || (t & (a.cv.s2 - 1))) continue;
                        o2 = t >> sh2;
                    } else {
                        if (t < 0 || t % a.cv.s2) continue;
                        o2 = t / a.cv.s2;
                    }
                    if (o2 < a.O.n2 && (o2 >> 6) == chunk) mask |= 1ull << (o2 & 63);
                }
            }
        }
    }
    return mask;
}

// The same walk for the first NCH chunks of 64 bins at once (O2 <= 64 * NCH): the fibers are read once, not once
// per chunk.  The chunk of a bin is matched against constants, so the masks stay in registers.
template <int NCH>
__device__ __forceinline__ void column_masks(const OutArgs &a, int b, int o0, int o1, int part, int step,
                                             unsigned long long (&mask)[NCH])
{
#pragma unroll
    for (int c = 0; c < NCH; c++) mask[c] = 0;
    const int K01 = a.cv.K0 * a.cv.K1;
    const bool pow2 = (a.cv.s2 & (a.cv.s2 - 1)) == 0;
    const int sh2 = __ffs(a.cv.s2) - 1;
    for (int k01 = part; k01 < K01; k01 += step) {
        const int k0 = k01 / a.cv.K1, k1 = k01 - k0 * a.cv.K1;
        int x0 = o0 * a.cv.s0 - a.cv.p0 + k0;
        int x1 = o1 * a.cv.s1 - a.cv.p1 + k1;
        if (x0 < 0 || x0 >= a.S.n0 || x1 < 0 || x1 >= a.S.n1) continue;
        int pc = (b * a.S.n0 + x0) * a.S.n1 + x1;
        int ps, pe;
        fiber_range(a.z_ptr, pc, a.in_rows, ps, pe);
        for (int e0 = ps; e0 < pe; e0 += 4) {
            int z[4];
#pragma unroll
            for (int q = 0; q < 4; q++) z[q] = a.z_idx[min(e0 + q, pe - 1)];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                if (e0 + q >= pe) continue;
                for (int k2 = 0; k2 < a.cv.K2; k2++) {
                    int t = z[q] + a.cv.p2 - k2;
                    int o2;
                    if (pow2) {
                        if (t < 0 || (t & (a.cv.s2 - 1))) continue;
                        o2 = t >> sh2;
                    } else {
                        if (t < 0 || t % a.cv.s2) continue;
                        o2 = t / a.cv.s2;
                    }
                    if (o2 >= a.O.n2) continue;
                    const unsigned long long bit = 1ull << (o2 & 63);
                    const int ch = o2 >> 6;
#pragma unroll
                    for (int c = 0; c < NCH; c++) mask[c] |= ch == c ? bit : 0ull;
                }
            }
        }
    }
}

constexpr int kMaskChunks = 8;                   // chunks of 64 bins (O2 <= 512) up to which every column's masks are kept
constexpr long kMaskWordsMax = 1L << 24;         // ... and 64-bit mask words (128 MB) up to which they are kept at all
__host__ __device__ inline int mask_chunks(int O2) { return (O2 + 63) >> 6; }
inline bool keeps_masks(const sph_geom *g)
{
    const int nchunk = mask_chunks(g->O[2]);
    return nchunk <= kMaskChunks && (long)g->B * g->O[0] * g->O[1] * nchunk <= kMaskWordsMax;
}

constexpr int kColLanes = 16;                    // lanes that share one output column
constexpr int kCountCols = 16;                   // output columns per workgroup of the count kernel
constexpr int kCountThreads = kCountCols * kColLanes;

// OR over the 16 lanes of a column group (all 16 are active together).
__device__ __forceinline__ unsigned long long or_reduce16(unsigned long long m)
{
    unsigned lo = (unsigned)m, hi = (unsigned)(m >> 32);
#pragma unroll
    for (int off = 1; off < kColLanes; off <<= 1) {
        lo |= __shfl_xor(lo, off, kWave);
        hi |= __shfl_xor(hi, off, kWave);
    }
    return ((unsigned long long)hi << 32) | lo;
}

// Active bins of one output column, counted by its 16 lanes in one walk over the fibers that reach it; the
// masks of its nchunk <= NCH chunks go to masks[oc * nchunk + chunk] (masks may be null).
template <int NCH>
__device__ __forceinline__ int count_column(const OutArgs &a, int b, int o0, int o1, int part, unsigned long long *masks,
                                            int oc, int nchunk)
{
    unsigned long long m[NCH];
    column_masks<NCH>(a, b, o0, o1, part, kColLanes, m);
    int cnt = 0;
#pragma unroll
    for (int c = 0; c < NCH; c++) {
        m[c] = or_reduce16(m[c]);
        cnt += __popcll(m[c]);
        if (masks && part == 0 && c < nchunk) masks[(long)oc * nchunk + c] = m[c];
    }
    return cnt;
}

// Scratch of the output-coordinate kernels: the state of the scan of the counts (sph_scan, one 64-bit word per
// tile of 2048 columns) at its head, the columns' bin masks behind it.
inline long scan_state_ints(long ncol) { return (long)(sph_scan::state_bytes(ncol) / 4); }

// Per-column counts.  16 lanes share an output column (one input column (k0, k1) each, K0*K1 = 9 of them busy
// for a 3x3x3 kernel), so the fibers that reach a column are walked side by side and small grids still fill
// the chip.  The counts go to oz_ptr, which sph_scan then scans in place: a scan folded into this kernel
// (workgroups numbered by a ticket, decoupled look-back) was measured slower than the two kernels, because
// every workgroup then pays an atomic on the one ticket counter and same-address device-scope atomics queue
// at about 20 ns each, while the counting wants thousands of small workgroups (131 072 columns: 74 us with
// 2048 workgroups of 64 columns, 31 us with 256 of 512 columns, against 19 us here + 6 us of scan).
// `masks` (O2 <= 512 only, else null) keeps each column's bin masks for the fill kernel.
__global__ __launch_bounds__(kCountThreads) void outcoords_count_kernel(OutArgs a, int32_t *counts,
                                                                        unsigned long long *masks, int *scan_state,
                                                                        int scan_state_n)
{
    const int ncol = a.B * a.O.n0 * a.O.n1;
    const int tid = threadIdx.x;
    // the scan that follows on the stream finds its state cleared (saves the launch of a fill kernel)
    if (blockIdx.x == 0)
        for (int i = tid; i < scan_state_n; i += kCountThreads) scan_state[i] = 0;
    const int part = tid % kColLanes, cl = tid / kColLanes;
    const int oc = blockIdx.x * kCountCols + cl;
    if (oc >= ncol) return; // whole 16-lane groups leave together
    const int nchunk = mask_chunks(a.O.n2);
    const int b = oc / (a.O.n0 * a.O.n1);
    const int rem = oc - b * (a.O.n0 * a.O.n1);
    const int o0 = rem / a.O.n1, o1 = rem % a.O.n1;
    int cnt = 0;
    if (nchunk == 1) {
        cnt = count_column<1>(a, b, o0, o1, part, masks, oc, nchunk);
    } else if (nchunk <= 2) {
        cnt = count_column<2>(a, b, o0, o1, part, masks, oc, nchunk);
    } else if (nchunk <= 4) {
        cnt = count_column<4>(a, b, o0, o1, part, masks, oc, nchunk);
    } else if (nchunk <= kMaskChunks) {
        cnt = count_column<kMaskChunks>(a, b, o0, o1, part, masks, oc, nchunk);
    } else { // deeper grids: one walk per chunk, nothing kept
        for (int ch = 0; ch < nchunk; ch++) cnt += __popcll(or_reduce16(column_mask(a, b, o0, o1, ch, part, kColLanes)));
    }
    if (part == 0) counts[oc] = cnt;
}

// oz_ptr holds the inclusive scan of the counts; one thread writes the bins of one column.
__global__ __launch_bounds__(kThreads) void outcoords_fill_kernel(OutArgs a, const int32_t *oz_ptr, int32_t *oz_idx,
                                                                  int out_rows, const unsigned long long *masks,
                                                                  int32_t *row_cols)
{
    const int ncol = a.B * a.O.n0 * a.O.n1;
    const int oc = blockIdx.x * kThreads + threadIdx.x;
    if (oc >= ncol) return;
    int pos = oc ? oz_ptr[oc - 1] : 0;
    const int end = oz_ptr[oc];
    if (end <= pos) return;
    int b = oc / (a.O.n0 * a.O.n1);
    int rem = oc - b * (a.O.n0 * a.O.n1);
    int o0 = rem / a.O.n1, o1 = rem % a.O.n1;
    int nchunk = (a.O.n2 + 63) >> 6;
    for (int ch = 0; ch < nchunk; ch++) {
        unsigned long long m = masks ? masks[(long)oc * nchunk + ch] : column_mask(a, b, o0, o1, ch, 0, 1);
        while (m) {
            int bit = __ffsll((long long)m) - 1;
            if (pos < out_rows) {
                oz_idx[pos] = ch * 64 + bit;
                if (row_cols) row_cols[pos] = oc;
            }
            pos++;
            m &= m - 1;
        }
    }
}

// ---------------------------------------------------------------------------
// Conversions to / from the reference's padded rule tensors.
// ---------------------------------------------------------------------------
__global__ void fill_i32_kernel(int32_t *p, long n, int32_t v)
{
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    long stride = (long)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}

// nbr[owner * KV + k] = gather for every used slot of the book.
__global__ void nbr_from_book_kernel(sph_book book, int cap, int ntiles, int32_t *nbr)
{
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x; // slot index over ntiles*cap*16
    long total = (long)ntiles * cap * SPH_GROUP;
    if (i >= total) return;
    long grp = i / SPH_GROUP;
    int tile = (int)(grp / cap);
    int g = (int)(grp - (long)tile * cap);
    if (g >= book.tile_ngrp[tile]) return;
    int owner = book.grp_owner[i];
    if (owner < 0) return;
    nbr[(long)owner * book.KV + book.grp_k[grp]] = book.grp_gather[i];
}

// One thread per (reference tile, k).  The tile covers output columns
// [t0*T0, +T0) x [t1*T1, +T1) of every batch sample (debug_utils.h:37-42);
// walking b, o0, o1, row ascending yields the list in ascending output row,
// which for sorted fibers is also ascending input row.
template <bool FILL>
__global__ void padded_kernel(const int32_t *oz_ptr, int out_rows, int B, int O0, int O1, int T0, int T1,
                              int KV, const int32_t *nbr, int tile_n_max, int32_t *rule_size,
                              int32_t *rules)
{
    int tgw = (O1 + T1 - 1) / T1;
    int ntile = ((O0 + T0 - 1) / T0) * tgw;
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (long)ntile * KV) return;
    int t = (int)(i / KV), k = (int)(i - (long)t * KV);
    int t0 = t / tgw, t1 = t - t0 * tgw;
    int cnt = 0;
    for (int b = 0; b < B; b++)
        for (int o0 = t0 * T0; o0 < min((t0 + 1) * T0, O0); o0++)
            for (int o1 = t1 * T1; o1 < min((t1 + 1) * T1, O1); o1++) {
                int c = (b * O0 + o0) * O1 + o1;
                int s, e;
                fiber_range(oz_ptr, c, out_rows, s, e);
                for (int j = s; j < e; j++) {
                    int in = nbr[(long)j * KV + k];
                    if (in < 0) continue;
                    if (FILL && cnt < tile_n_max) {
                        long base = ((long)t * KV + k) * 2 * tile_n_max;
                        rules[base + cnt] = in;
                        rules[base + tile_n_max + cnt] = j;
                    }
                    cnt++;
                }
            }
    if (!FILL) rule_size[i] = cnt;
}

__global__ void nbr_from_padded_kernel(const int32_t *rules, const int32_t *rule_size, int ntile, int KV,
                                       int tile_n_max, int in_rows, int out_rows, int transposed,
                                       int32_t *nbr)
{
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x; // over ntile*KV*tile_n_max
    long total = (long)ntile * KV * tile_n_max;
    if (i >= total) return;
    long tk = i / tile_n_max;
    int v = (int)(i - tk * tile_n_max);
    int n = rule_size[tk];
    if (v >= n) return;
    int k = (int)(tk % KV);
    int in = rules[tk * 2 * tile_n_max + v];
    int out = rules[tk * 2 * tile_n_max + tile_n_max + v];
    if (in < 0 || in >= in_rows || out < 0 || out >= out_rows) return;
    if (!transposed)
        nbr[(long)out * KV + k] = in;
    else
        nbr[(long)in * KV + k] = out;
}

inline ConvParams conv_params(const sph_geom *g)
{
    return ConvParams{g->K[0], g->K[1], g->K[2], g->stride[0], g->stride[1], g->stride[2],
                      g->pad[0], g->pad[1], g->pad[2]};
}

inline int book_has_groups(const sph_book *b) { return b->grp_k && b->grp_gather && b->grp_owner; }

// the groups may be left out (all three arrays null) by a caller that keeps the pairs by row
inline int book_ok(const sph_book *b)
{
    return b && b->tile_ngrp && b->tile_koff && b->rows >= 0 && b->KV > 0 && b->KV <= SPH_MAX_KV &&
           (book_has_groups(b) || (b->tile_nbr && !b->grp_k && !b->grp_gather && !b->grp_owner));
}

} // namespace

// ---------------------------------------------------------------------------
// Entry points
// ---------------------------------------------------------------------------
static thread_local char g_err[512] = "";

void sph_set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

SPH_EXPORT const char *sph_last_error(void) { return g_err; }
SPH_EXPORT int sph_abi_version(void) { return 7; }
SPH_EXPORT int sph_book_tiles(int rows) { return rows <= 0 ? 0 : sph_div_up(rows, R); }
SPH_EXPORT int sph_book_cap(int KV) { return KV * (R / SPH_GROUP); }

SPH_EXPORT int sph_tile_n_max(const sph_geom *g, int T0, int T1, int nnz)
{
    SPH_REQUIRE(g && T0 > 0 && T1 > 0, SPH_ERR_ARG, "sph_tile_n_max: bad argument");
    // rules.cu:21-34
    int in0 = g->stride[0] * (T0 - 1) + g->K[0];
    int in1 = g->stride[1] * (T1 - 1) + g->K[1];
    double sparsity = (double)nnz / ((double)g->B * g->S[0] * g->S[1] * g->S[2]);
    double size = (double)g->B * in0 * in1 * g->S[2] * sparsity * 2;
    return (int)(size + 64) & ~15;
}

SPH_EXPORT int sph_num_tiles(const sph_geom *g, int T0, int T1)
{
    SPH_REQUIRE(g && T0 > 0 && T1 > 0, SPH_ERR_ARG, "sph_num_tiles: bad argument");
    return sph_div_up(g->O[0], T0) * sph_div_up(g->O[1], T1);
}

static int rules_build(const char *who, const int32_t *z_idx, const int32_t *z_ptr, int in_rows, const int32_t *oz_idx,
                       const int32_t *oz_ptr, int out_rows, const sph_geom *g, int transposed, const sph_book *book,
                       const int32_t *row_cols, const SphPackJob *pack, void *stream)
{
    SPH_REQUIRE(sph_geom_ok(g), SPH_ERR_ARG, "%s: bad geometry (kernel volume <= %d)", who, SPH_MAX_KV);
    SPH_REQUIRE(book_ok(book), SPH_ERR_ARG, "%s: bad book", who);
    SPH_REQUIRE(z_ptr && oz_ptr && in_rows >= 0 && out_rows >= 0, SPH_ERR_ARG, "%s: bad argument", who);
    SPH_REQUIRE((in_rows == 0 || z_idx) && (out_rows == 0 || oz_idx), SPH_ERR_ARG, "%s: null index array", who);
    const int KV = g->K[0] * g->K[1] * g->K[2];
    SPH_REQUIRE(book->KV == KV, SPH_ERR_ARG, "%s: book.KV %d != kernel volume %d", who, book->KV, KV);
    SPH_REQUIRE(book->rows == (transposed ? in_rows : out_rows), SPH_ERR_ARG,
                "%s: book.rows %d does not match the stationary side", who, book->rows);

    BuildArgs a;
    Grid3 S{g->S[0], g->S[1], g->S[2]}, O{g->O[0], g->O[1], g->O[2]};
    if (!transposed) {
        a.q_idx = oz_idx; a.q_ptr = oz_ptr; a.q_rows = out_rows; a.Q = O;
        a.p_idx = z_idx;  a.p_ptr = z_ptr;  a.p_rows = in_rows;  a.P = S;
    } else {
        a.q_idx = z_idx;  a.q_ptr = z_ptr;  a.q_rows = in_rows;  a.Q = S;
        a.p_idx = oz_idx; a.p_ptr = oz_ptr; a.p_rows = out_rows; a.P = O;
    }
    a.B = g->B;
    a.q_rowcol = row_cols;
    a.cv = conv_params(g);
    a.by_q1 = fast_div((uint32_t)a.Q.n1);
    a.by_q01 = fast_div((uint32_t)a.Q.n0 * (uint32_t)a.Q.n1);
    a.cap = sph_book_cap(KV);
    a.book = *book;
    const int nt = sph_book_tiles(book->rows);
    a.tile_blocks = book->rows > 0 ? sph_xcd_grid(nt) : 0;
    int pack_blocks = 0;
    if (pack) {
        a.pack = *pack;
        pack_blocks = (int)((pack->total + kThreads - 1) / kThreads);
    } else {
        a.pack.total = 0;
    }
    if (a.tile_blocks + pack_blocks == 0) return SPH_OK;
    size_t lds = (size_t)R * KV * sizeof(int32_t) + emit_scratch_bytes(KV);
    // masks pay when a fiber of the gathered side serves several rows: four entries on average
    const long p_cols = (long)a.B * a.P.n0 * a.P.n1;
    const size_t lds_masks = (size_t)kMaskCols * (g->K[0] * g->K[1]) * (sizeof(unsigned long long) + sizeof(int32_t));
    a.long_fibers = a.P.n2 <= 64 && (long)a.p_rows >= 4 * p_cols && lds + lds_masks <= 64 * 1024;
    if (a.long_fibers) lds += lds_masks;
    hipStream_t st = (hipStream_t)stream;
    int rc = transposed ? allow_lds(build_book_kernel<true>, lds, who) : allow_lds(build_book_kernel<false>, lds, who);
    if (rc) return rc;
    if (!transposed)
        hipLaunchKernelGGL(build_book_kernel<false>, dim3(a.tile_blocks + pack_blocks), dim3(kThreads), lds, st, a);
    else
        hipLaunchKernelGGL(build_book_kernel<true>, dim3(a.tile_blocks + pack_blocks), dim3(kThreads), lds, st, a);
    return sph_check_launch(who);
}

SPH_EXPORT int sph_rules_build(const int32_t *z_idx, const int32_t *z_ptr, int in_rows,
                               const int32_t *oz_idx, const int32_t *oz_ptr, int out_rows,
                               const sph_geom *g, int transposed, const sph_book *book,
                               const int32_t *row_cols, void *stream)
{
    return rules_build("sph_rules_build", z_idx, z_ptr, in_rows, oz_idx, oz_ptr, out_rows, g, transposed, book, row_cols,
                       nullptr, stream);
}

SPH_EXPORT int sph_rules_build_pack(const int32_t *z_idx, const int32_t *z_ptr, int in_rows,
                                    const int32_t *oz_idx, const int32_t *oz_ptr, int out_rows,
                                    const sph_geom *g, int transposed, const sph_book *book,
                                    const int32_t *row_cols,
                                    sph_dtype dt, const void *w, int KV, int kdim, int ndim, long stride_k,
                                    long stride_kk, long stride_n, void *packed, void *stream)
{
    int rc = sph_pack_args_ok("sph_rules_build_pack", dt, w, packed, KV, kdim, ndim);
    if (rc) return rc;
    const SphPackJob p = sph_pack_job(dt, w, KV, kdim, ndim, stride_k, stride_kk, stride_n, packed);
    return rules_build("sph_rules_build_pack", z_idx, z_ptr, in_rows, oz_idx, oz_ptr, out_rows, g, transposed, book,
                       row_cols, &p, stream);
}

SPH_EXPORT int sph_outcoords_blocks(const sph_geom *g)
{
    SPH_REQUIRE(sph_geom_ok(g), SPH_ERR_ARG, "sph_outcoords_blocks: bad geometry");
    return sph_div_up(g->B * g->O[0] * g->O[1], kThreads);
}

// int32 entries of the scratch the two calls share: the state of the scan of the counts (a ticket and one
// 64-bit status word per tile of 2048 columns) and, behind it, every column's masks of active bins (one 64-bit
// word per 64 bins) -- kept for grids of up to 512 bins and 128 MB of masks; deeper or larger grids keep none
// and the fill kernel walks the fibers again
SPH_EXPORT int sph_outcoords_state_ints(const sph_geom *g)
{
    SPH_REQUIRE(sph_geom_ok(g), SPH_ERR_ARG, "sph_outcoords_state_ints: bad geometry");
    return (int)scan_state_ints((long)g->B * g->O[0] * g->O[1]);
}

SPH_EXPORT int sph_outcoords_scratch_ints(const sph_geom *g)
{
    SPH_REQUIRE(sph_geom_ok(g), SPH_ERR_ARG, "sph_outcoords_scratch_ints: bad geometry");
    const long ncol = (long)g->B * g->O[0] * g->O[1];
    const int nchunk = mask_chunks(g->O[2]);
    const long n = scan_state_ints(ncol) + (keeps_masks(g) ? 2 * ncol * nchunk : 0);
    SPH_REQUIRE(n < 2147483647L, SPH_ERR_UNSUPPORTED, "sph_outcoords_scratch_ints: grid too large");
    return (int)n;
}

static unsigned long long *outcoords_masks(const sph_geom *g, int32_t *scratch)
{
    if (!keeps_masks(g)) return nullptr;
    return (unsigned long long *)(scratch + scan_state_ints((long)g->B * g->O[0] * g->O[1]));
}

static OutArgs out_args(const int32_t *z_idx, const int32_t *z_ptr, int in_rows, const sph_geom *g)
{
    OutArgs a;
    a.z_idx = z_idx; a.z_ptr = z_ptr; a.in_rows = in_rows; a.B = g->B;
    a.S = Grid3{g->S[0], g->S[1], g->S[2]};
    a.O = Grid3{g->O[0], g->O[1], g->O[2]};
    a.cv = conv_params(g);
    return a;
}

static int outcoords_count(const char *who, const int32_t *z_idx, const int32_t *z_ptr, int in_rows, const sph_geom *g,
                           int32_t *oz_ptr, int32_t *scratch, int32_t *total, void *stream)
{
    SPH_REQUIRE(sph_geom_ok(g), SPH_ERR_ARG, "%s: bad geometry", who);
    SPH_REQUIRE(z_ptr && oz_ptr && scratch && in_rows >= 0 && (in_rows == 0 || z_idx), SPH_ERR_ARG, "%s: null argument", who);
    SPH_REQUIRE((uintptr_t)scratch % 8 == 0, SPH_ERR_ARG, "%s: scratch must be 8-byte aligned", who);
    const long ncol = (long)g->B * g->O[0] * g->O[1];
    const unsigned nblocks = (unsigned)((ncol + kCountCols - 1) / kCountCols);
    hipLaunchKernelGGL(outcoords_count_kernel, dim3(nblocks), dim3(kCountThreads), 0, (hipStream_t)stream,
                       out_args(z_idx, z_ptr, in_rows, g), oz_ptr, outcoords_masks(g, scratch), (int *)scratch,
                       sph_scan::state_ints(ncol));
    int rc = sph_check_launch(who);
    if (rc) return rc;
    // counts -> inclusive scan in place; the last tile also writes the row count
    hipError_t e = sph_scan::launch<sph_scan::Plus, true>(oz_ptr, oz_ptr, ncol, scratch, 0, (hipStream_t)stream, total,
                                                          /*clear_state=*/false);
    if (e != hipSuccess) {
        sph_set_error("%s: scan: %s", who, hipGetErrorString(e));
        return SPH_ERR_LAUNCH;
    }
    return sph_check_launch(who);
}

SPH_EXPORT int sph_outcoords_count(const int32_t *z_idx, const int32_t *z_ptr, int in_rows,
                                   const sph_geom *g, int32_t *oz_ptr, int32_t *scratch,
                                   int32_t *total_dev, void *stream)
{
    return outcoords_count("sph_outcoords_count", z_idx, z_ptr, in_rows, g, oz_ptr, scratch, total_dev, stream);
}

// ---------------------------------------------------------------------------
// sph_outcoords_count for callers that cannot allocate: the scratch is an array of the library's own.
// Each GPU holds its own copy of the array at its own address, found once per device.
// ---------------------------------------------------------------------------
constexpr long kStaticCols = SPH_STATIC_MAX_COLUMNS; // output columns (B * O0 * O1) the library's own scratch provides for
constexpr long kStaticInts = 256 + 2 * (kStaticCols / sph_scan::kTile) + 2 * kStaticCols; // scan state (rounded up) + masks
static __device__ __align__(256) int32_t sph_static_scratch[kStaticInts]; // 8.0 MiB per GPU
constexpr int kMaxDevices = 64;
static int32_t *g_static_ptr[kMaxDevices];
static std::mutex g_static_mutex;

// device address of this GPU's copy of the array (the array's name is no device address in host code)
static int static_scratch_ptr(const char *who, int32_t **out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        sph_set_error("%s: hipGetDevice: %s (device %d)", who, hipGetErrorString(e), dev);
        return SPH_ERR_LAUNCH;
    }
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (!g_static_ptr[dev]) {
        int32_t *p = nullptr;
        e = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(sph_static_scratch));
        if (e != hipSuccess || !p) {
            sph_set_error("%s: hipGetSymbolAddress: %s", who, hipGetErrorString(e));
            return SPH_ERR_LAUNCH;
        }
        g_static_ptr[dev] = p;
    }
    *out = g_static_ptr[dev];
    return SPH_OK;
}

SPH_EXPORT int sph_outcoords_count_static(const int32_t *z_idx, const int32_t *z_ptr, int in_rows,
                                          const sph_geom *g, int32_t *oz_ptr, int32_t *total_dev,
                                          const int32_t **scratch_out, void *stream)
{
    const char *who = "sph_outcoords_count_static";
    SPH_REQUIRE(sph_geom_ok(g), SPH_ERR_ARG, "%s: bad geometry", who);
    const long ncol = (long)g->B * g->O[0] * g->O[1];
    // a column keeps one 64-bit mask per 64 bins of O2 (up to 512 bins; deeper grids keep none)
    const int nchunk = mask_chunks(g->O[2]);
    const long need = ncol * (nchunk <= kMaskChunks ? nchunk : 1);
    SPH_REQUIRE(need <= kStaticCols, SPH_ERR_UNSUPPORTED,
                "%s: %ld output columns (B*O0*O1) of %d bins need %ld mask words, the library's own scratch provides for "
                "%ld: use sph_outcoords_count with a scratch of the caller's", who, ncol, g->O[2], need, kStaticCols);
    int32_t *ptr = nullptr;
    int rc = static_scratch_ptr(who, &ptr);
    if (rc) return rc;
    rc = outcoords_count(who, z_idx, z_ptr, in_rows, g, oz_ptr, ptr, total_dev, stream);
    if (rc == SPH_OK && scratch_out) *scratch_out = ptr;
    return rc;
}

SPH_EXPORT int sph_outcoords_fill(const int32_t *z_idx, const int32_t *z_ptr, int in_rows,
                                  const sph_geom *g, const int32_t *scratch, int32_t *oz_ptr,
                                  int32_t *oz_idx, int out_rows, int32_t *row_cols, void *stream)
{
    SPH_REQUIRE(sph_geom_ok(g), SPH_ERR_ARG, "sph_outcoords_fill: bad geometry");
    SPH_REQUIRE(z_ptr && oz_ptr && scratch && out_rows >= 0 && (out_rows == 0 || oz_idx) &&
                    (in_rows == 0 || z_idx), SPH_ERR_ARG, "sph_outcoords_fill: null argument");
    const int nb = sph_outcoords_blocks(g);
    hipLaunchKernelGGL(outcoords_fill_kernel, dim3(nb), dim3(kThreads), 0, (hipStream_t)stream,
                       out_args(z_idx, z_ptr, in_rows, g), (const int32_t *)oz_ptr, oz_idx, out_rows,
                       (const unsigned long long *)outcoords_masks(g, (int32_t *)scratch), row_cols);
    return sph_check_launch("sph_outcoords_fill");
}

SPH_EXPORT int sph_rules_to_padded_count(const sph_book *fwd_book, const int32_t *oz_ptr,
                                         const sph_geom *g, int T0, int T1, int32_t *nbr,
                                         int32_t *rule_size, void *stream)
{
    SPH_REQUIRE(sph_geom_ok(g) && T0 > 0 && T1 > 0, SPH_ERR_ARG, "sph_rules_to_padded_count: bad geometry");
    SPH_REQUIRE(book_ok(fwd_book) && book_has_groups(fwd_book) && oz_ptr && nbr && rule_size, SPH_ERR_ARG,
                "sph_rules_to_padded_count: null argument (the book must hold its groups)");
    hipStream_t st = (hipStream_t)stream;
    const int KV = fwd_book->KV, rows = fwd_book->rows;
    const int nt = sph_book_tiles(rows), cap = sph_book_cap(KV);
    long n = (long)rows * KV;
    if (n > 0) {
        hipLaunchKernelGGL(fill_i32_kernel, dim3((unsigned)min((n + 255) / 256, 65535L)), dim3(256), 0, st, nbr, n, -1);
        long slots = (long)nt * cap * SPH_GROUP;
        hipLaunchKernelGGL(nbr_from_book_kernel, dim3((unsigned)((slots + 255) / 256)), dim3(256), 0, st,
                           *fwd_book, cap, nt, nbr);
    }
    long ntk = (long)sph_num_tiles(g, T0, T1) * KV;
    hipLaunchKernelGGL(padded_kernel<false>, dim3((unsigned)((ntk + 255) / 256)), dim3(256), 0, st, oz_ptr,
                       rows, g->B, g->O[0], g->O[1], T0, T1, KV, nbr, 0, rule_size, (int32_t *)nullptr);
    return sph_check_launch("sph_rules_to_padded_count");
}

SPH_EXPORT int sph_rules_to_padded_fill(const int32_t *oz_ptr, const sph_geom *g, int T0, int T1,
                                        const int32_t *nbr, int out_rows, int KV, int tile_n_max,
                                        int32_t *rules, void *stream)
{
    SPH_REQUIRE(sph_geom_ok(g) && T0 > 0 && T1 > 0 && tile_n_max > 0, SPH_ERR_ARG, "sph_rules_to_padded_fill: bad geometry");
    SPH_REQUIRE(oz_ptr && nbr && rules && out_rows >= 0, SPH_ERR_ARG, "sph_rules_to_padded_fill: null argument");
    hipStream_t st = (hipStream_t)stream;
    long ntk = (long)sph_num_tiles(g, T0, T1) * KV;
    long n = ntk * 2 * tile_n_max;
    hipLaunchKernelGGL(fill_i32_kernel, dim3((unsigned)min((n + 255) / 256, 65535L)), dim3(256), 0, st, rules, n, -1);
    hipLaunchKernelGGL(padded_kernel<true>, dim3((unsigned)((ntk + 255) / 256)), dim3(256), 0, st, oz_ptr,
                       out_rows, g->B, g->O[0], g->O[1], T0, T1, KV, nbr, tile_n_max, (int32_t *)nullptr, rules);
    return sph_check_launch("sph_rules_to_padded_fill");
}

SPH_EXPORT int sph_rules_from_padded(const int32_t *rules, const int32_t *rule_size, int ntile, int KV,
                                     int tile_n_max, int in_rows, int out_rows, int transposed,
                                     int32_t *nbr, const sph_book *book, void *stream)
{
    SPH_REQUIRE(rules && rule_size && nbr && book_ok(book), SPH_ERR_ARG, "sph_rules_from_padded: null argument");
    SPH_REQUIRE(ntile > 0 && KV > 0 && KV <= SPH_MAX_KV && tile_n_max > 0 && in_rows >= 0 && out_rows >= 0,
                SPH_ERR_ARG, "sph_rules_from_padded: bad size");
    const int rows = transposed ? in_rows : out_rows;
    SPH_REQUIRE(book->rows == rows && book->KV == KV, SPH_ERR_ARG, "sph_rules_from_padded: book does not match");
    if (rows == 0) return SPH_OK;
    hipStream_t st = (hipStream_t)stream;
    long n = (long)rows * KV;
    hipLaunchKernelGGL(fill_i32_kernel, dim3((unsigned)min((n + 255) / 256, 65535L)), dim3(256), 0, st, nbr, n, -1);
    long total = (long)ntile * KV * tile_n_max;
    hipLaunchKernelGGL(nbr_from_padded_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, rules,
                       rule_size, ntile, KV, tile_n_max, in_rows, out_rows, transposed, nbr);
    const int nt = sph_book_tiles(rows);
    const size_t lds = (size_t)R * KV * sizeof(int32_t) + emit_scratch_bytes(KV);
    int rc = allow_lds(book_from_nbr_kernel, lds, "sph_rules_from_padded");
    if (rc) return rc;
    hipLaunchKernelGGL(book_from_nbr_kernel, dim3(nt), dim3(kThreads), lds, st,
                       nbr, rows, KV, sph_book_cap(KV), *book);
    return sph_check_launch("sph_rules_from_padded");
}

// One thread per column writes the column's number to its rows.
static __global__ void row_columns_kernel(const int32_t *z_ptr, int ncol, int rows, int32_t *row_cols)
{
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= ncol) return;
    int e = z_ptr[c], s = c ? z_ptr[c - 1] : 0;
    e = e < rows ? e : rows;
    for (int r = s < 0 ? 0 : s; r < e; r++) row_cols[r] = c;
}

SPH_EXPORT int sph_row_columns(const int32_t *z_ptr, int ncol, int rows, int32_t *row_cols, void *stream)
{
    SPH_REQUIRE(z_ptr && ncol > 0 && rows >= 0 && (rows == 0 || row_cols), SPH_ERR_ARG, "sph_row_columns: bad argument");
    if (rows == 0) return SPH_OK;
    hipLaunchKernelGGL(row_columns_kernel, dim3((unsigned)sph_div_up(ncol, 256)), dim3(256), 0, (hipStream_t)stream, z_ptr,
                       ncol, rows, row_cols);
    return sph_check_launch("sph_row_columns");
}
