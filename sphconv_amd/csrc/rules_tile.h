// Device code of the rule kernels that more than one translation unit uses: the map of a tile's rows to their
// columns, the fiber join that fills the tile's neighbour table in LDS, and the compaction of that table into
// per-offset lists and groups of 16.  rules.hip wraps it into the kernel that writes a rule book; fused.hip into
// the kernel that goes on to convolve the tile without writing the book.
#pragma once
#include "common.h"
#include "pack.h"
#include "tile_consts.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;

struct Grid3 {
    int n0, n1, n2;
};

// Division of a 32-bit unsigned number by a divisor fixed per launch: a multiplication and two shifts with
// constants made on the host (Granlund and Montgomery's round-up method, exact for every 32-bit numerator),
// where the compiler's division by a run-time value is some thirty instructions in a row.
struct FastDiv {
    uint32_t mul, sh1, sh2;
};
inline FastDiv fast_div(uint32_t d)
{
    uint32_t l = 0;
    while ((1ull << l) < d) l++;
    const uint32_t m = (uint32_t)((((1ull << l) - d) << 32) / d + 1);
    return FastDiv{m, l < 1 ? l : 1, l < 1 ? 0 : l - 1};
}
__device__ __forceinline__ uint32_t div_by(uint32_t n, const FastDiv &f)
{
    const uint32_t t = __umulhi(f.mul, n);
    return (t + ((n - t) >> f.sh1)) >> f.sh2;
}

struct ConvParams {
    int K0, K1, K2;
    int s0, s1, s2;
    int p0, p1, p2;
};

__device__ __forceinline__ int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

// Row range [start, end) of column c, clamped to [0, rows] so that inconsistent
// caller data can never index outside the row arrays.
__device__ __forceinline__ void fiber_range(const int32_t *ptr, int c, int rows, int &start, int &end)
{
    end = clampi(ptr[c], 0, rows);
    start = c ? clampi(ptr[c - 1], 0, rows) : 0;
    if (start > end) start = end;
}

// Narrows down the first column c in [0, n) with a[c] > target (n if none): returns
// lo <= c with c - lo < max_span.  All kThreads threads of the block work together:
// every round probes kThreads evenly spaced positions of the remaining window, so a
// round cuts the window by a factor of kThreads.  (Probes are scattered, one cache
// line each, and cost far more in the vector memory path than the coalesced column
// walk that follows; hence few probes and an early stop.)  max_span = 1 gives the
// exact column.  s_first: 2 * kWaves LDS ints (the rounds alternate between the halves,
// so a round needs one barrier).  meanwhile() runs once, while the first round's probes are in flight,
// and in front of a barrier: the place for LDS initialisation.  Must be called by the whole block.
template <int NT, class F>
__device__ int block_upper_bound(const int32_t *a, int n, int target, int max_span, int *s_first, F &&meanwhile)
{
    int lo = 0, hi = n;
    const int tid = threadIdx.x;
    bool first = true;
    for (int round = 0; hi - lo >= max_span; round ^= 1) {
        int span = hi - lo;
        int step = (span + NT - 1) / NT;
        long pos = (long)lo + (long)tid * step;
        int val = (pos < hi) ? a[pos] : 0x7fffffff; // positions >= hi are known to exceed
        if (first) meanwhile();
        first = false;
        // first probe above the target: per wave by a ballot, over the waves through LDS
        const unsigned long long above = __ballot(val > target);
        int *mine = s_first + round * (NT / kWave);
        if ((tid & (kWave - 1)) == 0) mine[tid / kWave] = above ? (tid & ~(kWave - 1)) + __ffsll((long long)above) - 1 : NT;
        lds_barrier();
        int f = NT;
#pragma unroll
        for (int w = 0; w < (NT / kWave); w++) f = min(f, mine[w]);
        if (f == NT) {
            lo = lo + (NT - 1) * step + 1;
        } else {
            long nh = (long)lo + (long)f * step;
            int new_hi = nh < hi ? (int)nh : hi;
            int new_lo = (f == 0) ? lo : lo + (f - 1) * step + 1;
            hi = new_hi;
            lo = new_lo;
        }
    }
    if (first) { // no round at all
        meanwhile();
        lds_barrier();
    }
    return lo;
}

// ---------------------------------------------------------------------------
// Shared tail of the book builders: the block holds, in LDS, a table
// nbr[row_local * KV + k] = gathered row or -1 for the R rows of tile `tile`
// (first row r0; rows behind the tile's last one hold -1).  Emits the tile's
// groups: per k, rows in ascending order, 16 per group, last group padded with -1.
//   pass 1: a wave takes an offset k: two ballots over the column k of the table
//           give every row with a pair its rank in the k-list, and the row writes
//           its number into the list's place in LDS (sel[k][rank]);
//   scan  : first group of every k, and one descriptor word per group;
//   pass 2: one thread per output SLOT reads its group's descriptor, the row at its
//           rank and the row's table entry, and stores -- consecutive threads store
//           consecutive slots, so the book is written coalesced.
// A tile's time is the length of its waves' dependent chains (the same with one
// workgroup per CU as with three): every step above is a handful of instructions per
// item, batched so that the LDS round trips of several items overlap.
// ---------------------------------------------------------------------------
// Lives in dynamic LDS behind the neighbour table, sized by the kernel volume (a 3x3x3 kernel needs 4.5 KB
// where the largest volume needs 21 KB).
struct EmitScratch {
    int *cnt;           // [KV] pairs of offset k
    int *goff;          // [KV + 1] first group of offset k
    int *ginfo;         // [KV * (R / SPH_GROUP)] per group: k | rank of its first slot << 8 | cnt[k] << 16
    unsigned long long *rmask; // [2] rows of the tile that have a pair at the offset emit_lists was asked about, as a bit set
    unsigned char *sel; // [KV][R] rows of offset k's list
};
__host__ __device__ inline size_t emit_scratch_bytes(int KV)
{
    size_t b = (size_t)KV * sizeof(int) + (size_t)(KV + 1) * sizeof(int) + (size_t)KV * (R / SPH_GROUP) * sizeof(int);
    b = (b + 7) & ~(size_t)7;
    b += 2 * sizeof(unsigned long long) + (size_t)KV * R;
    b = (b + 7) & ~(size_t)7;
    // the compact copy of a tile's groups (compact_groups below) takes the same place
    const size_t compact = (size_t)64 * SPH_GROUP * 5 + 64;
    return b > compact ? b : compact;
}
// `base` must be 8-byte aligned.
__device__ __forceinline__ EmitScratch emit_scratch_at(void *base, int KV)
{
    EmitScratch sc;
    sc.cnt = (int *)base;
    sc.goff = sc.cnt + KV;
    sc.ginfo = sc.goff + KV + 1;
    sc.rmask = (unsigned long long *)(((uintptr_t)(sc.ginfo + KV * (R / SPH_GROUP)) + 7) & ~(uintptr_t)7);
    sc.sel = (unsigned char *)(sc.rmask + 2);
    return sc;
}

// Passes 1 and the scan: the per-offset lists (sc.sel, sc.cnt), the first group of every offset (sc.goff) and one
// descriptor per group (sc.ginfo) in LDS; returns the tile's number of groups.  kmask >= 0: the rows that have a
// pair at offset kmask go to sc.rmask as a bit set.  Ends behind a barrier.
template <int NT>
__device__ __forceinline__ int emit_lists(const int32_t *nbr, int KV, const EmitScratch &sc, int kmask = -1)
{
    static_assert(R == 128 && kWave == 64, "two ballots cover a tile's rows");
    static_assert(R / SPH_GROUP <= 8 && R <= 128, "a group descriptor packs k, a rank and a count into 8 bits each");
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;

    // a wave takes every (NT / kWave)-th offset, eight of them per round with all their table reads in flight together
    // (one LDS round trip per round instead of one per offset)
    constexpr int kEmitBatch = 8;
    for (int kb = wave; kb < KV; kb += (NT / kWave) * kEmitBatch) {
        int v_lo[kEmitBatch], v_hi[kEmitBatch];
#pragma unroll
        for (int q = 0; q < kEmitBatch; q++) {
            const int k = min(kb + q * (NT / kWave), KV - 1);
            v_lo[q] = nbr[lane * KV + k];
            v_hi[q] = nbr[(kWave + lane) * KV + k];
        }
#pragma unroll
        for (int q = 0; q < kEmitBatch; q++) {
            const int k = min(kb + q * (NT / kWave), KV - 1); // behind the last offset: the last one again, same values
            {
                const unsigned long long m0 = __ballot(v_lo[q] >= 0), m1 = __ballot(v_hi[q] >= 0);
                const int c0 = __popcll(m0);
                // set bits below this lane = the row's rank among the rows of its half
                const int b0 = __builtin_amdgcn_mbcnt_hi((unsigned)(m0 >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m0, 0));
                const int b1 = __builtin_amdgcn_mbcnt_hi((unsigned)(m1 >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m1, 0));
                unsigned char *list = sc.sel + k * R;
                if (v_lo[q] >= 0) list[b0] = (unsigned char)lane;
                if (v_hi[q] >= 0) list[c0 + b1] = (unsigned char)(kWave + lane);
                sc.cnt[k] = c0 + __popcll(m1); // every lane the same value
                if (k == kmask && lane < 2) sc.rmask[lane] = lane ? m1 : m0;
            }
        }
    }
    lds_barrier();
    if (wave == 0) {
        // exclusive scan of the per-offset group counts by one wave (KV <= 128: two passes)
        int carry = 0;
        for (int k0 = 0; k0 < KV; k0 += kWave) {
            const int k = k0 + lane;
            const int c = (k < KV) ? sc.cnt[k] : 0;
            const int v = (c + SPH_GROUP - 1) / SPH_GROUP;
            const int incl = wave_inclusive_sum(v);
            if (k < KV) {
                const int first = carry + incl - v;
                sc.goff[k] = first;
                for (int g = 0; g < v; g++) sc.ginfo[first + g] = k | (g * SPH_GROUP) << 8 | c << 16;
            }
            carry += __builtin_amdgcn_readlane(incl, kWave - 1);
        }
        if (lane == 0) sc.goff[KV] = carry;
    }
    lds_barrier();
    return sc.goff[KV];
}

// Pass 2: the tile's groups, group counts and offsets to the book in global memory, by the threads
// tid0, tid0 + nthreads, ... of the workgroup (all of them: tid0 = threadIdx.x, nthreads = kThreads).
__device__ __forceinline__ void emit_store(const int32_t *nbr, int r0, int KV, int tile, int cap, const EmitScratch &sc,
                                           const sph_book &book, int tid0, int nthreads)
{
    const int tid = tid0;
    if (tid == 0) book.tile_ngrp[tile] = sc.goff[KV];
    for (int k = tid; k <= KV; k += nthreads)
        book.tile_koff[(long)tile * (KV + 1) + k] = (uint16_t)sc.goff[k];
    const int ngrp = sc.goff[KV];
    const long gbase_tile = (long)tile * cap;
    int32_t *out_gather = book.grp_gather + gbase_tile * SPH_GROUP, *out_owner = book.grp_owner + gbase_tile * SPH_GROUP;
    // a thread's slots (slot, slot + kThreads, ...) four at a time: every step of the chain descriptor -> row ->
    // table entry is one LDS round trip for the four together
    constexpr int kEmitSlots = 4;
    const int nslots = ngrp * SPH_GROUP;
    for (int s0 = tid; s0 < nslots; s0 += nthreads * kEmitSlots) {
        int info[kEmitSlots], row[kEmitSlots], gat[kEmitSlots];
#pragma unroll
        for (int q = 0; q < kEmitSlots; q++) info[q] = sc.ginfo[min(s0 + q * nthreads, nslots - 1) / SPH_GROUP];
#pragma unroll
        for (int q = 0; q < kEmitSlots; q++) {
            // s0 and s0 + q * nthreads share their place in the group (nthreads is a multiple of the group size)
            const int k = info[q] & 0xff, j = ((info[q] >> 8) & 0xff) + (tid & (SPH_GROUP - 1));
            row[q] = j < (info[q] >> 16) ? sc.sel[k * R + j] : -1;
        }
#pragma unroll
        for (int q = 0; q < kEmitSlots; q++) gat[q] = nbr[max(row[q], 0) * KV + (info[q] & 0xff)];
#pragma unroll
        for (int q = 0; q < kEmitSlots; q++) {
            const int slot = s0 + q * nthreads;
            if (slot < nslots) {
                out_gather[slot] = row[q] >= 0 ? gat[q] : -1;
                out_owner[slot] = row[q] >= 0 ? r0 + row[q] : -1;
            }
        }
    }
    for (int g = tid; g < ngrp; g += nthreads) book.grp_k[gbase_tile + g] = sc.ginfo[g] & 0xff;
}

// The same pairs by stationary row, book.tile_nbr [tile][k][row of the tile], coalesced.
__device__ __forceinline__ void emit_nbr_store(const int32_t *nbr, int KV, int tile, const sph_book &book, int tid0, int nthreads)
{
    int32_t *dst = book.tile_nbr + (long)tile * KV * R;
    for (int i = tid0; i < KV * R; i += nthreads) {
        const int k = i / R, r = i - k * R;
        dst[i] = nbr[r * KV + k];
    }
}

// ---------------------------------------------------------------------------
// The tile's groups from the table straight to a compact copy in LDS, without lists (kernel volumes of up to 32,
// tiles of up to kCompactGroups groups).  A wave takes the offsets wave, wave + NW, ...: an offset's column of the
// table is two registers per lane (rows lane and lane + 64), two ballots count its pairs; behind one barrier every
// wave reads all counts and scans them in its own registers, so it knows where every offset's groups start, and a
// row's rank in its offset's list (the ballot bits below it) is its slot.  Rows ascending inside an offset, offsets
// ascending: the order emit_lists + emit_store produce, at two barriers instead of five and without the chain
// descriptor -> row -> table entry per slot.  k_last >= 0 puts that offset's groups behind all others (the
// one-launch kernel gives them to other waves); rows with a pair at k_last are reported in s_cov (two words).
// ---------------------------------------------------------------------------
constexpr int kCompactGroups = 64;
struct CompactGroups {
    int32_t *gat;            // [kCompactGroups * SPH_GROUP] gathered row or -1
    unsigned char *own, *gk; // [kCompactGroups * SPH_GROUP] owner row inside the tile; [kCompactGroups] offset of the group
};
__host__ __device__ inline size_t compact_bytes() { return (size_t)kCompactGroups * SPH_GROUP * 5 + kCompactGroups; }
__device__ __forceinline__ CompactGroups compact_at(void *base) // 16-byte aligned
{
    CompactGroups cg;
    cg.gat = (int32_t *)base;
    cg.own = (unsigned char *)(cg.gat + kCompactGroups * SPH_GROUP);
    cg.gk = cg.own + kCompactGroups * SPH_GROUP;
    return cg;
}
struct CompactInfo {
    int ngrp, n0, nc; // groups of the tile; of all offsets but k_last; of k_last (0 without one)
    int gc_lo;        // groups of the offsets below k_last
    int first;        // per lane: first group, in the book's order, of offset `lane`
    bool fits;        // ngrp <= kCompactGroups: the compact copy was written
};
template <int NT>
__device__ __forceinline__ CompactInfo compact_groups(const int32_t *nbr, int KV, int k_last, const CompactGroups &cg,
                                                      unsigned long long *s_cov)
{
    static_assert(R == 2 * kWave, "two ballots cover a tile's rows");
    constexpr int NW = NT / kWave;
    constexpr int KPW = (32 + NW - 1) / NW; // KV <= 32
    __shared__ int s_cnt[32];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    for (int i = tid; i < kCompactGroups * SPH_GROUP / 4; i += NT) ((int4 *)cg.gat)[i] = make_int4(-1, -1, -1, -1);
    int e_lo[KPW], e_hi[KPW];
#pragma unroll
    for (int i = 0; i < KPW; i++) {
        const int k = wave + NW * i;
        e_lo[i] = k < KV ? nbr[lane * KV + k] : -1;
        e_hi[i] = k < KV ? nbr[(lane + kWave) * KV + k] : -1;
    }
#pragma unroll
    for (int i = 0; i < KPW; i++) {
        const int k = wave + NW * i;
        const int c = __popcll(__ballot(e_lo[i] >= 0)) + __popcll(__ballot(e_hi[i] >= 0));
        if (lane == 0 && k < KV) s_cnt[k] = c;
    }
    lds_barrier();
    CompactInfo ci;
    const int mine = lane < KV ? (s_cnt[lane] + SPH_GROUP - 1) / SPH_GROUP : 0; // groups of offset `lane`
    const int incl = wave_inclusive_sum(lane == k_last ? 0 : mine);
    ci.nc = k_last >= 0 ? __builtin_amdgcn_readlane(mine, max(k_last, 0)) : 0;
    ci.n0 = __builtin_amdgcn_readlane(incl, kWave - 1);
    ci.ngrp = ci.n0 + ci.nc;
    ci.gc_lo = k_last >= 0 ? __builtin_amdgcn_readlane(incl, max(k_last, 0)) : ci.n0;
    ci.first = lane < k_last || k_last < 0 ? incl - mine : (lane == k_last ? ci.gc_lo : incl - mine + ci.nc);
    ci.fits = ci.ngrp <= kCompactGroups;
    if (!ci.fits) return ci;
    const int place = lane == k_last ? ci.n0 : incl - mine; // first group of offset `lane` in the compact copy
#pragma unroll
    for (int i = 0; i < KPW; i++) {
        const int k = wave + NW * i;
        if (k >= KV) break;
        const unsigned long long b_lo = __ballot(e_lo[i] >= 0), b_hi = __ballot(e_hi[i] >= 0);
        const int g0 = __builtin_amdgcn_readlane(place, k), ng = __builtin_amdgcn_readlane(mine, k);
        if (e_lo[i] >= 0) {
            const int d = g0 * SPH_GROUP + __builtin_amdgcn_mbcnt_hi((unsigned)(b_lo >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)b_lo, 0));
            cg.gat[d] = e_lo[i];
            cg.own[d] = (unsigned char)lane;
        }
        if (e_hi[i] >= 0) {
            const int d = g0 * SPH_GROUP + __popcll(b_lo) +
                          __builtin_amdgcn_mbcnt_hi((unsigned)(b_hi >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)b_hi, 0));
            cg.gat[d] = e_hi[i];
            cg.own[d] = (unsigned char)(lane + kWave);
        }
        if (lane < ng) cg.gk[g0 + lane] = (unsigned char)k;
        if (s_cov && k == k_last && lane == 0) {
            s_cov[0] = b_lo;
            s_cov[1] = b_hi;
        }
    }
    if (s_cov && ci.nc == 0 && tid < 2) s_cov[tid] = 0ull;
    lds_barrier();
    return ci;
}

// The book's part of a tile from its compact copy (compact_groups with ci.fits), by all NT threads: group p of the
// copy is the book's group p (offsets below k_last), p + nc (offsets above it) or p - n0 + gc_lo (k_last's own).
template <int NT>
__device__ __forceinline__ void compact_store(const CompactGroups &cg, const CompactInfo &ci, int k_last, int r0, int KV, int tile,
                                              int cap, const sph_book &book)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const long gbase = (long)tile * cap;
    if (tid < kWave) {
        uint16_t *koff = book.tile_koff + (long)tile * (KV + 1);
        if (lane < KV) koff[lane] = (uint16_t)ci.first;
        if (lane == 0) {
            koff[KV] = (uint16_t)ci.ngrp;
            book.tile_ngrp[tile] = ci.ngrp;
        }
    }
    for (int s = tid; s < ci.ngrp * SPH_GROUP; s += NT) {
        const int p = s / SPH_GROUP;
        const int g = p < ci.gc_lo ? p : (p < ci.n0 ? p + ci.nc : p - ci.n0 + ci.gc_lo);
        const int gi = cg.gat[s], d = g * SPH_GROUP + (s & (SPH_GROUP - 1));
        book.grp_gather[gbase * SPH_GROUP + d] = gi;
        book.grp_owner[gbase * SPH_GROUP + d] = gi >= 0 ? r0 + (int)cg.own[s] : -1;
        if ((s & (SPH_GROUP - 1)) == 0) book.grp_k[gbase + g] = cg.gk[p];
    }
}

// Everything the book keeps of one tile, from the table in LDS.
template <int NT>
__device__ __forceinline__ void emit_groups(const int32_t *nbr, int nrows, int r0, int KV, int tile, int cap,
                                            const EmitScratch &sc, const sph_book &book)
{
    if (book.tile_nbr) emit_nbr_store(nbr, KV, tile, book, threadIdx.x, NT);
    if (!book.grp_gather) return; // the caller keeps the pairs by row only: no groups, and no group counts either
    if (KV <= 32) {
        // the compact copy takes the place of the list scratch (and of the masks of the mask join behind it, which
        // the table no longer needs)
        const CompactGroups cg = compact_at(sc.cnt);
        const CompactInfo ci = compact_groups<NT>(nbr, KV, -1, cg, nullptr);
        if (ci.fits) { // workgroup-uniform
            compact_store<NT>(cg, ci, -1, r0, KV, tile, cap, book);
            return;
        }
        lds_barrier(); // the lists below overwrite what the other waves may still be counting from
    }
    emit_lists<NT>(nbr, KV, sc);
    emit_store(nbr, r0, KV, tile, cap, sc, book, threadIdx.x, NT);
}

// ---------------------------------------------------------------------------
// Book builder by fiber join.  One block per tile of R stationary rows.
//   1. map the tile's rows to their columns (block-wide search in q_ptr, then a
//      walk over the covering columns);
//   2. for every (row, k0, k1): locate the one column of the other grid that
//      can pair with it and compare its fiber entries' S2 coordinate;
//   3. emit_groups (the caller).
// TRANSPOSED = false: stationary rows are outputs, x_d = o_d*s_d - p_d + k_d.
// TRANSPOSED = true : stationary rows are inputs,  o_d = (x_d + p_d - k_d)/s_d.
// ---------------------------------------------------------------------------
struct BuildArgs {
    const int32_t *q_idx, *q_ptr; // stationary side
    const int32_t *p_idx, *p_ptr; // gathered side
    int q_rows, p_rows;
    int B;
    Grid3 Q, P;
    ConvParams cv;
    int cap;
    sph_book book;
    // optional passenger: workgroups behind the tile workgroups pack a weight (total == 0: none)
    SphPackJob pack;
    int tile_blocks;
    // gathered-side fibers are long (several entries on average) and their bins fit a 64-bit mask:
    // join through per-column occupancy masks instead of walking a fiber once per row
    int long_fibers;
    FastDiv by_q1, by_q01; // division by Q.n1 and by Q.n0 * Q.n1
    // optional: column of every stationary row (q_rows entries; what the producer of the coordinates knew when it
    // wrote them).  Null: the columns are searched for in q_ptr.  Every entry is checked against q_ptr before it is
    // believed, so a wrong table costs time and never changes the result.
    const int32_t *q_rowcol;
};

constexpr int kMaskCols = 32;  // distinct columns of a tile the mask join provides for
constexpr int kMaskWalk = 16;  // fiber entries fetched together when a mask is built

// Fills s_nbr[row of the tile * KV + k] = gathered row or -1 for tile `tile` (which must hold at least one row) by
// the whole workgroup of kThreads threads; returns behind a barrier.  s_masks: LDS for the mask join (used when
// a.long_fibers; kMaskCols * K0 * K1 * 12 bytes, 8-byte aligned).
// MASKS = false leaves the mask join (and its 3 KB of static LDS) out of the kernel.
template <bool TRANSPOSED, bool MASKS, int NT>
__device__ __forceinline__ void tile_table(const BuildArgs &a, int tile, int32_t *s_nbr, void *s_masks)
{
    __shared__ int s_col[R];
    __shared__ int s_first[2 * (NT / kWave)], s_flag[2];

    const int tid = threadIdx.x;
    const int KV = a.cv.K0 * a.cv.K1 * a.cv.K2;
    const int K01 = a.cv.K0 * a.cv.K1;
    const int r0 = tile * R;
    const int r1 = min(r0 + R, a.q_rows);
    const int nrows = r1 - r0;
    const int q_ncol = a.B * a.Q.n0 * a.Q.n1;

    // the tile's own S2 coordinates do not depend on the column search: fetch them first.  A row belongs to
    // the NT / R threads that share its number: each keeps the row's coordinates in registers.
    static_assert(NT % R == 0, "a thread's items must share a row");
    const int my_rl = tid & (R - 1);
    const int my_zz = (my_rl < nrows) ? a.q_idx[r0 + my_rl] : 0;

    // 1. rows -> columns.  The walk below tolerates starting early (columns before the
    // tile hold none of its rows), so the search stops once the window is below one
    // walk step: a single round of probes for grids of up to 131072 columns.
    // With a table of the rows' columns the search is one coalesced load; every entry is checked against the two
    // pointers that bound its column (for a submanifold layer the join below asks for the same two), and one entry
    // that fails sends the whole tile to the search.
    bool hinted = false;
    if (a.q_rowcol) {
        for (int i = tid; i < R * KV / 4; i += NT) ((int4 *)s_nbr)[i] = make_int4(-1, -1, -1, -1);
        const int r = r0 + my_rl;
        int c = my_rl < nrows ? a.q_rowcol[r] : 0;
        const bool inside = (unsigned)c < (unsigned)q_ncol;
        c = inside ? c : 0;
        const int pe = a.q_ptr[c], ps = c ? a.q_ptr[c - 1] : 0;
        const bool good = my_rl >= nrows || (inside && ps <= r && r < pe);
        const unsigned long long bad = __ballot(!good);
        if (tid < R) s_col[tid] = my_rl < nrows ? c : -1;
        if ((tid & (kWave - 1)) == 0) s_first[(NT / kWave) + tid / kWave] = bad != 0; // the half the search's first round leaves alone
        lds_barrier();
        int any_bad = 0;
#pragma unroll
        for (int w = 0; w < (NT / kWave); w++) any_bad |= s_first[(NT / kWave) + w];
        hinted = !any_bad;
    }
    constexpr int kWalk = 2 * NT; // columns per walk step, two consecutive ones per thread
    int c_first = q_ncol;
    if (!hinted)
        c_first = block_upper_bound<NT>(a.q_ptr, q_ncol, r0, kWalk, s_first, [&]() {
            for (int i = tid; i < R * KV / 4; i += NT) ((int4 *)s_nbr)[i] = make_int4(-1, -1, -1, -1); // R * KV is a multiple of 4
            for (int i = tid; i < R; i += NT) s_col[i] = -1;
        });
    bool done = (c_first >= q_ncol);
    for (int cb = c_first, step = 0; !done; cb += kWalk, step ^= 1) { // the steps alternate between two flags: one barrier each
        const int last = min(cb + kWalk - 1, q_ncol - 1);
        const int c = cb + 2 * tid;
        if (c <= last) {
            // q_ptr[c-1], q_ptr[c], q_ptr[c+1] bound the fibers of columns c and c+1
            int p0 = c ? clampi(a.q_ptr[c - 1], 0, a.q_rows) : 0;
            int p1 = clampi(a.q_ptr[c], 0, a.q_rows);
            int p2 = (c + 1 <= last) ? clampi(a.q_ptr[c + 1], 0, a.q_rows) : p1;
            if (p1 < p0) p1 = p0;
            if (p2 < p1) p2 = p1;
            for (int r = max(p0, r0); r < min(p1, r1); r++) s_col[r - r0] = c;
            for (int r = max(p1, r0); r < min(p2, r1); r++) s_col[r - r0] = c + 1;
            if (c == last || c + 1 == last) s_flag[step] = (p2 >= r1) || (last == q_ncol - 1);
        }
        lds_barrier();
        done = s_flag[step] != 0;
    }
    // the row's column -> (batch, S0, S1), by every thread for its own row
    const int my_c = my_rl < nrows ? s_col[my_rl] : -1;
    const bool my_ok = my_c >= 0;
    const int my_b = (int)div_by((uint32_t)max(my_c, 0), a.by_q01);
    const int my_rem = max(my_c, 0) - my_b * (a.Q.n0 * a.Q.n1);
    const int my_c0 = (int)div_by((uint32_t)my_rem, a.by_q1), my_c1 = my_rem - my_c0 * a.Q.n1;

    // 2a. join through masks (long fibers).  The tile's rows share few columns, and every row of
    // a column would walk the same K0*K1 fibers of the other grid: walk each (column, k0, k1)
    // fiber once into a 64-bit occupancy mask, then every (row, k0, k1, k2) is a bit test and a
    // popcount (position inside the sorted fiber).  A fiber that is not strictly ascending or
    // leaves the 64 bins sends the whole tile to the general join below.
    bool by_masks = false;
    if constexpr (MASKS) if (a.long_fibers) {
        unsigned long long *s_cmask = (unsigned long long *)s_masks; // [K01][ncols], ncols <= kMaskCols
        int *s_cstart = (int *)(s_cmask + kMaskCols * K01);
        __shared__ int s_b[R], s_c0[R], s_c1[R], s_z[R];
        __shared__ int s_cj[R], s_rep[R], s_bad;
        if (tid < R && my_ok) {
            s_b[tid] = my_b;
            s_c0[tid] = my_c0;
            s_c1[tid] = my_c1;
            s_z[tid] = my_zz;
        }
        __shared__ unsigned long long s_bal[R / kWave];
        const int lane = tid & (kWave - 1), wave = tid / kWave;
        if (tid == 0) s_bad = 0;
        bool head = false;
        if (tid < R) {
            head = tid < nrows && s_col[tid] >= 0 && (tid == 0 || s_col[tid] != s_col[tid - 1]);
            const unsigned long long bal = __ballot(head);
            if (lane == 0) s_bal[wave] = bal;
        }
        lds_barrier();
        int ncols = 0;
        for (int w = 0; w < R / kWave; w++) ncols += __popcll(s_bal[w]);
        if (tid < R) {
            int incl = __popcll(s_bal[wave] & ((2ull << lane) - 1ull)); // heads at or before this row
            for (int w = 0; w < wave; w++) incl += __popcll(s_bal[w]);
            const int cj = (tid < nrows && s_col[tid] >= 0) ? incl - 1 : -1;
            s_cj[tid] = cj;
            if (head) s_rep[cj] = tid;
        }
        lds_barrier();
        if (ncols > kMaskCols) ncols = 0; // short fibers after all: general join
        for (int it = tid; it < ncols * K01; it += NT) {
            const int k01 = it / ncols, cj = it - k01 * ncols;
            const int rr = s_rep[cj];
            const int k0 = k01 / a.cv.K1, k1 = k01 - k0 * a.cv.K1;
            bool ok = true;
            int y0, y1;
            if (!TRANSPOSED) {
                y0 = s_c0[rr] * a.cv.s0 - a.cv.p0 + k0;
                y1 = s_c1[rr] * a.cv.s1 - a.cv.p1 + k1;
            } else {
                int t0 = s_c0[rr] + a.cv.p0 - k0, t1 = s_c1[rr] + a.cv.p1 - k1;
                if (t0 < 0 || t1 < 0 || t0 % a.cv.s0 || t1 % a.cv.s1) ok = false;
                y0 = t0 / a.cv.s0;
                y1 = t1 / a.cv.s1;
            }
            if (y0 < 0 || y0 >= a.P.n0 || y1 < 0 || y1 >= a.P.n1) ok = false;
            unsigned long long m = 0;
            int st = 0;
            if (ok) {
                int e;
                fiber_range(a.p_ptr, (s_b[rr] * a.P.n0 + y0) * a.P.n1 + y1, a.p_rows, st, e);
                int prev = -1;
                bool bad = false;
                for (int e0 = st; e0 < e; e0 += kMaskWalk) {
                    int v[kMaskWalk];
#pragma unroll
                    for (int q = 0; q < kMaskWalk; q++) v[q] = a.p_idx[min(e0 + q, e - 1)];
#pragma unroll
                    for (int q = 0; q < kMaskWalk; q++)
                        if (e0 + q < e) {
                            if ((unsigned)v[q] >= 64u || v[q] <= prev) bad = true;
                            else m |= 1ull << v[q];
                            prev = v[q];
                        }
                }
                if (bad) s_bad = 1;
            }
            s_cmask[it] = m;
            s_cstart[it] = st;
        }
        lds_barrier();
        by_masks = s_bad == 0 && ncols > 0;
        const bool pow2_s2 = (a.cv.s2 & (a.cv.s2 - 1)) == 0;
        const int sh_s2 = __ffs(a.cv.s2) - 1;
        if (by_masks) {
            for (int it = tid; it < K01 * R; it += NT) {
                const int rl = it & (R - 1), k01 = it / R;
                const int cj = s_cj[rl];
                if (cj < 0) continue;
                const unsigned long long m = s_cmask[k01 * ncols + cj];
                if (!m) continue;
                const int st = s_cstart[k01 * ncols + cj], zz = s_z[rl];
                for (int k2 = 0; k2 < a.cv.K2; k2++) {
                    int v;
                    if (!TRANSPOSED) {
                        v = zz * a.cv.s2 - a.cv.p2 + k2;
                    } else {
                        const int t = zz + a.cv.p2 - k2;
                        if (pow2_s2) { // uniform: strides 1, 2, 4, ... need no division
                            if (t < 0 || (t & (a.cv.s2 - 1))) continue;
                            v = t >> sh_s2;
                        } else {
                            if (t < 0 || t % a.cv.s2) continue;
                            v = t / a.cv.s2;
                        }
                    }
                    if ((unsigned)v < 64u && ((m >> v) & 1ull))
                        s_nbr[rl * KV + k01 * a.cv.K2 + k2] = st + __popcll(m & ((1ull << v) - 1ull));
                }
            }
        }
    }

    // 2. join.  item = (k01, row), consecutive lanes take consecutive rows.  Per pass a
    // thread first issues the two fiber-bound loads of all its items, then the first
    // three S2 coordinates of every fiber, and only then compares; longer fibers finish
    // in a loop.
    // NT is a multiple of R, so a thread meets the same row in every item: what depends on the row
    // only is fetched from LDS and multiplied once, and an item costs a handful of integer operations
    // (k0 = k01 / K1 by a 16-bit reciprocal, exact for the k01 < 256 that a kernel volume <= 128 allows)
    const int my_a0 = TRANSPOSED ? my_c0 + a.cv.p0 : my_c0 * a.cv.s0 - a.cv.p0;
    const int my_a1 = TRANSPOSED ? my_c1 + a.cv.p1 : my_c1 * a.cv.s1 - a.cv.p1;
    const int my_col0 = my_b * a.P.n0;
    const int my_slot = my_rl * KV;
    const unsigned inv_k1 = (65536u + a.cv.K1 - 1) / a.cv.K1;
    const bool unit_stride = a.cv.s0 == 1 && a.cv.s1 == 1;
    const bool pow2_stride = (a.cv.s0 & (a.cv.s0 - 1)) == 0 && (a.cv.s1 & (a.cv.s1 - 1)) == 0;
    const int sh_s0 = __ffs(a.cv.s0) - 1, sh_s1 = __ffs(a.cv.s1) - 1;
    // (row, k0, k1) items a thread joins per pass, all loads of a pass in flight together: a 3x3x3 kernel in one pass
    constexpr int kJoinItems = NT >= 256 ? 5 : 9;
    for (int base = 0; !by_masks && base < K01 * R; base += NT * kJoinItems) {
        int ps[kJoinItems], len[kJoinItems], slot[kJoinItems];
        int raw_e[kJoinItems], raw_s[kJoinItems];
        bool ok[kJoinItems];
#pragma unroll
        for (int j = 0; j < kJoinItems; j++) {
            const int k01 = (base + j * NT + tid) / R;
            ok[j] = k01 < K01 && my_ok;
            const int k0 = (int)(((unsigned)k01 * inv_k1) >> 16), k1 = k01 - k0 * a.cv.K1;
            int y0, y1;
            if (!TRANSPOSED) {
                y0 = my_a0 + k0;
                y1 = my_a1 + k1;
            } else {
                y0 = my_a0 - k0;
                y1 = my_a1 - k1;
                if (y0 < 0 || y1 < 0) ok[j] = false;
                if (pow2_stride) { // uniform branches: shifts for strides 1, 2, 4, ..., divisions for the others
                    if ((y0 & (a.cv.s0 - 1)) || (y1 & (a.cv.s1 - 1))) ok[j] = false;
                    y0 >>= sh_s0;
                    y1 >>= sh_s1;
                } else if (!unit_stride) {
                    if (y0 % a.cv.s0 || y1 % a.cv.s1) ok[j] = false;
                    y0 /= a.cv.s0;
                    y1 /= a.cv.s1;
                }
            }
            if (y0 < 0 || y0 >= a.P.n0 || y1 < 0 || y1 >= a.P.n1) ok[j] = false;
            const int pc = ok[j] ? (my_col0 + y0) * a.P.n1 + y1 : 0;
            raw_e[j] = a.p_ptr[pc];
            raw_s[j] = pc ? a.p_ptr[pc - 1] : 0;
            slot[j] = my_slot + k01 * a.cv.K2;
        }
        int z0[kJoinItems], z1[kJoinItems], z2[kJoinItems];
#pragma unroll
        for (int j = 0; j < kJoinItems; j++) {
            int e = clampi(raw_e[j], 0, a.p_rows), st = clampi(raw_s[j], 0, a.p_rows);
            if (st > e) st = e;
            ps[j] = st;
            len[j] = ok[j] ? e - st : 0;
            z0[j] = z1[j] = z2[j] = 0;
            if (len[j] > 0) z0[j] = a.p_idx[st];
            if (len[j] > 1) z1[j] = a.p_idx[st + 1];
            if (len[j] > 2) z2[j] = a.p_idx[st + 2];
        }
#pragma unroll
        for (int j = 0; j < kJoinItems; j++) {
            // k2 of a gathered-side entry with S2 coordinate v: forward v is an input
            // coordinate (k2 = v - (z*s2 - p2)), transposed v is an output coordinate
            // (k2 = z + p2 - v*s2)
            const int off = TRANSPOSED ? my_zz + a.cv.p2 : -(my_zz * a.cv.s2 - a.cv.p2);
            const int mul = TRANSPOSED ? -a.cv.s2 : 1;
            if (len[j] > 0) { int k2 = off + mul * z0[j]; if (k2 >= 0 && k2 < a.cv.K2) s_nbr[slot[j] + k2] = ps[j]; }
            if (len[j] > 1) { int k2 = off + mul * z1[j]; if (k2 >= 0 && k2 < a.cv.K2) s_nbr[slot[j] + k2] = ps[j] + 1; }
            if (len[j] > 2) { int k2 = off + mul * z2[j]; if (k2 >= 0 && k2 < a.cv.K2) s_nbr[slot[j] + k2] = ps[j] + 2; }
            // longer fibers: four entries per round, their loads in flight together
            for (int e = 3; e < len[j]; e += 4) {
                int v[4];
#pragma unroll
                for (int q = 0; q < 4; q++) v[q] = a.p_idx[ps[j] + min(e + q, len[j] - 1)];
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int k2 = off + mul * v[q];
                    if (e + q < len[j] && k2 >= 0 && k2 < a.cv.K2) s_nbr[slot[j] + k2] = ps[j] + e + q;
                }
            }
        }
    }
    lds_barrier();
}

} // namespace
