// Rule generation and forward convolution of one layer in ONE launch (sph_rules_conv).
//
// A tile's convolution needs only that tile's pairs, so the workgroup that has just built them in LDS
// (rules_tile.h: rows -> columns, fiber join, per-offset lists) goes straight on to convolve them
// (conv_wave.h: one wave, accumulators in LDS, MFMA per group of 16 pairs) instead of writing them to a book in
// global memory for a second kernel to read back: one launch less per uncached layer, no launch gap, none of the
// second kernel's start-up round trips, and the book's stores only when the caller wants the book kept (an
// indice_key that later layers share, a backward pass).  The reference needs three launches for the same work
// (prepareSubMGridKernel + getSubMRulesKernel, src/sphconv/rules.cu:339-384, then the convolution,
// src/sphconv/rule_conv.cu:171).
//
// LDS of a workgroup: region A holds the neighbour table and the list scratch while the rules are made and the
// accumulator tile afterwards; region B the tile's groups in compact form (gathered row, owner row, offset).  A
// tile with more groups than region B holds writes them to the book and convolves from there, as the two-kernel
// path would.
#include "common.h"
#include "pack.h"
#include "rules_tile.h"
#include "conv_wave.h"

namespace {

constexpr int kFusedGroups = kCompactGroups; // groups of a tile that region B holds (a LiDAR-like tile has 30 to 45)

struct FusedArgs {
    BuildArgs b;
    ConvArgs c;
    int nwtot;      // 16-column tiles of the output, padded to 1, 2 or 4
    int write_book; // also store the tile's groups (and the by-row table, if the book has one)
    int small_wg;   // two-wave workgroups (four fit a CU) whatever the tile count: for callers with scans in flight
};

inline size_t fused_region_a(int KV, int nwtot)
{
    const size_t acc = (size_t)(R + 1) * (nwtot * 16 + 4) * sizeof(uint32_t);
    const size_t tab = (size_t)R * KV * sizeof(int32_t) + emit_scratch_bytes(KV);
    return ((acc > tab ? acc : tab) + 15) & ~(size_t)15;
}
inline size_t fused_region_b() { return compact_bytes(); }


// NT threads per workgroup: 256 (four waves: more hands for the rule generation, at most three workgroups per CU
// by registers) or 128 (two waves: four workgroups per CU, for grids of more tiles than three per CU hold).
template <sph_dtype DT, int NS, int CT, bool MASKED, int NT>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(NT == 256 ? 3 : 2))) void rules_conv_kernel(FusedArgs fa, int region_a)
{
    extern __shared__ __attribute__((aligned(16))) uint32_t s_mem[];
    constexpr int NW = NT / kWave;
    constexpr int kRun = (R / SPH_GROUP + NW - 2) / (NW - 1); // groups of one offset per helper wave, at most
    const BuildArgs &b = fa.b;
    const ConvArgs &a = fa.c;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int tile = sph_xcd_tile(blockIdx.x, (b.q_rows + R - 1) / R);
    const int r0 = tile * R;
    if (r0 >= b.q_rows) return; // grid is padded to a multiple of the XCD count
    const int nrows = min(R, b.q_rows - r0);
    const int KV = b.cv.K0 * b.cv.K1 * b.cv.K2;

    int32_t *s_nbr = (int32_t *)s_mem;
    const EmitScratch sc = emit_scratch_at(s_nbr + R * KV, KV);
    int32_t *m_gat = (int32_t *)((char *)s_mem + region_a);
    unsigned char *m_own = (unsigned char *)(m_gat + kFusedGroups * SPH_GROUP);
    unsigned char *m_gk = m_own + kFusedGroups * SPH_GROUP;
    __shared__ unsigned long long s_cov[2];

    // 1. the tile's pairs: the table of (row, offset) -> gathered row
    tile_table<false, false, NT>(b, tile, s_nbr, nullptr);
    // 2. the groups, from the table straight to region B (compact_groups).  Those of the middle offset (in a
    // submanifold layer: every row's pair with itself, a run of eight full groups) go to the waves that would
    // otherwise wait, and are the first the tile is given: stored, not added.  Region B keeps them behind the
    // other groups.
    const int kc = KV / 2;
    const CompactGroups cg{m_gat, m_own, m_gk};
    const CompactInfo ci = compact_groups<NT>(s_nbr, KV, kc, cg, s_cov);
    int ngrp = ci.ngrp;
    const int n0 = ci.n0;
    const bool fits = ci.fits;
    if (fits && fa.write_book) {
        // the book is wanted too (a shared indice_key, a backward pass): region B holds all of it
        if (b.book.tile_nbr) emit_nbr_store(s_nbr, KV, tile, b.book, tid, NT);
        compact_store<NT>(cg, ci, kc, r0, KV, tile, b.cap, b.book);
    }
    if (!fits) {
        // the tile has more groups than region B holds: lists and group descriptors as build_book_kernel makes
        // them, stored to the book
        ngrp = emit_lists<NT>(s_nbr, KV, sc, kc);
        if (fa.write_book && b.book.tile_nbr) emit_nbr_store(s_nbr, KV, tile, b.book, tid, NT);
        emit_store(s_nbr, r0, KV, tile, b.cap, sc, b.book, tid, NT);
        // the conv wave reads the groups back from the book: the stores have left this CU once every wave has
        // waited for its own (the barrier below does), and the book's lines are in no cache of this CU yet
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
    }

    // 3. region A becomes the accumulator tile: the helper waves store the middle offset's products into it (and
    //    zero the rows that offset does not reach) while wave 0 requests its first rows and fragments;
    // 4. wave 0 adds the other groups one after the other.
    const int LDW = fa.nwtot * 16 + 4;
    if (fits) {
        if (wave == 0) {
            const LdsMeta meta{m_gat, m_own, m_gk, kFusedGroups, n0};
            conv_wave_groups<DT, NS, CT, MASKED>(a, fa.nwtot, meta, n0, s_mem, 0, lane, false, 1);
        } else {
            const LdsMeta meta{m_gat, m_own, m_gk, kFusedGroups, ngrp};
            conv_run_store<DT, NS, CT, MASKED, kRun>(a, fa.nwtot, meta, kc, n0 + wave - 1, NW - 1, ngrp, lane, s_mem, s_cov,
                                                     tid - kWave, NT - kWave);
            lds_barrier();
        }
    } else {
        for (int i = tid; i < (R + 1) * LDW / 4; i += NT) ((int4v *)s_mem)[i] = int4v{0, 0, 0, 0};
        lds_barrier();
        if (wave == 0) {
            const BookMeta meta(b.book, b.cap, tile, ngrp, r0, nrows, a.feat_rows);
            conv_wave_groups<DT, NS, CT, MASKED>(a, fa.nwtot, meta, ngrp, s_mem, 0, lane, false);
        }
    }
    lds_barrier();

    // 5. the tile goes to global memory once, by all threads, with the epilogue fused
    conv_wave_store<DT, CT>(a, fa.nwtot, s_mem, 0, r0, nrows, tid, NT);
}

template <sph_dtype DT, int NS, int CT, bool MASKED, int NT>
int launch_fused_nt(const FusedArgs &fa, int ntiles, hipStream_t st)
{
    const size_t ra = fused_region_a(fa.b.book.KV, fa.nwtot);
    const size_t lds = ra + fused_region_b();
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)rules_conv_kernel<DT, NS, CT, MASKED, NT>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) {
            sph_set_error("sph_rules_conv: hipFuncSetAttribute(%zu bytes of LDS): %s", lds, hipGetErrorString(e));
            return SPH_ERR_LAUNCH;
        }
    }
    hipLaunchKernelGGL((rules_conv_kernel<DT, NS, CT, MASKED, NT>), dim3(sph_xcd_grid(ntiles)), dim3(NT), lds, st, fa, (int)ra);
    return sph_check_launch("sph_rules_conv");
}

template <sph_dtype DT, int NS, int CT, bool MASKED>
int launch_fused(const FusedArgs &fa, int ntiles, hipStream_t st)
{
    // three workgroups of 256 threads per CU hold 768 tiles at once, four of 128 threads 1024 (and fp32 rows of 128
    // bytes into 64 columns do not fit the registers three workgroups leave a wave)
    if (fa.small_wg || ntiles > 768 || (DT == SPH_F32 && NS == 2 && CT == 4)) return launch_fused_nt<DT, NS, CT, MASKED, 128>(fa, ntiles, st);
    return launch_fused_nt<DT, NS, CT, MASKED, 256>(fa, ntiles, st);
}

template <sph_dtype DT, int NS, int CT>
int launch_fused_m(const FusedArgs &fa, int ntiles, hipStream_t st)
{
    if (fa.c.row_bytes < NS * 64) return launch_fused<DT, NS, CT, true>(fa, ntiles, st);
    return launch_fused<DT, NS, CT, false>(fa, ntiles, st);
}

template <sph_dtype DT, int NS>
int launch_fused_ct(const FusedArgs &fa, int ntiles, hipStream_t st)
{
    switch (fa.nwtot) {
    case 1: return launch_fused_m<DT, NS, 1>(fa, ntiles, st);
    case 2: return launch_fused_m<DT, NS, 2>(fa, ntiles, st);
    default: return launch_fused_m<DT, NS, 4>(fa, ntiles, st);
    }
}

template <sph_dtype DT>
int launch_fused_ns(const FusedArgs &fa, int ntiles, hipStream_t st)
{
    if (fa.c.nsteps == 1) return launch_fused_ct<DT, 1>(fa, ntiles, st);
    return launch_fused_ct<DT, 2>(fa, ntiles, st);
}

} // namespace


SPH_EXPORT int sph_rules_conv(const int32_t *z_idx, const int32_t *z_ptr, int in_rows, const int32_t *oz_idx,
                              const int32_t *oz_ptr, int out_rows, const sph_geom *g, const sph_book *book, int flags,
                              const int32_t *row_cols, sph_dtype dt, const void *feature, int kdim, const void *packed_w,
                              int ndim, const sph_epilogue *epi, void *out, void *stream)
{
    const char *who = "sph_rules_conv";
    SPH_REQUIRE(sph_geom_ok(g), SPH_ERR_ARG, "%s: bad geometry (kernel volume <= %d)", who, SPH_MAX_KV);
    SPH_REQUIRE(book && book->tile_ngrp && book->tile_koff && book->grp_k && book->grp_gather && book->grp_owner, SPH_ERR_ARG,
                "%s: the book must provide room for the groups (tiles that hold more than %d groups are convolved from it)",
                who, kFusedGroups);
    SPH_REQUIRE(z_ptr && oz_ptr && in_rows >= 0 && out_rows >= 0 && (in_rows == 0 || (z_idx && feature)) &&
                    (out_rows == 0 || (oz_idx && out)) && packed_w, SPH_ERR_ARG, "%s: null argument", who);
    SPH_REQUIRE((int)dt >= 0 && (int)dt <= 3, SPH_ERR_ARG, "%s: unknown dtype %d", who, (int)dt);
    SPH_REQUIRE(dt != SPH_I8 || (epi && epi->scale), SPH_ERR_ARG, "%s: int8 needs per-channel scales", who);
    const int KV = g->K[0] * g->K[1] * g->K[2];
    SPH_REQUIRE(book->KV == KV && book->rows == out_rows, SPH_ERR_ARG, "%s: the book is for %d offsets and %d rows, the call for %d and %d",
                who, book->KV, book->rows, KV, out_rows);
    SPH_REQUIRE(kdim > 0 && ndim > 0, SPH_ERR_ARG, "%s: bad channel count", who);
    if (out_rows == 0) return SPH_OK;

    const int es = sph_elem_size(dt);
    FusedArgs fa;
    ConvArgs &a = fa.c;
    a.feat = (const char *)feature;
    a.feat_rows = in_rows;
    a.kdim = kdim;
    a.row_bytes = kdim * es;
    a.wp = (const char *)packed_w;
    a.nsteps = sph_num_steps(dt, kdim);
    a.ndim = ndim;
    a.book = *book;
    a.cap = sph_book_cap(KV);
    a.scale = epi ? epi->scale : nullptr;
    a.shift = epi ? epi->shift : nullptr;
    a.relu = epi ? epi->relu : 0;
    a.out = (char *)out;
    a.aligned_in = (a.row_bytes % 16 == 0) && ((uintptr_t)feature % 16 == 0);
    a.aligned_out = ((ndim * es) % 16 == 0) && ((uintptr_t)out % 16 == 0);
    fa.nwtot = sph_pad_waves(ndim);
    fa.write_book = (flags & SPH_FUSED_WRITE_BOOK) != 0;
    fa.small_wg = (flags & SPH_FUSED_IN_FLIGHT) != 0;
    // what this kernel takes: whole 16-byte chunks of up to 128 bytes per row (with 256-byte rows the loop does not
    // fit the registers that three workgroups per CU leave a wave), up to 64 output columns, arrays below 2 GiB,
    // and a table of KV offsets per row that fits the accumulators' LDS
    const bool rows_ok = a.aligned_in && in_rows > 0 && (a.nsteps == 1 || a.nsteps == 2) &&
                         (double)in_rows * a.row_bytes < 2147483648.0 && in_rows < (1 << 24);
    SPH_REQUIRE(rows_ok && fa.nwtot <= 4 && KV <= 32 && (uintptr_t)packed_w % 16 == 0, SPH_ERR_UNSUPPORTED,
                "%s: takes rows of 16-byte multiples up to 128 bytes, up to 64 output columns and 32 kernel offsets: use "
                "sph_rules_build + sph_conv_apply", who);

    BuildArgs &b = fa.b;
    b.q_idx = oz_idx; b.q_ptr = oz_ptr; b.q_rows = out_rows; b.Q = Grid3{g->O[0], g->O[1], g->O[2]};
    b.p_idx = z_idx;  b.p_ptr = z_ptr;  b.p_rows = in_rows;  b.P = Grid3{g->S[0], g->S[1], g->S[2]};
    b.B = g->B;
    b.q_rowcol = row_cols;
    b.cv = ConvParams{g->K[0], g->K[1], g->K[2], g->stride[0], g->stride[1], g->stride[2], g->pad[0], g->pad[1], g->pad[2]};
    b.by_q1 = fast_div((uint32_t)b.Q.n1);
    b.by_q01 = fast_div((uint32_t)b.Q.n0 * (uint32_t)b.Q.n1);
    b.cap = a.cap;
    b.book = *book;
    b.pack.total = 0;
    b.tile_blocks = 0;
    b.long_fibers = 0;
    const int nt = sph_book_tiles(out_rows);
    hipStream_t st = (hipStream_t)stream;
    switch (dt) {
    case SPH_F32: return launch_fused_ns<SPH_F32>(fa, nt, st);
    case SPH_F16: return launch_fused_ns<SPH_F16>(fa, nt, st);
    case SPH_BF16: return launch_fused_ns<SPH_BF16>(fa, nt, st);
    default: return launch_fused_ns<SPH_I8>(fa, nt, st);
    }
}
