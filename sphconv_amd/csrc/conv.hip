// Gather-GEMM-scatter convolution for gfx950 (wave64, MFMA 16x16 tiles).
//
// Forward / dgrad (sph_conv_apply): the tile's pairs arrive as groups of 16 (one
// kernel offset per group).  Fast kernel (conv_wave_kernel): one wave owns a
// 128-row tile (x 64 output columns), gathers each group's 16 feature rows straight
// into MFMA operand registers (16 B per lane), multiplies by the pre-packed weight
// fragments of that offset and adds the result into its private LDS accumulator
// tile; the tile is written to HBM once, with the epilogue fused.  No barriers, no
// atomics, summation order fixed by the book.  conv_apply_kernel is the general
// fallback for unaligned or very long rows.  When the book also keeps its pairs by
// stationary row (dense neighbourhoods), conv_rows_kernel_* walks (offset, block of 16
// rows) steps with the accumulators in registers instead; with rows of up to 64 bytes and
// up to 32 output columns conv_rows_win_kernel does so from a copy of the gathered rows
// in LDS.
//
// wgrad (sph_conv_wgrad): work items are (kernel offset, chunk of 64 tiles, slice of 64
// groups); a wave gathers 32 pairs' rows with 16-byte loads into its own LDS area and
// reads MFMA operands with the pair index as the K dimension through transposing LDS
// reads; the [64,64] block stays in registers, one fp32 partial per workgroup, summed
// in a fixed order by a second kernel.  wgrad_kernel is the general fallback for rows
// that are not whole 16-byte chunks.
#include "common.h"
#include "pack.h"
#include "conv_wave.h"

#include <cstdlib>

namespace {

// ---------------------------------------------------------------------------
// Weight packing (layout and element copy: pack.h)
// ---------------------------------------------------------------------------
__global__ void pack_weight_kernel(SphPackJob p)
{
    sph_pack_element(p, (long)blockIdx.x * blockDim.x + threadIdx.x);
}

constexpr int kMetaGroups = 32; // groups whose indices are staged in LDS at a time

// General kernel (any row length and alignment; used when the rows are not a
// multiple of 16 bytes or longer than 256 bytes): NW waves per tile, wave w owns
// columns [16w, 16w+16), one group at a time, every wave gathers for itself.
// The MFMA is issued transposed: D^T[16 owner columns, 16 pairs] = W^T x A^T, so
// lane l ends up with columns 4*(l/16)..+3 of pair l%16.  NSTEP is always 0 (row
// length taken from the arguments).
template <sph_dtype DT, int NW, int NSTEP>
__global__ __launch_bounds__(NW * kWave) void conv_apply_kernel(ConvArgs a)
{
    typedef typename Traits<DT>::elem elem;
    typedef typename Traits<DT>::acc4 acc4;
    constexpr int LDW = NW * 16 + 4; // accumulator row stride in 32-bit words (16-byte multiple)
    extern __shared__ __attribute__((aligned(16))) uint32_t s_acc[]; // [R][LDW]
    __shared__ int s_k[kMetaGroups];
    __shared__ int2 s_meta[kMetaGroups * SPH_GROUP]; // (gathered row, owner row - r0)

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int tile = sph_xcd_tile(blockIdx.x, (a.book.rows + R - 1) / R);
    const int r0 = tile * R;
    if (r0 >= a.book.rows) return; // grid is padded to a multiple of the XCD count
    const int nrows = min(R, a.book.rows - r0);

    // each wave clears and later updates only its own 16 columns
    for (int i = lane; i < R * 4; i += kWave)
        *(int4v *)&s_acc[(i >> 2) * LDW + wave * 16 + (i & 3) * 4] = int4v{0, 0, 0, 0};

    const int ngrp = a.book.tile_ngrp[tile];
    const long gb0 = (long)tile * a.cap;
    const int acc_col = wave * 16 + (lane >> 4) * 4;
    const char *wlane = a.wp + (long)wave * (kWave * 16) + lane * 16;
    const long wstep = (long)NW * (kWave * 16);           // bytes between steps of one offset
    const int nsteps = NSTEP > 0 ? NSTEP : a.nsteps;

    for (int c0 = 0; c0 < ngrp; c0 += kMetaGroups) {
        const int nc = min(kMetaGroups, ngrp - c0);
        if (c0) __syncthreads(); // every wave is done with the previous chunk's indices
        for (int i = tid; i < nc * SPH_GROUP; i += NW * kWave) {
            int gi = a.book.grp_gather[(gb0 + c0) * SPH_GROUP + i];
            int rl = a.book.grp_owner[(gb0 + c0) * SPH_GROUP + i] - r0;
            if ((unsigned)rl >= (unsigned)nrows || (unsigned)gi >= (unsigned)a.feat_rows) gi = rl = -1;
            s_meta[i] = make_int2(gi, rl);
        }
        for (int i = tid; i < nc; i += NW * kWave) s_k[i] = a.book.grp_k[gb0 + c0 + i];
        __syncthreads();

        {
            for (int g = 0; g < nc; g++) {
                const int2 m = s_meta[g * SPH_GROUP + (lane & 15)];
                const char *wk = wlane + (long)s_k[g] * nsteps * wstep;
                acc4 d = {0, 0, 0, 0};
                for (int st = 0; st < nsteps; st++) {
                    int4v fa = load_a_frag<DT>(a, m.x, st, lane);
                    int4v fb = *(const int4v *)(wk + st * wstep);
                    d = mfma_step<DT>(fb, fa, d);
                }
                if (m.y >= 0) acc_add4<DT>(&s_acc[m.y * LDW + acc_col], d);
            }
        }
    }
    __syncthreads();

    // epilogue: LDS tile -> out rows [r0, r0+nrows), all ndim columns
    elem *out = (elem *)a.out + (long)r0 * a.ndim;
    constexpr int VE = 16 / (int)sizeof(elem);
    if (a.aligned_out) {
        const int cpr = a.ndim / VE; // 16-byte chunks per row
        for (int i = tid; i < nrows * cpr; i += NW * kWave) {
            int row = i / cpr, ch = i - row * cpr;
            union { int4v v; elem e[VE]; } u;
#pragma unroll
            for (int j = 0; j < VE; j++)
                u.e[j] = to_elem<DT>(epilogue_value<DT>(a, s_acc[row * LDW + ch * VE + j], ch * VE + j));
            *(int4v *)(out + (long)row * a.ndim + ch * VE) = u.v;
        }
    } else {
        for (int i = tid; i < nrows * a.ndim; i += NW * kWave) {
            int row = i / a.ndim, c = i - row * a.ndim;
            out[i] = to_elem<DT>(epilogue_value<DT>(a, s_acc[row * LDW + c], c));
        }
    }
}

// ---------------------------------------------------------------------------

template <sph_dtype DT, int NS, int CT, bool MASKED>
__global__ __launch_bounds__(128) void conv_wave_kernel(ConvArgs a, int nwtot)
{
    extern __shared__ __attribute__((aligned(16))) uint32_t s_acc[]; // [R + 1][LDW]
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;              // block of CT*16 columns
    const int tile = sph_xcd_tile(blockIdx.x, (a.book.rows + R - 1) / R);
    const int r0 = tile * R;
    if (r0 >= a.book.rows) return;
    const int nrows = min(R, a.book.rows - r0);
    const int col0 = wave * CT * 16;           // first column of this wave
    const int ngrp = min(max(a.book.tile_ngrp[tile], 0), a.cap);
    const BookMeta meta(a.book, a.cap, tile, ngrp, r0, nrows, a.feat_rows);
    conv_wave_groups<DT, NS, CT, MASKED>(a, nwtot, meta, ngrp, s_acc, col0, lane, true);
    conv_wave_store<DT, CT>(a, nwtot, s_acc, col0, r0, nrows, lane, kWave);
}

// The same with two helper waves per tile (up to 64 output columns, rows of up to 128 bytes).  A submanifold book
// has a run of up to eight full groups at the middle offset (every row's pair with itself), which all use one set
// of weight fragments: the helper waves load those fragments once, take the run's groups between them, multiply
// from zero and store the products to the owners' accumulator rows behind wave 0's clear and before its first
// sum, while wave 0's first rows and fragments are on their way.  Wave 0's chain is then the tile's other groups
// only (26 instead of 34 at LiDAR sparsity), and the run costs 8 fragment loads instead of 64.  A tile whose middle
// offset holds fewer than two groups (strided books) is wave 0's alone, and the helper waves leave at once.
constexpr int kRunHelpers = 2;
template <sph_dtype DT, int NS, int CT, bool MASKED>
__global__ __launch_bounds__(kWave * (1 + kRunHelpers)) __attribute__((amdgpu_waves_per_eu(3))) void conv_wave_run_kernel(ConvArgs a, int nwtot)
{
    extern __shared__ __attribute__((aligned(16))) uint32_t s_acc[]; // [R + 1][LDW]
    constexpr int kRun = (R / SPH_GROUP + kRunHelpers - 1) / kRunHelpers;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int tile = sph_xcd_tile(blockIdx.x, (a.book.rows + R - 1) / R);
    const int r0 = tile * R;
    if (r0 >= a.book.rows) return;
    const int nrows = min(R, a.book.rows - r0);
    const int KV = a.book.KV, kc = KV / 2;
    const int ngrp = min(max(a.book.tile_ngrp[tile], 0), a.cap);
    const unsigned short *ko = a.book.tile_koff + (long)tile * (KV + 1) + kc;
    const int run_lo = min((int)ko[0], ngrp);
    const int run_n = min(max((int)ko[1] - run_lo, 0), min(ngrp - run_lo, R / SPH_GROUP));
    const bool shared = run_n >= 2; // workgroup-uniform
    if (wave == 0) {
        const BookMeta meta(a.book, a.cap, tile, shared ? ngrp - run_n : ngrp, r0, nrows, a.feat_rows, run_lo, shared ? run_n : 0);
        conv_wave_groups<DT, NS, CT, MASKED>(a, nwtot, meta, meta.ngrp, s_acc, 0, lane, true, shared ? 2 : 0);
    } else {
        if (!shared) return;
        const BookMeta meta(a.book, a.cap, tile, ngrp, r0, nrows, a.feat_rows);
        conv_run_store<DT, NS, CT, MASKED, kRun>(a, nwtot, meta, kc, run_lo + wave - 1, kRunHelpers, run_lo + run_n, lane, s_acc,
                                                 nullptr, -1, 0, true);
        lds_barrier();
    }
    if (shared) { // the helper waves have waited for the tile: all three write it out
        lds_barrier();
        conv_wave_store<DT, CT>(a, nwtot, s_acc, 0, r0, nrows, tid, kWave * (1 + kRunHelpers));
    } else {
        conv_wave_store<DT, CT>(a, nwtot, s_acc, 0, r0, nrows, lane, kWave);
    }
}

// ---------------------------------------------------------------------------
// Walk by stationary row (book.tile_nbr): for dense neighbourhoods.
//
// The grouped kernel above pays per group of 16 pairs (weight fragments through the L1,
// an LDS read-modify-write of the owners' accumulators), which is the right price when a
// row has two or three pairs.  From about ten pairs per row upwards it is cheaper to take
// every (offset, block of 16 consecutive rows) in turn, whatever it holds: the 16 gathered
// rows (zeros where a row has no pair at this offset) times the offset's weight, added to
// accumulators that never leave the registers (8 blocks x 64 columns = 128 per lane).
// 27 weight loads per tile instead of one per group, no accumulators in LDS, no owner
// indirection; the price is one MFMA step per (offset, block) even when it is nearly empty.
// One wave per tile and 64 output columns.  The tile's table is staged in LDS; gathers are
// requested two to four stages (of 4 sixteen-byte chunks per lane) ahead of their use.
// Measured at 64->64 fp16 on a full grid: 164 us against 387 us by groups; without any
// load the same instruction stream takes 91 us, twice what its MFMAs alone need (independent
// 16x16x32 MFMAs issue every 16 cycles): a stage's selects, LDS exchange and waits are in
// series with its MFMAs, and two waves per SIMD do not cover them.
// ---------------------------------------------------------------------------
// WS = waves that share a tile's rows (1, or 4 when the grid has fewer tiles than the chip has SIMDs: the
// kernel then lasts as long as one wave's chain of KV * 8 steps, and four waves with two blocks each
// shorten it).
template <sph_dtype DT, int NS, int CT, bool MASKED, int WS>
__device__ __forceinline__ void conv_rows_body(const ConvArgs &a, int nwtot)
{
    typedef typename Traits<DT>::elem elem;
    typedef typename Traits<DT>::acc4 acc4;
    constexpr int NB = R / SPH_GROUP / WS; // blocks of 16 rows per wave
    constexpr int BPS0 = NS >= 4 ? 1 : 4 / NS;
    constexpr int BPS = BPS0 < NB ? BPS0 : NB; // blocks per stage: a stage gathers up to 4 sixteen-byte chunks per lane
    constexpr int SPK = NB / BPS;         // stages per offset
    // measured: 128-byte rows want four stages of gathers in flight and one set of weight registers; 64-byte
    // rows (few MFMAs per stage) two stages and the next offset's weights requested an offset ahead; a
    // wave that takes a quarter of the rows has the registers for four offsets of weights
    constexpr int D = (NS >= 2 || WS > 1) ? 4 : 2; // stages in flight
    constexpr int KW = WS > 1 ? 4 / SPK : (NS >= 2 ? 1 : 2); // sets of weight fragment registers
    constexpr int U = (D > SPK * KW) ? D : SPK * KW; // stages per unrolled round (all powers of two)
    extern __shared__ __attribute__((aligned(16))) int32_t s_nb[]; // [KV][R] gathered row or -1

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave / WS;         // block of CT*16 columns
    const int part = (tid / kWave) % WS;       // which blocks of the tile
    const int blk0 = part * NB;
    const int tile = sph_xcd_tile(blockIdx.x, (a.book.rows + R - 1) / R);
    const int r0 = tile * R;
    if (r0 >= a.book.rows) return; // whole workgroups leave: no barrier is missed
    const int nrows = min(R, a.book.rows - r0);
    const int col0 = wave * CT * 16;
    const int KV = a.book.KV;
    const int S = KV * SPK;
    const char *wlane = a.wp + ((long)(wave * CT)) * (kWave * 16) + lane * 16;
    const long wstep = (long)nwtot * (kWave * 16);

    // the tile's table goes to LDS once (validated on the way): every stage then finds its rows
    // with one LDS read per block instead of a dependent global load
    {
        const int4v *src = (const int4v *)(a.book.tile_nbr + (long)tile * KV * R);
        for (int i = tid; i < KV * R / 4; i += blockDim.x) {
            int4v v = src[i];
            v.x = (unsigned)v.x < (unsigned)a.feat_rows ? v.x : -1;
            v.y = (unsigned)v.y < (unsigned)a.feat_rows ? v.y : -1;
            v.z = (unsigned)v.z < (unsigned)a.feat_rows ? v.z : -1;
            v.w = (unsigned)v.w < (unsigned)a.feat_rows ? v.w : -1;
            ((int4v *)s_nb)[i] = v;
        }
    }
    __syncthreads();

    // Gathers are requested with the four lanes of a quad on the four 16-byte chunks of ONE row's 64-byte
    // step (one tag look-up per quad; with a lane per row of the MFMA layout every quad would touch four
    // rows).  They reach the MFMA layout (lane = pair + 16 * chunk) through a wave-private LDS buffer:
    // [chunk set][16 rows][80 bytes] (the 16-byte pad makes both the write and the read conflict-free).
    // With 64-byte rows (one step) the exchange costs more than the look-ups it saves: there a lane loads
    // its MFMA operand directly.
    constexpr bool QUAD = NS >= 2;
    constexpr int kTrRow = 80, kTrSet = SPH_GROUP * kTrRow;
    char *tr = (char *)(s_nb + KV * R) + (tid / kWave) * (BPS * NS * kTrSet);
    int4v fa[D][BPS][NS], fw[KW][NS][CT];
    int rq[D][BPS];
    acc4 acc[NB][CT];
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
        for (int c = 0; c < CT; c++) acc[j][c] = acc4{0, 0, 0, 0};

    // stage s = (k, q): offset k = s / SPK, blocks q*BPS .. q*BPS+BPS-1 of the tile, every 64-byte step of
    // their rows; stages past the end re-read the last offset
    auto issue = [&](int s, int q, int4v (&f)[BPS][NS], int (&rows)[BPS]) {
        const int k = min(s / SPK, KV - 1);
#pragma unroll
        for (int j = 0; j < BPS; j++) {
            rows[j] = s_nb[k * R + (blk0 + q * BPS + j) * SPH_GROUP + (QUAD ? lane >> 2 : lane & 15)];
            const char *row = a.feat + (long)max(rows[j], 0) * a.row_bytes;
#pragma unroll
            for (int st = 0; st < NS; st++) {
                const int off = st * 64 + (QUAD ? lane & 3 : lane >> 4) * 16;
                f[j][st] = *(const int4v *)(row + (off < a.row_bytes ? off : 0));
            }
        }
    };
    auto load_w = [&](int k, int4v (&w)[NS][CT]) {
        const char *wk = wlane + (long)min(k, KV - 1) * NS * wstep;
#pragma unroll
        for (int st = 0; st < NS; st++)
#pragma unroll
            for (int c = 0; c < CT; c++) w[st][c] = *(const int4v *)(wk + st * wstep + (long)c * (kWave * 16));
    };

#pragma unroll
    for (int p = 0; p < KW; p++) load_w(p, fw[p]);
#pragma unroll
    for (int u = 0; u < D; u++) issue(u, u % SPK, fa[u], rq[u]);
    for (int s0 = 0; s0 < S; s0 += U) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int s = s0 + u;
            const int d = u % D, q = u % SPK, p = (u / SPK) % KW; // compile-time after unrolling
            __builtin_amdgcn_sched_barrier(0);
            if (s < S) {
                // zeros for rows without a pair and beyond the row's end; quad layout -> LDS -> MFMA layout
                int4v x[BPS][NS];
#pragma unroll
                for (int j = 0; j < BPS; j++)
#pragma unroll
                    for (int st = 0; st < NS; st++) {
                        bool live = rq[d][j] >= 0;
                        if constexpr (MASKED) live = live && (st * 64 + (QUAD ? lane & 3 : lane >> 4) * 16 < a.row_bytes);
                        x[j][st] = live ? fa[d][j][st] : int4v{0, 0, 0, 0};
                        if constexpr (QUAD)
                            *(int4v *)(tr + (j * NS + st) * kTrSet + (lane >> 2) * kTrRow + (lane & 3) * 16) = x[j][st];
                    }
                if constexpr (QUAD) {
                    asm volatile("" ::: "memory"); // other lanes' chunks: keep the reads behind the writes
#pragma unroll
                    for (int j = 0; j < BPS; j++)
#pragma unroll
                        for (int st = 0; st < NS; st++)
                            x[j][st] = *(const int4v *)(tr + (j * NS + st) * kTrSet + (lane & 15) * kTrRow + (lane >> 4) * 16);
                }
                asm volatile("" ::: "memory");
#pragma unroll
                for (int j = 0; j < BPS; j++)
#pragma unroll
                    for (int st = 0; st < NS; st++)
#pragma unroll
                        for (int c = 0; c < CT; c++)
                            acc[q * BPS + j][c] = mfma_step<DT>(fw[p][st][c], x[j][st], acc[q * BPS + j][c]);
            }
            __builtin_amdgcn_sched_barrier(0);
            // the offset is done: its weight registers take the fragments of offset k + KW; the row buffers
            // just consumed take stage s + D
            if (q == SPK - 1) load_w(s / SPK + KW, fw[p]);
            issue(s + D, (u + D) % SPK, fa[d], rq[d]);
        }
    }

    // epilogue: a lane holds four consecutive columns of one row per block and column tile
    const bool plain = DT != SPH_I8 && !a.scale && !a.shift && !a.relu;
    const bool relu = DT != SPH_I8 && a.relu;
    float sc[CT][4], sh[CT][4];
#pragma unroll
    for (int c = 0; c < CT; c++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int col = min(col0 + c * 16 + (lane >> 4) * 4 + j, a.ndim - 1);
            sc[c][j] = a.scale ? a.scale[col] : 1.f;
            sh[c][j] = (DT != SPH_I8 && a.shift) ? a.shift[col] : 0.f;
        }
    elem *out = (elem *)a.out + (long)r0 * a.ndim;
    auto store_block = [&](int b, const acc4 (&ac)[CT]) {
        const int row = b * SPH_GROUP + (lane & 15);
        if (row >= nrows) return;
#pragma unroll
        for (int c = 0; c < CT; c++) {
            const int col = col0 + c * 16 + (lane >> 4) * 4;
            if (col >= a.ndim) continue;
            union { elem e[4]; uint32_t w[sizeof(elem)]; } u;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float v = DT == SPH_I8 ? (float)(int)ac[c][j] : (float)ac[c][j];
                if (!plain) {
                    v = v * sc[c][j] + sh[c][j];
                    if (relu) v = v > 0.f ? v : 0.f;
                }
                u.e[j] = to_elem<DT>(v);
            }
            uint32_t *dst = (uint32_t *)(out + (long)row * a.ndim + col);
#pragma unroll
            for (int q = 0; q < (int)sizeof(elem); q++) dst[q] = u.w[q];
        }
    };
#pragma unroll
    for (int j = 0; j < NB; j++) store_block(blk0 + j, acc[j]);
}

// The accumulators of a wave are CT*32 registers; the wrappers tell the compiler how many waves per
// SIMD to leave room for (4 column tiles: 2, 2 tiles: 3, 1 tile: 4), i.e. how many registers the
// gathers in flight may take.
template <sph_dtype DT, int NS, int CT, bool MASKED>
__global__ __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(2))) void conv_rows_kernel_w2(ConvArgs a, int nwtot)
{
    conv_rows_body<DT, NS, CT, MASKED, 1>(a, nwtot);
}
template <sph_dtype DT, int NS, int CT, bool MASKED>
__global__ __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(3))) void conv_rows_kernel_w3(ConvArgs a, int nwtot)
{
    conv_rows_body<DT, NS, CT, MASKED, 1>(a, nwtot);
}
template <sph_dtype DT, int NS, int CT, bool MASKED>
__global__ __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(4))) void conv_rows_kernel_w4(ConvArgs a, int nwtot)
{
    conv_rows_body<DT, NS, CT, MASKED, 1>(a, nwtot);
}
// four waves per tile and block of columns
template <sph_dtype DT, int NS, int CT, bool MASKED>
__global__ __launch_bounds__(512) void conv_rows_kernel_split(ConvArgs a, int nwtot)
{
    conv_rows_body<DT, NS, CT, MASKED, 4>(a, nwtot);
}


// ---------------------------------------------------------------------------
// By stationary row, gathered rows staged in LDS: rows of up to 64 bytes (one MFMA K step), up to 32
// output columns, one wave per tile.
//
// With one K step a (offset, block) step is one or two MFMAs behind a gather of 16 rows; the plain by-row
// kernel then waits for its gathers (every one a miss of the vector L1: a tile's 27 offsets ask for each
// neighbouring row about ten times, with the other waves' traffic in between).  The rows a tile's offsets
// gather lie close together in the feature array: for 9 consecutive offsets (one value of k0 in a 3x3x3
// kernel) they are the tile's own range of rows of one line of the grid, a column more on either side.
// So the offsets are taken in phases of 9: the wave finds the range [lo, hi] of rows the phase gathers,
// brings it to LDS as it lies (direct global -> LDS loads, all in flight at once), rewrites the phase's
// table as one byte per (offset, row) (place in the window; slots without a pair point at a row of zeros
// behind it), and every step's gather is then one 16-byte LDS read per lane, with nothing to select
// afterwards.  A phase whose rows do not fit the window (a tile that straddles two lines of the grid,
// strided layers with wide footprints) gathers from the feature array instead.  The order of summation
// per row is the plain kernel's (offsets ascending), so results are bit-identical.  Bounds: the LDS
// (about 10 cycles per 16-row read and CU, against 8 for the step's two MFMAs) and, per phase, one round
// trip for the window; the registers (accumulators, three offsets of weights, the next table) allow two
// waves per SIMD, and with 64 output columns they do not suffice (the compiler spills and the kernel
// halves its speed), so those layers stay with the plain kernel.
// Measured, fp16, grid 4x32x1024x32 at 40 % occupancy (1.68 M rows, 10.9 pairs per row): 32->32 178 us
// against 250 us with gathers from the feature array, 16->32 156 against 210.
// ---------------------------------------------------------------------------
constexpr int kWinPhase = 9;           // offsets per window
constexpr int kWinBytes = 16 * 1024;   // bytes of feature rows a window holds (up to 255 rows)
constexpr int kWinTab = kWinPhase * R; // one byte per (offset, row)
constexpr int kWinMaxRows = 255;       // most rows of a window: a byte names any of them or the row of zeros

template <sph_dtype DT, int CT, bool MASKED>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2))) void conv_rows_win_kernel(ConvArgs a, int nwtot)
{
    typedef typename Traits<DT>::elem elem;
    typedef typename Traits<DT>::acc4 acc4;
    typedef int int2v __attribute__((ext_vector_type(2)));
    constexpr int NB = R / SPH_GROUP;        // 8 blocks of 16 rows
    constexpr int HB = 4;                    // blocks per stage
    constexpr int SPO = NB / HB;             // stages per offset
    constexpr int TL = kWinPhase * R / 2 / kWave; // int2 table entries per lane and phase
    constexpr int WR = 3;                    // sets of weight fragments: requested three offsets ahead
    static_assert(kWinPhase % WR == 0, "the ring must divide a phase");
    extern __shared__ __attribute__((aligned(16))) char s_mem[];
    uint8_t *s_tab = (uint8_t *)s_mem;       // [kWinPhase][SPO][16 rows][HB blocks]
    char *s_win = s_mem + kWinTab;           // the window's rows, as they lie in the feature array
    int32_t *s_tab32 = (int32_t *)s_win;     // a phase without a window: [kWinPhase][R] rows of the feature array

    const int lane = threadIdx.x & (kWave - 1);
    const int tile = sph_xcd_tile(blockIdx.x, (a.book.rows + R - 1) / R);
    const int r0 = tile * R;
    if (r0 >= a.book.rows) return;
    const int nrows = min(R, a.book.rows - r0);
    const int KV = a.book.KV;
    const int rb = a.row_bytes;
    const int nph = (KV + kWinPhase - 1) / kWinPhase;
    const char *wlane = a.wp + lane * 16;
    const long wstep = (long)nwtot * (kWave * 16);
    const int chunk = lane >> 4;
    const bool live_chunk = chunk * 16 < rb;
    const int choff = live_chunk ? chunk * 16 : 0;

    acc4 acc[NB][CT];
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
        for (int c = 0; c < CT; c++) acc[j][c] = acc4{0, 0, 0, 0};

    int2v tn[TL]; // the next phase's table, on its way while this phase is worked through
    auto load_tab = [&](int ph) {
        const int phc = min(ph, nph - 1);
        const int2v *src = (const int2v *)(a.book.tile_nbr + ((long)tile * KV + phc * kWinPhase) * R);
        const int n2 = min(kWinPhase, KV - phc * kWinPhase) * R / 2;
#pragma unroll
        for (int i = 0; i < TL; i++) {
            const int e = lane + kWave * i;
            tn[i] = src[e < n2 ? e : 0];
        }
    };
    auto load_w = [&](int k, int4v (&w)[CT]) {
        const char *wk = wlane + (long)min(k, KV - 1) * wstep;
#pragma unroll
        for (int c = 0; c < CT; c++) w[c] = *(const int4v *)(wk + (long)c * (kWave * 16));
    };

    int4v wr[WR][CT];
    load_tab(0);
#pragma unroll
    for (int i = 0; i < WR; i++) load_w(i, wr[i]);
    for (int ph = 0; ph < nph; ph++) {
        const int k0 = ph * kWinPhase;
        const int nk = min(kWinPhase, KV - k0);
        // this phase's table: validate, find the range of rows it gathers
        int2v t[TL];
        int lo = 0x7fffffff, hi = -1;
#pragma unroll
        for (int i = 0; i < TL; i++) {
            const int e = lane + kWave * i;
            int2v v = tn[i];
            const bool in = e < nk * R / 2;
            v.x = (in && (unsigned)v.x < (unsigned)a.feat_rows) ? v.x : -1;
            v.y = (in && (unsigned)v.y < (unsigned)a.feat_rows) ? v.y : -1;
            if (v.x >= 0) { lo = min(lo, v.x); hi = max(hi, v.x); }
            if (v.y >= 0) { lo = min(lo, v.y); hi = max(hi, v.y); }
            t[i] = v;
        }
        load_tab(ph + 1);
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) {
            lo = min(lo, __shfl_xor(lo, o, kWave));
            hi = max(hi, __shfl_xor(hi, o, kWave));
        }
        lo = __builtin_amdgcn_readfirstlane(lo);
        hi = __builtin_amdgcn_readfirstlane(hi);
        if (hi < 0) { // no pair at these offsets
#pragma unroll
            for (int i = 0; i < WR; i++) load_w(k0 + kWinPhase + i, wr[i]);
            continue;
        }
        // a window holds rows lo..hi and, behind them, one row of zeros that slots without a pair read
        const int nrow = hi - lo + 1;
        const bool win = nrow <= kWinMaxRows && nrow * rb <= kWinBytes;
        // direct loads write LDS behind the back of the LDS unit's own queue: the last phase's reads must
        // have returned before the window is overwritten
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (win) {
#pragma unroll
            for (int i = 0; i < TL; i++) {
                // entries 2e and 2e + 1 of the phase: offset e / 64, row 2e % 128 and the next one (same block)
                const int e = lane + kWave * i;
                const int row = (2 * e) & (R - 1), blk = row >> 4, n = row & 15;
                uint8_t *dst = s_tab + (e >> 6) * R + (blk / HB) * (SPH_GROUP * HB) + n * HB + blk % HB;
                dst[0] = (uint8_t)(t[i].x >= 0 ? t[i].x - lo : nrow);
                dst[HB] = (uint8_t)(t[i].y >= 0 ? t[i].y - lo : nrow);
            }
            // lane l of load i fills the 16 bytes at i * 1024 + l * 16 of the window
            const int nbytes = nrow * rb;
            const int nld = (nbytes + kWave * 16 - 1) / (kWave * 16);
            const char *src = a.feat + (long)lo * rb;
            for (int i = 0; i < nld; i++) {
                const char *g = src + min((i * kWave + lane) * 16, nbytes - 16);
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)g,
                                                 (__attribute__((address_space(3))) void *)(s_win + i * (kWave * 16)), 16, 0, 0);
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (lane * 16 < rb) *(int4v *)(s_win + nbytes + lane * 16) = int4v{0, 0, 0, 0}; // behind the loads: their last kilobyte may reach here
            // stages (offset, HB blocks): table entries two stages ahead, rows one stage ahead
            constexpr int ns = kWinPhase * SPO;
            auto tab = [&](int st, int (&id)[HB]) {
                const int sc = min(st, ns - 1);
                const uint8_t *p = s_tab + (sc / SPO) * R + (sc % SPO) * (SPH_GROUP * HB) + (lane & 15) * HB;
                const uint32_t pk = HB == 4 ? *(const uint32_t *)p : *(const uint16_t *)p;
#pragma unroll
                for (int j = 0; j < HB; j++) id[j] = (pk >> (8 * j)) & 255;
            };
            auto rows = [&](const int (&id)[HB], int4v (&x)[HB]) {
#pragma unroll
                for (int j = 0; j < HB; j++) {
                    // lanes on 16-byte chunks behind the row's end read zeros too
                    const int r = (MASKED && !live_chunk) ? nrow : id[j];
                    x[j] = *(const int4v *)(s_win + (__umul24(r, rb) + choff));
                }
            };
            int id1[HB], id2[HB];
            int4v x1[HB];
            tab(0, id1);
            tab(1, id2);
            rows(id1, x1);
            auto round = [&](int k9) {
#pragma unroll
                for (int i = 0; i < WR; i++) {
#pragma unroll
                    for (int h = 0; h < SPO; h++) {
                        const int st = (k9 + i) * SPO + h;
                        int4v xc[HB];
#pragma unroll
                        for (int j = 0; j < HB; j++) { xc[j] = x1[j]; id1[j] = id2[j]; }
                        rows(id1, x1);
                        tab(st + 2, id2);
#pragma unroll
                        for (int j = 0; j < HB; j++)
#pragma unroll
                            for (int c = 0; c < CT; c++) acc[h * HB + j][c] = mfma_step<DT>(wr[i][c], xc[j], acc[h * HB + j][c]);
                    }
                    load_w(k0 + k9 + i + WR, wr[i]);
                }
            };
            // a whole phase as straight-line code (the compiler then counts the weight loads in flight exactly);
            // offsets past the kernel's last find a table of empty slots
#pragma unroll
            for (int k9 = 0; k9 < kWinPhase; k9 += WR) round(k9);
        } else {
            // the rows lie too far apart: gathers from the feature array, one offset at a time
#pragma unroll
            for (int i = 0; i < TL; i++) ((int2v *)s_tab32)[lane + kWave * i] = t[i];
#pragma unroll 1
            for (int k9 = 0; k9 < nk; k9++) {
                int4v w[CT];
                load_w(k0 + k9, w);
#pragma unroll
                for (int h = 0; h < SPO; h++) {
                    int id[HB];
                    int4v x[HB];
#pragma unroll
                    for (int j = 0; j < HB; j++) {
                        id[j] = s_tab32[k9 * R + (h * HB + j) * SPH_GROUP + (lane & 15)];
                        x[j] = *(const int4v *)(a.feat + (long)max(id[j], 0) * rb + choff);
                    }
#pragma unroll
                    for (int j = 0; j < HB; j++) {
                        bool live = id[j] >= 0;
                        if constexpr (MASKED) live = live && live_chunk;
                        const int4v y = live ? x[j] : int4v{0, 0, 0, 0};
#pragma unroll
                        for (int c = 0; c < CT; c++) acc[h * HB + j][c] = mfma_step<DT>(w[c], y, acc[h * HB + j][c]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int i = 0; i < WR; i++) load_w(k0 + kWinPhase + i, wr[i]);
        }
    }

    // epilogue: a lane holds four consecutive columns of one row per block and column tile
    const bool plain = DT != SPH_I8 && !a.scale && !a.shift && !a.relu;
    const bool relu = DT != SPH_I8 && a.relu;
    float sc[CT][4], sh[CT][4];
#pragma unroll
    for (int c = 0; c < CT; c++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int col = min(c * 16 + (lane >> 4) * 4 + j, a.ndim - 1);
            sc[c][j] = a.scale ? a.scale[col] : 1.f;
            sh[c][j] = (DT != SPH_I8 && a.shift) ? a.shift[col] : 0.f;
        }
    elem *out = (elem *)a.out + (long)r0 * a.ndim;
#pragma unroll
    for (int b = 0; b < NB; b++) {
        const int row = b * SPH_GROUP + (lane & 15);
        if (row >= nrows) continue;
#pragma unroll
        for (int c = 0; c < CT; c++) {
            const int col = c * 16 + (lane >> 4) * 4;
            if (col >= a.ndim) continue;
            union { elem e[4]; uint32_t w[sizeof(elem)]; } u;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float v = DT == SPH_I8 ? (float)(int)acc[b][c][j] : (float)acc[b][c][j];
                if (!plain) {
                    v = v * sc[c][j] + sh[c][j];
                    if (relu) v = v > 0.f ? v : 0.f;
                }
                u.e[j] = to_elem<DT>(v);
            }
            uint32_t *dst = (uint32_t *)(out + (long)row * a.ndim + col);
#pragma unroll
            for (int q = 0; q < (int)sizeof(elem); q++) dst[q] = u.w[q];
        }
    }
}

// ---------------------------------------------------------------------------
// wgrad
// ---------------------------------------------------------------------------
struct WgradArgs {
    const char *feat;
    int in_rows, iC;
    const char *dout;
    int out_rows, oC;
    sph_book book;
    int cap, ntiles, nchunk;
    float *partial;
    int *flags;      // wave kernel: one per partial slot, 1 = the slot was written
    int nslice;      // wave kernel: workgroups per chunk at the centre offset (slices h, h + nslice, ... each)
    int all_slices;  // wave kernel: every offset has its later slices' workgroups (small grids), not only the centre
    int nslots;
};

constexpr int kWgThreads = 256;
constexpr int kWgWaves = kWgThreads / kWave;
constexpr int kMaxTilesPerWave = 16; // (128/16)^2 / 4 waves

template <sph_dtype DT>
__global__ __launch_bounds__(kWgThreads) void wgrad_kernel(WgradArgs a)
{
    typedef typename Traits<DT>::elem elem;
    constexpr int KW = Traits<DT>::KW;
    constexpr int PB = 4 * KW;            // pairs per batch = K of one super step
    constexpr int LDP = PB + 16 / (int)sizeof(elem); // padded pair stride, keeps 16-byte alignment
    extern __shared__ char s_raw[];
    const int iCp = (a.iC + 15) & ~15, oCp = (a.oC + 15) & ~15;
    elem *At = (elem *)s_raw;               // [iCp][LDP]
    elem *Gt = At + (long)iCp * LDP;        // [oCp][LDP]
    __shared__ int s_in[PB], s_out[PB];

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int KV = a.book.KV;
    const int k = blockIdx.x / a.nchunk, chunk = blockIdx.x - k * a.nchunk;
    const int tpc = (a.ntiles + a.nchunk - 1) / a.nchunk;
    const int t0 = chunk * tpc, t1 = min(t0 + tpc, a.ntiles);
    const int MI = iCp / 16, NI = oCp / 16, MT = MI * NI;

    float4v acc[kMaxTilesPerWave];
#pragma unroll
    for (int j = 0; j < kMaxTilesPerWave; j++) acc[j] = float4v{0, 0, 0, 0};

    for (int t = t0; t < t1; t++) {
        const int g0 = a.book.tile_koff[(long)t * (KV + 1) + k];
        const int g1 = a.book.tile_koff[(long)t * (KV + 1) + k + 1];
        for (int gb = g0; gb < g1; gb += PB / SPH_GROUP) {
            __syncthreads(); // previous batch fully consumed
            if (tid < PB) {
                int g = gb + tid / SPH_GROUP;
                int vi = -1, vo = -1;
                if (g < g1) {
                    long slot = ((long)t * a.cap + g) * SPH_GROUP + (tid & (SPH_GROUP - 1));
                    vi = a.book.grp_gather[slot];
                    vo = a.book.grp_owner[slot];
                }
                if ((unsigned)vi >= (unsigned)a.in_rows || (unsigned)vo >= (unsigned)a.out_rows) vi = vo = -1;
                s_in[tid] = vi;
                s_out[tid] = vo;
            }
            __syncthreads();
            for (int e = tid; e < PB * iCp; e += kWgThreads) {
                int p = e / iCp, c = e - p * iCp;
                int row = s_in[p];
                elem v = (elem)0;
                if (row >= 0 && c < a.iC) v = ((const elem *)a.feat)[(long)row * a.iC + c];
                At[c * LDP + p] = v;
            }
            for (int e = tid; e < PB * oCp; e += kWgThreads) {
                int p = e / oCp, c = e - p * oCp;
                int row = s_out[p];
                elem v = (elem)0;
                if (row >= 0 && c < a.oC) v = ((const elem *)a.dout)[(long)row * a.oC + c];
                Gt[c * LDP + p] = v;
            }
            __syncthreads();
#pragma unroll
            for (int j = 0; j < kMaxTilesPerWave; j++) {
                int ti = wave + j * kWgWaves;
                if (ti < MT) {
                    int mi = ti / NI, ni = ti - mi * NI;
                    int4v fa = *(const int4v *)(At + (mi * 16 + (lane & 15)) * LDP + (lane >> 4) * KW);
                    int4v fb = *(const int4v *)(Gt + (ni * 16 + (lane & 15)) * LDP + (lane >> 4) * KW);
                    acc[j] = mfma_step<DT>(fa, fb, acc[j]);
                }
            }
        }
    }
    float *part = a.partial + ((long)k * a.nchunk + chunk) * a.iC * a.oC;
#pragma unroll
    for (int j = 0; j < kMaxTilesPerWave; j++) {
        int ti = wave + j * kWgWaves;
        if (ti < MT) {
            int mi = ti / NI, ni = ti - mi * NI;
            int co = ni * 16 + (lane & 15);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                int ci = mi * 16 + (lane >> 4) * 4 + r;
                if (ci < a.iC && co < a.oC) part[(long)ci * a.oC + co] = acc[j][r];
            }
        }
    }
}

template <typename OUT>
__global__ void wgrad_reduce_kernel(const float *partial, int KV, int nchunk, int per_k, OUT *dw)
{
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (long)KV * per_k) return;
    int k = (int)(i / per_k), e = (int)(i - (long)k * per_k);
    const float *p = partial + (long)k * nchunk * per_k + e;
    float s = 0.f;
    for (int c = 0; c < nchunk; c++) s += p[(long)c * per_k];
    dw[i] = (OUT)s;
}

// ---------------------------------------------------------------------------
// wgrad, fast path (rows are whole 16-byte chunks).
//
// Work item = (offset k, chunk of 64 tiles, slice of 64 groups of that chunk's groups at
// k, 64x64 block of [iC,oC]).  A chunk holds at most 64*8 groups per offset; four
// workgroups are launched per (offset, chunk), workgroup h takes slices h and h+4, and
// those whose first slice lies beyond the chunk's real group count exit at once (a
// submanifold book has 8 groups per tile at the centre offset and about one elsewhere:
// slicing by groups, not tiles, is what balances the grid).
// The four waves of the workgroup take the slice's batches (32 pairs; 16 for fp32) round
// robin and never synchronise until the end: a wave gathers the batch's feature rows and
// d_out rows with 16-byte loads into its own LDS area in natural [pair][channel] order,
// and reads MFMA operands with the pair index as the K dimension through transposing
// LDS reads (16-bit types) or strided 4-byte reads (fp32).  The block lives in registers;
// the workgroup's four blocks are summed through LDS into one fp32 partial, and
// wgrad_slot_reduce_kernel adds the written slots in a fixed order.
// What bounds it (64->64 fp16, 8 waves per CU): LDS traffic (8 KiB staged and 8 KiB read
// back per batch and wave) and the MFMAs, about equally.
// ---------------------------------------------------------------------------
constexpr int kWsTiles = 64;   // tiles per chunk (one lane each)
constexpr int kWsSlice = 64;   // groups per slice
constexpr int kWsSlices = 8;   // most workgroups per chunk at the centre offset (workgroup h takes slices h, h + nslice, ...);
                               // WgradArgs::nslice = 8 on small books, 4 on large ones; one workgroup elsewhere
constexpr int kWsBlock = 64;   // channels per block side

typedef short short4v __attribute__((ext_vector_type(4)));

// MFMA operand of 16 channels x one batch of pairs from a staging area laid out
// [pair][channel], row stride rs bytes.  16-bit types: lane (m = lane%16, q = lane/16)
// receives pairs 8q..8q+7 of channel m through two transposing reads (element j of lane
// 4a+b = the b-th element at the address given by lane a+4j of the same 16 lanes).
// fp32: component j of lane (m, q) = pair 4j+q of channel m.
template <sph_dtype DT>
__device__ __forceinline__ int wgrad_frag_offset(int rs, int lane)
{
    if constexpr (sizeof(typename Traits<DT>::elem) == 2) {
        const int s = lane & 15, q = lane >> 4;
        return (8 * q + (s >> 2)) * rs + 4 * (s & 3) * 2;
    } else {
        return (lane >> 4) * rs + (lane & 15) * 4;
    }
}
template <sph_dtype DT>
__device__ __forceinline__ int4v wgrad_frag(const char *p, int rs)
{
    if constexpr (sizeof(typename Traits<DT>::elem) == 2) {
        typedef __attribute__((address_space(3))) short4v lds_s4;
        short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4 *)p);
        short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4 *)(p + 4 * rs));
        union { struct { short4v l, h; } s; int4v v; } u;
        u.s.l = lo; u.s.h = hi;
        return u.v;
    } else {
        union { float f[4]; int4v v; } u;
#pragma unroll
        for (int j = 0; j < 4; j++) u.f[j] = *(const float *)(p + 4 * j * rs);
        return u.v;
    }
}

template <sph_dtype DT, int MI, int NI>
__global__ __launch_bounds__(256, 2) void wgrad_wave_kernel(WgradArgs a)
{
    typedef typename Traits<DT>::elem elem;
    constexpr int E = (int)sizeof(elem);
    constexpr int GPB = E == 2 ? 2 : 1;                // groups per batch: one MFMA super step of 32 or 16 pairs
    constexpr int PB = GPB * SPH_GROUP;                // pairs per batch
    // MI, NI: 16-channel tiles of the block's two sides (1, 2 or 4; narrower blocks are zero padded).
    // A batch of rows of MI tiles is MI 16-byte loads per lane.
    extern __shared__ __attribute__((aligned(16))) char s_raw[];

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int KV = a.book.KV;
    // Work items u = chunk*KV + k are dealt to the XCDs in contiguous runs (workgroups go to
    // the XCDs round robin): the offsets of one chunk gather the same ~2 MiB of rows, which
    // then stay in that XCD's L2.  The slice index is slowest, so that the first slices --
    // often the only ones with work -- spread over all XCDs and start first.
    const int items = KV * a.nchunk, items_grid = (items + SPH_NUM_XCD - 1) / SPH_NUM_XCD * SPH_NUM_XCD;
    int h, chunk, k;
    if ((int)blockIdx.x < items_grid) {
        h = 0;
        const int u = sph_xcd_tile(blockIdx.x, items);
        if (u >= items) return;
        chunk = u / KV;
        k = u - chunk * KV;
    } else {
        // Later slices: a submanifold book has 8 groups per tile at the centre offset and about one elsewhere, and
        // a workgroup without work still costs its dispatch (three quarters of the grid found none when every offset
        // had four).  So only the centre offset has them, numbered first, and at the other offsets the first
        // workgroup takes every slice -- unless the grid is small (all_slices): then a dense book's offsets need
        // their four workgroups each to fill the chip, and they follow the centre's.
        const int kc = KV / 2, v = (int)blockIdx.x - items_grid, nc = (a.nslice - 1) * a.nchunk;
        if (v < nc) {
            h = 1 + v / a.nchunk;
            chunk = v % a.nchunk;
            k = kc;
        } else {
            const int r = v - nc, per = a.nchunk * (KV - 1);
            if (!a.all_slices || KV == 1 || r >= (a.nslice - 1) * per) return;
            h = 1 + r / per;
            const int q = r % per, kk = q % (KV - 1);
            chunk = q / (KV - 1);
            k = kk + (kk >= kc ? 1 : 0);
        }
    }
    const int slice_step = (a.all_slices || k == KV / 2) ? a.nslice : 1;
    const int sbn = (a.oC + kWsBlock - 1) / kWsBlock;
    const int ci0 = (blockIdx.y / sbn) * kWsBlock, co0 = (blockIdx.y % sbn) * kWsBlock;
    const int cA = min(kWsBlock, a.iC - ci0), cG = min(kWsBlock, a.oC - co0);
    const int slot = (k * a.nchunk + chunk) * a.nslice + h;

    // groups of this offset in the chunk's tiles: lane = tile, prefix sums over the wave
    const int t0 = chunk * kWsTiles;
    int g0 = 0, n = 0;
    if (t0 + lane < a.ntiles) {
        const unsigned short *ko = a.book.tile_koff + (long)(t0 + lane) * (KV + 1) + k;
        g0 = min((int)ko[0], a.cap);
        n = min(max((int)ko[1] - g0, 0), min(a.cap - g0, R / SPH_GROUP));
    }
    const int incl = wave_inclusive_sum(n); // lane shifts of the vector ALU, no LDS round trip per step
    const int total = __builtin_amdgcn_readlane(incl, kWave - 1);
    if (slice_step == 1 && tid < a.nslice - 1 && blockIdx.y == 0) a.flags[slot + 1 + tid] = 0; // slots nobody fills
    if (h * kWsSlice >= total) {
        if (tid == 0 && blockIdx.y == 0) a.flags[slot] = 0;
        return;
    }

    // wave-private staging: feature rows then d_out rows, [pair][channels + 16 bytes]
    constexpr int rsA = MI * 16 * E + 16, rsG = NI * 16 * E + 16;
    const int cprA = cA * E / 16, cprG = cG * E / 16;      // real 16-byte chunks per row
    char *xa = s_raw + (size_t)wave * PB * (rsA + rsG);
    char *xg = xa + PB * rsA;
    for (int i = lane; i < PB * (rsA + rsG) / 16; i += kWave) ((int4v *)xa)[i] = int4v{0, 0, 0, 0};

    float4v acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++) acc[i][j] = float4v{0, 0, 0, 0};

    // Per-lane constants of the row copies: which pair and 16-byte chunk each of the lane's
    // loads moves, its offset in the source row and in the staging area (-1: none).
    int pairA[MI], srcA[MI], dstA[MI], pairG[NI], srcG[NI], dstG[NI];
    // (rows of 32, 64 or 128 bytes are 2, 4 or 8 chunks: a shift instead of the forty instructions of a division)
    const bool p2A = (cprA & (cprA - 1)) == 0, p2G = (cprG & (cprG - 1)) == 0;
    const int shA = __ffs(cprA) - 1, shG = __ffs(cprG) - 1;
#pragma unroll
    for (int it = 0; it < MI; it++) {
        const int i = it * kWave + lane;
        const int pa = p2A ? i >> shA : i / cprA, ca = i - pa * cprA;
        pairA[it] = min(pa, PB - 1); srcA[it] = ci0 * E + ca * 16; dstA[it] = pa < PB ? pa * rsA + ca * 16 : -1;
    }
#pragma unroll
    for (int it = 0; it < NI; it++) {
        const int i = it * kWave + lane;
        const int pg = p2G ? i >> shG : i / cprG, cg = i - pg * cprG;
        pairG[it] = min(pg, PB - 1); srcG[it] = co0 * E + cg * 16; dstG[it] = pg < PB ? pg * rsG + cg * 16 : -1;
    }
    const unsigned strideA = a.iC * E, strideG = a.oC * E;   // arrays are below 4 GiB (checked by the launcher)

    // Book slot of every group of a slice: lane l looks up flattened group s0+l (the tile
    // whose prefix range holds it, by binary search over the tile lanes) once per slice.
    const long slot_max = (long)a.ntiles * a.cap * SPH_GROUP - 1;
    auto slot_bases = [&](int s0) -> int {
        const int f = s0 + lane;
        int lo = 0;
#pragma unroll
        for (int step = kWave / 2; step >= 1; step >>= 1) {
            const int v = __shfl(incl, lo + step - 1, kWave);
            if (v <= f) lo += step;
        }
        lo = min(lo, kWave - 1);
        const int g = __shfl(g0, lo, kWave) + f - (__shfl(incl, lo, kWave) - __shfl(n, lo, kWave));
        const long sl = ((long)(t0 + lo) * a.cap + g) * SPH_GROUP;
        return (int)min(max(sl, 0L), slot_max - (SPH_GROUP - 1));   // ntiles*cap*16 fits 31 bits (checked by the launcher)
    };
    // Book entries of batch b of the slice: lane l < 32 loads the gathered (input) row of pair
    // l%PB, lane 32+l its owner (output) row.  The load is unconditional; the value is only
    // looked at once all of the wave's index loads are on their way.
    auto load_idx = [&](int bases, int s0, int s1, int b, bool &valid) -> int {
        const int pr = lane & (PB - 1);
        const int fl = GPB * b + (pr >> 4);                 // group within the slice
        valid = s0 + fl < s1;
        const int base = __shfl(bases, fl & (kWave - 1), kWave);
        return (lane < 32 ? a.book.grp_gather : a.book.grp_owner)[base + (pr & 15)];
    };
    // Row loads are unconditional (clamped to row 0; in_rows and out_rows are positive here)
    // so that several batches stay in flight; slots without a pair are zeroed when the rows
    // are staged.  Returns the mask of pairs that exist.
    auto gather = [&](int idx, int4v (&ra)[MI], int4v (&rg)[NI]) -> unsigned {
        // all lane exchanges first, then all loads: one wait on the LDS queue instead of one per row
        const int other = __shfl_xor(idx, 32, kWave);
        int rowA[MI], rowG[NI];
#pragma unroll
        for (int it = 0; it < MI; it++) rowA[it] = __shfl(idx, pairA[it], kWave);
#pragma unroll
        for (int it = 0; it < NI; it++) rowG[it] = __shfl(idx, 32 + pairG[it], kWave);
        __builtin_amdgcn_sched_barrier(0);
        const unsigned ok = (unsigned)__ballot(idx >= 0 && other >= 0);
#pragma unroll
        for (int it = 0; it < MI; it++)
            ra[it] = *(const int4v *)(a.feat + ((unsigned)max(rowA[it], 0) * strideA + (unsigned)srcA[it]));
#pragma unroll
        for (int it = 0; it < NI; it++)
            rg[it] = *(const int4v *)(a.dout + ((unsigned)max(rowG[it], 0) * strideG + (unsigned)srcG[it]));
        return ok;
    };
    auto stage = [&](unsigned ok, const int4v (&ra)[MI], const int4v (&rg)[NI]) {
#pragma unroll
        for (int it = 0; it < MI; it++)
            if (dstA[it] >= 0) *(int4v *)(xa + dstA[it]) = ((ok >> pairA[it]) & 1) ? ra[it] : int4v{0, 0, 0, 0};
#pragma unroll
        for (int it = 0; it < NI; it++)
            if (dstG[it] >= 0) *(int4v *)(xg + dstG[it]) = ((ok >> pairG[it]) & 1) ? rg[it] : int4v{0, 0, 0, 0};
    };
    const char *fragA = xa + wgrad_frag_offset<DT>(rsA, lane), *fragG = xg + wgrad_frag_offset<DT>(rsG, lane);
    auto multiply = [&]() {
        int4v fa[MI], fb[NI];
#pragma unroll
        for (int i = 0; i < MI; i++) fa[i] = wgrad_frag<DT>(fragA + i * 16 * E, rsA);
#pragma unroll
        for (int i = 0; i < NI; i++) fb[i] = wgrad_frag<DT>(fragG + i * 16 * E, rsG);
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int j = 0; j < NI; j++) acc[i][j] = mfma_step<DT>(fa[i], fb[j], acc[i][j]);
    };

    // Per slice, this wave owns batches wave, wave+4, ... (at most NB).  All their index
    // entries are requested at once; then the rows run DEPTH-1 batches ahead of their
    // staging through DEPTH register sets, and staging runs one batch ahead of the MFMAs.
    // The single staging area is safe because LDS operations of a wave execute in order.
    constexpr int NB = kWsSlice / GPB / 4;
    constexpr int DEPTH = 3;
    for (int s0 = h * kWsSlice; s0 < total; s0 += slice_step * kWsSlice) {
        const int s1 = min(total, s0 + kWsSlice);
        const int nbatch = (s1 - s0 + GPB - 1) / GPB;
        const int bases = slot_bases(s0);
        int idx[NB];
        bool valid[NB];
#pragma unroll
        for (int j = 0; j < NB; j++) idx[j] = load_idx(bases, s0, s1, wave + 4 * j, valid[j]);
#pragma unroll
        for (int j = 0; j < NB; j++)
            idx[j] = (valid[j] && (unsigned)idx[j] < (unsigned)(lane < 32 ? a.in_rows : a.out_rows)) ? idx[j] : -1;
        int4v ra[DEPTH][MI], rg[DEPTH][NI];
        unsigned ok[DEPTH];
#pragma unroll
        for (int j = 0; j < DEPTH - 1; j++)
            if (j < NB) ok[j] = gather(idx[j], ra[j], rg[j]);
#pragma unroll
        for (int j = 0; j < NB; j++) {
            if (wave + 4 * j < nbatch) {     // wave-uniform
                if (j + DEPTH - 1 < NB)
                    ok[(j + DEPTH - 1) % DEPTH] = gather(idx[j + DEPTH - 1], ra[(j + DEPTH - 1) % DEPTH], rg[(j + DEPTH - 1) % DEPTH]);
                if (j > 0) multiply();            // batch j-1, from LDS
                asm volatile("" ::: "memory");    // keep the staging writes behind the transposing reads
                stage(ok[j % DEPTH], ra[j % DEPTH], rg[j % DEPTH]);
                asm volatile("" ::: "memory");
            }
        }
        if (wave < nbatch) multiply();            // the last staged batch
    }

    // Sum the four waves' blocks through LDS (over the staging areas), pairwise: (0+2, 1+3),
    // then (0+1).  The partial is stored in accumulator order -- tile (i,j), lane, 4 values:
    // element [16i + 4(lane/16) + r][16j + lane%16] -- as 16-byte stores; the reduction kernel
    // puts it back in [iC,oC] order.
    float4v *red = (float4v *)s_raw;
    constexpr int BLK = MI * NI * kWave;   // float4 per block
    __syncthreads();
    if (wave >= 2) {
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int j = 0; j < NI; j++) red[(wave - 2) * BLK + (i * NI + j) * kWave + lane] = acc[i][j];
    }
    __syncthreads();
    if (wave < 2) {
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int j = 0; j < NI; j++) acc[i][j] += red[wave * BLK + (i * NI + j) * kWave + lane];
    }
    __syncthreads();
    if (wave == 1) {
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int j = 0; j < NI; j++) red[(i * NI + j) * kWave + lane] = acc[i][j];
    }
    __syncthreads();
    if (wave == 0) {
        float4v *part = (float4v *)(a.partial + ((long)slot * gridDim.y + blockIdx.y) * (kWsBlock * kWsBlock));
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int j = 0; j < NI; j++) part[(i * NI + j) * kWave + lane] = acc[i][j] + red[(i * NI + j) * kWave + lane];
        if (lane == 0 && blockIdx.y == 0) a.flags[slot] = 1;
    }
}

// dw[k][ci][co] = sum of the written slots of offset k, in slot order.  A slot holds one
// 64x64 block per (iC,oC) block pair, each in accumulator order of MI x NI tiles (see
// wgrad_wave_kernel).  A thread owns one 16-byte item of a block (four ci of one co), so the
// slots are read as they were written; a workgroup covers 32 consecutive items, its 8 groups of
// 32 threads each add every 8th slot (up to sixteen loads in flight), and the 8 sub-sums are added in a
// fixed order.
template <typename OUT>
__global__ __launch_bounds__(256) void wgrad_slot_reduce_kernel(const float *partial, const int *flags, int slots_per_k,
                                                                int iC, int oC, int mi_tiles, int ni_tiles, OUT *dw)
{
    __shared__ float4v s_sum[8][32];
    __shared__ unsigned long long s_flags[16];
    const int k = blockIdx.z, b = blockIdx.y, t = threadIdx.x & 31, j = threadIdx.x >> 5;
    const int q = blockIdx.x * 32 + t;       // 16-byte item of the block, in accumulator order
    const int sbn = (oC + kWsBlock - 1) / kWsBlock, nblk = ((iC + kWsBlock - 1) / kWsBlock) * sbn;
    const int tile = q >> 6, lane = q & 63;
    const bool live = tile < mi_tiles * ni_tiles;
    const long blk = (long)kWsBlock * kWsBlock, step = (long)nblk * blk;
    const float *p = partial + ((long)k * slots_per_k * nblk + b) * blk + q * 4;
    const int *f = flags + (long)k * slots_per_k;
    float4v s = {0.f, 0.f, 0.f, 0.f};
    // The flags of 1024 slots at a time become 16 ballot words in LDS, so that a thread's data loads do not
    // wait for flag loads: per round a thread takes its 16 candidates of two words (slots j, j+8, ... of each),
    // the loads of the written ones in flight together, and adds them in slot order.
    for (int base = 0; base < slots_per_k; base += 1024) {
        __syncthreads();
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const int c = base + w * 256 + (int)threadIdx.x;
            const unsigned long long m = __ballot(c < slots_per_k && f[c] != 0);
            if ((threadIdx.x & (kWave - 1)) == 0) s_flags[w * 4 + (threadIdx.x >> 6)] = m;
        }
        __syncthreads();
        if (!live) continue;
        const int nwords = min(16, (slots_per_k - base + 63) >> 6);
        for (int w0 = 0; w0 < nwords; w0 += 2) {
            const unsigned long long m0 = s_flags[w0] >> j, m1 = w0 + 1 < nwords ? s_flags[w0 + 1] >> j : 0ull;
            float4v v[16];
#pragma unroll
            for (int u = 0; u < 16; u++) {
                const unsigned long long m = u < 8 ? m0 : m1;
                const int cc = base + (w0 + (u >> 3)) * 64 + j + 8 * (u & 7);
                v[u] = float4v{0.f, 0.f, 0.f, 0.f};
                if ((m >> (8 * (u & 7))) & 1ull) v[u] = *(const float4v *)(p + cc * step);
            }
#pragma unroll
            for (int u = 0; u < 16; u++) s += v[u];
        }
    }
    s_sum[j][t] = s;
    __syncthreads();
    if (j == 0 && live) {
        float4v r = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int g = 0; g < 8; g++) r += s_sum[g][t];
        // accumulator order inside the block: tile (li/16, lj/16), lane = 16*((li%16)/4) + lj%16, value li%4
        const int ci = (b / sbn) * kWsBlock + (tile / ni_tiles) * 16 + (lane >> 4) * 4;
        const int co = (b % sbn) * kWsBlock + (tile % ni_tiles) * 16 + (lane & 15);
        if (co < oC) {
#pragma unroll
            for (int v = 0; v < 4; v++)
                if (ci + v < iC) dw[((long)k * iC + ci + v) * oC + co] = (OUT)r[v];
        }
    }
}

inline int elem_size(sph_dtype dt) { return sph_elem_size(dt); }
inline int frag_elems(sph_dtype dt) { return sph_frag_elems(dt); }
inline int pad_waves(int ndim) { return sph_pad_waves(ndim); }
inline int num_steps(sph_dtype dt, int kdim) { return sph_num_steps(dt, kdim); }
inline int wgrad_chunks(int ntiles) { return ntiles < 32 ? (ntiles < 1 ? 1 : ntiles) : 32; }

template <typename K>
inline int set_lds(K kernel, size_t bytes)
{
    if (bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (e != hipSuccess) {
            sph_set_error("hipFuncSetAttribute(%zu bytes of LDS): %s", bytes, hipGetErrorString(e));
            return SPH_ERR_LAUNCH;
        }
    }
    return SPH_OK;
}

template <sph_dtype DT, int NW, int NSTEP>
int launch_conv_ns(const ConvArgs &a, int ntiles, hipStream_t st)
{
    size_t lds = (size_t)R * (NW * 16 + 4) * sizeof(uint32_t);
    int rc = set_lds(conv_apply_kernel<DT, NW, NSTEP>, lds);
    if (rc) return rc;
    hipLaunchKernelGGL((conv_apply_kernel<DT, NW, NSTEP>), dim3(sph_xcd_grid(ntiles)), dim3(NW * kWave), lds, st, a);
    return sph_check_launch("sph_conv_apply");
}

template <sph_dtype DT, int NS, int CT, bool MASKED>
int launch_conv_wave(const ConvArgs &a, int nwtot, int ntiles, hipStream_t st)
{
    size_t lds = (size_t)(R + 1) * (nwtot * 16 + 4) * sizeof(uint32_t); // + scratch row
    const int waves = (nwtot + CT - 1) / CT;
    if constexpr (NS <= 2 && !(DT == SPH_F32 && NS == 2 && CT == 4)) {
        // one wave's worth of columns, rows of up to 128 bytes: helper waves for the middle offset's run (fp32 rows
        // of 128 bytes into 64 columns do not fit the registers three waves per SIMD leave)
        // (narrow layers on large grids keep the one-wave kernel: a group is one fragment load and one MFMA there,
        // and the helper waves' barriers cost a full chip more than the run saves: 16 -> 16 on 4912 tiles 22.6 / 25.8 us)
        if (waves == 1 && a.book.tile_koff && a.book.middle_run && (NS * CT >= 4 || ntiles <= 1024)) {
            int rc = set_lds(conv_wave_run_kernel<DT, NS, CT, MASKED>, lds);
            if (rc) return rc;
            hipLaunchKernelGGL((conv_wave_run_kernel<DT, NS, CT, MASKED>), dim3(sph_xcd_grid(ntiles)), dim3(kWave * (1 + kRunHelpers)),
                               lds, st, a, nwtot);
            return sph_check_launch("sph_conv_apply");
        }
    }
    int rc = set_lds(conv_wave_kernel<DT, NS, CT, MASKED>, lds);
    if (rc) return rc;
    hipLaunchKernelGGL((conv_wave_kernel<DT, NS, CT, MASKED>), dim3(sph_xcd_grid(ntiles)), dim3(waves * kWave), lds, st, a, nwtot);
    return sph_check_launch("sph_conv_apply");
}

template <sph_dtype DT, int NS, int CT>
int launch_conv_wave_m(const ConvArgs &a, int nwtot, int ntiles, hipStream_t st)
{
    // rows that end inside the last 64-byte step need its tail masked
    if (a.row_bytes < NS * 64) return launch_conv_wave<DT, NS, CT, true>(a, nwtot, ntiles, st);
    return launch_conv_wave<DT, NS, CT, false>(a, nwtot, ntiles, st);
}

template <sph_dtype DT, int NS>
int launch_conv_wave_ct(const ConvArgs &a, int nwtot, int ntiles, hipStream_t st)
{
    switch (nwtot) { // at most two waves per workgroup (launch bound of the kernel)
    case 1: return launch_conv_wave_m<DT, NS, 1>(a, nwtot, ntiles, st);
    case 2: return launch_conv_wave_m<DT, NS, 2>(a, nwtot, ntiles, st);
    default:
        // int8 rows are 64 bytes: on a full chip two waves per tile (32 columns each, the rows gathered twice)
        // are faster than one (configuration 5a: 50.5 -> 45.5 us); with 128-byte fp16 rows they are slower (123 -> 151 us)
        // (up to 64 output columns only: more would be four waves, beyond the kernel's launch bound).  A book with a
        // run at its middle offset takes one wave of 64 columns and two helper waves instead (5a: 36.7 -> 35.1 us).
        if constexpr (DT == SPH_I8)
            if (ntiles > 1024 && nwtot <= 4 && !a.book.middle_run) return launch_conv_wave_m<DT, NS, 2>(a, nwtot, ntiles, st);
        return launch_conv_wave_m<DT, NS, 4>(a, nwtot, ntiles, st);
    }
}

template <sph_dtype DT, int NS, int CT, bool MASKED>
int launch_conv_rows_m(const ConvArgs &a, int nwtot, int ntiles, hipStream_t st)
{
    const int waves = (nwtot + CT - 1) / CT;
    // fewer tiles than SIMDs: the kernel lasts one wave's chain, so four waves share a tile's rows
    const int ws = ntiles <= 1024 ? 4 : 1;
    // the table, and for 128-byte rows a wave's exchange buffer (up to 4 chunk sets of 16 rows x 80 bytes)
    const size_t lds = (size_t)a.book.KV * R * sizeof(int32_t) + (NS >= 2 ? (size_t)waves * ws * 4 * SPH_GROUP * 80 : 0);
    const dim3 grid(sph_xcd_grid(ntiles)), block(waves * ws * kWave);
    if constexpr (NS == 1 && CT <= 2) {
        // one K step, up to 32 columns: the gathered rows go through an LDS window (with 64 columns the
        // accumulators leave no registers for that kernel's pipeline)
        if (ws == 1 && waves == 1) {
            hipLaunchKernelGGL((conv_rows_win_kernel<DT, CT, MASKED>), grid, dim3(kWave), kWinTab + kWinBytes + 64, st, a, nwtot);
            return sph_check_launch("sph_conv_apply");
        }
    }
    if (ws == 4) hipLaunchKernelGGL((conv_rows_kernel_split<DT, NS, CT, MASKED>), grid, block, lds, st, a, nwtot);
    else if constexpr (CT >= 4) hipLaunchKernelGGL((conv_rows_kernel_w2<DT, NS, CT, MASKED>), grid, block, lds, st, a, nwtot);
    else if constexpr (CT == 2) hipLaunchKernelGGL((conv_rows_kernel_w3<DT, NS, CT, MASKED>), grid, block, lds, st, a, nwtot);
    else hipLaunchKernelGGL((conv_rows_kernel_w4<DT, NS, CT, MASKED>), grid, block, lds, st, a, nwtot);
    return sph_check_launch("sph_conv_apply");
}

template <sph_dtype DT, int NS, int CT>
int launch_conv_rows(const ConvArgs &a, int nwtot, int ntiles, hipStream_t st)
{
    if (a.row_bytes < NS * 64) return launch_conv_rows_m<DT, NS, CT, true>(a, nwtot, ntiles, st);
    return launch_conv_rows_m<DT, NS, CT, false>(a, nwtot, ntiles, st);
}

template <sph_dtype DT, int NS>
int launch_conv_rows_ct(const ConvArgs &a, int nwtot, int ntiles, hipStream_t st)
{
    switch (nwtot) {
    case 1: return launch_conv_rows<DT, NS, 1>(a, nwtot, ntiles, st);
    case 2: return launch_conv_rows<DT, NS, 2>(a, nwtot, ntiles, st);
    default: return launch_conv_rows<DT, NS, 4>(a, nwtot, ntiles, st);
    }
}

template <sph_dtype DT, int NW>
int launch_conv(const ConvArgs &a, int ntiles, hipStream_t st)
{
    // by stationary row, when the book keeps that form (rows of up to 128 bytes; its table must fit LDS)
    if (rows_path_ok(a)) {
        if (a.nsteps == 1) return launch_conv_rows_ct<DT, 1>(a, NW, ntiles, st);
        return launch_conv_rows_ct<DT, 2>(a, NW, ntiles, st);
    }
    // the one-wave-per-tile kernel addresses the feature array through a buffer descriptor with 31-bit offsets
    // made by a 24-bit multiply
    const bool small = (double)a.feat_rows * a.row_bytes < 2147483648.0 && a.feat_rows < (1 << 24);
    if (a.aligned_in && a.feat_rows > 0 && small) {
        switch (a.nsteps) {
        case 1: return launch_conv_wave_ct<DT, 1>(a, NW, ntiles, st);
        case 2: return launch_conv_wave_ct<DT, 2>(a, NW, ntiles, st);
        case 4: return launch_conv_wave_ct<DT, 4>(a, NW, ntiles, st);
        default: break;
        }
    }
    return launch_conv_ns<DT, NW, 0>(a, ntiles, st); // rows not a multiple of 16 bytes, or more than 256 bytes, or 2 GiB of them
}

template <sph_dtype DT>
int launch_conv_nw(const ConvArgs &a, int nw, int ntiles, hipStream_t st)
{
    switch (nw) {
    case 1: return launch_conv<DT, 1>(a, ntiles, st);
    case 2: return launch_conv<DT, 2>(a, ntiles, st);
    case 4: return launch_conv<DT, 4>(a, ntiles, st);
    default: return launch_conv<DT, 8>(a, ntiles, st);
    }
}

// 16-channel tiles of one side of the widest block: 1, 2 or 4
inline int wgrad_tiles(int channels)
{
    const int t = sph_div_up(channels < kWsBlock ? channels : kWsBlock, 16);
    return t <= 1 ? 1 : (t <= 2 ? 2 : 4);
}
inline size_t wgrad_wave_lds(int e, int mi, int ni)
{
    const int pb = (e == 2 ? 2 : 1) * SPH_GROUP;
    const size_t stage = (size_t)4 * pb * ((mi * 16 * e + 16) + (ni * 16 * e + 16));
    const size_t red = (size_t)2 * mi * ni * kWave * 4 * sizeof(float); // two waves' blocks at once
    return stage > red ? stage : red;
}
inline int wgrad_wave_chunks(int ntiles) { return ntiles < 1 ? 1 : sph_div_up(ntiles, kWsTiles); }
inline bool wgrad_wave_ok(sph_dtype dt, int iC, int oC)
{
    const int e = elem_size(dt);
    return (iC * e) % 16 == 0 && (oC * e) % 16 == 0;
}

template <sph_dtype DT>
int launch_wgrad(const WgradArgs &a0, void *dw, bool f32_out, hipStream_t st)
{
    typedef typename Traits<DT>::elem elem;
    const int KV = a0.book.KV;
    const int per_k = a0.iC * a0.oC;
    const long total = (long)KV * per_k;
    const bool aligned = ((uintptr_t)a0.feat % 16 == 0) && ((uintptr_t)a0.dout % 16 == 0);
    const bool small = (double)a0.in_rows * a0.iC * sizeof(elem) < 4294967296.0 &&
                       (double)a0.out_rows * a0.oC * sizeof(elem) < 4294967296.0 &&
                       (double)a0.ntiles * a0.cap * SPH_GROUP < 2147483648.0;
    if (wgrad_wave_ok(DT, a0.iC, a0.oC) && aligned && small && a0.in_rows > 0 && a0.out_rows > 0) {
        WgradArgs a = a0;
        const int sb = sph_div_up(a.iC, kWsBlock) * sph_div_up(a.oC, kWsBlock);
        a.nchunk = wgrad_wave_chunks(a.ntiles);
        // the centre offset's chain is what a small book's kernel lasts: eight workgroups share it there; on large
        // books four, which halves the partial blocks to write and add (measured: headline scan 29 -> 23.5 us with
        // eight, 8 scans 109 -> 115 us)
        a.nslice = a.nchunk <= 16 ? kWsSlices : kWsSlices / 2;
        a.nslots = KV * a.nchunk * a.nslice;
        a.flags = (int *)(a.partial + (size_t)a.nslots * sb * kWsBlock * kWsBlock);
        // later slices for every offset only where the whole grid stays small (measured: a full 4x4x128x4 grid, one
        // chunk, 15 us with them and 33 us without; 8 chunks 32 against 35 us; from 12 chunks on the shorter grid wins)
        a.all_slices = KV * a.nchunk * 4 <= 1024;
        const dim3 grid(sph_xcd_grid(KV * a.nchunk) + (a.nslice - 1) * a.nchunk * (a.all_slices ? KV : 1), sb);
        const int mi = wgrad_tiles(a.iC), ni = wgrad_tiles(a.oC);
        int rc;
#define SPH_WGRAD_CASE(M, N)                                                                      \
    if (mi == M && ni == N) {                                                                     \
        const size_t lds = wgrad_wave_lds((int)sizeof(elem), M, N);                               \
        rc = set_lds(wgrad_wave_kernel<DT, M, N>, lds);                                           \
        if (rc) return rc;                                                                        \
        hipLaunchKernelGGL((wgrad_wave_kernel<DT, M, N>), grid, dim3(256), lds, st, a);           \
    }
        SPH_WGRAD_CASE(1, 1) SPH_WGRAD_CASE(1, 2) SPH_WGRAD_CASE(1, 4)
        SPH_WGRAD_CASE(2, 1) SPH_WGRAD_CASE(2, 2) SPH_WGRAD_CASE(2, 4)
        SPH_WGRAD_CASE(4, 1) SPH_WGRAD_CASE(4, 2) SPH_WGRAD_CASE(4, 4)
#undef SPH_WGRAD_CASE
        rc = sph_check_launch("sph_conv_wgrad");
        if (rc) return rc;
        if (f32_out)
            hipLaunchKernelGGL(wgrad_slot_reduce_kernel<float>, dim3((unsigned)(mi * ni * 2), sb, KV), dim3(256), 0, st,
                               a.partial, a.flags, a.nchunk * a.nslice, a.iC, a.oC, mi, ni, (float *)dw);
        else
            hipLaunchKernelGGL(wgrad_slot_reduce_kernel<elem>, dim3((unsigned)(mi * ni * 2), sb, KV), dim3(256), 0, st,
                               a.partial, a.flags, a.nchunk * a.nslice, a.iC, a.oC, mi, ni, (elem *)dw);
        return sph_check_launch("sph_conv_wgrad(reduce)");
    }
    const WgradArgs &a = a0;
    constexpr int LDP = 4 * Traits<DT>::KW + 16 / (int)sizeof(elem);
    const int iCp = (a.iC + 15) & ~15, oCp = (a.oC + 15) & ~15;
    size_t lds = (size_t)(iCp + oCp) * LDP * sizeof(elem);
    hipLaunchKernelGGL(wgrad_kernel<DT>, dim3(KV * a.nchunk), dim3(kWgThreads), lds, st, a);
    int rc = sph_check_launch("sph_conv_wgrad");
    if (rc) return rc;
    if (f32_out)
        hipLaunchKernelGGL(wgrad_reduce_kernel<float>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                           a.partial, KV, a.nchunk, per_k, (float *)dw);
    else
        hipLaunchKernelGGL(wgrad_reduce_kernel<elem>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                           a.partial, KV, a.nchunk, per_k, (elem *)dw);
    return sph_check_launch("sph_conv_wgrad(reduce)");
}

inline int book_has_groups(const sph_book *b) { return b->grp_k && b->grp_gather && b->grp_owner; }

// the groups may be missing (all three arrays null) in a book that keeps its pairs by row
inline int book_ok(const sph_book *b)
{
    return b && b->tile_ngrp && b->tile_koff && b->rows >= 0 && b->KV > 0 && b->KV <= SPH_MAX_KV &&
           (book_has_groups(b) || (b->tile_nbr && !b->grp_k && !b->grp_gather && !b->grp_owner));
}

} // namespace

SPH_EXPORT size_t sph_weight_packed_bytes(sph_dtype dt, int KV, int kdim, int ndim)
{
    if (KV <= 0 || kdim <= 0 || ndim <= 0 || (int)dt < 0 || (int)dt > 3) return 0;
    return (size_t)KV * num_steps(dt, kdim) * pad_waves(ndim) * kWave * 16;
}

SPH_EXPORT int sph_weight_pack(sph_dtype dt, const void *w, int KV, int kdim, int ndim, long stride_k,
                               long stride_kk, long stride_n, void *packed, void *stream)
{
    int rc = sph_pack_args_ok("sph_weight_pack", dt, w, packed, KV, kdim, ndim);
    if (rc) return rc;
    const SphPackJob p = sph_pack_job(dt, w, KV, kdim, ndim, stride_k, stride_kk, stride_n, packed);
    hipLaunchKernelGGL(pack_weight_kernel, dim3((unsigned)((p.total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, p);
    return sph_check_launch("sph_weight_pack");
}

SPH_EXPORT int sph_conv_apply(sph_dtype dt, const void *feature, int feature_rows, int kdim,
                              const void *packed_w, int ndim, const sph_book *book,
                              const sph_epilogue *epi, void *out, void *stream)
{
    SPH_REQUIRE(book_ok(book), SPH_ERR_ARG, "sph_conv_apply: bad book");
    SPH_REQUIRE(packed_w && feature_rows >= 0 && (feature_rows == 0 || feature), SPH_ERR_ARG, "sph_conv_apply: null pointer");
    SPH_REQUIRE((int)dt >= 0 && (int)dt <= 3, SPH_ERR_ARG, "sph_conv_apply: unknown dtype %d", (int)dt);
    SPH_REQUIRE(kdim > 0 && kdim <= SPH_MAX_CHANNELS, SPH_ERR_UNSUPPORTED,
                "sph_conv_apply: %d input channels not in 1..%d", kdim, SPH_MAX_CHANNELS);
    SPH_REQUIRE(ndim > 0 && ndim <= 128, SPH_ERR_UNSUPPORTED, "sph_conv_apply: %d output channels not in 1..128", ndim);
    SPH_REQUIRE(dt != SPH_I8 || (epi && epi->scale), SPH_ERR_ARG, "sph_conv_apply: int8 needs per-channel scales");
    if (book->rows == 0) return SPH_OK;
    SPH_REQUIRE(out, SPH_ERR_ARG, "sph_conv_apply: null output");
    const int es = elem_size(dt);
    ConvArgs a;
    a.feat = (const char *)feature;
    a.feat_rows = feature_rows;
    a.kdim = kdim;
    a.row_bytes = kdim * es;
    a.wp = (const char *)packed_w;
    a.nsteps = num_steps(dt, kdim);
    a.ndim = ndim;
    a.book = *book;
    a.cap = sph_book_cap(book->KV);
    a.scale = epi ? epi->scale : nullptr;
    a.shift = epi ? epi->shift : nullptr;
    a.relu = epi ? epi->relu : 0;
    a.out = (char *)out;
    a.aligned_in = (a.row_bytes % 16 == 0) && ((uintptr_t)feature % 16 == 0);
    a.aligned_out = ((ndim * es) % 16 == 0) && ((uintptr_t)out % 16 == 0);
    SPH_REQUIRE((uintptr_t)packed_w % 16 == 0, SPH_ERR_ARG, "sph_conv_apply: packed weight must be 16-byte aligned");
    SPH_REQUIRE(book_has_groups(book) || rows_path_ok(a), SPH_ERR_ARG,
                "sph_conv_apply: the book holds no groups and this call cannot go by rows (rows of 16-byte multiples up to "
                "128 bytes, 16-byte aligned arrays)");
    const int nw = pad_waves(ndim), nt = sph_book_tiles(book->rows);
    hipStream_t st = (hipStream_t)stream;
    switch (dt) {
    case SPH_F32: return launch_conv_nw<SPH_F32>(a, nw, nt, st);
    case SPH_F16: return launch_conv_nw<SPH_F16>(a, nw, nt, st);
    case SPH_BF16: return launch_conv_nw<SPH_BF16>(a, nw, nt, st);
    default: return launch_conv_nw<SPH_I8>(a, nw, nt, st);
    }
}

SPH_EXPORT size_t sph_wgrad_partial_elems(int KV, int iC, int oC, int out_rows)
{
    if (KV <= 0 || iC <= 0 || oC <= 0) return 0;
    const int ntiles = sph_book_tiles(out_rows);
    const size_t general = (size_t)KV * wgrad_chunks(ntiles) * iC * oC;
    const size_t slots = (size_t)KV * wgrad_wave_chunks(ntiles) * kWsSlices;
    const size_t blocks = (size_t)sph_div_up(iC, kWsBlock) * sph_div_up(oC, kWsBlock);
    const size_t fast = slots * blocks * kWsBlock * kWsBlock + slots; // 64x64 blocks + one flag word per slot
    return general > fast ? general : fast;
}

SPH_EXPORT int sph_conv_wgrad(sph_dtype dt, const void *feature, int in_rows, int iC, const void *d_out,
                              int oC, const sph_book *fwd_book, float *partial, void *d_weight, int d_weight_f32,
                              void *stream)
{
    SPH_REQUIRE(book_ok(fwd_book) && book_has_groups(fwd_book), SPH_ERR_ARG, "sph_conv_wgrad: bad book (it must hold its groups)");
    SPH_REQUIRE(partial && d_weight, SPH_ERR_ARG, "sph_conv_wgrad: null pointer");
    SPH_REQUIRE(dt == SPH_F32 || dt == SPH_F16 || dt == SPH_BF16, SPH_ERR_UNSUPPORTED,
                "sph_conv_wgrad: dtype %d has no weight gradient", (int)dt);
    SPH_REQUIRE(iC > 0 && iC <= 128 && oC > 0 && oC <= 128, SPH_ERR_UNSUPPORTED,
                "sph_conv_wgrad: channels %d->%d not in 1..128", iC, oC);
    SPH_REQUIRE((in_rows == 0 || feature) && (fwd_book->rows == 0 || d_out), SPH_ERR_ARG, "sph_conv_wgrad: null pointer");
    WgradArgs a;
    a.feat = (const char *)feature;
    a.in_rows = in_rows;
    a.iC = iC;
    a.dout = (const char *)d_out;
    a.out_rows = fwd_book->rows;
    a.oC = oC;
    a.book = *fwd_book;
    a.cap = sph_book_cap(fwd_book->KV);
    a.ntiles = sph_book_tiles(fwd_book->rows);
    a.nchunk = wgrad_chunks(a.ntiles);
    a.partial = partial;
    a.nslots = 0;
    a.flags = nullptr;
    a.all_slices = 0;
    a.nslice = kWsSlices;
    hipStream_t st = (hipStream_t)stream;
    switch (dt) {
    case SPH_F32: return launch_wgrad<SPH_F32>(a, d_weight, true, st);
    case SPH_F16: return launch_wgrad<SPH_F16>(a, d_weight, d_weight_f32 != 0, st);
    default: return launch_wgrad<SPH_BF16>(a, d_weight, d_weight_f32 != 0, st);
    }
}
