// Device code of the grouped convolution (one wave per tile of 128 stationary rows and up to 64 output columns)
// that more than one translation unit uses: conv.hip wraps it into the kernel that reads the tile's groups from a
// rule book in global memory, fused.hip into the kernel that has just made them in LDS.
#pragma once
#include "common.h"
#include "pack.h"
#include "tile_consts.h"

namespace {



typedef int int4v __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));

template <sph_dtype DT> struct Traits;
template <> struct Traits<SPH_F32> {
    typedef float elem;
    typedef float4v acc4;
    static constexpr int KW = 4; // elements per 16-byte fragment
};
template <> struct Traits<SPH_F16> {
    typedef _Float16 elem;
    typedef float4v acc4;
    static constexpr int KW = 8;
};
template <> struct Traits<SPH_BF16> {
    typedef __bf16 elem;
    typedef float4v acc4;
    static constexpr int KW = 8;
};
template <> struct Traits<SPH_I8> {
    typedef int8_t elem;
    typedef int4v acc4;
    static constexpr int KW = 16;
};

// One "super step" consumes 64 bytes of every gathered row: lane l supplies the
// 16 bytes at offset 16*(l/16) of row l%16 (A) / of column l%16 (B).  Any
// assignment of K indices to lanes is valid as long as A and B agree.
template <sph_dtype DT>
__device__ __forceinline__ typename Traits<DT>::acc4 mfma_step(int4v a, int4v b, typename Traits<DT>::acc4 d);

template <>
__device__ __forceinline__ float4v mfma_step<SPH_F32>(int4v a, int4v b, float4v d)
{
    const float4v af = __builtin_bit_cast(float4v, a), bf = __builtin_bit_cast(float4v, b);
    d = __builtin_amdgcn_mfma_f32_16x16x4f32(af.x, bf.x, d, 0, 0, 0);
    d = __builtin_amdgcn_mfma_f32_16x16x4f32(af.y, bf.y, d, 0, 0, 0);
    d = __builtin_amdgcn_mfma_f32_16x16x4f32(af.z, bf.z, d, 0, 0, 0);
    d = __builtin_amdgcn_mfma_f32_16x16x4f32(af.w, bf.w, d, 0, 0, 0);
    return d;
}
template <>
__device__ __forceinline__ float4v mfma_step<SPH_F16>(int4v a, int4v b, float4v d)
{
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), d, 0, 0, 0);
}
template <>
__device__ __forceinline__ float4v mfma_step<SPH_BF16>(int4v a, int4v b, float4v d)
{
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8, a), __builtin_bit_cast(bf8, b), d, 0, 0, 0);
}
template <>
__device__ __forceinline__ int4v mfma_step<SPH_I8>(int4v a, int4v b, int4v d)
{
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, d, 0, 0, 0);
}

struct ConvArgs {
    const char *feat;
    int feat_rows, kdim, row_bytes;
    const char *wp;
    int nsteps, ndim;
    sph_book book;
    int cap;
    const float *scale, *shift;
    int relu;
    char *out;
    int aligned_in, aligned_out;
};

// can sph_conv_apply walk this call by stationary row?
inline bool rows_path_ok(const ConvArgs &a)
{
    return a.aligned_in && a.aligned_out && a.feat_rows > 0 && a.book.tile_nbr && (a.nsteps == 1 || a.nsteps == 2) &&
           (size_t)a.book.KV * R * sizeof(int32_t) <= 48 * 1024 && (uintptr_t)a.book.tile_nbr % 16 == 0;
}

template <sph_dtype DT>
__device__ __forceinline__ int4v load_a_frag(const ConvArgs &a, int in_row, int st, int lane)
{
    typedef typename Traits<DT>::elem elem;
    constexpr int KW = Traits<DT>::KW;
    int4v f = {0, 0, 0, 0};
    if ((unsigned)in_row >= (unsigned)a.feat_rows) return f;
    const int byte_off = st * 64 + (lane >> 4) * 16;
    const char *row = a.feat + (long)in_row * a.row_bytes;
    if (a.aligned_in) {
        if (byte_off < a.row_bytes) f = *(const int4v *)(row + byte_off);
    } else {
        union { int4v v; elem e[KW]; } u;
        u.v = f;
        const int c0 = byte_off / (int)sizeof(elem);
#pragma unroll
        for (int j = 0; j < KW; j++)
            if (c0 + j < a.kdim) u.e[j] = ((const elem *)row)[c0 + j];
        f = u.v;
    }
    return f;
}

template <sph_dtype DT>
__device__ __forceinline__ float epilogue_value(const ConvArgs &a, uint32_t raw, int c)
{
    float v;
    if (DT == SPH_I8)
        v = (float)(int32_t)raw;
    else
        v = __builtin_bit_cast(float, raw);
    if (a.scale) v = v * a.scale[c];
    if (DT != SPH_I8) {
        if (a.shift) v = v + a.shift[c];
        if (a.relu) v = v > 0.f ? v : 0.f;
    }
    return v;
}

template <sph_dtype DT>
__device__ __forceinline__ typename Traits<DT>::elem to_elem(float v)
{
    typedef typename Traits<DT>::elem elem;
    if (DT == SPH_I8) {
        float r = __builtin_rintf(v);
        r = r < -128.f ? -128.f : (r > 127.f ? 127.f : r);
        return (elem)(int)r;
    }
    return (elem)v;
}

// Adds the four accumulators a lane holds after a transposed MFMA (four consecutive
// output columns of ONE owner row) into the LDS tile with a single 16-byte
// read-modify-write.  The address range belongs to this wave only, so additions
// happen in program order and the sum is reproducible.  (LDS float atomics
// serialise per lane and measured 2x slower.)
template <sph_dtype DT>
__device__ __forceinline__ void acc_add4(uint32_t *p, typename Traits<DT>::acc4 d)
{
    typedef typename Traits<DT>::acc4 acc4;
    acc4 v = *(acc4 *)p;
    v += d;
    *(acc4 *)p = v;
}

// ---------------------------------------------------------------------------
// One wave per tile and per block of 64 output columns.
//
// At LiDAR sizes (a few hundred tiles) every workgroup of the grid is resident at
// once, so the kernel lasts as long as ONE tile's dependent chain; barriers and
// fragment exchange between waves only lengthen that chain.  Here a wave owns a
// tile (x 64 columns) outright: it gathers each group's rows once (16 B per lane,
// already MFMA operand order), loads the offset's weight fragments, and accumulates
// into its own LDS tile: the accumulator rows of the group's owners are read as the
// C operand of the MFMAs and written back.  No barrier, no atomics, summation order
// = book order.  Indices run two blocks ahead; gathers and weight fragments are
// requested three to four groups before their use, their address arithmetic is
// interleaved with the MFMAs.  Measured bounds of the loop at 64->64 fp16: the
// vector-memory return path (8 KiB of weight fragments + 2 KiB of rows per group),
// then the LDS read-MFMA-write chain, then the MFMAs themselves.
// ---------------------------------------------------------------------------
constexpr int kBlk = 4; // groups per pipeline block (4 x 16 index entries = one 64-lane load)
constexpr int kRsrcFlags = 0x00020000; // raw buffer descriptor, 32-bit data format

// Where a tile's groups come from.  load(g0, ...) requests the indices of groups g0 .. g0+3 (lane l: entry l%16 of
// group g0 + l/16; lanes 0..3: the groups' offsets) and returns raw values; finish(g0, ...) validates them one or
// two blocks later, just before they are used: touching a loaded value earlier would make the wave wait for it,
// and with it for every load issued before.  After finish: gi = gathered row or -1, ow = owner row inside the tile
// or -1, kk = offset (0 for groups behind the tile's last).
//
// The book in global memory, through buffer descriptors (a read beyond the tile's capacity returns zeros).
struct BookMeta {
    __amdgpu_buffer_rsrc_t r_gat, r_own, r_gk;
    int cap, ngrp, r0, nrows, feat_rows, KV;
    int skip_lo, skip_n; // groups [skip_lo, skip_lo + skip_n) of the book are somebody else's: group g >= skip_lo is the book's g + skip_n
    __device__ __forceinline__ BookMeta(const sph_book &book, int cap_, int tile, int ngrp_, int r0_, int nrows_, int feat_rows_,
                                        int skip_lo_ = 0, int skip_n_ = 0)
        : cap(cap_), ngrp(ngrp_), r0(r0_), nrows(nrows_), feat_rows(feat_rows_), KV(book.KV), skip_lo(skip_lo_), skip_n(skip_n_)
    {
        const long gb0 = (long)tile * cap;
        r_gat = __builtin_amdgcn_make_buffer_rsrc((void *)(book.grp_gather + gb0 * SPH_GROUP), 0, cap * SPH_GROUP * 4, kRsrcFlags);
        r_own = __builtin_amdgcn_make_buffer_rsrc((void *)(book.grp_owner + gb0 * SPH_GROUP), 0, cap * SPH_GROUP * 4, kRsrcFlags);
        r_gk = __builtin_amdgcn_make_buffer_rsrc((void *)(book.grp_k + gb0), 0, cap * 4, kRsrcFlags);
    }
    __device__ __forceinline__ int book_group(int g) const { return min(g < skip_lo ? g : g + skip_n, cap - 1); }
    __device__ __forceinline__ void load(int g0, int lane, int &gi, int &ow, int &kk) const
    {
        // lane l: entry l % 16 of group g0 + l / 16, inside this tile's capacity
        const int slot = (book_group(g0 + (lane >> 4)) * SPH_GROUP + (lane & 15)) * 4;
        gi = __builtin_amdgcn_raw_buffer_load_b32(r_gat, slot, 0, 0);
        ow = __builtin_amdgcn_raw_buffer_load_b32(r_own, slot, 0, 0);
        kk = __builtin_amdgcn_raw_buffer_load_b32(r_gk, book_group(g0 + (lane & (kBlk - 1))) * 4, 0, 0);
    }
    __device__ __forceinline__ void finish(int g0, int lane, int &gi, int &ow, int &kk) const
    {
        const int g = g0 + (lane >> 4);
        const int vow = ow - r0;
        const bool ok = g < ngrp && (unsigned)vow < (unsigned)nrows && (unsigned)gi < (unsigned)feat_rows;
        gi = ok ? gi : -1;
        ow = ok ? vow : -1;
        kk = (g0 + (lane & (kBlk - 1)) < ngrp && (unsigned)kk < (unsigned)KV) ? kk : 0;
    }
    // one slot of a run of groups (conv_run_store): gathered row or -1, owner row inside the tile
    __device__ __forceinline__ void slot(int s, int &gi, int &ow) const
    {
        const int off = min(s, cap * SPH_GROUP - 1) * 4;
        gi = __builtin_amdgcn_raw_buffer_load_b32(r_gat, off, 0, 0);
        ow = __builtin_amdgcn_raw_buffer_load_b32(r_own, off, 0, 0) - r0;
        const bool ok = (unsigned)ow < (unsigned)nrows && (unsigned)gi < (unsigned)feat_rows;
        gi = ok ? gi : -1;
    }
};

// The tile's groups in LDS, as the workgroup has just compacted them: gat[slot] = gathered row or -1,
// own[slot] = owner row inside the tile (any value where gat is -1), gk[group] = offset; `room` groups fit.
struct LdsMeta {
    const int32_t *gat;
    const unsigned char *own, *gk;
    int room, ngrp;
    __device__ __forceinline__ void load(int g0, int lane, int &gi, int &ow, int &kk) const
    {
        const int gs = min(g0, room - kBlk);
        gi = gat[gs * SPH_GROUP + lane];
        ow = own[gs * SPH_GROUP + lane];
        kk = gk[gs + (lane & (kBlk - 1))];
    }
    __device__ __forceinline__ void finish(int g0, int lane, int &gi, int &ow, int &kk) const
    {
        const bool inside = g0 <= room - kBlk;
        const bool ok = inside && g0 + (lane >> 4) < ngrp && gi >= 0;
        gi = ok ? gi : -1;
        ow = ok ? ow : -1;
        kk = (inside && g0 + (lane & (kBlk - 1)) < ngrp) ? kk : 0;
    }
    __device__ __forceinline__ void slot(int s, int &gi, int &ow) const
    {
        gi = gat[s];
        ow = own[s];
    }
};

// Clears the wave's CT*16 columns of the accumulator tile (and of the scratch row behind it).
template <int CT>
__device__ __forceinline__ void conv_wave_clear(uint32_t *s_acc, int LDW, int col0, int lane)
{
    for (int i = lane; i < (R + 1) * CT * 4; i += kWave)
        *(int4v *)&s_acc[(i / (CT * 4)) * LDW + col0 + (i % (CT * 4)) * 4] = int4v{0, 0, 0, 0};
}

// The tile's groups, one after the other, into the wave's columns [col0, col0 + CT*16) of s_acc ([R + 1][LDW]
// 32-bit words, cleared by the caller, by clear() below while the first indices are on their way, or by the other
// waves of the workgroup meanwhile: wait_clear then makes this wave meet them at that many barriers before its first
// sum).
//
// One group: the accumulator rows of the group's owners are requested first and are the C operand of the MFMAs
// (the matrix unit does the addition; adding the products with the vector ALU instead was measured 6 % slower:
// sixteen more instructions per group on a wave that has its SIMD to itself); once a step's MFMAs are issued its
// fragment registers take the fragments of the group two ahead (two sets of fragment registers; a ring of four
// sets requested three groups ahead is no faster and costs 64 registers), and the gathered rows' registers the
// same slot of the next block.  Everything a block of four groups needs from its indices -- accumulator
// addresses, byte offsets of the rows to gather -- is computed at the top of the block from eight lane permutes
// issued together, so no group waits for a permute of its own.
template <sph_dtype DT, int NS, int CT, bool MASKED, class Meta>
__device__ __forceinline__ void conv_wave_groups(const ConvArgs &a, int nwtot, const Meta &meta, int ngrp, uint32_t *s_acc,
                                                 int col0, int lane, bool clear, int wait_clear = 0)
{
    typedef typename Traits<DT>::acc4 acc4;
    const int LDW = nwtot * 16 + 4;
    // Every load of the loop goes through a buffer descriptor: the address is a scalar base plus a 32-bit lane
    // offset (plus a scalar offset for the weight's kernel offset), so no load costs 64-bit vector arithmetic,
    // and a read beyond the array returns zeros instead of faulting.  (The launcher sends arrays of 2 GiB or more,
    // or of 2^24 rows or more, to the general kernel: lane offsets are 31-bit and made by a 24-bit multiply.)
    const __amdgpu_buffer_rsrc_t r_feat = __builtin_amdgcn_make_buffer_rsrc((void *)a.feat, 0, a.feat_rows * a.row_bytes, kRsrcFlags);
    // weight fragment of (offset k, step st, column tile c): k*NS*nwtot + st*nwtot + c  (1 KiB each)
    const int wstep = nwtot * (kWave * 16);
    const __amdgpu_buffer_rsrc_t r_w = __builtin_amdgcn_make_buffer_rsrc((void *)a.wp, 0, a.book.KV * NS * wstep, kRsrcFlags);
    int woff[NS]; // lane offset of the wave's first column tile at step st
#pragma unroll
    for (int st = 0; st < NS; st++) woff[st] = st * wstep + (col0 / 16) * (kWave * 16) + lane * 16;
    const int lane_chunk = (lane >> 4) * 16;
    const int acc_lane = (col0 + (lane >> 4) * 4) * 4; // byte offset of the lane's four columns inside an accumulator row

    // Every load below is unconditional and straight-line (indices are clamped to
    // memory that is always allocated, results of invalid slots are discarded by
    // selects): the compiler can then count outstanding loads exactly and only waits
    // for the ones an instruction needs.
    // Gathers only load (from an address clamped into the feature array); slots that hold
    // no pair and the tail of rows shorter than the step are zeroed when the fragment is
    // used, not here -- a select on the loaded value would stall the wave on the load.
    auto load_a = [&](int row_off, int4v (&fa)[NS]) {
#pragma unroll
        for (int st = 0; st < NS; st++)
            fa[st] = __builtin_bit_cast(int4v, __builtin_amdgcn_raw_buffer_load_b128(r_feat, row_off + st * 64, 0, 0));
    };
    auto load_w = [&](int k, int4v (&fw)[NS][CT]) {
        const int wk = k * (NS * wstep); // scalar
#pragma unroll
        for (int st = 0; st < NS; st++)
#pragma unroll
            for (int c = 0; c < CT; c++)
                fw[st][c] = __builtin_bit_cast(int4v, __builtin_amdgcn_raw_buffer_load_b128(r_w, woff[st] + c * (kWave * 16), wk, 0));
    };
    // Byte offset of the row slot u of a block gathers (a row shorter than the step: the tail is the next row's,
    // masked later), and accumulator address of its pair: the owner's row, or the scratch row behind the tile for
    // a padding slot (which multiplies whatever row 0 holds): no branch, no select on data.
    auto row_offset = [&](int gi_blk, int u) -> int {
        const int in_row = __shfl(gi_blk, u * SPH_GROUP + (lane & 15), kWave);
        return (int)__umul24((unsigned)max(in_row, 0), (unsigned)a.row_bytes) + lane_chunk;
    };
    auto acc_ptr = [&](int ow_blk, int u) -> uint32_t * {
        const int rl = __shfl(ow_blk, u * SPH_GROUP + (lane & 15), kWave);
        return (uint32_t *)((char *)s_acc + (int)__umul24((unsigned)(rl >= 0 ? rl : R), (unsigned)(LDW * 4)) + acc_lane);
    };
    auto group_step = [&](int4v (&fw)[NS][CT], int4v (&fa)[NS], uint32_t *p, int k_next2, int row_next) {
        acc4 d[CT];
#pragma unroll
        for (int c = 0; c < CT; c++) d[c] = *(const acc4 *)(p + c * 16);
        const int wk2 = k_next2 * (NS * wstep); // scalar
#pragma unroll
        for (int st = 0; st < NS; st++) {
            int4v x = fa[st];
            if constexpr (MASKED) { // rows shorter than the steps, e.g. 4 fp32 channels = 16 of 64 bytes: zero the tail
                const bool live = st * 64 + (lane >> 4) * 16 < a.row_bytes;
                x = live ? x : int4v{0, 0, 0, 0};
            }
#pragma unroll
            for (int c = 0; c < CT; c++) d[c] = mfma_step<DT>(fw[st][c], x, d[c]);
#pragma unroll
            for (int c = 0; c < CT; c++)
                fw[st][c] = __builtin_bit_cast(int4v, __builtin_amdgcn_raw_buffer_load_b128(r_w, woff[st] + c * (kWave * 16), wk2, 0));
        }
        load_a(row_next, fa);
#pragma unroll
        for (int c = 0; c < CT; c++) *(acc4 *)(p + c * 16) = d[c];
        __builtin_amdgcn_sched_group_barrier(0x100, CT, 0); // the accumulator reads first
#pragma unroll
        for (int i = 0; i < NS * CT; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // one MFMA
            __builtin_amdgcn_sched_group_barrier(0x006, 2, 0); // VALU / SALU
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); // one VMEM read
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    // Pipeline: indices run two blocks ahead, the gathers of slot u one block, fragments two groups.
    int gi_n, ow_n, k_n;       // indices of the next block
    int gi_nn, ow_nn, k_nn;    // indices of the block after it
    int4v a_0[NS], a_1[NS], a_2[NS], a_3[NS]; // gathered rows of slot u
    int4v w_0[NS][CT], w_1[NS][CT];           // fragments of the even / odd groups
    int ow_c, k_c;

    meta.load(0, lane, gi_n, ow_n, k_n);
    meta.load(kBlk, lane, gi_nn, ow_nn, k_nn);
    // clear the accumulator tile (and the scratch row) while the first indices are on their way
    if (clear) conv_wave_clear<CT>(s_acc, LDW, col0, lane);
    meta.finish(0, lane, gi_n, ow_n, k_n);
    // The first loads are issued in the order the loop issues them, pinned against the scheduler: the compiler
    // places one wait count per use for every path into the loop, and a start in another order would make every
    // block of the loop wait for more loads than it needs.
    {
        const int r0 = row_offset(gi_n, 0), r1 = row_offset(gi_n, 1), r2 = row_offset(gi_n, 2), r3 = row_offset(gi_n, 3);
        load_a(r0, a_0);
        __builtin_amdgcn_sched_barrier(0);
        load_w(__builtin_amdgcn_readlane(k_n, 0), w_0);
        __builtin_amdgcn_sched_barrier(0);
        load_a(r1, a_1);
        __builtin_amdgcn_sched_barrier(0);
        load_w(__builtin_amdgcn_readlane(k_n, 1), w_1);
        __builtin_amdgcn_sched_barrier(0);
        load_a(r2, a_2);
        load_a(r3, a_3);
        __builtin_amdgcn_sched_barrier(0);
    }
    // the other waves of the workgroup prepare the tile meanwhile: they start behind the first barrier (the tile is
    // clear by then) or have started already, and are done at the last
    for (int i = 0; i < wait_clear; i++) lds_barrier();
    for (int g0 = 0; g0 < ngrp; g0 += kBlk) {
        ow_c = ow_n; k_c = k_n;
        gi_n = gi_nn; ow_n = ow_nn; k_n = k_nn;
        meta.finish(g0 + kBlk, lane, gi_n, ow_n, k_n);   // loaded one block ago
        meta.load(g0 + 2 * kBlk, lane, gi_nn, ow_nn, k_nn);
        uint32_t *p_0 = acc_ptr(ow_c, 0), *p_1 = acc_ptr(ow_c, 1), *p_2 = acc_ptr(ow_c, 2), *p_3 = acc_ptr(ow_c, 3);
        const int r_0 = row_offset(gi_n, 0), r_1 = row_offset(gi_n, 1), r_2 = row_offset(gi_n, 2), r_3 = row_offset(gi_n, 3);
        __builtin_amdgcn_sched_barrier(0);
        group_step(w_0, a_0, p_0, __builtin_amdgcn_readlane(k_c, 2), r_0);
        group_step(w_1, a_1, p_1, __builtin_amdgcn_readlane(k_c, 3), r_1);
        group_step(w_0, a_2, p_2, __builtin_amdgcn_readlane(k_n, 0), r_2);
        group_step(w_1, a_3, p_3, __builtin_amdgcn_readlane(k_n, 1), r_3);
    }
}

// A run of groups of ONE offset shared out to helper waves: this wave takes groups g_first, g_first + g_step, ...
// below g_end (kRunGroups of them at most) of the compact arrays, loads the offset's fragments once, and STORES the
// products to the owners' accumulator rows: for the first offset a tile is given, before any sum is in the tile.
// Owner rows of one offset's groups are all different, so the helper waves' stores never meet (the scratch row
// takes the padding slots of all of them, and is never read for a result).  Rows without a pair at this offset
// (bit clear in `covered`, two 64-bit words) are zeroed by the thread that `zrow` names (-1: none).
template <sph_dtype DT, int NS, int CT, bool MASKED, int kRunGroups, class Meta>
__device__ __forceinline__ void conv_run_store(const ConvArgs &a, int nwtot, const Meta &m, int k, int g_first, int g_step,
                                               int g_end, int lane, uint32_t *s_acc, const unsigned long long *covered, int zrow,
                                               int zrow_step, bool wait_clear = false)
{
    typedef typename Traits<DT>::acc4 acc4;
    const int LDW = nwtot * 16 + 4;
    const __amdgpu_buffer_rsrc_t r_feat = __builtin_amdgcn_make_buffer_rsrc((void *)a.feat, 0, a.feat_rows * a.row_bytes, kRsrcFlags);
    const int wstep = nwtot * (kWave * 16);
    const __amdgpu_buffer_rsrc_t r_w = __builtin_amdgcn_make_buffer_rsrc((void *)a.wp, 0, a.book.KV * NS * wstep, kRsrcFlags);
    int4v fw[NS][CT], fa[kRunGroups][NS];
    int ow[kRunGroups], gi[kRunGroups];
#pragma unroll
    for (int j = 0; j < kRunGroups; j++) {
        const int g = g_first + j * g_step;
        m.slot(min(g, g_end - 1) * SPH_GROUP + (lane & 15), gi[j], ow[j]);
    }
#pragma unroll
    for (int st = 0; st < NS; st++)
#pragma unroll
        for (int c = 0; c < CT; c++)
            fw[st][c] = __builtin_bit_cast(int4v, __builtin_amdgcn_raw_buffer_load_b128(r_w, st * wstep + c * (kWave * 16) + lane * 16,
                                                                                          k * (NS * wstep), 0));
#pragma unroll
    for (int j = 0; j < kRunGroups; j++) {
        const bool ok = g_first + j * g_step < g_end && gi[j] >= 0;
        ow[j] = ok ? ow[j] : R;
        const int row_off = (int)__umul24((unsigned)(ok ? gi[j] : 0), (unsigned)a.row_bytes) + (lane >> 4) * 16;
#pragma unroll
        for (int st = 0; st < NS; st++)
            fa[j][st] = __builtin_bit_cast(int4v, __builtin_amdgcn_raw_buffer_load_b128(r_feat, row_off + st * 64, 0, 0));
    }
    // rows the offset does not reach start from zero (while the loads are on their way)
    if (covered)
        for (int r = zrow; r >= 0 && r < R; r += zrow_step)
            if (!((covered[r >> 6] >> (r & 63)) & 1ull))
                for (int i = 0; i < LDW / 4; i++) ((int4v *)(s_acc + r * LDW))[i] = int4v{0, 0, 0, 0};
    if (wait_clear) lds_barrier(); // somebody else clears the tile: not before that
#pragma unroll
    for (int j = 0; j < kRunGroups; j++) {
        acc4 prod[CT];
#pragma unroll
        for (int st = 0; st < NS; st++) {
            int4v x = fa[j][st];
            if constexpr (MASKED) {
                const bool live = st * 64 + (lane >> 4) * 16 < a.row_bytes;
                x = live ? x : int4v{0, 0, 0, 0};
            }
#pragma unroll
            for (int c = 0; c < CT; c++) prod[c] = mfma_step<DT>(fw[st][c], x, st == 0 ? acc4{0, 0, 0, 0} : prod[c]);
        }
        uint32_t *p = (uint32_t *)((char *)s_acc + (int)__umul24((unsigned)ow[j], (unsigned)(LDW * 4)) + (lane >> 4) * 16);
#pragma unroll
        for (int c = 0; c < CT; c++) *(acc4 *)(p + c * 16) = prod[c];
    }
}

// Epilogue: columns [col0, col0 + CT*16) of the tile's rows [0, nrows) from s_acc to out rows r0.., by the
// threads t, t + nthr, ... (a wave alone: t = lane, nthr = 64).
template <sph_dtype DT, int CT>
__device__ __forceinline__ void conv_wave_store(const ConvArgs &a, int nwtot, const uint32_t *s_acc, int col0, int r0, int nrows,
                                                int t, int nthr)
{
    typedef typename Traits<DT>::elem elem;
    const int LDW = nwtot * 16 + 4;
    constexpr int VE = 16 / (int)sizeof(elem);
    const int ncols = min(CT * 16, a.ndim - col0);
    if (ncols <= 0) return;
    elem *out = (elem *)a.out + (long)r0 * a.ndim + col0;
    const bool plain = DT != SPH_I8 && !a.scale && !a.shift && !a.relu;
    if (a.aligned_out && ncols % VE == 0) {
        // thread = (row within a pass, 16-byte chunk of the row): VE accumulators -> one 16-byte store
        const int cpr = ncols / VE;                 // chunks per row (power of two here)
        const int ch = t % cpr, rstep = nthr / cpr;
        if (plain) {
            // four rows per pass: their LDS reads are all issued before the first conversion
            constexpr int UR = 4;
            for (int row0 = t / cpr; row0 < nrows; row0 += UR * rstep) {
                float4v f[UR][VE / 4];
#pragma unroll
                for (int q = 0; q < UR; q++) {
                    const int row = min(row0 + q * rstep, nrows - 1);
#pragma unroll
                    for (int j = 0; j < VE / 4; j++)
                        f[q][j] = *(const float4v *)&s_acc[row * LDW + col0 + ch * VE + j * 4];
                }
#pragma unroll
                for (int q = 0; q < UR; q++) {
                    const int row = row0 + q * rstep;
                    union { int4v v; elem e[VE]; } u;
#pragma unroll
                    for (int j = 0; j < VE / 4; j++) {
                        u.e[4 * j] = (elem)f[q][j].x; u.e[4 * j + 1] = (elem)f[q][j].y;
                        u.e[4 * j + 2] = (elem)f[q][j].z; u.e[4 * j + 3] = (elem)f[q][j].w;
                    }
                    if (row < nrows) *(int4v *)(out + (long)row * a.ndim + ch * VE) = u.v;
                }
            }
        } else {
            // scale / shift of this thread's VE columns stay in registers for all rows
            float sc[VE], sh[VE];
#pragma unroll
            for (int j = 0; j < VE; j++) {
                sc[j] = a.scale ? a.scale[col0 + ch * VE + j] : 1.f;
                sh[j] = (DT != SPH_I8 && a.shift) ? a.shift[col0 + ch * VE + j] : 0.f;
            }
            const bool relu = DT != SPH_I8 && a.relu;
            constexpr int UR = VE > 8 ? 2 : 4;
            for (int row0 = t / cpr; row0 < nrows; row0 += UR * rstep) {
                int4v f[UR][VE / 4];
#pragma unroll
                for (int q = 0; q < UR; q++) {
                    const int row = min(row0 + q * rstep, nrows - 1);
#pragma unroll
                    for (int j = 0; j < VE / 4; j++)
                        f[q][j] = *(const int4v *)&s_acc[row * LDW + col0 + ch * VE + j * 4];
                }
#pragma unroll
                for (int q = 0; q < UR; q++) {
                    const int row = row0 + q * rstep;
                    union { int4v v; elem e[VE]; } u;
#pragma unroll
                    for (int j = 0; j < VE; j++) {
                        const int raw = j % 4 == 0 ? f[q][j / 4].x : (j % 4 == 1 ? f[q][j / 4].y : (j % 4 == 2 ? f[q][j / 4].z : f[q][j / 4].w));
                        float v = DT == SPH_I8 ? (float)raw : __builtin_bit_cast(float, raw);
                        v = v * sc[j] + sh[j];
                        if (relu) v = v > 0.f ? v : 0.f;
                        u.e[j] = to_elem<DT>(v);
                    }
                    if (row < nrows) *(int4v *)(out + (long)row * a.ndim + ch * VE) = u.v;
                }
            }
        }
    } else {
        for (int i = t; i < nrows * ncols; i += nthr) {
            int row = i / ncols, c = i - row * ncols;
            out[(long)row * a.ndim + c] = to_elem<DT>(epilogue_value<DT>(a, s_acc[row * LDW + col0 + c], col0 + c));
        }
    }
}

} // namespace
