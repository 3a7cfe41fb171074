// Weight packing shared by the stand-alone kernel (sph_weight_pack) and by the rule kernel
// launch that carries it as extra workgroups (sph_rules_build_pack).
//
// packed[k][step][ntile][lane][KW] holds weight element (k, kk, n) with
//   kk = step*4*KW + KW*(lane/16) + j,  n = ntile*16 + lane%16,  KW = 16 / element size,
// zero padded: the order in which an MFMA lane reads its 16-byte operand fragment.
// The copy is a permutation of elements, so it only depends on the element size.
#pragma once
#include "common.h"

struct SphPackJob {
    const void *w;
    void *packed;
    int elem_size;          // 1, 2 or 4 bytes
    int KV, kdim, ndim, nsteps, ntn;
    long sk, skk, sn;       // element strides of w over (k, kk, n)
    long total;             // elements of the packed copy
};

static inline int sph_elem_size(sph_dtype dt) { return dt == SPH_F32 ? 4 : (dt == SPH_I8 ? 1 : 2); }
static inline int sph_frag_elems(sph_dtype dt) { return 16 / sph_elem_size(dt); }
// output-column tiles of 16, padded to 1, 2, 4 or 8
static inline int sph_pad_waves(int ndim)
{
    int nt = sph_div_up(ndim, 16);
    return nt <= 1 ? 1 : (nt <= 2 ? 2 : (nt <= 4 ? 4 : 8));
}
// MFMA super steps (64 bytes of every row each) of a contraction over kdim elements
static inline int sph_num_steps(sph_dtype dt, int kdim) { return sph_div_up(kdim, 4 * sph_frag_elems(dt)); }
static inline SphPackJob sph_pack_job(sph_dtype dt, const void *w, int KV, int kdim, int ndim, long sk, long skk,
                                      long sn, void *packed)
{
    SphPackJob p;
    p.w = w; p.packed = packed; p.elem_size = sph_elem_size(dt);
    p.KV = KV; p.kdim = kdim; p.ndim = ndim;
    p.nsteps = sph_num_steps(dt, kdim); p.ntn = sph_pad_waves(ndim);
    p.sk = sk; p.skk = skk; p.sn = sn;
    p.total = (long)KV * p.nsteps * p.ntn * 64 * sph_frag_elems(dt);
    return p;
}
// argument checks shared by the entry points that pack; returns 0 or an error code (message set)
static inline int sph_pack_args_ok(const char *who, sph_dtype dt, const void *w, void *packed, int KV, int kdim, int ndim)
{
    if (!w || !packed) { sph_set_error("%s: null pointer", who); return SPH_ERR_ARG; }
    if ((int)dt < 0 || (int)dt > 3) { sph_set_error("%s: unknown dtype %d", who, (int)dt); return SPH_ERR_ARG; }
    if (KV <= 0 || KV > SPH_MAX_KV) { sph_set_error("%s: kernel volume %d not in 1..%d", who, KV, SPH_MAX_KV); return SPH_ERR_UNSUPPORTED; }
    if (kdim <= 0 || kdim > SPH_MAX_CHANNELS) { sph_set_error("%s: %d input channels not in 1..%d", who, kdim, SPH_MAX_CHANNELS); return SPH_ERR_UNSUPPORTED; }
    if (ndim <= 0 || ndim > 128) { sph_set_error("%s: %d output channels not in 1..128", who, ndim); return SPH_ERR_UNSUPPORTED; }
    return SPH_OK;
}

#ifdef __HIPCC__
template <typename T>
__device__ __forceinline__ void sph_pack_elements(const SphPackJob &p, long i)
{
    constexpr int KW = 16 / (int)sizeof(T);
    if (i >= p.total) return;
    const int j = (int)(i % KW);
    long t = i / KW;
    const int lane = (int)(t % 64);
    t /= 64;
    const int nt = (int)(t % p.ntn);
    t /= p.ntn;
    const int st = (int)(t % p.nsteps);
    const int k = (int)(t / p.nsteps);
    const int kk = st * 4 * KW + KW * (lane >> 4) + j;
    const int n = nt * 16 + (lane & 15);
    T v = (T)0;
    if (kk < p.kdim && n < p.ndim) v = ((const T *)p.w)[k * p.sk + kk * p.skk + n * p.sn];
    ((T *)p.packed)[i] = v;
}

// element i of the job, whatever its type
__device__ __forceinline__ void sph_pack_element(const SphPackJob &p, long i)
{
    if (p.elem_size == 2) sph_pack_elements<uint16_t>(p, i);
    else if (p.elem_size == 4) sph_pack_elements<uint32_t>(p, i);
    else sph_pack_elements<uint8_t>(p, i);
}
#endif
