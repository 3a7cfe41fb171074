// Scan of an int32 array in one pass over the data (decoupled look-back across workgroups).
//
// A workgroup takes a tile of 2048 elements: every thread loads 8 consecutive ones, the tile is scanned
// through registers, wave shuffles and LDS, the workgroup publishes the tile's aggregate in a status word,
// and its first wave looks back over the status words of the preceding tiles, 64 at a time, until it meets
// one that already knows its inclusive prefix.  Workgroups number themselves by a ticket, so every
// predecessor of a workgroup is already running and the look-back cannot wait for a workgroup that has not
// been scheduled.  The state (ticket + one 64-bit word per tile: flag in the two top bits, value in the low
// 32) is cleared by a fill kernel in front of the scan.  In-place (out == in) is allowed.
#pragma once
#include <climits>
#include <cstdint>
#include <hip/hip_runtime.h>

namespace sph_scan {

constexpr int kThreads = 256;
constexpr int kItems = 8;
constexpr int kTile = kThreads * kItems;
constexpr int kWaveSize = 64;
constexpr unsigned long long kAggregate = 1ull << 62; // value = the tile's own aggregate
constexpr unsigned long long kInclusive = 2ull << 62; // value = aggregate of everything up to and including the tile

struct Plus {
    static __host__ __device__ __forceinline__ int identity() { return 0; }
    static __host__ __device__ __forceinline__ int op(int a, int b) { return a + b; }
};
struct Max {
    static __host__ __device__ __forceinline__ int identity() { return INT_MIN; }
    static __host__ __device__ __forceinline__ int op(int a, int b) { return a > b ? a : b; }
};

inline int tiles(long n) { return (int)((n + kTile - 1) / kTile); }
// bytes of state a scan of n elements needs (a multiple of 256)
inline size_t state_bytes(long n) { return ((size_t)(2 + 2 * (long)tiles(n > 0 ? n : 1)) * 4 + 255) & ~(size_t)255; }

static __global__ void clear_state_kernel(int *state, int nints)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < nints) state[i] = 0;
}

// out[i] = op(in[0], ..., in[i]) (INCLUSIVE) or op(init, in[0], ..., in[i-1]) (exclusive; init counts first).
// *total (may be null; any address the GPU can write, e.g. pinned host memory) receives op over all n elements
// (and init, for an exclusive scan).
template <class OP, bool INCLUSIVE>
__global__ __launch_bounds__(kThreads) void scan_kernel(const int32_t *in, int32_t *out, long n, int *state, int init,
                                                        int32_t *total)
{
    __shared__ int s_ticket;
    __shared__ int s_wave[kThreads / kWaveSize];
    __shared__ int s_prefix;
    unsigned long long *status = (unsigned long long *)(state + 2);
    const int tid = threadIdx.x, lane = tid & (kWaveSize - 1), wave = tid / kWaveSize;
    if (tid == 0) s_ticket = atomicAdd(&state[0], 1);
    __syncthreads();
    const int t = s_ticket;
    const long base = (long)t * kTile + (long)tid * kItems;

    int v[kItems];
    if (base + kItems <= n && ((uintptr_t)in & 15) == 0) {
        const int4 a = *(const int4 *)(in + base), b = *(const int4 *)(in + base + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
#pragma unroll
        for (int i = 0; i < kItems; i++) v[i] = base + i < n ? in[base + i] : OP::identity();
    }
    // inclusive scan of the thread's items, then of the threads' totals over the wave
#pragma unroll
    for (int i = 1; i < kItems; i++) v[i] = OP::op(v[i - 1], v[i]);
    int incl = v[kItems - 1];
#pragma unroll
    for (int off = 1; off < kWaveSize; off <<= 1) {
        const int u = __shfl_up(incl, off, kWaveSize);
        if (lane >= off) incl = OP::op(u, incl);
    }
    if (lane == kWaveSize - 1) s_wave[wave] = incl;
    __syncthreads();
    int wave_excl = OP::identity(), agg = OP::identity();
#pragma unroll
    for (int w = 0; w < kThreads / kWaveSize; w++) {
        if (w < wave) wave_excl = OP::op(wave_excl, s_wave[w]);
        agg = OP::op(agg, s_wave[w]);
    }

    if (wave == 0) {
        int excl = INCLUSIVE ? OP::identity() : init; // what precedes the first tile (later tiles: their look-back)
        if (t > 0) {
            if (lane == 0)
                __hip_atomic_store(&status[t], kAggregate | (unsigned)agg, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            int acc = OP::identity();
            for (int b = t - 1;;) {
                const int idx = b - lane; // lane 0 looks at the nearest predecessor
                const unsigned long long w =
                    idx >= 0 ? __hip_atomic_load(&status[idx], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0ull;
                const unsigned long long flag = idx >= 0 ? w >> 62 : 3ull; // 3: before the first tile
                const unsigned long long done = __ballot(flag >= 2), empty = __ballot(flag == 0);
                const int fi = done ? __ffsll((long long)done) - 1 : kWaveSize; // nearest tile that ends the look-back
                const unsigned long long need = fi >= kWaveSize - 1 ? ~0ull : (2ull << fi) - 1ull;
                if (empty & need) { // a predecessor on the way has not published yet
                    __builtin_amdgcn_s_sleep(1);
                    continue;
                }
                // fold lanes fi..0 (farthest first, so that the order of a non-commutative use would be kept)
                int x = (lane <= fi && flag != 3ull) ? (int)(unsigned)w : OP::identity();
#pragma unroll
                for (int off = 1; off < kWaveSize; off <<= 1) {
                    const int u = __shfl_down(x, off, kWaveSize);
                    if (lane + off < kWaveSize) x = OP::op(u, x);
                }
                acc = OP::op(__shfl(x, 0, kWaveSize), acc);
                if (fi < kWaveSize) break;
                b -= kWaveSize;
            }
            excl = acc; // tile 0's published prefix already holds init
        }
        if (lane == 0) {
            __hip_atomic_store(&status[t], kInclusive | (unsigned)OP::op(excl, agg), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
            s_prefix = excl;
            if (total && t == (int)gridDim.x - 1) *total = OP::op(excl, agg);
        }
    }
    __syncthreads();
    // what precedes this thread's first item
    int before = OP::op(s_prefix, wave_excl);
    const int up = __shfl_up(incl, 1, kWaveSize);
    if (lane > 0) before = OP::op(before, up);
    int o[kItems];
#pragma unroll
    for (int i = 0; i < kItems; i++) {
        if (INCLUSIVE)
            o[i] = OP::op(before, v[i]);
        else
            o[i] = i == 0 ? before : OP::op(before, v[i - 1]);
    }
    if (base + kItems <= n && ((uintptr_t)out & 15) == 0) {
        *(int4 *)(out + base) = make_int4(o[0], o[1], o[2], o[3]);
        *(int4 *)(out + base + 4) = make_int4(o[4], o[5], o[6], o[7]);
    } else {
#pragma unroll
        for (int i = 0; i < kItems; i++)
            if (base + i < n) out[base + i] = o[i];
    }
}

// ints of the state that must be zero when the scan kernel starts
inline int state_ints(long n) { return 2 + 2 * tiles(n > 0 ? n : 1); }

// Enqueues the scan of n elements on st; state: state_bytes(n) bytes of device memory, 8-byte aligned.
// clear_state = false: a kernel enqueued before on the same stream has already zeroed the first state_ints(n) ints.
template <class OP, bool INCLUSIVE>
inline hipError_t launch(const int32_t *in, int32_t *out, long n, void *state, int init, hipStream_t st,
                         int32_t *total = nullptr, bool clear_state = true)
{
    if (n <= 0) return hipSuccess;
    const int nt = tiles(n), nints = state_ints(n);
    if (clear_state)
        hipLaunchKernelGGL(clear_state_kernel, dim3((nints + 255) / 256), dim3(256), 0, st, (int *)state, nints);
    hipLaunchKernelGGL((scan_kernel<OP, INCLUSIVE>), dim3(nt), dim3(kThreads), 0, st, in, out, n, (int *)state, init,
                       total);
    return hipGetLastError();
}

} // namespace sph_scan
