// Shared device/host helpers of libcherryq (gfx950 only).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cq {

constexpr int kTileCols = 256;  // output columns per workgroup tile (256 B of one byte row)
constexpr int kUnitK = 128;     // compacted normal positions per work unit
constexpr int kCherryUnit = 32; // cherry rows per work unit
constexpr int kXcds = 8;        // MI355X: 8 accelerator complex dies, workgroups dealt round-robin

__host__ __device__ constexpr int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Work decomposition shared by host launch code and kernels.
struct Plan {
    int tiles;          // column tiles of kTileCols
    int units_normal;   // ceil(Kn / 128)
    int units_total;    // units_normal + ceil(C / 32)
    int units_per_wg;   // consecutive units reduced inside one workgroup
    int splits;         // workgroups per column tile (split-K factor)
};

__host__ __device__ inline Plan make_plan(int K, int N, int C, int units_per_wg) {
    Plan p;
    p.tiles = ceil_div(N, kTileCols);
    p.units_normal = ceil_div(K - C, kUnitK);
    p.units_total = p.units_normal + ceil_div(C, kCherryUnit);
    p.units_per_wg = units_per_wg;
    p.splits = ceil_div(p.units_total, units_per_wg);
    if (p.splits < 1) p.splits = 1;
    return p;
}

// Workgroups are dealt to the 8 XCDs round-robin by their linear id.  Renumber so that
// consecutive logical ids (all K-splits of one column tile) run on the same XCD and share
// its L2 for the activation vector, the scales and the split-K partials.
__device__ inline int xcd_remap(int bid, int total) {
    int per = total / kXcds;
    int body = per * kXcds;
    if (bid >= body) return bid;  // ragged tail keeps its id
    return (bid % kXcds) * per + bid / kXcds;
}

__device__ inline float to_float(__half h) { return __half2float(h); }
__device__ inline float to_float(float f) { return f; }
template <typename T> __device__ inline T from_float(float f);
template <> __device__ inline __half from_float<__half>(float f) { return __float2half_rn(f); }
template <> __device__ inline float from_float<float>(float f) { return f; }

// upper bound of k in (idx[m] - m): number of cherry columns at or before the k-th normal
// column, so that normal[k] = k + gather_offset(k).
template <typename IDX>
__device__ inline int gather_offset(const IDX *__restrict__ idx, int C, int k) {
    int lo = 0, hi = C;
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        bool le = (int)idx[mid] - mid <= k;
        lo = le ? mid + 1 : lo;
        hi = le ? hi : mid;
    }
    return lo;
}

// Split-K epilogue.  Every workgroup of a column tile stores its partial sums, then takes a
// ticket; the workgroup that draws the last ticket adds the partials in split order (a fixed
// order, so results do not depend on scheduling) and writes `mul` with a single rounding.
// `vals[b][c]` are this thread's partial sums for columns n0 + c, batch rows b < B.
template <typename IO, int MAXB, int COLS>
__device__ inline void splitk_finish(float (&vals)[MAXB][COLS], int B, int N, int n0, bool active,
                                     int tile, int split, int splits, float *__restrict__ partial,
                                     unsigned *__restrict__ tickets, IO *__restrict__ mul,
                                     int accumulate) {
    if (splits > 1) {
        if (active) {
#pragma unroll
            for (int b = 0; b < MAXB; b++)
                if (b < B) {
                    float *p = partial + ((size_t)split * B + b) * N + n0;
#pragma unroll
                    for (int c = 0; c < COLS; c++) p[c] = vals[b][c];
                }
        }
        __shared__ int s_last;
        __threadfence();
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned old = __hip_atomic_fetch_add(&tickets[tile], 1u, __ATOMIC_ACQ_REL,
                                                  __HIP_MEMORY_SCOPE_AGENT);
            s_last = (old == (unsigned)(splits - 1));
        }
        __syncthreads();
        if (!s_last) return;
        __threadfence();
        if (active) {
#pragma unroll
            for (int b = 0; b < MAXB; b++)
                if (b < B) {
#pragma unroll
                    for (int c = 0; c < COLS; c++) vals[b][c] = 0.f;
                    for (int s = 0; s < splits; s++) {
                        const float *p = partial + ((size_t)s * B + b) * N + n0;
#pragma unroll
                        for (int c = 0; c < COLS; c++)
                            vals[b][c] += __builtin_nontemporal_load(p + c);
                    }
                }
        }
        if (threadIdx.x == 0)
            __hip_atomic_store(&tickets[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (active) {
#pragma unroll
        for (int b = 0; b < MAXB; b++)
            if (b < B) {
                IO *o = mul + (size_t)b * N + n0;
#pragma unroll
                for (int c = 0; c < COLS; c++) {
                    float v = vals[b][c];
                    if (accumulate) v += to_float(o[c]);
                    o[c] = from_float<IO>(v);
                }
            }
    }
}

}  // namespace cq
