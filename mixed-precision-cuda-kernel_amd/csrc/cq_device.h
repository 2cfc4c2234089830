// Shared device/host helpers of libcherryq (gfx950 only).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cq {

constexpr int kTileCols = 256;  // output columns per workgroup tile (256 B of one byte row)
constexpr int kUnitK = 128;     // compacted normal positions per work unit (generic kernel)
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

__host__ __device__ inline Plan make_plan(int K, int N, int C, int units_per_wg, int unit_k = kUnitK) {
    Plan p;
    p.tiles = ceil_div(N, kTileCols);
    p.units_normal = ceil_div(K - C, unit_k);
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

// ---- cross-lane reductions without LDS ---------------------------------------------------------
// all-reduce over the 16 lanes of a DPP row by rotations 8, 4, 2, 1
__device__ inline float row_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x122, 0xf, 0xf, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x121, 0xf, 0xf, false));
    return v;
}

__device__ inline int row_max(int v) {
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x128, 0xf, 0xf, false));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x124, 0xf, 0xf, false));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x122, 0xf, 0xf, false));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x121, 0xf, 0xf, false));
    return v;
}

// v_permlane32_swap_b32 exchanges lanes 32..63 of its first operand with lanes 0..31 of its
// second; v_permlane16_swap_b32 exchanges the odd 16-lane rows of the first with the even rows
// of the second.  Written as inline assembly because the compiler builtin of this toolchain
// returns the first result twice; the s_nop pad the VALU->permlane-swap data hazards that the
// compiler cannot see through an asm statement.
//
// swap32_add: lanes < 32 return a[l] + a[l+32], lanes >= 32 return b[l-32] + b[l].
__device__ inline float swap32_add(float a, float b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return a + b;
}

// swap16_add: even rows return a[row] + a[row+1], odd rows return b[row-1] + b[row].
__device__ inline float swap16_add(float a, float b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return a + b;
}

// all lanes of the wavefront receive the sum / maximum over its 64 lanes
__device__ inline float wave_sum_all(float v) {
    v = row_sum(v);
    v = swap16_add(v, v);
    return swap32_add(v, v);
}

__device__ inline float row_max_f(float v) {
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false)));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, false)));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x122, 0xf, 0xf, false)));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x121, 0xf, 0xf, false)));
    return v;
}

__device__ inline float wave_max_all(float v) {
    v = row_max_f(v);
    float a = v, b = v;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    v = fmaxf(a, b);
    a = v;
    b = v;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return fmaxf(a, b);
}

// Split-K epilogue: one 64-bit atomic per output element.
//
// Each output element owns a 64-bit accumulator word in the workspace:
//     bits 63..8  running sum of the partial sums, two's-complement fixed point, 2^-34 units
//     bits  7..0  number of workgroups that have contributed so far
// A workgroup adds  (fixed(partial) << 8) + 1  with a single agent-scope atomic that returns
// the previous word.  Integer addition is associative, so the total does not depend on the order
// in which workgroups arrive, and the thread that sees the count reach `splits` holds the
// complete sum: it converts it back, writes `mul` with one rounding and stores 0 to the word,
// which is thereby ready for the next call.  One memory round trip, no barrier, no second pass.
//
// Fixed point loses nothing that fp16 output can show: the resolution 2^-34 is 2^10 times finer
// than the smallest fp16 subnormal step, and the range +-2^21 is 32 times fp16's largest value.
// The contract that follows: every workgroup's partial sum is rounded to a multiple of 2^-34 and,
// with fp16 tensors, clamped to +-(2^21 - 1) (a NaN partial is clamped too and reads as one end
// of the range: the output becomes an infinity, not NaN); the running total must stay within +-2^21, which it does whenever the partial sums of
// one sign add up to less than that -- beyond it the 56-bit field wraps.  With fp32 tensors,
// whose results may legitimately exceed 2^21, a partial of 2^13 or more (255 smaller ones
// cannot leave the range) or one that is not finite is instead added to a float side accumulator of the same output (`side`, one float per
// accumulator word, zero-kept like the words) and joins the total when the output is finished:
// range and NaN / Inf behave as in fp32, only the 2^-34 absolute resolution remains.
// Agent-scope release/acquire fences are deliberately not used: on this multi-XCD part they
// write back and invalidate a whole L2 and serialise the workgroups.
constexpr float kFixScale = 17179869184.0f;        // 2^34
constexpr double kFixInvScale = 1.0 / 17179869184.0;
constexpr float kFixClamp = 2097151.0f;             // 2^21 - 1
constexpr int kMaxSplits = 255;
constexpr float kWideEscape = 8192.0f;              // 2^21 / 256: kMaxSplits partials below it cannot leave the range

// Workspace layout of a call with B rows: min(B, 16) * N accumulator words (rounded up to 256
// bytes), then as many floats: the side accumulators of the fp32-tensor entry point.
__host__ inline size_t splitk_words_bytes(int B, int N) {
    return ((size_t)(B < 16 ? (B < 1 ? 1 : B) : 16) * (size_t)N * sizeof(unsigned long long) + 255) / 256 * 256;
}
__host__ inline size_t splitk_side_bytes(int B, int N) {
    return ((size_t)(B < 16 ? (B < 1 ? 1 : B) : 16) * (size_t)N * sizeof(float) + 255) / 256 * 256;
}
__host__ inline float *splitk_side(void *workspace, int B, int N) {
    return reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + splitk_words_bytes(B, N));
}

__device__ inline unsigned long long splitk_encode(float partial) {
    float p = fminf(fmaxf(partial, -kFixClamp), kFixClamp);
    long long q = __double2ll_rn((double)p * (double)kFixScale);
    return ((unsigned long long)q << 8) + 1ull;
}

// `vals[b][c]` are this thread's partial sums for columns n0 + c, batch rows b < B.
template <typename IO, int MAXB, int COLS>
__device__ inline void splitk_finish(float (&vals)[MAXB][COLS], int B, int N, int n0, bool active, int splits,
                                     unsigned long long *__restrict__ acc, IO *__restrict__ mul,
                                     int accumulate, float *__restrict__ side = nullptr) {
    constexpr bool kWide = sizeof(IO) == 4;  // fp32 tensors: out-of-range partials take the side accumulator
    if (!active) return;
    if (splits > 1) {
        unsigned long long now[MAXB][COLS];
#pragma unroll
        for (int b = 0; b < MAXB; b++)
            if (b < B) {
#pragma unroll
                for (int c = 0; c < COLS; c++) {
                    if (kWide && !(fabsf(vals[b][c]) < kWideEscape)) {
                        // the float add must have completed before this workgroup is counted as
                        // arrived: wait for its return value
                        float old = __hip_atomic_fetch_add(side + (size_t)b * N + n0 + c, vals[b][c], __ATOMIC_RELAXED,
                                                           __HIP_MEMORY_SCOPE_AGENT);
                        asm volatile("" ::"v"(old) : "memory");
                        vals[b][c] = 0.f;
                    }
                    const unsigned long long add = splitk_encode(vals[b][c]);
                    now[b][c] = __hip_atomic_fetch_add(acc + (size_t)b * N + n0 + c, add, __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT) + add;
                }
            }
#pragma unroll
        for (int b = 0; b < MAXB; b++)
            if (b < B) {
#pragma unroll
                for (int c = 0; c < COLS; c++) {
                    if ((int)(now[b][c] & 0xffull) != splits) continue;  // someone else finishes this one
                    __hip_atomic_store(acc + (size_t)b * N + n0 + c, 0ull, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                    float v = (float)((double)((long long)now[b][c] >> 8) * kFixInvScale);
                    if (kWide) {
                        float *sp = side + (size_t)b * N + n0 + c;
                        const float extra = __hip_atomic_load(sp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        if (!(extra == 0.f)) {
                            __hip_atomic_store(sp, 0.f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            v += extra;
                        }
                    }
                    IO *o = mul + (size_t)b * N + n0 + c;
                    if (accumulate) v += to_float(*o);
                    *o = from_float<IO>(v);
                }
            }
        return;
    }
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

// Attention over a head's positions dealt to several workgroups: slice s of a head leaves the
// maximum m[s] of its scores, the sum l[s] of exp(score - m[s]) and its own softmax-weighted sum of
// value rows; the head's result is sum_s c[s] * result[s] with c[s] = exp(m[s] - M) l[s] / sum of
// the same over the slices, M the largest m.  An empty slice has l = 0 (and m = -inf): factor 0.
// One slice alone gets exactly 1.
constexpr int kAttnMaxSlices = 8;
template <int NS>
__device__ inline void attn_combine_weights(const float (&m)[NS], const float (&l)[NS], float (&c)[NS]) {
    float M = m[0];
#pragma unroll
    for (int s = 1; s < NS; s++) M = fmaxf(M, m[s]);
    float w[NS], L = 0.f;
#pragma unroll
    for (int s = 0; s < NS; s++) {
        w[s] = l[s] > 0.f ? __expf(m[s] - M) * l[s] : 0.f;
        L += w[s];
    }
#pragma unroll
    for (int s = 0; s < NS; s++) c[s] = L > 0.f ? w[s] / L : 0.f;
}

}  // namespace cq
