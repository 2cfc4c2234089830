// QAT-side fake quantisation on the device: weight (N, K) -> weight with every non-cherry input
// channel replaced by its group-wise quantise-dequantise value, in ONE pass over the matrix
// (read once, written once), in the weight's own dtype (fp16 or fp32).
//
// Arithmetic follows the reference's training forward, llama/cherry_linear.py:77-99
// (_adjust_weight: groups of G consecutive COMPACTED normal columns, cherry columns untouched,
// optional straight-through form  (q - w) + w) with llama/quantizer.py:148-152 (scale) and
// :165-170 (transform).  Every torch operation there rounds to the weight dtype, so with
// rnd() = "round to the weight dtype" (identity for fp32):
//   s = rnd( rnd(max|w| + 1e-6f) / 2^(b-1) )
//   r = clamp( rnd(w / s), -Q, Q ),  Q = rnd(2^(b-1) - 0.01)
//   q = rnd( (rnd(rint(rnd(r - 0.5))) + 0.5) ) * s, rounded
// and, for the straight-through form, rnd( rnd(q - w) + w ) on every column.
//
// One workgroup walks whole rows.  The cherry channels become a bit mask over the K columns in
// LDS (so the indices need neither be sorted nor distinct, as in the reference's scatter) with
// a prefix count per 32-column word: a column's compacted position is its index minus the
// cherries before it.  Pass 1 over a row folds |w| into one LDS maximum per group, pass 2
// re-reads the row (it is still in cache) and writes the result.
#include "cq_common.cuh"
#include "cq_kernels.h"

#pragma clang fp contract(off)

namespace cq {

constexpr int kFqMaxWords = 2048;    // 32-column mask words: K <= 65536
constexpr int kFqMaxGroups = 4096;   // quantisation groups per row
constexpr int kFqThreads = 256;

bool fake_quant_supported(int K, int C, int G) {
    (void)C;
    if (K <= 0 || K > kFqMaxWords * 32 || G <= 0) return false;
    // the group count is at most ceil(K / G) whatever the indices hold
    return ceil_div(K, G) <= kFqMaxGroups;
}

template <typename T>
struct FqType;
template <>
struct FqType<__half> {
    static __device__ __forceinline__ float rnd(float x) { return __half2float(__float2half_rn(x)); }
    static __device__ __forceinline__ float get(const __half *p) { return __half2float(*p); }
    static __device__ __forceinline__ void put(__half *p, float v) { *p = __float2half_rn(v); }
    static __device__ __forceinline__ void load8(const __half *p, float (&v)[8]) {
        const uint4 r = *reinterpret_cast<const uint4 *>(p);
        const uint32_t d[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 8; i++)
            v[i] = __half2float(__ushort_as_half((unsigned short)(d[i >> 1] >> (16 * (i & 1)))));
    }
    static __device__ __forceinline__ void store8(__half *p, const float (&v)[8]) {
        uint32_t d[4];
#pragma unroll
        for (int i = 0; i < 4; i++)
            d[i] = (uint32_t)__half_as_ushort(__float2half_rn(v[2 * i])) |
                   ((uint32_t)__half_as_ushort(__float2half_rn(v[2 * i + 1])) << 16);
        *reinterpret_cast<uint4 *>(p) = make_uint4(d[0], d[1], d[2], d[3]);
    }
};
template <>
struct FqType<float> {
    static __device__ __forceinline__ float rnd(float x) { return x; }
    static __device__ __forceinline__ float get(const float *p) { return *p; }
    static __device__ __forceinline__ void put(float *p, float v) { *p = v; }
    static __device__ __forceinline__ void load8(const float *p, float (&v)[8]) {
        const float4 a = *reinterpret_cast<const float4 *>(p), b = *reinterpret_cast<const float4 *>(p + 4);
        v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
    }
    static __device__ __forceinline__ void store8(float *p, const float (&v)[8]) {
        *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4 *>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
};

// `w` and `out` may be the same buffer: a thread reads a chunk in pass 2 before it writes it, and
// nothing else reads that chunk afterwards.
template <typename T>
__global__ __launch_bounds__(kFqThreads) void fake_quant_kernel(const T *w, const int32_t *__restrict__ idx, T *out,
                                                               int K, int N, int C, int G, int bits, int ste,
                                                               int vec_ok) {
    using F = FqType<T>;
    __shared__ uint32_t s_mask[kFqMaxWords];  // bit j & 31 of word j >> 5: column j is a cherry
    __shared__ uint32_t s_pre[kFqMaxWords];   // cherries in the words before
    __shared__ uint32_t s_grp[kFqMaxGroups];  // per group: max |w| as float bits, then the scale
    __shared__ uint32_t s_scan[kFqThreads];
    const int t = threadIdx.x;

    for (int i = t; i < kFqMaxWords; i += kFqThreads) s_mask[i] = 0;
    __syncthreads();
    for (int m = t; m < C; m += kFqThreads) {
        const int j = idx[m];
        if (j >= 0 && j < K) atomicOr(&s_mask[j >> 5], 1u << (j & 31));
    }
    __syncthreads();
    // exclusive prefix of the words' popcounts: 8 words per thread, then a scan over the threads
    uint32_t mine = 0;
#pragma unroll
    for (int i = 0; i < kFqMaxWords / kFqThreads; i++) mine += __popc(s_mask[t * (kFqMaxWords / kFqThreads) + i]);
    s_scan[t] = mine;
    __syncthreads();
    for (int d = 1; d < kFqThreads; d <<= 1) {
        const uint32_t add = t >= d ? s_scan[t - d] : 0;
        __syncthreads();
        s_scan[t] += add;
        __syncthreads();
    }
    {
        uint32_t run = s_scan[t] - mine;
#pragma unroll
        for (int i = 0; i < kFqMaxWords / kFqThreads; i++) {
            const int wd = t * (kFqMaxWords / kFqThreads) + i;
            s_pre[wd] = run;
            run += __popc(s_mask[wd]);
        }
    }
    const int Kn = K - (int)s_scan[kFqThreads - 1];
    const int groups = ceil_div(Kn, G);
    __syncthreads();

    const float half_levels = (float)(1 << (bits - 1));
    const float qmax = F::rnd((float)((double)(1 << (bits - 1)) - 1e-2));
    const int chunks = ceil_div(K, 8);

    for (int n = blockIdx.x; n < N; n += gridDim.x) {
        const T *wr = w + (size_t)n * K;
        T *orow = out + (size_t)n * K;
        for (int g = t; g < groups; g += kFqThreads) s_grp[g] = 0;
        __syncthreads();

        // ---- pass 1: group maxima
        for (int c = t; c < chunks; c += kFqThreads) {
            const int j0 = 8 * c;
            const int valid = min(8, K - j0);
            float v[8];
            if (vec_ok) {
                F::load8(wr + j0, v);
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++) v[i] = i < valid ? F::get(wr + j0 + i) : 0.f;
            }
            const uint32_t word = s_mask[j0 >> 5];
            const uint32_t mb = (word >> (j0 & 31)) & 0xffu;
            if (mb == (valid == 8 ? 0xffu : ((1u << valid) - 1u))) continue;  // cherries only
            int pos = j0 - (int)s_pre[j0 >> 5] - __popc(word & ((1u << (j0 & 31)) - 1u));
            int g = pos / G;
            int bound = (g + 1) * G;
            uint32_t mx = 0;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                if (i >= valid || ((mb >> i) & 1u)) continue;
                if (pos >= bound) {
                    atomicMax(&s_grp[g], mx);
                    mx = 0;
                    do {
                        g++;
                        bound += G;
                    } while (pos >= bound);
                }
                mx = max(mx, __float_as_uint(fabsf(v[i])));
                pos++;
            }
            atomicMax(&s_grp[g], mx);
        }
        __syncthreads();
        for (int g = t; g < groups; g += kFqThreads) {
            const float a = F::rnd(__uint_as_float(s_grp[g]) + 1e-6f);
            s_grp[g] = __float_as_uint(F::rnd(a / half_levels));
        }
        __syncthreads();

        // ---- pass 2: quantise-dequantise, write
        for (int c = t; c < chunks; c += kFqThreads) {
            const int j0 = 8 * c;
            const int valid = min(8, K - j0);
            float v[8], o[8];
            if (vec_ok) {
                F::load8(wr + j0, v);
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++) v[i] = i < valid ? F::get(wr + j0 + i) : 0.f;
            }
            const uint32_t word = s_mask[j0 >> 5];
            const uint32_t mb = (word >> (j0 & 31)) & 0xffu;
            int pos = j0 - (int)s_pre[j0 >> 5] - __popc(word & ((1u << (j0 & 31)) - 1u));
            int g = min(pos / G, max(groups - 1, 0));
            int bound = (g + 1) * G;
            float s = groups > 0 ? __uint_as_float(s_grp[g]) : 1.f;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                o[i] = v[i];
                if (i < valid && !((mb >> i) & 1u)) {
                    if (pos >= bound) {
                        do {
                            g++;
                            bound += G;
                        } while (pos >= bound);
                        s = __uint_as_float(s_grp[g]);
                    }
                    float r = F::rnd(v[i] / s);
                    r = fminf(fmaxf(r, -qmax), qmax);
                    r = F::rnd(r - 0.5f);
                    r = F::rnd(rintf(r));
                    r = F::rnd(r + 0.5f);
                    o[i] = F::rnd(r * s);
                    pos++;
                }
                if (ste) o[i] = F::rnd(F::rnd(o[i] - v[i]) + v[i]);
            }
            if (vec_ok) {
                F::store8(orow + j0, o);
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++)
                    if (i < valid) F::put(orow + j0 + i, o[i]);
            }
        }
        // the next row's pass 1 is two barriers away from its first write to s_grp's scales
        __syncthreads();
    }
}

template <typename T>
static hipError_t launch_fake_quant_t(int bits, const T *w, const int32_t *idx, T *out, int K, int N, int C, int G,
                                      int ste, hipStream_t stream) {
    // 16-byte accesses need whole chunks and 16-byte aligned rows; anything else goes element-wise
    const int vec_ok = K % 8 == 0 && ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    const int grid = min(N, 256 * 4);  // 33 KB of LDS: four workgroups per CU, every one walks rows
    hipLaunchKernelGGL(fake_quant_kernel<T>, dim3(grid), dim3(kFqThreads), 0, stream, w, idx, out, K, N, C, G, bits,
                       ste, vec_ok);
    return hipGetLastError();
}

hipError_t launch_fake_quant(int bits, bool fp32, const void *w, const int32_t *idx, void *out, int K, int N, int C,
                             int G, int ste, hipStream_t stream) {
    if (fp32)
        return launch_fake_quant_t<float>(bits, reinterpret_cast<const float *>(w), idx,
                                          reinterpret_cast<float *>(out), K, N, C, G, ste, stream);
    return launch_fake_quant_t<__half>(bits, reinterpret_cast<const __half *>(w), idx,
                                       reinterpret_cast<__half *>(out), K, N, C, G, ste, stream);
}

}  // namespace cq
