// QAT-side fake quantisation on the device: weight (N, K) -> weight with every non-cherry input
// channel replaced by its group-wise quantise-dequantise value, in ONE launch (the matrix is read
// from memory once and written once), in the weight's own dtype (fp16 or fp32).
//
// Arithmetic follows the reference's training forward, llama/cherry_linear.py:77-99
// (_adjust_weight: groups of G consecutive COMPACTED normal columns, cherry columns untouched,
// optional straight-through form  (q - w) + w) with llama/quantizer.py:148-152 (scale) and
// :165-170 (transform).  Every torch operation there rounds to the weight dtype, so with
// rnd() = "round to the weight dtype" (identity for fp32):
//   s = rnd( rnd(max|w| + 1e-6f) / 2^(b-1) )
//   r = clamp( rnd(w / s), -Q, Q ),  Q = rnd(2^(b-1) - 0.01)
//   q = rnd( (rint(rnd(r - 0.5)) + 0.5) * s )
// and, for the straight-through form, rnd( rnd(q - w) + w ) on every column.
//
// One workgroup walks whole rows.  The cherry channels become a bit mask over the K columns in
// LDS (so the indices need neither be sorted nor distinct, as in the reference's scatter) with
// a prefix count per 32-column word: a column's compacted position is its index minus the
// cherries before it.  Pass 1 over a row folds |w| into one LDS maximum per group, pass 2
// re-reads the row (it is still in cache) and writes the result.
//
// The kernel is bound by vector ALU work, not by memory, so the common case (rows of whole
// 16-byte chunks, groups of at least 8) runs WITHOUT branches that depend on the data: a chunk
// of 8 columns touches at most two groups, `first_b` (a 256 x 9 table in LDS over the chunk's
// cherry bits and the room left in the first group) says from which element on the second
// group's scale applies, and cherry elements are computed like the others and then replaced by
// the original bits.  A per-chunk "fast path when no cherry and no group boundary falls into the
// chunk" measured slower than no fast path at all: with 1 chunk in 32 taking the other branch,
// nearly every wavefront executes both.
#include "cq_device.h"
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

typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef unsigned short us2_t __attribute__((ext_vector_type(2)));

// 0 or 0xffffffff from bit i of m
__device__ __forceinline__ uint32_t bit_mask(uint32_t m, int i) { return (uint32_t)__builtin_amdgcn_sbfe((int)m, i, 1); }
// per 16-bit half of a pair (elements 2p, 2p+1): 0xffff where the element's bit of m is set
__device__ __forceinline__ uint32_t pair_mask(uint32_t m, int p) {
    return (bit_mask(m, 2 * p) & 0x0000ffffu) | (bit_mask(m, 2 * p + 1) & 0xffff0000u);
}
__device__ __forceinline__ uint32_t select_bits(uint32_t mask, uint32_t if_set, uint32_t if_clear) {
    return (if_set & mask) | (if_clear & ~mask);
}

// What a chunk of 8 columns needs to know about its groups: elements whose bit in `in_a` is set
// use scale `a`, the others scale `b`; bits of `cherry` mark elements that are left untouched.
struct ChunkScales {
    float sa, sb;       // the scales as fp32 values
    uint32_t in_a;      // 8 bits
    uint32_t cherry;    // 8 bits
};

// Per dtype: a chunk of 8 consecutive weights in registers, and the arithmetic on it.
template <typename T>
struct FqType;

template <>
struct FqType<__half> {
    struct Raw { uint32_t d[4]; };
    static __device__ __forceinline__ float rnd(float x) { return __half2float(__float2half_rn(x)); }
    static __device__ __forceinline__ Raw load(const __half *p, bool vec, int valid) {
        Raw r;
        if (vec) {
            const uint4 q = *reinterpret_cast<const uint4 *>(p);
            r.d[0] = q.x, r.d[1] = q.y, r.d[2] = q.z, r.d[3] = q.w;
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t lo = 2 * i < valid ? __half_as_ushort(p[2 * i]) : 0u;
                const uint32_t hi = 2 * i + 1 < valid ? __half_as_ushort(p[2 * i + 1]) : 0u;
                r.d[i] = lo | (hi << 16);
            }
        }
        return r;
    }
    static __device__ __forceinline__ void store(__half *p, const Raw &r, bool vec, int valid) {
        if (vec) {
            *reinterpret_cast<uint4 *>(p) = make_uint4(r.d[0], r.d[1], r.d[2], r.d[3]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (i < valid) p[i] = __ushort_as_half((unsigned short)(r.d[i >> 1] >> (16 * (i & 1))));
        }
    }
    static __device__ __forceinline__ float get(const Raw &r, int i) {
        return __half2float(__ushort_as_half((unsigned short)(r.d[i >> 1] >> (16 * (i & 1)))));
    }
    static __device__ __forceinline__ void set(Raw &r, int i, float v) {
        const uint32_t h = __half_as_ushort(__float2half_rn(v));
        r.d[i >> 1] = (i & 1) ? ((r.d[i >> 1] & 0x0000ffffu) | (h << 16)) : ((r.d[i >> 1] & 0xffff0000u) | h);
    }
    // RN16(w / s) without the IEEE division sequence: one Newton step on w * (1/s) leaves less
    // than one fp32 ulp of error, and a quotient of two 11-bit significands that is not itself
    // an fp16 rounding boundary stays more than 2^-23 (relative) away from every boundary, so
    // the rounding to fp16 sees the same side as the exact quotient.
    static __device__ __forceinline__ float quot32(float w, float s, float rs) {
        const float q0 = w * rs;
        const float e = __builtin_fmaf(-q0, s, w);
        return __builtin_fmaf(e, rs, q0);
    }
    static __device__ __forceinline__ float one(float w, float s, float qmax) {
        float r = rnd(quot32(w, s, __builtin_amdgcn_rcpf(s)));
        r = fminf(fmaxf(r, -qmax), qmax);
        r = rnd(r - 0.5f);
        r = rintf(r) + 0.5f;  // both exact in fp16 for |r| <= 8.5
        return rnd(r * s);
    }
    // max |w| per group of the chunk, as fp32 bits (|fp16| bit patterns order like the values)
    static __device__ __forceinline__ void absmax(const Raw &v, const ChunkScales &cs, uint32_t &ma, uint32_t &mb) {
        us2_t xa = {0, 0}, xb = {0, 0};
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const uint32_t a = v.d[p] & 0x7fff7fffu & ~pair_mask(cs.cherry, p);
            const uint32_t ina = pair_mask(cs.in_a, p);
            xa = __builtin_elementwise_max(xa, __builtin_bit_cast(us2_t, a & ina));
            xb = __builtin_elementwise_max(xb, __builtin_bit_cast(us2_t, a & ~ina));
        }
        ma = __float_as_uint(__half2float(__ushort_as_half(max(xa[0], xa[1]))));
        mb = __float_as_uint(__half2float(__ushort_as_half(max(xb[0], xb[1]))));
    }
    // fp16 addition and multiplication round like "fp32 operation, then round to fp16" (the
    // fp32 result of two fp16 operands is exact or far from any fp16 tie), so everything after
    // the quotient runs on packed fp16 instructions
    static __device__ __forceinline__ Raw all(const Raw &w, const ChunkScales &cs, float qmax, int ste) {
        const float rsa = __builtin_amdgcn_rcpf(cs.sa), rsb = __builtin_amdgcn_rcpf(cs.sb);
        const uint32_t sa16 = __half_as_ushort(__float2half_rn(cs.sa)), sb16 = __half_as_ushort(__float2half_rn(cs.sb));
        const uint32_t aa = sa16 | (sa16 << 16), bb = sb16 | (sb16 << 16);
        const _Float16 qh = (_Float16)qmax;
        const h2_t hi = {qh, qh}, lo = {-qh, -qh}, half2 = {(_Float16)0.5f, (_Float16)0.5f};
        Raw o;
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const h2_t wv = __builtin_bit_cast(h2_t, w.d[p]);
            const h2_t s2 = __builtin_bit_cast(h2_t, select_bits(pair_mask(cs.in_a, p), aa, bb));
            const float rs0 = __uint_as_float(select_bits(bit_mask(cs.in_a, 2 * p), __float_as_uint(rsa), __float_as_uint(rsb)));
            const float rs1 = __uint_as_float(select_bits(bit_mask(cs.in_a, 2 * p + 1), __float_as_uint(rsa), __float_as_uint(rsb)));
            h2_t r = {(_Float16)quot32((float)wv[0], (float)s2[0], rs0), (_Float16)quot32((float)wv[1], (float)s2[1], rs1)};
            r = __builtin_elementwise_min(__builtin_elementwise_max(r, lo), hi);
            r = r - half2;
            r = __builtin_elementwise_rint(r) + half2;
            const h2_t q = r * s2;
            uint32_t bits = select_bits(pair_mask(cs.cherry, p), w.d[p], __builtin_bit_cast(uint32_t, q));
            if (ste) {
                const h2_t qq = __builtin_bit_cast(h2_t, bits);
                bits = __builtin_bit_cast(uint32_t, (h2_t)((qq - wv) + wv));
            }
            o.d[p] = bits;
        }
        return o;
    }
};

template <>
struct FqType<float> {
    struct Raw { float v[8]; };
    static __device__ __forceinline__ float rnd(float x) { return x; }
    static __device__ __forceinline__ Raw load(const float *p, bool vec, int valid) {
        Raw r;
        if (vec) {
            const float4 a = *reinterpret_cast<const float4 *>(p), b = *reinterpret_cast<const float4 *>(p + 4);
            r.v[0] = a.x, r.v[1] = a.y, r.v[2] = a.z, r.v[3] = a.w, r.v[4] = b.x, r.v[5] = b.y, r.v[6] = b.z, r.v[7] = b.w;
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) r.v[i] = i < valid ? p[i] : 0.f;
        }
        return r;
    }
    static __device__ __forceinline__ void store(float *p, const Raw &r, bool vec, int valid) {
        if (vec) {
            *reinterpret_cast<float4 *>(p) = make_float4(r.v[0], r.v[1], r.v[2], r.v[3]);
            *reinterpret_cast<float4 *>(p + 4) = make_float4(r.v[4], r.v[5], r.v[6], r.v[7]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (i < valid) p[i] = r.v[i];
        }
    }
    static __device__ __forceinline__ float get(const Raw &r, int i) { return r.v[i]; }
    static __device__ __forceinline__ void set(Raw &r, int i, float v) { r.v[i] = v; }
    // fp32 weights: the correctly rounded division, as torch's
    static __device__ __forceinline__ float one(float w, float s, float qmax) {
        float r = w / s;
        r = fminf(fmaxf(r, -qmax), qmax);
        r = rintf(r - 0.5f) + 0.5f;
        return r * s;
    }
    static __device__ __forceinline__ void absmax(const Raw &v, const ChunkScales &cs, uint32_t &ma, uint32_t &mb) {
        ma = 0, mb = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t a = __float_as_uint(v.v[i]) & 0x7fffffffu & ~bit_mask(cs.cherry, i);
            const uint32_t ina = bit_mask(cs.in_a, i);
            ma = max(ma, a & ina);
            mb = max(mb, a & ~ina);
        }
    }
    static __device__ __forceinline__ Raw all(const Raw &w, const ChunkScales &cs, float qmax, int ste) {
        Raw o;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float s = __uint_as_float(select_bits(bit_mask(cs.in_a, i), __float_as_uint(cs.sa), __float_as_uint(cs.sb)));
            float q = __uint_as_float(select_bits(bit_mask(cs.cherry, i), __float_as_uint(w.v[i]),
                                                  __float_as_uint(one(w.v[i], s, qmax))));
            if (ste) q = (q - w.v[i]) + w.v[i];
            o.v[i] = q;
        }
        return o;
    }
};

// `w` and `out` may be the same buffer: a thread reads a chunk in pass 2 before it writes it, and
// nothing else reads that chunk afterwards.
// UNIFORM: rows are whole, 16-byte aligned chunks and G >= 8 (a chunk meets at most two groups).
template <typename T, bool UNIFORM>
__global__ __launch_bounds__(kFqThreads) void fake_quant_kernel(const T *w, const int32_t *__restrict__ idx, T *out,
                                                               int K, int N, int C, int G, int gshift, int bits,
                                                               int ste, int vec_ok) {
    using F = FqType<T>;
    using Raw = typename F::Raw;
    __shared__ uint32_t s_mask[kFqMaxWords];  // bit j & 31 of word j >> 5: column j is a cherry
    __shared__ uint32_t s_pre[kFqMaxWords];   // cherries in the words before
    __shared__ uint32_t s_grp[kFqMaxGroups];  // per group: max |w| as float bits, then the scale
    __shared__ uint32_t s_scan[kFqThreads];
    // first_b[cherry bits][room]: index of the first element of a chunk that belongs to the NEXT
    // group when the current one has room for `room` (0..8, 8 = at least 8) more normal elements
    __shared__ uint8_t s_first_b[256 * 9];
    const int t = threadIdx.x;

    for (int i = t; i < kFqMaxWords; i += kFqThreads) s_mask[i] = 0;
    if (UNIFORM) {
        for (int e = t; e < 256 * 9; e += kFqThreads) {
            const uint32_t cherry = e / 9;
            int room = e % 9, first = 8;
            for (int i = 0; i < 8; i++) {
                if ((cherry >> i) & 1u) continue;
                if (room == 0) {
                    first = i;
                    break;
                }
                room--;
            }
            s_first_b[e] = (uint8_t)first;
        }
    }
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
    const int last_group = max(groups - 1, 0);

    // compacted position of column j0 (a multiple of 8) and the cherry bits of its chunk
    auto locate = [&](int j0, uint32_t &cherry) {
        const uint32_t word = s_mask[j0 >> 5];
        cherry = (word >> (j0 & 31)) & 0xffu;
        return j0 - (int)s_pre[j0 >> 5] - __popc(word & ((1u << (j0 & 31)) - 1u));
    };
    // group of the chunk's first normal element (clamped: a chunk of trailing cherries has none)
    // and which elements still belong to it
    auto split = [&](int j0, int &g, ChunkScales &cs) {
        const int pos = locate(j0, cs.cherry);
        g = min(gshift >= 0 ? pos >> gshift : pos / G, last_group);
        const int room = min(max((g + 1) * G - pos, 0), 8);
        cs.in_a = (1u << s_first_b[cs.cherry * 9 + room]) - 1u;
    };

    for (int n = blockIdx.x; n < N; n += gridDim.x) {
        const T *wr = w + (size_t)n * K;
        T *orow = out + (size_t)n * K;
        for (int g = t; g < groups; g += kFqThreads) s_grp[g] = 0;
        __syncthreads();

        // ---- pass 1: group maxima
        for (int c = t; c < chunks; c += kFqThreads) {
            const int j0 = 8 * c;
            if (UNIFORM) {
                const Raw v = F::load(wr + j0, true, 8);
                ChunkScales cs;
                int g;
                split(j0, g, cs);
                uint32_t ma, mb;
                F::absmax(v, cs, ma, mb);
                if (groups > 0) {
                    atomicMax(&s_grp[g], ma);
                    if (cs.in_a != 0xffu) atomicMax(&s_grp[min(g + 1, last_group)], mb);
                }
            } else {
                const int valid = min(8, K - j0);
                const Raw v = F::load(wr + j0, vec_ok, valid);
                uint32_t cherry;
                int pos = locate(j0, cherry);
                if (cherry == (valid == 8 ? 0xffu : ((1u << valid) - 1u))) continue;  // cherries only
                int g = pos / G;
                int bound = (g + 1) * G;
                uint32_t mx = 0;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    if (i >= valid || ((cherry >> i) & 1u)) continue;
                    if (pos >= bound) {
                        atomicMax(&s_grp[g], mx);
                        mx = 0;
                        do {
                            g++;
                            bound += G;
                        } while (pos >= bound);
                    }
                    mx = max(mx, __float_as_uint(fabsf(F::get(v, i))));
                    pos++;
                }
                atomicMax(&s_grp[g], mx);
            }
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
            if (UNIFORM) {
                const Raw v = F::load(wr + j0, true, 8);
                ChunkScales cs;
                int g;
                split(j0, g, cs);
                if (groups == 0) cs.cherry = 0xffu;
                cs.sa = groups > 0 ? __uint_as_float(s_grp[g]) : 1.f;
                cs.sb = groups > 0 ? __uint_as_float(s_grp[min(g + 1, last_group)]) : 1.f;
                F::store(orow + j0, F::all(v, cs, qmax, ste), true, 8);
            } else {
                const int valid = min(8, K - j0);
                const Raw v = F::load(wr + j0, vec_ok, valid);
                uint32_t cherry;
                int pos = locate(j0, cherry);
                int g = min(pos / G, last_group);
                int bound = (g + 1) * G;
                float s = groups > 0 ? __uint_as_float(s_grp[g]) : 1.f;
                Raw o = v;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const float wv = F::get(v, i);
                    float ov = wv;
                    if (i < valid && !((cherry >> i) & 1u)) {
                        if (pos >= bound) {
                            do {
                                g++;
                                bound += G;
                            } while (pos >= bound);
                            s = __uint_as_float(s_grp[g]);
                        }
                        ov = F::one(wv, s, qmax);
                        pos++;
                    }
                    // the straight-through expression is evaluated on cherry channels too
                    if (ste) ov = F::rnd(F::rnd(ov - wv) + wv);
                    F::set(o, i, ov);
                }
                F::store(orow + j0, o, vec_ok, valid);
            }
        }
        // the next row clears s_grp: not before every thread has read its scales
        __syncthreads();
    }
}

template <typename T>
static hipError_t launch_fake_quant_t(int bits, const T *w, const int32_t *idx, T *out, int K, int N, int C, int G,
                                      int ste, hipStream_t stream) {
    // 16-byte accesses need whole chunks and 16-byte aligned rows; anything else goes element-wise
    const int vec_ok = K % 8 == 0 && ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    const int gshift = (G & (G - 1)) == 0 ? __builtin_ctz((unsigned)G) : -1;
    const int grid = min(N, 256 * 4);  // 36 KB of LDS: four workgroups per CU, every one walks rows
    if (vec_ok && G >= 8)
        hipLaunchKernelGGL((fake_quant_kernel<T, true>), dim3(grid), dim3(kFqThreads), 0, stream, w, idx, out, K, N, C,
                           G, gshift, bits, ste, vec_ok);
    else
        hipLaunchKernelGGL((fake_quant_kernel<T, false>), dim3(grid), dim3(kFqThreads), 0, stream, w, idx, out, K, N,
                           C, G, gshift, bits, ste, vec_ok);
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
