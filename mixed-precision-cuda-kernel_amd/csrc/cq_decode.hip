// Batch-1 decode-step glue for a LLaMA-shaped decoder around the CherryQ linears: the operations
// between two fused matvecs, each as ONE launch so that a token step is a short chain of kernels
// (captured in a HIP graph by the caller) instead of dozens of element-wise launches.
//
// Semantics follow the reference's model code (llama/modeling_llama_quant.py): RMSNorm :75-89,
// rotary embedding :95-147 and apply_rotary_pos_emb :179-210, attention with KV cache :391-402 /
// :671-696, SiLU-gated MLP :251.  fp16 storage, fp32 arithmetic inside a kernel, roundings at the
// points where the reference's fp16 tensors are materialised.
#include "cq_device.h"
#include "cq_kernels.h"

// The rotary embedding rounds every product and every sum to fp16 separately, as the reference's
// fp16 tensor operations do; contraction would merge a product and a sum into one rounding.
#pragma clang fp contract(off)

namespace cq {

// wavefront-wide sum / maximum, delivered to every lane (DPP rotations and permlane swaps, no LDS)
__device__ inline float wave_sum(float v) { return wave_sum_all(v); }
__device__ inline float wave_max(float v) { return wave_max_all(v); }

// h <- h + delta (skipped when delta is null);  y <- weight * fp16(h * rsqrt(mean(h^2) + eps))
// One workgroup; a thread takes 4 consecutive elements (one 8-byte access) per pass.  H % 4 == 0.
__global__ __launch_bounds__(1024) void add_rmsnorm_kernel(__half *__restrict__ h, const __half *__restrict__ delta,
                                                           const __half *__restrict__ weight, __half *__restrict__ y,
                                                           int H, float eps) {
    __shared__ float s_part[16];
    const int t = threadIdx.x;
    float ss = 0.f;
    for (int i = 4 * t; i < H; i += 4096) {
        const uint2 raw = *reinterpret_cast<const uint2 *>(h + i);
        float v[4] = {__half2float(__ushort_as_half(raw.x & 0xffff)), __half2float(__ushort_as_half(raw.x >> 16)),
                      __half2float(__ushort_as_half(raw.y & 0xffff)), __half2float(__ushort_as_half(raw.y >> 16))};
        if (delta) {
            const uint2 dr = *reinterpret_cast<const uint2 *>(delta + i);
            const float d[4] = {__half2float(__ushort_as_half(dr.x & 0xffff)), __half2float(__ushort_as_half(dr.x >> 16)),
                                __half2float(__ushort_as_half(dr.y & 0xffff)), __half2float(__ushort_as_half(dr.y >> 16))};
            unsigned short o[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                o[e] = __half_as_ushort(__float2half_rn(v[e] + d[e]));
                v[e] = __half2float(__ushort_as_half(o[e]));
            }
            *reinterpret_cast<uint2 *>(h + i) = make_uint2(o[0] | (uint32_t)o[1] << 16, o[2] | (uint32_t)o[3] << 16);
        }
#pragma unroll
        for (int e = 0; e < 4; e++) ss += v[e] * v[e];
    }
    ss = wave_sum(ss);
    if ((t & 63) == 0) s_part[t >> 6] = ss;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < 16; w++) tot += s_part[w];
    const float rs = rsqrtf(tot / (float)H + eps);
    for (int i = 4 * t; i < H; i += 4096) {
        const uint2 raw = *reinterpret_cast<const uint2 *>(h + i);
        const uint2 wr = *reinterpret_cast<const uint2 *>(weight + i);
        const uint32_t hv[4] = {raw.x & 0xffff, raw.x >> 16, raw.y & 0xffff, raw.y >> 16};
        const uint32_t wv[4] = {wr.x & 0xffff, wr.x >> 16, wr.y & 0xffff, wr.y >> 16};
        unsigned short o[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float n = __half2float(__float2half_rn(__half2float(__ushort_as_half(hv[e])) * rs));
            o[e] = __half_as_ushort(__float2half_rn(__half2float(__ushort_as_half(wv[e])) * n));
        }
        *reinterpret_cast<uint2 *>(y + i) = make_uint2(o[0] | (uint32_t)o[1] << 16, o[2] | (uint32_t)o[3] << 16);
    }
}

// theta^(-2 i / head_dim), the rotary frequency of dimension pair i.  The library routine powf is a
// call of several hundred instructions on the critical path of every decode step.  For a
// power-of-two head_dim the exponent x = (2 i / head_dim) * log2(theta) is split into an integer
// and a fraction in [-0.5, 0.5] without rounding error beyond that of log2(theta), which the host
// passes as an unevaluated sum of two floats; 2^-fraction is one v_exp_f32 (about 1 ulp), so the
// result is within about 2 ulp of the exact value, like powf's.  Other head dims use powf.
struct RopeBase {
    float theta, log2_hi, log2_lo;
};

static RopeBase rope_base(float theta) {
    const double l = log2((double)theta);
    RopeBase b;
    b.theta = theta;
    b.log2_hi = (float)l;
    b.log2_lo = (float)(l - (double)b.log2_hi);
    return b;
}

__device__ inline float rope_inv_freq(int i, int head_dim, const RopeBase &b) {
    if (head_dim & (head_dim - 1)) return powf(b.theta, -2.0f * (float)i / (float)head_dim);
    const float fi = (float)(2 * i);                 // exact
    const float p = fi * b.log2_hi;
    const float e = fmaf(fi, b.log2_hi, -p);         // exact error of the product
    const float inv_hd = 1.0f / (float)head_dim;     // exact: a power of two
    const float ps = p * inv_hd;                     // exact scaling
    const float n = rintf(ps);
    const float frac = (ps - n) + (e + fi * b.log2_lo) * inv_hd;  // ps - n is exact
    return ldexpf(__builtin_amdgcn_exp2f(-frac), -(int)n);
}

// Rotary embedding of q (in place) and k, and the KV-cache write at position *pos.
// One workgroup per head (q heads first, then kv heads), head_dim / 2 threads.
// Cache layout: [kv_head][max_len][head_dim].
__global__ void rope_cache_kernel(__half *__restrict__ q, const __half *__restrict__ k, const __half *__restrict__ v,
                                  __half *__restrict__ k_cache, __half *__restrict__ v_cache,
                                  const int *__restrict__ pos_ptr, int n_heads, int n_kv_heads, int head_dim,
                                  int max_len, RopeBase base) {
    const int pos = *pos_ptr;
    const int head = blockIdx.x, i = threadIdx.x, half_dim = head_dim / 2;
    if (i >= half_dim || (unsigned)pos >= (unsigned)max_len) return;  // also a negative position: nothing is written
    const float inv_freq = rope_inv_freq(i, head_dim, base);
    float sn, cs;
    sincosf((float)pos * inv_freq, &sn, &cs);
    const float c = __half2float(__float2half_rn(cs)), s = __half2float(__float2half_rn(sn));
    auto rot = [&](float x1, float x2, __half &o1, __half &o2) {
        // x * cos + rotate_half(x) * sin with every product and the sum rounded to fp16
        const float a1 = __half2float(__float2half_rn(x1 * c)), b1 = __half2float(__float2half_rn(-x2 * s));
        const float a2 = __half2float(__float2half_rn(x2 * c)), b2 = __half2float(__float2half_rn(x1 * s));
        o1 = __float2half_rn(a1 + b1);
        o2 = __float2half_rn(a2 + b2);
    };
    if (head < n_heads) {
        __half *qh = q + (size_t)head * head_dim;
        __half o1, o2;
        rot(__half2float(qh[i]), __half2float(qh[i + half_dim]), o1, o2);
        qh[i] = o1;
        qh[i + half_dim] = o2;
    } else {
        const int kh = head - n_heads;
        const __half *ksrc = k + (size_t)kh * head_dim;
        const __half *vsrc = v + (size_t)kh * head_dim;
        __half *kd = k_cache + ((size_t)kh * max_len + pos) * head_dim;
        __half *vd = v_cache + ((size_t)kh * max_len + pos) * head_dim;
        __half o1, o2;
        rot(__half2float(ksrc[i]), __half2float(ksrc[i + half_dim]), o1, o2);
        kd[i] = o1;
        kd[i + half_dim] = o2;
        vd[i] = vsrc[i];
        vd[i + half_dim] = vsrc[i + half_dim];
    }
}

// Single-query attention over the cache positions 0 .. *pos, one workgroup (256 threads) per head.
// The 256 threads form 16 rows of 16 lanes; a row takes one cache position at a time, each lane
// 8 of the 128 dimensions (one 16-byte load), so 16 positions are in flight per iteration.
// softmax in fp32, probabilities rounded to fp16 before the value product (as the eager path of
// the reference does), fp32 accumulation.  head_dim must be 128, max_len <= kMaxAttnLen.
constexpr int kMaxAttnLen = 4096;

__device__ inline float row16_sum(float v) { return row_sum(v); }

__device__ inline void unpack8(const uint4 &u, float (&f)[8]) {
    const __half2 *h = reinterpret_cast<const __half2 *>(&u);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        f[2 * i] = __low2float(h[i]);
        f[2 * i + 1] = __high2float(h[i]);
    }
}

__global__ __launch_bounds__(256) void attn_decode_kernel(const __half *__restrict__ q,
                                                          const __half *__restrict__ k_cache,
                                                          const __half *__restrict__ v_cache,
                                                          __half *__restrict__ out, const int *__restrict__ pos_ptr,
                                                          int n_heads, int n_kv_heads, int max_len, float scale) {
    __shared__ float s_score[kMaxAttnLen];
    __shared__ float s_red[8];
    __shared__ float s_acc[16][128];
    const int head = blockIdx.x, t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int row = t >> 4, l16 = t & 15;
    const int kvh = head / (n_heads / n_kv_heads);
    const int pos = *pos_ptr;
    if ((unsigned)pos >= (unsigned)max_len) {
        // a position outside the cache (negative, or at / beyond max_len) reads nothing; the
        // output is NaN so that the caller's mistake shows in everything computed from it
        if (t < 128) out[(size_t)head * 128 + t] = __ushort_as_half((unsigned short)0x7e00);
        return;
    }
    const int len = pos + 1;
    const uint4 *kb = reinterpret_cast<const uint4 *>(k_cache + (size_t)kvh * max_len * 128);
    const uint4 *vb = reinterpret_cast<const uint4 *>(v_cache + (size_t)kvh * max_len * 128);
    float qf[8];
    unpack8(reinterpret_cast<const uint4 *>(q + (size_t)head * 128)[l16], qf);
    for (int j = row; j < len; j += 16) {
        float kf[8];
        unpack8(kb[(size_t)j * 16 + l16], kf);
        float d = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) d += qf[i] * kf[i];
        d = row16_sum(d);
        if (l16 == 0) s_score[j] = __half2float(__float2half_rn(d)) * scale;  // fp16 q k^T, then / sqrt(d)
    }
    __syncthreads();
    float m = -INFINITY;
    for (int j = t; j < len; j += 256) m = fmaxf(m, s_score[j]);
    m = wave_max(m);
    if (lane == 0) s_red[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
    float sum = 0.f;
    for (int j = t; j < len; j += 256) {
        const float e = __expf(s_score[j] - m);
        s_score[j] = e;
        sum += e;
    }
    sum = wave_sum(sum);
    if (lane == 0) s_red[4 + wave] = sum;
    __syncthreads();
    const float inv = 1.f / (s_red[4] + s_red[5] + s_red[6] + s_red[7]);
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = 0.f;
    for (int j = row; j < len; j += 16) {
        const float p = __half2float(__float2half_rn(s_score[j] * inv));
        float vf[8];
        unpack8(vb[(size_t)j * 16 + l16], vf);
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] += p * vf[i];
    }
#pragma unroll
    for (int i = 0; i < 8; i++) s_acc[row][8 * l16 + i] = acc[i];
    __syncthreads();
    if (t < 128) {
        float o = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++) o += s_acc[r][t];
        out[(size_t)head * 128 + t] = __float2half_rn(o);
    }
}

// Rotary embedding, KV-cache write and single-query attention of one token in ONE launch: one
// workgroup of 1024 threads (64 rows of 16 lanes) per query head.  The workgroup rotates its own
// q and its kv head's k in LDS and attends to the new position from there, so no workgroup reads
// a cache row that another one writes in the same launch; the first query head of each kv group
// stores the rotated k and the v row into the caches for later tokens.  Arithmetic and rounding
// points are those of rope_cache_kernel followed by attn_decode_kernel.
// (No __restrict__ on the inputs: loads through a read-only restrict pointer may be moved anywhere,
// and the order of this kernel's first requests matters.)
__global__ __launch_bounds__(1024) void rope_attn_decode_kernel(
    const __half *q, const __half *k, const __half *v, __half *k_cache, __half *v_cache, __half *__restrict__ out,
    const int *__restrict__ pos_ptr, int n_heads, int n_kv_heads, int max_len, RopeBase base, float scale) {
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    __shared__ float s_score[kMaxAttnLen];
    __shared__ float s_red[32];
    __shared__ float s_acc[16][128];
    __shared__ __attribute__((aligned(16))) unsigned short s_qh[128], s_kh[128];  // rotated q, k as fp16
    const int head = blockIdx.x, t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int row = t >> 4, l16 = t & 15;
    const int rep = n_heads / n_kv_heads, kvh = head / rep;
    const uint4 *kb = reinterpret_cast<const uint4 *>(k_cache + (size_t)kvh * max_len * 128);
    const uint4 *vb = reinterpret_cast<const uint4 *>(v_cache + (size_t)kvh * max_len * 128);
    // Order of the requests = order of use: the new token's q (threads 0..63), k and v (threads
    // 64..127) and the position, every K row of the first pass; the V rows behind the first barrier.
    // The cache rows are requested before the position is known (rows up to max_len exist; those
    // at or beyond the position are ignored below): one memory round trip in front of the arithmetic.
    // Every request is an unconditional buffer load (rows past the cache read zeros through the
    // descriptor; every thread requests the small values, threads from 128 on drop them): all of
    // them sit in one basic block in this order, so the wait in front of the rotation counts only
    // the requests issued before it -- behind a branch the compiler waits for everything that is
    // outstanding, V rows included, and plain loads it moves next to their first use.
    typedef uint32_t u4_t __attribute__((ext_vector_type(4)));
    constexpr uint32_t kFlags = 0x00020000u;
    const __amdgpu_buffer_rsrc_t rq = __builtin_amdgcn_make_buffer_rsrc((void *)(q + (size_t)head * 128), 0, 256, kFlags);
    const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc((void *)(k + (size_t)kvh * 128), 0, 256, kFlags);
    const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc((void *)(v + (size_t)kvh * 128), 0, 256, kFlags);
    const __amdgpu_buffer_rsrc_t rkc = __builtin_amdgcn_make_buffer_rsrc((void *)kb, 0, max_len * 256, kFlags);
    const __amdgpu_buffer_rsrc_t rvc = __builtin_amdgcn_make_buffer_rsrc((void *)vb, 0, max_len * 256, kFlags);
    const int ci = t & 63;
    const unsigned short q1 = __builtin_amdgcn_raw_buffer_load_b16(rq, ci * 2, 0, 0), q2 = __builtin_amdgcn_raw_buffer_load_b16(rq, ci * 2 + 128, 0, 0);
    const unsigned short k1 = __builtin_amdgcn_raw_buffer_load_b16(rk, ci * 2, 0, 0), k2 = __builtin_amdgcn_raw_buffer_load_b16(rk, ci * 2 + 128, 0, 0);
    const __half v1 = __ushort_as_half(__builtin_amdgcn_raw_buffer_load_b16(rv, ci * 2, 0, 0));
    const __half v2 = __ushort_as_half(__builtin_amdgcn_raw_buffer_load_b16(rv, ci * 2 + 128, 0, 0));
    asm volatile("" ::: "memory");   // (keeps the groups of requests in this order through the compiler)
    __builtin_amdgcn_sched_barrier(0);
    uint4 k_first[4], v_first[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const u4_t r = __builtin_amdgcn_raw_buffer_load_b128(rkc, (row + 64 * u) * 256 + l16 * 16, 0, 0);
        k_first[u] = make_uint4(r[0], r[1], r[2], r[3]);
    }
    asm volatile("" ::: "memory");   // (keeps the groups of requests in this order through the compiler)
    __builtin_amdgcn_sched_barrier(0);
    const __half r1 = __ushort_as_half((t & 64) ? k1 : q1), r2 = __ushort_as_half((t & 64) ? k2 : q2);
    const float x1 = __half2float(r1), x2 = __half2float(r2);
    const float inv_freq = rope_inv_freq(t & 63, 128, base);  // does not need the position
    const int pos = *pos_ptr;
    if ((unsigned)pos >= (unsigned)max_len) {  // outside the cache: nothing read or written, the output is NaN
        if (t < 128) out[(size_t)head * 128 + t] = __ushort_as_half((unsigned short)0x7e00);
        return;
    }
    if (t < 128) {
        const int i = t & 63;
        const bool is_k = t >= 64;
        float sn, cs;
        sincosf((float)pos * inv_freq, &sn, &cs);
        const float c = __half2float(__float2half_rn(cs)), sr = __half2float(__float2half_rn(sn));
        const float a1 = __half2float(__float2half_rn(x1 * c)), b1 = __half2float(__float2half_rn(-x2 * sr));
        const float a2 = __half2float(__float2half_rn(x2 * c)), b2 = __half2float(__float2half_rn(x1 * sr));
        const __half o1 = __float2half_rn(a1 + b1), o2 = __float2half_rn(a2 + b2);
        unsigned short *dst = is_k ? s_kh : s_qh;
        dst[i] = __half_as_ushort(o1);
        dst[i + 64] = __half_as_ushort(o2);
        if (is_k && head % rep == 0) {
            __half *kd = k_cache + ((size_t)kvh * max_len + pos) * 128;
            __half *vd = v_cache + ((size_t)kvh * max_len + pos) * 128;
            kd[i] = o1;
            kd[i + 64] = o2;
            vd[i] = v1;
            vd[i + 64] = v2;
        }
    }
    __syncthreads();
    // The V rows are requested only now: a wavefront reaches a barrier when its requests have been
    // ACCEPTED, and one compute unit accepts about 32 KB per microsecond -- with the V rows in front
    // of it the barrier opened when all 128 KB of a 256-position cache had been taken (3 to 4 us);
    // they are not needed before the softmax is done and travel while the scores are formed.
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const u4_t r = __builtin_amdgcn_raw_buffer_load_b128(rvc, (row + 64 * u) * 256 + l16 * 16, 0, 0);
        v_first[u] = make_uint4(r[0], r[1], r[2], r[3]);
    }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    // q . k over the lane's 8 dimensions as four packed fp16 dot products (fp32 accumulation), the 16
    // lanes of a row then add up with DPP rotations
    const uint4 qv = *reinterpret_cast<const uint4 *>(&s_qh[8 * l16]);
    auto dot8 = [&](const uint4 &kv) {
        float d = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, kv.x), __builtin_bit_cast(half2_t, qv.x), 0.f, false);
        d = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, kv.y), __builtin_bit_cast(half2_t, qv.y), d, false);
        d = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, kv.z), __builtin_bit_cast(half2_t, qv.z), d, false);
        d = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, kv.w), __builtin_bit_cast(half2_t, qv.w), d, false);
        return row_sum(d);
    };
    // scores of the cached positions 0 .. pos-1, four rows of loads in flight per thread; the running
    // maximum rides along, so that the softmax needs no pass of its own for it
    float m = -INFINITY;
    for (int j0 = row; j0 < pos; j0 += 256) {
        uint4 kk[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int j = j0 + 64 * u;
            if (j0 == row)
                kk[u] = k_first[u];
            else
                kk[u] = j < pos ? kb[(size_t)j * 16 + l16] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int j = j0 + 64 * u;
            const float sc = __half2float(__float2half_rn(dot8(kk[u]))) * scale;  // fp16 q k^T, then / sqrt(d)
            if (j < pos) {
                m = fmaxf(m, sc);
                if (l16 == 0) s_score[j] = sc;
            }
        }
    }
    if (row == 0) {  // the new position, from LDS
        const float sc = __half2float(__float2half_rn(dot8(*reinterpret_cast<const uint4 *>(&s_kh[8 * l16])))) * scale;
        m = fmaxf(m, sc);
        if (l16 == 0) s_score[pos] = sc;
    }
    m = wave_max_all(m);
    if (lane == 0) s_red[wave] = m;
    __syncthreads();
    const int len = pos + 1;
    m = s_red[0];
#pragma unroll
    for (int w = 1; w < 16; w++) m = fmaxf(m, s_red[w]);
    float sum = 0.f;
    for (int j = t; j < len; j += 1024) {
        const float e = __expf(s_score[j] - m);
        s_score[j] = e;
        sum += e;
    }
    sum = wave_sum_all(sum);
    if (lane == 0) s_red[16 + wave] = sum;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < 16; w++) tot += s_red[16 + w];
    const float inv = 1.f / tot;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = 0.f;
    for (int j0 = row; j0 < pos; j0 += 256) {
        uint4 vv[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int j = j0 + 64 * u;
            if (j0 == row)
                vv[u] = j < pos ? v_first[u] : make_uint4(0, 0, 0, 0);  // rows past the position may hold anything
            else
                vv[u] = j < pos ? vb[(size_t)j * 16 + l16] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int j = j0 + 64 * u;
            const float p = j < pos ? __half2float(__float2half_rn(s_score[j] * inv)) : 0.f;
            float vf[8];
            unpack8(vv[u], vf);
#pragma unroll
            for (int i = 0; i < 8; i++) acc[i] = fmaf(p, vf[i], acc[i]);
        }
    }
    if (row == 0) {
        const float p = __half2float(__float2half_rn(s_score[pos] * inv));
        float vf[8];
        unpack8(reinterpret_cast<const uint4 *>(v + (size_t)kvh * 128)[l16], vf);
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = fmaf(p, vf[i], acc[i]);
    }
    // the four 16-lane rows of a wavefront hold partial sums for the same 128 dimensions: two
    // halving exchanges leave every lane with 2 of its 8 dimensions summed over the four rows
    {
        float h4[4], q2[2];
#pragma unroll
        for (int i = 0; i < 4; i++) h4[i] = swap32_add(acc[i], acc[4 + i]);  // lanes >= 32: dimensions 4..7
#pragma unroll
        for (int i = 0; i < 2; i++) q2[i] = swap16_add(h4[i], h4[2 + i]);    // odd rows: + 2
        const int d0 = 8 * l16 + 4 * (lane >> 5) + 2 * ((lane >> 4) & 1);
        s_acc[wave][d0] = q2[0];
        s_acc[wave][d0 + 1] = q2[1];
    }
    __syncthreads();
    if (t < 128) {
        float o = 0.f;
#pragma unroll
        for (int w = 0; w < 16; w++) o += s_acc[w][t];
        out[(size_t)head * 128 + t] = __float2half_rn(o);
    }
}

// rope_attn_decode_kernel with a head's positions dealt to `slices` workgroups (grid = n_heads *
// slices; workgroup b works on head b % n_heads, slice b / n_heads = the blocks of 64 positions
// slice, slice + slices, slice + 2 slices, ... so that the slices stay balanced at every position).
// One workgroup per head requests the head's whole K and V (128 KB at 256 positions, 4 MB at 4096)
// through ONE compute unit, which accepts about 32 KB at a time; with 32 heads only 32 of the 256
// compute units pull data.  A slice is a softmax of its own: it stores
// fp16(sum_j fp16(e_j / l) v_j) with e_j = exp(score_j - m), m and l its scores' maximum and sum of
// e_j, and (m, l) as two floats; a slice without positions stores zeros and (-inf, 0).
// attn_combine_weights() turns the (m, l) of a head's slices into the factors of the slices'
// results; the reader of the partial results (the output projection while it stages its input, or
// attn_combine_kernel) applies them.  With one slice the stored result is rope_attn_decode_kernel's,
// bit for bit, and its factor is exactly 1.  The slice that owns the new position attends to it
// from LDS and (first query head of a kv group) stores the rotated k and the v row into the caches.
__global__ __launch_bounds__(1024) void rope_attn_split_kernel(
    const __half *__restrict__ q, const __half *__restrict__ k, const __half *__restrict__ v,
    __half *__restrict__ k_cache, __half *__restrict__ v_cache, __half *__restrict__ part, float *__restrict__ ml,
    const int *__restrict__ pos_ptr, int n_heads, int n_kv_heads, int max_len, int slices, RopeBase base, float scale) {
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    __shared__ float s_score[kMaxAttnLen];   // indexed by 64 * (the slice's block number) + position % 64
    __shared__ float s_red[32];
    __shared__ float s_acc[16][128];
    __shared__ __attribute__((aligned(16))) unsigned short s_qh[128], s_kh[128];  // rotated q, k as fp16
    const int head = blockIdx.x % n_heads, slice = blockIdx.x / n_heads;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int row = t >> 4, l16 = t & 15;
    const int rep = n_heads / n_kv_heads, kvh = head / rep;
    const uint4 *kb = reinterpret_cast<const uint4 *>(k_cache + (size_t)kvh * max_len * 128);
    const uint4 *vb = reinterpret_cast<const uint4 *>(v_cache + (size_t)kvh * max_len * 128);
    auto position = [&](int lb) { return 64 * (slice + slices * lb) + row; };  // this thread's row of the slice's block lb
    // A cache that four blocks per slice cover is requested whole before the position is known (one
    // memory round trip in front of the arithmetic); of a longer one only the rows up to the
    // position are read, after it has arrived (rows beyond it would be most of the traffic).
    const bool early = max_len <= 256 * slices;
    uint4 k_first[4], v_first[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const int j = position(u);
        k_first[u] = early && j < max_len ? kb[(size_t)j * 16 + l16] : make_uint4(0, 0, 0, 0);
        v_first[u] = early && j < max_len ? vb[(size_t)j * 16 + l16] : make_uint4(0, 0, 0, 0);
    }
    float x1 = 0.f, x2 = 0.f, inv_freq = 0.f;
    __half v1 = __float2half(0.f), v2 = v1;
    if (t < 128) {
        const int i = t & 63;
        const __half *src = t >= 64 ? k + (size_t)kvh * 128 : q + (size_t)head * 128;
        x1 = __half2float(src[i]);
        x2 = __half2float(src[i + 64]);
        if (t >= 64) {
            v1 = v[(size_t)kvh * 128 + i];
            v2 = v[(size_t)kvh * 128 + i + 64];
        }
        inv_freq = rope_inv_freq(i, 128, base);
    }
    const int pos = *pos_ptr;
    __half *pdst = part + ((size_t)slice * n_heads + head) * 128;
    float *mdst = ml + ((size_t)slice * n_heads + head) * 2;
    if ((unsigned)pos >= (unsigned)max_len) {  // outside the cache: nothing read or written, the output is NaN
        if (t < 128) pdst[t] = __ushort_as_half((unsigned short)0x7e00);
        if (t == 0) {
            mdst[0] = 0.f;
            mdst[1] = 1.f;
        }
        return;
    }
    const int used = pos / 64 + 1;  // blocks that hold positions 0 .. pos
    if (slice >= used) {            // nothing to attend to in this slice
        if (t < 128) pdst[t] = __float2half(0.f);
        if (t == 0) {
            mdst[0] = -INFINITY;
            mdst[1] = 0.f;
        }
        return;
    }
    const bool has_new = (used - 1) % slices == slice;  // the new position lies in this slice's last block
    const int nblk = (used - slice + slices - 1) / slices;
    const int len = 64 * nblk - (has_new ? 63 - pos % 64 : 0);  // positions of this slice, the new one included
    const int cached = len - (has_new ? 1 : 0);
    if (!early) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int j = position(u);
            k_first[u] = j < pos ? kb[(size_t)j * 16 + l16] : make_uint4(0, 0, 0, 0);
            v_first[u] = j < pos ? vb[(size_t)j * 16 + l16] : make_uint4(0, 0, 0, 0);
        }
    }
    if (t < 128) {
        const int i = t & 63;
        const bool is_k = t >= 64;
        float sn, cs;
        sincosf((float)pos * inv_freq, &sn, &cs);
        const float c = __half2float(__float2half_rn(cs)), sr = __half2float(__float2half_rn(sn));
        const float a1 = __half2float(__float2half_rn(x1 * c)), b1 = __half2float(__float2half_rn(-x2 * sr));
        const float a2 = __half2float(__float2half_rn(x2 * c)), b2 = __half2float(__float2half_rn(x1 * sr));
        const __half o1 = __float2half_rn(a1 + b1), o2 = __float2half_rn(a2 + b2);
        unsigned short *dst = is_k ? s_kh : s_qh;
        dst[i] = __half_as_ushort(o1);
        dst[i + 64] = __half_as_ushort(o2);
        if (is_k && has_new && head % rep == 0) {
            __half *kd = k_cache + ((size_t)kvh * max_len + pos) * 128;
            __half *vd = v_cache + ((size_t)kvh * max_len + pos) * 128;
            kd[i] = o1;
            kd[i + 64] = o2;
            vd[i] = v1;
            vd[i + 64] = v2;
        }
    }
    __syncthreads();
    const uint4 qv = *reinterpret_cast<const uint4 *>(&s_qh[8 * l16]);
    auto dot8 = [&](const uint4 &kv) {
        float d = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, kv.x), __builtin_bit_cast(half2_t, qv.x), 0.f, false);
        d = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, kv.y), __builtin_bit_cast(half2_t, qv.y), d, false);
        d = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, kv.z), __builtin_bit_cast(half2_t, qv.z), d, false);
        d = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, kv.w), __builtin_bit_cast(half2_t, qv.w), d, false);
        return row_sum(d);
    };
    float m = -INFINITY;
    for (int lb0 = 0; 64 * lb0 < cached; lb0 += 4) {
        uint4 kk[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int j = position(lb0 + u);
            if (lb0 == 0)
                kk[u] = k_first[u];
            else
                kk[u] = j < pos ? kb[(size_t)j * 16 + l16] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const float sc = __half2float(__float2half_rn(dot8(kk[u]))) * scale;
            if (position(lb0 + u) < pos) {
                m = fmaxf(m, sc);
                if (l16 == 0) s_score[64 * (lb0 + u) + row] = sc;
            }
        }
    }
    if (has_new && row == 0) {  // the new position, from LDS
        const float sc = __half2float(__float2half_rn(dot8(*reinterpret_cast<const uint4 *>(&s_kh[8 * l16])))) * scale;
        m = fmaxf(m, sc);
        if (l16 == 0) s_score[len - 1] = sc;
    }
    m = wave_max_all(m);
    if (lane == 0) s_red[wave] = m;
    __syncthreads();
    m = s_red[0];
#pragma unroll
    for (int w = 1; w < 16; w++) m = fmaxf(m, s_red[w]);
    float sum = 0.f;
    for (int j = t; j < len; j += 1024) {
        const float e = __expf(s_score[j] - m);
        s_score[j] = e;
        sum += e;
    }
    sum = wave_sum_all(sum);
    if (lane == 0) s_red[16 + wave] = sum;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < 16; w++) tot += s_red[16 + w];
    const float inv = 1.f / tot;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = 0.f;
    for (int lb0 = 0; 64 * lb0 < cached; lb0 += 4) {
        uint4 vv[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int j = position(lb0 + u);
            if (lb0 == 0)
                vv[u] = j < pos ? v_first[u] : make_uint4(0, 0, 0, 0);  // rows past the position may hold anything
            else
                vv[u] = j < pos ? vb[(size_t)j * 16 + l16] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const float p = position(lb0 + u) < pos ? __half2float(__float2half_rn(s_score[64 * (lb0 + u) + row] * inv)) : 0.f;
            float vf[8];
            unpack8(vv[u], vf);
#pragma unroll
            for (int i = 0; i < 8; i++) acc[i] = fmaf(p, vf[i], acc[i]);
        }
    }
    if (has_new && row == 0) {
        const float p = __half2float(__float2half_rn(s_score[len - 1] * inv));
        float vf[8];
        unpack8(reinterpret_cast<const uint4 *>(v + (size_t)kvh * 128)[l16], vf);
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = fmaf(p, vf[i], acc[i]);
    }
    {
        float h4[4], q2[2];
#pragma unroll
        for (int i = 0; i < 4; i++) h4[i] = swap32_add(acc[i], acc[4 + i]);
#pragma unroll
        for (int i = 0; i < 2; i++) q2[i] = swap16_add(h4[i], h4[2 + i]);
        const int d0 = 8 * l16 + 4 * (lane >> 5) + 2 * ((lane >> 4) & 1);
        s_acc[wave][d0] = q2[0];
        s_acc[wave][d0 + 1] = q2[1];
    }
    __syncthreads();
    if (t < 128) {
        float o = 0.f;
#pragma unroll
        for (int w = 0; w < 16; w++) o += s_acc[w][t];
        pdst[t] = __float2half_rn(o);
    }
    if (t == 0) {
        mdst[0] = m;
        mdst[1] = tot;
    }
}

// out[head][d] <- fp16(sum_s c_s * part[s][head][d]) with the factors of attn_combine_weights();
// one thread per output element.  (The output projection over a weight stream applies the same
// factors while it stages its input; this kernel serves every other reader.)
__global__ __launch_bounds__(256) void attn_combine_kernel(const __half *__restrict__ part, const float *__restrict__ ml,
                                                           __half *__restrict__ out, int n_heads, int slices) {
    const int i = blockIdx.x * 256 + threadIdx.x, n = n_heads * 128;
    if (i >= n) return;
    const int head = i >> 7;
    float mv[kAttnMaxSlices], lv[kAttnMaxSlices], c[kAttnMaxSlices];
#pragma unroll
    for (int s = 0; s < kAttnMaxSlices; s++) {
        const bool on = s < slices;
        mv[s] = on ? ml[((size_t)s * n_heads + head) * 2] : -INFINITY;
        lv[s] = on ? ml[((size_t)s * n_heads + head) * 2 + 1] : 0.f;
    }
    attn_combine_weights(mv, lv, c);
    float o = 0.f;
#pragma unroll
    for (int s = 0; s < kAttnMaxSlices; s++)
        if (s < slices) o = fmaf(c[s], __half2float(part[(size_t)s * n + i]), o);
    out[i] = __float2half_rn(o);
}

// out <- fp16(silu(gate)) * up
__global__ __launch_bounds__(256) void silu_mul_kernel(const __half *__restrict__ gate, const __half *__restrict__ up,
                                                       __half *__restrict__ out, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float g = __half2float(gate[i]);
    const float a = __half2float(__float2half_rn(g / (1.f + __expf(-g))));
    out[i] = __float2half_rn(a * __half2float(up[i]));
}

// Unquantised fp16 head: logits[v] = fp16(sum_k act[k] * W[v][k]) with W (vocab, hidden) row-major
// as the reference's lm_head holds it (llama/modeling_llama_quant.py:1132), fp32 accumulation, and
// act = weight * fp16(h * rsqrt(mean(h^2) + eps)) -- the final RMSNorm (:1064), with the rounding
// points of add_rmsnorm_kernel -- or act = h when no norm weight is given.  The matrix is the
// largest single read of a token step (262 MB for 32000 x 4096), so the kernel is a plain
// HBM stream: every wavefront keeps the whole activation row in registers (CH pieces of 16 bytes
// per lane), normalises it itself (no LDS, no barrier) and then takes rows v = w, w + waves, ...,
// one row = CH loads of 1 KB, the next row's loads in flight while the current one is multiplied.
// RAGGED: the hidden size Hr is not a multiple of 512 (CH = ceil(Hr / 512)); lanes whose piece of the
// last 1 KB lies past the row read nothing and multiply zeros.
typedef uint32_t hu4 __attribute__((ext_vector_type(4)));

template <int CH, bool RAGGED>
__global__ __launch_bounds__(256) void head_kernel(const __half *__restrict__ h, const __half *__restrict__ norm_w,
                                                   float eps, const __half *__restrict__ W,
                                                   __half *__restrict__ logits, int V, int Hr) {
    const int H = RAGGED ? Hr : 512 * CH;
    const int lane = threadIdx.x & 63;
    const int w = blockIdx.x * 4 + (threadIdx.x >> 6), nw = gridDim.x * 4;
    const hu4 zero = {0u, 0u, 0u, 0u};
    auto has = [&](int c) { return !RAGGED || c < CH - 1 || ((CH - 1) * 64 + lane) * 8 < H; };  // (H % 8 == 0)
    auto load_row = [&](hu4 (&dst)[CH], int v) {
        const hu4 *row = reinterpret_cast<const hu4 *>(W + (size_t)v * H);
#pragma unroll
        for (int c = 0; c < CH; c++) dst[c] = has(c) ? __builtin_nontemporal_load(row + c * 64 + lane) : zero;
    };
    float x[CH][8];
    {
        hu4 xr[CH];
#pragma unroll
        for (int c = 0; c < CH; c++) xr[c] = has(c) ? reinterpret_cast<const hu4 *>(h)[c * 64 + lane] : zero;
        if (norm_w) {
            hu4 nr[CH];
#pragma unroll
            for (int c = 0; c < CH; c++) nr[c] = has(c) ? reinterpret_cast<const hu4 *>(norm_w)[c * 64 + lane] : zero;
            float ss = 0.f;
#pragma unroll
            for (int c = 0; c < CH; c++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float a = __half2float(__ushort_as_half((unsigned short)(xr[c][j] & 0xffffu)));
                    const float b = __half2float(__ushort_as_half((unsigned short)(xr[c][j] >> 16)));
                    ss += a * a + b * b;
                }
            ss = wave_sum_all(ss);
            const float rs = rsqrtf(ss / (float)H + eps);
#pragma unroll
            for (int c = 0; c < CH; c++)
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const float xv = __half2float(__ushort_as_half((unsigned short)(xr[c][j >> 1] >> (16 * (j & 1)))));
                    const float wv = __half2float(__ushort_as_half((unsigned short)(nr[c][j >> 1] >> (16 * (j & 1)))));
                    const float n = __half2float(__float2half_rn(xv * rs));
                    x[c][j] = __half2float(__float2half_rn(wv * n));
                }
        } else {
#pragma unroll
            for (int c = 0; c < CH; c++)
#pragma unroll
                for (int j = 0; j < 8; j++)
                    x[c][j] = __half2float(__ushort_as_half((unsigned short)(xr[c][j >> 1] >> (16 * (j & 1)))));
        }
    }
    auto finish_row = [&](const hu4 (&r)[CH], int v) {
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int c = 0; c < CH; c++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                a0 = fmaf(__half2float(__ushort_as_half((unsigned short)(r[c][j] & 0xffffu))), x[c][2 * j], a0);
                a1 = fmaf(__half2float(__ushort_as_half((unsigned short)(r[c][j] >> 16))), x[c][2 * j + 1], a1);
            }
        const float tot = wave_sum_all(a0 + a1);
        if (lane == 0) logits[v] = __float2half_rn(tot);
    };
    hu4 ra[CH], rb[CH];
    int v = w;
    if (v < V) load_row(ra, v);
    while (v < V) {
        if (v + nw < V) load_row(rb, v + nw);
        finish_row(ra, v);
        v += nw;
        if (v >= V) break;
        if (v + nw < V) load_row(ra, v + nw);
        finish_row(rb, v);
        v += nw;
    }
}

bool head_supported(int vocab, int hidden) { return vocab > 0 && hidden >= 8 && hidden <= 8192 && hidden % 8 == 0; }

hipError_t launch_head(const __half *h, const __half *norm_w, float eps, const __half *W, __half *logits, int vocab,
                       int hidden, hipStream_t stream) {
    if (!head_supported(vocab, hidden)) return hipErrorInvalidValue;
    int grid = ceil_div(vocab, 4);
    if (grid > 1024) grid = 1024;  // four wavefronts per SIMD
    const bool ragged = hidden % 512 != 0;
    switch (ceil_div(hidden, 512)) {
#define CQ_HEAD_CASE(CH_)                                                                                                       \
    case CH_:                                                                                                                   \
        if (ragged)                                                                                                             \
            hipLaunchKernelGGL((head_kernel<CH_, true>), dim3(grid), dim3(256), 0, stream, h, norm_w, eps, W, logits, vocab, hidden);  \
        else                                                                                                                    \
            hipLaunchKernelGGL((head_kernel<CH_, false>), dim3(grid), dim3(256), 0, stream, h, norm_w, eps, W, logits, vocab, hidden); \
        break;
        CQ_HEAD_CASE(1) CQ_HEAD_CASE(2) CQ_HEAD_CASE(3) CQ_HEAD_CASE(4) CQ_HEAD_CASE(5) CQ_HEAD_CASE(6) CQ_HEAD_CASE(7)
        CQ_HEAD_CASE(8) CQ_HEAD_CASE(9) CQ_HEAD_CASE(10) CQ_HEAD_CASE(11) CQ_HEAD_CASE(12) CQ_HEAD_CASE(13)
        CQ_HEAD_CASE(14) CQ_HEAD_CASE(15) CQ_HEAD_CASE(16)
#undef CQ_HEAD_CASE
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// Tail of a greedy decoding step, one workgroup: next = argmax(logits) (lowest index among equal
// maxima), recorded in *next_token and history[*pos]; the next token's embedding row becomes the
// hidden state of the following step; *pos += 1.  What the reference's generation loop does on
// the host between two forward passes (benchmark_perplexity.py:92-109), kept on the device so
// that a replayed graph needs no host work per token.
__global__ __launch_bounds__(1024) void argmax_embed_kernel(const __half *__restrict__ logits, int vocab,
                                                            const __half *__restrict__ embed, int hidden,
                                                            __half *__restrict__ hid, long long *__restrict__ next_token,
                                                            long long *__restrict__ history, int history_len,
                                                            int *__restrict__ pos_ptr) {
    __shared__ float s_val[16];
    __shared__ int s_idx[16];
    __shared__ int s_best;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    // 8 logits per 16-byte load; the tail that is not a multiple of 8 is read element-wise
    const int vec_end = vocab & ~7;
    for (int i = 8 * t; i < vec_end; i += 8 * 1024) {
        float f[8];
        unpack8(*reinterpret_cast<const uint4 *>(logits + i), f);
#pragma unroll
        for (int e = 0; e < 8; e++)
            if (f[e] > best) {
                best = f[e];
                best_i = i + e;
            }
    }
    for (int i = vec_end + t; i < vocab; i += 1024) {
        const float f = __half2float(logits[i]);
        if (f > best) {
            best = f;
            best_i = i;
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o);
        const int oi = __shfl_xor(best_i, o);
        if (ov > best || (ov == best && oi < best_i)) {
            best = ov;
            best_i = oi;
        }
    }
    if (lane == 0) {
        s_val[wave] = best;
        s_idx[wave] = best_i;
    }
    __syncthreads();
    if (t == 0) {
        for (int w = 1; w < 16; w++)
            if (s_val[w] > best || (s_val[w] == best && s_idx[w] < best_i)) {
                best = s_val[w];
                best_i = s_idx[w];
            }
        if (best_i >= vocab) best_i = 0;  // every logit was NaN or -inf
        s_best = best_i;
        const int pos = *pos_ptr;
        *next_token = best_i;
        if (history && pos >= 0 && pos < history_len) history[pos] = best_i;
        *pos_ptr = pos + 1;
    }
    __syncthreads();
    const __half *row = embed + (size_t)s_best * hidden;
    for (int i = t; i < hidden; i += 1024) hid[i] = row[i];
}

hipError_t launch_argmax_embed(const __half *logits, int vocab, const __half *embed, int hidden, __half *hid,
                               long long *next_token, long long *history, int history_len, int *pos,
                               hipStream_t stream) {
    hipLaunchKernelGGL(argmax_embed_kernel, dim3(1), dim3(1024), 0, stream, logits, vocab, embed, hidden, hid,
                       next_token, history, history_len, pos);
    return hipGetLastError();
}

hipError_t launch_add_rmsnorm(__half *h, const __half *delta, const __half *weight, __half *y, int H, float eps,
                              hipStream_t stream) {
    hipLaunchKernelGGL(add_rmsnorm_kernel, dim3(1), dim3(1024), 0, stream, h, delta, weight, y, H, eps);
    return hipGetLastError();
}

hipError_t launch_rope_cache(__half *q, const __half *k, const __half *v, __half *k_cache, __half *v_cache,
                             const int *pos, int n_heads, int n_kv_heads, int head_dim, int max_len, float theta,
                             hipStream_t stream) {
    hipLaunchKernelGGL(rope_cache_kernel, dim3(n_heads + n_kv_heads), dim3(head_dim / 2), 0, stream, q, k, v, k_cache,
                       v_cache, pos, n_heads, n_kv_heads, head_dim, max_len, rope_base(theta));
    return hipGetLastError();
}

hipError_t launch_attn_decode(const __half *q, const __half *k_cache, const __half *v_cache, __half *out,
                              const int *pos, int n_heads, int n_kv_heads, int max_len, float scale,
                              hipStream_t stream) {
    hipLaunchKernelGGL(attn_decode_kernel, dim3(n_heads), dim3(256), 0, stream, q, k_cache, v_cache, out, pos, n_heads,
                       n_kv_heads, max_len, scale);
    return hipGetLastError();
}

hipError_t launch_rope_attn_decode(const __half *q, const __half *k, const __half *v, __half *k_cache,
                                   __half *v_cache, __half *out, const int *pos, int n_heads, int n_kv_heads,
                                   int max_len, float theta, float scale, hipStream_t stream) {
    hipLaunchKernelGGL(rope_attn_decode_kernel, dim3(n_heads), dim3(1024), 0, stream, q, k, v, k_cache, v_cache, out,
                       pos, n_heads, n_kv_heads, max_len, rope_base(theta), scale);
    return hipGetLastError();
}

hipError_t launch_rope_attn_split(const __half *q, const __half *k, const __half *v, __half *k_cache, __half *v_cache,
                                  __half *part, float *ml, const int *pos, int n_heads, int n_kv_heads, int max_len,
                                  int slices, float theta, float scale, hipStream_t stream) {
    // 60 KB of unused dynamic LDS on top of the 25 KB the kernel declares: more than half of a compute
    // unit's, so that the workgroups spread one per compute unit instead of sharing one's memory pipeline
    hipLaunchKernelGGL(rope_attn_split_kernel, dim3(n_heads * slices), dim3(1024), 60 * 1024, stream, q, k, v, k_cache, v_cache,
                       part, ml, pos, n_heads, n_kv_heads, max_len, slices, rope_base(theta), scale);
    return hipGetLastError();
}

hipError_t launch_attn_combine(const __half *part, const float *ml, __half *out, int n_heads, int slices,
                               hipStream_t stream) {
    hipLaunchKernelGGL(attn_combine_kernel, dim3(ceil_div(n_heads * 128, 256)), dim3(256), 0, stream, part, ml, out,
                       n_heads, slices);
    return hipGetLastError();
}

hipError_t launch_silu_mul(const __half *gate, const __half *up, __half *out, int n, hipStream_t stream) {
    hipLaunchKernelGGL(silu_mul_kernel, dim3(ceil_div(n, 256)), dim3(256), 0, stream, gate, up, out, n);
    return hipGetLastError();
}

int attn_max_len() { return kMaxAttnLen; }

}  // namespace cq
