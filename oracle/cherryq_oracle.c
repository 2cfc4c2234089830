/*
 * CPU oracle (plain C) for CherryQ's mixed-precision quantized linear.
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP path and the timed CPU baseline.
 * Nothing in the product library links or loads this file.
 *
 * It restates the reference's CPU path, QuantLinear.unpack() followed by
 * nn.functional.linear (llama/qlinear.py:120-162 and :194-195), plus the arithmetic
 * contract of the fused entry points (csrc/quant_cuda_kernel.cu:718-835, 558-672).
 * Parity status: pinned against the numpy oracle (itself pinned by the golden vectors
 * recorded from the reference's Python) in tests/test_oracle_c.py.
 *
 * Build: see oracle/Makefile.  All tensors are row-major and contiguous; fp16 values are
 * passed as uint16_t bit patterns.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ---- IEEE binary16 <-> binary32, round to nearest even ---------------------------- */

static inline float h2f(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static inline uint16_t f2h(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | (absx > 0x7F800000u ? 0x200u : 0));
    if (absx >= 0x477FF000u) /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7C00u);
    if (absx < 0x38800000u) { /* subnormal half or zero */
        if (absx < 0x33000000u) return (uint16_t)sign; /* < 2^-25 -> 0 */
        int e = (int)(absx >> 23);
        uint32_t man = (absx & 0x7FFFFFu) | 0x800000u;
        int shift = 126 - e; /* 14..24 */
        uint32_t half = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1u))) half++;
        return (uint16_t)(sign | half);
    }
    uint32_t half = ((absx >> 13) - (112u << 10));
    uint32_t rem = absx & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++;
    return (uint16_t)(sign | half);
}

uint16_t cherryq_oracle_f2h(float f) { return f2h(f); }
float cherryq_oracle_h2f(uint16_t h) { return h2f(h); }

int cherryq_oracle_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ---- codes ------------------------------------------------------------------------ */

/* Code of compacted normal position k, column n.  4-bit: llama/qlinear.py:89-94 /
 * csrc/quant_cuda_kernel.cu:811-829.  3-bit: little-endian 24-bit unit over three byte
 * rows, llama/qlinear.py:95-114 / csrc/quant_cuda_kernel.cu:649-667. */
static inline unsigned code_at(const uint8_t *qw, int bits, long n_cols, long k, long n) {
    if (bits == 4) {
        unsigned b = qw[(k >> 1) * n_cols + n];
        return (b >> (4 * (k & 1))) & 15u;
    }
    long t = k >> 3;
    unsigned w24 = (unsigned)qw[(3 * t) * n_cols + n] | ((unsigned)qw[(3 * t + 1) * n_cols + n] << 8) |
                   ((unsigned)qw[(3 * t + 2) * n_cols + n] << 16);
    return (w24 >> (3 * (k & 7))) & 7u;
}

/* normal[k]: ascending complement of the sorted cherry indices (llama/qlinear.py:75-76) */
static void build_normal(const int16_t *idx, int C, int K, int32_t *normal) {
    int c = 0, j = 0;
    for (int k = 0; k < K; k++) {
        if (c < C && idx[c] == k) { c++; continue; }
        normal[j++] = k;
    }
}

/* ---- QuantLinear.unpack(): dense (N, K) fp16 -------------------------------------- */
/* llama/qlinear.py:120-162 with FullSymQuantizer.dequantize (llama/quantizer.py:160-163):
 * normal column normal[k] <- RN16( (fp16(u - 2^(b-1)) + 0.5) * s[k/G, n] ), cherry column
 * idx[c] <- cherry_weight[c, n].  (q + 0.5) is exact in fp16 and the product of a 4-bit
 * and an 11-bit significand is exact in float, so one rounding remains. */
int cherryq_oracle_unpack(int bits, const uint8_t *qweight, const uint16_t *scales,
                          const uint16_t *cherry_weight, const int16_t *cherry_indices,
                          int K, int N, int C, int G, uint16_t *dense) {
    if (bits != 3 && bits != 4) return -1;
    int Kn = K - C;
    int32_t *normal = (int32_t *)malloc(sizeof(int32_t) * (size_t)(K > 0 ? K : 1));
    if (!normal) return -2;
    build_normal(cherry_indices, C, K, normal);
    const float cb = (float)(1 << (bits - 1)) - 0.5f;
#pragma omp parallel for schedule(static)
    for (long n = 0; n < N; n++) {
        uint16_t *row = dense + n * (long)K;
        for (long k = 0; k < Kn; k++) {
            float s = h2f(scales[(k / G) * (long)N + n]);
            float v = ((float)code_at(qweight, bits, N, k, n) - cb) * s;
            row[normal[k]] = f2h(v);
        }
        for (int c = 0; c < C; c++) row[cherry_indices[c]] = cherry_weight[(long)c * N + n];
    }
    free(normal);
    return 0;
}

/* ---- nn.functional.linear on fp16 operands ---------------------------------------- */
/* llama/qlinear.py:194-195.  Exactly converted operands, double accumulation, one
 * rounding to fp16 (torch leaves the CPU summation order unspecified). */
int cherryq_oracle_linear(const uint16_t *x, const uint16_t *dense, int B, int K, int N,
                          uint16_t *y, double *y_f64) {
    float *xf = (float *)malloc(sizeof(float) * (size_t)B * K);
    if (!xf) return -2;
    for (long i = 0; i < (long)B * K; i++) xf[i] = h2f(x[i]);
#pragma omp parallel for schedule(static)
    for (long n = 0; n < N; n++) {
        const uint16_t *row = dense + n * (long)K;
        for (int b = 0; b < B; b++) {
            const float *xb = xf + (long)b * K;
            double a0 = 0, a1 = 0, a2 = 0, a3 = 0;
            long k = 0;
            for (; k + 4 <= K; k += 4) {
                a0 += (double)h2f(row[k]) * xb[k];
                a1 += (double)h2f(row[k + 1]) * xb[k + 1];
                a2 += (double)h2f(row[k + 2]) * xb[k + 2];
                a3 += (double)h2f(row[k + 3]) * xb[k + 3];
            }
            for (; k < K; k++) a0 += (double)h2f(row[k]) * xb[k];
            double a = (a0 + a1) + (a2 + a3);
            if (y_f64) y_f64[(long)b * N + n] = a;
            if (y) y[(long)b * N + n] = f2h((float)a);
        }
    }
    free(xf);
    return 0;
}

/* ---- fused entry-point contract, un-rounded weights, double accumulation ---------- */
/* mul[b,n] += sum_k (u[k,n]-c_b) s[k/G,n] x[b,normal[k]] + sum_c cw[c,n] x[b,idx[c]]
 * csrc/quant_cuda_kernel.cu:797-834 (normal blocks) and 738-762 (cherry blocks). */
int cherryq_oracle_fused(int bits, const uint16_t *x, const uint8_t *qweight,
                         const uint16_t *cherry_weight, const int16_t *cherry_indices,
                         const uint16_t *scales, int B, int K, int N, int C, int G, double *y) {
    if (bits != 3 && bits != 4) return -1;
    int Kn = K - C;
    int32_t *normal = (int32_t *)malloc(sizeof(int32_t) * (size_t)(K > 0 ? K : 1));
    if (!normal) return -2;
    build_normal(cherry_indices, C, K, normal);
    const double cb = (double)(1 << (bits - 1)) - 0.5;
#pragma omp parallel for schedule(static)
    for (long n = 0; n < N; n++) {
        for (int b = 0; b < B; b++) {
            const uint16_t *xb = x + (long)b * K;
            double acc = 0;
            for (long g0 = 0; g0 < Kn; g0 += G) {
                double part = 0;
                long g1 = g0 + G < Kn ? g0 + G : Kn;
                for (long k = g0; k < g1; k++)
                    part += ((double)code_at(qweight, bits, N, k, n) - cb) * (double)h2f(xb[normal[k]]);
                acc += part * (double)h2f(scales[(g0 / G) * (long)N + n]);
            }
            for (int c = 0; c < C; c++)
                acc += (double)h2f(cherry_weight[(long)c * N + n]) * (double)h2f(xb[cherry_indices[c]]);
            y[(long)b * N + n] = acc;
        }
    }
    free(normal);
    return 0;
}

/* ---- the reference CPU path end to end: unpack() then linear() -------------------- */
/* llama/qlinear.py:183-195 (first call under dmode(layerwise_dequantize=False)). */
int cherryq_oracle_dequant_matmul(int bits, const uint16_t *x, const uint8_t *qweight,
                                  const uint16_t *cherry_weight, const int16_t *cherry_indices,
                                  const uint16_t *scales, int B, int K, int N, int C, int G,
                                  uint16_t *dense_scratch, uint16_t *y) {
    int rc = cherryq_oracle_unpack(bits, qweight, scales, cherry_weight, cherry_indices, K, N, C, G,
                                   dense_scratch);
    if (rc) return rc;
    return cherryq_oracle_linear(x, dense_scratch, B, K, N, y, NULL);
}

/* ---- Dequantize{3,4}Normal: dense fp32 (Kn, N) of the compacted normal part -------- */
/* csrc/quant_cuda_kernel.cu:869-922 (3-bit); the 4-bit kernel (956-1010) is stated with
 * the evident intent, i.e. the same indexing with 64 byte rows per 128 positions. */
int cherryq_oracle_dequantize_normal(int bits, const uint8_t *qweight, const float *scales,
                                     float *out, int height, int N, int cherry_size, int G) {
    if (bits != 3 && bits != 4) return -1;
    long Kn = height - cherry_size;
    const float cb = (float)(1 << (bits - 1)) - 0.5f;
#pragma omp parallel for schedule(static)
    for (long k = 0; k < Kn; k++)
        for (long n = 0; n < N; n++)
            out[k * N + n] = ((float)code_at(qweight, bits, N, k, n) - cb) * scales[(k / G) * (long)N + n];
    return 0;
}
