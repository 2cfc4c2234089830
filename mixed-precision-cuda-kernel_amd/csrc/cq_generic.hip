// Generic fused dequant + matmul kernel: any batch (in chunks of kMaxB rows), 3/4 bit, group
// sizes that are multiples of 32, fp16 or fp32 I/O.  One wavefront per workgroup; lanes run
// across 256 output columns (one dword = 4 columns of a byte row per lane), the K dimension
// is walked in units of 128 compacted positions and split across workgroups.  This is the
// reference-shaped path for everything the specialised kernels (cq_matvec.hip) do not take.
//
// Arithmetic contract: csrc/quant_cuda_kernel.cu:718-835 (4-bit), 558-672 / 316-438 (3-bit,
// group multiple of 128 / group 64), 441-556 / 191-314 (fp32 I/O), with fp32 accumulation
// kept until a single final rounding instead of one fp16 atomic per 128 positions (:833).
#include "cq_common.cuh"
#include "cq_kernels.h"

namespace cq {

constexpr int kMaxB = 8;

template <int BITS>
__device__ inline void decode8(const uint32_t *w, int col, float (&v)[8]);

// 4-bit: four byte rows hold eight codes of a column, low nibble first.
template <>
__device__ inline void decode8<4>(const uint32_t *w, int col, float (&v)[8]) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
        uint32_t byte = (w[r] >> (8 * col)) & 0xFFu;
        v[2 * r] = (float)(byte & 15u) - 7.5f;
        v[2 * r + 1] = (float)(byte >> 4) - 7.5f;
    }
}

// 3-bit: three byte rows form a little-endian 24-bit word of eight codes.
template <>
__device__ inline void decode8<3>(const uint32_t *w, int col, float (&v)[8]) {
    uint32_t w24 = ((w[0] >> (8 * col)) & 0xFFu) | (((w[1] >> (8 * col)) & 0xFFu) << 8) |
                   (((w[2] >> (8 * col)) & 0xFFu) << 16);
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = (float)((w24 >> (3 * i)) & 7u) - 3.5f;
}

template <int BITS, typename IO, typename IDX>
__global__ __launch_bounds__(64) void generic_kernel(
    const IO *__restrict__ vec, const uint8_t *__restrict__ qweight,
    const IO *__restrict__ cherry_weight, const IDX *__restrict__ cherry_indices,
    const IO *__restrict__ scales, IO *__restrict__ mul, unsigned long long *__restrict__ acc_words, int B,
    int K, int N, int C, int G, int accumulate, Plan plan) {
    const int lane = threadIdx.x;
    const int lid = xcd_remap(blockIdx.x, gridDim.x);
    const int tile = lid / plan.splits;
    const int split = lid % plan.splits;
    const int n0 = tile * kTileCols + lane * 4;
    const bool active = n0 < N;
    const int Kn = K - C;
    const int qrows = Kn / 8 * BITS;
    constexpr int kRowsPer8 = BITS;  // byte rows per 8 codes

    __shared__ float xs[kMaxB][kUnitK];
    float acc[kMaxB][4];
#pragma unroll
    for (int b = 0; b < kMaxB; b++)
#pragma unroll
        for (int c = 0; c < 4; c++) acc[b][c] = 0.f;

    const int u_begin = split * plan.units_per_wg;
    const int u_end = min(u_begin + plan.units_per_wg, plan.units_total);
    for (int u = u_begin; u < u_end; u++) {
        __syncthreads();
        if (u < plan.units_normal) {
            const int kbase = u * kUnitK;
            for (int j = lane; j < kUnitK; j += 64) {
                int k = kbase + j;
                int src = k + gather_offset(cherry_indices, C, k);
                for (int b = 0; b < B; b++)
                    xs[b][j] = (k < Kn) ? to_float(vec[(size_t)b * K + src]) : 0.f;
            }
            __syncthreads();
            if (active) {
                // 128 positions in slices of 32 so that a group boundary (G % 32 == 0) never
                // falls inside a slice
                for (int sl = 0; sl < 4; sl++) {
                    int k0 = kbase + 32 * sl;
                    if (k0 >= Kn) break;
                    float sc[4];
                    {
                        const IO *sp = scales + (size_t)(k0 / G) * N + n0;
#pragma unroll
                        for (int c = 0; c < 4; c++) sc[c] = to_float(sp[c]);
                    }
                    float part[kMaxB][4];
#pragma unroll
                    for (int b = 0; b < kMaxB; b++)
#pragma unroll
                        for (int c = 0; c < 4; c++) part[b][c] = 0.f;
                    for (int e = 0; e < 4; e++) {  // 8 codes per step
                        int kk = k0 + 8 * e;
                        if (kk >= Kn) break;
                        int r0 = kk / 8 * kRowsPer8;
                        uint32_t w[kRowsPer8];
#pragma unroll
                        for (int r = 0; r < kRowsPer8; r++)
                            w[r] = (r0 + r < qrows)
                                       ? *reinterpret_cast<const uint32_t *>(qweight + (size_t)(r0 + r) * N + n0)
                                       : 0u;
#pragma unroll
                        for (int c = 0; c < 4; c++) {
                            float v[8];
                            decode8<BITS>(w, c, v);
#pragma unroll
                            for (int b = 0; b < kMaxB; b++)
                                if (b < B) {
                                    const float *xb = &xs[b][32 * sl + 8 * e];
#pragma unroll
                                    for (int i = 0; i < 8; i++) part[b][c] += v[i] * xb[i];
                                }
                        }
                    }
#pragma unroll
                    for (int b = 0; b < kMaxB; b++)
#pragma unroll
                        for (int c = 0; c < 4; c++) acc[b][c] += sc[c] * part[b][c];
                }
            }
        } else {
            // cherry rows: dense fp16/fp32 weights times the activations of the cherry channels
            const int c0 = (u - plan.units_normal) * kCherryUnit;
            const int cn = min(kCherryUnit, C - c0);
            if (lane < cn)
                for (int b = 0; b < B; b++)
                    xs[b][lane] = to_float(vec[(size_t)b * K + (int)cherry_indices[c0 + lane]]);
            __syncthreads();
            if (active) {
                for (int j = 0; j < cn; j++) {
                    const IO *wp = cherry_weight + (size_t)(c0 + j) * N + n0;
                    float wv[4];
#pragma unroll
                    for (int c = 0; c < 4; c++) wv[c] = to_float(wp[c]);
#pragma unroll
                    for (int b = 0; b < kMaxB; b++)
                        if (b < B) {
                            float xv = xs[b][j];
#pragma unroll
                            for (int c = 0; c < 4; c++) acc[b][c] += wv[c] * xv;
                        }
                }
            }
        }
    }
    splitk_finish<IO, kMaxB, 4>(acc, B, N, n0, active, plan.splits, acc_words, mul, accumulate);
}

template <int BITS, typename IO, typename IDX>
hipError_t launch_generic(const IO *vec, const uint8_t *qweight, const IO *cherry_weight,
                          const IDX *cherry_indices, const IO *scales, IO *mul, int B, int K, int N,
                          int C, int G, int accumulate, void *workspace, hipStream_t stream) {
    int upw = 4;
    while (make_plan(K, N, C, upw).splits > kMaxSplits) upw <<= 1;
    Plan plan = make_plan(K, N, C, upw);
    unsigned long long *acc_words = reinterpret_cast<unsigned long long *>(workspace);
    for (int b0 = 0; b0 < B; b0 += kMaxB) {
        int nb = min(kMaxB, B - b0);
        hipLaunchKernelGGL((generic_kernel<BITS, IO, IDX>), dim3(plan.tiles * plan.splits), dim3(64), 0,
                           stream, vec + (size_t)b0 * K, qweight, cherry_weight, cherry_indices, scales,
                           mul + (size_t)b0 * N, acc_words, nb, K, N, C, G, accumulate, plan);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

template hipError_t launch_generic<4, __half, int16_t>(const __half *, const uint8_t *, const __half *,
                                                       const int16_t *, const __half *, __half *, int, int,
                                                       int, int, int, int, void *, hipStream_t);
template hipError_t launch_generic<3, __half, int16_t>(const __half *, const uint8_t *, const __half *,
                                                       const int16_t *, const __half *, __half *, int, int,
                                                       int, int, int, int, void *, hipStream_t);
template hipError_t launch_generic<3, float, int32_t>(const float *, const uint8_t *, const float *,
                                                      const int32_t *, const float *, float *, int, int, int,
                                                      int, int, int, void *, hipStream_t);

// ---- dense dequant of the compacted normal part, fp32 (Kn, N) ------------------------------
// out[k, n] = (code(k, n) - c_b) * scales[k / G, n]; csrc/quant_cuda_kernel.cu:869-922.
template <int BITS>
__global__ __launch_bounds__(256) void dequant_normal_kernel(const uint8_t *__restrict__ qweight,
                                                             const float *__restrict__ scales,
                                                             float *__restrict__ out, int Kn, int N, int G) {
    const int n0 = (blockIdx.x * 256 + threadIdx.x) * 4;
    const int k0 = blockIdx.y * 8;
    if (n0 >= N || k0 >= Kn) return;
    uint32_t w[BITS];
#pragma unroll
    for (int r = 0; r < BITS; r++)
        w[r] = *reinterpret_cast<const uint32_t *>(qweight + (size_t)(k0 / 8 * BITS + r) * N + n0);
    const float4 s = *reinterpret_cast<const float4 *>(scales + (size_t)(k0 / G) * N + n0);
    const float sc[4] = {s.x, s.y, s.z, s.w};
    float v[4][8];
#pragma unroll
    for (int c = 0; c < 4; c++) decode8<BITS>(w, c, v[c]);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        float4 o = make_float4(v[0][i] * sc[0], v[1][i] * sc[1], v[2][i] * sc[2], v[3][i] * sc[3]);
        *reinterpret_cast<float4 *>(out + (size_t)(k0 + i) * N + n0) = o;
    }
}

hipError_t launch_dequant_normal(int bits, const uint8_t *qweight, const float *scales, float *out, int Kn,
                                 int N, int G, hipStream_t stream) {
    if (Kn == 0 || N == 0) return hipSuccess;
    dim3 grid(ceil_div(N, 1024), Kn / 8);
    if (bits == 4)
        hipLaunchKernelGGL(dequant_normal_kernel<4>, grid, dim3(256), 0, stream, qweight, scales, out, Kn, N, G);
    else
        hipLaunchKernelGGL(dequant_normal_kernel<3>, grid, dim3(256), 0, stream, qweight, scales, out, Kn, N, G);
    return hipGetLastError();
}

// ---- QuantLinear.unpack(): dense (N, K) fp16 -----------------------------------------------
// llama/qlinear.py:120-162.  A workgroup dequantises a 64-position x 64-column block, turns it
// through LDS and writes 128-byte row segments of the transposed (N, K) result.  Normal
// positions scatter to their original columns normal[k] = k + gather_offset(k); the cherry
// columns are copied by the trailing blocks of the grid.
template <int BITS>
__global__ __launch_bounds__(256) void unpack_kernel(const uint8_t *__restrict__ qweight,
                                                     const __half *__restrict__ cherry_weight,
                                                     const int16_t *__restrict__ cherry_indices,
                                                     const __half *__restrict__ scales,
                                                     __half *__restrict__ dense, int K, int N, int C, int G,
                                                     int kblocks) {
    __shared__ __half tile[64][64 + 2];
    __shared__ int dst[64];
    const int Kn = K - C;
    const int nb = blockIdx.x * 64;
    const int t = threadIdx.x;
    if ((int)blockIdx.y < kblocks) {
        const int kb = blockIdx.y * 64;
        if (t < 64) {
            int k = kb + t;
            dst[t] = (k < Kn) ? k + gather_offset(cherry_indices, C, k) : -1;
        }
        // 8 units of 8 positions x 16 column quads = 128 work items, two per pass of 256 threads
        if (t < 128) {
            const int unit = t >> 4, quad = t & 15;
            const int k0 = kb + unit * 8, n0 = nb + quad * 4;
            if (k0 < Kn && n0 < N) {
                uint32_t w[BITS];
#pragma unroll
                for (int r = 0; r < BITS; r++)
                    w[r] = *reinterpret_cast<const uint32_t *>(qweight + (size_t)(k0 / 8 * BITS + r) * N + n0);
                const __half *sp = scales + (size_t)(k0 / G) * N + n0;
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    float v[8];
                    decode8<BITS>(w, c, v);
                    // (code - c_b) has 4 significant bits and the fp16 scale 11: the float
                    // product is exact, so this is the single rounding the reference performs
                    float s = __half2float(sp[c]);
#pragma unroll
                    for (int i = 0; i < 8; i++) tile[quad * 4 + c][unit * 8 + i] = __float2half_rn(v[i] * s);
                }
            }
        }
        __syncthreads();
        // thread -> (row n = t / 4 .. , 16 consecutive positions)
        const int nl = t >> 2, seg = (t & 3) * 16;
        if (nb + nl < N) {
            __half *row = dense + (size_t)(nb + nl) * K;
            for (int j = 0; j < 16; j++) {
                int d = dst[seg + j];
                if (d >= 0) row[d] = tile[nl][seg + j];
            }
        }
    } else {
        // cherry columns: dense[n, idx[c]] = cherry_weight[c, n]
        const int cblk = blockIdx.y - kblocks;
        for (int i = t; i < 64 * 64; i += 256) {
            int c = cblk * 64 + (i >> 6), n = nb + (i & 63);
            if (c < C && n < N) dense[(size_t)n * K + (int)cherry_indices[c]] = cherry_weight[(size_t)c * N + n];
        }
    }
}

hipError_t launch_unpack(int bits, const uint8_t *qweight, const __half *cherry_weight,
                         const int16_t *cherry_indices, const __half *scales, __half *dense, int K, int N,
                         int C, int G, hipStream_t stream) {
    const int Kn = K - C;
    const int kblocks = ceil_div(Kn, 64);
    dim3 grid(ceil_div(N, 64), kblocks + ceil_div(C, 64));
    if (grid.x == 0 || grid.y == 0) return hipSuccess;
    if (bits == 4)
        hipLaunchKernelGGL(unpack_kernel<4>, grid, dim3(256), 0, stream, qweight, cherry_weight, cherry_indices,
                           scales, dense, K, N, C, G, kblocks);
    else
        hipLaunchKernelGGL(unpack_kernel<3>, grid, dim3(256), 0, stream, qweight, cherry_weight, cherry_indices,
                           scales, dense, K, N, C, G, kblocks);
    return hipGetLastError();
}

}  // namespace cq
