// Device-side pack(): dense fp16 weight (N, K) + sorted cherry channels -> the packed buffers
// (scales, qweight, cherry_weight), bit for bit what the host path computes.
//
// Arithmetic follows the reference's offline path: llama/qlinear.py:67-118 (column split, code
// offset, byte layout), llama/cherry_linear.py:69-75 (groups over the COMPACTED normal columns),
// llama/quantizer.py:148-158 (scale and rounding rule).  For fp16 weights every torch operation
// there is "compute in fp32, round to fp16":
//   s    = RN16( f32( RN16( f32(max|w|) + 1e-6f ) ) / 2^(b-1) )
//   q    = rint( clamp( f32( RN16( f32(w) / f32(s) ) ), -qmax, qmax ) - 0.5 ),  qmax = 2^(b-1) - 0.01
//   code = q + 2^(b-1)
// (fp32 division followed by rounding to fp16 equals the correctly rounded fp16 quotient: 24 >= 2*11+2.)
#include "cq_device.h"
#include "cq_kernels.h"

namespace cq {

// source channel of compacted normal position k: k + #{m : idx[m] - m <= k}
__device__ inline int normal_source(const int16_t *__restrict__ idx, int C, int k) {
    int lo = 0, hi = C;
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if ((int)idx[mid] - mid <= k) lo = mid + 1; else hi = mid;
    }
    return k + lo;
}

// One wavefront per (group, output row): scales[g, n].
__global__ __launch_bounds__(256) void pack_scales_kernel(const __half *__restrict__ w,
                                                          const int16_t *__restrict__ idx,
                                                          __half *__restrict__ scales, int K, int N, int C, int G,
                                                          int bits) {
    const int lane = threadIdx.x & 63;
    const long long item = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int Kn = K - C, ng = ceil_div(Kn, G);
    if (item >= (long long)ng * N) return;
    const int g = (int)(item / N), n = (int)(item % N);
    const int k0 = g * G, k1 = min(k0 + G, Kn);
    float mx = 0.f;
    for (int k = k0 + lane; k < k1; k += 64)
        mx = fmaxf(mx, fabsf(__half2float(w[(size_t)n * K + normal_source(idx, C, k)])));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if (lane == 0) {
        const float a = __half2float(__float2half_rn(mx + 1e-6f));
        scales[(size_t)g * N + n] = __float2half_rn(a / (float)(1 << (bits - 1)));
    }
}

// Tile of 64 output rows x 128 compacted positions per workgroup: the weights are read along K
// (contiguous in the dense layout), staged in LDS, and the packed bytes written along N
// (contiguous in the packed layout).
template <int BITS>
__global__ __launch_bounds__(256) void pack_codes_kernel(const __half *__restrict__ w,
                                                         const int16_t *__restrict__ idx,
                                                         const __half *__restrict__ scales,
                                                         uint8_t *__restrict__ qweight, int K, int N, int C, int G) {
    __shared__ unsigned short s_w[64][130];
    const int Kn = K - C;
    const int k0 = blockIdx.x * 128, n0 = blockIdx.y * 64;
    const int t = threadIdx.x;
    for (int e = t; e < 64 * 128; e += 256) {
        const int nl = e >> 7, kl = e & 127;
        const int n = n0 + nl, k = k0 + kl;
        unsigned short v = 0;
        if (n < N && k < Kn) v = __half_as_ushort(w[(size_t)n * K + normal_source(idx, C, k)]);
        s_w[nl][kl] = v;
    }
    __syncthreads();
    const float qmax = (float)(1 << (BITS - 1)) - 1e-2f;
    for (int e = t; e < 16 * 64; e += 256) {
        const int nl = e & 63, j = e >> 6;  // unit of 8 positions
        const int n = n0 + nl, k = k0 + 8 * j;
        if (n >= N || k >= Kn) continue;
        uint32_t word = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            // a group boundary can fall inside a unit when G is not a multiple of 8
            const float s = __half2float(scales[(size_t)((k + i) / G) * N + n]);
            const float x = __half2float(__ushort_as_half(s_w[nl][8 * j + i]));
            float r = __half2float(__float2half_rn(x / s));
            r = fminf(fmaxf(r, -qmax), qmax) - 0.5f;
            const int code = (int)rintf(r) + (1 << (BITS - 1));
            word |= (uint32_t)(code & ((1 << BITS) - 1)) << (BITS * i);
        }
        const size_t row = (size_t)(k / 8) * BITS;
#pragma unroll
        for (int b = 0; b < BITS; b++) qweight[(row + b) * N + n] = (uint8_t)(word >> (8 * b));
    }
}

// cherry_weight[c, n] = w[n, idx[c]]
__global__ __launch_bounds__(256) void pack_cherry_kernel(const __half *__restrict__ w,
                                                          const int16_t *__restrict__ idx,
                                                          __half *__restrict__ cherry_weight, int K, int N, int C) {
    const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
    if (e >= (long long)C * N) return;
    const int c = (int)(e / N), n = (int)(e % N);
    cherry_weight[e] = w[(size_t)n * K + idx[c]];
}

hipError_t launch_pack(int bits, const __half *w, const int16_t *idx, uint8_t *qweight, __half *scales,
                       __half *cherry_weight, int K, int N, int C, int G, hipStream_t stream) {
    const int Kn = K - C;
    if (Kn > 0) {
        const long long items = (long long)ceil_div(Kn, G) * N;
        hipLaunchKernelGGL(pack_scales_kernel, dim3((unsigned)((items + 3) / 4)), dim3(256), 0, stream, w, idx, scales,
                           K, N, C, G, bits);
        const dim3 grid(ceil_div(Kn, 128), ceil_div(N, 64));
        if (bits == 4)
            hipLaunchKernelGGL(pack_codes_kernel<4>, grid, dim3(256), 0, stream, w, idx, scales, qweight, K, N, C, G);
        else
            hipLaunchKernelGGL(pack_codes_kernel<3>, grid, dim3(256), 0, stream, w, idx, scales, qweight, K, N, C, G);
    }
    if (C > 0)
        hipLaunchKernelGGL(pack_cherry_kernel, dim3((unsigned)(((long long)C * N + 255) / 256)), dim3(256), 0, stream,
                           w, idx, cherry_weight, K, N, C);
    return hipGetLastError();
}

}  // namespace cq
