// Generic fused dequant + matmul kernel: any batch (in chunks of kMaxB rows), 3/4 bit, group
// sizes that are multiples of 32, fp16 or fp32 I/O.  One wavefront per workgroup; lanes run
// across 256 output columns (one dword = 4 columns of a byte row per lane), the K dimension
// is walked in units of 128 compacted positions and split across workgroups.  This is the
// reference-shaped path for everything the specialised kernels (cq_matvec.hip) do not take.
//
// Arithmetic contract: csrc/quant_cuda_kernel.cu:718-835 (4-bit), 558-672 / 316-438 (3-bit,
// group multiple of 128 / group 64), 441-556 / 191-314 (fp32 I/O), with fp32 accumulation
// kept until a single final rounding instead of one fp16 atomic per 128 positions (:833).
#include "cq_device.h"
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
    const IO *__restrict__ scales, IO *__restrict__ mul, unsigned long long *__restrict__ acc_words,
    float *__restrict__ side, int B, int K, int N, int C, int G, int accumulate, Plan plan) {
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
    splitk_finish<IO, kMaxB, 4>(acc, B, N, n0, active, plan.splits, acc_words, mul, accumulate, side);
}

template <int BITS, typename IO, typename IDX>
hipError_t launch_generic(const IO *vec, const uint8_t *qweight, const IO *cherry_weight,
                          const IDX *cherry_indices, const IO *scales, IO *mul, int B, int K, int N,
                          int C, int G, int accumulate, void *workspace, hipStream_t stream) {
    int upw = 4;
    while (make_plan(K, N, C, upw).splits > kMaxSplits) upw <<= 1;
    Plan plan = make_plan(K, N, C, upw);
    unsigned long long *acc_words = reinterpret_cast<unsigned long long *>(workspace);
    float *side = sizeof(IO) == 4 ? splitk_side(workspace, B, N) : nullptr;  // fp32 tensors only
    for (int b0 = 0; b0 < B; b0 += kMaxB) {
        int nb = min(kMaxB, B - b0);
        hipLaunchKernelGGL((generic_kernel<BITS, IO, IDX>), dim3(plan.tiles * plan.splits), dim3(64), 0,
                           stream, vec + (size_t)b0 * K, qweight, cherry_weight, cherry_indices, scales,
                           mul + (size_t)b0 * N, acc_words, side, nb, K, N, C, G, accumulate, plan);
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

// Dense (N, K) fp16 weight, bit for bit what QuantLinear.unpack() computes on the host,
// llama/qlinear.py:120-162.  A workgroup owns 128 consecutive columns of the DENSE weight and 64
// of its rows: it decodes the (at most 17) packed 8-position units whose normal columns fall
// into that range into LDS, stages the cherry rows of the range next to them, and writes every
// dense row as 16-byte stores, 256 bytes contiguous per row.  Column d of the dense weight is
// cherry c when idx[c] == d, else normal position d - #{idx < d}.
constexpr int kUnpackCols = 128;
constexpr int kUnpackRows = 64;
constexpr int kUnpackUnits = kUnpackCols / 8 + 1;

template <typename IDX>
__device__ inline int cherries_below(const IDX *__restrict__ idx, int C, int d) {
    int lo = 0, hi = C;
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if ((int)idx[mid] < d) lo = mid + 1; else hi = mid;
    }
    return lo;
}

constexpr int kUnpackMaxBlocks = 4;  // row blocks of kUnpackRows a workgroup may walk

template <int BITS>
__global__ __launch_bounds__(256) void unpack_kernel(const uint8_t *__restrict__ qweight,
                                                     const __half *__restrict__ cherry_weight,
                                                     const int16_t *__restrict__ cherry_indices,
                                                     const __half *__restrict__ scales,
                                                     __half *__restrict__ dense, int K, int N, int C, int G,
                                                     int blocks) {
    __shared__ unsigned short s_norm[kUnpackRows][kUnpackUnits * 8 + 2];
    __shared__ unsigned short s_ch[kUnpackCols][kUnpackRows];
    __shared__ short s_src[kUnpackCols];
    // the index list is searched several times per thread: from LDS when it fits (a search in global
    // memory is a chain of dependent loads in front of everything else the workgroup does)
    constexpr int kIdxCap = 2048;
    __shared__ int16_t s_idx[kIdxCap];
    const int Kn = K - C;
    const int d0 = blockIdx.x * kUnpackCols, d1 = min(d0 + kUnpackCols, K);
    const int t = threadIdx.x;
    const int16_t *idx = cherry_indices;
    if (C <= kIdxCap) {
        for (int i = t; i < C; i += 256) s_idx[i] = cherry_indices[i];
        __syncthreads();
        idx = s_idx;
    }
    const int c_lo = cherries_below(idx, C, d0), c_hi = cherries_below(idx, C, d1);
    const int k_lo = d0 - c_lo, k_hi = d1 - c_hi;  // normal positions of this column range
    const int ku0 = k_lo & ~7;
    const int units = k_hi > k_lo ? ceil_div(k_hi - ku0, 8) : 0;
    if (t < kUnpackCols) {
        const int d = d0 + t;
        short src = 0;
        if (d < d1) {
            const int c = cherries_below(idx, C, d);
            src = (c < C && (int)idx[c] == d) ? (short)(-1 - (c - c_lo)) : (short)(d - c - ku0);
        }
        s_src[t] = src;
    }
    __syncthreads();
    // a thread writes the same 8-column segment of every row it handles: its sources are read once
    static_assert(256 % (kUnpackCols / 8) == 0, "a thread keeps its segment across rows");
    const int seg = t & 15;
    const int dseg = d0 + 8 * seg;
    int src[8];
#pragma unroll
    for (int j = 0; j < 8; j++) src[j] = s_src[8 * seg + j];

    // The column range's geometry is found once; the workgroup then walks `blocks` blocks of
    // kUnpackRows rows, with the packed codes of the next block requested before the current one
    // is written out.  units * 16 items of (8 positions x 4 rows) per block: with the usual 17
    // units that is 272 for 256 threads, so a thread may own two.
    constexpr int kItems = (kUnpackUnits * 16 + 255) / 256;
    uint32_t w[kItems][BITS];
    uint2 sraw[kItems];
    bool live[kItems];
    auto request = [&](int n0) {
#pragma unroll
        for (int it = 0; it < kItems; it++) {
            const int e = t + 256 * it;
            const int u = e >> 4, quad = e & 15;
            const int k0 = ku0 + 8 * u, nq = n0 + 4 * quad;
            live[it] = e < units * 16 && k0 < Kn && nq < N;
            if (live[it]) {
#pragma unroll
                for (int r = 0; r < BITS; r++)
                    w[it][r] = *reinterpret_cast<const uint32_t *>(qweight + (size_t)(k0 / 8 * BITS + r) * N + nq);
                sraw[it] = *reinterpret_cast<const uint2 *>(scales + (size_t)(k0 / G) * N + nq);
            }
        }
    };
    const int nb0 = blockIdx.y * blocks * kUnpackRows;
    request(nb0);
    for (int b = 0; b < blocks; b++) {
        const int n0 = nb0 + b * kUnpackRows;
        if (n0 >= N) break;  // uniform
        for (int e = t; e < (c_hi - c_lo) * kUnpackRows; e += 256) {
            const int c = e / kUnpackRows, nl = e % kUnpackRows;
            s_ch[c][nl] = n0 + nl < N ? __half_as_ushort(cherry_weight[(size_t)(c_lo + c) * N + n0 + nl]) : 0;
        }
#pragma unroll
        for (int it = 0; it < kItems; it++) {
            if (!live[it]) continue;
            const int e = t + 256 * it;
            const int u = e >> 4, quad = e & 15;
            const uint32_t sbits[4] = {sraw[it].x & 0xffffu, sraw[it].x >> 16, sraw[it].y & 0xffffu, sraw[it].y >> 16};
#pragma unroll
            for (int c = 0; c < 4; c++) {
                float v[8];
                decode8<BITS>(w[it], c, v);
                // (code - c_b) has 4 significant bits and the fp16 scale 11: the float product is
                // exact, so this is the single rounding the reference performs
                const float sc = __half2float(__ushort_as_half((unsigned short)sbits[c]));
#pragma unroll
                for (int i = 0; i < 8; i++)
                    s_norm[4 * quad + c][8 * u + i] = __half_as_ushort(__float2half_rn(v[i] * sc));
            }
        }
        __syncthreads();
        if (b + 1 < blocks && n0 + kUnpackRows < N) request(n0 + kUnpackRows);
        if (dseg < d1) {
#pragma unroll
            for (int i = 0; i < kUnpackRows * (kUnpackCols / 8) / 256; i++) {
                const int nl = (t >> 4) + 16 * i;
                if (n0 + nl >= N) continue;
                unsigned short h[8];
#pragma unroll
                for (int j = 0; j < 8; j++) h[j] = src[j] >= 0 ? s_norm[nl][src[j]] : s_ch[-1 - src[j]][nl];
                uint4 out;
                out.x = h[0] | (uint32_t)h[1] << 16;
                out.y = h[2] | (uint32_t)h[3] << 16;
                out.z = h[4] | (uint32_t)h[5] << 16;
                out.w = h[6] | (uint32_t)h[7] << 16;
                *reinterpret_cast<uint4 *>(dense + (size_t)(n0 + nl) * K + dseg) = out;
            }
        }
        __syncthreads();  // the next block's decode overwrites s_norm / s_ch
    }
}

hipError_t launch_unpack(int bits, const uint8_t *qweight, const __half *cherry_weight,
                         const int16_t *cherry_indices, const __half *scales, __half *dense, int K, int N,
                         int C, int G, hipStream_t stream) {
    if (K <= 0 || N <= 0) return hipSuccess;
    // more row blocks per workgroup hide the load latency better, as long as the launch still
    // gives every CU several workgroups
    auto workgroups = [&](int b) { return (long)ceil_div(K, kUnpackCols) * ceil_div(N, kUnpackRows * b); };
    const int blocks = workgroups(kUnpackMaxBlocks) >= 4096 ? kUnpackMaxBlocks : workgroups(2) >= 512 ? 2 : 1;
    dim3 grid(ceil_div(K, kUnpackCols), ceil_div(N, kUnpackRows * blocks));
    if (bits == 4)
        hipLaunchKernelGGL(unpack_kernel<4>, grid, dim3(256), 0, stream, qweight, cherry_weight, cherry_indices,
                           scales, dense, K, N, C, G, blocks);
    else
        hipLaunchKernelGGL(unpack_kernel<3>, grid, dim3(256), 0, stream, qweight, cherry_weight, cherry_indices,
                           scales, dense, K, N, C, G, blocks);
    return hipGetLastError();
}

}  // namespace cq
