// 3-bit fused dequant + matmul on fp32 tensors (fp32 activations, scales, cherry rows and
// outputs, int32 channel indices): the variant behind vecquant3matmul_cherryq(..., fp16=False),
// the call the reference's benchmark_speed.py:20-45 times (batch 16, 4096 -> 13824).
//
// The weight stream is tiled as in the fp16 kernels (cq_matvec.hip / cq_batch.hip): a wavefront
// owns units of 128 compacted positions x 256 columns, four lane groups split the positions, a
// lane owns 16 adjacent columns and loads dwordx4.  The arithmetic stays in fp32 and runs on the
// matrix cores as v_mfma_f32_16x16x4_f32:
//
//   D[batch row][column] += sum over 4 positions  A[batch row][position] * B[position][column]
//
//   B (weights)  from registers: for one of the lane's 16 columns, two v_perm_b32 collect the
//                column's three bytes of an 8-position unit, v_bfe_u32 + v_cvt_f32_u32 + one
//                subtraction give the eight values code - 3.5 exactly (as the reference forms
//                them, csrc/quant_cuda_kernel.cu:280-305); each is the B operand of one MFMA
//                whose four K slots are the four lane groups' positions.
//   A (activations) prepared once per call by a small kernel in the per-lane operand order
//                (gathered around the cherry channels, zero padded to 16 rows).
//   Per unit the fp32 tile is multiplied by the group's scale and added to the totals, which is
//   where the reference applies the scale too (:312).
//
// Cherry rows are further units whose B operands are the fp32 rows themselves.  Across the
// workgroup's wavefronts the totals meet in LDS, across workgroups in one 64-bit fixed-point
// atomic per output element (cq_device.h).  Up to 16 rows per pass; more rows are further
// passes over the weights.
//
// Arithmetic contract: csrc/quant_cuda_kernel.cu:191-314 (group 64) and 441-556 (group 128):
// fp32 products and sums; the summation order differs (the reference adds 64 or 128 products in
// sequence per thread and combines blocks with fp32 atomics in arrival order).
#include "cq_device.h"
#include "cq_kernels.h"

namespace cq {

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kF32Rows = 16;   // MFMA M dimension; smaller batches are zero padded
constexpr int kF32Waves = 4;   // wavefronts per workgroup
constexpr uint32_t kRsrcFlagsF = 0x00020000u;
constexpr uint32_t kOobF = 0x80000000u;

size_t f32_scratch_bytes(int K, int C) {
    const Plan p = make_plan(K, 8, C, 1, kUnitK);
    return ((size_t)p.units_total * 8 * 64 * sizeof(float4) + 255) / 256 * 256;
}

// ---- activation preparation ------------------------------------------------------------------
// xa[(u * 8 + f) * 64 + lane], lane = (q, i): normal unit u, f = 2 t + h holds
// x[row i][positions 128 u + 32 q + 8 t + 4 h + 0..3]; cherry unit: f = 0, 1 hold
// x[row i][idx[c0 + 8 q + 0..7]].  Rows >= B and positions past the end read as 0.
__global__ __launch_bounds__(256) void f32_prep_kernel(const float *__restrict__ x,
                                                       const int32_t *__restrict__ cherry_indices,
                                                       float4 *__restrict__ xa, int B, int K, int C,
                                                       int units_normal) {
    const int u = blockIdx.x, t = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int q = lane >> 4, i = lane & 15;
    const int Kn = K - C;
    float v[8];
    if (u >= units_normal) {
        if (t != 0) return;
        const int c0 = (u - units_normal) * kCherryUnit + 8 * q;
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = (c0 + j < C && i < B) ? x[(size_t)i * K + cherry_indices[c0 + j]] : 0.f;
    } else {
        const int k0 = u * kUnitK + 32 * q + 8 * t;
        int low = gather_offset(cherry_indices, C, k0);
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int k = k0 + j;
            while (low < C && cherry_indices[low] - low <= k) low++;
            v[j] = (k < Kn && i < B) ? x[(size_t)i * K + k + low] : 0.f;
        }
    }
    xa[((size_t)u * 8 + 2 * t) * 64 + lane] = make_float4(v[0], v[1], v[2], v[3]);
    xa[((size_t)u * 8 + 2 * t + 1) * 64 + lane] = make_float4(v[4], v[5], v[6], v[7]);
}

// ---- main kernel -------------------------------------------------------------------------------
__global__ __launch_bounds__(64 * kF32Waves) __attribute__((amdgpu_waves_per_eu(2, 2))) void f32_kernel(
    const uint8_t *__restrict__ qweight, const float *__restrict__ cherry_weight, const float *__restrict__ scales,
    float *__restrict__ mul, const float4 *__restrict__ xa, unsigned long long *__restrict__ acc_words,
    float *__restrict__ side, int B, int K, int N, int C, int G, int accumulate, Plan plan, int units_per_wave) {
    __shared__ float s_red[kF32Waves][kF32Rows][kTileCols];  // 64 KB

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kq = lane >> 4, nl = lane & 15;
    const int tile = blockIdx.x % plan.tiles;
    const int split = blockIdx.x / plan.tiles;
    const int Kn = K - C;
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc((void *)qweight, 0, Kn / 8 * 3 * N, kRsrcFlagsF);
    const __amdgpu_buffer_rsrc_t rs =
        __builtin_amdgcn_make_buffer_rsrc((void *)scales, 0, ceil_div(Kn, G) * N * 4, kRsrcFlagsF);
    const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc((void *)cherry_weight, 0, C * N * 4, kRsrcFlagsF);
    const int n0 = tile * kTileCols + nl * 16;
    const bool col_ok = n0 < N;

    // tot[c][r]: column n0 + c, batch row 4 * kq + r
    float4_t tot[16];
#pragma unroll
    for (int c = 0; c < 16; c++) tot[c] = (float4_t){0.f, 0.f, 0.f, 0.f};

    const int u0 = split * plan.units_per_wg + wave;
    for (int it = 0; it < units_per_wave; it++) {
        const int u = u0 + it * kF32Waves;
        if (u >= plan.units_total) break;
        const float4 *xau = xa + (size_t)u * 8 * 64 + lane;
        if (u < plan.units_normal) {
            // 12 byte rows x 16 columns, the group's 16 scales, 32 activations
            u32x4 w[12];
            const uint32_t woff = col_ok ? (uint32_t)((u * 48 + kq * 12) * N + n0) : kOobF;
#pragma unroll
            for (int i = 0; i < 12; i++) w[i] = __builtin_amdgcn_raw_buffer_load_b128(rw, woff + (uint32_t)(i * N), 0, 2);
            const int g = (u * kUnitK) / G;
            const uint32_t soff = col_ok ? (uint32_t)(g * N + n0) * 4u : kOobF;
            u32x4 sc[4];
#pragma unroll
            for (int i = 0; i < 4; i++) sc[i] = __builtin_amdgcn_raw_buffer_load_b128(rs, soff + 16u * i, 0, 0);
            float4 a[8];
#pragma unroll
            for (int f = 0; f < 8; f++) a[f] = xau[f * 64];

            float4_t d[16];
#pragma unroll
            for (int c = 0; c < 16; c++) d[c] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const float av[8] = {a[2 * t].x, a[2 * t].y, a[2 * t].z, a[2 * t].w,
                                     a[2 * t + 1].x, a[2 * t + 1].y, a[2 * t + 1].z, a[2 * t + 1].w};
                // bytes (row 3t, row 3t+1, row 3t+2) of column c -> one 24-bit unit of 8 codes
                uint32_t unit[16];
#pragma unroll
                for (int c = 0; c < 16; c++) {
                    const int dw = c >> 2, cb = c & 3;
                    const uint32_t p01 = __builtin_amdgcn_perm(w[3 * t + 1][dw], w[3 * t][dw],
                                                               0x0c0c0000u | (uint32_t)((4 + cb) << 8) | (uint32_t)cb);
                    unit[c] = __builtin_amdgcn_perm(w[3 * t + 2][dw], p01, 0x0c000100u | (uint32_t)((4 + cb) << 16));
                }
                // consecutive MFMAs go to different accumulators
#pragma unroll
                for (int j = 0; j < 8; j++)
#pragma unroll
                    for (int c = 0; c < 16; c++) {
                        const float wv = (float)((unit[c] >> (3 * j)) & 7u) - 3.5f;
                        d[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[j], wv, d[c], 0, 0, 0);
                    }
            }
#pragma unroll
            for (int c = 0; c < 16; c++) {
                const float s = __uint_as_float(sc[c >> 2][c & 3]);
#pragma unroll
                for (int r = 0; r < 4; r++) tot[c][r] += s * d[c][r];
            }
        } else {
            // 32 cherry rows, 8 per lane group; B operands are the fp32 rows themselves
            const int c0 = (u - plan.units_normal) * kCherryUnit + 8 * kq;
            const float4 a0 = xau[0], a1 = xau[64];
            const float av[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
#pragma unroll
            for (int j = 0; j < 8; j++) {
                // rows past C read as 0 through the buffer bounds; their activations are 0 as well
                const uint32_t coff = col_ok ? (uint32_t)((c0 + j) * N + n0) * 4u : kOobF;
                u32x4 cw[4];
#pragma unroll
                for (int i = 0; i < 4; i++) cw[i] = __builtin_amdgcn_raw_buffer_load_b128(rc, coff + 16u * i, 0, 2);
#pragma unroll
                for (int c = 0; c < 16; c++)
                    tot[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[j], __uint_as_float(cw[c >> 2][c & 3]), tot[c], 0,
                                                                  0, 0);
            }
        }
    }

    // ---- across the workgroup's wavefronts through LDS.  Column 16 nl + c is stored at
    // 16 nl + ((c + nl) & 15): for a fixed c the 16 lanes of a row then hit 16 different banks.
#pragma unroll
    for (int c = 0; c < 16; c++)
#pragma unroll
        for (int r = 0; r < 4; r++) s_red[wave][4 * kq + r][16 * nl + ((c + nl) & 15)] = tot[c][r];
    __syncthreads();
    float vals[kF32Rows][1];
    {
        const int sw = (tid & ~15) | (((tid & 15) + (tid >> 4)) & 15);  // where column `tid` was stored
#pragma unroll
        for (int b = 0; b < kF32Rows; b++)
            vals[b][0] = (s_red[0][b][sw] + s_red[1][b][sw]) + (s_red[2][b][sw] + s_red[3][b][sw]);
    }
    const int n = tile * kTileCols + tid;
    splitk_finish<float, kF32Rows, 1>(vals, B, N, n, n < N, plan.splits, acc_words, mul, accumulate, side);
}

bool f32_supported(int B, int K, int N, int C, int G) {
    if (B < 1) return false;
    if (G % kUnitK) return false;  // a unit must not straddle a group
    if (K - C <= 0) return false;
    const long long wbytes = (long long)(K - C) / 8 * 3 * N;
    const long long cbytes = (long long)C * N * 4;
    const long long sbytes = (long long)ceil_div(K - C, G) * N * 4;
    if (wbytes >= 0x7fff0000ll || cbytes >= 0x7fff0000ll || sbytes >= 0x7fff0000ll) return false;
    return true;
}

hipError_t launch_f32(const float *vec, const uint8_t *qweight, const float *cherry_weight,
                      const int32_t *cherry_indices, const float *scales, float *mul, int B, int K, int N, int C,
                      int G, int accumulate, void *workspace, void *scratch, hipStream_t stream) {
    const Plan unit_plan = make_plan(K, N, C, 1, kUnitK);
    // as few units per wave as keep the grid within one resident round (two workgroups per CU)
    // and the split count within the counter field of the accumulator words
    int upv = 1;
    while (upv < 64 && (unit_plan.tiles * ceil_div(unit_plan.units_total, kF32Waves * upv) > 512 ||
                        ceil_div(unit_plan.units_total, kF32Waves * upv) > kMaxSplits))
        upv++;
    const Plan plan = make_plan(K, N, C, kF32Waves * upv, kUnitK);
    float4 *xa = reinterpret_cast<float4 *>(scratch);
    for (int b0 = 0; b0 < B; b0 += kF32Rows) {
        const int nb = min(kF32Rows, B - b0);
        hipLaunchKernelGGL(f32_prep_kernel, dim3(plan.units_total), dim3(256), 0, stream, vec + (size_t)b0 * K,
                           cherry_indices, xa, nb, K, C, plan.units_normal);
        hipLaunchKernelGGL(f32_kernel, dim3(plan.tiles * plan.splits), dim3(64 * kF32Waves), 0, stream, qweight,
                           cherry_weight, scales, mul + (size_t)b0 * N, xa, reinterpret_cast<unsigned long long *>(workspace),
                           splitk_side(workspace, B, N), nb, K, N, C, G, accumulate, plan, upv);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

}  // namespace cq
