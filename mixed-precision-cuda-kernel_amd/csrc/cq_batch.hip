// Small-batch fused dequant + matmul (2 <= batch <= 16 rows per pass) on the gfx950 matrix cores.
//
// The weight stream is tiled exactly as in the batch-1 kernel (cq_matvec.hip): a wavefront owns
// units of 128 compacted positions x 256 columns, four lane groups split the positions, a lane
// owns 16 adjacent columns and loads dwordx4.  The arithmetic goes to v_mfma_f32_16x16x32_f16:
//
//   D[batch row][column] += sum over 32 positions  A[batch row][position] * B[position][column]
//
//   B (weights)  comes straight from registers.  For one of the lane's 16 columns, two
//                v_perm_b32 interleave that column's bytes of consecutive byte rows and masks cut
//                out code pairs; a masked field at bit p of a 16-bit half IS the fp16 subnormal
//                code * 2^(p-24), which the matrix core multiplies exactly.  Four such dwords are
//                the 8 positions a lane group contributes to one MFMA.  No int->float conversion,
//                no LDS staging of dequantised tiles.
//   A (activations) is prepared once per call by a small kernel in exactly the per-lane operand
//                order: gathered around the cherry channels, zero padded to 16 rows, scaled by
//                2^(sh - p) so that every field position p is compensated exactly (sh normalises
//                each row of each unit to the top of the fp16 range), together with the row sums
//                needed for the grid offset  -c_b * sum(x).
//   The MFMA's K dimension runs across the four lane groups, so the K reduction inside a unit
//   costs nothing; per unit the fp32 tile is scaled by the group scale and added to the totals.
//
// Cherry rows (dense fp16) run through the same MFMA with operands packed by v_perm_b32.
// Across workgroups the K splits meet, for calls with few outputs, in one 64-bit fixed-point atomic
// per output element (cq_device.h), and for larger ones in per-split partial tiles plus one
// ticket per column tile (agent-scope sc1 stores / loads, no cache-wide fences; the last
// workgroup adds the partials in split order).  Both are independent of arrival order.
//
// Arithmetic contract: csrc/quant_cuda_kernel.cu:797-834 (the reference loops its batch-1 body
// over the batch rows, re-reading the weights for every row); fp32 accumulation, one rounding.
#include "cq_device.h"
#include "cq_kernels.h"

namespace cq {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kBatchRows = 16;        // MFMA M dimension; smaller batches are zero padded
constexpr int kBatchWaves = 4;        // wavefronts per workgroup
constexpr int kBatchAtomicOutputs = 8 * 14336;  // calls with at most this many outputs use the atomic split-K epilogue
constexpr int kBatchMaxSplits = 8;    // bounds the partial-tile scratch and the last workgroup's reads
constexpr uint32_t kRsrcFlagsB = 0x00020000u;
constexpr uint32_t kOobB = 0x80000000u;

// position order inside one 8-position MFMA slice of a lane group, and the bit position p of
// each code's field inside its 16-bit half (value seen by the matrix core = code * 2^(p-24))
//   4-bit: ord = {0, 2, 1, 3, 4, 6, 5, 7}   p = {0, 0, 4, 4, 0, 0, 4, 4}
//   3-bit: ord = {0, 3, 1, 4, 5, 6, 2, 7}   p = {0, 1, 3, 4, 7, 2, 6, 5}
template <int BITS>
__host__ __device__ constexpr int slice_ord(int kk) {
    return BITS == 4 ? ((kk & 4) | ((kk & 1) << 1) | ((kk >> 1) & 1)) : (int)((0x72654130u >> (4 * kk)) & 7u);
}
template <int BITS>
__host__ __device__ constexpr int slice_pos(int kk) {
    return BITS == 4 ? ((kk & 2) ? 4 : 0) : (int)((0x56274310u >> (4 * kk)) & 7u);
}
static_assert(slice_ord<4>(1) == 2 && slice_ord<4>(2) == 1 && slice_ord<4>(6) == 5 && slice_pos<4>(3) == 4, "");
static_assert(slice_ord<3>(1) == 3 && slice_ord<3>(6) == 2 && slice_pos<3>(4) == 7 && slice_pos<3>(7) == 5, "");

BatchWorkspace batch_workspace(int K, int N, int C) {
    BatchWorkspace w;
    const Plan p = make_plan(K, N, C, 1, kUnitK);
    // zero-kept workspace: the accumulator words of the other kernels, then the tickets
    w.tickets = ((size_t)kBatchRows * (size_t)N * sizeof(unsigned long long) + 255) / 256 * 256;
    w.workspace_total = w.tickets + ((size_t)p.tiles * sizeof(unsigned) + 255) / 256 * 256;
    // uninitialised scratch
    size_t off = 0;
    w.partial = off;
    off += (size_t)kBatchMaxSplits * kBatchRows * (size_t)N * sizeof(float);
    off = (off + 255) / 256 * 256;
    w.xa = off;
    off += (size_t)p.units_total * 4096;
    w.rowsum = off;
    off += (size_t)p.units_total * kBatchRows * sizeof(float);
    w.rowshift = off;
    off += (size_t)p.units_total * kBatchRows * sizeof(int);
    w.scratch_total = (off + 255) / 256 * 256;
    return w;
}

// ---- activation preparation ------------------------------------------------------------------
// One workgroup per unit.  Normal unit u: thread (step s, lane (q, i)) produces the 8 fp16 values
// lane (q, i) feeds to the MFMA of step s: x[row i][positions 128u + 32q + 8s + ord[0..7]], gathered
// around the cherry channels, times 2^(sh - p).  Cherry unit: one step, raw x[row i][idx[c]].
template <int BITS>
__global__ __launch_bounds__(256) void batch_prep_kernel(const __half *__restrict__ x,
                                                         const int16_t *__restrict__ cherry_indices,
                                                         uint4 *__restrict__ xa, float *__restrict__ rowsum,
                                                         int *__restrict__ rowshift, int B, int K, int C,
                                                         int units_normal) {
    __shared__ unsigned s_max[kBatchRows];
    __shared__ float s_part[kBatchRows][16];
    const int u = blockIdx.x, t = threadIdx.x;
    const int s = t >> 6, lane = t & 63, q = lane >> 4, i = lane & 15;
    const int Kn = K - C;
    if (u >= units_normal) {
        if (t < 64) {
            const int c0 = (u - units_normal) * kCherryUnit + 8 * q;
            unsigned short h[8];
#pragma unroll
            for (int kk = 0; kk < 8; kk++) {
                const int c = c0 + kk;
                h[kk] = (c < C && i < B) ? __half_as_ushort(x[(size_t)i * K + (int)cherry_indices[c]]) : 0;
            }
            xa[(size_t)u * 256 + lane] = make_uint4(h[0] | h[1] << 16, h[2] | h[3] << 16, h[4] | h[5] << 16,
                                                    h[6] | h[7] << 16);
        }
        return;
    }
    // t[m] = idx[m] - m is non-decreasing; position k sits after every cherry m with t[m] <= k.
    // Stage t in LDS (one pass over the indices) and walk this thread's 8 consecutive positions.
    constexpr int kCap = 2048;
    __shared__ int s_t[kCap];
    if (t < kBatchRows) s_max[t] = 0;
    const bool staged = C <= kCap;
    if (staged)
        for (int mm = t; mm < C; mm += 256) s_t[mm] = (int)cherry_indices[mm] - mm;
    __syncthreads();
    const int kb = u * kUnitK + 32 * q + 8 * s;
    int lows[8];
    if (staged) {
        int lo = 0, hi = C;
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            const bool le = s_t[mid] <= kb;
            lo = le ? mid + 1 : lo;
            hi = le ? hi : mid;
        }
        lows[0] = lo;
#pragma unroll
        for (int j = 1; j < 8; j++) {
            while (lo < C && s_t[lo] <= kb + j) lo++;
            lows[j] = lo;
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++) lows[j] = gather_offset(cherry_indices, C, kb + j);
    }
    float v[8];
    unsigned m = 0;
    float sum = 0.f;
#pragma unroll
    for (int kk = 0; kk < 8; kk++) {
        const int j = slice_ord<BITS>(kk);
        const int k = kb + j;
        unsigned short hb = 0;
        if (k < Kn && i < B) hb = __half_as_ushort(x[(size_t)i * K + k + lows[j]]);
        v[kk] = __half2float(__ushort_as_half(hb));
        m = max(m, (unsigned)(hb & 0x7fffu));
        sum += v[kk];
    }
    atomicMax(&s_max[i], m);
    s_part[i][s * 4 + q] = sum;
    __syncthreads();
    const int sh = 29 - (int)(s_max[i] >> 10);
    unsigned short h[8];
#pragma unroll
    for (int kk = 0; kk < 8; kk++)
        h[kk] = __half_as_ushort(__float2half_rn(ldexpf(v[kk], sh - slice_pos<BITS>(kk))));
    xa[(size_t)u * 256 + t] = make_uint4(h[0] | h[1] << 16, h[2] | h[3] << 16, h[4] | h[5] << 16, h[6] | h[7] << 16);
    if (t < kBatchRows) {
        float tot = 0.f;
#pragma unroll
        for (int p = 0; p < 16; p++) tot += s_part[t][p];  // fixed order
        rowsum[u * kBatchRows + t] = tot;
        rowshift[u * kBatchRows + t] = 29 - (int)(s_max[t] >> 10);
    }
}

// ---- main kernel -------------------------------------------------------------------------------
// Everything one unit needs from memory.
struct UnitRegs {
    u32x4 w[16];    // 16 (12) byte rows x 16 columns
    u32x4 sc0, sc1; // 16 group scales (fp16)
    uint4 a[4];     // prepared activations, one MFMA A operand per step
    float4 rsum;    // row sums of the activations for the lane's 4 batch rows
    int4 rsh;       // their normalisation shifts
};

struct BatchCtx {
    __amdgpu_buffer_rsrc_t rw, rs, rc;
    const uint4 *xa;
    const float *rowsum;
    const int *rowshift;
    int N, G, units_normal, lane, kq, n0;
    bool col_ok;
};

template <int BITS>
__device__ __forceinline__ void issue_unit(UnitRegs &r, const BatchCtx &cx, int u) {
    constexpr int R = BITS == 4 ? 16 : 12;
    const uint4 *xau = cx.xa + (size_t)u * 256 + cx.lane;
    const uint32_t woff = cx.col_ok ? (uint32_t)((u * 4 * R + cx.kq * R) * cx.N + cx.n0) : kOobB;
#pragma unroll
    for (int i = 0; i < R; i++)
        r.w[i] = __builtin_amdgcn_raw_buffer_load_b128(cx.rw, woff + (uint32_t)(i * cx.N), 0, 2);
    const int g = (u * kUnitK) / cx.G;
    const uint32_t soff = cx.col_ok ? (uint32_t)(g * cx.N + cx.n0) * 2u : kOobB;
    r.sc0 = __builtin_amdgcn_raw_buffer_load_b128(cx.rs, soff, 0, 0);
    r.sc1 = __builtin_amdgcn_raw_buffer_load_b128(cx.rs, soff + 16, 0, 0);
#pragma unroll
    for (int s = 0; s < 4; s++) r.a[s] = xau[s * 64];
    r.rsum = *reinterpret_cast<const float4 *>(cx.rowsum + u * kBatchRows + 4 * cx.kq);
    r.rsh = *reinterpret_cast<const int4 *>(cx.rowshift + u * kBatchRows + 4 * cx.kq);
}

// tot[c][r]: column n0 + c, batch row 4 * kq + r
template <int BITS>
__device__ __forceinline__ void compute_unit(const UnitRegs &r, float4_t (&tot)[16]) {
    constexpr float kGrid = BITS == 4 ? 7.5f : 3.5f;
    float4_t d[16];
#pragma unroll
    for (int c = 0; c < 16; c++) d[c] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; s++) {
        const half8_t av = __builtin_bit_cast(half8_t, r.a[s]);
#pragma unroll
        for (int dw = 0; dw < 4; dw++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                u32x4 b;
                if (BITS == 4) {
                    const uint32_t sel = 0x0c000c00u | (uint32_t)(j << 16) | (uint32_t)(4 + j);
                    const uint32_t p0 = __builtin_amdgcn_perm(r.w[4 * s][dw], r.w[4 * s + 1][dw], sel);
                    const uint32_t p1 = __builtin_amdgcn_perm(r.w[4 * s + 2][dw], r.w[4 * s + 3][dw], sel);
                    b = (u32x4){p0 & 0x000f000fu, p0 & 0x00f000f0u, p1 & 0x000f000fu, p1 & 0x00f000f0u};
                } else {
                    const uint32_t sel = 0x0c000000u | (uint32_t)(j << 16) | (uint32_t)(j << 8) | (uint32_t)(4 + j);
                    const uint32_t p1 = __builtin_amdgcn_perm(r.w[3 * s][dw], r.w[3 * s + 1][dw], sel);
                    const uint32_t p2 = __builtin_amdgcn_perm(r.w[3 * s + 1][dw], r.w[3 * s + 2][dw], sel);
                    b = (u32x4){p1 & 0x000e0007u, p1 & 0x00700038u, p2 & 0x001c0380u,
                                (p1 & 0x000001c0u) | (p2 & 0x00e00000u)};
                }
                d[4 * dw + j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, __builtin_bit_cast(half8_t, b),
                                                                      d[4 * dw + j], 0, 0, 0);
            }
        }
    }
    // tile -> totals: undo the normalisation, apply the grid offset and the group scale
    const float f[4] = {ldexpf(1.f, 24 - r.rsh.x), ldexpf(1.f, 24 - r.rsh.y), ldexpf(1.f, 24 - r.rsh.z),
                        ldexpf(1.f, 24 - r.rsh.w)};
    const float o[4] = {-kGrid * r.rsum.x, -kGrid * r.rsum.y, -kGrid * r.rsum.z, -kGrid * r.rsum.w};
#pragma unroll
    for (int c = 0; c < 16; c++) {
        const uint32_t sw = c < 8 ? r.sc0[c >> 1] : r.sc1[(c - 8) >> 1];
        const float sc = __half2float(__ushort_as_half((unsigned short)((c & 1) ? (sw >> 16) : (sw & 0xffffu))));
#pragma unroll
        for (int q = 0; q < 4; q++) tot[c][q] += sc * (d[c][q] * f[q] + o[q]);
    }
}

// cherry unit: 32 dense fp16 rows, 8 per lane group; B operands packed by v_perm_b32
__device__ __forceinline__ void cherry_unit(const BatchCtx &cx, int u, float4_t (&tot)[16]) {
    const int c0 = (u - cx.units_normal) * kCherryUnit + 8 * cx.kq;
    const uint32_t coff = cx.col_ok ? (uint32_t)(c0 * cx.N + cx.n0) * 2u : kOobB;
    u32x4 cw[8][2];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        cw[i][0] = __builtin_amdgcn_raw_buffer_load_b128(cx.rc, coff + (uint32_t)(i * cx.N * 2), 0, 2);
        cw[i][1] = __builtin_amdgcn_raw_buffer_load_b128(cx.rc, coff + (uint32_t)(i * cx.N * 2) + 16, 0, 2);
    }
    const half8_t av = __builtin_bit_cast(half8_t, cx.xa[(size_t)u * 256 + cx.lane]);
#pragma unroll
    for (int c = 0; c < 16; c++) {
        const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;  // (row r half, row r+1 half)
        u32x4 b;
#pragma unroll
        for (int rp = 0; rp < 4; rp++)
            b[rp] = __builtin_amdgcn_perm(cw[2 * rp + 1][c >> 3][(c & 7) >> 1], cw[2 * rp][c >> 3][(c & 7) >> 1], sel);
        tot[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, __builtin_bit_cast(half8_t, b), tot[c], 0, 0, 0);
    }
}

template <int BITS>
__global__ __launch_bounds__(64 * kBatchWaves) __attribute__((amdgpu_waves_per_eu(2, 2))) void batch_kernel(
    const uint8_t *__restrict__ qweight, const __half *__restrict__ cherry_weight,
    const __half *__restrict__ scales, __half *__restrict__ mul, const uint4 *__restrict__ xa,
    const float *__restrict__ rowsum, const int *__restrict__ rowshift, float *__restrict__ partial,
    unsigned *__restrict__ tickets, unsigned long long *__restrict__ acc_words, int atomic_epilogue, int B, int K,
    int N, int C, int G, int accumulate, Plan plan, int units_per_wave) {
    __shared__ float s_red[kBatchWaves][kBatchRows][kTileCols];  // 64 KB

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kq = lane >> 4, nl = lane & 15;
    const int tile = blockIdx.x % plan.tiles;
    const int split = blockIdx.x / plan.tiles;
    const int Kn = K - C;
    BatchCtx cx;
    cx.rw = __builtin_amdgcn_make_buffer_rsrc((void *)qweight, 0, Kn / 8 * BITS * N, kRsrcFlagsB);
    cx.rs = __builtin_amdgcn_make_buffer_rsrc((void *)scales, 0, ceil_div(Kn, G) * N * 2, kRsrcFlagsB);
    cx.rc = __builtin_amdgcn_make_buffer_rsrc((void *)cherry_weight, 0, C * N * 2, kRsrcFlagsB);
    cx.xa = xa;
    cx.rowsum = rowsum;
    cx.rowshift = rowshift;
    cx.N = N;
    cx.G = G;
    cx.units_normal = plan.units_normal;
    cx.lane = lane;
    cx.kq = kq;
    cx.n0 = tile * kTileCols + nl * 16;
    cx.col_ok = cx.n0 < N;

    float4_t tot[16];
#pragma unroll
    for (int c = 0; c < 16; c++) tot[c] = (float4_t){0.f, 0.f, 0.f, 0.f};

    // this wave's units: u0, u0 + 4, u0 + 8, ...  (the 4 waves interleave).  One register set per
    // wave keeps the kernel at two waves per SIMD, which overlap each other's loads and MFMAs.
    const int u0 = split * plan.units_per_wg + wave;
    for (int it = 0; it < units_per_wave; it++) {
        const int ua = u0 + it * kBatchWaves;
        if (ua < plan.units_normal) {
            UnitRegs ra;
            issue_unit<BITS>(ra, cx, ua);
            compute_unit<BITS>(ra, tot);
        }
    }
    for (int it = 0; it < units_per_wave; it++) {
        const int u = u0 + it * kBatchWaves;
        if (u >= plan.units_normal && u < plan.units_total) cherry_unit(cx, u, tot);
    }

    // ---- across the workgroup's wavefronts through LDS.  Column 16 nl + c is stored at
    // 16 nl + ((c + nl) & 15): for a fixed c the 16 lanes of a row then hit 16 different banks.
#pragma unroll
    for (int c = 0; c < 16; c++)
#pragma unroll
        for (int r = 0; r < 4; r++) s_red[wave][4 * kq + r][16 * nl + ((c + nl) & 15)] = tot[c][r];
    __syncthreads();
    float vals[kBatchRows];
    {
        const int sw = (tid & ~15) | (((tid & 15) + (tid >> 4)) & 15);  // where column `tid` was stored
#pragma unroll
        for (int b = 0; b < kBatchRows; b++)
            vals[b] = (s_red[0][b][sw] + s_red[1][b][sw]) + (s_red[2][b][sw] + s_red[3][b][sw]);
    }
    const int n = tile * kTileCols + tid;
    const bool active = n < N;

    // ---- across workgroups: per-split partial tiles + one ticket per column tile.  (One atomic
    // per output element, as in the batch-1 kernel, is slower here: 16 rows make 16x the atomics.)
    // Partials travel as agent-scope sc1 stores / loads, no cache-wide fences; see cq_device.h.
    if (atomic_epilogue) {
        // few enough outputs: one 64-bit fixed-point atomic per output element, as in the batch-1
        // kernel (order-independent, leaves the words zero), instead of partial tiles + ticket
        float v2[kBatchRows][1];
#pragma unroll
        for (int b = 0; b < kBatchRows; b++) v2[b][0] = vals[b];
        splitk_finish<__half, kBatchRows, 1>(v2, B, N, n, active, plan.splits, acc_words, mul, accumulate);
        return;
    }
    if (plan.splits > 1) {
        if (active)
#pragma unroll
            for (int b = 0; b < kBatchRows; b++)
                if (b < B)
                    __hip_atomic_store(partial + ((size_t)split * kBatchRows + b) * N + n, vals[b], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
        int *s_last = reinterpret_cast<int *>(&s_red[0][0][0]);  // the tile has been consumed
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (tid == 0) {
            unsigned old = __hip_atomic_fetch_add(&tickets[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            *s_last = (old == (unsigned)(plan.splits - 1));
        }
        __syncthreads();
        if (!*s_last) return;
        if (tid == 0) __hip_atomic_store(&tickets[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (active) {
#pragma unroll
            for (int b = 0; b < kBatchRows; b++) vals[b] = 0.f;
            // up to 3 splits (48 loads) in flight at a time, added in split order
            for (int s0 = 0; s0 < plan.splits; s0 += 3) {
                float p[3][kBatchRows];
#pragma unroll
                for (int ds = 0; ds < 3; ds++)
#pragma unroll
                    for (int b = 0; b < kBatchRows; b++)
                        p[ds][b] = (b < B && s0 + ds < plan.splits)
                                       ? __hip_atomic_load(partial + ((size_t)(s0 + ds) * kBatchRows + b) * N + n,
                                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                       : 0.f;
#pragma unroll
                for (int ds = 0; ds < 3; ds++)
#pragma unroll
                    for (int b = 0; b < kBatchRows; b++) vals[b] += p[ds][b];
            }
        }
    }
    if (active) {
#pragma unroll
        for (int b = 0; b < kBatchRows; b++)
            if (b < B) {
                __half *o = mul + (size_t)b * N + n;
                float v = vals[b];
                if (accumulate) v += __half2float(*o);
                *o = __float2half_rn(v);
            }
    }
}

bool batch_supported(int bits, int B, int K, int N, int C, int G) {
    (void)bits;
    (void)N;
    if (B < 2) return false;
    if (G % kUnitK) return false;  // a unit must not straddle a group
    if (K - C <= 0) return false;
    const long long wbytes = (long long)(K - C) / 8 * 4 * N;
    const long long cbytes = (long long)C * N * 2;
    if (wbytes >= 0x7fff0000ll || cbytes >= 0x7fff0000ll) return false;
    return true;
}

template <int BITS>
static hipError_t launch_batch_bits(const __half *vec, const uint8_t *qweight, const __half *cherry_weight,
                                    const int16_t *cherry_indices, const __half *scales, __half *mul, int B, int K,
                                    int N, int C, int G, int accumulate, void *workspace, void *scratch,
                                    hipStream_t stream) {
    const BatchWorkspace ws = batch_workspace(K, N, C);
    char *base = reinterpret_cast<char *>(scratch);
    uint4 *xa = reinterpret_cast<uint4 *>(base + ws.xa);
    float *rowsum = reinterpret_cast<float *>(base + ws.rowsum);
    int *rowshift = reinterpret_cast<int *>(base + ws.rowshift);
    float *partial = reinterpret_cast<float *>(base + ws.partial);
    unsigned *tickets = reinterpret_cast<unsigned *>(reinterpret_cast<char *>(workspace) + ws.tickets);
    const Plan unit_plan = make_plan(K, N, C, 1, kUnitK);
    for (int b0 = 0; b0 < B; b0 += kBatchRows) {
        const int nb = min(kBatchRows, B - b0);
        // Split-K epilogue.  Up to ~115k outputs (8 rows of a 13B MLP layer, 16 rows of a 5120-wide
        // one): one fixed-point atomic per output element, as in the batch-1 kernel (measured
        // 5-25 % faster there than the alternative, and up to 15 % slower above).  More outputs:
        // per-split partial tiles + a ticket, the last workgroup of a tile adds them.
        const int atomic_epilogue = (long long)nb * N <= kBatchAtomicOutputs;
        // Units per wave.  Atomic epilogue: as few as keep the grid within one resident round
        // (two workgroups per CU), so that nearly every wave's loads go out at once.  Partial
        // tiles: as few as keep the split count within the partial workspace; more only when the
        // grid would otherwise exceed ~4 workgroups per CU (less split-K traffic).
        int upv = 1;
        if (atomic_epilogue) {
            while (upv < 64 && (unit_plan.tiles * ceil_div(unit_plan.units_total, kBatchWaves * upv) > 512 ||
                                ceil_div(unit_plan.units_total, kBatchWaves * upv) > kMaxSplits))
                upv++;
        } else {
            while (ceil_div(unit_plan.units_total, kBatchWaves * upv) > kBatchMaxSplits) upv++;
            while (upv < 8 && unit_plan.tiles * ceil_div(unit_plan.units_total, kBatchWaves * (upv + 1)) >= 1024) upv++;
        }
        const Plan plan = make_plan(K, N, C, kBatchWaves * upv, kUnitK);
        hipLaunchKernelGGL(batch_prep_kernel<BITS>, dim3(plan.units_total), dim3(256), 0, stream, vec + (size_t)b0 * K,
                           cherry_indices, xa, rowsum, rowshift, nb, K, C, plan.units_normal);
        hipLaunchKernelGGL(batch_kernel<BITS>, dim3(plan.tiles * plan.splits), dim3(64 * kBatchWaves), 0, stream,
                           qweight, cherry_weight, scales, mul + (size_t)b0 * N, xa, rowsum, rowshift, partial, tickets,
                           reinterpret_cast<unsigned long long *>(workspace), atomic_epilogue, nb, K, N, C, G,
                           accumulate, plan, upv);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

hipError_t launch_batch(int bits, const __half *vec, const uint8_t *qweight, const __half *cherry_weight,
                        const int16_t *cherry_indices, const __half *scales, __half *mul, int B, int K, int N, int C,
                        int G, int accumulate, void *workspace, void *scratch, hipStream_t stream) {
    if (bits == 4)
        return launch_batch_bits<4>(vec, qweight, cherry_weight, cherry_indices, scales, mul, B, K, N, C, G, accumulate,
                                    workspace, scratch, stream);
    return launch_batch_bits<3>(vec, qweight, cherry_weight, cherry_indices, scales, mul, B, K, N, C, G, accumulate,
                                workspace, scratch, stream);
}

}  // namespace cq
