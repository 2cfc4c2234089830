// Fused dequant + matvec for 1 to 4 activation rows on gfx950, built as an HBM stream over the
// checkpoint layout (matvec_kernel<BITS, NW, KPL, NORM, ROWS>).
//
// Work unit: 4 * KPL compacted normal positions (KPL = 16: 64 positions, 8 / 6 KB of 4- / 3-bit
// weights; KPL = 32: 128 positions) x 256 output columns, or 32 cherry rows x 256 columns.  One
// wavefront owns one unit: the 64 lanes form 4 lane groups (16-lane DPP rows) that split the
// positions four ways, and the 16 lanes of a row each own 16 adjacent columns, so every load is
// a dwordx4 and a row of lanes reads 256 contiguous bytes of one byte row.  A wavefront issues
// all its weight loads up front and consumes them in order as they land.  NW (1, 2 or 4)
// wavefronts -- consecutive units of one column tile -- form a workgroup; the K reduction runs
// lane -> DPP row -> permlane swaps across rows -> LDS across wavefronts -> split-K partials
// across workgroups (one 64-bit fixed-point atomic per output, cq_device.h).  The launch
// geometry (KPL, NW) follows the size of the layer: matvec_geometry() below.  NORM fuses an
// RMSNorm of the activation row into its staging, ROWS = 2 runs two activation rows through the
// same dot2 sequence, ROWS = 4 up to four through 4x4x4 matrix-core instructions; a gate vector
// (silu(gate) * x) and several layers per launch are run-time options of the staging.
//
// Codes never pass through an int->float conversion.  A code field masked in place inside a
// 16-bit half is the fp16 subnormal  code * 2^(p-24)  (p = bit position of the field), which
// v_dot2_f32_f16 multiplies exactly against fp16 activations and accumulates in fp32:
//   4-bit: two byte rows are interleaved per column with one v_perm_b32; the low-nibble pair
//          and the high-nibble pair are two masks and two dot2 (5 VALU ops per 4 weights).
//   3-bit: three byte rows of a column give the 24-bit unit in two v_perm_b32; four masks pick
//          the code pairs (0,3) (1,4) (5,6) (2,7), whose different bit positions are folded
//          into the activations as exact powers of two (11 VALU ops per 8 weights).
// The grid offset c_b = 7.5 / 3.5 is applied once per lane group as  -c_b * sum(x).
//
// Arithmetic contract: csrc/quant_cuda_kernel.cu:718-835 (4-bit) and 558-672 / 316-438
// (3-bit); fp32 accumulation throughout, one rounding to fp16 at the end.
#include "cq_device.h"
#include "cq_kernels.h"

namespace cq {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kMaxFastCherries = 128;  // two 64-lane chunks of cherry indices
constexpr uint32_t kRsrcFlags = 0x00020000u;
constexpr uint32_t kOob = 0x80000000u;  // byte offset beyond any buffer this kernel accepts
constexpr int kStreamPolicy = 2;  // cache policy of the weight stream: nt (read once)

__device__ inline float fdot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a), __builtin_bit_cast(half2_t, b), c, false);
}

// fp16 pair (silu(gate) rounded to fp16) * up, rounded to fp16: the gated-MLP activation the
// reference materialises between its up/gate and down projections, applied while the down
// projection stages its activations.
__device__ inline uint32_t silu_mul_pair(uint32_t gate, uint32_t up) {
    uint32_t r = 0;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const float g = __half2float(__ushort_as_half((unsigned short)(gate >> (16 * i))));
        const float u = __half2float(__ushort_as_half((unsigned short)(up >> (16 * i))));
        const float a = __half2float(__float2half_rn(g / (1.f + __expf(-g))));
        r |= (uint32_t)__half_as_ushort(__float2half_rn(a * u)) << (16 * i);
    }
    return r;
}

// weight * fp16(x * rs) per half of a pair: RMSNorm applied while the activations are staged
__device__ inline uint32_t norm_pair(uint32_t xp, uint32_t wp, float rs) {
    uint32_t r = 0;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const float xv = __half2float(__ushort_as_half((unsigned short)(xp >> (16 * i))));
        const float wv = __half2float(__ushort_as_half((unsigned short)(wp >> (16 * i))));
        const float nv = __half2float(__float2half_rn(xv * rs));
        r |= (uint32_t)__half_as_ushort(__float2half_rn(wv * nv)) << (16 * i);
    }
    return r;
}

constexpr int kNormLoads = 4;  // 16-byte loads per thread for the fused RMSNorm's sum of squares

// rsqrt(mean(x^2) + eps) from the workgroup's shared pass over x (chunk = this thread's loads).
// Holds a workgroup barrier: when the fused norm is on, every wavefront of the workgroup calls it
// exactly once, whichever unit path it is on.  The fences are LDS-only so that the unit's
// weight loads stay in flight across the barrier.
template <int NW>
__device__ inline float norm_scale(const u32x4 (&chunk)[kNormLoads], float *s_ss, int wave, int lane, int K,
                                   float eps) {
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kNormLoads; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float a = __half2float(__ushort_as_half((unsigned short)(chunk[i][j] & 0xffffu)));
            const float b = __half2float(__ushort_as_half((unsigned short)(chunk[i][j] >> 16)));
            ss += a * a + b * b;
        }
    ss = wave_sum_all(ss);
    if (lane == 0) s_ss[wave] = ss;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    float t = 0.f;
#pragma unroll
    for (int wv = 0; wv < NW; wv++) t += s_ss[wv];
    return rsqrtf(t / (float)K + eps);
}

__device__ inline float half_bits_to_float(uint32_t h) {
    return __half2float(__ushort_as_half((unsigned short)h));
}

// KPL = compacted positions per lane group (16 or 32); a unit is 4 * KPL positions.
template <int BITS, int KPL>
struct Geo {
    static constexpr int kUnit = 4 * KPL;
    static constexpr int kRowsPerLaneGroup = KPL * BITS / 8;  // byte rows holding KPL positions
    static constexpr int kRowsPerUnit = 4 * kRowsPerLaneGroup;
    static constexpr int kPairs = KPL / 2;  // activation pair dwords per lane group
};

// NW = wavefronts (= units) per workgroup: 4, or 2 or 1 when the layer is so small
// that larger workgroups would leave CUs without work.
// ROWS = activation rows handled in the same pass (1, 2 or 4); `rows` (<= ROWS) of them exist, the
// others read zeros.  The codes are decoded once.  ROWS == 2: every row adds its own dot2 products.
// ROWS == 4: the masked code fields of 4 positions are the B operand and one row's activations
// the A operand of v_mfma_f32_4x4x4_16B_f16 (16 independent 4 x 4 x 4 products, one per group of
// four lanes), which costs about what the two dot2 of the one-row kernel cost.  The norm / gate
// prologues exist for one row only.
template <int BITS, int NW, int KPL, bool NORM, int ROWS>
__global__ __launch_bounds__(64 * NW) void matvec_kernel(
    const __half *__restrict__ x, MatvecPrologue pro, MatvecGroup grp,
    unsigned long long *__restrict__ acc_words, int K, int C, int G, int accumulate, Plan plan, int rows) {
    static_assert(ROWS == 1 || !NORM, "the fused prologues take one row");
    using G_ = Geo<BITS, KPL>;
    constexpr int R = G_::kRowsPerLaneGroup;
    constexpr int UK = G_::kUnit;
    __shared__ uint32_t s_win[NW][ROWS][128];  // per wave and row: 256 fp16 activations starting at the unit's first position
    __shared__ uint32_t s_pair[NW][ROWS][64];  // per wave and row: activation pairs laid out for the dot2 operands

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    // wave-uniform by construction; telling the compiler makes every branch on the unit index a
    // scalar branch, so a wavefront executes exactly one of the unit paths below
    const int wave = NORM ? __builtin_amdgcn_readfirstlane(tid >> 6) : tid >> 6;
    const int kq = lane >> 4, nl = lane & 15;
    const __half *__restrict__ x_gate = ROWS == 1 ? pro.gate : nullptr;
    // NORM is a template parameter so that the plain kernel does not pay the registers
    const __half *__restrict__ norm_w = NORM ? pro.norm_weight : nullptr;
    // Consecutive workgroups take neighbouring column tiles of the same rows, so that the
    // workgroups in flight at any moment read whole byte rows (DRAM page locality); walking one
    // 256-byte strip down the rows instead costs ~40 % of the bandwidth on square layers.
    // A launch covers up to kMaxGroup layers that share the activation vector (q/k/v, gate/up):
    // plan.tiles counts the column tiles of all of them and a workgroup picks its layer by tile.
    const int gtile = blockIdx.x % plan.tiles;
    const int split = blockIdx.x / plan.tiles;
    MatvecMember mm = grp.m[0];
#pragma unroll
    for (int i = 1; i < kMaxGroup; i++)
        if (i < grp.count && gtile >= grp.m[i].tile_begin) mm = grp.m[i];
    const uint8_t *__restrict__ qweight = mm.qweight;
    const __half *__restrict__ cherry_weight = mm.cherry_weight;
    const int16_t *__restrict__ cherry_indices = mm.cherry_indices;
    const __half *__restrict__ scales = mm.scales;
    __half *__restrict__ mul = mm.mul;
    const int N = mm.N;
    const int tile = gtile - mm.tile_begin;
    acc_words += (size_t)mm.tile_begin * kTileCols;
    const int u = split * NW + wave;
    const int n0 = tile * kTileCols + nl * 16;
    const bool col_ok = n0 < N;
    const int Kn = K - C;

    float tot[ROWS][16];
#pragma unroll
    for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int c = 0; c < 16; c++) tot[r][c] = 0.f;

    // Fused RMSNorm: the workgroup's threads share one pass over the K activations (16 bytes per
    // load, reads past the end return 0) for the sum of squares.  The loads are issued here, ahead
    // of the unit's own loads; they are consumed in norm_scale() after those have been issued.
    __shared__ float s_ss[NW];
    u32x4 nchunk[kNormLoads];
    if (norm_w) {
        const __amdgpu_buffer_rsrc_t rn = __builtin_amdgcn_make_buffer_rsrc((void *)x, 0, K * 2, kRsrcFlags);
#pragma unroll
        for (int i = 0; i < kNormLoads; i++)
            nchunk[i] = __builtin_amdgcn_raw_buffer_load_b128(rn, (uint32_t)(tid + i * 64 * NW) * 16u, 0, 0);
    }
    if (u < plan.units_normal) {
        const int ubase = u * UK;
        // ---- small operands first: vmcnt retires in order, so these can be waited on while
        // the weight loads issued after them are still in flight
        const __amdgpu_buffer_rsrc_t ri =
            __builtin_amdgcn_make_buffer_rsrc((void *)cherry_indices, 0, C * 2, kRsrcFlags);
        const int i0 = (short)__builtin_amdgcn_raw_buffer_load_b16(ri, lane * 2, 0, 0);
        const int i1 = (short)__builtin_amdgcn_raw_buffer_load_b16(ri, (lane + 64) * 2, 0, 0);
        // rows beyond `rows` lie outside the descriptor and read as zeros
        const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)x, 0, rows * K * 2, kRsrcFlags);
        uint32_t win0[ROWS], win1[ROWS];
        if (ROWS == 1) {
            win0[0] = __builtin_amdgcn_raw_buffer_load_b32(rx, (ubase + 2 * lane) * 2, 0, 0);
            win1[0] = __builtin_amdgcn_raw_buffer_load_b32(rx, (ubase + 128 + 2 * lane) * 2, 0, 0);
        } else {
            // a window that runs past the end of its row must not read the next row's activations
            const bool in0 = ubase + 2 * lane < K, in1 = ubase + 128 + 2 * lane < K;
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                const uint32_t roff = (uint32_t)(r * K) * 2u;
                win0[r] = __builtin_amdgcn_raw_buffer_load_b32(rx, (in0 && r < rows) ? roff + (ubase + 2 * lane) * 2 : kOob, 0, 0);
                win1[r] = __builtin_amdgcn_raw_buffer_load_b32(rx, (in1 && r < rows) ? roff + (ubase + 128 + 2 * lane) * 2 : kOob, 0, 0);
            }
        }
        uint32_t nw0 = 0, nw1 = 0;
        if (norm_w) {
            const __amdgpu_buffer_rsrc_t rnw = __builtin_amdgcn_make_buffer_rsrc((void *)norm_w, 0, K * 2, kRsrcFlags);
            nw0 = __builtin_amdgcn_raw_buffer_load_b32(rnw, (ubase + 2 * lane) * 2, 0, 0);
            nw1 = __builtin_amdgcn_raw_buffer_load_b32(rnw, (ubase + 128 + 2 * lane) * 2, 0, 0);
        }
        uint32_t gat0 = 0, gat1 = 0;
        if (x_gate) {
            const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc((void *)x_gate, 0, K * 2, kRsrcFlags);
            gat0 = __builtin_amdgcn_raw_buffer_load_b32(rg, (ubase + 2 * lane) * 2, 0, 0);
            gat1 = __builtin_amdgcn_raw_buffer_load_b32(rg, (ubase + 128 + 2 * lane) * 2, 0, 0);
        }
        const int ng = ceil_div(Kn, G);
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)scales, 0, ng * N * 2, kRsrcFlags);
        const int g = (ubase + KPL * kq) / G;
        const uint32_t soff = col_ok ? (uint32_t)(g * N + n0) * 2u : kOob;
        const u32x4 sc0 = __builtin_amdgcn_raw_buffer_load_b128(rs, soff, 0, 0);
        const u32x4 sc1 = __builtin_amdgcn_raw_buffer_load_b128(rs, soff + 16, 0, 0);

        // ---- the weight stream: R byte rows x 16 columns per lane, rows past the end read 0
        const int qrows = Kn / 8 * BITS;
        const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc((void *)qweight, 0, qrows * N, kRsrcFlags);
        const uint32_t woff = col_ok ? (uint32_t)((u * G_::kRowsPerUnit + kq * R) * N + n0) : kOob;
        u32x4 w[R];
#pragma unroll
        for (int r = 0; r < R; r++)
            w[r] = __builtin_amdgcn_raw_buffer_load_b128(rw, woff + (uint32_t)(r * N), 0, kStreamPolicy);

        // ---- gather the unit's 128 activations around the cherry channels
        // t[m] = idx[m] - m is non-decreasing; position k sits after every m with t[m] <= k
        const int t0 = lane < C ? i0 - lane : 0x7fffffff;
        const int t1 = lane + 64 < C ? i1 - (lane + 64) : 0x7fffffff;
        if (x_gate) {
            win0[0] = silu_mul_pair(gat0, win0[0]);
            win1[0] = silu_mul_pair(gat1, win1[0]);
        }
        if (norm_w) {
            const float rs = norm_scale<NW>(nchunk, s_ss, wave, lane, K, pro.eps);
            win0[0] = norm_pair(win0[0], nw0, rs);
            win1[0] = norm_pair(win1[0], nw1, rs);
        }
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            s_win[wave][r][lane] = win0[r];
            s_win[wave][r][64 + lane] = win1[r];
        }
        // positions this lane prepares, relative to the lane group's first position
        int j0, j1, p0 = 0, p1 = 0;
        if (BITS == 4) {
            j0 = 4 * (nl >> 1) + (nl & 1);  // even lanes: (4p, 4p+2), odd lanes: (4p+1, 4p+3)
            j1 = j0 + 2;
            if (ROWS == 4) p0 = p1 = 4 * (nl & 1);  // the matrix-core path keeps one accumulator: high nibbles sit at bit 4
        } else {
            const int q = nl & 3, t8 = 8 * (nl >> 2);  // code pairs (0,3) (1,4) (5,6) (2,7) of a unit
            j0 = t8 + ((0x2510 >> (4 * q)) & 15);
            j1 = t8 + ((0x7643 >> (4 * q)) & 15);
            p0 = (0x6730 >> (4 * q)) & 15;  // bit position of the first code's field in its half
            p1 = (0x5241 >> (4 * q)) & 15;
        }
        const int k0 = ubase + KPL * kq + j0, k1 = ubase + KPL * kq + j1;
        int low0 = __popcll(__ballot(t0 < ubase)) + __popcll(__ballot(t1 < ubase));
        int low1 = low0;
        {
            unsigned long long m = __ballot(t0 >= ubase && t0 < ubase + UK);
            while (m) {
                int j = __builtin_ctzll(m);
                int tj = __builtin_amdgcn_readlane(t0, j);
                low0 += tj <= k0;
                low1 += tj <= k1;
                m &= m - 1;
            }
            m = __ballot(t1 >= ubase && t1 < ubase + UK);
            while (m) {
                int j = __builtin_ctzll(m);
                int tj = __builtin_amdgcn_readlane(t1, j);
                low0 += tj <= k0;
                low1 += tj <= k1;
                m &= m - 1;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        const bool prep = nl < G_::kPairs;  // lanes that prepare an activation pair
        float xsum[ROWS];
        int sh[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            const unsigned short *winh = reinterpret_cast<const unsigned short *>(&s_win[wave][r][0]);
            uint32_t h0 = (prep && k0 < Kn) ? winh[(k0 - ubase) + low0] : 0u;
            uint32_t h1 = (prep && k1 < Kn) ? winh[(k1 - ubase) + low1] : 0u;
            xsum[r] = row_sum(half_bits_to_float(h0) + half_bits_to_float(h1));
            sh[r] = 0;
            if (BITS == 3 || ROWS == 4) {
                // scale the lane group's activations so that the largest has biased exponent 29;
                // the per-field factors 2^-p (p <= 7) then stay far inside the fp16 normal range
                const int e = row_max((int)max(h0 & 0x7fffu, h1 & 0x7fffu)) >> 10;
                sh[r] = 29 - e;
                h0 = __half_as_ushort(__float2half_rn(ldexpf(half_bits_to_float(h0), sh[r] - p0)));
                h1 = __half_as_ushort(__float2half_rn(ldexpf(half_bits_to_float(h1), sh[r] - p1)));
            }
            s_pair[wave][r][lane] = h0 | (h1 << 16);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        // ROWS == 4: v_mfma_f32_4x4x4_16B_f16 works on 16 blocks of 4 lanes; lane t of a block feeds
        // row t's activations (A, 4 positions) and its own column's code fields (B, the same 4
        // positions) and receives its column's sums for all four rows, so a lane holds the
        // activations of ONE row, as in the one-row kernel.
        constexpr int XR = ROWS == 4 ? 1 : ROWS;
        u32x4 xq[XR][G_::kPairs / 4];
#pragma unroll
        for (int r = 0; r < XR; r++)
#pragma unroll
            for (int i = 0; i < G_::kPairs / 4; i++)
                xq[r][i] = *reinterpret_cast<const u32x4 *>(&s_pair[wave][ROWS == 4 ? (lane & 3) : r][16 * kq + 4 * i]);

        if (ROWS == 4) {
            // d[c][r]: this lane's column c, activation row r
            float4_t d[16];
#pragma unroll
            for (int c = 0; c < 16; c++) d[c] = (float4_t){0.f, 0.f, 0.f, 0.f};
            if (BITS == 4) {
#pragma unroll
                for (int p = 0; p < R / 2; p++) {
                    const half4_t av = __builtin_bit_cast(half4_t, (u32x2){xq[0][p >> 1][(p & 1) * 2], xq[0][p >> 1][(p & 1) * 2 + 1]});
#pragma unroll
                    for (int dd = 0; dd < 4; dd++) {
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const uint32_t pr = __builtin_amdgcn_perm(w[2 * p][dd], w[2 * p + 1][dd],
                                                                      0x0c000c00u | (uint32_t)(j << 16) | (uint32_t)(4 + j));
                            const half4_t bv = __builtin_bit_cast(half4_t, (u32x2){pr & 0x000f000fu, pr & 0x00f000f0u});
                            d[4 * dd + j] = __builtin_amdgcn_mfma_f32_4x4x4f16(av, bv, d[4 * dd + j], 0, 0, 0);
                        }
                    }
                }
            } else {
#pragma unroll
                for (int t = 0; t < R / 3; t++) {
                    const half4_t a0 = __builtin_bit_cast(half4_t, (u32x2){xq[0][t][0], xq[0][t][1]});
                    const half4_t a1 = __builtin_bit_cast(half4_t, (u32x2){xq[0][t][2], xq[0][t][3]});
#pragma unroll
                    for (int dd = 0; dd < 4; dd++) {
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const uint32_t sel = 0x0c000000u | (uint32_t)(j << 16) | (uint32_t)(j << 8) | (uint32_t)(4 + j);
                            const uint32_t p1 = __builtin_amdgcn_perm(w[3 * t][dd], w[3 * t + 1][dd], sel);
                            const uint32_t p2 = __builtin_amdgcn_perm(w[3 * t + 1][dd], w[3 * t + 2][dd], sel);
                            const half4_t b0 = __builtin_bit_cast(half4_t, (u32x2){p1 & 0x000e0007u, p1 & 0x00700038u});
                            const half4_t b1 = __builtin_bit_cast(
                                half4_t, (u32x2){p2 & 0x001c0380u, (p1 & 0x000001c0u) | (p2 & 0x00e00000u)});
                            d[4 * dd + j] = __builtin_amdgcn_mfma_f32_4x4x4f16(a0, b0, d[4 * dd + j], 0, 0, 0);
                            d[4 * dd + j] = __builtin_amdgcn_mfma_f32_4x4x4f16(a1, b1, d[4 * dd + j], 0, 0, 0);
                        }
                    }
                }
            }
            constexpr float kGrid = BITS == 4 ? -7.5f : -3.5f;
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                const float corr = kGrid * xsum[r];
#pragma unroll
                for (int c = 0; c < 16; c++) {
                    const uint32_t sw = c < 8 ? sc0[c >> 1] : sc1[(c - 8) >> 1];
                    const float s = half_bits_to_float((c & 1) ? (sw >> 16) : (sw & 0xffffu));
                    tot[r][c] = (ldexpf(d[c][r], 24 - sh[r]) + corr) * s;
                }
            }
        } else if (BITS == 4) {
            float lo[ROWS][16], hi[ROWS][16];
#pragma unroll
            for (int r = 0; r < ROWS; r++)
#pragma unroll
                for (int c = 0; c < 16; c++) lo[r][c] = hi[r][c] = 0.f;
#pragma unroll
            for (int p = 0; p < R / 2; p++) {
#pragma unroll
                for (int d = 0; d < 4; d++) {
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        // bytes (row 2p col j, 0, row 2p+1 col j, 0)
                        const uint32_t pr = __builtin_amdgcn_perm(w[2 * p][d], w[2 * p + 1][d],
                                                                  0x0c000c00u | (uint32_t)(j << 16) | (uint32_t)(4 + j));
                        const uint32_t ce = pr & 0x000f000fu, co = pr & 0x00f000f0u;
#pragma unroll
                        for (int r = 0; r < ROWS; r++) {
                            lo[r][4 * d + j] = fdot2(ce, xq[r][p >> 1][(p & 1) * 2], lo[r][4 * d + j]);
                            hi[r][4 * d + j] = fdot2(co, xq[r][p >> 1][(p & 1) * 2 + 1], hi[r][4 * d + j]);
                        }
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                const float corr = -7.5f * xsum[r];
#pragma unroll
                for (int c = 0; c < 16; c++) {
                    const uint32_t sw = c < 8 ? sc0[c >> 1] : sc1[(c - 8) >> 1];
                    const float s = half_bits_to_float((c & 1) ? (sw >> 16) : (sw & 0xffffu));
                    tot[r][c] = (lo[r][c] * 16777216.0f + hi[r][c] * 1048576.0f + corr) * s;
                }
            }
        } else {
            float acc[ROWS][16];
#pragma unroll
            for (int r = 0; r < ROWS; r++)
#pragma unroll
                for (int c = 0; c < 16; c++) acc[r][c] = 0.f;
#pragma unroll
            for (int t = 0; t < R / 3; t++) {
#pragma unroll
                for (int d = 0; d < 4; d++) {
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const uint32_t sel = 0x0c000000u | (uint32_t)(j << 16) | (uint32_t)(j << 8) | (uint32_t)(4 + j);
                        // p1 = bits 0..15 of the 24-bit unit | its bits 8..15 again in the high half
                        // p2 = bits 8..23 of the unit        | its bits 16..23 in the high half
                        const uint32_t p1 = __builtin_amdgcn_perm(w[3 * t][d], w[3 * t + 1][d], sel);
                        const uint32_t p2 = __builtin_amdgcn_perm(w[3 * t + 1][d], w[3 * t + 2][d], sel);
                        const uint32_t c03 = p1 & 0x000e0007u, c14 = p1 & 0x00700038u, c56 = p2 & 0x001c0380u;
                        const uint32_t c27 = (p1 & 0x000001c0u) | (p2 & 0x00e00000u);
#pragma unroll
                        for (int r = 0; r < ROWS; r++) {
                            float a = acc[r][4 * d + j];
                            a = fdot2(c03, xq[r][t][0], a);  // codes 0 | 3
                            a = fdot2(c14, xq[r][t][1], a);  // codes 1 | 4
                            a = fdot2(c56, xq[r][t][2], a);  // codes 5 | 6
                            a = fdot2(c27, xq[r][t][3], a);  // codes 2 | 7
                            acc[r][4 * d + j] = a;
                        }
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                const float corr = -3.5f * xsum[r];
#pragma unroll
                for (int c = 0; c < 16; c++) {
                    const uint32_t sw = c < 8 ? sc0[c >> 1] : sc1[(c - 8) >> 1];
                    const float s = half_bits_to_float((c & 1) ? (sw >> 16) : (sw & 0xffffu));
                    tot[r][c] = (ldexpf(acc[r][c], 24 - sh[r]) + corr) * s;
                }
            }
        }
    } else if (u < plan.units_total) {
        // ---- cherry unit: 32 rows of fp16 weights, 8 per lane group, times x[idx[c]]
        const int c0 = (u - plan.units_normal) * kCherryUnit + 8 * kq;
        const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc((void *)cherry_weight, 0, C * N * 2, kRsrcFlags);
        const uint32_t coff = col_ok ? (uint32_t)(c0 * N + n0) * 2u : kOob;
        // the activation gather x[idx[c]] is a dependent chain; run it before the weight loads are
        // queued, while this wave has nothing else outstanding
        const __amdgpu_buffer_rsrc_t ri =
            __builtin_amdgcn_make_buffer_rsrc((void *)cherry_indices, 0, C * 2, kRsrcFlags);
        const int ci = (unsigned short)__builtin_amdgcn_raw_buffer_load_b16(ri, (c0 + (nl & 7)) * 2, 0, 0);
        const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)x, 0, rows * K * 2, kRsrcFlags);
        const uint32_t xoff = (nl < 8 && c0 + nl < C) ? (uint32_t)ci * 2u : kOob;
        uint32_t xrow[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; r++)
            xrow[r] = __builtin_amdgcn_raw_buffer_load_b16(rx, (r < rows && xoff != kOob) ? xoff + (uint32_t)(r * K) * 2u : kOob, 0, 0);
        uint32_t xraw = xrow[0];
        if (x_gate) {
            const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc((void *)x_gate, 0, K * 2, kRsrcFlags);
            const uint32_t graw = __builtin_amdgcn_raw_buffer_load_b16(rg, xoff, 0, 0);
            xraw = silu_mul_pair(graw & 0xffffu, xraw & 0xffffu) & 0xffffu;
        }
        uint32_t nwraw = 0;
        if (norm_w) {
            const __amdgpu_buffer_rsrc_t rnw = __builtin_amdgcn_make_buffer_rsrc((void *)norm_w, 0, K * 2, kRsrcFlags);
            nwraw = __builtin_amdgcn_raw_buffer_load_b16(rnw, xoff, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);  // keep the weight loads behind the gather in the queue
        u32x4 cw[8][2];
#pragma unroll
        for (int r = 0; r < 8; r++) {
            cw[r][0] = __builtin_amdgcn_raw_buffer_load_b128(rc, coff + (uint32_t)(r * N * 2), 0, kStreamPolicy);
            cw[r][1] = __builtin_amdgcn_raw_buffer_load_b128(rc, coff + (uint32_t)(r * N * 2) + 16, 0, kStreamPolicy);
        }
        if (norm_w) {
            const float rs = norm_scale<NW>(nchunk, s_ss, wave, lane, K, pro.eps);
            xraw = norm_pair(xraw & 0xffffu, nwraw & 0xffffu, rs) & 0xffffu;
        }
        xrow[0] = xraw;
#pragma unroll
        for (int r = 0; r < ROWS; r++) s_pair[wave][r][lane] = __builtin_bit_cast(uint32_t, half_bits_to_float(xrow[r]));
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        float xc[ROWS][8];
#pragma unroll
        for (int b = 0; b < ROWS; b++)
#pragma unroll
            for (int r = 0; r < 8; r++) xc[b][r] = __builtin_bit_cast(float, s_pair[wave][b][16 * kq + r]);
#pragma unroll
        for (int r = 0; r < 8; r++) {
#pragma unroll
            for (int c = 0; c < 16; c++) {
                const uint32_t ww = cw[r][c >> 3][(c & 7) >> 1];
                const float wf = half_bits_to_float((c & 1) ? (ww >> 16) : (ww & 0xffffu));
#pragma unroll
                for (int b = 0; b < ROWS; b++) tot[b][c] += wf * xc[b][r];
            }
        }
    } else if (norm_w) {
        // a wavefront without a unit still owes the workgroup its barrier
        (void)norm_scale<NW>(nchunk, s_ss, wave, lane, K, pro.eps);
    }

    // ---- reduce over the four lane groups; lane group kq ends up with columns 4kq .. 4kq+3
    float q4[ROWS][4];
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        float h8[8];
#pragma unroll
        for (int i = 0; i < 8; i++) h8[i] = swap32_add(tot[r][i], tot[r][8 + i]);
#pragma unroll
        for (int i = 0; i < 4; i++) q4[r][i] = swap16_add(h8[i], h8[4 + i]);
    }
    if (NW == 1) {
        const int n = n0 + 4 * kq;
        splitk_finish<__half, ROWS, 4>(q4, rows, N, n, n < N, plan.splits, acc_words, mul, accumulate);
    } else {
        // ---- across the workgroup's wavefronts through LDS, then 4 / NW columns per thread
        __shared__ float s_red[NW][ROWS][kTileCols];
#pragma unroll
        for (int r = 0; r < ROWS; r++)
            *reinterpret_cast<float4 *>(&s_red[wave][r][16 * nl + 4 * kq]) = make_float4(q4[r][0], q4[r][1], q4[r][2], q4[r][3]);
        __syncthreads();
        constexpr int CPT = 4 / NW;  // columns per thread
        float vals[ROWS][CPT];
#pragma unroll
        for (int r = 0; r < ROWS; r++)
#pragma unroll
            for (int c = 0; c < CPT; c++) {
                float v = 0.f;
#pragma unroll
                for (int wv = 0; wv < NW; wv++) v += s_red[wv][r][(tid * CPT + c) & (kTileCols - 1)];
                vals[r][c] = v;
            }
        const int n = tile * kTileCols + tid * CPT;
        splitk_finish<__half, ROWS, CPT>(vals, rows, N, n, n < N && tid * CPT < kTileCols, plan.splits, acc_words, mul,
                                         accumulate);
    }
}

bool matvec_supported(int bits, int B, int K, int N, int C, int G) {
    (void)bits;
    if (B < 1 || B > kMatvecMaxRows) return false;
    if (C > kMaxFastCherries) return false;
    if (G % 32) return false;
    // byte offsets are 32-bit and kOob must lie beyond every buffer
    const long long wbytes = (long long)(K - C) / 8 * 4 * N;
    const long long cbytes = (long long)C * N * 2;
    const long long sbytes = (long long)ceil_div(K - C, G) * N * 2;
    if (wbytes >= 0x7fff0000ll || cbytes >= 0x7fff0000ll || sbytes >= 0x7fff0000ll) return false;
    if (K - C <= 0) return false;
    // the split count of the geometry the launch will really use (it depends on the size of the
    // layer and on the row count) must fit the 8-bit arrival counter of the split-K word
    return matvec_geometry(bits, K, N, C, B).splits <= kMaxSplits;
}


// Two to four rows take this kernel rather than the matrix-core batch path whenever it takes the
// shape: no preparation launch, atomics instead of partial tiles.  Measured on the 4096 -> 11008
// 4-bit layer: 2 rows 9.5 us (batch path 13.6), 3 rows 11.0 (14.1), 4 rows 11.5 (14.5); 8192 ->
// 28672: 28.2 (35.8) and 34.3 (37.6).  Two rows run the dot2 instantiation (the 4 x 4 MFMA one
// costs 11.4 us there), three and four the MFMA one.
bool matvec_rows_preferred(int bits, int B, int K, int N, int C, int G) {
    return B >= 2 && matvec_supported(bits, B, K, N, C, G);
}

template <int BITS, int NW, int KPL>
static hipError_t launch_matvec_nw(const __half *vec, const MatvecPrologue &pro, const MatvecGroup &grp, int tiles,
                                   int K, int C, int G, int accumulate, void *workspace, hipStream_t stream,
                                   int rows) {
    // the fused norm reads K activations with kNormLoads 16-byte loads per thread
    if (pro.norm_weight && K > kNormLoads * 8 * 64 * NW) return hipErrorNotSupported;
    if (rows > 1 && (pro.norm_weight || pro.gate || grp.count != 1)) return hipErrorNotSupported;
    Plan plan = make_plan(K, kTileCols, C, NW, 4 * KPL);
    if (plan.splits > kMaxSplits) return hipErrorNotSupported;  // would wrap the split-K arrival counter
    plan.tiles = tiles;
    const dim3 grid(plan.tiles * plan.splits), block(64 * NW);
    unsigned long long *acc = reinterpret_cast<unsigned long long *>(workspace);
    if (rows > 2)
        hipLaunchKernelGGL((matvec_kernel<BITS, NW, KPL, false, 4>), grid, block, 0, stream, vec, pro, grp, acc, K, C,
                           G, accumulate, plan, rows);
    else if (rows == 2)
        hipLaunchKernelGGL((matvec_kernel<BITS, NW, KPL, false, 2>), grid, block, 0, stream, vec, pro, grp, acc, K, C,
                           G, accumulate, plan, rows);
    else if (pro.norm_weight)
        hipLaunchKernelGGL((matvec_kernel<BITS, NW, KPL, true, 1>), grid, block, 0, stream, vec, pro, grp, acc, K, C,
                           G, accumulate, plan, 1);
    else
        hipLaunchKernelGGL((matvec_kernel<BITS, NW, KPL, false, 1>), grid, block, 0, stream, vec, pro, grp, acc, K, C,
                           G, accumulate, plan, 1);
    return hipGetLastError();
}

// Geometry, from sweeps over the LLaMA-7B/13B/70B layer shapes on MI355X (3- and 4-bit, single and
// grouped launches): 64-position units (8 KB per wave: more wavefronts in flight, half the
// decode left to do when a wave's data lands) up to 28 MB of packed weights, 128-position units
// (half the wavefronts and split-K atomics) above; four wavefronts per workgroup throughout --
// eight make the workgroup barrier and the per-CU placement coarser and were slower nearly
// everywhere, fewer multiply the split-K atomics.  Only layers too small to give every second
// CU a workgroup use fewer wavefronts per workgroup.
int matvec_kpl(int bits, int K, int N, int C) {
    const long long bytes = (long long)(K - C) / 8 * bits * N;
    return bytes < (28ll << 20) ? 16 : 32;
}

int matvec_waves_per_wg(int K, int N, int C, int kpl) {
    int nw = 4;
    while (nw > 1) {
        const Plan p = make_plan(K, N, C, nw, 4 * kpl);
        if (p.tiles * p.splits >= 128) break;
        nw >>= 1;
    }
    while (nw < 4 && make_plan(K, N, C, nw, 4 * kpl).splits > kMaxSplits) nw <<= 1;
    return nw;
}

// The launch geometry of a call: positions per lane and unit (16: 64-position units, 32: 128),
// wavefronts per workgroup, and the resulting workgroups per column tile.  One function for the
// support checks and the launch, so that they cannot disagree.
// three and four rows: 128-position units whatever the size -- every row multiplies the split-K
// atomics (0.85 us per row on the 4096 -> 11008 layer with 64-position units), half as many
// splits outweigh the coarser grid (4 rows: 13.1 -> 11.5 us; two rows: 9.5 -> 10.1, left alone)
MatvecGeometry matvec_geometry(int bits, int K, int n_total, int C, int rows) {
    MatvecGeometry g;
    g.kpl = rows > 2 ? 32 : matvec_kpl(bits, K, n_total, C);
    g.nw = matvec_waves_per_wg(K, n_total, C, g.kpl);
    g.splits = make_plan(K, kTileCols, C, g.nw, 4 * g.kpl).splits;
    if (g.splits > kMaxSplits && g.kpl == 16) {  // very long rows of a small layer: coarser units
        g.kpl = 32;
        g.nw = matvec_waves_per_wg(K, n_total, C, g.kpl);
        g.splits = make_plan(K, kTileCols, C, g.nw, 4 * g.kpl).splits;
    }
    return g;
}

bool matvec_norm_supported(int bits, int K, int n_total, int C) {
    const MatvecGeometry g = matvec_geometry(bits, K, n_total, C, 1);
    return g.splits <= kMaxSplits && K <= kNormLoads * 8 * 64 * g.nw;
}

static hipError_t launch_matvec_rows_group(int bits, const __half *vec, const MatvecPrologue &pro,
                                           const MatvecMember *members, int count, int K, int C, int G,
                                           int accumulate, void *workspace, hipStream_t stream, int rows) {
    MatvecGroup grp = {};
    grp.count = count;
    int tiles = 0, n_total = 0;
    for (int i = 0; i < count; i++) {
        grp.m[i] = members[i];
        grp.m[i].tile_begin = tiles;
        tiles += ceil_div(members[i].N, kTileCols);
        n_total += members[i].N;
    }
    for (int i = count; i < kMaxGroup; i++) grp.m[i] = grp.m[0];
    // geometry from the group's total size: the launch streams all members' weights together
    const MatvecGeometry geo = matvec_geometry(bits, K, n_total, C, rows);
    if (geo.splits > kMaxSplits) return hipErrorNotSupported;
    const int kpl = geo.kpl, nw = geo.nw;
#define CQ_LAUNCH(B, W, P)                                                                                   \
    return launch_matvec_nw<B, W, P>(vec, pro, grp, tiles, K, C, G, accumulate, workspace, stream, rows)
#define CQ_PICK_NW(B, P)                                                                                     \
    do {                                                                                                     \
        if (nw >= 4) CQ_LAUNCH(B, 4, P);                                                                     \
        if (nw == 2) CQ_LAUNCH(B, 2, P);                                                                     \
        CQ_LAUNCH(B, 1, P);                                                                                  \
    } while (0)
    if (bits == 4) {
        if (kpl == 16) CQ_PICK_NW(4, 16);
        CQ_PICK_NW(4, 32);
    }
    if (kpl == 16) CQ_PICK_NW(3, 16);
    CQ_PICK_NW(3, 32);
#undef CQ_PICK_NW
#undef CQ_LAUNCH
}

hipError_t launch_matvec_group(int bits, const __half *vec, const MatvecPrologue &pro, const MatvecMember *members,
                               int count, int K, int C, int G, int accumulate, void *workspace,
                               hipStream_t stream) {
    return launch_matvec_rows_group(bits, vec, pro, members, count, K, C, G, accumulate, workspace, stream, 1);
}

hipError_t launch_matvec(int bits, const __half *vec, const uint8_t *qweight, const __half *cherry_weight,
                         const int16_t *cherry_indices, const __half *scales, __half *mul, int K, int N, int C,
                         int G, int accumulate, void *workspace, hipStream_t stream) {
    MatvecMember m = {qweight, cherry_weight, cherry_indices, scales, mul, N, 0};
    return launch_matvec_group(bits, vec, MatvecPrologue{nullptr, nullptr, 0.f}, &m, 1, K, C, G, accumulate,
                               workspace, stream);
}

// 2..kMatvecMaxRows activation rows (vec (rows, K), mul (rows, N), one accumulator word per
// output in `workspace`) in one pass over the weights.
hipError_t launch_matvec_rows(int bits, const __half *vec, const uint8_t *qweight, const __half *cherry_weight,
                              const int16_t *cherry_indices, const __half *scales, __half *mul, int rows, int K,
                              int N, int C, int G, int accumulate, void *workspace, hipStream_t stream) {
    MatvecMember m = {qweight, cherry_weight, cherry_indices, scales, mul, N, 0};
    return launch_matvec_rows_group(bits, vec, MatvecPrologue{nullptr, nullptr, 0.f}, &m, 1, K, C, G, accumulate,
                                    workspace, stream, rows);
}

}  // namespace cq
