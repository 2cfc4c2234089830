// Batch-1 matvec over the repacked weight stream, one workgroup per compute unit (gfx950).
//
// Same stream, same arithmetic and the same tile ownership as stream_kernel in cq_stream.hip (a
// team of W wavefronts owns a tile of 16 columns over all of K; no split-K, no atomics, one
// rounding from fp32), but the launch is shaped by what the memory pipeline of a compute unit
// does, as per-wavefront timestamps of the older kernel showed it:
//
//   * A compute unit accepts vector loads only as earlier ones return (about 32 KB can be
//     outstanding).  A wavefront that requests all its units up front therefore sits in the issue
//     stage for microseconds, a barrier behind it opens only when the slowest wavefront has got
//     its last request accepted, and whatever another workgroup of the same compute unit requests
//     later -- its activations -- waits behind all of that.  So there is ONE workgroup per compute
//     unit (the launch asks for more than half of the LDS), its staging wavefronts come first in
//     the workgroup and request the activations before any weight request exists, and a computing
//     wavefront requests only D0 units before the barrier and keeps a ring of D afterwards: the
//     requests of all wavefronts interleave, every wavefront's data arrives at the pace it
//     consumes it, and the last data to arrive is one unit per wavefront, not one wavefront's
//     whole share.
//   * The activations are staged without a workgroup barrier of their own: staging wavefront j
//     requests exactly the raw slice its NB blocks of 512 compacted positions can touch (the
//     positions themselves plus up to 128 cherry columns in front), copies it to its place in LDS
//     and gathers from there.  Neighbouring slices overlap; both owners write the same values.
//   * TEAMS teams per workgroup, each on a tile of its own: team t of workgroup b takes the tiles
//     b + G (t + TEAMS j), j = 0, 1, ... of the workgroup's layer (G workgroups work on that layer),
//     the ring of loads running across tile boundaries.
//
// Measured on MI355X (us per launch in a graph of 2000, weights from HBM; stream_kernel -> this):
// 4096 -> 11008 4-bit 6.35 -> 5.60, 3-bit 6.08 -> 5.08; 4096 -> 4096 3.98 -> 3.66; 4096 -> 32000
// 13.7 -> 11.9; 8192 -> 8192 8.85 -> 7.6; 8192 -> 28672 21.4 -> 20.2; 8192 -> 1024 5.26 -> 4.1.
//
// Arithmetic contract: csrc/quant_cuda_kernel.cu:718-835 (4-bit) and 558-672 (3-bit) of the
// reference; replaces the per-thread decode loops at :811-831 / :649-667.
#include <mutex>

#include "cq_stream_dev.h"

namespace cq {

constexpr int kCuMaxWalk = 16;   // tiles one team takes at most
constexpr int kCuCus = 256;      // compute units of an MI355X
constexpr int kCuMaxDevices = 64;

// weight * fp16(x * rs) on both halves of a pair (the rounding points of add_rmsnorm_kernel)
__device__ inline uint32_t cu_norm_pair(uint32_t xp, uint32_t wp, float rs) {
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

struct CuGroup {  // members 1 and 2 of a group launch (member 0 travels in the leading arguments)
    const uint8_t *stream[2];
    __half *mul[2];
    int N[2];
    int wg_begin[2];  // first workgroup of members 1 and 2
    int wgs[2];       // workgroups of members 1 and 2
    int count;
};

// S staging wavefronts (wavefronts 0 .. S-1, NB blocks of 512 compacted positions each), then
// TEAMS teams of W computing wavefronts; computing wavefront c of a team takes the units c, c + W,
// ... (L at most) of every tile the team comes to.  The leading arguments (14 dwords) are what the
// first loads of a workgroup need; the file is built with a kernel-argument preload count that
// puts them into scalar registers before the wavefronts start.
template <int BITS, int W, int L, int TEAMS, int S, int NB, int D0, int D, bool NORM, bool GROUP>
__global__ __launch_bounds__(64 * (W * TEAMS + S)) void stream_cu_kernel(
    const __half *__restrict__ x, const uint8_t *__restrict__ stream0, __half *__restrict__ mul0, int K, int C, int ng,
    int N0, uint32_t hdr_bytes, uint32_t off_cherry, uint32_t off_units, uint32_t record_bytes, int wgs0, int accumulate,
    const __half *__restrict__ norm_w, float eps, CuGroup grp) {
    constexpr int NC = W * TEAMS;  // computing wavefronts
    constexpr int NT = 64 * (NC + S);
    constexpr int UB = BITS == 4 ? 1024 : 768;
    constexpr float kGrid = BITS == 4 ? -7.5f : -3.5f;
    constexpr int XS = NB + 1;  // 16-byte loads per lane that cover a staging wavefront's raw slice
    static_assert(D0 <= D && D <= L && L % D == 0 && L % 4 == 0, "ring slots are fixed per unit across tiles");
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kq = lane >> 4, nn = lane & 15;

    // which layer this workgroup works for (members are consecutive ranges of workgroups); the
    // candidates are pinned in scalar registers first so that the selects stay selects
    const uint8_t *__restrict__ stream = stream0;
    __half *__restrict__ mul = mul0;
    int N = N0, bid = blockIdx.x, G = wgs0;
    if constexpr (GROUP) {
        const uint8_t *s1 = grp.stream[0], *s2 = grp.stream[1];
        __half *o1 = grp.mul[0], *o2 = grp.mul[1];
        int n1 = grp.N[0], n2 = grp.N[1], b1 = grp.wg_begin[0], b2 = grp.wg_begin[1], g1 = grp.wgs[0], g2 = grp.wgs[1],
            cnt = grp.count;
        asm volatile("" : "+s"(stream), "+s"(s1), "+s"(s2), "+s"(mul), "+s"(o1), "+s"(o2));
        asm volatile("" : "+s"(N), "+s"(n1), "+s"(n2), "+s"(b1), "+s"(b2), "+s"(g1), "+s"(g2), "+s"(cnt));
        const bool m1 = cnt > 1 && bid >= b1, m2 = cnt > 2 && bid >= b2;
        stream = m2 ? s2 : m1 ? s1 : stream;
        mul = m2 ? o2 : m1 ? o1 : mul;
        N = m2 ? n2 : m1 ? n1 : N;
        G = m2 ? g2 : m1 ? g1 : G;
        bid -= m2 ? b2 : m1 ? b1 : 0;
    }
    const int ntiles = (N + kStreamTileCols - 1) / kStreamTileCols;
    const int Knp512 = (ng * kStreamUnitK + 511) & ~511;
    const int nblk = Knp512 >> 9;
    // LDS: raw activations (slice by slice, zeros past the row) | compacted activations | unit sums | partial outputs
    unsigned short *s_raw = reinterpret_cast<unsigned short *>(smem);
    unsigned short *s_xs = s_raw + Knp512 + 512 * NB + 8;
    float *s_xsum = reinterpret_cast<float *>(s_xs + Knp512);
    float *s_red = s_xsum + 4 * nblk;
    const int tstride = G * TEAMS;
    const int P = (ntiles + tstride - 1) / tstride;  // tiles the busiest team walks

    if (wave < S) {
        // ---- staging wavefront: its slice of the row, its blocks' gather table; gather; unit sums
        __builtin_amdgcn_s_setprio(3);
        const int b0 = wave * NB, b1 = min(nblk, b0 + NB);
        const bool active = b0 < nblk, last = active && b1 == nblk;
        const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)x, 0, K * 2, kSFlags);
        const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc((void *)stream, 0, (int)hdr_bytes, kSFlags);
        su4 xr[XS];
        su2 tb[NB];
#pragma unroll
        for (int i = 0; i < XS; i++)
            xr[i] = __builtin_amdgcn_raw_buffer_load_b128(rx, active ? (uint32_t)(b0 * 512 + i * 512 + lane * 8) * 2u : kSOob, 0, 0);
#pragma unroll
        for (int i = 0; i < NB; i++)
            tb[i] = __builtin_amdgcn_raw_buffer_load_b64(rh, b0 + i < b1 ? (uint32_t)((b0 + i) * 512 + lane * 8) : kSOob, 0, 0);
        if constexpr (NORM) {
            su4 nr[XS];
            const __amdgpu_buffer_rsrc_t rn = __builtin_amdgcn_make_buffer_rsrc((void *)norm_w, 0, K * 2, kSFlags);
#pragma unroll
            for (int i = 0; i < XS; i++)
                nr[i] = __builtin_amdgcn_raw_buffer_load_b128(rn, active ? (uint32_t)(b0 * 512 + i * 512 + lane * 8) * 2u : kSOob, 0, 0);
            // sum of squares over the part of the row that only this wavefront holds: its own
            // blocks' positions, and for the last one everything behind them (zeros past the row)
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < XS; i++)
                if (i < b1 - b0 || last) {
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const float a = __half2float(__ushort_as_half((unsigned short)(xr[i][j] & 0xffffu)));
                        const float b = __half2float(__ushort_as_half((unsigned short)(xr[i][j] >> 16)));
                        ss += a * a + b * b;
                    }
                }
            ss = wave_sum_all(ss);
            if (lane == 0) s_red[wave] = ss;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
            float t = 0.f;
#pragma unroll
            for (int wv = 0; wv < S; wv++) t += s_red[wv];
            const float rs = rsqrtf(t / (float)K + eps);
#pragma unroll
            for (int i = 0; i < XS; i++) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    xr[i][j] = cu_norm_pair(xr[i][j], nr[i][j], rs);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        if (active) {
#pragma unroll
            for (int i = 0; i < XS; i++) reinterpret_cast<su4 *>(s_raw + b0 * 512 + i * 512)[lane] = xr[i];
#pragma unroll
            for (int i = 0; i < NB; i++) {
                const int blk = b0 + i;
                if (blk < b1) {
                    const su2 t = tb[i];
                    unsigned short h[8];
#pragma unroll
                    for (int j = 0; j < 8; j++)
                        h[j] = s_raw[blk * 512 + 64 * j + lane + (int)((t[j >> 2] >> (8 * (j & 3))) & 0xffu)];
                    float f[4];
#pragma unroll
                    for (int j = 0; j < 8; j++) s_xs[blk * 512 + 64 * j + lane] = h[j];
#pragma unroll
                    for (int u = 0; u < 4; u++)
                        f[u] = __half2float(__ushort_as_half(h[2 * u])) + __half2float(__ushort_as_half(h[2 * u + 1]));
                    // the block's four unit sums in one pass: the two swaps leave unit 0 | 2 | 1 | 3 in
                    // the four 16-lane rows, the rotations finish each row
                    const float s01 = swap32_add(f[0], f[1]);
                    const float s23 = swap32_add(f[2], f[3]);
                    const float r = row_sum(swap16_add(s01, s23));
                    if (nn == 0) s_xsum[blk * 4 + ((kq >> 1) | ((kq & 1) << 1))] = r;
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
    } else {
        // ---- computing wavefront
        const int cwv = wave - S;
        const int team = cwv / W, cls = cwv % W;
        const __amdgpu_buffer_rsrc_t rt = __builtin_amdgcn_make_buffer_rsrc(
            (void *)(stream + hdr_bytes), 0, (int)min((unsigned long long)ntiles * record_bytes, 0xffffffffull), kSFlags);
        const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc((void *)stream, 0, (int)hdr_bytes, kSFlags);
        uint32_t sc[L / 4];
        su4 wbuf[D];
        su4 cw[4];
        su4 civ[4];
        const bool cherry_wave = cls == W - 1;
        int tcur = bid + G * team;
        bool vcur = tcur < ntiles;
        uint32_t tb = (uint32_t)tcur * record_bytes;
        auto load_cherry = [&](uint32_t base, bool valid) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int lg = 4 * j + kq;
                cw[j] = __builtin_amdgcn_raw_buffer_load_b128(
                    rt, valid && 8 * lg < C ? off_cherry + (uint32_t)(lg * 16 + nn) * 16u : kSOob, base, 2);
            }
        };
        // lane group kq keeps the scales of the units i with i % 4 == kq (every lane group ends up
        // with the same MFMA results, so each finishes a quarter of the units)
        const uint32_t sc_off = (uint32_t)((cls + kq * W) * 32 + nn * 2);
        auto load_scale = [&](int i4, uint32_t base, bool valid) -> uint32_t {
            return __builtin_amdgcn_raw_buffer_load_b16(rt, valid && cls + (4 * i4 + kq) * W < ng ? sc_off : kSOob,
                                                        base + 4 * i4 * W * 32, 0);
        };
        // a unit past the last one of the column, or of a tile that does not exist, reads zeros:
        // the vector offset alone lies outside the descriptor
        const uint32_t w_off = off_units + (uint32_t)(cls * UB + lane * (BITS * 4));
        auto load_unit = [&](int i, uint32_t base, bool valid) -> su4 {
            const uint32_t off = valid && cls + i * W < ng ? w_off : kSOob;
            if constexpr (BITS == 4) {
                return __builtin_amdgcn_raw_buffer_load_b128(rt, off, base + i * W * UB, 2);
            } else {
                const su3 v = __builtin_amdgcn_raw_buffer_load_b96(rt, off, base + i * W * UB, 2);
                return (su4){v[0], v[1], v[2], 0u};
            }
        };
        if (cherry_wave) {
            // the cherry columns of the lane's A operands (positions 32 q + 8 kq + 0..7 of the list) and the rows
#pragma unroll
            for (int q = 0; q < 4; q++)
                civ[q] = __builtin_amdgcn_raw_buffer_load_b128(rh, 32 * q < C ? (uint32_t)(Knp512 + 64 * q + 16 * kq) : kSOob, 0, 0);
            load_cherry(tb, vcur);
        }
#pragma unroll
        for (int i = 0; i < L / 4; i++) sc[i] = load_scale(i, tb, vcur);
#pragma unroll
        for (int i = 0; i < D0; i++) wbuf[i] = load_unit(i, tb, vcur);
        if constexpr (NORM) {
            __builtin_amdgcn_s_barrier();  // (the staging wavefronts exchange their sums of squares)
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
#pragma unroll
        for (int i = D0; i < D; i++) wbuf[i] = load_unit(i, tb, vcur);
        // cherry activations straight from the raw row in LDS; list entries past the last channel
        // name column K, which holds a zero (out-of-range part of the last slice)
        su4 ca[4];
        if (cherry_wave) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                if (32 * q < C) {
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const uint32_t c0 = min(civ[q][j] & 0xffffu, (uint32_t)K), c1 = min(civ[q][j] >> 16, (uint32_t)K);
                        ca[q][j] = (uint32_t)s_raw[c0] | ((uint32_t)s_raw[c1] << 16);
                    }
                }
            }
        }
#pragma unroll 1
        for (int j = 0; j < P; j++) {
            const int tnext = tcur + tstride;
            const bool vnext = tnext < ntiles;
            const uint32_t tbn = (uint32_t)tnext * record_bytes;
            float totc = 0.f;
            if (cherry_wave) {
                sf4_t dc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int q = 0; q < 4; q++)
                    if (32 * q < C) dc = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_h8(ca[q]), as_h8(cw[q]), dc, 0, 0, 0);
                totc = dc[0];
                load_cherry(tbn, vnext);
            }
            float tt = 0.f;
#pragma unroll
            for (int i = 0; i < L; i++) {
                // a unit past the column's last reads zero codes and a zero scale; its activations
                // and unit sum are those of unit 0, which every layer has
                const bool real = cls + i * W < ng;
                const int up = real ? cls + i * W : 0;
                const float sf = (i & 3) == kq ? __half2float(__ushort_as_half((unsigned short)sc[i >> 2])) : 0.f;
                const su4 w = wbuf[i % D];
                const float v = unit_dot<BITS>(w, s_xs + up * kStreamUnitK + 32 * kq);
                wbuf[i % D] = i + D < L ? load_unit(i + D, tb, vcur) : load_unit(i + D - L, tbn, vnext);
                tt += (v + kGrid * s_xsum[up]) * sf;
                if ((i & 3) == 3) sc[i >> 2] = load_scale(i >> 2, tbn, vnext);
            }
            // the four lane groups' quarters
            tt = swap32_add(tt, tt);
            tt = swap16_add(tt, tt) + totc;
            if (kq == 0) s_red[(j * NC + cwv) * 16 + nn] = tt;
            tcur = tnext;
            vcur = vnext;
            tb = tbn;
            if (!vcur) break;
        }
    }

    // ---- across a tile's wavefronts, then one store per output
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    for (int o = tid; o < 16 * P * TEAMS; o += NT) {
        const int jt = o >> 4, j = jt / TEAMS, team = jt - j * TEAMS;
        const int tile = bid + G * (team + TEAMS * j), n = tile * 16 + (o & 15);
        if (tile < ntiles && n < N) {
            float v = 0.f;
#pragma unroll
            for (int c = 0; c < W; c++) v += s_red[(j * NC + team * W + c) * 16 + (o & 15)];
            if (accumulate) v += __half2float(mul[n]);
            mul[n] = __float2half_rn(v);
        }
    }
}

// ---- launch geometries --------------------------------------------------------------------------
// By units per column (W * L must cover them, S * NB * 4 the blocks) and tiles per compute unit
// (one team per tile a compute unit gets, up to three).  Measured, 4-bit / 3-bit us per launch:
// 4096 -> 11008: W4 L8 x 3 teams, D0 = 3, D = 4: 5.60 / 5.08 (D0 2: 5.61 / 5.09; D0 = D = 4: 5.75 / 5.24;
//   D0 4 D 8: 5.96 / 5.41; everything up front, D0 = D = 8: 6.62 / 6.18; W2 L16 x 3: 5.73-5.96);
// 4096 -> 4096: W8 L4 x 1, D0 2 D 4: 3.66 / 3.54 (W4 L8 x 1: 3.74-4.12; 8 staging wavefronts of one block: 3.69);
// 8192 -> 8192: W8 L8 x 1 with 8 staging wavefronts, D0 2 D 4: 7.6 (D0 4 D 8: 7.85; 4 staging wavefronts: 8.2).
struct CuCfg {
    int W, L, TEAMS, S, NB, D0, D;
};
static constexpr CuCfg kCuCfgs[] = {
    {8, 4, 1, 4, 2, 2, 4},  // 0: up to 32 units, at most one tile per compute unit
    {4, 8, 2, 4, 2, 3, 4},  // 1: up to 32 units, up to two tiles per compute unit
    {4, 8, 3, 4, 2, 3, 4},  // 2: up to 32 units, more
    {8, 8, 1, 8, 2, 2, 4},  // 3: up to 64 units
};

static int cu_pick(int ng, int tiles_per_cu_ceil) {
    if (ng <= 32) return tiles_per_cu_ceil <= 1 ? 0 : tiles_per_cu_ceil == 2 ? 1 : 2;
    if (ng <= 64) return 3;
    return -1;
}

static size_t cu_lds_bytes(const StreamGeo &g, const CuCfg &c, int P) {
    const int Knp512 = (g.ng * kStreamUnitK + 511) & ~511;
    size_t need = (size_t)(Knp512 + 512 * c.NB + 8 + Knp512) * 2 + (size_t)(Knp512 / 128) * 4 +
                  (size_t)c.W * c.TEAMS * 16 * 4 * P;
    const size_t alone = 80 * 1024 + 1024;  // more than half of a compute unit's LDS: one workgroup per compute unit
    return need > alone ? need : alone;
}

// Workgroups per member: the launch's compute units are dealt in proportion to the members' tiles.
struct CuSplit {
    int wgs[kStreamMaxGroup], begin[kStreamMaxGroup], total, walk;
};
static CuSplit cu_split(const int *tiles, int count, int teams) {
    CuSplit s = {};
    int all = 0;
    for (int i = 0; i < count; i++) all += tiles[i];
    int left = all < kCuCus ? all : kCuCus;
    if (left < count) left = count;
    int tiles_left = all;
    for (int i = 0; i < count; i++) {
        // proportional share of what is left, at least one workgroup, never more than the member has tiles
        int w = i + 1 == count ? left : (int)(((long long)left * tiles[i] + tiles_left / 2) / (tiles_left > 0 ? tiles_left : 1));
        if (w < 1) w = 1;
        if (w > left - (count - 1 - i)) w = left - (count - 1 - i);
        if (w > tiles[i]) w = tiles[i];
        s.wgs[i] = w;
        s.begin[i] = s.total;
        s.total += w;
        left -= w;
        tiles_left -= tiles[i];
        const int p = ceil_div(tiles[i], w * teams);
        if (p > s.walk) s.walk = p;
    }
    return s;
}

bool stream_cu_supported(int bits, int K, int C, const int *Ns, int count) {
    if (count < 1 || count > kStreamMaxGroup) return false;
    int tiles[kStreamMaxGroup], all = 0;
    for (int i = 0; i < count; i++) {
        tiles[i] = ceil_div(Ns[i], kStreamTileCols);
        all += tiles[i];
    }
    const StreamGeo geo = stream_geo(bits, K, Ns[0], C);
    const int idx = cu_pick(geo.ng, ceil_div(all, kCuCus));
    if (idx < 0) return false;
    const CuCfg &c = kCuCfgs[idx];
    if (geo.ng > c.W * c.L || geo.ng * kStreamUnitK > c.S * c.NB * 512 || C > 128) return false;
    const CuSplit sp = cu_split(tiles, count, c.TEAMS);
    if (sp.walk > kCuMaxWalk) return false;
    return cu_lds_bytes(geo, c, sp.walk) <= 160 * 1024;
}

template <int BITS, int I, bool NORM, bool GROUP>
static hipError_t launch_cu_cfg(const __half *vec, const __half *norm_w, float eps, const StreamMember *members, int count,
                                const StreamGeo &geo, const CuSplit &sp, int accumulate, hipStream_t s) {
    constexpr CuCfg c = kCuCfgs[I];
    auto kern = stream_cu_kernel<BITS, c.W, c.L, c.TEAMS, c.S, c.NB, c.D0, c.D, NORM, GROUP>;
    const size_t lds = cu_lds_bytes(geo, c, sp.walk);
    {
        // per instantiation and device, once: the dynamic-LDS limit raised
        static std::mutex mu;
        static bool raised[kCuMaxDevices] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kCuMaxDevices) return hipErrorInvalidDevice;
        std::lock_guard<std::mutex> lock(mu);
        if (!raised[dev]) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return e;
            raised[dev] = true;
        }
    }
    CuGroup g = {};
    g.count = count;
    for (int i = 1; i < kStreamMaxGroup; i++) {
        const StreamMember &m = members[i < count ? i : 0];
        g.stream[i - 1] = m.stream;
        g.mul[i - 1] = m.mul;
        g.N[i - 1] = m.N;
        g.wg_begin[i - 1] = i < count ? sp.begin[i] : 0x7fffffff;
        g.wgs[i - 1] = i < count ? sp.wgs[i] : 1;
    }
    hipLaunchKernelGGL(kern, dim3(sp.total), dim3(64 * (c.W * c.TEAMS + c.S)), lds, s, vec, members[0].stream, members[0].mul,
                       geo.K, geo.C, geo.ng, members[0].N, geo.hdr_bytes, geo.off_cherry, geo.off_units, geo.record_bytes,
                       sp.wgs[0], accumulate, norm_w, eps, g);
    return hipGetLastError();
}

// `count` layers of the same bits / K / C that read the same activation row, in one launch;
// norm_w != nullptr fuses the RMSNorm of that row.  The caller has asked stream_cu_supported().
hipError_t launch_stream_cu(int bits, const __half *vec, const __half *norm_w, float eps, const StreamMember *members,
                            int count, int K, int C, int accumulate, hipStream_t s) {
    if (count < 1 || count > kStreamMaxGroup) return hipErrorInvalidValue;
    int tiles[kStreamMaxGroup], all = 0;
    for (int i = 0; i < count; i++) {
        tiles[i] = ceil_div(members[i].N, kStreamTileCols);
        all += tiles[i];
    }
    const StreamGeo geo = stream_geo(bits, K, members[0].N, C);
    const int idx = cu_pick(geo.ng, ceil_div(all, kCuCus));
    if (idx < 0) return hipErrorInvalidValue;
    const CuSplit sp = cu_split(tiles, count, kCuCfgs[idx].TEAMS);
    if (sp.walk > kCuMaxWalk) return hipErrorInvalidValue;
#define CQ_CU_GO(BITS_, I_)                                                                                          \
    do {                                                                                                             \
        if (norm_w) {                                                                                                \
            return count > 1 ? launch_cu_cfg<BITS_, I_, true, true>(vec, norm_w, eps, members, count, geo, sp, accumulate, s)   \
                             : launch_cu_cfg<BITS_, I_, true, false>(vec, norm_w, eps, members, count, geo, sp, accumulate, s); \
        }                                                                                                            \
        return count > 1 ? launch_cu_cfg<BITS_, I_, false, true>(vec, nullptr, 0.f, members, count, geo, sp, accumulate, s)     \
                         : launch_cu_cfg<BITS_, I_, false, false>(vec, nullptr, 0.f, members, count, geo, sp, accumulate, s);   \
    } while (0)
#define CQ_CU_BITS(BITS_)            \
    switch (idx) {                   \
        case 0: CQ_CU_GO(BITS_, 0);  \
        case 1: CQ_CU_GO(BITS_, 1);  \
        case 2: CQ_CU_GO(BITS_, 2);  \
        default: CQ_CU_GO(BITS_, 3); \
    }
    if (bits == 4) CQ_CU_BITS(4)
    CQ_CU_BITS(3)
#undef CQ_CU_BITS
#undef CQ_CU_GO
}

}  // namespace cq
