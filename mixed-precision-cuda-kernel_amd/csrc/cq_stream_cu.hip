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

constexpr int kCuPlain = 0, kCuNorm = 1, kCuGate = 2, kCuAttn = 3;
constexpr int kCuAttnSlices = 4;  // slices of a split attention that the kCuAttn prologue combines

// fp16(silu(gate)) * up, rounded to fp16, on both halves of a pair (the rounding points of silu_mul_kernel)
__device__ inline uint32_t cu_silu_mul_pair(uint32_t gate, uint32_t up) {
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

// What a workgroup works on, gathered from the kernel arguments by the two kernel shells below.
struct CuJob {
    const __half *x;
    const uint8_t *stream;  // the layer's stream (header, then tile records)
    __half *mul;
    const __half *norm_w;   // kCuNorm: the norm weight; kCuGate: the gate vector; kCuAttn: the slices' (maximum, sum) pairs
    float eps;
    int K, C, N;
    int G, bid;             // workgroups that share the layer, this one's index among them
    int accumulate, P;      // P: tiles the launch's busiest team walks
    const uint8_t *stream2, *stream3;  // MEM > 1: the second and third layer's stream
    __half *mul2, *mul3;               // ... and output
};

constexpr int kCuSeparate = 0, kCuSiluPair = 1;  // epilogues: every layer's result | fp16(fp16(silu(layer 0)) * layer 1)

// S staging wavefronts (wavefronts 0 .. S-1, NB blocks of 512 compacted positions each), then
// TEAMS teams of W computing wavefronts; computing wavefront c of a team takes the units c, c + W,
// ... (L at most) of every tile the team comes to.  WALK: some team has more than one tile.
// PRO: what the staging wavefronts do to the row on its way into LDS -- kCuPlain nothing,
// kCuNorm the RMSNorm norm_w * fp16(x * rsqrt(mean(x^2) + eps)), kCuGate the gated-MLP activation
// fp16(fp16(silu(gate)) * x) with the gate vector passed in the norm_w slot, kCuAttn the row
// formed from the partial results of an attention dealt to kCuAttnSlices workgroups per head
// (rope_attn_split_kernel): x holds [slices][K] fp16 partial results, the norm_w slot
// [slices][K / 128][2] floats, the row is fp16(sum_s c_s * partial_s) with attn_combine_weights()
// (the arithmetic of attn_combine_kernel, for an output projection that reads the heads' results).
// MEM > 1: MEM layers of the same shape that read the same row share a workgroup (2: gate_proj /
// up_proj, 3: q / k / v of equal widths): team t works on layer t % MEM, on the same tile index as
// the other teams of its slot t / MEM, so the tiles of all layers spread evenly over the compute
// units; each layer's compaction is staged by S / MEM of the staging wavefronts (the layers keep
// different cherry channels).  EPI: kCuSeparate stores every layer's result, kCuSiluPair (MEM 2)
// fp16(fp16(silu(layer 0)) * layer 1) of the two rounded results instead.
// EXTRA (one layer per workgroup, S == W, no walking): a workgroup whose compute unit gets one tile
// more than it has teams hands that tile to its staging wavefronts, which work on it as one more
// team once the row is staged.  q / k / v of 4096 columns each are 3 x 256 tiles on 85 / 85 / 86
// workgroups of three teams: 255 slots for 256 tiles, so one team of a member walked a second
// tile and the launch carried the walking code (7.23 us against 6.17 us for 3 x 255 tiles).
template <int BITS, int W, int L, int TEAMS, int S, int NB, int D0, int D, int PRO, bool WALK, int MEM = 1, int EPI = kCuSeparate,
          bool EXTRA = false>
__device__ __forceinline__ void stream_cu_body(const CuJob &job) {
    constexpr int NC = W * TEAMS;  // computing wavefronts
    constexpr int NCX = NC + (EXTRA ? S : 0);  // ... and the staging wavefronts when they take a tile of their own
    static_assert(!EXTRA || (S == W && MEM == 1 && !WALK && EPI == kCuSeparate), "the staging wavefronts as one more team");
    constexpr int NT = 64 * (NC + S);
    constexpr int UB = BITS == 4 ? 1024 : 768;
    constexpr float kGrid = BITS == 4 ? -7.5f : -3.5f;
    constexpr int XS = NB + 1;  // 16-byte loads per lane that cover a staging wavefront's raw slice
    static_assert(D0 <= D && D <= L && L % D == 0 && L % 4 == 0, "ring slots are fixed per unit across tiles");
    static_assert(MEM >= 1 && MEM <= 3 && TEAMS % MEM == 0 && S % MEM == 0 && (MEM == 1 || PRO != kCuGate), "teams and staging wavefronts per layer");
    static_assert(EPI == kCuSeparate || MEM == 2, "");
    constexpr int SM = S / MEM;            // staging wavefronts per layer
    constexpr int TSLOTS = TEAMS / MEM;    // tiles a workgroup works on at a time
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kq = lane >> 4, nn = lane & 15;
    const int K = job.K, C = job.C, N = job.N, G = job.G, bid = job.bid;
    // the layers' streams, pinned in scalar registers so that picking one by a wavefront's layer
    // stays a scalar select (left alone the compiler builds a table in scratch memory and indexes
    // it: a kernel with scratch launches microseconds slower and starts with a memory round trip)
    const uint8_t *st0 = job.stream, *st1 = MEM > 1 ? job.stream2 : job.stream, *st2 = MEM > 2 ? job.stream3 : job.stream;
    if constexpr (MEM > 1) asm volatile("" : "+s"(st0), "+s"(st1), "+s"(st2));
    auto stream_of = [&](int m) -> const uint8_t * { return MEM > 2 && m == 2 ? st2 : MEM > 1 && m == 1 ? st1 : st0; };
    // the record geometry of stream_geo(), from the shape (scalar arithmetic: cheaper than
    // kernel arguments that would not fit the preloaded ones)
    const int ng = (K - C + kStreamUnitK - 1) / kStreamUnitK;
    const int Knp512 = (ng * kStreamUnitK + 511) & ~511;
    const int nblk = Knp512 >> 9;
    const uint32_t off_cherry = ((uint32_t)ng * 32u + 255u) & ~255u;
    const uint32_t off_units = off_cherry + (((uint32_t)C * 32u + 255u) & ~255u);
    const uint32_t record_bytes = off_units + (uint32_t)ng * UB;
    const uint32_t hdr_bytes = ((uint32_t)(Knp512 + 2 * ((C + 31) & ~31)) + 255u) & ~255u;
    const int ntiles = (N + kStreamTileCols - 1) / kStreamTileCols;
    // LDS: raw activations (slice by slice, zeros past the row) | compacted activations | unit sums | partial outputs
    unsigned short *s_raw = reinterpret_cast<unsigned short *>(smem);
    unsigned short *s_xs = s_raw + Knp512 + 512 * NB + 8;                   // [MEM][Knp512]
    float *s_xsum = reinterpret_cast<float *>(s_xs + MEM * Knp512);         // [MEM][4 nblk]
    float *s_red = s_xsum + MEM * 4 * nblk;
    const int tstride = G * TSLOTS;

    // ---- a team's wavefront at work: wavefront `cls` of the team whose partial sums go to row `cwv` of
    // s_red, on tile slot `slot` of layer `mem`.  AFTER: called behind the workgroup barrier (the staging
    // wavefronts as one more team): no barrier inside, one tile.
    auto team_work = [&](auto after_tag, const int cwv, const int slot, const int cls, const int mem) {
        constexpr bool AFTER = decltype(after_tag)::value;
        const uint8_t *__restrict__ stream = stream_of(mem);
        const unsigned short *xs_m = s_xs + mem * Knp512;
        const float *xsum_m = s_xsum + mem * 4 * nblk;
        const __amdgpu_buffer_rsrc_t rt = __builtin_amdgcn_make_buffer_rsrc(
            (void *)(stream + hdr_bytes), 0, (int)min((unsigned long long)ntiles * record_bytes, 0xffffffffull), kSFlags);
        const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc((void *)stream, 0, (int)hdr_bytes, kSFlags);
        uint32_t sc[L / 4];
        su4 wbuf[D];
        su4 cw[4];
        su4 civ[4];
        const bool cherry_wave = cls == W - 1;
        constexpr bool WALKX = WALK && !AFTER;
        int tcur = bid + G * slot;
        bool vcur = tcur < ntiles;
        uint32_t tb = (uint32_t)tcur * record_bytes;
        auto load_cherry = [&](uint32_t base, bool valid) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int lg = 4 * j + kq;
                if (32 * j < C)
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
        // The barrier at which the staging wavefronts exchange their sums of squares (kCuNorm) opens
        // when every wavefront's requests so far have been ACCEPTED by the compute unit.  With several
        // layers per workgroup (two staging wavefronts per layer, four blocks each) the computing
        // wavefronts pass it before they request anything: RMSNorm + gate/up + SiLU 10.25 -> 9.92 us;
        // with one layer per workgroup the same order is slower (gate/up as a group 9.94 -> 10.43 us).
        constexpr bool kNormFirst = PRO == kCuNorm && MEM > 1;
        if constexpr (kNormFirst && !AFTER) __builtin_amdgcn_s_barrier();
        if (cherry_wave) {
            // the cherry columns of the lane's A operands (positions 32 q + 8 kq + 0..7 of the list) and the rows
#pragma unroll
            for (int q = 0; q < 4; q++)
                if (32 * q < C) civ[q] = __builtin_amdgcn_raw_buffer_load_b128(rh, (uint32_t)(Knp512 + 64 * q + 16 * kq), 0, 0);
            load_cherry(tb, vcur);
        }
#pragma unroll
        for (int i = 0; i < L / 4; i++) sc[i] = load_scale(i, tb, vcur);
#pragma unroll
        for (int i = 0; i < D0; i++) wbuf[i] = load_unit(i, tb, vcur);
        if constexpr (!AFTER) {
            if constexpr (PRO == kCuNorm && !kNormFirst) {
                __builtin_amdgcn_s_barrier();  // (the staging wavefronts exchange their sums of squares)
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
            __builtin_amdgcn_s_barrier();
        }
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
        const int P = WALKX ? job.P : 1;
#pragma unroll 1
        for (int j = 0; j < P; j++) {
            const int tnext = tcur + tstride;
            const bool vnext = WALKX && tnext < ntiles;
            const uint32_t tbn = (uint32_t)tnext * record_bytes;
            float totc = 0.f;
            if (cherry_wave) {
                sf4_t dc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int q = 0; q < 4; q++)
                    if (32 * q < C) dc = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_h8(ca[q]), as_h8(cw[q]), dc, 0, 0, 0);
                totc = dc[0];
                if constexpr (WALKX) load_cherry(tbn, vnext);
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
                const float v = unit_dot<BITS>(w, xs_m + up * kStreamUnitK + 32 * kq);
                if (i + D < L) wbuf[i % D] = load_unit(i + D, tb, vcur);
                else if constexpr (WALKX) wbuf[i % D] = load_unit(i + D - L, tbn, vnext);
                tt += (v + kGrid * xsum_m[up]) * sf;
                if constexpr (WALKX) {
                    if ((i & 3) == 3) sc[i >> 2] = load_scale(i >> 2, tbn, vnext);
                }
            }
            // the four lane groups' quarters
            tt = swap32_add(tt, tt);
            tt = swap16_add(tt, tt) + totc;
            if (kq == 0) s_red[(j * NCX + cwv) * 16 + nn] = tt;
            tcur = tnext;
            vcur = vnext;
            tb = tbn;
            if (!vcur) break;
        }
    };

    if (wave < S) {
        // ---- staging wavefront: its slice of the row, its blocks' gather table; gather; unit sums
        __builtin_amdgcn_s_setprio(3);
        const int mem = MEM > 1 ? wave / SM : 0, ws = wave - mem * SM;   // the layer it stages for, its index among that layer's
        const int b0 = ws * NB, b1 = min(nblk, b0 + NB);
        const bool active = b0 < nblk, last = active && b1 == nblk;
        const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)job.x, 0, K * 2, kSFlags);
        const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc((void *)stream_of(mem), 0,
                                                                            (int)hdr_bytes, kSFlags);
        unsigned short *xs_m = s_xs + mem * Knp512;
        float *xsum_m = s_xsum + mem * 4 * nblk;
        su4 xr[XS];
        su2 tb[NB];
#pragma unroll
        for (int i = 0; i < XS; i++)
            xr[i] = __builtin_amdgcn_raw_buffer_load_b128(rx, active ? (uint32_t)(b0 * 512 + i * 512 + lane * 8) * 2u : kSOob, 0, 0);
#pragma unroll
        for (int i = 0; i < NB; i++)
            tb[i] = __builtin_amdgcn_raw_buffer_load_b64(rh, b0 + i < b1 ? (uint32_t)((b0 + i) * 512 + lane * 8) : kSOob, 0, 0);
        if constexpr (PRO == kCuGate) {
            su4 gr[XS];
            const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc((void *)job.norm_w, 0, K * 2, kSFlags);
#pragma unroll
            for (int i = 0; i < XS; i++)
                gr[i] = __builtin_amdgcn_raw_buffer_load_b128(rg, active ? (uint32_t)(b0 * 512 + i * 512 + lane * 8) * 2u : kSOob, 0, 0);
#pragma unroll
            for (int i = 0; i < XS; i++) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    xr[i][j] = cu_silu_mul_pair(gr[i][j], xr[i][j]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        if constexpr (PRO == kCuAttn) {
            su4 pr[kCuAttnSlices - 1][XS];
            su2 mlr[kCuAttnSlices][XS];
            const int heads = K >> 7;
            const __amdgpu_buffer_rsrc_t rm = __builtin_amdgcn_make_buffer_rsrc((void *)job.norm_w, 0, kCuAttnSlices * heads * 8, kSFlags);
#pragma unroll
            for (int sl = 1; sl < kCuAttnSlices; sl++) {
                const __amdgpu_buffer_rsrc_t rp = __builtin_amdgcn_make_buffer_rsrc((void *)(job.x + (size_t)sl * K), 0, K * 2, kSFlags);
#pragma unroll
                for (int i = 0; i < XS; i++)
                    pr[sl - 1][i] = __builtin_amdgcn_raw_buffer_load_b128(rp, active ? (uint32_t)(b0 * 512 + i * 512 + lane * 8) * 2u : kSOob, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < XS; i++) {
                const int col = b0 * 512 + i * 512 + lane * 8;
#pragma unroll
                for (int sl = 0; sl < kCuAttnSlices; sl++)
                    mlr[sl][i] = __builtin_amdgcn_raw_buffer_load_b64(rm, active && col < K ? (uint32_t)(sl * heads + (col >> 7)) * 8u : kSOob, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < XS; i++) {
                float mv[kCuAttnSlices], lv[kCuAttnSlices], cf[kCuAttnSlices];
#pragma unroll
                for (int sl = 0; sl < kCuAttnSlices; sl++) {
                    mv[sl] = __uint_as_float(mlr[sl][i][0]);
                    lv[sl] = __uint_as_float(mlr[sl][i][1]);
                }
                attn_combine_weights(mv, lv, cf);
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    uint32_t r = 0;
#pragma unroll
                    for (int hf = 0; hf < 2; hf++) {
                        float o = fmaf(cf[0], __half2float(__ushort_as_half((unsigned short)(xr[i][j] >> (16 * hf)))), 0.f);
#pragma unroll
                        for (int sl = 1; sl < kCuAttnSlices; sl++)
                            o = fmaf(cf[sl], __half2float(__ushort_as_half((unsigned short)(pr[sl - 1][i][j] >> (16 * hf)))), o);
                        r |= (uint32_t)__half_as_ushort(__float2half_rn(o)) << (16 * hf);
                    }
                    xr[i][j] = r;
                }
            }
        }
        if constexpr (PRO == kCuNorm) {
            su4 nr[XS];
            const __amdgpu_buffer_rsrc_t rn = __builtin_amdgcn_make_buffer_rsrc((void *)job.norm_w, 0, K * 2, kSFlags);
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
            float t = 0.f;   // (with two layers each layer's staging wavefronts cover the whole row: the first layer's sums)
#pragma unroll
            for (int wv = 0; wv < SM; wv++) t += s_red[wv];
            const float rs = rsqrtf(t / (float)K + job.eps);
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
                    for (int j = 0; j < 8; j++) xs_m[blk * 512 + 64 * j + lane] = h[j];
#pragma unroll
                    for (int u = 0; u < 4; u++)
                        f[u] = __half2float(__ushort_as_half(h[2 * u])) + __half2float(__ushort_as_half(h[2 * u + 1]));
                    // the block's four unit sums in one pass: the two swaps leave unit 0 | 2 | 1 | 3 in
                    // the four 16-lane rows, the rotations finish each row
                    const float s01 = swap32_add(f[0], f[1]);
                    const float s23 = swap32_add(f[2], f[3]);
                    const float r = row_sum(swap16_add(s01, s23));
                    if (nn == 0) xsum_m[blk * 4 + ((kq >> 1) | ((kq & 1) << 1))] = r;
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        if constexpr (EXTRA) {
            // one more tile for this compute unit than it has teams: the staging wavefronts take it
            if (bid + G * TEAMS < ntiles) team_work(std::true_type{}, NC + wave, TEAMS, wave, 0);
        }
    } else {
        // ---- computing wavefront
        const int cwv = wave - S;
        const int team = cwv / W, cls = cwv % W;
        const int mem = MEM > 1 ? team % MEM : 0, slot = MEM > 1 ? team / MEM : team;   // the team's layer, its tile slot
        team_work(std::false_type{}, cwv, slot, cls, mem);
    }

    // ---- across a tile's wavefronts, then one store per output
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    const int P = WALK ? job.P : 1;
    constexpr int OUTS = EPI == kCuSiluPair ? TSLOTS : TEAMS + (EXTRA ? 1 : 0);   // 16-column pieces of output per walk step
    __half *mu0 = job.mul, *mu1 = MEM > 1 ? job.mul2 : job.mul, *mu2 = MEM > 2 ? job.mul3 : job.mul;
    if constexpr (MEM > 1) asm volatile("" : "+s"(mu0), "+s"(mu1), "+s"(mu2));
    for (int o = tid; o < 16 * P * OUTS; o += NT) {
        const int jt = o >> 4, j = jt / OUTS, t = jt - j * OUTS, col = o & 15;
        const int slot = EPI == kCuSiluPair ? t : t / MEM, mem = EPI == kCuSiluPair ? 0 : t - slot * MEM;
        const int tile = bid + G * (slot + TSLOTS * j), n = tile * 16 + col;
        if (tile < ntiles && n < N) {
            const float *red = s_red + (j * NCX + (slot * MEM + mem) * W) * 16 + col;
            if constexpr (EPI == kCuSiluPair) {
                float g = 0.f, u = 0.f;
#pragma unroll
                for (int c = 0; c < W; c++) {
                    g += red[c * 16];
                    u += red[(W + c) * 16];
                }
                // the two projections' results as they would be stored, then the activation of silu_mul_kernel
                const float g16 = __half2float(__float2half_rn(g)), u16 = __half2float(__float2half_rn(u));
                const float a = __half2float(__float2half_rn(g16 / (1.f + __expf(-g16))));
                mu0[n] = __float2half_rn(a * u16);
            } else {
                float v = 0.f;
#pragma unroll
                for (int c = 0; c < W; c++) v += red[c * 16];
                __half *__restrict__ mul = MEM > 2 && mem == 2 ? mu2 : MEM > 1 && mem == 1 ? mu1 : mu0;  // (per-lane select: vector registers)
                if (job.accumulate) v += __half2float(mul[n]);
                mul[n] = __float2half_rn(v);
            }
        }
    }
}

// The file is built with a kernel-argument preload count of 14 dwords: the dispatcher puts the
// leading arguments into scalar registers before a wavefront starts, so nothing that a
// wavefront's first requests depend on waits for a load from the argument segment (which costs
// most of a microsecond).  Both shells are laid out for that.

// one layer: x, stream, mul, K, C, N, workgroups, accumulate, P = 12 dwords
template <int BITS, int W, int L, int TEAMS, int S, int NB, int D0, int D, bool WALK>
__global__ __launch_bounds__(64 * (W * TEAMS + S)) void stream_cu_kernel(const __half *__restrict__ x,
                                                                          const uint8_t *__restrict__ stream,
                                                                          __half *__restrict__ mul, int K, int C, int N,
                                                                          int wgs, int accumulate, int P) {
    const CuJob job = {x, stream, mul, nullptr, 0.f, K, C, N, wgs, (int)blockIdx.x, accumulate, P, nullptr, nullptr, nullptr, nullptr};
    stream_cu_body<BITS, W, L, TEAMS, S, NB, D0, D, kCuPlain, WALK>(job);
}

// Up to three layers that read the same row (q / k / v, gate / up), consecutive ranges of
// workgroups per layer, optionally behind the fused RMSNorm or the gated-MLP activation (one
// layer then: the down projection).  Leading 14 dwords: x, norm_w (or the gate vector), the
// three streams, then packed K | C << 16, N0/8 | N1/8 << 16, N2/8 | P << 16 | accumulate << 31,
// first workgroup of member 1 | of member 2 << 10 | all workgroups << 20.
struct CuGroupTail {
    __half *mul[kStreamMaxGroup];
    float eps;
};
template <int BITS, int W, int L, int TEAMS, int S, int NB, int D0, int D, int PRO, bool WALK, bool EXTRA = false>
__global__ __launch_bounds__(64 * (W * TEAMS + S)) void stream_cu_group_kernel(
    const __half *__restrict__ x, const __half *__restrict__ norm_w, const uint8_t *__restrict__ stream0,
    const uint8_t *__restrict__ stream1, const uint8_t *__restrict__ stream2, uint32_t kc, uint32_t n01, uint32_t n2p,
    uint32_t wgb, CuGroupTail tail) {
    // the candidates are pinned in scalar registers first so that the selects stay selects (and do
    // not become one load at a selected argument address)
    const uint8_t *s0 = stream0, *s1 = stream1, *s2 = stream2;
    asm volatile("" : "+s"(s0), "+s"(s1), "+s"(s2));
    const int bid = blockIdx.x;
    const int b1 = (int)(wgb & 1023u), b2 = (int)((wgb >> 10) & 1023u), total = (int)(wgb >> 20);
    const bool m1 = bid >= b1, m2 = bid >= b2;  // (absent members start at `total`)
    __half *o0 = tail.mul[0], *o1 = tail.mul[1], *o2 = tail.mul[2];
    asm volatile("" : "+s"(o0), "+s"(o1), "+s"(o2));
    CuJob job;
    job.x = x;
    job.norm_w = norm_w;
    job.eps = tail.eps;
    job.stream = m2 ? s2 : m1 ? s1 : s0;
    job.mul = m2 ? o2 : m1 ? o1 : o0;
    job.K = (int)(kc & 0xffffu);
    job.C = (int)(kc >> 16);
    job.N = 8 * (int)(m2 ? (n2p & 0xffffu) : m1 ? (n01 >> 16) : (n01 & 0xffffu));
    job.G = m2 ? total - b2 : m1 ? b2 - b1 : b1;
    job.bid = bid - (m2 ? b2 : m1 ? b1 : 0);
    job.accumulate = (int)(n2p >> 31);
    job.P = (int)((n2p >> 16) & 0x7fffu);
    job.stream2 = job.stream3 = nullptr;
    job.mul2 = job.mul3 = nullptr;
    stream_cu_body<BITS, W, L, TEAMS, S, NB, D0, D, PRO, WALK, 1, kCuSeparate, EXTRA>(job);
}

// MEM = 2 or 3 layers of the SAME shape that read the same row, every workgroup working on the same
// columns of all of them.  EPI = kCuSiluPair (MEM 2): gate_proj and up_proj of a gated MLP, storing
// the activation fp16(fp16(silu(gate)) * up) that the down projection reads
// (llama/modeling_llama_quant.py:251) into mul[0] instead of the two results.  EPI = kCuSeparate
// with MEM 3 was measured for q / k / v and not kept.  Leading 14 dwords: x, norm_w, three streams, K | C << 16, N,
// workgroups | P << 16, eps; the outputs behind them.
struct CuMultiTail {
    __half *mul[kStreamMaxGroup];
};
template <int BITS, int W, int L, int TEAMS, int S, int NB, int D0, int D, int PRO, bool WALK, int MEM, int EPI>
__global__ __launch_bounds__(64 * (W * TEAMS + S)) void stream_cu_multi_kernel(
    const __half *__restrict__ x, const __half *__restrict__ norm_w, const uint8_t *__restrict__ stream0,
    const uint8_t *__restrict__ stream1, const uint8_t *__restrict__ stream2, uint32_t kc, int N, uint32_t wgs_p, float eps,
    CuMultiTail tail) {
    const CuJob job = {x, stream0, tail.mul[0], norm_w, eps, (int)(kc & 0xffffu), (int)(kc >> 16), N, (int)(wgs_p & 0xffffu),
                       (int)blockIdx.x, 0, (int)(wgs_p >> 16), stream1, stream2, tail.mul[1], tail.mul[2]};
    stream_cu_body<BITS, W, L, TEAMS, S, NB, D0, D, PRO, WALK, MEM, EPI>(job);
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
    {8, 4, 1, 4, 2, 2, 4},   // 0: up to 32 units, at most one tile per compute unit
    {4, 8, 2, 4, 2, 3, 4},   // 1: up to 32 units, up to two tiles per compute unit
    {4, 8, 3, 4, 2, 3, 4},   // 2: up to 32 units, more
    {8, 8, 1, 8, 2, 2, 4},   // 3: up to 64 units
    {11, 8, 1, 5, 5, 3, 4},  // 4: up to 88 units (11008 input channels)
    {8, 16, 1, 8, 4, 4, 8},  // 5: up to 128 units
    {8, 28, 1, 8, 7, 4, 7},  // 6: up to 224 units (28672 input channels)
    {5, 8, 2, 6, 2, 3, 4},   // 7: up to 40 units (5120 input channels), two teams
    {4, 28, 2, 8, 4, 4, 7},  // 8: up to 112 units (13824 input channels), two tiles per compute unit
    {12, 8, 1, 4, 6, 3, 4},  // 9: up to 96 units, one team of 12 (12288 -> 4096: 6.5 / 6.1 us against 7.2 / 6.7 for entry 5)
    {4, 12, 3, 4, 3, 3, 4},  // 10: up to 48 units, three teams and the staging wavefronts as a fourth (5120 -> 13824)
};
// entries whose staging wavefronts can work as one more team (as many of them as a team has wavefronts)
constexpr bool cu_cfg_extra(int i) { return kCuCfgs[i].S == kCuCfgs[i].W; }
// The LLaMA-13B widths (entries 7 and 8), us per launch, 4-bit / 3-bit, against the checkpoint layout's
// 5.87 / 5.57 (5120 -> 5120), 10.15 / 8.80 (5120 -> 13824), 10.24 / 8.81 (13824 -> 5120):
// 5120 -> 5120 (320 tiles): entry 7 4.52 / 4.65 (entry 3: 6.0 / 6.0; three teams of 4 x 12 units 5.4 / 5.9;
//   four teams of 3 x 16 units 6.2 / 6.5);
// 5120 -> 13824 (864 tiles): entry 7, teams walking two tiles, 8.2-8.3 / 8.1-8.2 (four teams of 3 x 16
//   units without walking 8.0 / 8.2 with a ring of 4, 9.0 / 8.7 with a ring of 8; 4 x 12 units x 3 teams
//   8.8 / 8.3; 2 x 20 units x 6 teams 8.6-8.8 / 8.8);
// 13824 -> 5120 (320 tiles of 108 units): entry 8 9.2 / 8.95 (entry 5, walking: 10.3; 6 x 20 units x 2
//   teams with 4 staging wavefronts 9.6 / 9.4; 7 x 16 units and 2 staging wavefronts of 14 blocks 11.7 / 11.6).
// Deep columns (entries 4 to 6) are the same kernel with more units per wavefront and more
// blocks per staging wavefront; the barrier then opens later (staging 22 blocks takes 1.3 us
// instead of 0.5), which the D0 units requested in front of it cover.  Measured: 11008 -> 4096
// 7.04 us on the checkpoint layout -> 5.93 (3-bit 6.76 -> 5.57; with 8 x 12 units and 8 staging
// wavefronts 6.01 / 5.59); 28672 -> 8192 23.5 -> 22.0; 13824 -> 5120 (3-bit, 320 tiles on 256
// compute units: a quarter of them walk two tiles) 10.2 against 8.93, so that shape stays on the
// checkpoint layout.
// (While a 3-bit unit still ended in two 16x16x16 MFMAs chained onto 16x16x32 results, tile-walking
// 3-bit instantiations with more than 8 units per wavefront and a short ring -- L = 12 or 16 with
// D = 4, L = 20 with D = 2, 4 or 5 -- returned wrong sums; unit_dot() explains.  The parity tests run
// every entry in both bit widths, with and without walking.)

constexpr int kCuAttnMaxCfg = 3;  // the attention-combining prologue exists for entries 0 .. 3 (output projections up to 64 units)

static int cu_pick(int ng, int tiles_per_cu_ceil) {
    if (ng <= 32) return tiles_per_cu_ceil <= 1 ? 0 : tiles_per_cu_ceil == 2 ? 1 : 2;
    if (ng <= 48 && tiles_per_cu_ceil >= 3 && tiles_per_cu_ceil <= 4) return 10;
    if (ng <= 40) return 7;
    if (ng <= 64) return 3;
    if (ng <= 88) return 4;
    if (ng <= 96) return 9;
    if (ng <= 112 && tiles_per_cu_ceil == 2) return 8;
    if (ng <= 128) return 5;
    if (ng <= 224) return 6;
    return -1;
}

static size_t cu_lds_bytes(const StreamGeo &g, const CuCfg &c, int P, int layers = 1) {
    const int Knp512 = (g.ng * kStreamUnitK + 511) & ~511;
    size_t need = (size_t)(Knp512 + 512 * c.NB + 8 + layers * Knp512) * 2 + (size_t)layers * (Knp512 / 128) * 4 +
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
    for (int i = 0; i < count; i++)
        if (Ns[i] % 8 || Ns[i] / 8 > 0xffff) return false;
    if (K > 0xffff || sp.total > 1023) return false;
    return cu_lds_bytes(geo, c, sp.walk) <= 160 * 1024;
}

// an output projection that forms its input row from split-attention partial results
bool stream_attn_out_supported(int bits, int K, int C, int N) {
    const int Ns[1] = {N};
    if (K % 128 || !stream_cu_supported(bits, K, C, Ns, 1)) return false;
    const StreamGeo geo = stream_geo(bits, K, N, C);
    return cu_pick(geo.ng, ceil_div(geo.ntiles, kCuCus)) <= kCuAttnMaxCfg;
}

template <typename KERN>
static hipError_t cu_raise_lds(KERN kern, bool *raised) {
    // per instantiation and device, once: the dynamic-LDS limit raised
    static std::mutex mu;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kCuMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mu);
    if (!raised[dev]) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        raised[dev] = true;
    }
    return hipSuccess;
}

template <int BITS, int I, int PRO, bool GROUP, bool WALK, bool EXTRA = false>
static hipError_t launch_cu_cfg(const __half *vec, const __half *norm_w, float eps, const StreamMember *members, int count,
                                const StreamGeo &geo, const CuSplit &sp, int accumulate, hipStream_t s) {
    constexpr CuCfg c = kCuCfgs[I];
    const size_t lds = cu_lds_bytes(geo, c, sp.walk) + (EXTRA ? (size_t)c.S * 16 * 4 : 0);
    const dim3 grid(sp.total), block(64 * (c.W * c.TEAMS + c.S));
    static bool raised[kCuMaxDevices] = {};
    if constexpr (!GROUP) {
        auto kern = stream_cu_kernel<BITS, c.W, c.L, c.TEAMS, c.S, c.NB, c.D0, c.D, WALK>;
        if (hipError_t e = cu_raise_lds(kern, raised)) return e;
        hipLaunchKernelGGL(kern, grid, block, lds, s, vec, members[0].stream, members[0].mul, geo.K, geo.C, members[0].N,
                           sp.wgs[0], accumulate, sp.walk);
    } else {
        auto kern = stream_cu_group_kernel<BITS, c.W, c.L, c.TEAMS, c.S, c.NB, c.D0, c.D, PRO, WALK, EXTRA>;
        if (hipError_t e = cu_raise_lds(kern, raised)) return e;
        CuGroupTail tail = {};
        const uint8_t *st[kStreamMaxGroup];
        uint32_t n8[kStreamMaxGroup], begin[kStreamMaxGroup];
        for (int i = 0; i < kStreamMaxGroup; i++) {
            const StreamMember &m = members[i < count ? i : 0];
            st[i] = m.stream;
            tail.mul[i] = m.mul;
            n8[i] = (uint32_t)(m.N / 8);
            begin[i] = (uint32_t)(i < count ? sp.begin[i] : sp.total);
        }
        tail.eps = eps;
        const uint32_t kc = (uint32_t)geo.K | ((uint32_t)geo.C << 16);
        const uint32_t n01 = n8[0] | (n8[1] << 16);
        const uint32_t n2p = n8[2] | ((uint32_t)sp.walk << 16) | (accumulate ? 0x80000000u : 0u);
        const uint32_t wgb = begin[1] | (begin[2] << 10) | ((uint32_t)sp.total << 20);
        hipLaunchKernelGGL(kern, grid, block, lds, s, vec, norm_w, st[0], st[1], st[2], kc, n01, n2p, wgb, tail);
    }
    return hipGetLastError();
}

// `count` layers of the same bits / K / C that read the same activation row, in one launch;
// norm_w != nullptr fuses the RMSNorm of that row, gate != nullptr (one layer, no norm) the
// gated-MLP activation fp16(fp16(silu(gate)) * vec).  The caller has asked stream_cu_supported().
hipError_t launch_stream_cu(int bits, const __half *vec, const __half *norm_w, float eps, const __half *gate,
                            const StreamMember *members, int count, int K, int C, int accumulate, hipStream_t s,
                            const float *attn_ml) {
    if (count < 1 || count > kStreamMaxGroup || (gate && (norm_w || count != 1))) return hipErrorInvalidValue;
    if (attn_ml && (gate || norm_w || count != 1 || K % 128)) return hipErrorInvalidValue;
    int tiles[kStreamMaxGroup], all = 0;
    for (int i = 0; i < count; i++) {
        tiles[i] = ceil_div(members[i].N, kStreamTileCols);
        all += tiles[i];
        if (members[i].N % 8 || members[i].N / 8 > 0xffff) return hipErrorInvalidValue;  // (the group shell packs N / 8 into 16 bits)
    }
    if (K > 0xffff) return hipErrorInvalidValue;
    const StreamGeo geo = stream_geo(bits, K, members[0].N, C);
    const int idx = cu_pick(geo.ng, ceil_div(all, kCuCus));
    if (idx < 0) return hipErrorInvalidValue;
    CuSplit sp = cu_split(tiles, count, kCuCfgs[idx].TEAMS);
    // one tile more than teams on some compute unit: the staging wavefronts take it instead of a team walking
    bool extra = false;
    if (sp.walk > 1 && cu_cfg_extra(idx) && !gate && !attn_ml) {
        const CuSplit sx = cu_split(tiles, count, kCuCfgs[idx].TEAMS + 1);
        if (sx.walk == 1) {
            sp = sx;
            extra = true;
        }
    }
    if (sp.walk > kCuMaxWalk || sp.total > 1023) return hipErrorInvalidValue;
    const bool group = count > 1 || norm_w != nullptr || gate != nullptr, walk = sp.walk > 1;
    const __half *ml_slot = reinterpret_cast<const __half *>(attn_ml);
#define CQ_CU_GO(BITS_, I_)                                                                                               \
    do {                                                                                                                  \
        if (extra) {                                                                                                      \
            if constexpr (cu_cfg_extra(I_))                                                                               \
                return norm_w ? launch_cu_cfg<BITS_, I_, kCuNorm, true, false, true>(vec, norm_w, eps, members, count, geo, sp, accumulate, s)    \
                              : launch_cu_cfg<BITS_, I_, kCuPlain, true, false, true>(vec, nullptr, 0.f, members, count, geo, sp, accumulate, s); \
            else                                                                                                          \
                return hipErrorInvalidValue;                                                                              \
        }                                                                                                                 \
        if (attn_ml) {                                                                                                    \
            if constexpr (I_ <= kCuAttnMaxCfg)                                                                            \
                return walk ? launch_cu_cfg<BITS_, I_, kCuAttn, true, true>(vec, ml_slot, 0.f, members, count, geo, sp, accumulate, s)   \
                            : launch_cu_cfg<BITS_, I_, kCuAttn, true, false>(vec, ml_slot, 0.f, members, count, geo, sp, accumulate, s); \
            else                                                                                                          \
                return hipErrorInvalidValue;                                                                              \
        }                                                                                                                 \
        if (!group)                                                                                                       \
            return walk ? launch_cu_cfg<BITS_, I_, kCuPlain, false, true>(vec, nullptr, 0.f, members, count, geo, sp, accumulate, s)   \
                        : launch_cu_cfg<BITS_, I_, kCuPlain, false, false>(vec, nullptr, 0.f, members, count, geo, sp, accumulate, s); \
        if (gate)                                                                                                         \
            return walk ? launch_cu_cfg<BITS_, I_, kCuGate, true, true>(vec, gate, 0.f, members, count, geo, sp, accumulate, s)        \
                        : launch_cu_cfg<BITS_, I_, kCuGate, true, false>(vec, gate, 0.f, members, count, geo, sp, accumulate, s);      \
        if (norm_w)                                                                                                       \
            return walk ? launch_cu_cfg<BITS_, I_, kCuNorm, true, true>(vec, norm_w, eps, members, count, geo, sp, accumulate, s)      \
                        : launch_cu_cfg<BITS_, I_, kCuNorm, true, false>(vec, norm_w, eps, members, count, geo, sp, accumulate, s);    \
        return walk ? launch_cu_cfg<BITS_, I_, kCuPlain, true, true>(vec, nullptr, 0.f, members, count, geo, sp, accumulate, s)        \
                    : launch_cu_cfg<BITS_, I_, kCuPlain, true, false>(vec, nullptr, 0.f, members, count, geo, sp, accumulate, s);      \
    } while (0)
#define CQ_CU_BITS(BITS_)            \
    switch (idx) {                   \
        case 0: CQ_CU_GO(BITS_, 0);  \
        case 1: CQ_CU_GO(BITS_, 1);  \
        case 2: CQ_CU_GO(BITS_, 2);  \
        case 3: CQ_CU_GO(BITS_, 3);  \
        case 4: CQ_CU_GO(BITS_, 4);  \
        case 5: CQ_CU_GO(BITS_, 5);  \
        case 6: CQ_CU_GO(BITS_, 6);  \
        case 7: CQ_CU_GO(BITS_, 7);  \
        case 8: CQ_CU_GO(BITS_, 8);  \
        case 9: CQ_CU_GO(BITS_, 9);  \
        default: CQ_CU_GO(BITS_, 10); \
    }
    if (bits == 4) CQ_CU_BITS(4)
    CQ_CU_BITS(3)
#undef CQ_CU_BITS
#undef CQ_CU_GO
}


// ---- two to four activation rows --------------------------------------------------------------------
// The matrix-core tile that the one-row kernel fills with 16 copies of its row takes four different
// rows at the same price: A row m holds activation row m % 4, so accumulator entry r of EVERY lane
// group is row r's sum and the lane groups still share the units' scales a quarter each.  Same
// launch shape as stream_cu_body (one workgroup per compute unit, staging wavefronts first, D0 units
// requested before the barrier, a ring of D behind it); what changes is the staging: a row's slice
// of NB blocks is a task, all wavefronts share the tasks of the B rows (the computing ones once
// their first requests are out), each passes its tasks through a piece of LDS of its own, and the
// rows' cherry activations are left in LDS for the teams' cherry wavefronts.
template <int BITS>
__device__ inline sf4_t unit_dot_rows(const su4 w, const unsigned short *xa) {
    const sf4_t zero4 = {0.f, 0.f, 0.f, 0.f};
    if constexpr (BITS == 4) {
        const su4 y = {w[0] >> 8, w[1] >> 8, w[2] >> 8, w[3] >> 8};
        const sh8_t a0 = *reinterpret_cast<const sh8_t *>(xa);
        const sh8_t a1 = *reinterpret_cast<const sh8_t *>(xa + 8);
        const sh8_t a2 = *reinterpret_cast<const sh8_t *>(xa + 16);
        const sh8_t a3 = *reinterpret_cast<const sh8_t *>(xa + 24);
        const su4 b0 = {w[0] & 0x000f000fu, y[0] & 0x000f000fu, w[1] & 0x000f000fu, y[1] & 0x000f000fu};
        const su4 b1 = {w[2] & 0x000f000fu, y[2] & 0x000f000fu, w[3] & 0x000f000fu, y[3] & 0x000f000fu};
        const su4 b2 = {w[0] & 0x00f000f0u, y[0] & 0x00f000f0u, w[1] & 0x00f000f0u, y[1] & 0x00f000f0u};
        const su4 b3 = {w[2] & 0x00f000f0u, y[2] & 0x00f000f0u, w[3] & 0x00f000f0u, y[3] & 0x00f000f0u};
        sf4_t dl = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, as_h8(b0), zero4, 0, 0, 0);
        sf4_t dh = __builtin_amdgcn_mfma_f32_16x16x32_f16(a2, as_h8(b2), zero4, 0, 0, 0);
        dl = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, as_h8(b1), dl, 0, 0, 0);
        dh = __builtin_amdgcn_mfma_f32_16x16x32_f16(a3, as_h8(b3), dh, 0, 0, 0);
        return dl * 16777216.0f + dh * 1048576.0f;
    } else {
        const su3 y = {w[0] >> 9, w[1] >> 9, w[2] >> 9};
        const sh8_t a0 = *reinterpret_cast<const sh8_t *>(xa);
        const sh8_t a2 = *reinterpret_cast<const sh8_t *>(xa + 8);
        const sh8_t a4 = *reinterpret_cast<const sh8_t *>(xa + 16);
        const sh8_t a1 = *reinterpret_cast<const sh8_t *>(xa + 24);
        const uint32_t z = (y[0] & 0x00400040u) | ((y[1] & 0x00400040u) << 1) | ((y[2] & 0x00400040u) << 2);
        const su4 b0 = {w[0] & 0x00070007u, w[1] & 0x00070007u, w[2] & 0x00070007u, y[0] & 0x00070007u};
        const su4 b2 = {w[0] & 0x00380038u, w[1] & 0x00380038u, w[2] & 0x00380038u, y[0] & 0x00380038u};
        const su4 b4 = {w[0] & 0x01c001c0u, w[1] & 0x01c001c0u, w[2] & 0x01c001c0u, z};
        const su4 b1 = {y[1] & 0x00070007u, y[2] & 0x00070007u, (y[1] >> 3) & 0x00070007u, (y[2] >> 3) & 0x00070007u};
        sf4_t d0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, as_h8(b0), zero4, 0, 0, 0);
        const sf4_t d3 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a2, as_h8(b2), zero4, 0, 0, 0);
        const sf4_t d6 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a4, as_h8(b4), zero4, 0, 0, 0);
        d0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, as_h8(b1), d0, 0, 0, 0);
        return d0 * 16777216.0f + d3 * 2097152.0f + d6 * 262144.0f;
    }
}

constexpr int kCuRows = 8;     // activation rows of a stream_cu_rows_kernel launch at most (R = 4 or 8; rows from B on are not staged)
constexpr int kCuRowsNB = 2;   // blocks of 512 compacted positions per staging task
constexpr int kCuRowsPad = 8;  // halves between the compacted rows in LDS: the four rows a load instruction reads lie in different banks

// R = 8: A row m holds activation row m % 8, lane groups kq and kq ^ 2 receive the same four rows
// (4 (kq & 1) + r) and share the units' scales half each.
// WALK: some team takes more than one tile (the requests of the next tile then join the ring).
template <int BITS, int W, int L, int TEAMS, int S, int NB, int D0, int D, int R, bool WALK>
__global__ __launch_bounds__(64 * (W * TEAMS + S)) void stream_cu_rows_kernel(const __half *__restrict__ x,
                                                                               const uint8_t *__restrict__ stream,
                                                                               __half *__restrict__ mul, int K, int C, int N,
                                                                               int G, int accumulate, int Pw, int B) {
    const int P = WALK ? Pw : 1;
    static_assert(R == 4 || R == 8, "rows per matrix-core tile");
    constexpr int NRED = 16 / R;   // lane groups that receive the same rows: they share the units' scales
    constexpr int NC = W * TEAMS;
    constexpr int NT = 64 * (NC + S);
    constexpr int UB = BITS == 4 ? 1024 : 768;
    constexpr float kGrid = BITS == 4 ? -7.5f : -3.5f;
    constexpr int NBR = kCuRowsNB;
    constexpr int XS = NBR + 1;
    constexpr int NW = NC + S;                          // all wavefronts stage: the computing ones once their first requests are out
    constexpr int TPW = (R * ((W * L + 4 * NBR - 1) / (4 * NBR)) + NW - 1) / NW;  // staging tasks (a row's slice of NBR blocks) per wavefront at most
    constexpr int PIECE = XS * 512 + 8;                 // halves of a wavefront's piece of LDS
    static_assert(D0 <= D && D <= L && L % D == 0 && L % 4 == 0, "ring slots are fixed per unit across tiles");
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kq = lane >> 4, nn = lane & 15;
    const int bid = blockIdx.x;
    const int ng = (K - C + kStreamUnitK - 1) / kStreamUnitK;
    const int Knp512 = (ng * kStreamUnitK + 511) & ~511;
    const int nblk = Knp512 >> 9;
    const uint32_t off_cherry = ((uint32_t)ng * 32u + 255u) & ~255u;
    const uint32_t off_units = off_cherry + (((uint32_t)C * 32u + 255u) & ~255u);
    const uint32_t record_bytes = off_units + (uint32_t)ng * UB;
    const uint32_t hdr_bytes = ((uint32_t)(Knp512 + 2 * ((C + 31) & ~31)) + 255u) & ~255u;
    const int ntiles = (N + kStreamTileCols - 1) / kStreamTileCols;
    // LDS: the wavefronts' pieces | compacted rows [R][Knp512 + pad] | unit sums [4 nblk][R] | cherry activations [R][128] | partial outputs [P][NC][R][16]
    const int XROW = Knp512 + kCuRowsPad;
    unsigned short *s_piece = reinterpret_cast<unsigned short *>(smem);
    unsigned short *s_xs = s_piece + NW * PIECE;
    float *s_xsum = reinterpret_cast<float *>(s_xs + R * XROW);
    unsigned short *s_cx = reinterpret_cast<unsigned short *>(s_xsum + 4 * nblk * R);
    float *s_red = reinterpret_cast<float *>(s_cx + R * 128);
    const int tstride = G * TEAMS;

    // ---- staging: task t = slice t % nslices (NBR blocks of 512 compacted positions) of row t / nslices;
    // wavefront w takes the tasks w, w + NW, ...: raw slice -> its piece of LDS -> gather, unit sums,
    // and the row's activations at the cherry channels whose columns start in the slice
    const int nslices = (nblk + NBR - 1) / NBR, ntasks = B * nslices;
    su4 xr[TPW][XS];
    su2 tbl[TPW][NBR];
    uint32_t cl[TPW][2];
    auto stage_request = [&]() {
        const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc((void *)stream, 0, (int)hdr_bytes, kSFlags);
#pragma unroll
        for (int tt = 0; tt < TPW; tt++) {
            const int task = wave + tt * NW;
            const bool on = task < ntasks;
            const int r = task / nslices, sl = task - r * nslices, b0 = sl * NBR, b1 = min(nblk, b0 + NBR);
            // (a descriptor per row: what lies behind the row's end reads as zeros)
            const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)(x + (size_t)(on ? r : 0) * K), 0, K * 2, kSFlags);
#pragma unroll
            for (int i = 0; i < XS; i++)
                xr[tt][i] = __builtin_amdgcn_raw_buffer_load_b128(rx, on ? (uint32_t)(b0 * 512 + i * 512 + lane * 8) * 2u : kSOob, 0, 0);
#pragma unroll
            for (int i = 0; i < NBR; i++)
                tbl[tt][i] = __builtin_amdgcn_raw_buffer_load_b64(rh, on && b0 + i < b1 ? (uint32_t)((b0 + i) * 512 + lane * 8) : kSOob, 0, 0);
#pragma unroll
            for (int h = 0; h < 2; h++)
                cl[tt][h] = __builtin_amdgcn_raw_buffer_load_b16(rh, on && lane + 64 * h < C ? (uint32_t)(Knp512 + 2 * (lane + 64 * h)) : kSOob, 0, 0);
        }
    };
    auto stage_process = [&]() {
        unsigned short *piece = s_piece + wave * PIECE;
#pragma unroll
        for (int tt = 0; tt < TPW; tt++) {
            const int task = wave + tt * NW;
            if (task < ntasks) {
                const int r = task / nslices, sl = task - r * nslices, b0 = sl * NBR, b1 = min(nblk, b0 + NBR);
                unsigned short *xs_r = s_xs + r * XROW;
#pragma unroll
                for (int i = 0; i < XS; i++) reinterpret_cast<su4 *>(piece + i * 512)[lane] = xr[tt][i];
#pragma unroll
                for (int i = 0; i < NBR; i++) {
                    const int blk = b0 + i;
                    if (blk < b1) {
                        const su2 t = tbl[tt][i];
                        unsigned short h[8];
#pragma unroll
                        for (int j = 0; j < 8; j++)
                            h[j] = piece[i * 512 + 64 * j + lane + (int)((t[j >> 2] >> (8 * (j & 3))) & 0xffu)];
                        float f[4];
#pragma unroll
                        for (int j = 0; j < 8; j++) xs_r[blk * 512 + 64 * j + lane] = h[j];
#pragma unroll
                        for (int u = 0; u < 4; u++)
                            f[u] = __half2float(__ushort_as_half(h[2 * u])) + __half2float(__ushort_as_half(h[2 * u + 1]));
                        const float s01 = swap32_add(f[0], f[1]);
                        const float s23 = swap32_add(f[2], f[3]);
                        const float rs = row_sum(swap16_add(s01, s23));
                        if (nn == 0) s_xsum[(blk * 4 + ((kq >> 1) | ((kq & 1) << 1))) * R + r] = rs;
                    }
                }
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const int e = lane + 64 * h, col = (int)(cl[tt][h] & 0xffffu);
                    const int owner = min(col / (NBR * 512), nslices - 1);
                    if (e < C) {
                        if (owner == sl) s_cx[r * 128 + e] = piece[col - b0 * 512];
                    } else if (sl == 0) {
                        s_cx[r * 128 + e] = 0;
                    }
                }
            }
            asm volatile("" ::: "memory");
            __builtin_amdgcn_wave_barrier();  // (the piece is rewritten for the next task)
        }
    };

    if (wave < S) {
        __builtin_amdgcn_s_setprio(3);
        stage_request();
        stage_process();
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
    } else {
        // ---- computing wavefront `cls` of team `team`, on tiles bid + G (team + TEAMS j)
        const int cwv = wave - S;
        const int team = cwv / W, cls = cwv % W;
        const __amdgpu_buffer_rsrc_t rt = __builtin_amdgcn_make_buffer_rsrc(
            (void *)(stream + hdr_bytes), 0, (int)min((unsigned long long)ntiles * record_bytes, 0xffffffffull), kSFlags);
        uint32_t sc[L / NRED];
        const int red_id = kq / (R / 4);            // which share of the units' scales this lane group keeps
        const int rowbase = 4 * (kq % (R / 4));     // accumulator entry r of this lane is row rowbase + r
        su4 wbuf[D];
        su4 cw[4];
        const bool cherry_wave = cls == W - 1;
        int tcur = bid + G * team;
        bool vcur = tcur < ntiles;
        uint32_t tb = (uint32_t)tcur * record_bytes;
        auto load_cherry = [&](uint32_t base, bool valid) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int lg = 4 * j + kq;
                if (32 * j < C)
                    cw[j] = __builtin_amdgcn_raw_buffer_load_b128(
                        rt, valid && 8 * lg < C ? off_cherry + (uint32_t)(lg * 16 + nn) * 16u : kSOob, base, 2);
            }
        };
        const uint32_t sc_off = (uint32_t)((cls + red_id * W) * 32 + nn * 2);
        auto load_scale = [&](int sl, uint32_t base, bool valid) -> uint32_t {
            return __builtin_amdgcn_raw_buffer_load_b16(rt, valid && cls + (NRED * sl + red_id) * W < ng ? sc_off : kSOob,
                                                        base + NRED * sl * W * 32, 0);
        };
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
        stage_request();   // (activations first: the barrier waits for them, not for the weights)
        __builtin_amdgcn_sched_barrier(0);
        if (cherry_wave) load_cherry(tb, vcur);
#pragma unroll
        for (int i = 0; i < L / NRED; i++) sc[i] = load_scale(i, tb, vcur);
#pragma unroll
        for (int i = 0; i < D0; i++) wbuf[i] = load_unit(i, tb, vcur);
        __builtin_amdgcn_sched_barrier(0);
        stage_process();
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
#pragma unroll
        for (int i = D0; i < D; i++) wbuf[i] = load_unit(i, tb, vcur);
        const unsigned short *xs_l = s_xs + (nn & (R - 1)) * XROW + 32 * kq;   // A row nn holds activation row nn % 4
        su4 ca[4];
        if (cherry_wave) {
#pragma unroll
            for (int q = 0; q < 4; q++)
                if (32 * q < C) ca[q] = *reinterpret_cast<const su4 *>(s_cx + (nn & (R - 1)) * 128 + 32 * q + 8 * kq);
        }
        const float *xsum_l = s_xsum + rowbase;
#pragma unroll 1
        for (int j = 0; j < P; j++) {
            const int tnext = tcur + tstride;
            const bool vnext = WALK && tnext < ntiles;
            const uint32_t tbn = (uint32_t)tnext * record_bytes;
            sf4_t dc = {0.f, 0.f, 0.f, 0.f};
            if (cherry_wave) {
#pragma unroll
                for (int q = 0; q < 4; q++)
                    if (32 * q < C) dc = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_h8(ca[q]), as_h8(cw[q]), dc, 0, 0, 0);
                if constexpr (WALK) load_cherry(tbn, vnext);
            }
            sf4_t tt = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < L; i++) {
                const bool real = cls + i * W < ng;
                const int up = real ? cls + i * W : 0;
                const float sf = (i % NRED) == red_id ? __half2float(__ushort_as_half((unsigned short)sc[i / NRED])) : 0.f;
                const su4 w = wbuf[i % D];
                const sf4_t v = unit_dot_rows<BITS>(w, xs_l + up * kStreamUnitK);
                if (i + D < L) wbuf[i % D] = load_unit(i + D, tb, vcur);
                else if constexpr (WALK) wbuf[i % D] = load_unit(i + D - L, tbn, vnext);
                const sf4_t xsum = *reinterpret_cast<const sf4_t *>(xsum_l + up * R);
                tt += (v + kGrid * xsum) * sf;
                if constexpr (WALK) {
                    if ((i % NRED) == NRED - 1) sc[i / NRED] = load_scale(i / NRED, tbn, vnext);
                }
            }
            // the shares of the lane groups that hold the same rows; every lane then stores R / 4 of its rows
            float fin[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float t = swap32_add(tt[r], tt[r]);
                if constexpr (NRED == 4) t = swap16_add(t, t);
                fin[r] = t + dc[r];
            }
            float *red = s_red + ((j * NC + cwv) * R + rowbase) * 16 + nn;
            if constexpr (R == 4) {
                red[kq * 16] = kq == 0 ? fin[0] : kq == 1 ? fin[1] : kq == 2 ? fin[2] : fin[3];
            } else {
                red[(2 * red_id) * 16] = red_id ? fin[2] : fin[0];
                red[(2 * red_id + 1) * 16] = red_id ? fin[3] : fin[1];
            }
            tcur = tnext;
            vcur = vnext;
            tb = tbn;
            if (!vcur) break;
        }
    }

    // ---- across a tile's wavefronts, then one store per output and row
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    for (int o = tid; o < 16 * R * P * TEAMS; o += NT) {
        const int col = o & 15, r = (o >> 4) & (R - 1), jt = o / (16 * R), j = jt / TEAMS, t = jt - j * TEAMS;
        const int tile = bid + G * (t + TEAMS * j), n = tile * 16 + col;
        if (tile < ntiles && n < N && r < B) {
            const float *red = s_red + ((j * NC + t * W) * R + r) * 16 + col;
            float v = 0.f;
#pragma unroll
            for (int c = 0; c < W; c++) v += red[c * R * 16];
            __half *o16 = mul + (size_t)r * N + n;
            if (accumulate) v += __half2float(*o16);
            *o16 = __float2half_rn(v);
        }
    }
}

static size_t cu_rows_lds_bytes(const StreamGeo &g, const CuCfg &c, int P, int R) {
    const int Knp512 = (g.ng * kStreamUnitK + 511) & ~511;
    size_t need = (size_t)(c.W * c.TEAMS + c.S) * ((kCuRowsNB + 1) * 512 + 8) * 2 + (size_t)R * (Knp512 + kCuRowsPad) * 2 + (size_t)(Knp512 / 128) * R * 4 +
                  (size_t)R * 128 * 2 + (size_t)P * c.W * c.TEAMS * R * 16 * 4;
    const size_t alone = 80 * 1024 + 1024;  // more than half of a compute unit's LDS: one workgroup per compute unit
    return need > alone ? need : alone;
}

// (entries 5, 6 and 8 -- more than 96 units per column, 16 wavefronts of 128 registers -- would spill with four rows' sums;
// eight rows of more than 48 units do not fit the LDS beside the wavefronts' staging pieces)
constexpr bool cu_rows_cfg(int i, int R) { return R == 4 ? i != 5 && i != 6 && i != 8 : i <= 2 || i == 7 || i == 10; }
static int cu_rows_tile(int B) { return B <= 4 ? 4 : 8; }

bool stream_cu_rows_supported(int bits, int B, int K, int N, int C) {
    if (B < 2 || B > kCuRows || N % 8) return false;
    const int Ns[1] = {N};
    if (!stream_cu_supported(bits, K, C, Ns, 1)) return false;
    const StreamGeo geo = stream_geo(bits, K, N, C);
    const int idx = cu_pick(geo.ng, ceil_div(geo.ntiles, kCuCus));
    if (!cu_rows_cfg(idx, cu_rows_tile(B))) return false;
    const int tiles[1] = {geo.ntiles};
    const CuSplit sp = cu_split(tiles, 1, kCuCfgs[idx].TEAMS);
    return cu_rows_lds_bytes(geo, kCuCfgs[idx], sp.walk, cu_rows_tile(B)) <= 160 * 1024;
}

template <int BITS, int I, int R>
static hipError_t launch_cu_rows_cfg(const __half *vec, const uint8_t *stream, __half *mul, int B, const StreamGeo &geo,
                                     const CuSplit &sp, int accumulate, hipStream_t s) {
    constexpr CuCfg c = kCuCfgs[I];
    if constexpr (!cu_rows_cfg(I, R)) {
        return hipErrorInvalidValue;
    } else {
        const size_t lds = cu_rows_lds_bytes(geo, c, sp.walk, R);
        const dim3 grid(sp.total), block(64 * (c.W * c.TEAMS + c.S));
        if (sp.walk > 1) {
            auto kern = stream_cu_rows_kernel<BITS, c.W, c.L, c.TEAMS, c.S, c.NB, c.D0, c.D, R, true>;
            static bool raised[kCuMaxDevices] = {};
            if (hipError_t e = cu_raise_lds(kern, raised)) return e;
            hipLaunchKernelGGL(kern, grid, block, lds, s, vec, stream, mul, geo.K, geo.C, geo.N, sp.wgs[0], accumulate, sp.walk, B);
        } else {
            auto kern = stream_cu_rows_kernel<BITS, c.W, c.L, c.TEAMS, c.S, c.NB, c.D0, c.D, R, false>;
            static bool raised[kCuMaxDevices] = {};
            if (hipError_t e = cu_raise_lds(kern, raised)) return e;
            hipLaunchKernelGGL(kern, grid, block, lds, s, vec, stream, mul, geo.K, geo.C, geo.N, sp.wgs[0], accumulate, sp.walk, B);
        }
        return hipGetLastError();
    }
}

// vec (B, K), mul (B, N), 2 <= B <= 8; the caller has asked stream_cu_rows_supported()
hipError_t launch_stream_cu_rows(int bits, const __half *vec, const uint8_t *stream, __half *mul, int B, int K, int N, int C,
                                 int accumulate, hipStream_t s) {
    const StreamGeo geo = stream_geo(bits, K, N, C);
    const int idx = cu_pick(geo.ng, ceil_div(geo.ntiles, kCuCus));
    if (idx < 0 || B < 2 || B > kCuRows || !cu_rows_cfg(idx, cu_rows_tile(B))) return hipErrorInvalidValue;
    const int tiles[1] = {geo.ntiles};
    const CuSplit sp = cu_split(tiles, 1, kCuCfgs[idx].TEAMS);
    if (sp.walk > kCuMaxWalk) return hipErrorInvalidValue;
#define CQ_ROWS_BITS(BITS_)                                                                               \
    switch (idx) {                                                                                        \
        case 0: return B <= 4 ? launch_cu_rows_cfg<BITS_, 0, 4>(vec, stream, mul, B, geo, sp, accumulate, s) : launch_cu_rows_cfg<BITS_, 0, 8>(vec, stream, mul, B, geo, sp, accumulate, s);          \
        case 1: return B <= 4 ? launch_cu_rows_cfg<BITS_, 1, 4>(vec, stream, mul, B, geo, sp, accumulate, s) : launch_cu_rows_cfg<BITS_, 1, 8>(vec, stream, mul, B, geo, sp, accumulate, s);          \
        case 2: return B <= 4 ? launch_cu_rows_cfg<BITS_, 2, 4>(vec, stream, mul, B, geo, sp, accumulate, s) : launch_cu_rows_cfg<BITS_, 2, 8>(vec, stream, mul, B, geo, sp, accumulate, s);          \
        case 3: return B <= 4 ? launch_cu_rows_cfg<BITS_, 3, 4>(vec, stream, mul, B, geo, sp, accumulate, s) : launch_cu_rows_cfg<BITS_, 3, 8>(vec, stream, mul, B, geo, sp, accumulate, s);          \
        case 4: return B <= 4 ? launch_cu_rows_cfg<BITS_, 4, 4>(vec, stream, mul, B, geo, sp, accumulate, s) : launch_cu_rows_cfg<BITS_, 4, 8>(vec, stream, mul, B, geo, sp, accumulate, s);          \
        case 7: return B <= 4 ? launch_cu_rows_cfg<BITS_, 7, 4>(vec, stream, mul, B, geo, sp, accumulate, s) : launch_cu_rows_cfg<BITS_, 7, 8>(vec, stream, mul, B, geo, sp, accumulate, s);          \
        case 9: return B <= 4 ? launch_cu_rows_cfg<BITS_, 9, 4>(vec, stream, mul, B, geo, sp, accumulate, s) : launch_cu_rows_cfg<BITS_, 9, 8>(vec, stream, mul, B, geo, sp, accumulate, s);          \
        default: return B <= 4 ? launch_cu_rows_cfg<BITS_, 10, 4>(vec, stream, mul, B, geo, sp, accumulate, s) : launch_cu_rows_cfg<BITS_, 10, 8>(vec, stream, mul, B, geo, sp, accumulate, s);        \
    }
    if (bits == 4) CQ_ROWS_BITS(4)
    CQ_ROWS_BITS(3)
#undef CQ_ROWS_BITS
}

// ---- several layers of one shape in every workgroup -----------------------------------------------
// gate_proj + up_proj -> fp16(fp16(silu(gate)) * up).  Up to 32 units per column: three pairs of
// two-wavefront teams (16 units per wavefront) and 2 + 2 staging wavefronts of four blocks, i.e. the
// three tiles per compute unit of the 4096 -> 11008 launch with both layers' tile t in one
// workgroup; up to 64 units: one pair of four-wavefront teams and 4 + 4 staging wavefronts.
// (Measured and not kept: q / k / v of equal widths the same way, three teams of three wavefronts
// and 2 + 2 + 2 staging wavefronts, one tile of each layer per compute unit instead of consecutive
// ranges of 85 / 85 / 86 workgroups: 8.25 us behind the RMSNorm against 7.24, 7.00 against 7.08
// without -- the later barrier costs what the even spread gains.)
// Measured, RMSNorm + gate/up + SiLU, 4-bit / 3-bit us (ring of 8 -> ring of 4): 2 x (4096 -> 11008) 10.67 /
// 9.72 -> 10.25 / 9.23; 2 x (8192 -> 28672) 41.2 / 33.9 -> 39.3 / 32.6; 2 x (5120 -> 13824) on the 64-unit
// entry 18.2 / 17.7, on the 48-unit entry 15.4 / 14.8 (two teams of 5 x 8 units: 15.8 / 14.8).
static constexpr CuCfg kCuPairCfgs[] = {
    {2, 16, 6, 4, 4, 3, 4},   // up to 32 units: three pairs of two-wavefront teams
    {3, 16, 4, 4, 6, 2, 4},   // up to 48 units: two pairs of three-wavefront teams
    {4, 16, 2, 8, 4, 2, 4},   // up to 64 units: one pair of four-wavefront teams
};

static int cu_pair_pick(int ng) { return ng <= 32 ? 0 : ng <= 48 ? 1 : ng <= 64 ? 2 : -1; }

bool stream_pair_supported(int bits, int K, int N, int C) {
    if ((bits != 3 && bits != 4) || K > 0xffff || C > 128 || N % 8) return false;
    const StreamGeo geo = stream_geo(bits, K, N, C);
    const int idx = cu_pair_pick(geo.ng);
    if (idx < 0) return false;
    const CuCfg &c = kCuPairCfgs[idx];
    if (geo.ng > c.W * c.L || geo.ng * kStreamUnitK > (c.S / 2) * c.NB * 512) return false;
    const int tiles[1] = {geo.ntiles};
    const CuSplit sp = cu_split(tiles, 1, c.TEAMS / 2);
    if (sp.walk > kCuMaxWalk || sp.total > 0xffff) return false;
    return cu_lds_bytes(geo, c, sp.walk, 2) <= 160 * 1024;
}

template <int BITS, int W, int L, int TEAMS, int S, int NB, int D0, int D, int PRO, bool WALK, int MEM, int EPI>
static hipError_t launch_multi_cfg(const __half *vec, const __half *norm_w, float eps, const uint8_t *const *streams,
                                   __half *const *muls, const StreamGeo &geo, const CuSplit &sp, hipStream_t s) {
    constexpr CuCfg c = {W, L, TEAMS, S, NB, D0, D};
    auto kern = stream_cu_multi_kernel<BITS, W, L, TEAMS, S, NB, D0, D, PRO, WALK, MEM, EPI>;
    static bool raised[kCuMaxDevices] = {};
    if (hipError_t e = cu_raise_lds(kern, raised)) return e;
    const size_t lds = cu_lds_bytes(geo, c, sp.walk, MEM);
    CuMultiTail tail = {{muls[0], muls[1], muls[MEM > 2 ? 2 : 1]}};
    hipLaunchKernelGGL(kern, dim3(sp.total), dim3(64 * (W * TEAMS + S)), lds, s, vec, norm_w, streams[0], streams[1],
                       streams[MEM > 2 ? 2 : 1], (uint32_t)geo.K | ((uint32_t)geo.C << 16), geo.N,
                       (uint32_t)sp.wgs[0] | ((uint32_t)sp.walk << 16), eps, tail);
    return hipGetLastError();
}

// act (1, N) = fp16(fp16(silu(vec' Wg^T)) * (vec' Wu^T)), vec' = vec or its RMSNorm; the caller has
// asked stream_pair_supported().
hipError_t launch_stream_pair(int bits, const __half *vec, const __half *norm_w, float eps, const uint8_t *stream_gate,
                              const uint8_t *stream_up, __half *act, int K, int N, int C, hipStream_t s) {
    const StreamGeo geo = stream_geo(bits, K, N, C);
    const int idx = cu_pair_pick(geo.ng);
    if (idx < 0) return hipErrorInvalidValue;
    const int tiles[1] = {geo.ntiles};
    const CuSplit sp = cu_split(tiles, 1, kCuPairCfgs[idx].TEAMS / 2);
    if (sp.walk > kCuMaxWalk) return hipErrorInvalidValue;
    const bool walk = sp.walk > 1;
    const uint8_t *streams[2] = {stream_gate, stream_up};
    __half *muls[2] = {act, act};
#define CQ_MULTI(BITS_, C_, PRO_, WALK_, MEM_, EPI_) \
    launch_multi_cfg<BITS_, C_.W, C_.L, C_.TEAMS, C_.S, C_.NB, C_.D0, C_.D, PRO_, WALK_, MEM_, EPI_>
#define CQ_PAIR_GO(BITS_, I_)                                                                                            \
    do {                                                                                                                 \
        constexpr CuCfg c = kCuPairCfgs[I_];                                                                             \
        if (norm_w)                                                                                                      \
            return walk ? CQ_MULTI(BITS_, c, kCuNorm, true, 2, kCuSiluPair)(vec, norm_w, eps, streams, muls, geo, sp, s)  \
                        : CQ_MULTI(BITS_, c, kCuNorm, false, 2, kCuSiluPair)(vec, norm_w, eps, streams, muls, geo, sp, s); \
        return walk ? CQ_MULTI(BITS_, c, kCuPlain, true, 2, kCuSiluPair)(vec, nullptr, 0.f, streams, muls, geo, sp, s)   \
                    : CQ_MULTI(BITS_, c, kCuPlain, false, 2, kCuSiluPair)(vec, nullptr, 0.f, streams, muls, geo, sp, s);  \
    } while (0)
    if (bits == 4) {
        if (idx == 0) CQ_PAIR_GO(4, 0);
        if (idx == 1) CQ_PAIR_GO(4, 1);
        CQ_PAIR_GO(4, 2);
    }
    if (idx == 0) CQ_PAIR_GO(3, 0);
    if (idx == 1) CQ_PAIR_GO(3, 1);
    CQ_PAIR_GO(3, 2);
#undef CQ_PAIR_GO
}

#undef CQ_MULTI

}  // namespace cq
