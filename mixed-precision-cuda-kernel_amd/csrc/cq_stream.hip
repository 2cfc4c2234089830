// Fused dequant + matvec over a load-time repacked weight stream (gfx950).
//
// The reference layout (qweight (Kn/8*b, N), N contiguous) forces a kernel to split K across
// workgroups: a byte row holds one or two positions of every column, so a wavefront that wants
// wide loads owns many columns and few positions, and the partial sums of many workgroups have to
// meet in memory.  The stream layout below is the same information rearranged once, at load time,
// for the way CDNA4 wants to consume it:
//
//   * 16 output columns form a tile; a tile's whole K range is one contiguous record
//         [scales: ng x 16 fp16][cherry rows: C x 16 fp16][units: ng x 1 KB (4-bit) / 768 B (3-bit)]
//     (sections padded to 256 bytes).  A workgroup owns whole tiles, so no partial sum ever leaves
//     the workgroup: no atomics, no workspace, one fp16 store per output.
//   * a unit is 128 compacted positions (one scale group when G = 128) x 16 columns.  Lane
//     (kq = lane / 16, n = lane % 16) holds the 32 codes of column n at positions
//     128 g + 32 kq + 0..31 in 4 (3) consecutive dwords, so a wavefront reads a unit as ONE
//     dwordx4 (dwordx3) load of 1 KB (768 B) contiguous bytes.
//   * inside a lane's dwords the codes sit where a single v_and_b32 turns them into an MFMA
//     operand: a field masked in place at bit p <= 8 of a 16-bit half IS the fp16 subnormal
//     code * 2^(p-24).  4-bit: fields at bit 0 and 4 of each half directly, the other two after
//     one shift by 8 (5 VALU instructions per 8 codes, no v_perm).  3-bit: fields at bit 0, 3, 6
//     directly, two more after one shift by 9 (and, for the last four positions, by 3 more), and
//     the 6 left-over bits of the three dwords form the last two codes (25 instructions per 32
//     codes) -- here the values truly straddle dwords.
//   * v_mfma_f32_16x16x32_f16 multiplies (4 steps per unit at either width): B = the lane's
//     masked fields, A = the activations of the same positions from LDS, and the MFMA's K
//     dimension runs across the four lane groups, so the reduction over a unit's 128 positions
//     costs nothing.  Fields of different bit positions go to different accumulators (scaled by
//     2^(24-p) afterwards), so the activations enter unscaled and every product is exact.
//   * the activation vector is compacted around the cherry channels ONCE per workgroup into LDS
//     (raw copy -> gather), together with the per-group sums for the grid offset -c_b * sum(x).
//
// Arithmetic contract: csrc/quant_cuda_kernel.cu:718-835 (4-bit) and 558-672 (3-bit) of the
// reference; fp32 accumulation, one rounding to fp16.  Replaces the per-thread decode loops at
// :811-831 / :649-667 and the serial batch loop :797-834.
#include <stdlib.h>

#include <mutex>
#include <type_traits>

#include "cq_stream_dev.h"

namespace cq {

static inline uint32_t align256(uint32_t v) { return (v + 255u) & ~255u; }

StreamGeo stream_geo(int bits, int K, int N, int C) {
    StreamGeo g;
    g.bits = bits;
    g.K = K;
    g.N = N;
    g.C = C;
    g.Kn = K - C;
    g.ng = ceil_div(K - C, kStreamUnitK);
    g.ntiles = ceil_div(N, kStreamTileCols);
    g.off_cherry = align256((uint32_t)g.ng * 32u);
    g.off_units = g.off_cherry + align256((uint32_t)C * 32u);
    g.record_bytes = g.off_units + (uint32_t)g.ng * (bits == 4 ? 1024u : 768u);
    g.hdr_bytes = align256((uint32_t)(((g.ng * kStreamUnitK + 511) & ~511) + 2 * ((C + 31) & ~31)));
    return g;
}

size_t stream_bytes(int bits, int K, int N, int C) {
    const StreamGeo g = stream_geo(bits, K, N, C);
    return g.hdr_bytes + (size_t)g.ntiles * g.record_bytes;
}

// ---- where code q (0..31) of a lane lives ----------------------------------------------------
// 4-bit: MFMA j = q / 8 takes slot r = q % 8 from dword 2 (j & 1) + r / 4, nibble {0, 4, 2, 6}[r % 4]
// (+ 1 for j >= 2, the fields that sit at bit 4 of their half).
__host__ __device__ constexpr int s4_dword(int q) { return 2 * ((q >> 3) & 1) + ((q & 7) >> 2); }
__host__ __device__ constexpr int s4_bit(int q) { return 4 * ((int)((0x6240u >> (4 * (q & 3))) & 15u) + (q >> 4)); }
// 3-bit: returns dword (0..2) and bit, or dword 3 for the two codes assembled from the left-over
// bits (bit 15 + 16 h of dwords 0, 1, 2 = code bits 0, 1, 2), with `bit` = 16 h.
__host__ __device__ constexpr int s3_dword(int q) {
    return q < 24 ? (((q & 7) < 6) ? ((q & 7) >> 1) : (q < 16 ? 0 : 3)) : 1 + ((q & 3) >> 1);
}
__host__ __device__ constexpr int s3_bit(int q) {
    const int h = q & 1;
    if (q < 24) {
        const int f = ((q & 7) < 6) ? (q >> 3) : (q >> 3) + 3;  // q < 16 only for the second form
        return ((q & 7) < 6 || q < 16) ? 16 * h + 3 * f : 16 * h;
    }
    return 16 * h + 3 * (q < 28 ? 3 : 4);
}

// ---- prepack: reference buffers -> stream ------------------------------------------------------
template <int BITS>
__device__ inline uint32_t ref_code(const uint8_t *__restrict__ qweight, int k, int n, int N) {
    if (BITS == 4) return (qweight[(size_t)(k >> 1) * N + n] >> (4 * (k & 1))) & 15u;
    const size_t r = (size_t)(k >> 3) * 3;
    const uint32_t w24 = qweight[r * N + n] | (qweight[(r + 1) * N + n] << 8) | (qweight[(r + 2) * N + n] << 16);
    return (w24 >> (3 * (k & 7))) & 7u;
}

template <int BITS>
__global__ __launch_bounds__(256) void stream_pack_kernel(const uint8_t *__restrict__ qweight,
                                                          const __half *__restrict__ cherry_weight,
                                                          const __half *__restrict__ scales,
                                                          uint8_t *__restrict__ stream, int G, StreamGeo geo) {
    const int tile = blockIdx.x;
    uint8_t *rec = stream + geo.hdr_bytes + (size_t)tile * geo.record_bytes;
    const int N = geo.N, Kn = geo.Kn;
    // sections the kernel never writes codes into start out zero (padding)
    for (uint32_t i = threadIdx.x; i < geo.off_units / 4; i += 256) reinterpret_cast<uint32_t *>(rec)[i] = 0u;
    __syncthreads();
    for (int i = threadIdx.x; i < geo.ng * 16; i += 256) {
        const int g = i >> 4, n = tile * 16 + (i & 15);
        reinterpret_cast<__half *>(rec)[i] = n < N ? scales[(size_t)(g * kStreamUnitK / G) * N + n] : __float2half(0.f);
    }
    for (int i = threadIdx.x; i < geo.C * 16; i += 256) {
        // piece (lg, nn): 8 halves = cherry rows 8 lg .. 8 lg + 7 of column nn
        const int piece = i >> 3, e = i & 7, lg = piece >> 4, n = tile * 16 + (piece & 15);
        reinterpret_cast<__half *>(rec + geo.off_cherry)[i] =
            n < N ? cherry_weight[(size_t)(8 * lg + e) * N + n] : __float2half(0.f);
    }
    constexpr int DW = BITS;  // dwords per lane and unit
    for (int i = threadIdx.x; i < geo.ng * 64; i += 256) {
        const int g = i >> 6, lane = i & 63, kq = lane >> 4, n = tile * 16 + (lane & 15);
        uint32_t d[4] = {0u, 0u, 0u, 0u};
        for (int q = 0; q < 32; q++) {
            const int k = g * kStreamUnitK + 32 * kq + q;
            const uint32_t code = (k < Kn && n < N) ? ref_code<BITS>(qweight, k, n, N) : 0u;
            if (BITS == 4) {
                d[s4_dword(q)] |= code << s4_bit(q);
            } else if (s3_dword(q) < 3) {
                d[s3_dword(q)] |= code << s3_bit(q);
            } else {
                const int b = s3_bit(q) + 15;
                d[0] |= (code & 1u) << b;
                d[1] |= ((code >> 1) & 1u) << b;
                d[2] |= ((code >> 2) & 1u) << b;
            }
        }
        uint32_t *o = reinterpret_cast<uint32_t *>(rec + geo.off_units + (size_t)g * (64 * DW * 4)) + lane * DW;
        for (int j = 0; j < DW; j++) o[j] = d[j];
    }
}

// stream -> reference buffers (the inverse; restores a state dict from a prepacked module)
template <int BITS>
__global__ __launch_bounds__(256) void stream_unpack_kernel(const uint8_t *__restrict__ stream,
                                                            uint8_t *__restrict__ qweight,
                                                            __half *__restrict__ cherry_weight,
                                                            __half *__restrict__ scales, int G, StreamGeo geo) {
    const int tile = blockIdx.x;
    const uint8_t *rec = stream + geo.hdr_bytes + (size_t)tile * geo.record_bytes;
    const int N = geo.N, Kn = geo.Kn;
    const int ngr = ceil_div(Kn, G);
    for (int i = threadIdx.x; i < ngr * 16; i += 256) {
        const int gr = i >> 4, n = tile * 16 + (i & 15);
        if (n < N) scales[(size_t)gr * N + n] = reinterpret_cast<const __half *>(rec)[(gr * (G / kStreamUnitK)) * 16 + (i & 15)];
    }
    for (int i = threadIdx.x; i < geo.C * 16; i += 256) {
        const int piece = i >> 3, e = i & 7, lg = piece >> 4, n = tile * 16 + (piece & 15);
        if (n < N) cherry_weight[(size_t)(8 * lg + e) * N + n] = reinterpret_cast<const __half *>(rec + geo.off_cherry)[i];
    }
    constexpr int DW = BITS;
    for (int i = threadIdx.x; i < geo.ng * 64; i += 256) {
        const int g = i >> 6, lane = i & 63, kq = lane >> 4, n = tile * 16 + (lane & 15);
        if (n >= N) continue;
        const uint32_t *o = reinterpret_cast<const uint32_t *>(rec + geo.off_units + (size_t)g * (64 * DW * 4)) + lane * DW;
        uint32_t d[4] = {0u, 0u, 0u, 0u};
        for (int j = 0; j < DW; j++) d[j] = o[j];
        uint32_t code[32];
        for (int q = 0; q < 32; q++) {
            if (BITS == 4) {
                code[q] = (d[s4_dword(q)] >> s4_bit(q)) & 15u;
            } else if (s3_dword(q) < 3) {
                code[q] = (d[s3_dword(q)] >> s3_bit(q)) & 7u;
            } else {
                const int b = s3_bit(q) + 15;
                code[q] = ((d[0] >> b) & 1u) | (((d[1] >> b) & 1u) << 1) | (((d[2] >> b) & 1u) << 2);
            }
        }
        const int k0 = g * kStreamUnitK + 32 * kq;
        if (BITS == 4) {
            for (int q = 0; q < 32; q += 2)
                if (k0 + q < Kn) qweight[(size_t)((k0 + q) >> 1) * N + n] = (uint8_t)(code[q] | (code[q + 1] << 4));
        } else {
            for (int q = 0; q < 32; q += 8) {
                if (k0 + q >= Kn) continue;
                uint32_t w24 = 0;
                for (int e = 0; e < 8; e++) w24 |= code[q + e] << (3 * e);
                const size_t r = (size_t)((k0 + q) >> 3) * 3;
                qweight[r * N + n] = (uint8_t)w24;
                qweight[(r + 1) * N + n] = (uint8_t)(w24 >> 8);
                qweight[(r + 2) * N + n] = (uint8_t)(w24 >> 16);
            }
        }
    }
}

// header: for every compacted position k the number of cherry columns in front of it, low(k) (the
// position reads activation column k + low(k); padding positions hold C and so read beyond the last
// column, where the kernel keeps zeros), one byte
// each, stored per block of 512 positions so that lane l of a wavefront finds the entries of
// positions l, l + 64, ..., l + 448 in 8 consecutive bytes; then the cherry columns (uint16,
// padded with K, the column the kernel keeps zero)
__global__ __launch_bounds__(256) void stream_header_kernel(const int16_t *__restrict__ cherry_indices,
                                                            uint8_t *__restrict__ hdr, StreamGeo geo) {
    const int Knp512 = (geo.ng * kStreamUnitK + 511) & ~511, Cp = (geo.C + 31) & ~31;
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < Knp512) {
        const int blk = i >> 9, l = (i >> 3) & 63, j = i & 7;
        const int k = blk * 512 + 64 * j + l;
        hdr[i] = (uint8_t)(k < geo.Kn ? gather_offset(cherry_indices, geo.C, k) : geo.C);
    } else if (i < Knp512 + Cp) {
        const int m = i - Knp512;
        reinterpret_cast<uint16_t *>(hdr + Knp512)[m] = (uint16_t)(m < geo.C ? (int)cherry_indices[m] : geo.K);
    }
    if (i >= Knp512 + 2 * Cp && i < (int)geo.hdr_bytes) hdr[i] = 0;  // padding of the header
}

__global__ __launch_bounds__(256) void stream_header_unpack_kernel(const uint8_t *__restrict__ hdr,
                                                                   int16_t *__restrict__ cherry_indices, StreamGeo geo) {
    const int Knp512 = (geo.ng * kStreamUnitK + 511) & ~511;
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < geo.C) cherry_indices[i] = (int16_t)reinterpret_cast<const uint16_t *>(hdr + Knp512)[i];
}

// weight * fp16(x * rs) on both halves of a pair (the rounding points of add_rmsnorm_kernel)
__device__ inline uint32_t stream_norm_pair(uint32_t xp, uint32_t wp, float rs) {
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

// A workgroup is W computing wavefronts plus S staging wavefronts and owns T tiles (W % T == 0):
// computing wavefront w works on tile w % T and takes the units g = w / T, w / T + W / T, ... of it
// (at most L), D loads in flight.  Staging wavefront j prepares NB consecutive blocks of 512
// compacted positions (S * NB blocks cover K); with S == 0 the computing wavefronts stage NB blocks
// each themselves.  P > 1: the workgroup walks up to P tiles of its member one after the other
// (launches with more tiles than the chip holds workgroups), the activations staged once.
//
// Order of events.  A CU admits vector loads only as fast as earlier ones return, so whatever a
// wavefront does after queueing weight loads waits in that queue with them.  Therefore: (1) every
// wavefront requests its 16 bytes per thread of the activation vector alone (those that stage
// also the gather table and the cherry columns from the stream header), copies them to LDS and
// meets the others -- under a microsecond after the start, nothing else being in the queues;
// (2) the computing wavefronts queue their cherry rows, scales and first D units, while the
// staging wavefronts, which never touch the weight stream, gather the activations into MFMA
// operand order (conflict-free: lane l takes positions l, l + 64, ...) and add up every unit's
// activations for the grid offset (S == 0: the computing wavefronts do so after queueing their
// loads -- LDS work does not wait behind vector loads); (3) all meet at a second workgroup
// barrier, then a computing wavefront consumes its units in order, refilling every slot it frees.
//
// Up to kStreamMaxGroup layers that read the same activation row (q / k / v, gate / up) share
// one launch: consecutive ranges of workgroups belong to consecutive members, each with its own
// stream (header and tile records) and output.  NORM: the row is RMS-normalised while it is
// staged -- norm_w * fp16(x * rsqrt(mean(x^2) + eps)), the rounding points of the decoder's
// separate norm kernel -- at the price of one more workgroup barrier.
template <int BITS, int W, int T, int D, int L, int S, int NB, int XL, bool NORM, bool GROUP, int P>
__global__ __launch_bounds__(64 * (W + S)) void stream_kernel(const __half *__restrict__ x,
                                                              const uint8_t *__restrict__ stream0, int K0,
                                                              uint32_t hdr_bytes0, StreamGroup grp,
                                                              const __half *__restrict__ norm_w, float eps,
                                                              int accumulate, StreamGeo geo, StreamWalk walk) {
    // x, stream0 (= grp.stream[0]), K0 (= geo.K) and hdr_bytes0 (= geo.hdr_bytes) lead the argument
    // list as plain scalars: what the first loads of a workgroup need sits in the first bytes of the
    // kernel-argument segment (and can be preloaded into scalar registers by the dispatcher when
    // the file is built with a kernel-argument preload count).
    static_assert(L % 4 == 0 && W % T == 0 && D <= L, "");
    static_assert(P == 1 || (T == 1 && L % D == 0 && GROUP), "walking several tiles: one tile at a time, ring slots fixed per unit");
    // Which member this workgroup works for.  Every member's fields are first pinned in scalar
    // registers: left to itself the compiler turns the selects into ONE load at a selected
    // kernel-argument address, i.e. a second, dependent memory round trip in front of the header
    // loads (measured: +1.1 us on the 4096 -> 11008 layer).  A single layer skips all of it.
    const int bid = blockIdx.x;
    const uint8_t *__restrict__ stream = stream0;
    __half *__restrict__ mul = grp.mul[0];
    int N = grp.N[0], wg = bid;
    int member_wgs = 1;  // (P > 1) workgroups that share this member's tiles: this one takes wg, wg + member_wgs, ...
    if constexpr (GROUP) {
        const uint8_t *s1 = grp.stream[1], *s2 = grp.stream[2];
        __half *o1 = grp.mul[1], *o2 = grp.mul[2];
        int n1 = grp.N[1], n2 = grp.N[2], t1 = grp.tile_begin[1], t2 = grp.tile_begin[2], cnt = grp.count;
        asm volatile("" : "+s"(stream), "+s"(s1), "+s"(s2), "+s"(mul), "+s"(o1), "+s"(o2));
        asm volatile("" : "+s"(N), "+s"(n1), "+s"(n2), "+s"(t1), "+s"(t2), "+s"(cnt));
        const bool m1 = cnt > 1 && bid >= t1, m2 = cnt > 2 && bid >= t2;
        stream = m2 ? s2 : m1 ? s1 : stream;
        mul = m2 ? o2 : m1 ? o1 : mul;
        N = m2 ? n2 : m1 ? n1 : N;
        wg = bid - (m2 ? t2 : m1 ? t1 : 0);  // workgroup index within the member
        if constexpr (P > 1) {
            int g0 = walk.wgs[0], g1 = walk.wgs[1], g2 = walk.wgs[2];
            asm volatile("" : "+s"(g0), "+s"(g1), "+s"(g2));
            member_wgs = m2 ? g2 : m1 ? g1 : g0;
        }
    }
    constexpr int WT = W / T;
    constexpr int NT = 64 * (W + S);
    constexpr int UB = BITS == 4 ? 1024 : 768;
    constexpr float kGrid = BITS == 4 ? -7.5f : -3.5f;
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kq = lane >> 4, nn = lane & 15;
    const bool stager = wave >= W;
    // The staging wavefronts are the critical path until the second barrier: they get the issue
    // slots first.  (Measured on 4096 -> 11008: 6.34 / 6.08 us against 6.48 / 6.24, 4-bit / 3-bit;
    // with 8 computing wavefronts 4.02 against 3.94 on 4096 -> 4096, and with the fused RMSNorm
    // 7.51 against 7.21 on the q/k/v group, so only here.)
    if constexpr (S > 0 && W == 4 && !NORM) {
        if (stager) __builtin_amdgcn_s_setprio(3);
    }
    const int K = K0, C = geo.C, ng = geo.ng;
    const int Knp = ng * kStreamUnitK;
    const int Cp = (C + 31) & ~31;
    const int Knp512 = (Knp + 511) & ~511;
    const int nblk = Knp512 >> 9;  // blocks of 512 positions
    // LDS: 16 spare bytes | raw activations (+ zeros) | compacted activations | cherry activations | unit sums | partial outputs
    unsigned short *s_raw = reinterpret_cast<unsigned short *>(smem + 16);
    unsigned short *s_xs = s_raw + K + kStreamRawPad;
    unsigned short *s_xc = s_xs + Knp512;
    float *s_xsum = reinterpret_cast<float *>(s_xc + Cp);
    float *s_red = s_xsum + 4 * nblk;

    // ---- (1) raw activations, everyone; gather table and cherry columns, staging wavefronts
    su4 xr[XL];
    su2 tb[NB];
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)x, 0, K * 2, kSFlags);
    const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc((void *)stream, 0, (int)hdr_bytes0, kSFlags);
#pragma unroll
    for (int i = 0; i < XL; i++)
        if (i * NT * 8 < K) xr[i] = __builtin_amdgcn_raw_buffer_load_b128(rx, (uint32_t)(tid + i * NT) * 16u, 0, 0);
    // S == 0: no staging wavefronts -- every computing wavefront stages NB blocks itself, between
    // queueing its weight loads and using them
    const int ws = S == 0 ? wave : wave - W;  // index among the wavefronts that stage
    const int b0 = ws * NB, b1 = min(nblk, b0 + NB);
    uint32_t ci0 = 0, ci1 = 0;
    if (stager || S == 0) {
#pragma unroll
        for (int i = 0; i < NB; i++)
            tb[i] = __builtin_amdgcn_raw_buffer_load_b64(rh, b0 + i < b1 ? (uint32_t)((b0 + i) * 512 + lane * 8) : kSOob, 0, 0);
        if (ws == 0) {
            ci0 = __builtin_amdgcn_raw_buffer_load_b16(rh, lane < Cp ? (uint32_t)(Knp512 + lane * 2) : kSOob, 0, 0);
            ci1 = __builtin_amdgcn_raw_buffer_load_b16(rh, lane + 64 < Cp ? (uint32_t)(Knp512 + (lane + 64) * 2) : kSOob, 0, 0);
        }
    }
    if constexpr (NORM) {
        su4 nr[XL];
        const __amdgpu_buffer_rsrc_t rn = __builtin_amdgcn_make_buffer_rsrc((void *)norm_w, 0, K * 2, kSFlags);
#pragma unroll
        for (int i = 0; i < XL; i++)
            if (i * NT * 8 < K) nr[i] = __builtin_amdgcn_raw_buffer_load_b128(rn, (uint32_t)(tid + i * NT) * 16u, 0, 0);
        float ss = 0.f;  // pieces past K read as zeros
#pragma unroll
        for (int i = 0; i < XL; i++)
            if (i * NT * 8 < K) {
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
        for (int wv = 0; wv < W + S; wv++) t += s_red[wv];
        const float rs = rsqrtf(t / (float)K + eps);
        // one dword at a time (the scheduling barriers keep the temporaries of different dwords
        // from being live together: this phase must not set the kernel's register count)
#pragma unroll
        for (int i = 0; i < XL; i++)
            if (i * NT * 8 < K) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    xr[i][j] = stream_norm_pair(xr[i][j], nr[i][j], rs);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
    }
#pragma unroll
    for (int i = 0; i < XL; i++)
        if (i * NT * 8 < K && (tid + i * NT) * 8 < K) reinterpret_cast<su4 *>(s_raw)[tid + i * NT] = xr[i];
    // zeros behind the activations: what padding positions (and padded cherry columns) read
    if (tid < kStreamRawPad / 8) reinterpret_cast<su4 *>(s_raw)[(K >> 3) + tid] = (su4){0u, 0u, 0u, 0u};
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");

    float tot = 0.f;
    // ---- (2b) xs[k] = x[k + low(k)] for the positions of blocks [b0, b1), and the sum of every unit
    auto stage_blocks = [&]() {
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
        if (ws == 0) {
            if (lane < Cp) s_xc[lane] = s_raw[ci0 & 0xffffu];
            if (lane + 64 < Cp) s_xc[lane + 64] = s_raw[ci1 & 0xffffu];
        }
    };
    // What a computing wavefront does between queueing its loads and using the staged activations:
    // it meets the staging wavefronts at a workgroup barrier (no polling of LDS, which takes LDS
    // cycles from the wavefronts that stage); without staging wavefronts it stages its own blocks first.
    auto staged_wait = [&]() {
        if constexpr (S == 0) stage_blocks();
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    };
    if (stager) {
        stage_blocks();
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
    } else {
        // ---- (2a) computing wavefront.  Lane group kq keeps the scales of the units i with
        // i % 4 == kq (every lane group ends up with the same MFMA results, so each finishes a
        // quarter of the units; the quarters are added at the end).  Every unit of a tile past the
        // last reads zeros through an empty descriptor.
        if constexpr (P > 1) {
            // ---- several tiles, one after the other: tile wg, wg + member_wgs, ... of this member.
            // The ring of D loads runs across tile boundaries (slot i % D always holds unit i of
            // some tile, L % D == 0), the cherry rows and scales of the next tile are requested as
            // soon as the registers of the current ones are free, and nothing but the running sum
            // is kept per tile: its 16 partial outputs per wavefront wait in LDS for the end.
            const int cls = wave;
            const int ntl = (N + kStreamTileCols - 1) / kStreamTileCols;
            const __amdgpu_buffer_rsrc_t rt = __builtin_amdgcn_make_buffer_rsrc(
                (void *)(stream + geo.hdr_bytes), 0, (int)min((unsigned long long)ntl * geo.record_bytes, 0xffffffffull), kSFlags);
            uint32_t sc[L / 4];
            su4 wbuf[D];
            su4 cw[4];
            const bool cherry_wave = cls == W - 1;
            int tcur = wg;
            bool vcur = tcur < ntl;
            uint32_t tb = (uint32_t)tcur * geo.record_bytes;
            auto load_cherry = [&](uint32_t base, bool valid) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int lg = 4 * j + kq;
                    cw[j] = __builtin_amdgcn_raw_buffer_load_b128(
                        rt, valid && 8 * lg < C ? geo.off_cherry + (uint32_t)(lg * 16 + nn) * 16u : kSOob, base, 2);
                }
            };
            const uint32_t sc_off = (uint32_t)((cls + kq * W) * 32 + nn * 2);
            auto load_scale = [&](int i4, uint32_t base, bool valid) -> uint32_t {
                return __builtin_amdgcn_raw_buffer_load_b16(rt, valid && cls + (4 * i4 + kq) * W < ng ? sc_off : kSOob,
                                                            base + 4 * i4 * W * 32, 0);
            };
            const uint32_t w_off = geo.off_units + (uint32_t)(cls * UB + lane * (BITS * 4));
            auto load_unit = [&](int i, uint32_t base, bool valid) -> su4 {
                const uint32_t off = valid && cls + i * W < ng ? w_off : kSOob;
                if constexpr (BITS == 4) {
                    return __builtin_amdgcn_raw_buffer_load_b128(rt, off, base + i * W * UB, 2);
                } else {
                    const su3 v = __builtin_amdgcn_raw_buffer_load_b96(rt, off, base + i * W * UB, 2);
                    return (su4){v[0], v[1], v[2], 0u};
                }
            };
            if (cherry_wave) load_cherry(tb, vcur);
#pragma unroll
            for (int i = 0; i < L / 4; i++) sc[i] = load_scale(i, tb, vcur);
#pragma unroll
            for (int i = 0; i < D; i++) wbuf[i] = load_unit(i, tb, vcur);
            staged_wait();
#pragma unroll 1
            for (int j = 0; j < P; j++) {
                const int tnext = tcur + member_wgs;
                const bool vnext = j + 1 < P && tnext < ntl;
                const uint32_t tbn = (uint32_t)tnext * geo.record_bytes;
                float totc = 0.f;
                if (cherry_wave) {
                    sf4_t dc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int q = 0; q < 4; q++)
                        if (32 * q < C) {
                            const sh8_t a = *reinterpret_cast<const sh8_t *>(s_xc + 32 * q + 8 * kq);
                            dc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, as_h8(cw[q]), dc, 0, 0, 0);
                        }
                    totc = dc[0];
                    load_cherry(tbn, vnext);
                }
                float tt = 0.f;
#pragma unroll
                for (int i = 0; i < L; i++) {
                    // a unit past the last one of the column reads zero codes and a zero scale; its
                    // activations are taken from unit 0, which every layer has and which is always
                    // staged, so that no stale LDS contents (NaN patterns) meet the zeros
                    const bool real = cls + i * W < ng;
                    const int up = real ? cls + i * W : 0;
                    const float sf = (i & 3) == kq ? __half2float(__ushort_as_half((unsigned short)sc[i >> 2])) : 0.f;
                    const su4 w = wbuf[i % D];
                    const float v = unit_dot<BITS>(w, s_xs + up * kStreamUnitK + 32 * kq);
                    wbuf[i % D] = i + D < L ? load_unit(i + D, tb, vcur) : load_unit(i + D - L, tbn, vnext);
                    tt += (v + kGrid * s_xsum[up]) * sf;
                    if ((i & 3) == 3) sc[i >> 2] = load_scale(i >> 2, tbn, vnext);
                }
                tt = swap32_add(tt, tt);
                tt = swap16_add(tt, tt) + totc;
                if (kq == 0) s_red[(j * W + wave) * 16 + nn] = tt;
                tcur = tnext;
                vcur = vnext;
                tb = tbn;
                if (!vcur) break;
            }
        } else {
            const int tl = wave % T, cls = wave / T;
            const int tile = wg * T + tl;
            const bool tile_ok = tile * kStreamTileCols < N;
            const __amdgpu_buffer_rsrc_t rt = __builtin_amdgcn_make_buffer_rsrc(
                (void *)(stream + geo.hdr_bytes + (size_t)(tile_ok ? tile : 0) * geo.record_bytes), 0,
                tile_ok ? (int)geo.record_bytes : 0, kSFlags);
            uint32_t sc[L / 4];
            su4 wbuf[D];
            su4 cw[4];
            const bool cherry_wave = cls == WT - 1;
            // cherry rows first: they are consumed first, which frees their registers for the units
            if (cherry_wave) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int lg = 4 * j + kq;
                    cw[j] = __builtin_amdgcn_raw_buffer_load_b128(
                        rt, 8 * lg < C ? geo.off_cherry + (uint32_t)(lg * 16 + nn) * 16u : kSOob, 0, 2);
                }
            }
            const uint32_t sc_off = (uint32_t)((cls + kq * WT) * 32 + nn * 2);
#pragma unroll
            for (int i = 0; i < L / 4; i++)
                sc[i] = __builtin_amdgcn_raw_buffer_load_b16(rt, cls + (4 * i + kq) * WT < ng ? sc_off : kSOob, 4 * i * WT * 32, 0);
            const uint32_t w_off = geo.off_units + (uint32_t)(cls * UB + lane * (BITS * 4));
            auto load_unit = [&](int i) -> su4 {
                // a unit past the last reads zeros: the vector offset alone lies outside the descriptor
                const uint32_t off = cls + i * WT < ng ? w_off : kSOob;
                if constexpr (BITS == 4) {
                    return __builtin_amdgcn_raw_buffer_load_b128(rt, off, i * WT * UB, 2);
                } else {
                    const su3 v = __builtin_amdgcn_raw_buffer_load_b96(rt, off, i * WT * UB, 2);
                    return (su4){v[0], v[1], v[2], 0u};
                }
            };
#pragma unroll
            for (int i = 0; i < D; i++) wbuf[i] = load_unit(i);
            // ---- (3) the staged activations are needed from here on
            staged_wait();
            float totc = 0.f;
            if (cherry_wave) {
                sf4_t dc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (32 * j < C) {
                        const sh8_t a = *reinterpret_cast<const sh8_t *>(s_xc + 32 * j + 8 * kq);
                        dc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, as_h8(cw[j]), dc, 0, 0, 0);
                    }
                totc = dc[0];
            }
            // units, in order; every consumed slot is refilled with the unit D further on
            const unsigned short *xa0 = s_xs + cls * kStreamUnitK + 32 * kq;
            const float *xsum0 = s_xsum + cls;
#pragma unroll
            for (int i = 0; i < L; i++) {
                if (cls + i * WT >= ng) break;
                const float sf = (i & 3) == kq ? __half2float(__ushort_as_half((unsigned short)sc[i >> 2])) : 0.f;
                const su4 w = wbuf[i % D];
                const float v = unit_dot<BITS>(w, xa0 + i * WT * kStreamUnitK);
                if (i + D < L) wbuf[i % D] = load_unit(i + D);
                tot += (v + kGrid * xsum0[i * WT]) * sf;
            }
            // the four lane groups' quarters
            tot = swap32_add(tot, tot);
            tot = swap16_add(tot, tot) + totc;
            if (kq == 0) s_red[wave * 16 + nn] = tot;
        }
    }

    // ---- across the tile's wavefronts, then one store per output
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    if constexpr (P > 1) {
        const int ntl = (N + kStreamTileCols - 1) / kStreamTileCols;
        for (int o = tid; o < 16 * P; o += NT) {
            const int j = o >> 4, tile = wg + j * member_wgs, n = tile * 16 + (o & 15);
            if (tile < ntl && n < N) {
                float v = 0.f;
#pragma unroll
                for (int c = 0; c < W; c++) v += s_red[(j * W + c) * 16 + (o & 15)];
                if (accumulate) v += __half2float(mul[n]);
                mul[n] = __float2half_rn(v);
            }
        }
    } else if (tid < 16 * T) {
        const int otl = tid >> 4, n = (wg * T + otl) * 16 + (tid & 15);
        if (n < N) {
            float v = 0.f;
#pragma unroll
            for (int c = 0; c < WT; c++) v += s_red[(c * T + otl) * 16 + (tid & 15)];
            if (accumulate) v += __half2float(mul[n]);
            mul[n] = __float2half_rn(v);
        }
    }
}

// ---- 2 to 16 activation rows over the stream --------------------------------------------------
// The matrix-core tile that the one-row kernel fills with 16 copies of one row takes 16 different
// rows at the same price: A = the rows' activations (lane (kq, n) reads row n), B = the masked
// code fields, D = 16 rows x 16 columns (lane (kq, n) ends up with rows 4 kq .. 4 kq + 3 of column n).
// A workgroup still owns whole columns -- no split-K, no workspace -- but needs the compacted
// activations of ALL rows in LDS (rows x K x 2 bytes: 128 KB for 16 rows of 4096), so (1) a small
// launch compacts the rows once into a scratch buffer (x[k + low(k)], the per-unit sums, the
// cherry activations), (2) the main launch has at most as many workgroups as the chip holds at a
// time, each copying that buffer into LDS once and then walking tiles wg, wg + G, ...

// one block of 512 compacted positions of one row per wavefront
__global__ __launch_bounds__(64) void stream_rows_prep_kernel(const __half *__restrict__ x,
                                                              const uint8_t *__restrict__ hdr,
                                                              unsigned short *__restrict__ xs,
                                                              float *__restrict__ xsum,
                                                              unsigned short *__restrict__ xc, StreamGeo geo) {
    const int blk = blockIdx.x, row = blockIdx.y, lane = threadIdx.x, kq = lane >> 4, nn = lane & 15;
    const int K = geo.K, Knp512 = (geo.ng * kStreamUnitK + 511) & ~511, Cp = (geo.C + 31) & ~31, nu = Knp512 >> 7;
    const unsigned short *xrow = reinterpret_cast<const unsigned short *>(x) + (size_t)row * K;
    // the table and the raw columns the block can touch (its 512 positions + up to 128 cherry
    // columns in front) are requested together; the gather then runs out of LDS: one memory round
    // trip instead of two dependent ones
    __shared__ __align__(16) unsigned short s_seg[512 + 128];
    const su2 t = *reinterpret_cast<const su2 *>(hdr + (size_t)blk * 512 + lane * 8);
    const int q0 = blk * 512 + lane * 8, q1 = blk * 512 + 512 + lane * 8;
    const su4 zero = {0u, 0u, 0u, 0u};
    const su4 v0 = q0 < K ? *reinterpret_cast<const su4 *>(xrow + q0) : zero;        // K % 8 == 0
    const su4 v1 = lane < 16 && q1 < K ? *reinterpret_cast<const su4 *>(xrow + q1) : zero;
    *reinterpret_cast<su4 *>(s_seg + lane * 8) = v0;
    if (lane < 16) *reinterpret_cast<su4 *>(s_seg + 512 + lane * 8) = v1;
    __syncthreads();
    unsigned short h[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        h[j] = s_seg[64 * j + lane + (int)((t[j >> 2] >> (8 * (j & 3))) & 0xffu)];  // columns >= K hold zeros
        xs[(size_t)row * Knp512 + blk * 512 + 64 * j + lane] = h[j];
    }
    float f[4];
#pragma unroll
    for (int u = 0; u < 4; u++)
        f[u] = __half2float(__ushort_as_half(h[2 * u])) + __half2float(__ushort_as_half(h[2 * u + 1]));
    const float s01 = swap32_add(f[0], f[1]);
    const float s23 = swap32_add(f[2], f[3]);
    const float r = row_sum(swap16_add(s01, s23));
    if (nn == 0) xsum[(size_t)row * nu + blk * 4 + ((kq >> 1) | ((kq & 1) << 1))] = r;
    if (blk == 0)
        for (int c = lane; c < Cp; c += 64) {
            const int col = reinterpret_cast<const uint16_t *>(hdr + Knp512)[c];
            xc[(size_t)row * Cp + c] = col < K ? xrow[col] : (unsigned short)0;
        }
}

// the four rows (4 kq .. 4 kq + 3) x one column that this lane holds of a unit's 16 x 16 product
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
        // positions 24..27 sit at bit 0, 28..31 at bit 3: moved to bit 0 so that one 16x16x32 step takes all eight
        const su4 b1 = {y[1] & 0x00070007u, y[2] & 0x00070007u, (y[1] >> 3) & 0x00070007u, (y[2] >> 3) & 0x00070007u};
        sf4_t d0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, as_h8(b0), zero4, 0, 0, 0);
        const sf4_t d3 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a2, as_h8(b2), zero4, 0, 0, 0);
        const sf4_t d6 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a4, as_h8(b4), zero4, 0, 0, 0);
        d0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, as_h8(b1), d0, 0, 0, 0);
        return d0 * 16777216.0f + d3 * 2097152.0f + d6 * 262144.0f;
    }
}

constexpr int kRowsSkew = 8;     // halves added to a row's stride in LDS: 16 rows' 16-byte reads hit 16 different bank groups

// TEAMS teams of W wavefronts, each team on a tile of its own; wavefront c of a team takes units
// c, c + W, ... (L at most) of every tile the team comes to, all L loads in flight, each slot
// refilled with the next tile's unit as soon as it is consumed.  Tiles are dealt so that the
// workgroups' loads stay even: team t of workgroup b takes tiles b + t * G, + TEAMS * G, ...
// STAGE: the workgroup compacts the rows itself (raw rows and the header's table through LDS)
// instead of reading rows that stream_rows_prep_kernel compacted -- one launch instead of two,
// possible while raw and compacted rows fit LDS together (8 rows of 4096).
template <int BITS, int W, int L, int TEAMS, bool STAGE>
__global__ __launch_bounds__(64 * W * TEAMS) void stream_rows_kernel(
    const unsigned short *__restrict__ xs_g, const float *__restrict__ xsum_g, const unsigned short *__restrict__ xc_g,
    const uint8_t *__restrict__ stream, __half *__restrict__ mul, int B, int accumulate, StreamGeo geo) {
    constexpr int NW = W * TEAMS, NT = 64 * NW;
    constexpr int UB = BITS == 4 ? 1024 : 768;
    constexpr float kGrid = BITS == 4 ? -7.5f : -3.5f;
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int team = wave / W, cls = wave % W;
    const int kq = lane >> 4, nn = lane & 15;
    const int K = geo.K, C = geo.C, ng = geo.ng, N = geo.N;
    const int Knp512 = (ng * kStreamUnitK + 511) & ~511, Cp = (C + 31) & ~31, nu = Knp512 >> 7;
    const int RS = Knp512 + kRowsSkew, CS = Cp + kRowsSkew;
    unsigned short *s_x = reinterpret_cast<unsigned short *>(smem);                 // [B][RS]
    unsigned short *s_xc = s_x + (size_t)B * RS;                                     // [B][CS]
    float *s_xsum = reinterpret_cast<float *>(s_xc + (size_t)B * CS);                // [16][nu] (rows >= B unused)
    float *s_red = s_xsum + 16 * nu;                                                 // [NW][256]

    if constexpr (STAGE) {
        // ---- (1) raw rows (each followed by 8 zeros: what padding positions read), the gather table
        // and the cherry columns -> LDS; then xs[r][p] = x[r][p + low(p)], unit sums, cherry activations
        const int XS = K + 8;                                                       // raw row stride
        unsigned short *s_raw = reinterpret_cast<unsigned short *>(s_red + NW * 256);  // [B][XS]
        uint8_t *s_tab = reinterpret_cast<uint8_t *>(s_raw + (size_t)B * XS);          // [Knp512]
        unsigned short *s_col = reinterpret_cast<unsigned short *>(s_tab + Knp512);    // [Cp]
        const int per_row = K >> 3, total = B * per_row;
        for (int base = 0; base < total; base += 4 * NT) {
            su4 v[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int c = base + i * NT + tid;
                if (c < total) v[i] = reinterpret_cast<const su4 *>(xs_g)[c];  // xs_g: the raw rows here
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int c = base + i * NT + tid;
                if (c < total) {
                    const int row = c / per_row, col = c - row * per_row;
                    *reinterpret_cast<su4 *>(s_raw + (size_t)row * XS + col * 8) = v[i];
                }
            }
        }
        for (int c = tid; c < B; c += NT) *reinterpret_cast<su4 *>(s_raw + (size_t)c * XS + K) = (su4){0u, 0u, 0u, 0u};
        for (int c = tid; c < (Knp512 >> 4); c += NT) reinterpret_cast<su4 *>(s_tab)[c] = reinterpret_cast<const su4 *>(stream)[c];
        for (int c = tid; c < Cp; c += NT) s_col[c] = reinterpret_cast<const unsigned short *>(stream + Knp512)[c];
        __syncthreads();
        const int nblk = Knp512 >> 9;
        for (int q = wave; q < B * nblk; q += NW) {  // (row, block of 512 positions) pairs
            const int row = q / nblk, blk = q - row * nblk;
            const su2 t = *reinterpret_cast<const su2 *>(s_tab + blk * 512 + lane * 8);
            const unsigned short *raw = s_raw + (size_t)row * XS;
            unsigned short h[8];
#pragma unroll
            for (int j = 0; j < 8; j++)
                h[j] = raw[min(blk * 512 + 64 * j + lane + (int)((t[j >> 2] >> (8 * (j & 3))) & 0xffu), K)];
#pragma unroll
            for (int j = 0; j < 8; j++) s_x[(size_t)row * RS + blk * 512 + 64 * j + lane] = h[j];
            float f[4];
#pragma unroll
            for (int u = 0; u < 4; u++)
                f[u] = __half2float(__ushort_as_half(h[2 * u])) + __half2float(__ushort_as_half(h[2 * u + 1]));
            const float s01 = swap32_add(f[0], f[1]);
            const float s23 = swap32_add(f[2], f[3]);
            const float r = row_sum(swap16_add(s01, s23));
            if (nn == 0) s_xsum[row * nu + blk * 4 + ((kq >> 1) | ((kq & 1) << 1))] = r;
        }
        for (int c = tid; c < B * Cp; c += NT) {
            const int row = c / Cp, m = c - row * Cp;
            s_xc[row * CS + m] = s_raw[(size_t)row * XS + min((int)s_col[m], K)];
        }
    } else {
        // ---- (1) the compacted rows, their unit sums and cherry activations: global -> LDS, 16 bytes a piece
        const int per_row = Knp512 >> 3, total = B * per_row;
        for (int base = 0; base < total; base += 8 * NT) {
            su4 v[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int c = base + i * NT + tid;
                if (c < total) v[i] = reinterpret_cast<const su4 *>(xs_g)[c];
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int c = base + i * NT + tid;
                if (c < total) {
                    const int row = c / per_row, col = c - row * per_row;
                    *reinterpret_cast<su4 *>(s_x + (size_t)row * RS + col * 8) = v[i];
                }
            }
        }
        for (int c = tid; c < B * nu; c += NT) s_xsum[c] = xsum_g[c];
        for (int c = tid; c < B * Cp; c += NT) s_xc[(c / Cp) * CS + c % Cp] = xc_g[c];
    }
    __syncthreads();

    // ---- (2) tiles
    const int ntl = (N + kStreamTileCols - 1) / kStreamTileCols;
    const int G = gridDim.x, stride = G * TEAMS;
    const __amdgpu_buffer_rsrc_t rt = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(stream + geo.hdr_bytes), 0, (int)min((unsigned long long)ntl * geo.record_bytes, 0xffffffffull), kSFlags);
    uint32_t sc[L];
    su4 wbuf[L];
    su4 cw[4];
    const bool cherry_wave = cls == W - 1;
    auto load_cherry = [&](uint32_t base, bool valid) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int lg = 4 * j + kq;
            cw[j] = __builtin_amdgcn_raw_buffer_load_b128(
                rt, valid && 8 * lg < C ? geo.off_cherry + (uint32_t)(lg * 16 + nn) * 16u : kSOob, base, 2);
        }
    };
    auto load_scale = [&](int i, uint32_t base, bool valid) -> uint32_t {
        return __builtin_amdgcn_raw_buffer_load_b16(rt, valid && cls + i * W < ng ? (uint32_t)(cls * 32 + nn * 2) : kSOob,
                                                    base + i * W * 32, 0);
    };
    const uint32_t w_off = geo.off_units + (uint32_t)(cls * UB + lane * (BITS * 4));
    auto load_unit = [&](int i, uint32_t base, bool valid) -> su4 {
        const uint32_t off = valid && cls + i * W < ng ? w_off : kSOob;
        if constexpr (BITS == 4) {
            return __builtin_amdgcn_raw_buffer_load_b128(rt, off, base + i * W * UB, 2);
        } else {
            const su3 v = __builtin_amdgcn_raw_buffer_load_b96(rt, off, base + i * W * UB, 2);
            return (su4){v[0], v[1], v[2], 0u};
        }
    };
    int tile = blockIdx.x + team * G;
    bool vcur = tile < ntl;
    uint32_t tb = (uint32_t)tile * geo.record_bytes;
    if (cherry_wave) load_cherry(tb, vcur);
#pragma unroll
    for (int i = 0; i < L; i++) sc[i] = load_scale(i, tb, vcur);
#pragma unroll
    for (int i = 0; i < L; i++) wbuf[i] = load_unit(i, tb, vcur);
    // lanes of rows that do not exist (n >= B) read row 0: their results are never stored
    const int arow = nn < B ? nn : 0;
    const unsigned short *xrow = s_x + (size_t)arow * RS + 32 * kq;
    const float *xsrow = s_xsum + (4 * kq) * nu;
    // the loop count is the same for every wavefront of the workgroup (barriers inside): as long as
    // the workgroup's first team, which has the lowest tile, has one
    for (int t0 = blockIdx.x; t0 < ntl; t0 += stride) {
        const int tnext = tile + stride;
        const bool vnext = tnext < ntl;
        const uint32_t tbn = (uint32_t)tnext * geo.record_bytes;
        sf4_t acc = {0.f, 0.f, 0.f, 0.f};
        if (cherry_wave) {
#pragma unroll
            for (int q = 0; q < 4; q++)
                if (32 * q < C) {
                    const sh8_t a = *reinterpret_cast<const sh8_t *>(s_xc + arow * CS + 32 * q + 8 * kq);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, as_h8(cw[q]), acc, 0, 0, 0);
                }
            load_cherry(tbn, vnext);
        }
#pragma unroll
        for (int i = 0; i < L; i++) {
            // a unit past the column's last reads zero codes and a zero scale; its activations and
            // unit sum are taken from unit 0, which every layer has (unit `cls` need not exist when
            // a column has fewer units than the team has wavefronts)
            const int up = cls + i * W < ng ? cls + i * W : 0;
            const float sf = __half2float(__ushort_as_half((unsigned short)sc[i]));
            const sf4_t v = unit_dot_rows<BITS>(wbuf[i], xrow + up * kStreamUnitK);
            wbuf[i] = load_unit(i, tbn, vnext);
            sc[i] = load_scale(i, tbn, vnext);
#pragma unroll
            for (int r = 0; r < 4; r++) acc[r] += (v[r] + kGrid * xsrow[r * nu + up]) * sf;
        }
        float *red = s_red + (size_t)wave * 256;
#pragma unroll
        for (int r = 0; r < 4; r++) red[(4 * kq + r) * 16 + nn] = acc[r];
        __syncthreads();
        // 256 outputs per team, summed over its W wavefronts by the team's first 256 threads (all of
        // them with 4 wavefronts, half of them with 8)
        {
            const int t = tid - team * 64 * W;
            if (t < 256 && vcur) {
                const int row = t >> 4, n = tile * kStreamTileCols + (t & 15);
                if (row < B && n < N) {
                    float v = 0.f;
#pragma unroll
                    for (int c = 0; c < W; c++) v += s_red[(size_t)(team * W + c) * 256 + t];
                    __half *o = mul + (size_t)row * N + n;
                    if (accumulate) v += __half2float(*o);
                    *o = __float2half_rn(v);
                }
            }
        }
        __syncthreads();
        tile = tnext;
        vcur = vnext;
        tb = tbn;
    }
}

// ---- rows kept in registers -------------------------------------------------------------------
// The A operands of a wavefront's units do not change from tile to tile, so a wavefront that walks
// tiles can hold them in registers: 8 units x 4 operands x 4 VGPRs = 128 VGPRs, loaded once from a
// buffer that a first launch wrote in operand order.  No LDS traffic for the activations, and 16
// rows of 8192 channels (256 KB, more than LDS holds) become possible.  One workgroup of 8
// wavefronts per compute unit: teams of W = ceil(units / 8) wavefronts, 8 / W teams.

// grid: one block per unit (+ one for the cherry activations), 256 threads.  xf[unit][m][lane][8]:
// lane (kq, n) gets row n (zeros from row B on), compacted positions 128 unit + 32 kq + 8 m + 0..7.
__global__ __launch_bounds__(256) void stream_rows_frag_kernel(const __half *__restrict__ x,
                                                               const uint8_t *__restrict__ hdr,
                                                               su4 *__restrict__ xf, float *__restrict__ xsum,
                                                               su4 *__restrict__ xcf, int B, StreamGeo geo) {
    __shared__ __align__(16) unsigned short s_seg[16][256 + 8];
    __shared__ uint8_t s_tab[128];
    const int u = blockIdx.x, t = threadIdx.x, lane = t & 63, m = t >> 6, kq = lane >> 4, nn = lane & 15;
    const int K = geo.K, Knp512 = (geo.ng * kStreamUnitK + 511) & ~511;
    const unsigned short *xh = reinterpret_cast<const unsigned short *>(x);
    if (u == geo.ng) {  // cherry activations: positions 32 m + 8 kq + 0..7 of the cherry list
        su4 v = {0u, 0u, 0u, 0u};
        unsigned short h[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int col = reinterpret_cast<const uint16_t *>(hdr + Knp512)[32 * m + 8 * kq + j];  // padding entries hold K
            h[j] = nn < B && 32 * m < ((geo.C + 31) & ~31) && col < K ? xh[(size_t)nn * K + col] : (unsigned short)0;
        }
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = (uint32_t)h[2 * j] | ((uint32_t)h[2 * j + 1] << 16);
        xcf[m * 64 + lane] = v;
        return;
    }
    // the unit's raw columns (its 128 positions + up to 128 cherry columns in front) of all rows, and its table bytes
    for (int c = t; c < 16 * 32; c += 256) {
        const int row = c >> 5, q = c & 31, pos = u * kStreamUnitK + q * 8;
        su4 v = {0u, 0u, 0u, 0u};
        if (row < B && pos < K) v = *reinterpret_cast<const su4 *>(xh + (size_t)row * K + pos);  // K % 8 == 0
        *reinterpret_cast<su4 *>(&s_seg[row][q * 8]) = v;
    }
    if (t < 128) {
        const int p = u * kStreamUnitK + t;
        s_tab[t] = hdr[(p >> 9) * 512 + (p & 63) * 8 + ((p & 511) >> 6)];
    }
    __syncthreads();
    {
        unsigned short h[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int i = 32 * kq + 8 * m + j;
            h[j] = s_seg[nn][i + s_tab[i]];  // columns >= K hold zeros
        }
        su4 v;
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = (uint32_t)h[2 * j] | ((uint32_t)h[2 * j + 1] << 16);
        xf[((size_t)u * 4 + m) * 64 + lane] = v;
    }
    {   // the unit's sum of activations per row: 16 threads per row, 8 positions each
        const int row = t >> 4, part = t & 15;
        float sacc = 0.f;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int i = part * 8 + j;
            sacc += __half2float(__ushort_as_half(s_seg[row][i + s_tab[i]]));
        }
        sacc = row_sum(sacc);
        if (part == 0) xsum[row * geo.ng + u] = sacc;
    }
}

template <int BITS, typename WB>
__device__ inline sf4_t unit_dot_regs(const WB w, const su4 (&a)[4]) {
    const sf4_t zero4 = {0.f, 0.f, 0.f, 0.f};
    if constexpr (BITS == 4) {
        const su4 y = {w[0] >> 8, w[1] >> 8, w[2] >> 8, w[3] >> 8};
        const su4 b0 = {w[0] & 0x000f000fu, y[0] & 0x000f000fu, w[1] & 0x000f000fu, y[1] & 0x000f000fu};
        const su4 b1 = {w[2] & 0x000f000fu, y[2] & 0x000f000fu, w[3] & 0x000f000fu, y[3] & 0x000f000fu};
        const su4 b2 = {w[0] & 0x00f000f0u, y[0] & 0x00f000f0u, w[1] & 0x00f000f0u, y[1] & 0x00f000f0u};
        const su4 b3 = {w[2] & 0x00f000f0u, y[2] & 0x00f000f0u, w[3] & 0x00f000f0u, y[3] & 0x00f000f0u};
        sf4_t dl = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_h8(a[0]), as_h8(b0), zero4, 0, 0, 0);
        sf4_t dh = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_h8(a[2]), as_h8(b2), zero4, 0, 0, 0);
        dl = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_h8(a[1]), as_h8(b1), dl, 0, 0, 0);
        dh = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_h8(a[3]), as_h8(b3), dh, 0, 0, 0);
        return dl * 16777216.0f + dh * 1048576.0f;
    } else {
        const su3 y = {w[0] >> 9, w[1] >> 9, w[2] >> 9};
        const uint32_t z = (y[0] & 0x00400040u) | ((y[1] & 0x00400040u) << 1) | ((y[2] & 0x00400040u) << 2);
        const su4 b0 = {w[0] & 0x00070007u, w[1] & 0x00070007u, w[2] & 0x00070007u, y[0] & 0x00070007u};
        const su4 b2 = {w[0] & 0x00380038u, w[1] & 0x00380038u, w[2] & 0x00380038u, y[0] & 0x00380038u};
        const su4 b4 = {w[0] & 0x01c001c0u, w[1] & 0x01c001c0u, w[2] & 0x01c001c0u, z};
        // positions 24..27 sit at bit 0, 28..31 at bit 3: moved to bit 0 so that one 16x16x32 step takes all eight
        const su4 b1 = {y[1] & 0x00070007u, y[2] & 0x00070007u, (y[1] >> 3) & 0x00070007u, (y[2] >> 3) & 0x00070007u};
        sf4_t d0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_h8(a[0]), as_h8(b0), zero4, 0, 0, 0);
        const sf4_t d3 = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_h8(a[1]), as_h8(b2), zero4, 0, 0, 0);
        const sf4_t d6 = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_h8(a[2]), as_h8(b4), zero4, 0, 0, 0);
        d0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_h8(a[3]), as_h8(b1), d0, 0, 0, 0);
        return d0 * 16777216.0f + d3 * 2097152.0f + d6 * 262144.0f;
    }
}

// W wavefronts per team, 8 / W teams, L units per wavefront (W * L units per column at most), the
// loads of R consecutive tiles of a team in flight (R * L per wavefront).
constexpr int kRowsRegChunk = 4;  // tile steps whose partial outputs stream_rows_reg_kernel keeps in LDS between two barriers

// KS > 1 (layers deeper than W * L units): the workgroups form KS slices, slice z takes units
// [z * US, (z + 1) * US) of every tile it visits and writes its fp32 partial sums to
// part[z][16][N]; rows_reduce_kernel adds the slices up.  The cherry channels belong to slice 0.
template <int BITS, int W, int L, int R, bool KSPLIT = false>
__global__ __launch_bounds__(512) void stream_rows_reg_kernel(const su4 *__restrict__ xf, const float *__restrict__ xsum_g,
                                                              const su4 *__restrict__ xcf,
                                                              const uint8_t *__restrict__ stream,
                                                              __half *__restrict__ mul, int B, int accumulate,
                                                              StreamGeo geo, float *__restrict__ part = nullptr,
                                                              int KS = 1, int US = 0) {
    constexpr int TEAMS = 8 / W;
    constexpr int UB = BITS == 4 ? 1024 : 768;
    constexpr float kGrid = BITS == 4 ? -7.5f : -3.5f;
    // partial outputs of kRowsRegChunk consecutive tile steps: [step][wavefront][16 rows x 16 columns].  A
    // wavefront reaches a barrier only when the compute unit has accepted all its requests so far, the
    // next tiles' weights included: two barriers per tile cost more than the arithmetic between
    // them, so the partial sums wait here and the workgroup meets once per chunk of steps.
    extern __shared__ __align__(16) unsigned char smem[];
    float *s_red = reinterpret_cast<float *>(smem);                  // [kRowsRegChunk][8][256]
    float *s_xsum = s_red + kRowsRegChunk * 8 * 256;                 // [16][ng]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int team = wave / W, cls = wave % W;
    const int kq = lane >> 4, nn = lane & 15;
    const int C = geo.C, ng = geo.ng, N = geo.N;
    const int G = KSPLIT ? gridDim.x / KS : gridDim.x;          // workgroups that share the tiles
    const int slice = KSPLIT ? blockIdx.x / G : 0, bx = KSPLIT ? blockIdx.x - slice * G : blockIdx.x;
    const int u0 = KSPLIT ? slice * US : 0;                       // the slice's first unit
    const int ucount = KSPLIT ? min(US, ng - u0) : ng;            // and how many it has
    // ---- requests, in the order their data is needed: the small shared operands (cherry
    // activations, unit sums: they go through LDS and gate the barrier), the wavefront's own A
    // operands, then the first R tiles' weights -- all queued BEFORE the barrier, so that the weight
    // stream is under way while the workgroup still waits for its activations
    const bool cherry_wave = cls == W - 1 && slice == 0;
    __shared__ su4 s_acr[4 * 64];  // the cherry operands (read once per tile by each team's last wavefront)
    su4 acr_v = {0u, 0u, 0u, 0u};
    if (tid < 4 * 64) acr_v = xcf[tid];
    constexpr int XJ = KSPLIT ? 8 : 4;  // 512 * XJ unit sums at most: 16 rows of 64 units, 256 when split
    float xs_v[XJ];
#pragma unroll
    for (int j = 0; j < XJ; j++) xs_v[j] = tid + 512 * j < 16 * ng ? xsum_g[tid + 512 * j] : 0.f;
    su4 areg[L][4];
#pragma unroll
    for (int i = 0; i < L; i++) {
        const int u = u0 + cls + i * W;
#pragma unroll
        for (int m = 0; m < 4; m++)
            areg[i][m] = cls + i * W < ucount && nn < B ? xf[((size_t)u * 4 + m) * 64 + lane] : (su4){0u, 0u, 0u, 0u};  // (rows from B on are zeros: not fetched)
    }
    __builtin_amdgcn_sched_barrier(0);

    const int ntl = (N + kStreamTileCols - 1) / kStreamTileCols;
    const int stride = G * TEAMS;
    const __amdgpu_buffer_rsrc_t rt = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(stream + geo.hdr_bytes), 0, (int)min((unsigned long long)ntl * geo.record_bytes, 0xffffffffull), kSFlags);
    typedef typename std::conditional<BITS == 4, su4, su3>::type WB;  // a unit: 4 or 3 dwords per lane
    uint32_t sc[R][L];
    WB wbuf[R][L];
    su4 cw[R][4];
    auto load_cherry = [&](su4 (&dst)[4], uint32_t base, bool valid) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int lg = 4 * j + kq;
            dst[j] = __builtin_amdgcn_raw_buffer_load_b128(
                rt, valid && 8 * lg < C ? geo.off_cherry + (uint32_t)(lg * 16 + nn) * 16u : kSOob, base, 2);
        }
    };
    auto load_scale = [&](int i, uint32_t base, bool valid) -> uint32_t {
        return __builtin_amdgcn_raw_buffer_load_b16(rt, valid && cls + i * W < ucount ? (uint32_t)((u0 + cls) * 32 + nn * 2) : kSOob,
                                                    base + i * W * 32, 0);
    };
    const uint32_t w_off = geo.off_units + (uint32_t)((u0 + cls) * UB + lane * (BITS * 4));
    auto load_unit = [&](int i, uint32_t base, bool valid) -> WB {
        const uint32_t off = valid && cls + i * W < ucount ? w_off : kSOob;
        if constexpr (BITS == 4) {
            return __builtin_amdgcn_raw_buffer_load_b128(rt, off, base + i * W * UB, 2);
        } else {
            return __builtin_amdgcn_raw_buffer_load_b96(rt, off, base + i * W * UB, 2);
        }
    };
    // slot s of the ring holds the tile the team reaches in its (R * j + s)-th step
    int tile[R];
    bool valid[R];
#pragma unroll
    for (int s = 0; s < R; s++) {
        tile[s] = bx + team * G + s * stride;
        valid[s] = tile[s] < ntl;
        const uint32_t tb = (uint32_t)tile[s] * geo.record_bytes;
        if (cherry_wave) load_cherry(cw[s], tb, valid[s]);
#pragma unroll
        for (int i = 0; i < L; i++) sc[s][i] = load_scale(i, tb, valid[s]);
#pragma unroll
        for (int i = 0; i < L; i++) wbuf[s][i] = load_unit(i, tb, valid[s]);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (tid < 4 * 64) s_acr[tid] = acr_v;
#pragma unroll
    for (int j = 0; j < XJ; j++)
        if (tid + 512 * j < 16 * ng) s_xsum[tid + 512 * j] = xs_v[j];
    __syncthreads();
    const float *xsrow = s_xsum + (4 * kq) * ng;
    // the loop count is the same for every wavefront of the workgroup (barriers inside): as long as
    // the workgroup's first team, which has the lowest tile, has one in slot 0
    int step = 0;   // tile steps of the workgroup so far (the same count in every wavefront)
    auto flush = [&](int first_step, int count) {
        // sums over a tile's wavefronts and the stores, for the `count` steps that started at `first_step`
        __syncthreads();
        for (int o = tid; o < count * TEAMS * 256; o += 512) {
            const int j = o / (TEAMS * 256), rem = o - j * TEAMS * 256, tm = rem >> 8, t = rem & 255;
            const int tl = bx + tm * G + (first_step + j) * stride;
            const int row = t >> 4, n = tl * kStreamTileCols + (t & 15);
            if (tl < ntl && row < B && n < N) {
                float v = 0.f;
#pragma unroll
                for (int c = 0; c < W; c++) v += s_red[(j * 8 + tm * W + c) * 256 + t];
                if constexpr (KSPLIT) {
                    part[((size_t)slice * 16 + row) * N + n] = v;
                } else {
                    __half *o16 = mul + (size_t)row * N + n;
                    if (accumulate) v += __half2float(*o16);
                    *o16 = __float2half_rn(v);
                }
            }
        }
        __syncthreads();
    };
    int chunk_first = 0;
    // the loop count is the same for every wavefront of the workgroup (barriers inside): as long as
    // the workgroup's first team, which has the lowest tile, has one in slot 0
    for (int t0 = bx; t0 < ntl; t0 += R * stride) {
#pragma unroll
        for (int s = 0; s < R; s++) {
            const int tnext = tile[s] + R * stride;
            const bool vnext = tnext < ntl;
            const uint32_t tbn = (uint32_t)tnext * geo.record_bytes;
            sf4_t acc = {0.f, 0.f, 0.f, 0.f};
            if (cherry_wave) {
#pragma unroll
                for (int q = 0; q < 4; q++)
                    if (32 * q < C)
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_h8(s_acr[q * 64 + lane]), as_h8(cw[s][q]), acc, 0, 0, 0);
                load_cherry(cw[s], tbn, vnext);
            }
#pragma unroll
            for (int i = 0; i < L; i++) {
                const int up = cls + i * W < ucount ? u0 + cls + i * W : 0;  // (a unit past the last: zero codes, zero scale, zero operands; unit 0's sum, which exists)
                const float sf = __half2float(__ushort_as_half((unsigned short)sc[s][i]));
                const sf4_t v = unit_dot_regs<BITS, WB>(wbuf[s][i], areg[i]);
                wbuf[s][i] = load_unit(i, tbn, vnext);
                sc[s][i] = load_scale(i, tbn, vnext);
#pragma unroll
                for (int r = 0; r < 4; r++) acc[r] += (v[r] + kGrid * xsrow[r * ng + up]) * sf;
            }
            float *red = s_red + ((step - chunk_first) * 8 + wave) * 256;
#pragma unroll
            for (int r = 0; r < 4; r++) red[(4 * kq + r) * 16 + nn] = acc[r];
            tile[s] = tnext;
            valid[s] = vnext;
            step++;
            if (step - chunk_first == kRowsRegChunk) {
                flush(chunk_first, kRowsRegChunk);
                chunk_first = step;
            }
        }
    }
    if (step > chunk_first) flush(chunk_first, step - chunk_first);
}

// Sum of the KS slices' partial outputs (part[z][16][N], fp32) of a split rows launch, rounded to
// fp16 once: out[b][n] = (accumulate ? out[b][n] : 0) + sum_z part[z][b][n].
__global__ __launch_bounds__(256) void rows_reduce_kernel(const float *__restrict__ part, __half *__restrict__ mul, int B, int N,
                                                          int KS, int accumulate) {
    const int n = blockIdx.x * 256 + threadIdx.x, row = blockIdx.y;
    if (n >= N || row >= B) return;
    float v = 0.f;
    for (int z = 0; z < KS; z++) v += part[((size_t)z * 16 + row) * N + n];
    __half *o16 = mul + (size_t)row * N + n;
    if (accumulate) v += __half2float(*o16);
    *o16 = __float2half_rn(v);
}

constexpr int kStreamWalk = 8;  // tiles one workgroup takes at most when a launch has more tiles than resident workgroups

static size_t stream_lds_bytes(const StreamGeo &g, int W, int tiles_per_wg = kStreamWalk) {
    const int Knp512 = (g.ng * kStreamUnitK + 511) & ~511, Cp = (g.C + 31) & ~31;
    return 16 + (size_t)(g.K + kStreamRawPad + Knp512 + Cp) * 2 + (size_t)(Knp512 / 128) * 4 +
           (size_t)W * 16 * 4 * tiles_per_wg;
}

// Launch geometries (W computing wavefronts, T tiles, D loads in flight, L units per wavefront at
// most, S staging wavefronts of NB blocks each), by the number of 128-position units of a column.
// One tile per workgroup throughout: whole tiles are the grain in which the work spreads over the
// CUs, and two tiles per workgroup measured 20-30 % slower on the 4096 -> 11008 layer for that
// reason.  All of a wavefront's loads are queued at once where the registers allow (D = L).
struct StreamCfg {
    int W, T, D, L, S, NB, max_units;
};
static constexpr StreamCfg kStreamCfgs[] = {
    {4, 1, 8, 8, 4, 2, 32},    // 0: K <= 4096 + cherries, more tiles than compute units
    {8, 1, 4, 4, 4, 2, 32},    // 1: K <= 4096 + cherries, about one tile per compute unit
    {8, 1, 8, 8, 0, 2, 64},    // 2: up to 64 units; the computing wavefronts stage the activations themselves
    {8, 1, 8, 12, 6, 4, 96},   // 3
    {8, 1, 8, 16, 4, 8, 128},  // 4
};
constexpr int kStreamCfgCount = sizeof(kStreamCfgs) / sizeof(kStreamCfgs[0]);


static int stream_pick(const StreamGeo &geo) {
    // Measured (us per launch, 4-bit / 3-bit; W computing + S staging wavefronts, L units each):
    // (entry 0 before its staging wavefronts got issue priority, which took 0.15 us off its single-layer figures)
    // 4096 -> 11008 (688 tiles): entry 0 6.49 / 6.25, entry 1 7.52 / 7.37, W4 L8 S0 6.90 / 6.56,
    //   W8 L4 S0 6.54 / 6.23, W4 L8 S1 6.39-7.76 (the single staging wavefront is the critical path and
    //   its speed moved by more than a microsecond with unrelated changes of the code: not used);
    // 4096 -> 4096 (256 tiles): entry 0 4.25, entry 1 3.93, W8 L4 S0 4.38;
    // RMSNorm + 3 x (4096 -> 4096) (768 tiles): entry 0 7.37, entry 1 11.6;
    // RMSNorm + 2 x (4096 -> 11008) (1376 tiles, workgroups walk two tiles): entry 0 10.9, entry 1 12.0;
    // 8192 -> 28672 (1792 tiles of 64 units, 7 per workgroup): entry 2 21.2, W8 L8 S4 22.2;
    // 8192 -> 8192: entry 2 9.5, entry 4 8.6; 5120 -> 13824 (3-bit): entry 2 10.4, W8 L12 S0 9.6.
    if (geo.ng <= 32) return geo.ntiles <= 320 ? 1 : 0;
    for (int i = 2; i < kStreamCfgCount; i++)
        if (geo.ng <= kStreamCfgs[i].max_units) return i;
    return -1;
}

constexpr int kStreamCus = 256;  // compute units of an MI355X

// Where the batch-1 matvec over the stream measured faster than the one over the checkpoint layout
// (us per launch, weights from HBM; checkpoint layout / stream): 4096 -> 4096 4.95 / 3.58 (3-bit
// 4.79 / 3.55), 4096 -> 11008 7.46 / 5.71 (6.79 / 5.15), 11008 -> 4096 7.04 / 5.91 (6.76 / 5.56),
// 8192 -> 8192 8.75 / 7.72, 8192 -> 1024 4.55 / 4.24, 8192 -> 28672 22.8 / 20.5, 28672 -> 8192 23.5 /
// 22.3, 5120 -> 5120 5.87 / 4.52 (5.57 / 4.65), 5120 -> 13824 10.15 / 8.2 (8.80 / 8.1), 13824 -> 5120
// 10.24 / 8.9 (8.81 / 8.5), 12288 -> 4096 7.90 / 6.5 (6.93 / 6.1), 8192 -> 5120 7.03 / 6.88 (6.50 / 6.71),
// 6144 -> 6144 6.75 / 6.40 (6.45 / 6.42), 5120 -> 20480 (3-bit) 12.3 / 10.2: everywhere the launch with
// one workgroup per compute unit takes the layer, within 3 % at worst.
bool stream_faster(int bits, int K, int N, int C) {
    const StreamGeo g = stream_geo(bits, K, N, C);
    if (g.ng <= 32) return true;
    return stream_cu_supported(bits, K, C, &N, 1);
}

// the launch shapes of this file (several workgroups per compute unit) take the layer
static bool stream_old_supported(const StreamGeo &geo) {
    const int i = stream_pick(geo);
    return i >= 0 && stream_lds_bytes(geo, kStreamCfgs[i].W) <= 160 * 1024;
}

bool stream_supported(int bits, int B, int K, int N, int C, int G) {
    if (bits != 3 && bits != 4) return false;
    if (B != 1) return false;
    if (G <= 0 || G % kStreamUnitK) return false;
    if (K - C <= 0 || C > 128 || K > 32768) return false;
    if (K % 8 || N % 8 || C % 8) return false;
    const StreamGeo geo = stream_geo(bits, K, N, C);
    // tile records are addressed with 32-bit byte offsets, and an offset with bit 31 set is how the
    // kernels read zeros for units that do not exist: the whole stream stays below 2 GiB
    if ((unsigned long long)geo.hdr_bytes + (unsigned long long)geo.ntiles * geo.record_bytes >= 0x7fff0000ull) return false;
    return stream_old_supported(geo) || stream_cu_supported(bits, K, C, &N, 1);
}

constexpr int kMaxDevices = 64;  // GPUs of one process that the per-device launch plans cover

struct DevicePlan {
    bool big_lds = false, asked = false;
    int regs[2] = {0, 0};
};
// vector registers per lane of a kernel (0 if the runtime does not say)
static int kernel_vgprs(const void *k) {
    hipFuncAttributes attr;
    if (hipFuncGetAttributes(&attr, k) == hipSuccess && attr.numRegs > 0) return attr.numRegs;
    (void)hipGetLastError();
    return 0;
}

template <int BITS, int I, bool NORM>
static hipError_t launch_stream_cfg(const __half *vec, const StreamGroup &grp, const __half *norm_w, float eps,
                                    int accumulate, const StreamGeo &geo, hipStream_t s) {
    constexpr StreamCfg c = kStreamCfgs[I];
    constexpr int XL = stream_x_loads(c.max_units, 64 * (c.W + c.S));
    // what the kernel's fixed-size register arrays assume
    if (geo.ng * kStreamUnitK > c.NB * 512 * (c.S ? c.S : c.W) || geo.K > XL * 8 * 64 * (c.W + c.S) || geo.ng > c.max_units ||
        ceil_div(geo.ng, c.W / c.T) > c.L)
        return hipErrorInvalidValue;
    // More tiles than the chip holds workgroups at a time: every workgroup walks several tiles of
    // its member (activations staged once, loads streaming across the tile boundaries) instead of
    // the launch running in rounds that each pay the start-up chain again.
    constexpr bool kCanWalk = c.T == 1 && c.L % c.D == 0;
    auto kern_one = stream_kernel<BITS, c.W, c.T, c.D, c.L, c.S, c.NB, XL, NORM, false, 1>;
    auto kern_grp = stream_kernel<BITS, c.W, c.T, c.D, c.L, c.S, c.NB, XL, NORM, true, 1>;
    auto kern_walk = stream_kernel<BITS, c.W, c.T, c.D, c.L, c.S, c.NB, XL, NORM, true, kCanWalk ? kStreamWalk : 1>;
    const size_t lds_walk = stream_lds_bytes(geo, c.W, kStreamWalk);
    if (stream_lds_bytes(geo, c.W, 1) > 160 * 1024) return hipErrorInvalidValue;
    // Per instantiation and device, found once under a lock (the entry points are re-entrant): the
    // 160 KB dynamic-LDS limit raised, and the register counts of the one-tile and the walking kernel.
    static std::mutex mu;
    static DevicePlan plans[kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    int regs_one = 0, regs_walk = 0;
    {
        std::lock_guard<std::mutex> lock(mu);
        DevicePlan &pl = plans[dev];
        if (lds_walk > 48 * 1024 && !pl.big_lds) {
            for (const void *k : {reinterpret_cast<const void *>(kern_one), reinterpret_cast<const void *>(kern_grp),
                                  reinterpret_cast<const void *>(kern_walk)}) {
                hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (e != hipSuccess) return e;
            }
            pl.big_lds = true;
        }
        if (kCanWalk && !pl.asked) {
            pl.regs[0] = kernel_vgprs(reinterpret_cast<const void *>(kern_grp));
            pl.regs[1] = kernel_vgprs(reinterpret_cast<const void *>(kern_walk));
            pl.asked = true;
        }
        regs_one = pl.regs[0];
        regs_walk = pl.regs[1];
    }
    // Workgroups that the chip holds at a time, of the kernel that takes one tile per workgroup and
    // of the one that walks (more registers): from the register counts (512 VGPRs per SIMD lane,
    // allocated in eights, at most 8 wavefronts per SIMD, four SIMDs) and the LDS.
    auto resident = [&](int regs, size_t lds_bytes) {
        int per_cu = 20 / (c.W + c.S);
        if (regs > 0) {
            int per_simd = 512 / ((regs + 7) / 8 * 8);
            if (per_simd > 8) per_simd = 8;
            per_cu = 4 * per_simd / (c.W + c.S);
        }
        const int by_lds = (int)((160 * 1024) / lds_bytes);
        if (per_cu > by_lds) per_cu = by_lds;
        return kStreamCus * (per_cu < 1 ? 1 : per_cu);
    };
    int slots_one = 0, slots_walk = 0;
    if (kCanWalk && lds_walk <= 160 * 1024) {
        slots_one = resident(regs_one, stream_lds_bytes(geo, c.W, 1));
        slots_walk = resident(regs_walk, lds_walk);
    }
    // one round of one-tile workgroups if they all fit; else as few tiles per workgroup as fill the chip once
    int per_wg = 1;
    if (kCanWalk && lds_walk <= 160 * 1024 && slots_one > 0 && geo.ntiles > slots_one) per_wg = ceil_div(geo.ntiles, slots_walk);
    if (per_wg > kStreamWalk) per_wg = kStreamWalk;
    const bool walk = per_wg > 1;
    const size_t lds = stream_lds_bytes(geo, c.W, walk ? kStreamWalk : 1);
    auto kern = walk ? kern_walk : grp.count > 1 ? kern_grp : kern_one;
    // members are told apart by workgroup index: each starts at a workgroup of its own
    // (The order of the kernel arguments is not free: with the walk fields inside StreamGroup, which
    // moves everything behind it by 8 bytes, the single-layer kernel measured 7.2 us instead of 6.5
    // on the 4096 -> 11008 layer, its instructions being the same.)
    StreamGroup g = grp;
    StreamWalk gw;
    int wgs = 0;
    for (int i = 0; i < kStreamMaxGroup; i++) {
        g.tile_begin[i] = wgs;
        const int tiles_i = ceil_div(ceil_div(grp.N[i], kStreamTileCols), c.T);
        gw.wgs[i] = ceil_div(tiles_i, per_wg);
        if (i < grp.count) wgs += gw.wgs[i];
    }
    const dim3 grid(wgs), block(64 * (c.W + c.S));
    hipLaunchKernelGGL(kern, grid, block, lds, s, vec, g.stream[0], geo.K, geo.hdr_bytes, g, norm_w, eps, accumulate, geo, gw);
    return hipGetLastError();
}

template <int BITS, bool NORM>
static hipError_t launch_stream_bits(const __half *vec, const StreamGroup &grp, const __half *norm_w, float eps,
                                     int accumulate, const StreamGeo &geo, hipStream_t s) {
    switch (stream_pick(geo)) {
        case 0: return launch_stream_cfg<BITS, 0, NORM>(vec, grp, norm_w, eps, accumulate, geo, s);
        case 1: return launch_stream_cfg<BITS, 1, NORM>(vec, grp, norm_w, eps, accumulate, geo, s);
        case 2: return launch_stream_cfg<BITS, 2, NORM>(vec, grp, norm_w, eps, accumulate, geo, s);
        case 3: return launch_stream_cfg<BITS, 3, NORM>(vec, grp, norm_w, eps, accumulate, geo, s);
        case 4: return launch_stream_cfg<BITS, 4, NORM>(vec, grp, norm_w, eps, accumulate, geo, s);
        default: return hipErrorInvalidValue;
    }
}

// Which of the two launch shapes takes a call: the one with one workgroup per compute unit
// (cq_stream_cu.hip) wherever it measured faster.
static bool stream_cu_preferred(int bits, int K, int C, const int *Ns, int count, bool norm) {
    if (!stream_cu_supported(bits, K, C, Ns, count)) return false;
    int tiles = 0;
    for (int i = 0; i < count; i++) tiles += ceil_div(Ns[i], kStreamTileCols);
    StreamGeo geo = stream_geo(bits, K, Ns[0], C);
    geo.ntiles = tiles;
    if (!stream_old_supported(geo)) return true;
    // measurement switch, read once: CHERRYQ_STREAM_CU=0 the older shape wherever it can, =1 the newer
    static const int forced = [] {
        const char *e = getenv("CHERRYQ_STREAM_CU");
        return e && e[0] == '0' ? 0 : e && e[0] == '1' ? 1 : -1;
    }();
    if (forced >= 0) return forced == 1;
    // Measured (us, older shape / one workgroup per compute unit; 4-bit unless noted): single layers
    // 4096 -> 11008 6.35 / 5.68, 4096 -> 4096 3.99 / 3.58, 8192 -> 8192 8.9 / 7.7, 5120 -> 5120 6.0 / 4.5,
    // 5120 -> 13824 10.7 / 8.2, 13824 -> 5120 11.6 / 8.9; RMSNorm + q/k/v (3 x 4096 -> 4096) 7.35 / 7.24
    // (3-bit 7.10 / 6.76), RMSNorm + gate/up (2 x 4096 -> 11008) 10.95 / 9.76 (3-bit 9.69 / 8.96), q/k/v
    // without norm 7.02 / 7.08, RMSNorm + 8192 -> (8192, 1024, 1024) 11.5 / 10.6, RMSNorm + 2 x (8192 ->
    // 28672) 40.2 / 38.9: the newer shape wherever it takes the launch.
    (void)norm;
    (void)geo;
    return true;
}


// `count` layers (at most kStreamMaxGroup) of the same bits / K / C that read the same activation
// row, in one launch; norm_w != nullptr fuses the RMSNorm of that row.
hipError_t launch_stream_group_old(int bits, const __half *vec, const __half *norm_w, float eps,
                                   const StreamMember *members, int count, int K, int C, int accumulate, hipStream_t s);

hipError_t launch_stream_group(int bits, const __half *vec, const __half *norm_w, float eps,
                               const StreamMember *members, int count, int K, int C, int accumulate, hipStream_t s) {
    if (count < 1 || count > kStreamMaxGroup) return hipErrorInvalidValue;
    int Ns[kStreamMaxGroup];
    for (int i = 0; i < count; i++) Ns[i] = members[i].N;
    if (stream_cu_preferred(bits, K, C, Ns, count, norm_w != nullptr))
        return launch_stream_cu(bits, vec, norm_w, eps, nullptr, members, count, K, C, accumulate, s);
    return launch_stream_group_old(bits, vec, norm_w, eps, members, count, K, C, accumulate, s);
}

// which of the two launch shapes cherryq_matvec_prepacked_f16 uses for a layer (for profiles and benchmarks)
bool stream_uses_cu(int bits, int K, int N, int C) { return stream_cu_preferred(bits, K, C, &N, 1, false); }

bool stream_gated_supported(int bits, int K, int N, int C) { return stream_cu_supported(bits, K, C, &N, 1); }

hipError_t launch_stream_gated(int bits, const __half *vec, const __half *gate, const uint8_t *stream, __half *mul,
                               int K, int N, int C, int accumulate, hipStream_t s) {
    const StreamMember m = {stream, mul, N};
    return launch_stream_cu(bits, vec, nullptr, 0.f, gate, &m, 1, K, C, accumulate, s);
}

hipError_t launch_stream_attn_out(int bits, const __half *part, const float *ml, const uint8_t *stream, __half *mul,
                                  int K, int N, int C, int accumulate, hipStream_t s) {
    const StreamMember m = {stream, mul, N};
    return launch_stream_cu(bits, part, nullptr, 0.f, nullptr, &m, 1, K, C, accumulate, s, ml);
}

int attn_max_slices() { return kAttnMaxSlices; }
int attn_out_slices() { return 4; }  // kCuAttnSlices of cq_stream_cu.hip

// the launch with one workgroup per tile (or per few tiles), several workgroups per compute unit
hipError_t launch_stream_group_old(int bits, const __half *vec, const __half *norm_w, float eps,
                                   const StreamMember *members, int count, int K, int C, int accumulate, hipStream_t s) {
    if (count < 1 || count > kStreamMaxGroup) return hipErrorInvalidValue;
    StreamGroup grp = {};
    grp.count = count;
    int tiles = 0, n_total = 0;
    for (int i = 0; i < kStreamMaxGroup; i++) {
        const StreamMember &m = members[i < count ? i : 0];
        grp.stream[i] = m.stream;
        grp.mul[i] = m.mul;
        grp.N[i] = m.N;
        grp.tile_begin[i] = tiles;
        if (i < count) {
            tiles += ceil_div(m.N, kStreamTileCols);
            n_total += m.N;
        }
    }
    // the geometry of one member (records, header) with the launch's total tile count
    StreamGeo geo = stream_geo(bits, K, members[0].N, C);
    geo.N = n_total;
    geo.ntiles = tiles;
    if (bits == 4)
        return norm_w ? launch_stream_bits<4, true>(vec, grp, norm_w, eps, accumulate, geo, s)
                      : launch_stream_bits<4, false>(vec, grp, nullptr, 0.f, accumulate, geo, s);
    return norm_w ? launch_stream_bits<3, true>(vec, grp, norm_w, eps, accumulate, geo, s)
                  : launch_stream_bits<3, false>(vec, grp, nullptr, 0.f, accumulate, geo, s);
}

hipError_t launch_stream(int bits, const __half *vec, const uint8_t *stream, __half *mul, int K, int N, int C,
                         int accumulate, hipStream_t s) {
    const StreamMember m = {stream, mul, N};
    return launch_stream_group(bits, vec, nullptr, 0.f, &m, 1, K, C, accumulate, s);
}

// Whether a group launch takes these layers (each must be supported on its own; the launch
// geometry follows the total number of tiles).
bool stream_group_supported(int bits, int K, int C, int G, const int *Ns, int count) {
    if (count < 1 || count > kStreamMaxGroup) return false;
    int tiles = 0;
    for (int i = 0; i < count; i++) {
        if (!stream_supported(bits, 1, K, Ns[i], C, G)) return false;
        tiles += ceil_div(Ns[i], kStreamTileCols);
    }
    StreamGeo geo = stream_geo(bits, K, Ns[0], C);
    geo.ntiles = tiles;
    return stream_old_supported(geo) || stream_cu_supported(bits, K, C, Ns, count);
}

// ---- 2 to 16 rows: sizes, support, launch
constexpr int kRowsMax = 16;

struct RowsScratch {
    size_t xs, xsum, xc, total;  // byte offsets of the compacted rows, their unit sums, their cherry activations
};
static RowsScratch rows_scratch(int B, const StreamGeo &g) {
    const size_t Knp512 = (size_t)((g.ng * kStreamUnitK + 511) & ~511), Cp = (size_t)((g.C + 31) & ~31);
    RowsScratch r;
    r.xs = 0;
    r.xsum = (B * Knp512 * 2 + 255) / 256 * 256;
    r.xc = r.xsum + (B * (Knp512 / 128) * 4 + 255) / 256 * 256;
    r.total = r.xc + (B * Cp * 2 + 255) / 256 * 256;
    return r;
}
static size_t rows_lds_bytes(int B, const StreamGeo &g, int waves, bool stage) {
    const size_t Knp512 = (size_t)((g.ng * kStreamUnitK + 511) & ~511), Cp = (size_t)((g.C + 31) & ~31);
    size_t bytes = B * (Knp512 + kRowsSkew) * 2 + B * (Cp + kRowsSkew) * 2 + 16 * (Knp512 / 128) * 4 + (size_t)waves * 256 * 4;
    if (stage) bytes += (size_t)B * (g.K + 8) * 2 + Knp512 + Cp * 2;
    return bytes;
}

// operand-order buffer of the register variant: units x 4 operands x 64 lanes x 16 bytes, the unit
// sums of 16 rows, the cherry operands
struct RowsFrag {
    size_t xf, xsum, xcf, total;
};
static RowsFrag rows_frag(const StreamGeo &g) {
    RowsFrag r;
    r.xf = 0;
    r.xsum = (size_t)g.ng * 4 * 64 * 16;
    r.xcf = r.xsum + ((size_t)16 * g.ng * 4 + 255) / 256 * 256;
    r.total = r.xcf + 4 * 64 * 16;
    return r;
}
// layers deeper than 64 units: slices of at most 64 units, each with its own share of the workgroups
constexpr int kRowsMaxSlices = 4;
// Measured (us per call, 4-bit, 16 rows; 2 / 3 / 4 / 5 / 8 slices): 11008 -> 4096 15.4 / 14.9 / 14.4 / 16.3 / 18.6,
// 28672 -> 8192 - / - / 32.6 / 37.9 / 34.0; 13824 -> 5120 3-bit 17.9 / 19.0 / 17.0 / 18.9 / 21.9.  Layers of up to
// 64 units are slower in slices (4096 -> 11008: 12.3 whole, 15.5 in two, 21.4 in four).
static int rows_slices(const StreamGeo &g) { return g.ng <= 64 ? 1 : kRowsMaxSlices; }

size_t stream_rows_scratch_bytes(int bits, int B, int K, int N, int C) {
    if (B < 2 || stream_cu_rows_supported(bits, B, K, N, C)) return 0;  // (one row, or the rows staged inside the one launch)
    const StreamGeo geo = stream_geo(bits, K, N, C);
    const int ks = rows_slices(geo);
    if (ks > 1) return rows_frag(geo).total + (size_t)ks * 16 * N * 4;  // the operands, then the slices' fp32 partial outputs
    const size_t a = rows_scratch(B < kRowsMax ? B : kRowsMax, geo).total, b = rows_frag(geo).total;
    return a > b ? a : b;
}

bool stream_rows_supported(int bits, int B, int K, int N, int C, int G) {
    if (B < 2 || B > kRowsMax) return false;
    if (!stream_supported(bits, 1, K, N, C, G)) return false;
    const StreamGeo geo = stream_geo(bits, K, N, C);
    // at most 8 units per wavefront, 8 wavefronts per team: 64 units, or up to 4 slices of that
    return ceil_div(geo.ng, rows_slices(geo)) <= 64;
}

template <int BITS, int W, int L, int TEAMS, bool STAGE>
static hipError_t launch_rows_cfg(const unsigned short *xs, const float *xsum, const unsigned short *xc,
                                  const uint8_t *stream, __half *mul, int B, int accumulate, const StreamGeo &geo,
                                  hipStream_t s) {
    auto kern = stream_rows_kernel<BITS, W, L, TEAMS, STAGE>;
    const size_t lds = rows_lds_bytes(B, geo, W * TEAMS, STAGE);
    if (lds > 160 * 1024 || ceil_div(geo.ng, W) > L) return hipErrorInvalidValue;
    if (lds > 48 * 1024) {
        static std::mutex mu;
        static bool big_lds[kMaxDevices] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
        std::lock_guard<std::mutex> lock(mu);
        if (!big_lds[dev]) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return e;
            big_lds[dev] = true;
        }
    }
    // one workgroup per compute unit (its teams share the rows in LDS); fewer when there are fewer tiles
    int grid = ceil_div(geo.ntiles, TEAMS);
    if (grid > kStreamCus) grid = kStreamCus;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * W * TEAMS), lds, s, xs, xsum, xc, stream, mul, B, accumulate, geo);
    return hipGetLastError();
}

// the kernels launch_stream_rows runs for a shape, as a profiler's kernel trace names them
const char *stream_rows_kernel_name(int bits, int B, int K, int N, int C) {
    const StreamGeo geo = stream_geo(bits, K, N, C);
    if (stream_cu_rows_supported(bits, B, K, N, C)) return "cq::stream_cu_rows_kernel";
    if (rows_slices(geo) > 1) return "cq::stream_rows_frag_kernel + cq::stream_rows_reg_kernel (slices of units) + cq::rows_reduce_kernel";
    if (B >= 8 || geo.ng > 32 || rows_lds_bytes(B, geo, 8, false) > 160 * 1024)
        return "cq::stream_rows_frag_kernel + cq::stream_rows_reg_kernel";
    return B <= 4 ? "cq::stream_rows_kernel (rows staged in the launch)" : "cq::stream_rows_prep_kernel + cq::stream_rows_kernel";
}

// vec (B, K), mul (B, N), 2 <= B <= 16; scratch: stream_rows_scratch_bytes(), 256-byte aligned
hipError_t launch_stream_rows(int bits, const __half *vec, const uint8_t *stream, __half *mul, int B, int K, int N,
                              int C, int accumulate, void *scratch, hipStream_t s) {
    const StreamGeo geo = stream_geo(bits, K, N, C);
    // two to eight rows in the one-workgroup-per-compute-unit shape where it takes the layer: no launch in
    // front, no scratch (4096 -> 11008, us: 2 rows 9.9 -> 6.6, 4 rows 10.5 -> 7.4, 8 rows 11.7 -> 8.6)
    if (stream_cu_rows_supported(bits, B, K, N, C))
        return launch_stream_cu_rows(bits, vec, stream, mul, B, K, N, C, accumulate, s);
    // Two main kernels.  Measured (us, whole call, 4-bit; rows in LDS / rows in registers): 4096 -> 11008
    // 5 rows 12.0 / 12.4, 8 rows 12.4 / 12.5, 16 rows 14.1 / 12.6; 4096 -> 4096 8 rows 9.9 / 9.4, 16 rows
    // 12.4 / 9.6; 8192 -> 28672 8 rows 35.2 / 27.6, 16 rows - / 29.2; 8192 -> 8192 8 rows 16.7 / 14.8.
    const int ks = rows_slices(geo);
    if (ks > 1) {
        // Deeper than 64 units: the tiles' units split over ks slices of workgroups (each keeps only
        // its slice of the operands in registers), fp32 partial outputs per slice, one more launch
        // that adds them up in slice order.  (The slice that finishes last adding them up inside the
        // launch -- device-scope fences around an arrival counter -- measured 50 us slower per call.)
        const RowsFrag f = rows_frag(geo);
        su4 *xf = reinterpret_cast<su4 *>(reinterpret_cast<char *>(scratch) + f.xf);
        float *xsum = reinterpret_cast<float *>(reinterpret_cast<char *>(scratch) + f.xsum);
        su4 *xcf = reinterpret_cast<su4 *>(reinterpret_cast<char *>(scratch) + f.xcf);
        float *part = reinterpret_cast<float *>(reinterpret_cast<char *>(scratch) + f.total);
        const int us = ceil_div(geo.ng, ks);
        if (us > 64) return hipErrorInvalidValue;
        const int per = geo.ntiles < kStreamCus / ks ? geo.ntiles : kStreamCus / ks;  // workgroups of one slice
        hipLaunchKernelGGL(stream_rows_frag_kernel, dim3(geo.ng + 1), dim3(256), 0, s, vec, stream, xf, xsum, xcf, B, geo);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        const size_t lds = (size_t)kRowsRegChunk * 8 * 256 * 4 + (size_t)16 * geo.ng * 4;
#define CQ_SPLIT_GO(BITS_, L_, R_)                                                                                     \
    hipLaunchKernelGGL((stream_rows_reg_kernel<BITS_, 8, L_, R_, true>), dim3(per * ks), dim3(512), lds, s, xf, xsum, xcf,  \
                       stream, mul, B, accumulate, geo, part, ks, us)
        if (bits == 4) {
            if (us <= 32) CQ_SPLIT_GO(4, 4, 2);
            else CQ_SPLIT_GO(4, 8, 1);
        } else {
            if (us <= 32) CQ_SPLIT_GO(3, 4, 2);
            else CQ_SPLIT_GO(3, 8, 1);
        }
#undef CQ_SPLIT_GO
        e = hipGetLastError();
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(rows_reduce_kernel, dim3(ceil_div(N, 256), B), dim3(256), 0, s, part, mul, B, N, ks, accumulate);
        return hipGetLastError();
    }
    if (B >= 8 || geo.ng > 32 || rows_lds_bytes(B, geo, 8, false) > 160 * 1024) {
        // the rows as matrix-core operands in a buffer, then the kernel that keeps them in registers
        const RowsFrag f = rows_frag(geo);
        su4 *xf = reinterpret_cast<su4 *>(reinterpret_cast<char *>(scratch) + f.xf);
        float *xsum = reinterpret_cast<float *>(reinterpret_cast<char *>(scratch) + f.xsum);
        su4 *xcf = reinterpret_cast<su4 *>(reinterpret_cast<char *>(scratch) + f.xcf);
        hipLaunchKernelGGL(stream_rows_frag_kernel, dim3(geo.ng + 1), dim3(256), 0, s, vec, stream, xf, xsum, xcf, B, geo);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        const bool w4 = geo.ng <= 32;
        const int grid = geo.ntiles < kStreamCus ? geo.ntiles : kStreamCus;  // one team of 8 wavefronts per workgroup
        const size_t lds = (size_t)kRowsRegChunk * 8 * 256 * 4 + (size_t)16 * geo.ng * 4;
#define CQ_REG_GO(BITS_, W_, L_, R_)                                                                                  \
    hipLaunchKernelGGL((stream_rows_reg_kernel<BITS_, W_, L_, R_>), dim3(grid), dim3(512), lds, s, xf, xsum, xcf, stream, mul,  \
                       B, accumulate, geo)
        // up to 32 units: 4 per wavefront and the loads of two tiles in flight (measured on 4096 ->
        // 11008, 16 rows: 12.6 us against 13.8 with two teams of 4 wavefronts x 8 units); else 8 per wavefront
        if (bits == 4) {
            if (w4) CQ_REG_GO(4, 8, 4, 2);
            else CQ_REG_GO(4, 8, 8, 1);
        } else {
            if (w4) CQ_REG_GO(3, 8, 4, 2);
            else CQ_REG_GO(3, 8, 8, 1);
        }
#undef CQ_REG_GO
        return hipGetLastError();
    }
    // teams of 8 wavefronts, 4 units each for rows of up to 32 units and 8 beyond; two teams per
    // workgroup when every compute unit gets at least two tiles
    const bool l4 = geo.ng <= 32;
    // (two teams of 8 units per wavefront do not fit the 128 registers of a 1024-thread workgroup: they
    // spilled, and a kernel with scratch memory also launches several microseconds slower)
    const int teams = l4 && geo.ntiles >= 2 * kStreamCus && rows_lds_bytes(B, geo, 16, false) <= 160 * 1024 ? 2 : 1;
    // compaction inside the workgroup for a few rows (measured on 4096 -> 11008: 2 rows 10.4 us against
    // 11.6 with the compaction launch, 4 rows 11.4 against 11.8, 8 rows 13.7 against 12.8)
    const bool stage = B <= 4 && (K % 8 == 0) && rows_lds_bytes(B, geo, 8 * teams, true) <= 160 * 1024;
    const unsigned short *xs;
    const float *xsum = nullptr;
    const unsigned short *xc = nullptr;
    if (stage) {
        xs = reinterpret_cast<const unsigned short *>(vec);
    } else {
        const RowsScratch sc = rows_scratch(B, geo);
        unsigned short *xs_w = reinterpret_cast<unsigned short *>(reinterpret_cast<char *>(scratch) + sc.xs);
        float *xsum_w = reinterpret_cast<float *>(reinterpret_cast<char *>(scratch) + sc.xsum);
        unsigned short *xc_w = reinterpret_cast<unsigned short *>(reinterpret_cast<char *>(scratch) + sc.xc);
        const int nblk = ((geo.ng * kStreamUnitK + 511) & ~511) >> 9;
        hipLaunchKernelGGL(stream_rows_prep_kernel, dim3(nblk, B), dim3(64), 0, s, vec, stream, xs_w, xsum_w, xc_w, geo);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        xs = xs_w;
        xsum = xsum_w;
        xc = xc_w;
    }
#define CQ_ROWS_GO(BITS_, W_, L_, T_)                                                                                \
    return stage ? launch_rows_cfg<BITS_, W_, L_, T_, true>(xs, xsum, xc, stream, mul, B, accumulate, geo, s)        \
                 : launch_rows_cfg<BITS_, W_, L_, T_, false>(xs, xsum, xc, stream, mul, B, accumulate, geo, s)
#define CQ_ROWS(BITS_)                                                                                               \
    do {                                                                                                             \
        if (l4 && teams == 2) CQ_ROWS_GO(BITS_, 8, 4, 2);                                                            \
        if (l4) CQ_ROWS_GO(BITS_, 8, 4, 1);                                                                          \
        CQ_ROWS_GO(BITS_, 8, 8, 1);                                                                                  \
    } while (0)
    if (bits == 4) CQ_ROWS(4);
    CQ_ROWS(3);
#undef CQ_ROWS
#undef CQ_ROWS_GO
}

hipError_t launch_stream_pack(int bits, const uint8_t *qweight, const __half *cherry_weight,
                              const int16_t *cherry_indices, const __half *scales, uint8_t *stream, int K, int N,
                              int C, int G, hipStream_t s) {
    const StreamGeo geo = stream_geo(bits, K, N, C);
    hipLaunchKernelGGL(stream_header_kernel, dim3(ceil_div((int)geo.hdr_bytes, 256)), dim3(256), 0, s, cherry_indices, stream,
                       geo);
    if (bits == 4)
        hipLaunchKernelGGL(stream_pack_kernel<4>, dim3(geo.ntiles), dim3(256), 0, s, qweight, cherry_weight, scales, stream, G, geo);
    else
        hipLaunchKernelGGL(stream_pack_kernel<3>, dim3(geo.ntiles), dim3(256), 0, s, qweight, cherry_weight, scales, stream, G, geo);
    return hipGetLastError();
}

hipError_t launch_stream_unpack(int bits, const uint8_t *stream, uint8_t *qweight, __half *cherry_weight,
                                int16_t *cherry_indices, __half *scales, int K, int N, int C, int G, hipStream_t s) {
    const StreamGeo geo = stream_geo(bits, K, N, C);
    if (C > 0)
        hipLaunchKernelGGL(stream_header_unpack_kernel, dim3(ceil_div(C, 256)), dim3(256), 0, s,
                           stream, cherry_indices, geo);
    if (bits == 4)
        hipLaunchKernelGGL(stream_unpack_kernel<4>, dim3(geo.ntiles), dim3(256), 0, s, stream, qweight, cherry_weight, scales, G, geo);
    else
        hipLaunchKernelGGL(stream_unpack_kernel<3>, dim3(geo.ntiles), dim3(256), 0, s, stream, qweight, cherry_weight, scales, G, geo);
    return hipGetLastError();
}

}  // namespace cq
