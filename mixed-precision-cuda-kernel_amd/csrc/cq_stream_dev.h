// Device-side pieces shared by the kernels that read the repacked weight stream (gfx950).
#pragma once

#include <type_traits>

#include "cq_device.h"
#include "cq_kernels.h"

namespace cq {

typedef _Float16 sh8_t __attribute__((ext_vector_type(8)));
typedef _Float16 sh4_t __attribute__((ext_vector_type(4)));
typedef float sf4_t __attribute__((ext_vector_type(4)));
typedef uint32_t su4 __attribute__((ext_vector_type(4)));
typedef uint32_t su3 __attribute__((ext_vector_type(3)));
typedef uint32_t su2 __attribute__((ext_vector_type(2)));
typedef _Float16 sh2_t __attribute__((ext_vector_type(2)));

constexpr uint32_t kSFlags = 0x00020000u;
constexpr uint32_t kSOob = 0x80000000u;
// 16-byte loads of raw activations per thread that cover the longest row a geometry takes
// (max_units units of 128 positions plus up to 128 cherry channels) with NT threads
__host__ __device__ constexpr int stream_x_loads(int max_units, int nt) {
    return (max_units * 128 + 128 + nt * 8 - 1) / (nt * 8);
}
constexpr int kStreamRawPad = 512 + 128 + 8;  // zero halves kept behind the raw activations in LDS

// ---- the matvec --------------------------------------------------------------------------------
__device__ inline sh8_t as_h8(su4 v) { return __builtin_bit_cast(sh8_t, v); }
__device__ inline sh4_t as_h4(su2 v) { return __builtin_bit_cast(sh4_t, v); }

// One unit (128 positions x 16 columns) against the activations of the same positions: the
// sum over the unit of x * code for the lane's column (row 0 of the MFMA tile, which every lane
// group receives because every row of A holds the same activations).
template <int BITS>
__device__ inline float unit_dot(const su4 w, const unsigned short *xa) {
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
        return dl[0] * 16777216.0f + dh[0] * 1048576.0f;
    } else {
        // Every step is a 16x16x32 MFMA.  (The last 8 positions were two 16x16x16 steps once, chained
        // onto the 16x16x32 results through their accumulators: kernels whose schedule packed
        // those chains tightly -- tile-walking ones with more than 8 units per wavefront and a short
        // ring -- then returned sums that were off by hundreds and changed from run to run, while a
        // scheduling barrier around each unit, or this form, made them right.  The shift that
        // brings positions 28..31 to bit 0 costs two instructions and no MFMA time.)
        const su3 y = {w[0] >> 9, w[1] >> 9, w[2] >> 9};
        const sh8_t a0 = *reinterpret_cast<const sh8_t *>(xa);        // positions 0..7: fields at bit 0
        const sh8_t a2 = *reinterpret_cast<const sh8_t *>(xa + 8);    // 8..15: bit 3
        const sh8_t a4 = *reinterpret_cast<const sh8_t *>(xa + 16);   // 16..23: bit 6
        const sh8_t a1 = *reinterpret_cast<const sh8_t *>(xa + 24);   // 24..27: bit 0, 28..31: bit 3 (moved to bit 0 below)
        const uint32_t z = (y[0] & 0x00400040u) | ((y[1] & 0x00400040u) << 1) | ((y[2] & 0x00400040u) << 2);
        const su4 b0 = {w[0] & 0x00070007u, w[1] & 0x00070007u, w[2] & 0x00070007u, y[0] & 0x00070007u};
        const su4 b2 = {w[0] & 0x00380038u, w[1] & 0x00380038u, w[2] & 0x00380038u, y[0] & 0x00380038u};
        const su4 b4 = {w[0] & 0x01c001c0u, w[1] & 0x01c001c0u, w[2] & 0x01c001c0u, z};
        const su4 b1 = {y[1] & 0x00070007u, y[2] & 0x00070007u, (y[1] >> 3) & 0x00070007u, (y[2] >> 3) & 0x00070007u};
        sf4_t d0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, as_h8(b0), zero4, 0, 0, 0);
        const sf4_t d3 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a2, as_h8(b2), zero4, 0, 0, 0);
        const sf4_t d6 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a4, as_h8(b4), zero4, 0, 0, 0);
        d0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, as_h8(b1), d0, 0, 0, 0);
        return d0[0] * 16777216.0f + d3[0] * 2097152.0f + d6[0] * 262144.0f;
    }
}

}  // namespace cq
