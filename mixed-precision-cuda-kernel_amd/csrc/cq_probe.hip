// Roofline reference kernels for the measurement script: what this GPU does with the same bytes
// when a kernel does nothing but read them, and what an empty launch costs.  They put the
// fused kernels' times in proportion; nothing in the product path calls them.
#include "cq_common.cuh"
#include "cq_kernels.h"

namespace cq {

typedef uint32_t u32x4p __attribute__((ext_vector_type(4)));

// Each workgroup reads 64 KB: 256 threads x 16 loads of 16 bytes, a wavefront covering 1 KB of
// contiguous memory per load (the access shape of the weight stream), read-once cache policy.
// The loads are all issued before the first is consumed.  The XOR of everything read is stored
// only if it equals a value the caller picks, which keeps the loads alive at no cost.
__global__ __launch_bounds__(256) void stream_read_kernel(const uint8_t *__restrict__ p, unsigned bytes,
                                                          uint32_t *__restrict__ sink, uint32_t magic) {
    const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void *)p, 0, (int)bytes, 0x00020000u);
    const uint32_t base = blockIdx.x * 65536u + threadIdx.x * 16u;
    u32x4p v[16];
#pragma unroll
    for (int i = 0; i < 16; i++) v[i] = __builtin_amdgcn_raw_buffer_load_b128(r, base + i * 4096u, 0, 2);
    uint32_t x = 0;
#pragma unroll
    for (int i = 0; i < 16; i++) x ^= v[i][0] ^ v[i][1] ^ v[i][2] ^ v[i][3];
    if (x == magic) sink[0] = x;
}

__global__ void empty_kernel() {}

hipError_t launch_probe_read(const void *buf, size_t bytes, void *sink, hipStream_t stream) {
    const unsigned wgs = (unsigned)((bytes + 65535) / 65536);
    if (wgs == 0) return hipSuccess;
    hipLaunchKernelGGL(stream_read_kernel, dim3(wgs), dim3(256), 0, stream, reinterpret_cast<const uint8_t *>(buf),
                       (unsigned)bytes, reinterpret_cast<uint32_t *>(sink), 0x9e3779b9u);
    return hipGetLastError();
}

hipError_t launch_probe_empty(hipStream_t stream) {
    hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(64), 0, stream);
    return hipGetLastError();
}

}  // namespace cq
