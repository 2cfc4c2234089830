// Roofline reference kernels for the measurement script (built into libcherryq_probe.so, a
// bench-only library; nothing in the product library links or calls them): what this GPU does with
// the same bytes when a kernel does nothing but read them, and what an empty launch costs.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef uint32_t u32x4p __attribute__((ext_vector_type(4)));

// Each workgroup of 256 threads reads LOADS * 4 KB: LOADS loads of 16 bytes per thread, a wavefront
// covering 1 KB of contiguous memory per load (the access shape of the weight streams), cache
// policy POLICY (0 = default, 2 = nt, read once).  The loads are all issued before the first is
// consumed.  The XOR of everything read is stored only if it equals a value the caller picks,
// which keeps the loads alive at no cost.
template <int LOADS, int POLICY>
__global__ __launch_bounds__(256) void stream_read_kernel(const uint8_t *__restrict__ p, unsigned bytes,
                                                          uint32_t *__restrict__ sink, uint32_t magic) {
    const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void *)p, 0, (int)bytes, 0x00020000u);
    const uint32_t base = blockIdx.x * (uint32_t)(LOADS * 4096) + threadIdx.x * 16u;
    u32x4p v[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; i++) v[i] = __builtin_amdgcn_raw_buffer_load_b128(r, base + i * 4096u, 0, POLICY);
    uint32_t x = 0;
#pragma unroll
    for (int i = 0; i < LOADS; i++) x ^= v[i][0] ^ v[i][1] ^ v[i][2] ^ v[i][3];
    if (x == magic) sink[0] = x;
}

__global__ void empty_kernel() {}

template <int LOADS, int POLICY>
int launch_read(const void *buf, size_t bytes, void *sink, hipStream_t stream) {
    const unsigned per = LOADS * 4096;
    const unsigned wgs = (unsigned)((bytes + per - 1) / per);
    if (wgs == 0) return 0;
    hipLaunchKernelGGL((stream_read_kernel<LOADS, POLICY>), dim3(wgs), dim3(256), 0, stream,
                       reinterpret_cast<const uint8_t *>(buf), (unsigned)bytes, reinterpret_cast<uint32_t *>(sink),
                       0x9e3779b9u);
    return (int)hipGetLastError();
}

}  // namespace

extern "C" {

// Reads `bytes` (< 2 GiB) of `buf` once.  kb_per_workgroup: 8, 16, 32 or 64; nt: read-once cache
// policy or the default one.  sink: 4 writable bytes (never written in practice).  Returns 0, a
// hipError_t, or -1 for an argument it does not take.
int cherryq_probe_stream_read(const void *buf, size_t bytes, void *sink, int kb_per_workgroup, int nt, void *stream) {
    if (!buf || !sink || bytes >= 0x7fff0000ull || (reinterpret_cast<uintptr_t>(buf) & 15)) return -1;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    switch (kb_per_workgroup * 2 + (nt ? 1 : 0)) {
        case 16: return launch_read<2, 0>(buf, bytes, sink, s);
        case 17: return launch_read<2, 2>(buf, bytes, sink, s);
        case 32: return launch_read<4, 0>(buf, bytes, sink, s);
        case 33: return launch_read<4, 2>(buf, bytes, sink, s);
        case 64: return launch_read<8, 0>(buf, bytes, sink, s);
        case 65: return launch_read<8, 2>(buf, bytes, sink, s);
        case 128: return launch_read<16, 0>(buf, bytes, sink, s);
        case 129: return launch_read<16, 2>(buf, bytes, sink, s);
        default: return -1;
    }
}

int cherryq_probe_empty_launch(void *stream) {
    hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(64), 0, reinterpret_cast<hipStream_t>(stream));
    return (int)hipGetLastError();
}

}  // extern "C"
