// extern "C" entry points of libcherryq: argument validation and kernel selection.
// Declarations and the reference interfaces they replace: include/cherryq.h.
#include "../../include/cherryq.h"

#include <stdlib.h>

#include <atomic>
#include <mutex>

#include "cq_device.h"
#include "cq_kernels.h"

namespace cq {

// Test hook: route every fused call through the generic kernel (a second, independently written
// HIP path that the tests cross-check the specialised kernels against).  Set by
// cherryq_set_force_generic(); the environment variable CHERRYQ_FORCE_GENERIC=1 is read once,
// at the first fused call, as the initial value.
static std::atomic<int> g_force_generic{-1};
static bool force_generic() {
    int v = g_force_generic.load(std::memory_order_relaxed);
    if (v < 0) {
        const char *e = getenv("CHERRYQ_FORCE_GENERIC");
        v = e && e[0] == '1' ? 1 : 0;
        int unset = -1;
        if (!g_force_generic.compare_exchange_strong(unset, v)) v = unset;  // a setter call came first
    }
    return v == 1;
}

// Size queries answer for any arguments; nonsensical ones are clamped, not rejected.
static void clamp_dims(int &B, int &K, int &N, int &C) {
    if (B < 1) B = 1;
    if (K < 8) K = 8;
    if (N < 8) N = 8;
    if (C < 0) C = 0;
    if (C > K) C = K;
}

// zero-kept: accumulator words (batch 1 and the generic kernel) and, for batches, the tickets
size_t workspace_bytes(int B, int K, int N, int C) {
    clamp_dims(B, K, N, C);
    size_t bytes = splitk_words_bytes(B, N) + splitk_side_bytes(B, N);
    if (B >= 2) {
        size_t b2 = batch_workspace(K, N, C).workspace_total;
        if (b2 > bytes) bytes = b2;
    }
    if (B >= kGemmMinRows) {
        size_t b3 = gemm_plan(B, K, N, C).workspace_bytes;
        if (b3 > bytes) bytes = b3;
    }
    return bytes;
}

// uninitialised: partial tiles and prepared activations of the matrix-core path
size_t scratch_bytes(int B, int K, int N, int C) {
    clamp_dims(B, K, N, C);
    size_t bytes = B >= 2 ? batch_workspace(K, N, C).scratch_total : 0;
    if (B >= 2 && f32_scratch_bytes(K, C) > bytes) bytes = f32_scratch_bytes(K, C);  // fp32-tensor variant
    if (B >= kGemmMinRows) {
        size_t b3 = gemm_plan(B, K, N, C).scratch_bytes;
        if (b3 > bytes) bytes = b3;
    }
    return bytes;
}

static inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

static int check_tensors(const void *vec, const void *qweight, const void *cherry_weight,
                         const void *cherry_indices, const void *scales, const void *mul, int B, int K, int N,
                         int C, int G) {
    if (B < 0 || K <= 0 || N <= 0 || C < 0 || C > K) return CHERRYQ_E_SHAPE;
    if (K % 8 || N % 8 || C % 8) return CHERRYQ_E_SHAPE;
    if (G <= 0 || G % 32) return CHERRYQ_E_GROUP;
    if (!vec || !mul) return CHERRYQ_E_NULL;
    if (K - C > 0 && (!qweight || !scales)) return CHERRYQ_E_NULL;
    if (C > 0 && (!cherry_weight || !cherry_indices)) return CHERRYQ_E_NULL;
    if (!aligned(qweight, 16) || !aligned(scales, 16) || !aligned(cherry_weight, 16) || !aligned(vec, 4) ||
        !aligned(mul, 16) || !aligned(cherry_indices, 4))
        return CHERRYQ_E_ALIGN;
    return CHERRYQ_OK;
}

static int check_common(const void *vec, const void *qweight, const void *cherry_weight,
                        const void *cherry_indices, const void *scales, const void *mul, int B, int K, int N,
                        int C, int G, void *workspace, size_t workspace_bytes_given, void *scratch,
                        size_t scratch_bytes_given) {
    const int rc = check_tensors(vec, qweight, cherry_weight, cherry_indices, scales, mul, B, K, N, C, G);
    if (rc) return rc;
    if (!workspace || !aligned(workspace, 256) || workspace_bytes_given < workspace_bytes(B, K, N, C))
        return CHERRYQ_E_WORKSPACE;
    const size_t need = scratch_bytes(B, K, N, C);
    if (need && (!scratch || !aligned(scratch, 256) || scratch_bytes_given < need)) return CHERRYQ_E_WORKSPACE;
    return CHERRYQ_OK;
}

template <int BITS>
static int matmul_f16(const void *vec, const uint8_t *qweight, const void *cherry_weight,
                      const int16_t *cherry_indices, const void *scales, void *mul, int B, int K, int N,
                      int C, int G, int accumulate, void *workspace, size_t wsb, void *scratch, size_t scb,
                      void *stream) {
    int rc = check_common(vec, qweight, cherry_weight, cherry_indices, scales, mul, B, K, N, C, G, workspace,
                          wsb, scratch, scb);
    if (rc) return rc;
    if (C > 0 && K > 32768) return CHERRYQ_E_SHAPE;  // int16 channel indices cannot name the columns
    if (B == 0) return CHERRYQ_OK;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const __half *x = reinterpret_cast<const __half *>(vec);
    const __half *cw = reinterpret_cast<const __half *>(cherry_weight);
    const __half *sc = reinterpret_cast<const __half *>(scales);
    __half *y = reinterpret_cast<__half *>(mul);
    hipError_t e;
    if (!force_generic() && B == 1 && matvec_supported(BITS, B, K, N, C, G)) {
        e = launch_matvec(BITS, x, qweight, cw, cherry_indices, sc, y, K, N, C, G, accumulate, workspace, s);
    } else if (!force_generic() && matvec_rows_preferred(BITS, B, K, N, C, G)) {
        e = launch_matvec_rows(BITS, x, qweight, cw, cherry_indices, sc, y, B, K, N, C, G, accumulate, workspace, s);
    } else if (!force_generic() && B >= kGemmMinRows && gemm_supported(BITS, B, K, N, C, G)) {
        e = launch_gemm(BITS, x, qweight, cw, cherry_indices, sc, y, B, K, N, C, G, accumulate, workspace, scratch, s);
    } else if (!force_generic() && batch_supported(BITS, B, K, N, C, G)) {
        e = launch_batch(BITS, x, qweight, cw, cherry_indices, sc, y, B, K, N, C, G, accumulate, workspace, scratch, s);
    } else {
        e = launch_generic<BITS, __half, int16_t>(x, qweight, cw, cherry_indices, sc, y, B, K, N, C, G,
                                                  accumulate, workspace, s);
    }
    return (int)e;
}

}  // namespace cq

extern "C" {

int cherryq_version(void) { return CHERRYQ_VERSION; }

void cherryq_set_force_generic(int on) { cq::g_force_generic.store(on ? 1 : 0); }

const char *cherryq_status_string(int status) {
    switch (status) {
        case CHERRYQ_OK: return "ok";
        case CHERRYQ_E_NULL: return "a required pointer is NULL";
        case CHERRYQ_E_SHAPE: return "dimensions inconsistent with the packed buffer schema";
        case CHERRYQ_E_GROUP: return "unsupported group_size for this entry point";
        case CHERRYQ_E_WORKSPACE: return "workspace missing, misaligned or too small";
        case CHERRYQ_E_BITS: return "w_bits must be 3 or 4";
        case CHERRYQ_E_ALIGN: return "a pointer is not aligned as the kernels require";
        case CHERRYQ_E_UNSUPPORTED: return "request not implemented by this build";
        case CHERRYQ_E_STATIC_LIMIT:
            return "request exceeds the fixed workspace of the entry point that does not allocate "
                   "(at most 4 rows and batch * out_features <= 131072)";
        default: break;
    }
    if (status > 0) return hipGetErrorString((hipError_t)status);
    return "unknown status";
}

size_t cherryq_workspace_bytes(int batch, int in_features, int out_features, int num_cherries) {
    return cq::workspace_bytes(batch, in_features, out_features, num_cherries);
}

size_t cherryq_scratch_bytes(int batch, int in_features, int out_features, int num_cherries) {
    return cq::scratch_bytes(batch, in_features, out_features, num_cherries);
}

size_t cherryq_scratch_bytes_f32(int batch, int in_features, int out_features, int num_cherries) {
    int B = batch, K = in_features, N = out_features, C = num_cherries;
    cq::clamp_dims(B, K, N, C);
    const size_t f32 = cq::f32_scratch_bytes(K, C);
    const size_t common = cq::scratch_bytes(B, K, N, C);
    return f32 > common ? f32 : common;
}

int cherryq_vecquant4matmul_f16(const void *vec, const uint8_t *qweight, const void *cherry_weight,
                                const int16_t *cherry_indices, const void *scales, void *mul, int batch,
                                int in_features, int out_features, int num_cherries, int group_size,
                                int accumulate, void *workspace, size_t workspace_bytes, void *scratch,
                                size_t scratch_bytes, void *stream) {
    if (group_size < 128) return CHERRYQ_E_GROUP;  // csrc/quant_cuda_kernel.cu:684
    return cq::matmul_f16<4>(vec, qweight, cherry_weight, cherry_indices, scales, mul, batch, in_features,
                             out_features, num_cherries, group_size, accumulate, workspace, workspace_bytes,
                             scratch, scratch_bytes, stream);
}

int cherryq_vecquant3matmul_f16(const void *vec, const uint8_t *qweight, const void *cherry_weight,
                                const int16_t *cherry_indices, const void *scales, void *mul, int batch,
                                int in_features, int out_features, int num_cherries, int group_size,
                                int accumulate, void *workspace, size_t workspace_bytes, void *scratch,
                                size_t scratch_bytes, void *stream) {
    return cq::matmul_f16<3>(vec, qweight, cherry_weight, cherry_indices, scales, mul, batch, in_features,
                             out_features, num_cherries, group_size, accumulate, workspace, workspace_bytes,
                             scratch, scratch_bytes, stream);
}

int cherryq_vecquant3matmul_f32(const float *vec, const uint8_t *qweight, const float *cherry_weight,
                                const int32_t *cherry_indices, const float *scales, float *mul, int batch,
                                int in_features, int out_features, int num_cherries, int group_size,
                                int accumulate, void *workspace, size_t workspace_bytes, void *scratch,
                                size_t scratch_bytes, void *stream) {
    int rc = cq::check_common(vec, qweight, cherry_weight, cherry_indices, scales, mul, batch, in_features,
                              out_features, num_cherries, group_size, workspace, workspace_bytes, scratch,
                              scratch_bytes);
    if (rc) return rc;
    if (batch == 0) return CHERRYQ_OK;
    // one row: the matrix-core kernel when the caller brought its scratch buffer, else the generic one
    const bool has_scratch = scratch && cq::aligned(scratch, 256) &&
                             scratch_bytes >= cq::f32_scratch_bytes(in_features, num_cherries);
    if (!cq::force_generic() && (batch >= 2 || has_scratch) &&
        cq::f32_supported(batch, in_features, out_features, num_cherries, group_size))
        return (int)cq::launch_f32(vec, qweight, cherry_weight, cherry_indices, scales, mul, batch, in_features,
                                   out_features, num_cherries, group_size, accumulate, workspace, scratch,
                                   reinterpret_cast<hipStream_t>(stream));
    return (int)cq::launch_generic<3, float, int32_t>(vec, qweight, cherry_weight, cherry_indices, scales, mul,
                                                      batch, in_features, out_features, num_cherries,
                                                      group_size, accumulate, workspace,
                                                      reinterpret_cast<hipStream_t>(stream));
}

static int dequantize_normal(int bits, const uint8_t *qweight, const float *scales, float *out, int height,
                             int N, int C, int G, void *stream) {
    if (height <= 0 || N <= 0 || C < 0 || C > height || height % 8 || N % 8 || C % 8) return CHERRYQ_E_SHAPE;
    if (G <= 0 || G % 8) return CHERRYQ_E_GROUP;
    if (height - C == 0) return CHERRYQ_OK;
    if (!qweight || !scales || !out) return CHERRYQ_E_NULL;
    if (!cq::aligned(qweight, 4) || !cq::aligned(scales, 16) || !cq::aligned(out, 16)) return CHERRYQ_E_ALIGN;
    return (int)cq::launch_dequant_normal(bits, qweight, scales, out, height - C, N, G,
                                          reinterpret_cast<hipStream_t>(stream));
}

int cherryq_dequantize3_normal_f32(const uint8_t *qweight, const float *scales, float *out, int height,
                                   int out_features, int cherry_size, int group_size, void *stream) {
    return dequantize_normal(3, qweight, scales, out, height, out_features, cherry_size, group_size, stream);
}

int cherryq_dequantize4_normal_f32(const uint8_t *qweight, const float *scales, float *out, int height,
                                   int out_features, int cherry_size, int group_size, void *stream) {
    return dequantize_normal(4, qweight, scales, out, height, out_features, cherry_size, group_size, stream);
}

int cherryq_unpack_f16(int w_bits, const uint8_t *qweight, const void *cherry_weight,
                       const int16_t *cherry_indices, const void *scales, void *dense, int in_features,
                       int out_features, int num_cherries, int group_size, void *stream) {
    if (w_bits != 3 && w_bits != 4) return CHERRYQ_E_BITS;
    int K = in_features, N = out_features, C = num_cherries;
    if (K <= 0 || N <= 0 || C < 0 || C > K || K % 8 || N % 8 || C % 8) return CHERRYQ_E_SHAPE;
    if (C > 0 && K > 32768) return CHERRYQ_E_SHAPE;  // int16 channel indices cannot name the columns
    if (group_size <= 0 || group_size % 8) return CHERRYQ_E_GROUP;
    if (!dense) return CHERRYQ_E_NULL;
    if (K - C > 0 && (!qweight || !scales)) return CHERRYQ_E_NULL;
    if (C > 0 && (!cherry_weight || !cherry_indices)) return CHERRYQ_E_NULL;
    if (!cq::aligned(qweight, 4) || !cq::aligned(scales, 8) || !cq::aligned(dense, 16)) return CHERRYQ_E_ALIGN;
    return (int)cq::launch_unpack(w_bits, qweight, reinterpret_cast<const __half *>(cherry_weight),
                                  cherry_indices, reinterpret_cast<const __half *>(scales),
                                  reinterpret_cast<__half *>(dense), K, N, C, group_size,
                                  reinterpret_cast<hipStream_t>(stream));
}

// ---- device-side pack, fake quantisation ----------------------------------------------------

int cherryq_pack_f16(int w_bits, const void *weight, const int16_t *cherry_indices, uint8_t *qweight, void *scales,
                     void *cherry_weight, int in_features, int out_features, int num_cherries, int group_size,
                     void *stream) {
    if (w_bits != 3 && w_bits != 4) return CHERRYQ_E_BITS;
    const int K = in_features, N = out_features, C = num_cherries;
    if (K <= 0 || N <= 0 || C < 0 || C > K || K % 8 || C % 8) return CHERRYQ_E_SHAPE;
    if (C > 0 && K > 32768) return CHERRYQ_E_SHAPE;  // int16 channel indices cannot name the columns
    if (group_size <= 0) return CHERRYQ_E_GROUP;
    if (!weight) return CHERRYQ_E_NULL;
    if (K - C > 0 && (!qweight || !scales)) return CHERRYQ_E_NULL;
    if (C > 0 && (!cherry_indices || !cherry_weight)) return CHERRYQ_E_NULL;
    return (int)cq::launch_pack(w_bits, reinterpret_cast<const __half *>(weight), cherry_indices, qweight,
                                reinterpret_cast<__half *>(scales), reinterpret_cast<__half *>(cherry_weight), K, N,
                                C, group_size, reinterpret_cast<hipStream_t>(stream));
}

static int fake_quant_entry(bool fp32, int w_bits, const void *weight, const int32_t *cherry_indices, void *out,
                            int in_features, int out_features, int num_cherries, int group_size, int ste,
                            void *stream) {
    if (w_bits < 2 || w_bits > 4) return CHERRYQ_E_BITS;
    const int K = in_features, N = out_features, C = num_cherries;
    if (K <= 0 || N <= 0 || C < 0) return CHERRYQ_E_SHAPE;
    if (group_size <= 0) return CHERRYQ_E_GROUP;
    if (!weight || !out || (C > 0 && !cherry_indices)) return CHERRYQ_E_NULL;
    if (!cq::aligned(weight, fp32 ? 4 : 2) || !cq::aligned(out, fp32 ? 4 : 2)) return CHERRYQ_E_ALIGN;
    if (!cq::fake_quant_supported(K, C, group_size)) return CHERRYQ_E_UNSUPPORTED;
    return (int)cq::launch_fake_quant(w_bits, fp32, weight, cherry_indices, out, K, N, C, group_size, ste,
                                      reinterpret_cast<hipStream_t>(stream));
}

int cherryq_fake_quant_f16(int w_bits, const void *weight, const int32_t *cherry_indices, void *out, int in_features,
                           int out_features, int num_cherries, int group_size, int ste, void *stream) {
    return fake_quant_entry(false, w_bits, weight, cherry_indices, out, in_features, out_features, num_cherries,
                            group_size, ste, stream);
}

int cherryq_fake_quant_f32(int w_bits, const void *weight, const int32_t *cherry_indices, void *out, int in_features,
                           int out_features, int num_cherries, int group_size, int ste, void *stream) {
    return fake_quant_entry(true, w_bits, weight, cherry_indices, out, in_features, out_features, num_cherries,
                            group_size, ste, stream);
}

// ---- the entry point that allocates nothing (see include/cherryq.h) -----------------------------

}  // extern "C"

namespace cq {

// The split-K accumulator words of cherryq_vecquant_matmul_f16_static: 4 rows x 32768 columns of
// 8 bytes.  Zero at load time; the kernels return every word they used to zero.
constexpr size_t kStaticWorkspaceBytes = CHERRYQ_STATIC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned long long scratch[kStaticWorkspaceBytes / sizeof(unsigned long long)];

constexpr int kStaticMaxDevices = 64;
static std::mutex g_static_mutex;
static void *g_static_ptr[kStaticMaxDevices];    // each GPU's own copy of `scratch`, from hipGetSymbolAddress
static bool g_static_dirty[kStaticMaxDevices];   // a launch failed after the array may have been touched

__global__ __launch_bounds__(256) void static_clear_kernel(unsigned long long *p, unsigned words) {
    for (unsigned i = blockIdx.x * 256 + threadIdx.x; i < words; i += gridDim.x * 256) p[i] = 0ull;
}

template <int BITS>
static int matmul_f16_static(const void *vec, const uint8_t *qweight, const void *cherry_weight,
                             const int16_t *cherry_indices, const void *scales, void *mul, int B, int K, int N, int C,
                             int G, int accumulate, void *stream) {
    if (B < 0 || K <= 0 || N <= 0) return CHERRYQ_E_SHAPE;
    if (B > kMatvecMaxRows) return CHERRYQ_E_STATIC_LIMIT;
    const size_t need = ((size_t)(B < 1 ? 1 : B) * (size_t)N * sizeof(unsigned long long) + 255) / 256 * 256;
    if (need > kStaticWorkspaceBytes) return CHERRYQ_E_STATIC_LIMIT;
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kStaticMaxDevices) return CHERRYQ_E_UNSUPPORTED;
    void *ws = nullptr;
    bool dirty = false;
    {
        std::lock_guard<std::mutex> lock(g_static_mutex);
        if (!g_static_ptr[dev]) {  // once per device, with that device current
            void *ptr = nullptr;
            e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
            if (e != hipSuccess) return (int)e;
            if (!ptr) return CHERRYQ_E_NULL;
            g_static_ptr[dev] = ptr;
        }
        ws = g_static_ptr[dev];
        dirty = g_static_dirty[dev];
        g_static_dirty[dev] = true;  // until this call's launches are known to have been accepted
    }
    // the checks of the entry point this one is a variant of; on rejection nothing was launched
    int rc = check_tensors(vec, qweight, cherry_weight, cherry_indices, scales, mul, B, K, N, C, G);
    if (rc == CHERRYQ_OK && C > 0 && K > 32768) rc = CHERRYQ_E_SHAPE;
    if (rc != CHERRYQ_OK || B == 0) {
        std::lock_guard<std::mutex> lock(g_static_mutex);
        g_static_dirty[dev] = dirty;
        return rc;
    }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (dirty) {
        hipLaunchKernelGGL(static_clear_kernel, dim3(256), dim3(256), 0, s, reinterpret_cast<unsigned long long *>(ws),
                           (unsigned)(kStaticWorkspaceBytes / sizeof(unsigned long long)));
        e = hipGetLastError();
        if (e != hipSuccess) return (int)e;
    }
    const __half *x = reinterpret_cast<const __half *>(vec);
    const __half *cw = reinterpret_cast<const __half *>(cherry_weight);
    const __half *sc = reinterpret_cast<const __half *>(scales);
    __half *y = reinterpret_cast<__half *>(mul);
    if (!force_generic() && B == 1 && matvec_supported(BITS, B, K, N, C, G))
        e = launch_matvec(BITS, x, qweight, cw, cherry_indices, sc, y, K, N, C, G, accumulate, ws, s);
    else if (!force_generic() && matvec_rows_preferred(BITS, B, K, N, C, G))
        e = launch_matvec_rows(BITS, x, qweight, cw, cherry_indices, sc, y, B, K, N, C, G, accumulate, ws, s);
    else  // the general kernel: same accumulator words, no other buffer
        e = launch_generic<BITS, __half, int16_t>(x, qweight, cw, cherry_indices, sc, y, B, K, N, C, G, accumulate, ws, s);
    if (e == hipSuccess) {
        std::lock_guard<std::mutex> lock(g_static_mutex);
        g_static_dirty[dev] = false;
    }
    return (int)e;
}

}  // namespace cq

extern "C" {

int cherryq_vecquant_matmul_f16_static(int w_bits, const void *vec, const uint8_t *qweight, const void *cherry_weight,
                                       const int16_t *cherry_indices, const void *scales, void *mul, int batch,
                                       int in_features, int out_features, int num_cherries, int group_size,
                                       int accumulate, void *stream) {
    if (w_bits == 4) {
        if (group_size < 128) return CHERRYQ_E_GROUP;
        return cq::matmul_f16_static<4>(vec, qweight, cherry_weight, cherry_indices, scales, mul, batch, in_features,
                                        out_features, num_cherries, group_size, accumulate, stream);
    }
    if (w_bits == 3)
        return cq::matmul_f16_static<3>(vec, qweight, cherry_weight, cherry_indices, scales, mul, batch, in_features,
                                        out_features, num_cherries, group_size, accumulate, stream);
    return CHERRYQ_E_BITS;
}

// ---- load-time repacked weight stream (see include/cherryq.h) -----------------------------------

size_t cherryq_prepack_bytes(int w_bits, int in_features, int out_features, int num_cherries) {
    if ((w_bits != 3 && w_bits != 4) || in_features <= 0 || out_features <= 0 || num_cherries < 0 ||
        num_cherries >= in_features)
        return 0;
    return cq::stream_bytes(w_bits, in_features, out_features, num_cherries);
}

int cherryq_prepack_supported(int w_bits, int batch, int in_features, int out_features, int num_cherries,
                              int group_size) {
    if (batch >= 2)
        return cq::stream_rows_supported(w_bits, batch, in_features, out_features, num_cherries, group_size) ? 1 : 0;
    return cq::stream_supported(w_bits, batch, in_features, out_features, num_cherries, group_size) ? 1 : 0;
}

size_t cherryq_prepacked_scratch_bytes(int w_bits, int batch, int in_features, int out_features, int num_cherries) {
    if ((w_bits != 3 && w_bits != 4) || batch < 2 || in_features <= 0 || out_features <= 0 || num_cherries < 0 ||
        num_cherries >= in_features)
        return 0;
    return cq::stream_rows_scratch_bytes(w_bits, batch, in_features, out_features, num_cherries);
}

int cherryq_prepack_recommended(int w_bits, int in_features, int out_features, int num_cherries, int group_size) {
    if (!cq::stream_supported(w_bits, 1, in_features, out_features, num_cherries, group_size)) return 0;
    return cq::stream_faster(w_bits, in_features, out_features, num_cherries) ? 1 : 0;
}

int cherryq_prepack_rows_recommended(int w_bits, int batch, int in_features, int out_features, int num_cherries,
                                     int group_size) {
    if (batch == 1) return cherryq_prepack_recommended(w_bits, in_features, out_features, num_cherries, group_size);
    if (batch < 1 || !cherryq_prepack_supported(w_bits, batch, in_features, out_features, num_cherries, group_size)) return 0;
    if (cq::stream_cu_rows_supported(w_bits, batch, in_features, out_features, num_cherries)) return 1;
    const int units = (in_features - num_cherries + cq::kStreamUnitK - 1) / cq::kStreamUnitK;
    return batch >= (units <= 32 ? 4 : 8) ? 1 : 0;
}

const char *cherryq_matvec_prepacked_kernel_name(int w_bits, int in_features, int out_features, int num_cherries) {
    if (!cq::stream_supported(w_bits, 1, in_features, out_features, num_cherries, cq::kStreamUnitK)) return "";
    return cq::stream_uses_cu(w_bits, in_features, out_features, num_cherries) ? "cq::stream_cu_kernel" : "cq::stream_kernel";
}

const char *cherryq_matmul_prepacked_kernel_name(int w_bits, int batch, int in_features, int out_features, int num_cherries) {
    if (batch == 1) return cherryq_matvec_prepacked_kernel_name(w_bits, in_features, out_features, num_cherries);
    if (!cq::stream_rows_supported(w_bits, batch, in_features, out_features, num_cherries, cq::kStreamUnitK)) return "";
    return cq::stream_rows_kernel_name(w_bits, batch, in_features, out_features, num_cherries);
}

static int prepack_check(int w_bits, int K, int N, int C, int G, size_t stream_bytes_given) {
    if (w_bits != 3 && w_bits != 4) return CHERRYQ_E_BITS;
    if (K <= 0 || N <= 0 || C < 0 || C >= K || K % 8 || N % 8 || C % 8) return CHERRYQ_E_SHAPE;
    if (C > 0 && K > 32768) return CHERRYQ_E_SHAPE;  // int16 channel indices cannot name the columns
    if (G <= 0 || G % cq::kStreamUnitK) return CHERRYQ_E_GROUP;
    if (!cq::stream_supported(w_bits, 1, K, N, C, G)) return CHERRYQ_E_UNSUPPORTED;
    if (stream_bytes_given < cq::stream_bytes(w_bits, K, N, C)) return CHERRYQ_E_WORKSPACE;
    return CHERRYQ_OK;
}

int cherryq_prepack_f16(int w_bits, const uint8_t *qweight, const void *cherry_weight, const int16_t *cherry_indices,
                        const void *scales, void *stream, size_t stream_bytes, int in_features, int out_features,
                        int num_cherries, int group_size, void *hip_stream) {
    int rc = prepack_check(w_bits, in_features, out_features, num_cherries, group_size, stream_bytes);
    if (rc) return rc;
    if (!qweight || !scales || !stream || (num_cherries > 0 && (!cherry_weight || !cherry_indices))) return CHERRYQ_E_NULL;
    if (!cq::aligned(stream, 256)) return CHERRYQ_E_ALIGN;
    return (int)cq::launch_stream_pack(w_bits, qweight, reinterpret_cast<const __half *>(cherry_weight), cherry_indices,
                                       reinterpret_cast<const __half *>(scales), reinterpret_cast<uint8_t *>(stream),
                                       in_features, out_features, num_cherries, group_size,
                                       reinterpret_cast<hipStream_t>(hip_stream));
}

int cherryq_unprepack_f16(int w_bits, const void *stream, size_t stream_bytes, uint8_t *qweight, void *cherry_weight,
                          int16_t *cherry_indices, void *scales, int in_features, int out_features, int num_cherries,
                          int group_size, void *hip_stream) {
    int rc = prepack_check(w_bits, in_features, out_features, num_cherries, group_size, stream_bytes);
    if (rc) return rc;
    if (!qweight || !scales || !stream || (num_cherries > 0 && (!cherry_weight || !cherry_indices))) return CHERRYQ_E_NULL;
    if (!cq::aligned(stream, 256)) return CHERRYQ_E_ALIGN;
    return (int)cq::launch_stream_unpack(w_bits, reinterpret_cast<const uint8_t *>(stream), qweight,
                                         reinterpret_cast<__half *>(cherry_weight), cherry_indices,
                                         reinterpret_cast<__half *>(scales), in_features, out_features, num_cherries,
                                         group_size, reinterpret_cast<hipStream_t>(hip_stream));
}

int cherryq_matvec_prepacked_f16(int w_bits, const void *vec, const void *stream, size_t stream_bytes, void *mul,
                                 int batch, int in_features, int out_features, int num_cherries, int accumulate,
                                 void *hip_stream) {
    int rc = prepack_check(w_bits, in_features, out_features, num_cherries, cq::kStreamUnitK, stream_bytes);
    if (rc) return rc;
    if (batch < 0) return CHERRYQ_E_SHAPE;
    if (batch == 0) return CHERRYQ_OK;
    if (batch != 1) return CHERRYQ_E_UNSUPPORTED;
    if (!vec || !stream || !mul) return CHERRYQ_E_NULL;
    if (!cq::aligned(stream, 256) || !cq::aligned(vec, 16) || !cq::aligned(mul, 2)) return CHERRYQ_E_ALIGN;
    return (int)cq::launch_stream(w_bits, reinterpret_cast<const __half *>(vec), reinterpret_cast<const uint8_t *>(stream),
                                  reinterpret_cast<__half *>(mul), in_features, out_features, num_cherries, accumulate,
                                  reinterpret_cast<hipStream_t>(hip_stream));
}

int cherryq_matmul_prepacked_f16(int w_bits, const void *vec, const void *stream, size_t stream_bytes, void *mul,
                                 int batch, int in_features, int out_features, int num_cherries, int accumulate,
                                 void *scratch, size_t scratch_bytes, void *hip_stream) {
    if (batch == 1)
        return cherryq_matvec_prepacked_f16(w_bits, vec, stream, stream_bytes, mul, batch, in_features, out_features,
                                            num_cherries, accumulate, hip_stream);
    int rc = prepack_check(w_bits, in_features, out_features, num_cherries, cq::kStreamUnitK, stream_bytes);
    if (rc) return rc;
    if (batch < 0) return CHERRYQ_E_SHAPE;
    if (batch == 0) return CHERRYQ_OK;
    if (!cq::stream_rows_supported(w_bits, batch, in_features, out_features, num_cherries, cq::kStreamUnitK))
        return CHERRYQ_E_UNSUPPORTED;
    if (!vec || !stream || !mul) return CHERRYQ_E_NULL;
    if (!cq::aligned(stream, 256) || !cq::aligned(vec, 16) || !cq::aligned(mul, 2)) return CHERRYQ_E_ALIGN;
    const size_t need = cq::stream_rows_scratch_bytes(w_bits, batch, in_features, out_features, num_cherries);
    if (need && (!scratch || !cq::aligned(scratch, 256) || scratch_bytes < need)) return CHERRYQ_E_WORKSPACE;
    return (int)cq::launch_stream_rows(w_bits, reinterpret_cast<const __half *>(vec), reinterpret_cast<const uint8_t *>(stream),
                                       reinterpret_cast<__half *>(mul), batch, in_features, out_features, num_cherries,
                                       accumulate, scratch, reinterpret_cast<hipStream_t>(hip_stream));
}

int cherryq_decode_matvec_group_prepacked_f16(int w_bits, const void *vec, const void *norm_weight, float eps,
                                              const cherryq_stream_layer *layers, int n_layers, int in_features,
                                              int num_cherries, int accumulate, void *hip_stream) {
    if (w_bits != 3 && w_bits != 4) return CHERRYQ_E_BITS;
    if (!layers || !vec) return CHERRYQ_E_NULL;
    if (n_layers < 1 || n_layers > cq::kStreamMaxGroup) return CHERRYQ_E_SHAPE;
    if (!cq::aligned(vec, 16) || (norm_weight && !cq::aligned(norm_weight, 16))) return CHERRYQ_E_ALIGN;
    cq::StreamMember members[cq::kStreamMaxGroup];
    int outs[cq::kStreamMaxGroup];
    for (int i = 0; i < n_layers; i++) {
        const cherryq_stream_layer &l = layers[i];
        const int rc = prepack_check(w_bits, in_features, l.out_features, num_cherries, cq::kStreamUnitK, l.stream_bytes);
        if (rc) return rc;
        if (!l.stream || !l.mul) return CHERRYQ_E_NULL;
        if (!cq::aligned(l.stream, 256) || !cq::aligned(l.mul, 2)) return CHERRYQ_E_ALIGN;
        members[i] = {reinterpret_cast<const uint8_t *>(l.stream), reinterpret_cast<__half *>(l.mul), l.out_features};
        outs[i] = l.out_features;
    }
    if (!cq::stream_group_supported(w_bits, in_features, num_cherries, cq::kStreamUnitK, outs, n_layers))
        return CHERRYQ_E_UNSUPPORTED;
    return (int)cq::launch_stream_group(w_bits, reinterpret_cast<const __half *>(vec),
                                        reinterpret_cast<const __half *>(norm_weight), eps, members, n_layers,
                                        in_features, num_cherries, accumulate, reinterpret_cast<hipStream_t>(hip_stream));
}

int cherryq_decode_gate_up_prepacked_f16(int w_bits, const void *vec, const void *norm_weight, float eps,
                                         const void *gate_stream, size_t gate_stream_bytes, const void *up_stream,
                                         size_t up_stream_bytes, void *act, int in_features, int out_features,
                                         int num_cherries, void *hip_stream) {
    int rc = prepack_check(w_bits, in_features, out_features, num_cherries, cq::kStreamUnitK, gate_stream_bytes);
    if (rc) return rc;
    rc = prepack_check(w_bits, in_features, out_features, num_cherries, cq::kStreamUnitK, up_stream_bytes);
    if (rc) return rc;
    if (!vec || !gate_stream || !up_stream || !act) return CHERRYQ_E_NULL;
    if (!cq::aligned(gate_stream, 256) || !cq::aligned(up_stream, 256) || !cq::aligned(vec, 16) ||
        (norm_weight && !cq::aligned(norm_weight, 16)) || !cq::aligned(act, 2))
        return CHERRYQ_E_ALIGN;
    if (!cq::stream_pair_supported(w_bits, in_features, out_features, num_cherries)) return CHERRYQ_E_UNSUPPORTED;
    return (int)cq::launch_stream_pair(w_bits, reinterpret_cast<const __half *>(vec), reinterpret_cast<const __half *>(norm_weight),
                                       eps, reinterpret_cast<const uint8_t *>(gate_stream),
                                       reinterpret_cast<const uint8_t *>(up_stream), reinterpret_cast<__half *>(act),
                                       in_features, out_features, num_cherries, reinterpret_cast<hipStream_t>(hip_stream));
}

int cherryq_decode_gate_up_prepacked_supported(int w_bits, int in_features, int out_features, int num_cherries) {
    if (!cq::stream_supported(w_bits, 1, in_features, out_features, num_cherries, cq::kStreamUnitK)) return 0;
    return cq::stream_pair_supported(w_bits, in_features, out_features, num_cherries) ? 1 : 0;
}

int cherryq_decode_matvec_gated_prepacked_f16(int w_bits, const void *vec, const void *vec_gate, const void *stream,
                                              size_t stream_bytes, void *mul, int in_features, int out_features,
                                              int num_cherries, int accumulate, void *hip_stream) {
    int rc = prepack_check(w_bits, in_features, out_features, num_cherries, cq::kStreamUnitK, stream_bytes);
    if (rc) return rc;
    if (!vec || !vec_gate || !stream || !mul) return CHERRYQ_E_NULL;
    if (!cq::aligned(stream, 256) || !cq::aligned(vec, 16) || !cq::aligned(vec_gate, 16) || !cq::aligned(mul, 2))
        return CHERRYQ_E_ALIGN;
    if (!cq::stream_gated_supported(w_bits, in_features, out_features, num_cherries)) return CHERRYQ_E_UNSUPPORTED;
    return (int)cq::launch_stream_gated(w_bits, reinterpret_cast<const __half *>(vec), reinterpret_cast<const __half *>(vec_gate),
                                        reinterpret_cast<const uint8_t *>(stream), reinterpret_cast<__half *>(mul), in_features,
                                        out_features, num_cherries, accumulate, reinterpret_cast<hipStream_t>(hip_stream));
}

int cherryq_decode_matvec_attention_prepacked_supported(int w_bits, int in_features, int out_features, int num_cherries) {
    if ((w_bits != 3 && w_bits != 4) || in_features <= 0 || out_features <= 0 || num_cherries < 0) return 0;
    if (in_features % 8 || out_features % 8 || num_cherries % 8 || num_cherries >= in_features) return 0;
    return cq::stream_attn_out_supported(w_bits, in_features, num_cherries, out_features) ? 1 : 0;
}

int cherryq_decode_matvec_attention_prepacked_f16(int w_bits, const void *partial, const float *max_sum, int slices,
                                                  const void *stream, size_t stream_bytes, void *mul, int in_features,
                                                  int out_features, int num_cherries, int accumulate, void *hip_stream) {
    int rc = prepack_check(w_bits, in_features, out_features, num_cherries, cq::kStreamUnitK, stream_bytes);
    if (rc) return rc;
    if (!partial || !max_sum || !stream || !mul) return CHERRYQ_E_NULL;
    if (slices != cq::attn_out_slices() || in_features % 128) return CHERRYQ_E_SHAPE;
    if (!cq::aligned(stream, 256) || !cq::aligned(partial, 16) || !cq::aligned(max_sum, 8) || !cq::aligned(mul, 2))
        return CHERRYQ_E_ALIGN;
    if (!cq::stream_attn_out_supported(w_bits, in_features, num_cherries, out_features)) return CHERRYQ_E_UNSUPPORTED;
    return (int)cq::launch_stream_attn_out(w_bits, reinterpret_cast<const __half *>(partial), max_sum,
                                           reinterpret_cast<const uint8_t *>(stream), reinterpret_cast<__half *>(mul),
                                           in_features, out_features, num_cherries, accumulate,
                                           reinterpret_cast<hipStream_t>(hip_stream));
}

// ---- decode-step entry points (see include/cherryq.h) ------------------------------------------

size_t cherryq_group_workspace_bytes(int n_layers, const int *out_features) {
    size_t bytes = 0;
    for (int i = 0; i < n_layers; i++) {
        const int n = out_features && out_features[i] > 0 ? out_features[i] : 8;
        bytes += (size_t)((n + 255) / 256) * 256 * sizeof(unsigned long long);
    }
    return bytes;
}

int cherryq_decode_matvec_group_f16(int w_bits, const void *vec, const void *vec_gate, const void *norm_weight,
                                    float eps, const cherryq_layer *layers, int n_layers, int in_features,
                                    int num_cherries, int group_size, int accumulate, void *workspace,
                                    size_t workspace_bytes, void *stream) {
    using namespace cq;
    if (w_bits != 3 && w_bits != 4) return CHERRYQ_E_BITS;
    if (!layers) return CHERRYQ_E_NULL;
    if (n_layers < 1 || n_layers > kMaxGroup) return CHERRYQ_E_SHAPE;
    const int K = in_features, C = num_cherries, G = group_size;
    if (C > 0 && K > 32768) return CHERRYQ_E_SHAPE;  // int16 channel indices cannot name the columns
    int outs[kMaxGroup];
    for (int i = 0; i < n_layers; i++) outs[i] = layers[i].out_features;
    if (workspace_bytes < cherryq_group_workspace_bytes(n_layers, outs)) return CHERRYQ_E_WORKSPACE;
    if (vec_gate && !aligned(vec_gate, 4)) return CHERRYQ_E_ALIGN;
    if (norm_weight && (!aligned(norm_weight, 4) || !aligned(vec, 16))) return CHERRYQ_E_ALIGN;
    bool fast = !force_generic();
    MatvecMember members[kMaxGroup];
    for (int i = 0; i < n_layers; i++) {
        const cherryq_layer &l = layers[i];
        int rc = check_common(vec, l.qweight, l.cherry_weight, l.cherry_indices, l.scales, l.mul, 1, K,
                              l.out_features, C, G, workspace, workspace_bytes, nullptr, 0);
        if (rc) return rc;
        fast = fast && matvec_supported(w_bits, 1, K, l.out_features, C, G);
        members[i] = {l.qweight, reinterpret_cast<const __half *>(l.cherry_weight), l.cherry_indices,
                      reinterpret_cast<const __half *>(l.scales), reinterpret_cast<__half *>(l.mul), l.out_features, 0};
    }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    int n_total = 0;
    for (int i = 0; i < n_layers; i++) n_total += outs[i];
    // one launch streams all members: its geometry follows their total size
    fast = fast && matvec_geometry(w_bits, K, n_total, C, 1).splits <= kMaxSplits;
    if (norm_weight && (!fast || !matvec_norm_supported(w_bits, K, n_total, C))) return CHERRYQ_E_UNSUPPORTED;
    if (fast) {
        const MatvecPrologue pro = {reinterpret_cast<const __half *>(vec_gate),
                                    reinterpret_cast<const __half *>(norm_weight), eps};
        return (int)launch_matvec_group(w_bits, reinterpret_cast<const __half *>(vec), pro, members, n_layers, K, C,
                                        G, accumulate, workspace, s);
    }
    // shapes the streaming kernel does not take: one launch per layer, no fused activation
    if (vec_gate) return CHERRYQ_E_UNSUPPORTED;
    for (int i = 0; i < n_layers; i++) {
        const cherryq_layer &l = layers[i];
        int rc = w_bits == 4 ? matmul_f16<4>(vec, l.qweight, l.cherry_weight, l.cherry_indices, l.scales, l.mul, 1, K,
                                             l.out_features, C, G, accumulate, workspace, workspace_bytes, nullptr,
                                             0, stream)
                             : matmul_f16<3>(vec, l.qweight, l.cherry_weight, l.cherry_indices, l.scales, l.mul, 1, K,
                                             l.out_features, C, G, accumulate, workspace, workspace_bytes, nullptr,
                                             0, stream);
        if (rc) return rc;
    }
    return CHERRYQ_OK;
}

int cherryq_decode_add_rmsnorm_f16(void *hidden, const void *delta, const void *weight, void *normed,
                                   int hidden_size, float eps, void *stream) {
    if (!hidden || !weight || !normed) return CHERRYQ_E_NULL;
    if (hidden_size <= 0 || hidden_size % 4) return CHERRYQ_E_SHAPE;
    if (!cq::aligned(hidden, 8) || !cq::aligned(weight, 8) || !cq::aligned(normed, 8) || (delta && !cq::aligned(delta, 8)))
        return CHERRYQ_E_ALIGN;
    return (int)cq::launch_add_rmsnorm(reinterpret_cast<__half *>(hidden), reinterpret_cast<const __half *>(delta),
                                       reinterpret_cast<const __half *>(weight), reinterpret_cast<__half *>(normed),
                                       hidden_size, eps, reinterpret_cast<hipStream_t>(stream));
}

int cherryq_decode_rope_cache_f16(void *q, const void *k, const void *v, void *k_cache, void *v_cache,
                                  const int *position, int n_heads, int n_kv_heads, int head_dim, int max_len,
                                  float theta, void *stream) {
    if (!q || !k || !v || !k_cache || !v_cache || !position) return CHERRYQ_E_NULL;
    if (n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads || head_dim <= 0 || head_dim % 2 ||
        head_dim > 2048 || max_len <= 0)
        return CHERRYQ_E_SHAPE;
    return (int)cq::launch_rope_cache(reinterpret_cast<__half *>(q), reinterpret_cast<const __half *>(k),
                                      reinterpret_cast<const __half *>(v), reinterpret_cast<__half *>(k_cache),
                                      reinterpret_cast<__half *>(v_cache), position, n_heads, n_kv_heads, head_dim,
                                      max_len, theta, reinterpret_cast<hipStream_t>(stream));
}

int cherryq_decode_attention_f16(const void *q, const void *k_cache, const void *v_cache, void *out,
                                 const int *position, int n_heads, int n_kv_heads, int head_dim, int max_len,
                                 void *stream) {
    if (!q || !k_cache || !v_cache || !out || !position) return CHERRYQ_E_NULL;
    if (n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads || max_len <= 0 || max_len > cq::attn_max_len())
        return CHERRYQ_E_SHAPE;
    if (head_dim != 128) return CHERRYQ_E_UNSUPPORTED;
    return (int)cq::launch_attn_decode(reinterpret_cast<const __half *>(q), reinterpret_cast<const __half *>(k_cache),
                                       reinterpret_cast<const __half *>(v_cache), reinterpret_cast<__half *>(out),
                                       position, n_heads, n_kv_heads, max_len, 1.0f / sqrtf((float)head_dim),
                                       reinterpret_cast<hipStream_t>(stream));
}

int cherryq_decode_rope_attention_f16(const void *q, const void *k, const void *v, void *k_cache, void *v_cache,
                                      void *out, const int *position, int n_heads, int n_kv_heads, int head_dim,
                                      int max_len, float theta, void *stream) {
    if (!q || !k || !v || !k_cache || !v_cache || !out || !position) return CHERRYQ_E_NULL;
    if (n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads || max_len <= 0 || max_len > cq::attn_max_len())
        return CHERRYQ_E_SHAPE;
    if (head_dim != 128) return CHERRYQ_E_UNSUPPORTED;
    if (!cq::aligned(q, 16) || !cq::aligned(k, 16) || !cq::aligned(v, 16) || !cq::aligned(k_cache, 16) ||
        !cq::aligned(v_cache, 16) || !cq::aligned(out, 2))
        return CHERRYQ_E_ALIGN;
    return (int)cq::launch_rope_attn_decode(
        reinterpret_cast<const __half *>(q), reinterpret_cast<const __half *>(k), reinterpret_cast<const __half *>(v),
        reinterpret_cast<__half *>(k_cache), reinterpret_cast<__half *>(v_cache), reinterpret_cast<__half *>(out),
        position, n_heads, n_kv_heads, max_len, theta, 1.0f / sqrtf((float)head_dim),
        reinterpret_cast<hipStream_t>(stream));
}

int cherryq_decode_attention_max_slices(void) { return cq::attn_max_slices(); }
int cherryq_decode_attention_projection_slices(void) { return cq::attn_out_slices(); }

int cherryq_decode_rope_attention_split_f16(const void *q, const void *k, const void *v, void *k_cache, void *v_cache,
                                            void *partial, float *max_sum, int slices, const int *position, int n_heads,
                                            int n_kv_heads, int head_dim, int max_len, float theta, void *stream) {
    if (!q || !k || !v || !k_cache || !v_cache || !partial || !max_sum || !position) return CHERRYQ_E_NULL;
    if (n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads || max_len <= 0 || max_len > cq::attn_max_len() ||
        slices < 1 || slices > cq::attn_max_slices())
        return CHERRYQ_E_SHAPE;
    if (head_dim != 128) return CHERRYQ_E_UNSUPPORTED;
    if (!cq::aligned(q, 16) || !cq::aligned(k, 16) || !cq::aligned(v, 16) || !cq::aligned(k_cache, 16) ||
        !cq::aligned(v_cache, 16) || !cq::aligned(partial, 16) || !cq::aligned(max_sum, 8))
        return CHERRYQ_E_ALIGN;
    return (int)cq::launch_rope_attn_split(
        reinterpret_cast<const __half *>(q), reinterpret_cast<const __half *>(k), reinterpret_cast<const __half *>(v),
        reinterpret_cast<__half *>(k_cache), reinterpret_cast<__half *>(v_cache), reinterpret_cast<__half *>(partial),
        max_sum, position, n_heads, n_kv_heads, max_len, slices, theta, 1.0f / sqrtf((float)head_dim),
        reinterpret_cast<hipStream_t>(stream));
}

int cherryq_decode_attention_combine_f16(const void *partial, const float *max_sum, int slices, void *out, int n_heads,
                                         int head_dim, void *stream) {
    if (!partial || !max_sum || !out) return CHERRYQ_E_NULL;
    if (n_heads <= 0 || slices < 1 || slices > cq::attn_max_slices()) return CHERRYQ_E_SHAPE;
    if (head_dim != 128) return CHERRYQ_E_UNSUPPORTED;
    if (!cq::aligned(partial, 2) || !cq::aligned(max_sum, 4) || !cq::aligned(out, 2)) return CHERRYQ_E_ALIGN;
    return (int)cq::launch_attn_combine(reinterpret_cast<const __half *>(partial), max_sum,
                                        reinterpret_cast<__half *>(out), n_heads, slices,
                                        reinterpret_cast<hipStream_t>(stream));
}

int cherryq_decode_head_supported(int vocab, int hidden_size) { return cq::head_supported(vocab, hidden_size) ? 1 : 0; }

int cherryq_decode_head_f16(const void *hidden, const void *norm_weight, float eps, const void *lm_head, void *logits,
                            int vocab, int hidden_size, void *stream) {
    if (!hidden || !lm_head || !logits) return CHERRYQ_E_NULL;
    if (vocab <= 0 || hidden_size <= 0) return CHERRYQ_E_SHAPE;
    if (!cq::head_supported(vocab, hidden_size)) return CHERRYQ_E_UNSUPPORTED;
    if (!cq::aligned(hidden, 16) || !cq::aligned(lm_head, 16) || !cq::aligned(logits, 2) ||
        (norm_weight && !cq::aligned(norm_weight, 16)))
        return CHERRYQ_E_ALIGN;
    return (int)cq::launch_head(reinterpret_cast<const __half *>(hidden), reinterpret_cast<const __half *>(norm_weight), eps,
                                reinterpret_cast<const __half *>(lm_head), reinterpret_cast<__half *>(logits), vocab,
                                hidden_size, reinterpret_cast<hipStream_t>(stream));
}

int cherryq_decode_argmax_embed_f16(const void *logits, int vocab, const void *embed, int hidden, void *hidden_out,
                                    long long *next_token, long long *history, int history_len, int *position,
                                    void *stream) {
    if (!logits || !embed || !hidden_out || !next_token || !position) return CHERRYQ_E_NULL;
    if (vocab <= 0 || hidden <= 0 || history_len < 0) return CHERRYQ_E_SHAPE;
    if (!cq::aligned(logits, 16) || !cq::aligned(embed, 2) || !cq::aligned(hidden_out, 2) ||
        !cq::aligned(next_token, 8) || !cq::aligned(history, 8))
        return CHERRYQ_E_ALIGN;
    return (int)cq::launch_argmax_embed(reinterpret_cast<const __half *>(logits), vocab,
                                        reinterpret_cast<const __half *>(embed), hidden,
                                        reinterpret_cast<__half *>(hidden_out), next_token, history, history_len,
                                        position, reinterpret_cast<hipStream_t>(stream));
}

int cherryq_decode_silu_mul_f16(const void *gate, const void *up, void *out, int n, void *stream) {
    if (!gate || !up || !out) return CHERRYQ_E_NULL;
    if (n <= 0) return CHERRYQ_E_SHAPE;
    return (int)cq::launch_silu_mul(reinterpret_cast<const __half *>(gate), reinterpret_cast<const __half *>(up),
                                    reinterpret_cast<__half *>(out), n, reinterpret_cast<hipStream_t>(stream));
}

}  // extern "C"
