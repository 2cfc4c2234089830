// Internal launch interface between the C ABI (cq_api.hip) and the kernel files.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace cq {

size_t workspace_bytes(int B, int K, int N, int C);

// cq_generic.hip
template <int BITS, typename IO, typename IDX>
hipError_t launch_generic(const IO *vec, const uint8_t *qweight, const IO *cherry_weight,
                          const IDX *cherry_indices, const IO *scales, IO *mul, int B, int K, int N,
                          int C, int G, int accumulate, void *workspace, hipStream_t stream);
hipError_t launch_dequant_normal(int bits, const uint8_t *qweight, const float *scales, float *out, int Kn,
                                 int N, int G, hipStream_t stream);
hipError_t launch_unpack(int bits, const uint8_t *qweight, const __half *cherry_weight,
                         const int16_t *cherry_indices, const __half *scales, __half *dense, int K, int N,
                         int C, int G, hipStream_t stream);

// cq_matvec.hip: HBM-streaming matvec for 1..kMatvecMaxRows activation rows.  Returns false when
// the shape is not one it takes.
constexpr int kMatvecMaxRows = 4;
struct MatvecGeometry {
    int kpl;     // positions per lane and unit: 16 (64-position units) or 32 (128)
    int nw;      // wavefronts (= units) per workgroup
    int splits;  // workgroups per column tile; must not exceed 255 (8-bit arrival counter)
};
MatvecGeometry matvec_geometry(int bits, int K, int n_total, int C, int rows);
bool matvec_supported(int bits, int B, int K, int N, int C, int G);
bool matvec_rows_preferred(int bits, int B, int K, int N, int C, int G);  // 2..4 rows: this kernel rather than the batch one
hipError_t launch_matvec_rows(int bits, const __half *vec, const uint8_t *qweight, const __half *cherry_weight,
                              const int16_t *cherry_indices, const __half *scales, __half *mul, int rows, int K,
                              int N, int C, int G, int accumulate, void *workspace, hipStream_t stream);
hipError_t launch_matvec(int bits, const __half *vec, const uint8_t *qweight, const __half *cherry_weight,
                         const int16_t *cherry_indices, const __half *scales, __half *mul, int K, int N,
                         int C, int G, int accumulate, void *workspace, hipStream_t stream);

// One launch over up to kMaxGroup layers that share the activation vector, K, C and G (q/k/v or
// gate/up of a decoder block).  The zero-kept workspace needs 8 bytes per column of every
// member, each member's columns rounded up to a multiple of 256.
constexpr int kMaxGroup = 4;
struct MatvecMember {
    const uint8_t *qweight;
    const __half *cherry_weight;
    const int16_t *cherry_indices;
    const __half *scales;
    __half *mul;
    int N;
    int tile_begin;  // filled in by the launcher
};
struct MatvecGroup {
    MatvecMember m[kMaxGroup];
    int count;
};
// What the kernel does to the activation vector while staging it (at most one of the two):
// gate != null: act = fp16(fp16(silu(gate)) * vec);
// norm_weight != null: act = norm_weight * fp16(vec * rsqrt(mean(vec^2) + eps)).
struct MatvecPrologue {
    const __half *gate;
    const __half *norm_weight;
    float eps;
};
bool matvec_norm_supported(int bits, int K, int n_total, int C);
hipError_t launch_matvec_group(int bits, const __half *vec, const MatvecPrologue &pro, const MatvecMember *members,
                               int count, int K, int C, int G, int accumulate, void *workspace,
                               hipStream_t stream);

// cq_batch.hip: 2..16 batch rows per pass on the matrix cores.
struct BatchWorkspace {
    size_t tickets, workspace_total;                       // zero-kept workspace: offset, size
    size_t partial, xa, rowsum, rowshift, scratch_total;  // uninitialised scratch: offsets, size
};
BatchWorkspace batch_workspace(int K, int N, int C);
bool batch_supported(int bits, int B, int K, int N, int C, int G);
hipError_t launch_batch(int bits, const __half *vec, const uint8_t *qweight, const __half *cherry_weight,
                        const int16_t *cherry_indices, const __half *scales, __half *mul, int B, int K, int N,
                        int C, int G, int accumulate, void *workspace, void *scratch, hipStream_t stream);
size_t scratch_bytes(int B, int K, int N, int C);

// cq_gemm.hip: more than 16 rows (prompt processing) -- dequantise into LDS, fp16 MFMA tiles.
struct GemmPlan {
    int tm;                           // rows of an output tile: 128, 64 (calls of up to 64 rows) or 32 (up to 32)
    int mtiles, ntiles;               // tm x 128 output tiles
    int steps_normal, steps_total;    // K steps of 64 positions: packed part, then the cherry rows
    int Kp, Mp;                       // padded sizes of the compacted activation copy
    int splits, steps_per_split;      // K splits (grid.y)
    size_t workspace_bytes;           // zero-kept: one ticket per output tile
    size_t a_bytes, partial_bytes;    // scratch: compacted activations, then the per-split partial tiles
    size_t scratch_bytes;
};
constexpr int kGemmMinRows = 17;  // fewer rows go through the 16-row kernel
GemmPlan gemm_plan(int M, int K, int N, int C);
bool gemm_supported(int bits, int M, int K, int N, int C, int G);
hipError_t launch_gemm(int bits, const __half *vec, const uint8_t *qweight, const __half *cherry_weight,
                       const int16_t *cherry_indices, const __half *scales, __half *mul, int M, int K, int N, int C,
                       int G, int accumulate, void *workspace, void *scratch, hipStream_t stream);

// cq_stream.hip: batch-1 matvec over a load-time repacked weight stream (tiles of 16 columns, each
// tile's whole K range contiguous; no split-K, no workspace).
constexpr int kStreamTileCols = 16;
constexpr int kStreamUnitK = 128;
struct StreamGeo {
    int bits, K, N, C, Kn, ng, ntiles;
    uint32_t off_cherry, off_units, record_bytes;  // byte offsets inside a tile record, record size
    uint32_t hdr_bytes;                             // gather table + cherry columns in front of the tiles
};
constexpr int kStreamMaxGroup = 3;
struct StreamMember {  // one layer of a group launch
    const uint8_t *stream;
    __half *mul;
    int N;
};
struct StreamWalk {  // kernel argument of launches whose workgroups walk several tiles: workgroups per member
    int wgs[kStreamMaxGroup];
};
struct StreamGroup {  // kernel argument: the members' streams, outputs, widths and first workgroups
    const uint8_t *stream[kStreamMaxGroup];
    __half *mul[kStreamMaxGroup];
    int N[kStreamMaxGroup];
    int tile_begin[kStreamMaxGroup];  // first workgroup of each member
    int count;
};
StreamGeo stream_geo(int bits, int K, int N, int C);
hipError_t launch_stream_group(int bits, const __half *vec, const __half *norm_w, float eps,
                               const StreamMember *members, int count, int K, int C, int accumulate, hipStream_t s);
bool stream_group_supported(int bits, int K, int C, int G, const int *Ns, int count);
// 2 to 16 activation rows over the stream: a compaction launch into `scratch`, then the main launch
bool stream_cu_rows_supported(int bits, int B, int K, int N, int C);
hipError_t launch_stream_cu_rows(int bits, const __half *vec, const uint8_t *stream, __half *mul, int B, int K, int N, int C,
                                 int accumulate, hipStream_t s);
const char *stream_rows_kernel_name(int bits, int B, int K, int N, int C);
size_t stream_rows_scratch_bytes(int bits, int B, int K, int N, int C);
bool stream_rows_supported(int bits, int B, int K, int N, int C, int G);
hipError_t launch_stream_rows(int bits, const __half *vec, const uint8_t *stream, __half *mul, int B, int K, int N,
                              int C, int accumulate, void *scratch, hipStream_t s);
// cq_stream_cu.hip: the same launch with one workgroup per compute unit (up to 64 units per column)
bool stream_cu_supported(int bits, int K, int C, const int *Ns, int count);
hipError_t launch_stream_cu(int bits, const __half *vec, const __half *norm_w, float eps, const __half *gate,
                            const StreamMember *members, int count, int K, int C, int accumulate, hipStream_t s,
                            const float *attn_ml = nullptr);
// one repacked layer whose input row is formed from the partial results of launch_rope_attn_split
// with attn_out_slices() slices (part [slices][K] fp16, ml [slices][K / 128][2] fp32): the output projection
bool stream_attn_out_supported(int bits, int K, int C, int N);
hipError_t launch_stream_attn_out(int bits, const __half *part, const float *ml, const uint8_t *stream, __half *mul,
                                  int K, int N, int C, int accumulate, hipStream_t s);
int attn_max_slices();
int attn_out_slices();  // slices launch_stream_attn_out combines
// gate_proj and up_proj (same shape, same row) in one launch that stores fp16(fp16(silu(gate)) * up)
bool stream_pair_supported(int bits, int K, int N, int C);
hipError_t launch_stream_pair(int bits, const __half *vec, const __half *norm_w, float eps, const uint8_t *stream_gate,
                              const uint8_t *stream_up, __half *act, int K, int N, int C, hipStream_t s);
// one repacked layer behind the gated-MLP activation fp16(fp16(silu(gate)) * vec) (the down projection)
bool stream_gated_supported(int bits, int K, int N, int C);
hipError_t launch_stream_gated(int bits, const __half *vec, const __half *gate, const uint8_t *stream, __half *mul,
                               int K, int N, int C, int accumulate, hipStream_t s);
size_t stream_bytes(int bits, int K, int N, int C);
bool stream_faster(int bits, int K, int N, int C);
bool stream_uses_cu(int bits, int K, int N, int C);
bool stream_supported(int bits, int B, int K, int N, int C, int G);
hipError_t launch_stream(int bits, const __half *vec, const uint8_t *stream, __half *mul, int K, int N, int C,
                         int accumulate, hipStream_t s);
hipError_t launch_stream_pack(int bits, const uint8_t *qweight, const __half *cherry_weight,
                              const int16_t *cherry_indices, const __half *scales, uint8_t *stream, int K, int N,
                              int C, int G, hipStream_t s);
hipError_t launch_stream_unpack(int bits, const uint8_t *stream, uint8_t *qweight, __half *cherry_weight,
                                int16_t *cherry_indices, __half *scales, int K, int N, int C, int G, hipStream_t s);

// cq_pack.hip: dense fp16 weight -> packed buffers on the device.
hipError_t launch_pack(int bits, const __half *w, const int16_t *idx, uint8_t *qweight, __half *scales,
                       __half *cherry_weight, int K, int N, int C, int G, hipStream_t stream);

// cq_f32.hip: the 3-bit fp32-tensor variant on the fp32 matrix-core instruction, 2 rows and more.
bool f32_supported(int B, int K, int N, int C, int G);
size_t f32_scratch_bytes(int K, int C);
hipError_t launch_f32(const float *vec, const uint8_t *qweight, const float *cherry_weight,
                      const int32_t *cherry_indices, const float *scales, float *mul, int B, int K, int N, int C,
                      int G, int accumulate, void *workspace, void *scratch, hipStream_t stream);

// cq_fakequant.hip: training-side quantise-dequantise of the non-cherry columns, fp16 or fp32.
bool fake_quant_supported(int K, int C, int G);
hipError_t launch_fake_quant(int bits, bool fp32, const void *w, const int32_t *idx, void *out, int K, int N, int C,
                             int G, int ste, hipStream_t stream);

// cq_decode.hip: batch-1 decode-step glue kernels.
hipError_t launch_add_rmsnorm(__half *h, const __half *delta, const __half *weight, __half *y, int H, float eps,
                              hipStream_t stream);
hipError_t launch_rope_cache(__half *q, const __half *k, const __half *v, __half *k_cache, __half *v_cache,
                             const int *pos, int n_heads, int n_kv_heads, int head_dim, int max_len, float theta,
                             hipStream_t stream);
hipError_t launch_attn_decode(const __half *q, const __half *k_cache, const __half *v_cache, __half *out,
                              const int *pos, int n_heads, int n_kv_heads, int max_len, float scale,
                              hipStream_t stream);
hipError_t launch_rope_attn_decode(const __half *q, const __half *k, const __half *v, __half *k_cache,
                                   __half *v_cache, __half *out, const int *pos, int n_heads, int n_kv_heads,
                                   int max_len, float theta, float scale, hipStream_t stream);
// Attention with a head's positions dealt to `slices` workgroups (1 .. kAttnMaxSlices): partial results
// part[slices][n_heads * 128] fp16 and (maximum, sum) pairs ml[slices][n_heads][2] fp32; the combine
// kernel (or the output projection's staging, launch_stream_attn_out) forms the heads' results.
hipError_t launch_rope_attn_split(const __half *q, const __half *k, const __half *v, __half *k_cache, __half *v_cache,
                                  __half *part, float *ml, const int *pos, int n_heads, int n_kv_heads, int max_len,
                                  int slices, float theta, float scale, hipStream_t stream);
hipError_t launch_attn_combine(const __half *part, const float *ml, __half *out, int n_heads, int slices,
                               hipStream_t stream);
hipError_t launch_argmax_embed(const __half *logits, int vocab, const __half *embed, int hidden, __half *hid,
                               long long *next_token, long long *history, int history_len, int *pos,
                               hipStream_t stream);
// fp16 head with the final RMSNorm fused (norm_w may be null); hidden a multiple of 512, at most 8192
bool head_supported(int vocab, int hidden);
hipError_t launch_head(const __half *h, const __half *norm_w, float eps, const __half *W, __half *logits, int vocab,
                       int hidden, hipStream_t stream);
hipError_t launch_silu_mul(const __half *gate, const __half *up, __half *out, int n, hipStream_t stream);
int attn_max_len();

}  // namespace cq
