/*
 * libcherryq -- C ABI of the MI355X (gfx950) implementation of CherryQ's mixed-precision
 * quantized linear: packed 3/4-bit group-wise weights + fp16 "cherry" input channels.
 *
 * This header is the drop-in boundary.  It replaces the pybind11 module `quant_cuda` of
 * the reference (csrc/quant_cuda.cpp:72-77) and the four host launchers behind it
 * (csrc/quant_cuda_kernel.cu:117-188, 675-716, 838-866, 925-953).  All pointers are
 * device pointers owned by the caller; nothing here allocates, frees or synchronises.
 * Every call enqueues work on `stream` (a hipStream_t passed as void*; NULL = the null
 * stream) of the device that is current in the calling thread, and returns at once.
 *
 * Tensor layouts (row-major, contiguous), with K = in_features, N = out_features,
 * C = num_cherries, Kn = K - C, b = w_bits, G = group_size:
 *   vec            (B, K)            fp16 (or fp32 for the *_f32 entry point)
 *   qweight        (Kn/8*b, N)       uint8   llama/qlinear.py:51-54, packing :86-116
 *   cherry_weight  (C, N)            fp16    llama/qlinear.py:47-50
 *   cherry_indices (C,)              int16, ascending (int32 for *_f32)  llama/qlinear.py:43-46
 *   scales         (ceil(Kn/G), N)   fp16    llama/qlinear.py:55-58
 *   mul            (B, N)            fp16, accumulated into (mul += x W^T) when
 *                                    `accumulate` != 0, overwritten otherwise
 *
 * K, N and C are multiples of 8 (rows of whole 16-byte pieces); with int16 indices and C > 0,
 * K is at most 32768.
 *
 * Return value: 0 on success; negative = rejected argument (CHERRYQ_E_*); positive = a
 * hipError_t reported by the launch.  cherryq_status_string() names either.
 */
#ifndef CHERRYQ_H
#define CHERRYQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CHERRYQ_VERSION 1

enum {
    CHERRYQ_OK = 0,
    CHERRYQ_E_NULL = -1,        /* a required pointer is NULL */
    CHERRYQ_E_SHAPE = -2,       /* dimensions inconsistent with the buffer schema */
    CHERRYQ_E_GROUP = -3,       /* unsupported group size for this entry point */
    CHERRYQ_E_WORKSPACE = -4,   /* workspace missing, misaligned or too small */
    CHERRYQ_E_BITS = -5,        /* w_bits is not 3 or 4 */
    CHERRYQ_E_ALIGN = -6,       /* a pointer is not aligned as the kernels require */
    CHERRYQ_E_UNSUPPORTED = -7, /* valid request that this build does not implement */
    CHERRYQ_E_STATIC_LIMIT = -8 /* beyond the fixed workspace of cherryq_vecquant_matmul_f16_static */
};

int cherryq_version(void);
/* Test hook, not part of the reference interface: on != 0 routes every fused call through the
 * library's general kernel instead of the specialised ones (the tests compare the two). */
void cherryq_set_force_generic(int on);
const char *cherryq_status_string(int status);

/*
 * Device memory the fused entry points need beside their operands (the reference's kernels need
 * none: they add fp16 partials into `mul` with atomics, csrc/quant_cuda_kernel.cu:833).
 *
 * workspace: where the K splits of different workgroups meet -- one 64-bit accumulator word per
 *   output element (fixed-point running sum plus an arrival count, added with a single atomic)
 *   and one arrival ticket per 256-column tile.  At least cherryq_workspace_bytes() bytes,
 *   256-byte aligned.  It must be all zero before the first call; every call leaves it all zero
 *   again, whatever the shapes of earlier calls were.  The one exception: a call that returns a
 *   positive value (the runtime refused or aborted a launch) may leave words behind -- zero the
 *   workspace again (hipMemsetAsync, or a fill kernel under capture) before reusing it.
 *   Numerical contract of the accumulator words (batch 1 to 4, and every shape that takes the
 *   general kernel): each workgroup's partial sum is rounded to a multiple of 2^-34 and, with fp16
 *   tensors, clamped to +-(2^21 - 1); the running total must stay within +-2^21 (32 times fp16's
 *   largest value).  Within that range the sum is exact and independent of the order in which
 *   workgroups arrive, so results are deterministic; totals beyond fp16's range come out as
 *   infinities of the right sign.  Outside it -- partial sums of one sign that add up beyond 2^21 --
 *   the total wraps and the result is unspecified; a NaN activation gives infinite outputs
 *   (either sign), not NaN.  With fp32 tensors (cherryq_vecquant3matmul_f32) partials of 2^13
 *   and more, infinities and NaN are carried in a float side accumulator instead: range and
 *   special values behave as in fp32, the absolute resolution stays 2^-34 per partial.
 * scratch: uninitialised memory for the batched paths (batch >= 2): per-split partial tiles and
 *   the activations laid out in matrix-core operand order.  At least cherryq_scratch_bytes()
 *   bytes (0 for batch 1, then it may be NULL), 256-byte aligned.
 * Both sizes depend on the batch: up to 16 rows run in the streaming or the small-batch kernel, more (prompt
 * processing) in the tiled GEMM kernel, whose compacted copy of the activations and partial
 * tiles grow with the number of rows.  Size the buffers for the largest batch that will be passed.
 * Calls that may overlap in time (different streams) must use different workspace and scratch.
 * cherryq_scratch_bytes_f32() is the scratch size for the fp32-tensor entry point, which is not 0
 * at batch 1: with such a buffer one row runs on the matrix-core kernel too, without (NULL) on a
 * slower general one.
 */
size_t cherryq_workspace_bytes(int batch, int in_features, int out_features, int num_cherries);
size_t cherryq_scratch_bytes(int batch, int in_features, int out_features, int num_cherries);
size_t cherryq_scratch_bytes_f32(int batch, int in_features, int out_features, int num_cherries);

/*
 * Replaces quant_cuda.vecquant4matmul_cherryq (csrc/quant_cuda.cpp:56-69,
 * csrc/quant_cuda_kernel.cu:675-835).  group_size must be a multiple of 32 that is
 * >= 128 (the reference rejects < 128, :684, and silently assumes a multiple of 128).
 */
int cherryq_vecquant4matmul_f16(const void *vec, const uint8_t *qweight, const void *cherry_weight,
                                const int16_t *cherry_indices, const void *scales, void *mul,
                                int batch, int in_features, int out_features, int num_cherries,
                                int group_size, int accumulate, void *workspace,
                                size_t workspace_bytes, void *scratch, size_t scratch_bytes,
                                void *stream);

/*
 * Replaces quant_cuda.vecquant3matmul_cherryq with fp16=True (csrc/quant_cuda.cpp:41-54,
 * csrc/quant_cuda_kernel.cu:117-188, kernels :316-438 for group 64 and :558-672 for
 * multiples of 128).  group_size must be a multiple of 32; the reference silently does
 * nothing for group sizes other than 64 or a multiple of 128.
 */
int cherryq_vecquant3matmul_f16(const void *vec, const uint8_t *qweight, const void *cherry_weight,
                                const int16_t *cherry_indices, const void *scales, void *mul,
                                int batch, int in_features, int out_features, int num_cherries,
                                int group_size, int accumulate, void *workspace,
                                size_t workspace_bytes, void *scratch, size_t scratch_bytes,
                                void *stream);

/*
 * Replaces quant_cuda.vecquant3matmul_cherryq with fp16=False: fp32 vec / cherry_weight /
 * scales / mul and int32 cherry_indices (csrc/quant_cuda_kernel.cu:191-314, 441-556;
 * caller: benchmark_speed.py:20-32).
 */
int cherryq_vecquant3matmul_f32(const float *vec, const uint8_t *qweight, const float *cherry_weight,
                                const int32_t *cherry_indices, const float *scales, float *mul,
                                int batch, int in_features, int out_features, int num_cherries,
                                int group_size, int accumulate, void *workspace,
                                size_t workspace_bytes, void *scratch, size_t scratch_bytes,
                                void *stream);

/*
 * Replace quant_cuda.Dequantize3Normal / Dequantize4Normal (csrc/quant_cuda.cpp:26-38,
 * csrc/quant_cuda_kernel.cu:838-1010): out[k, n] = (code(k, n) - c_b) * scales[k / G, n]
 * for the Kn compacted normal positions, fp32 scales and fp32 out of shape (>= Kn, N).
 * `height` is in_features.  The reference's 4-bit launcher indexes rows with the 3-bit
 * block height (:934, :964) and so covers only part of the matrix; this one covers all
 * of it.
 */
int cherryq_dequantize3_normal_f32(const uint8_t *qweight, const float *scales, float *out,
                                   int height, int out_features, int cherry_size, int group_size,
                                   void *stream);
int cherryq_dequantize4_normal_f32(const uint8_t *qweight, const float *scales, float *out,
                                   int height, int out_features, int cherry_size, int group_size,
                                   void *stream);

/*
 * Device-side QuantLinear.unpack() (llama/qlinear.py:120-162): the dense (N, K) fp16
 * weight, normal column normal[k] = RN16((code - c_b) * scale) bit for bit as the
 * reference's torch code computes it, cherry column idx[c] = cherry_weight[c, :].
 */
int cherryq_unpack_f16(int w_bits, const uint8_t *qweight, const void *cherry_weight,
                       const int16_t *cherry_indices, const void *scales, void *dense,
                       int in_features, int out_features, int num_cherries, int group_size,
                       void *stream);

/*
 * pack() on the device: dense fp16 `weight` (out_features, in_features), row-major, and the
 * ASCENDING cherry channels -> qweight, scales (ceil(Kn/group_size), out_features) and
 * cherry_weight (num_cherries, out_features), bit for bit what QuantLinear.pack() computes on
 * the host for fp16 weights (llama/qlinear.py:67-118 with llama/cherry_linear.py:69-75 and
 * FullSymQuantizer.get_scaling_factor / quantize, llama/quantizer.py:148-158).  cherry_indices
 * must hold distinct channels in [0, in_features).  No workspace.
 */
int cherryq_pack_f16(int w_bits, const void *weight, const int16_t *cherry_indices, uint8_t *qweight,
                     void *scales, void *cherry_weight, int in_features, int out_features, int num_cherries,
                     int group_size, void *stream);

/*
 * The training-side forward's weight (QuantLinear._adjust_weight, llama/cherry_linear.py:77-99
 * of the reference): `out` = `weight` (out_features, in_features), row-major, with every
 * NON-cherry input channel replaced by FullSymQuantizer.transform of it
 * (llama/quantizer.py:165-170) under per-row scales of `group_size` consecutive compacted normal
 * channels (llama/cherry_linear.py:69-75, llama/quantizer.py:148-152), every operation rounded
 * to the weight's dtype as torch does: bit for bit the reference's result for fp16 and fp32
 * weights.  ste != 0 gives the straight-through form the training branch feeds to the matmul,
 * (q - w) + w evaluated in the weight dtype on every channel (:97-98); ste == 0 is what
 * prepare_weight_for_inference stores (:48-61).  w_bits 2..4.  cherry_indices (int32, as the
 * QAT module keeps them) need be neither sorted nor distinct; entries outside
 * [0, in_features) are ignored.  `out` may be `weight` itself.  No workspace.  Returns
 * CHERRYQ_E_UNSUPPORTED beyond 65536 input channels or 4096 groups per row.
 */
int cherryq_fake_quant_f16(int w_bits, const void *weight, const int32_t *cherry_indices, void *out,
                           int in_features, int out_features, int num_cherries, int group_size, int ste,
                           void *stream);
int cherryq_fake_quant_f32(int w_bits, const void *weight, const int32_t *cherry_indices, void *out,
                           int in_features, int out_features, int num_cherries, int group_size, int ste,
                           void *stream);

/*
 * cherryq_vecquant{3,4}matmul_f16 for callers that cannot allocate device memory or carry a
 * workspace around (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference.  Same arguments without workspace / scratch, same
 * kernels and results for 1 to 4 activation rows; the split-K accumulator words live in a
 * fixed array of CHERRYQ_STATIC_WORKSPACE_BYTES inside the library's device code (held by every
 * GPU the library runs on until the process ends), so batch * out_features may not exceed
 * 131072 and batch may not exceed 4: beyond that the call returns CHERRYQ_E_STATIC_LIMIT and
 * launches nothing.  The call makes no hipMalloc / hipFree and no allocating library call; its
 * first call on a device looks the array's address up (hipGetSymbolAddress) and should happen
 * outside a stream capture.  All calls on one GPU share that GPU's array: calls that may overlap
 * in time on one GPU (different streams) race -- serialise them or use the entry points above
 * with workspaces of their own.  The kernels return every word they used to zero; if a launch
 * is refused by the runtime, the next call clears the whole array first (a fill kernel on the
 * call's stream, no hipMemset).
 */
#define CHERRYQ_STATIC_WORKSPACE_BYTES (1u << 20)
int cherryq_vecquant_matmul_f16_static(int w_bits, const void *vec, const uint8_t *qweight, const void *cherry_weight,
                                       const int16_t *cherry_indices, const void *scales, void *mul, int batch,
                                       int in_features, int out_features, int num_cherries, int group_size,
                                       int accumulate, void *stream);

/*
 * Load-time repack of a packed layer into a weight stream laid out for this GPU, and the batch-1
 * matvec over it.  The reference has no counterpart: its kernels read the checkpoint layout
 * directly (csrc/quant_cuda_kernel.cu:811-831 4-bit, :649-667 3-bit) and so does every entry point
 * above.  The stream holds the same information -- every code, scale, cherry row and cherry index,
 * bit for bit; cherryq_unprepack_f16 is the exact inverse -- rearranged so that 16 output columns'
 * whole input range is one contiguous record of 1 KB (768 B for 3 bits) pieces that a wavefront
 * loads with one instruction and masks straight into matrix-core operands.  A workgroup then owns
 * whole output columns: no partial sums leave it, so the call needs no workspace, uses no atomics
 * and rounds once from fp32, like the entry points above.  Arithmetic contract and result are
 * those of cherryq_vecquant{3,4}matmul_f16 at batch 1 (mul = or += vec W^T).
 *
 * stream: cherryq_prepack_bytes() bytes, 256-byte aligned, written by cherryq_prepack_f16 once
 * per layer.  group_size must be a multiple of 128 (the stream stores one scale row per 128
 * positions); cherryq_prepack_supported() says whether a shape is taken at all (at most 128
 * cherry channels, at most 28672 + 128 input channels, a stream of less than 2 GiB, batch 1).  vec
 * must be 16-byte aligned.
 */
size_t cherryq_prepack_bytes(int w_bits, int in_features, int out_features, int num_cherries);
int cherryq_prepack_supported(int w_bits, int batch, int in_features, int out_features, int num_cherries,
                              int group_size);
/* 1 where the matvec over the stream measured faster on MI355X than the one over the checkpoint
 * layout (today: every shape the launch with one workgroup per compute unit takes -- every
 * LLaMA-7B, -13B and -70B projection among them; within 3 % at worst on the shapes measured), 0
 * elsewhere or if unsupported: what a loader asks before spending the extra copy of the weights. */
int cherryq_prepack_recommended(int w_bits, int in_features, int out_features, int num_cherries, int group_size);
/* The same for `batch` activation rows, for a caller that holds both layouts: 1 where
 * cherryq_matmul_prepacked_f16 measured faster on MI355X than cherryq_vecquant{3,4}matmul_f16 over
 * the checkpoint layout -- one row as above; 2 to 4 rows wherever the four-row form of the
 * one-workgroup-per-compute-unit kernel takes the layer (up to 96 units of 128 input channels);
 * from 4 rows on layers of up to 32 units and from 8 rows on deeper ones otherwise; 0 beyond 16
 * rows.  No counterpart in the reference (its kernel loops over the rows, quant_cuda_kernel.cu:797). */
int cherryq_prepack_rows_recommended(int w_bits, int batch, int in_features, int out_features, int num_cherries,
                                     int group_size);
/* The kernel cherryq_matvec_prepacked_f16 launches for a layer, as it appears in a profiler's
 * kernel trace (without template arguments): "cq::stream_cu_kernel" (one workgroup per compute
 * unit) or "cq::stream_kernel"; "" for shapes the entry point does not take. */
const char *cherryq_matvec_prepacked_kernel_name(int w_bits, int in_features, int out_features, int num_cherries);
/* The same for cherryq_matmul_prepacked_f16 with `batch` rows (2 to 16): its kernels in launch order, joined by " + ". */
const char *cherryq_matmul_prepacked_kernel_name(int w_bits, int batch, int in_features, int out_features, int num_cherries);
int cherryq_prepack_f16(int w_bits, const uint8_t *qweight, const void *cherry_weight, const int16_t *cherry_indices,
                        const void *scales, void *stream, size_t stream_bytes, int in_features, int out_features,
                        int num_cherries, int group_size, void *hip_stream);
int cherryq_unprepack_f16(int w_bits, const void *stream, size_t stream_bytes, uint8_t *qweight, void *cherry_weight,
                          int16_t *cherry_indices, void *scales, int in_features, int out_features, int num_cherries,
                          int group_size, void *hip_stream);
int cherryq_matvec_prepacked_f16(int w_bits, const void *vec, const void *stream, size_t stream_bytes, void *mul,
                                 int batch, int in_features, int out_features, int num_cherries, int accumulate,
                                 void *hip_stream);

/*
 * The same over 2 to 16 activation rows (vec (batch, in_features), mul (batch, out_features)): the
 * matrix-core tile that the one-row kernel fills with copies of one row takes 16 different rows
 * at the same price, still without split-K or workspace.  Two to four rows (layers of up to 96
 * units of 128 input channels) and five to eight rows (up to 48 units) run in the one-row kernel's
 * own launch shape, tile row m holding activation row m mod 4 or 8: one launch, no scratch buffer
 * (cherryq_prepacked_scratch_bytes() is 0 and scratch may be NULL).  Otherwise the compacted activations of all rows
 * are brought into matrix-core operand order once (a first small launch into an uninitialised
 * scratch buffer of cherryq_prepacked_scratch_bytes() bytes, 256-byte aligned; for up to 4 rows
 * inside the main launch) and then stay in LDS or in registers while a workgroup walks its
 * tiles.  Layers deeper than 8192 + 128 input channels (64 units of 128 positions), up to 256
 * units, are taken in four slices of units with fp32 partial outputs in the scratch buffer and one
 * more launch that adds them.  batch == 1 forwards to
 * cherryq_matvec_prepacked_f16 (scratch may then be NULL).  cherryq_prepack_supported(w_bits,
 * batch, ...) says whether a batch is taken.  vec must be 16-byte aligned (the rows are read as
 * 16-byte pieces; in_features is a multiple of 8, so every row then is).
 */
size_t cherryq_prepacked_scratch_bytes(int w_bits, int batch, int in_features, int out_features, int num_cherries);
int cherryq_matmul_prepacked_f16(int w_bits, const void *vec, const void *stream, size_t stream_bytes, void *mul,
                                 int batch, int in_features, int out_features, int num_cherries, int accumulate,
                                 void *scratch, size_t scratch_bytes, void *hip_stream);

/*
 * The decode step's grouped launch over repacked layers (the counterpart of
 * cherryq_decode_matvec_group_f16 below for layers held as weight streams): 1 to 3 layers that
 * share w_bits, in_features and num_cherries and read the same (1, in_features) row -- q / k / v,
 * gate / up, or one projection alone -- in ONE launch; layers[i].mul (+)= act W_i^T with
 * act = vec, or norm_weight * fp16(vec * rsqrt(mean(vec^2) + eps)) when norm_weight is given
 * (the RMSNorm in front of the projections, llama/modeling_llama_quant.py:75-89, fused into the
 * activation staging).  No workspace.  vec and norm_weight 16-byte aligned.
 */
typedef struct cherryq_stream_layer {
    const void *stream;   /* written by cherryq_prepack_f16 */
    size_t stream_bytes;
    void *mul;            /* (1, out_features) fp16 */
    int out_features;
} cherryq_stream_layer;
int cherryq_decode_matvec_group_prepacked_f16(int w_bits, const void *vec, const void *norm_weight /* may be NULL */,
                                              float eps, const cherryq_stream_layer *layers, int n_layers,
                                              int in_features, int num_cherries, int accumulate, void *hip_stream);

/*
 * gate_proj and up_proj of a gated MLP (two repacked layers of the same shape that read the same
 * row) in ONE launch that stores the activation the down projection reads,
 * act = fp16(fp16(silu(g)) * u) with g = fp16(vec' Wg^T), u = fp16(vec' Wu^T) and vec' = vec or
 * its RMSNorm (norm_weight given) -- llama/modeling_llama_quant.py:251 with the rounding points of
 * its fp16 tensors -- instead of the two results: pairs of wavefront teams work on the same 16
 * columns of both layers and meet in LDS.  No workspace; act (1, out_features) fp16 is overwritten.
 * cherryq_decode_gate_up_prepacked_supported() says whether a shape is taken (up to 8192 + 128
 * input channels).  No counterpart in the reference, whose three projections are separate calls.
 */
int cherryq_decode_gate_up_prepacked_supported(int w_bits, int in_features, int out_features, int num_cherries);
int cherryq_decode_gate_up_prepacked_f16(int w_bits, const void *vec, const void *norm_weight /* may be NULL */, float eps,
                                         const void *gate_stream, size_t gate_stream_bytes, const void *up_stream,
                                         size_t up_stream_bytes, void *act, int in_features, int out_features,
                                         int num_cherries, void *hip_stream);

/*
 * The down projection of a gated MLP over a repacked layer: mul (+)= act W^T with
 * act = fp16(fp16(silu(vec_gate)) * vec), the activation llama/modeling_llama_quant.py:251 forms
 * between the gate / up and the down projection, computed while the row is staged (the
 * counterpart of cherryq_decode_matvec_group_f16's vec_gate for layers held as weight streams).
 * One launch, no workspace.  vec and vec_gate: (1, in_features) fp16, 16-byte aligned.
 */
int cherryq_decode_matvec_gated_prepacked_f16(int w_bits, const void *vec, const void *vec_gate, const void *stream,
                                              size_t stream_bytes, void *mul, int in_features, int out_features,
                                              int num_cherries, int accumulate, void *hip_stream);

/*
 * The output projection of the attention block over a repacked layer, reading the partial results
 * of cherryq_decode_rope_attention_split_f16 (slices must be cherryq_decode_attention_projection_slices();
 * in_features = n_heads * 128): mul (+)= act W^T with act the combined heads' results, formed with
 * the arithmetic of cherryq_decode_attention_combine_f16 while the row is staged.  One launch, no
 * workspace.  partial 16-byte, max_sum 8-byte aligned.
 */
int cherryq_decode_matvec_attention_prepacked_supported(int w_bits, int in_features, int out_features, int num_cherries);
int cherryq_decode_matvec_attention_prepacked_f16(int w_bits, const void *partial, const float *max_sum, int slices,
                                                  const void *stream, size_t stream_bytes, void *mul, int in_features,
                                                  int out_features, int num_cherries, int accumulate, void *hip_stream);

/*
 * One batch-1 launch over 1..4 packed layers that read the SAME activation vector and share
 * in_features, num_cherries, group_size and w_bits: q/k/v_proj (llama/modeling_llama_quant.py
 * :346-348 of the reference) or gate/up_proj (:251).  Arithmetic per layer is that of
 * cherryq_vecquant{3,4}matmul_f16 at batch 1; the point is that the layers' weight streams
 * overlap inside one grid instead of running as short launches one after another.
 * When vec_gate is non-NULL the activations are fp16(fp16(silu(vec_gate)) * vec), the
 * gated-MLP product that feeds down_proj (:251), formed while the kernel stages its activations.
 * When norm_weight is non-NULL, vec is the un-normalised hidden state and the activations are
 * norm_weight * fp16(vec * rsqrt(mean(vec^2) + eps)), the RMSNorm of :75-89 in front of q/k/v
 * and gate/up, each workgroup taking the sum of squares itself (vec must be 16-byte aligned).
 * workspace: zero-kept like the matmul workspace, cherryq_group_workspace_bytes() bytes.
 * Returns CHERRYQ_E_UNSUPPORTED for vec_gate / norm_weight with shapes the streaming kernel
 * does not take (the caller then runs the separate decode entry points below).
 */
typedef struct cherryq_layer {
    const uint8_t *qweight;
    const void *cherry_weight;
    const int16_t *cherry_indices;
    const void *scales;
    void *mul;
    int out_features;
} cherryq_layer;
size_t cherryq_group_workspace_bytes(int n_layers, const int *out_features);
int cherryq_decode_matvec_group_f16(int w_bits, const void *vec, const void *vec_gate /* may be NULL */,
                                    const void *norm_weight /* may be NULL */, float eps,
                                    const cherryq_layer *layers, int n_layers, int in_features,
                                    int num_cherries, int group_size, int accumulate, void *workspace,
                                    size_t workspace_bytes, void *stream);

/*
 * Decode-step glue for a LLaMA-shaped decoder, batch 1, fp16: what sits between two fused
 * matvecs in the caller's token step (llama/modeling_llama_quant.py of the reference: RMSNorm
 * :75-89, rotary embedding :179-210, attention over the KV cache :391-402 and :671-696, gated
 * MLP :251), one launch each, so that the step can be captured as a short HIP graph.  They have
 * no counterpart in the reference's extension, which leaves these operations to PyTorch.
 * `position` is a device pointer to the current token position (so a captured graph can be
 * replayed while the caller increments it); caches are [kv_head][max_len][head_dim].
 */
int cherryq_decode_add_rmsnorm_f16(void *hidden, const void *delta /* may be NULL */, const void *weight,
                                   void *normed, int hidden_size, float eps, void *stream);
int cherryq_decode_rope_cache_f16(void *q, const void *k, const void *v, void *k_cache, void *v_cache,
                                  const int *position, int n_heads, int n_kv_heads, int head_dim, int max_len,
                                  float theta, void *stream);
int cherryq_decode_attention_f16(const void *q, const void *k_cache, const void *v_cache, void *out,
                                 const int *position, int n_heads, int n_kv_heads, int head_dim, int max_len,
                                 void *stream);
/* rope_cache followed by attention for the same token, as one launch (q is not modified). */
int cherryq_decode_rope_attention_f16(const void *q, const void *k, const void *v, void *k_cache, void *v_cache,
                                      void *out, const int *position, int n_heads, int n_kv_heads,
                                      int head_dim, int max_len, float theta, void *stream);
/*
 * The same with a head's positions dealt to `slices` workgroups (1 .. cherryq_decode_attention_max_slices(),
 * which is 8): slice s takes the blocks of 64 positions s, s + slices, s + 2 slices, ..., is a softmax
 * of its own, and stores its result into
 * partial[s][n_heads * head_dim] (fp16) and the maximum of its scores and the sum of their
 * exponentials into max_sum[s][n_heads][2] (fp32).  A head's result is sum_s c_s partial[s] with
 * c_s = exp(max_s - max) sum_s / sum_t exp(max_t - max) sum_t; cherryq_decode_attention_combine_f16
 * forms it (fp16), and cherryq_decode_matvec_attention_prepacked_f16 is an output projection
 * (llama/modeling_llama_quant.py:404, o_proj) over a repacked layer that forms it while it stages its
 * input (for cherryq_decode_attention_projection_slices() = 4 slices), so that split attention +
 * projection stay two launches.  With slices = 1, and up to position 63 with any number, the combined
 * result equals cherryq_decode_rope_attention_f16's bit for bit; otherwise it differs by the
 * roundings of the partial results (about 4e-4 relative).  One workgroup per head reads the
 * head's whole cache through one compute unit: 50 us per layer at 4000 positions of 32 heads
 * against 22 us with 4 slices (18 against 11 at 1000 positions; at 256 positions the two are within
 * 0.5 us and the combining costs more than that).  No counterpart in the reference.
 */
int cherryq_decode_attention_max_slices(void);
int cherryq_decode_attention_projection_slices(void);
int cherryq_decode_rope_attention_split_f16(const void *q, const void *k, const void *v, void *k_cache, void *v_cache,
                                            void *partial, float *max_sum, int slices, const int *position, int n_heads,
                                            int n_kv_heads, int head_dim, int max_len, float theta, void *stream);
int cherryq_decode_attention_combine_f16(const void *partial, const float *max_sum, int slices, void *out, int n_heads,
                                         int head_dim, void *stream);
/*
 * Unquantised fp16 head of the decode step: logits (vocab fp16) = act W^T with lm_head W (vocab,
 * hidden_size) row-major as the reference holds it (llama/modeling_llama_quant.py:1132), fp32
 * accumulation, one rounding; act = norm_weight * fp16(hidden * rsqrt(mean(hidden^2) + eps)), the
 * final RMSNorm (:1064, :75-89) fused into the launch, or hidden itself when norm_weight is NULL.
 * A plain HBM stream over the matrix (the largest single read of a token step).  hidden_size a
 * multiple of 8, at most 8192 (cherryq_decode_head_supported); hidden, norm_weight, lm_head
 * 16-byte aligned.
 */
int cherryq_decode_head_supported(int vocab, int hidden_size);
int cherryq_decode_head_f16(const void *hidden, const void *norm_weight /* may be NULL */, float eps,
                            const void *lm_head, void *logits, int vocab, int hidden_size, void *stream);

/*
 * Tail of a greedy step: *next_token = argmax(logits[0..vocab)) (lowest index among equal maxima),
 * history[*position] = that token when history is non-NULL and the position lies below
 * history_len, hidden_out[0..hidden) = embed[token] (the next step's input), *position += 1.
 * The host side of the reference's generation loop (benchmark_perplexity.py:92-109).
 */
int cherryq_decode_argmax_embed_f16(const void *logits, int vocab, const void *embed, int hidden,
                                    void *hidden_out, long long *next_token, long long *history /* may be NULL */,
                                    int history_len, int *position, void *stream);
int cherryq_decode_silu_mul_f16(const void *gate, const void *up, void *out, int n, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* CHERRYQ_H */
