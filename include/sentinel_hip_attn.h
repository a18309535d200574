/*
 * sentinel_hip_attn.h - C ABI of the MI355X (gfx950) causal flash-attention forward / backward.
 *
 * These entry points stand where Sentinel's CUDA attention dispatch stands: they take the same
 * tensors, geometry and column window as
 *     CudaFlashAttention::forwardMultiHead   (sentinel/NeuralNet/Cuda/CudaFlashAttention.hpp:30,
 *                                             sentinel/NeuralNet/Cuda/CudaFlashAttention.cu:1543-1609)
 *     CudaFlashAttention::backwardMultiHead  (sentinel/NeuralNet/Cuda/CudaFlashAttention.hpp:40,
 *                                             sentinel/NeuralNet/Cuda/CudaFlashAttention.cu:1615-1700)
 * as called from CudaCausalSelfAttention::attendFullSequence / ::backward
 * (sentinel/NeuralNet/Cuda/CudaCausalSelfAttention.cu:237-249, :421-438), but as plain pointers and
 * sizes: the caller owns every buffer, nothing is allocated, freed or synchronised inside a call, and
 * all work is enqueued on the stream that is passed in (capture-safe).
 *
 * Differences from the CUDA path they replace, all additive:
 *   - head_dim up to 128 (the CUDA path stops at 64, CudaFlashAttention.hpp:16);
 *   - grouped-query attention is native: k / v / dk / dv have kv_heads heads and query head h reads
 *     kv head h / (q_heads / kv_heads), so no expanded K/V copies and no gradient reduction pass
 *     (replaces expandKvHeadsInto / reduceKvHeadGradsInto, CudaCausalSelfAttention.cu:27-44);
 *   - dq, dk and dv are overwritten deterministically (no atomics); pre-zeroed buffers, as the
 *     CUDA caller provides (CudaCausalSelfAttention.cu:392-394), are fine but not required;
 *   - any seq_len >= 1 and any stride are accepted (no multiple-of-4 rule).
 */
#ifndef SENTINEL_HIP_ATTN_H
#define SENTINEL_HIP_ATTN_H

#include <stddef.h>

#if defined(__GNUC__)
#define SENTINEL_HIP_API __attribute__((visibility("default")))
#else
#define SENTINEL_HIP_API
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* Return codes. The C++ shim maps INVALID_ARGUMENT and UNSUPPORTED to std::invalid_argument and
 * RUNTIME to std::runtime_error, the exception types of validateMultiHeadShape / resolveColumnWindow
 * (CudaFlashAttention.cu:1458-1471, :1533-1539) and throwIfCudaFailed (:1608). */
enum {
    SENTINEL_HIP_OK = 0,
    SENTINEL_HIP_INVALID_ARGUMENT = 1, /* null pointer, bad head geometry, bad column window */
    SENTINEL_HIP_UNSUPPORTED = 2,      /* head_dim / dtype / layout combination has no kernel: use the dense path */
    SENTINEL_HIP_RUNTIME = 3           /* no device, launch failure */
};

/* element type of q, k, v, out, d_out, dq, dk, dv (lse and delta are always float) */
enum { SENTINEL_HIP_F32 = 0, SENTINEL_HIP_BF16 = 1, SENTINEL_HIP_F16 = 2 };

/* arithmetic used for the matrix products */
enum {
    SENTINEL_HIP_COMPUTE_AUTO = -1, /* F32 io -> F32 arithmetic; BF16 / F16 io -> MFMA in that type */
    SENTINEL_HIP_COMPUTE_F32 = 0,   /* exact fp32 FMA path (any head_dim <= 128) */
    SENTINEL_HIP_COMPUTE_BF16 = 1,  /* bf16 MFMA, fp32 accumulation: the kernels are tiled for head_dim 64 and 128; fp32
                                       column tensors of any head_dim that is a multiple of 8 (<= 128) run on them too,
                                       zero-padded to 64 / 128 by the conversion pass they go through anyway (the CUDA
                                       path's generic kernel takes any head_dim <= 64, CudaFlashAttention.cu:1596-1599);
                                       16-bit [B,H,T,d] tensors need head_dim 64 or 128 */
    SENTINEL_HIP_COMPUTE_F16 = 2    /* fp16 MFMA, fp32 accumulation: same rules */
};

/*
 * Tensor layouts.
 *  SENTINEL_HIP_LAYOUT_COLUMNS  Sentinel's device layout (CudaFlashAttention.cu:129-135):
 *        element(head, dim, column) = base[(head * head_dim + dim) * stride_columns + column]
 *        pack p occupies columns [column_start + p * seq_len, column_start + (p + 1) * seq_len);
 *        lse is q_heads x stride_columns. Columns outside the pack window are never written.
 *        With 16-bit arithmetic the operands are converted into the workspace by passes of their own; the results
 *        (out, dq, dk, dv) are written by the attention kernels themselves, as the fp32 values of their accumulators
 *        (rounded to the arithmetic type they equal the BHTD layout's results).
 *  SENTINEL_HIP_LAYOUT_BHTD     contiguous [pack_count, heads, seq_len, head_dim]; lse is
 *        [pack_count, q_heads, seq_len]; stride_columns and column_start are ignored.
 * delta workspace (both layouts): q_heads x (pack_count * seq_len) floats, the shape the CUDA caller
 * keeps in CudaCausalSelfAttention::flashDelta (CudaFlashAttention.cu:1640).
 */
enum { SENTINEL_HIP_LAYOUT_COLUMNS = 0, SENTINEL_HIP_LAYOUT_BHTD = 1 };

/*
 * Workspace flags, OR-ed into the `layout` argument. They matter where a workspace is used at all (COLUMNS layout with
 * MFMA arithmetic) and are ignored elsewhere. The CUDA layer keeps flashLogSumExp from its forward call for its
 * backward call (CudaCausalSelfAttention.cu:237-249, :421-438); a caller that keeps the workspace the same way saves
 * the backward four of its five conversion passes:
 *  SENTINEL_HIP_WORKSPACE_KEEP   forward: `workspace` is sized for the BACKWARD call
 *        (sentinel_hip_flash_workspace_bytes(..., backward = 1)) and the 16-bit copies of q, k, v (rotated, if the call
 *        rotates) and out are left in it where the backward call looks for them.
 *  SENTINEL_HIP_WORKSPACE_REUSE  backward: `workspace` is the one a KEEP forward call with the same tensors, geometry,
 *        mask and rotation filled, untouched since: q, k, v and out are not read or converted again, only d_out is
 *        (the q / k / v / out pointers are still validated but not dereferenced). Passing a workspace that was not
 *        filled that way gives wrong gradients: nothing can check it.
 */
enum { SENTINEL_HIP_WORKSPACE_KEEP = 0x100, SENTINEL_HIP_WORKSPACE_REUSE = 0x200 };

/*
 * Scratch the caller must provide for a configuration (bytes; 0 when none is needed). Only the
 * COLUMNS layout with MFMA arithmetic needs any (type-converted [B,H,T,d] copies of the operands).
 * `backward` != 0 sizes it for sentinel_hip_flash_bwd, else for sentinel_hip_flash_fwd.
 */
SENTINEL_HIP_API size_t sentinel_hip_flash_workspace_bytes(int io_dtype, int compute_dtype, int layout, int q_heads, int kv_heads,
                                          int head_dim, int seq_len, int pack_count, int backward);

/*
 * out = softmax(scale * Q K^T [+ causal mask]) V and lse = max + ln(sum exp) per query, natural log of
 * the scaled scores (CudaFlashAttention.cu:1260-1264). Replaces CudaFlashAttention::forwardMultiHead.
 * `scale` must be positive and finite (the caller passes 1/sqrt(head_dim), CudaCausalSelfAttention.cu:212).
 * `stream` is a hipStream_t (NULL = default stream).
 */
SENTINEL_HIP_API int sentinel_hip_flash_fwd(const void* q, const void* k, const void* v, void* out, float* lse, int io_dtype,
                           int compute_dtype, int layout, int q_heads, int kv_heads, int head_dim, int stride_columns,
                           int column_start, int seq_len, int pack_count, float scale, int causal, void* workspace,
                           size_t workspace_bytes, void* stream);

/*
 * dq, dk, dv from d_out with P recomputed from lse and D = rowsum(d_out * out) written to `delta`.
 * Replaces CudaFlashAttention::backwardMultiHead (which launches the Delta kernel and one backward
 * kernel, CudaFlashAttention.cu:1640-1699).
 */
SENTINEL_HIP_API int sentinel_hip_flash_bwd(const void* q, const void* k, const void* v, const void* out, const float* lse,
                           const void* d_out, void* dq, void* dk, void* dv, float* delta, int io_dtype,
                           int compute_dtype, int layout, int q_heads, int kv_heads, int head_dim, int stride_columns,
                           int column_start, int seq_len, int pack_count, float scale, int causal, void* workspace,
                           size_t workspace_bytes, void* stream);

/*
 * Rotary position embedding: the step on either side of the attention core.
 *
 * Tables are fp32 [table_positions][head_dim / 2] in device memory, row = position, as the caller keeps them
 * in CudaCausalSelfAttention::cosTable / sinTable (built by RotaryEmbedding, Layers/RotaryEmbedding.cpp:8-29).
 *
 * sentinel_hip_rope_rotate rotates the (even, odd) row pairs of every head of an fp32 column-layout matrix in
 * place. Column c of the `columns` columns from column_start uses table position
 *      segment_length > 0 ? c % segment_length : position_offset + c.
 * Replaces CudaOps::rotaryRotateInPlace (inverse = 0) and CudaOps::rotaryRotateInverseInPlace (inverse != 0)
 * (Cuda/CudaOps.cu:362-402, host side :1318-1360), with their argument checks. The arithmetic is plain fp32
 * multiply / add (no fused multiply-add), so results are bit-identical to the host RotaryEmbedding.
 */
SENTINEL_HIP_API int sentinel_hip_rope_rotate(float* tensor, int heads, int head_dim, int stride_columns, int column_start,
                             int columns, int position_offset, int segment_length, const float* cos_table,
                             const float* sin_table, int table_positions, int inverse, void* stream);

/*
 * destination[i] = source[i] rounded to nearest even in `dtype` (SENTINEL_HIP_BF16 or SENTINEL_HIP_F16), for
 * element_count fp32 values in device memory; fp16 values beyond its range become infinities. The operand cast of the
 * layer's mixed-precision projection GEMMs: replaces CudaAmp::castFloatBufferToHalf (Cuda/CudaAmp.hpp:83,
 * Cuda/CudaAmp.cu:467-473, :523-527), which CudaMatrix::multiplyInto runs on both operands when
 * CudaAmp::preferMixedPrecision is set (Cuda/CudaMatmul.cu:413, Cuda/CudaAmp.cu:892-918). source must be 4-byte and
 * destination 2-byte aligned (16-byte aligned buffers take the wide path); element_count 0 is a no-op.
 */
SENTINEL_HIP_API int sentinel_hip_cast_to_16bit(const float* source, void* destination, size_t element_count, int dtype,
                               void* stream);

/*
 * sentinel_hip_flash_fwd / _bwd on UNROTATED q and k: token t of every pack is rotated with table row
 * position_offset + t on the way into the kernels, and dq, dk come back rotated back (gradients with respect
 * to the unrotated tensors). One call replaces the sequence the CUDA layer runs around the attention core:
 * rotaryRotateInPlace(query), rotaryRotateInPlace(key) (Cuda/CudaCausalSelfAttention.cu:206-207), forwardMultiHead
 * / backwardMultiHead, rotaryRotateInverseInPlace(queryGradient), (keyGradient) (:508-509), with
 * segmentLength = seq_len. The rotation rides on the layout conversion, so these exist for the configuration
 * that has one (COLUMNS layout, fp32 tensors, 16-bit arithmetic); anything else returns
 * SENTINEL_HIP_UNSUPPORTED and the caller rotates with sentinel_hip_rope_rotate. Workspace as for the plain calls.
 */
SENTINEL_HIP_API int sentinel_hip_flash_fwd_rope(const void* q, const void* k, const void* v, void* out, float* lse,
                                const float* cos_table, const float* sin_table, int table_positions, int position_offset,
                                int io_dtype, int compute_dtype, int layout, int q_heads, int kv_heads, int head_dim,
                                int stride_columns, int column_start, int seq_len, int pack_count, float scale, int causal,
                                void* workspace, size_t workspace_bytes, void* stream);
SENTINEL_HIP_API int sentinel_hip_flash_bwd_rope(const void* q, const void* k, const void* v, const void* out, const float* lse,
                                const void* d_out, void* dq, void* dk, void* dv, float* delta, const float* cos_table,
                                const float* sin_table, int table_positions, int position_offset, int io_dtype,
                                int compute_dtype, int layout, int q_heads, int kv_heads, int head_dim, int stride_columns,
                                int column_start, int seq_len, int pack_count, float scale, int causal, void* workspace,
                                size_t workspace_bytes, void* stream);

/*
 * The same with Sentinel's sparse attention mask on top of the causal one: a key is visible to a query iff
 *   key <= query and (key < global_token_count or window_size <= 0 or key >= query - window_size + 1)
 * (CausalSelfAttention::allowsKey, sentinel/NeuralNet/Layers/CausalSelfAttention.cpp:95-100; on the device
 * CudaOps::applySparseAttentionMaskInPlace and zeroForbiddenScoreGradientsInPlace, Cuda/CudaOps.cu:1262-1275). The
 * CUDA layer turns flash attention off for such layers (canUseFlashAttention, Cuda/CudaCausalSelfAttention.cu:46-57)
 * and materialises T x T scores per head (:255-314); here the kernels skip the key tiles no query of a tile can
 * see, so the work is O(T * window) instead of O(T^2). window_size <= 0 or >= seq_len is the plain causal mask (the
 * global tokens then change nothing). causal must be 1 with a window. cos_table / sin_table may both be NULL (no
 * rotation); otherwise as sentinel_hip_flash_fwd_rope. Workspace as for the plain calls.
 */
SENTINEL_HIP_API int sentinel_hip_flash_fwd_sparse(const void* q, const void* k, const void* v, void* out, float* lse,
                                  const float* cos_table, const float* sin_table, int table_positions,
                                  int position_offset, int window_size, int global_token_count, int io_dtype,
                                  int compute_dtype, int layout, int q_heads, int kv_heads, int head_dim,
                                  int stride_columns, int column_start, int seq_len, int pack_count, float scale,
                                  int causal, void* workspace, size_t workspace_bytes, void* stream);
SENTINEL_HIP_API int sentinel_hip_flash_bwd_sparse(const void* q, const void* k, const void* v, const void* out, const float* lse,
                                  const void* d_out, void* dq, void* dk, void* dv, float* delta,
                                  const float* cos_table, const float* sin_table, int table_positions,
                                  int position_offset, int window_size, int global_token_count, int io_dtype,
                                  int compute_dtype, int layout, int q_heads, int kv_heads, int head_dim,
                                  int stride_columns, int column_start, int seq_len, int pack_count, float scale,
                                  int causal, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Generation step: attention of ONE query position (the newest token, rows q_heads*head_dim of `query`, already
 * rotated) against the first `length` positions of an append-only K/V cache in Sentinel's layout: fp32
 * [(kv_head*head_dim + dim), position] with cache_stride positions per row (CudaKvCache::key / ::value,
 * Cuda/CudaKvCache.hpp:9-29; the new token's K/V are appended before the call, so length includes it).
 * out = q_heads*head_dim floats, the attended vector before the output projection.
 * Replaces the per-head loop of CudaCausalSelfAttention::attendCachedQuery
 * (Cuda/CudaCausalSelfAttention.cu:318-341; extractHead x3, GEMM, scale, mask, softmax, GEMM, writeHead per head)
 * with two launches that read the cache once; grouped-query heads share the reads. window_size /
 * global_token_count are the layer's sparse-mask parameters (applySparseAttentionMaskInPlace with
 * queryPositionStart = length - 1, :333): the query sees positions below global_token_count and the last
 * window_size positions, and only those parts of the cache are read; window_size <= 0 or >= length sees all.
 * Workspace: sentinel_hip_decode_workspace_bytes.
 */
SENTINEL_HIP_API size_t sentinel_hip_decode_workspace_bytes(int q_heads, int head_dim, int length);
SENTINEL_HIP_API int sentinel_hip_decode_attention(const float* query, const float* key_cache, const float* value_cache, float* out,
                                  int q_heads, int kv_heads, int head_dim, int cache_stride, int length, float scale,
                                  int window_size, int global_token_count, void* workspace, size_t workspace_bytes,
                                  void* stream);

/*
 * sentinel_hip_decode_attention without a workspace argument and without any allocation. It has no counterpart in
 * the reference; it is for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc. The partial results live in a device array that is part of the library
 * (SENTINEL_HIP_DECODE_STATIC_SCRATCH_BYTES per GPU, held until the process ends); a call whose
 * sentinel_hip_decode_workspace_bytes(q_heads, head_dim, length) exceeds it returns SENTINEL_HIP_INVALID_ARGUMENT.
 * Arguments, results and kernels are those of sentinel_hip_decode_attention. All calls on one GPU share that GPU's
 * array: calls that overlap in time on one GPU (different streams, threads) race; calls on one stream do not. The
 * first call on a device looks the array's address up (no allocation, no synchronisation); make it before capture.
 */
#define SENTINEL_HIP_DECODE_STATIC_SCRATCH_BYTES ((size_t)4 << 20)
SENTINEL_HIP_API int sentinel_hip_decode_attention_static(const float* query, const float* key_cache, const float* value_cache,
                                         float* out, int q_heads, int kv_heads, int head_dim, int cache_stride, int length,
                                         float scale, int window_size, int global_token_count, void* stream);

/*
 * Dense (materialising) attention path of the layer: the scores of one (head, pack) are a keys x queries fp32 matrix,
 * element (key, query) at base[key * query_count + query]; matrix b of a batch starts b * batch_stride elements on.
 *
 * sentinel_hip_dense_softmax_fwd, in place: P = softmax over keys of scale * S with forbidden pairs set to -1e9 first.
 * Replaces the per-head sequence CudaOps::scaleInPlace, applySparseAttentionMaskInPlace, softmaxInto
 * (Cuda/CudaCausalSelfAttention.cu:272-275; device bodies Cuda/CudaOps.cu:249-309) for a whole batch of heads with one
 * launch. A pair is allowed when key <= query and (key < global_token_count or window_size <= 0 or
 * key >= query - window_size + 1), positions being key and query_position_start + query, or, with segment_length > 0,
 * key % segment_length and query % segment_length of the same segment (CudaOps.cu:257-283).
 *
 * sentinel_hip_dense_softmax_bwd, in place over probability_gradient: dS = scale * P * (dP - sum over keys of dP * P),
 * zero on forbidden pairs. Replaces CudaOps::softmaxBackwardInto, zeroForbiddenScoreGradientsInPlace, scaleInPlace
 * (Cuda/CudaCausalSelfAttention.cu:455-457; Cuda/CudaOps.cu:311-344).
 */
SENTINEL_HIP_API int sentinel_hip_dense_softmax_fwd(float* scores, int batch, long long batch_stride, int key_count,
                                                    int query_count, int query_position_start, int window_size,
                                                    int global_token_count, int segment_length, float scale, void* stream);
SENTINEL_HIP_API int sentinel_hip_dense_softmax_bwd(const float* probabilities, long long probability_batch_stride,
                                                    float* probability_gradient, long long gradient_batch_stride, int batch,
                                                    int key_count, int query_count, int query_position_start, int window_size,
                                                    int global_token_count, int segment_length, float scale, void* stream);

/* Largest head_dim any kernel here accepts (the CUDA path's CudaFlashAttention::maxHeadDimension is 64). */
SENTINEL_HIP_API int sentinel_hip_flash_max_head_dim(void);

/* 1 when a HIP device is usable (stands for CudaMatmul::isAvailable, CudaFlashAttention.cu:1545). */
SENTINEL_HIP_API int sentinel_hip_device_available(void);

/* Fixed text for a return code. */
SENTINEL_HIP_API const char* sentinel_hip_strerror(int code);

/* Detail of the last non-OK return on the calling thread ("" if none). */
SENTINEL_HIP_API const char* sentinel_hip_last_error(void);

/*
 * Optional per-kernel timing (diagnostics). Stands for the cudaEvent phase breakdown of
 * CudaLanguageModel::runTrainProfileDemo (sentinel/NeuralNet/Cuda/CudaLanguageModel.cu:4203-4211, :4378).
 * While enabled, every kernel launched by the entry points above is bracketed by two hipEvents on its
 * stream (so such calls must not be captured into a graph). sentinel_hip_flash_collect_timings waits for
 * the recorded events, adds the durations up per kernel name since the previous collect, writes at most
 * `capacity` entries (names are static strings) and returns the number written.
 */
SENTINEL_HIP_API int sentinel_hip_flash_set_timing(int enabled); /* returns the previous setting */
SENTINEL_HIP_API int sentinel_hip_flash_collect_timings(const char** names_out, float* total_ms_out, int* launches_out,
                                                        int capacity);

#ifdef __cplusplus
}
#endif
#endif /* SENTINEL_HIP_ATTN_H */
