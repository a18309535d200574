/*
 * TEST INFRASTRUCTURE ONLY - CPU oracle for Sentinel's causal attention.
 *
 * This is a plain C++ restatement of the host (OpenMP) attention path of
 * ToldByNun/sentinel, used to check the HIP kernels and as the CPU baseline
 * in bench.py.  Nothing in the shipped library links, loads or calls it.
 *
 * Tensors use Sentinel's device layout (Cuda/CudaFlashAttention.cu:129-135):
 *   element(head, dim, column) = base[(head * headDim + dim) * strideColumns + column]
 * with packCount sequences of seqLen columns starting at colStart.  q / d_out /
 * out / dq have qHeads heads, k / v / dk / dv have kvHeads heads, lse is
 * qHeads x strideColumns.
 */
#ifndef SENTINEL_ATTENTION_ORACLE_H
#define SENTINEL_ATTENTION_ORACLE_H

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Forward (and backward when d_out != NULL) of causal multi-head attention.
 *
 *  out, lse            forward results (lse may be NULL); columns outside the
 *                      pack window are left untouched
 *  d_out, dq, dk, dv   backward: all four non-NULL or all four NULL; dk / dv
 *                      are OVERWRITTEN inside the pack window (zero, then the
 *                      group's query heads are added in increasing order)
 *  causal              1 = Sentinel's mask (key > query forbidden); 0 = no mask
 *                      (the CPU reference has no such mode; kept for the device
 *                      API's `causal` flag)
 *  packParallel        1 = OpenMP over packs with serial inner loops (mirrors
 *                      the train loop, Network/LanguageModel.cpp:1109-1125);
 *                      0 = packs in order, gemm / softmax internally parallel
 *                      under the reference's own thresholds
 *
 * Returns 0, or -1 on invalid geometry.
 */
int sentinel_oracle_attention(const float* q, const float* k, const float* v,
                              float* out, float* lse,
                              const float* d_out, float* dq, float* dk, float* dv,
                              int qHeads, int kvHeads, int headDim,
                              int strideColumns, int colStart, int seqLen, int packCount,
                              float scale, int causal, int packParallel);

/*
 * The same with Sentinel's sparse mask on top of the causal one (CausalSelfAttention::allowsKey,
 * Layers/CausalSelfAttention.cpp:95-100): key <= query and (key < globalTokenCount or windowSize <= 0 or
 * key >= query - windowSize + 1).  Restates the dense masked path (applyAttentionMaskInPlace :109-120, score
 * gradients zeroed :338-343); the reference's sparse-compute path (:128-168, :296-330) skips the forbidden pairs
 * instead and agrees up to summation order.  windowSize = 0, globalTokenCount = 0 is sentinel_oracle_attention.
 * Pinned bit-exactly against the reference's compiled layer with preferSparseCompute = false, to rounding with
 * preferSparseCompute = true, and against a float64 masked softmax (tests/test_oracle_sparse.py).
 * Returns -1 for a window / global tokens without the causal flag.
 */
int sentinel_oracle_attention_sparse(const float* q, const float* k, const float* v,
                                     float* out, float* lse,
                                     const float* d_out, float* dq, float* dk, float* dv,
                                     int qHeads, int kvHeads, int headDim,
                                     int strideColumns, int colStart, int seqLen, int packCount,
                                     float scale, int causal, int packParallel,
                                     int windowSize, int globalTokenCount);

/* D[head][column] = sum_dim out * d_out (Cuda/CudaFlashAttention.cu:576-596). */
int sentinel_oracle_delta(const float* out, const float* d_out, float* delta,
                          int qHeads, int headDim, int strideColumns, int colStart,
                          int seqLen, int packCount);

/* C = op(A) * op(B) with the reference's blocking and summation order
 * (Math/Matrix.cpp:106-148); exported so tests can pin it on its own. */
int sentinel_oracle_gemm(const float* a, int aRows, int aCols, const float* b, int bRows, int bCols,
                         float* c, int transposeA, int transposeB);

/* column softmax (Activations/Softmax.cpp:10-44); rows x cols, row-major */
int sentinel_oracle_softmax_columns(const float* logits, float* out, int rows, int cols);

/*
 * Rotary position embedding, the step on either side of the attention core.
 *
 * sentinel_oracle_rope_tables: cos / sin tables [positions][headDim / 2] exactly as the
 * reference builds them (Layers/RotaryEmbedding.cpp:8-29: float pow, cos, sin).
 * sentinel_oracle_rope_rotate: rotates the (even, odd) row pairs of every head in place
 * (Layers/RotaryEmbedding.cpp:39-59; inverse :61-81).  Column c of the `columns` columns
 * starting at colStart uses table position  segmentLength > 0 ? c % segmentLength :
 * positionOffset + c  (the device rule, Cuda/CudaOps.cu:362-402; the host layer is the
 * case positionOffset = 0, segmentLength = 0).  Returns -1 on invalid geometry or a
 * position past the table (Cuda/CudaOps.cu:1319-1330).
 * Pinned bit-exactly against the reference's compiled RotaryEmbedding (tests/golden,
 * tests/test_oracle_rope.py) and by rotation invariants.
 */
int sentinel_oracle_rope_tables(int headDim, int positions, float base, float* cosTable, float* sinTable);
int sentinel_oracle_rope_rotate(float* tensor, int heads, int headDim, int strideColumns, int colStart, int columns,
                                int positionOffset, int segmentLength, const float* cosTable, const float* sinTable,
                                int tablePositions, int inverse);

/*
 * The whole attention layer around the core, one sequence (embeddingDim x seqLen, row-major):
 *   Q = Wq X, K = Wk X, V = Wv X; RoPE on Q and K; causal attention (scale 1/sqrt(headDim));
 *   Y = Wo A                                              (Layers/CausalSelfAttention.cpp:212-264)
 * and, when d_y != NULL, its backward                     (Layers/CausalSelfAttention.cpp:266-368):
 *   dWo = dY A^T, dA = Wo^T dY, core backward, inverse RoPE on dQ, dK,
 *   dWq = dQ X^T, dWk = dK X^T, dWv = dV X^T, dX = Wq^T dQ + Wk^T dK + Wv^T dV.
 * wq: (qHeads*headDim) x E, wk / wv: (kvHeads*headDim) x E, wo: E x (qHeads*headDim); gradients have the
 * shapes of what they differentiate. Composed from the functions above, so it inherits their pins; the
 * composition itself is pinned bit-exactly against the reference's compiled layer (tests/golden/layer_kat.npz,
 * tests/test_oracle_layer.py) and by finite differences.
 * Returns 0, -1 on invalid geometry.
 */
int sentinel_oracle_layer(const float* x, const float* wq, const float* wk, const float* wv, const float* wo,
                          const float* d_y, float* y, float* d_x, float* d_wq, float* d_wk, float* d_wv, float* d_wo,
                          int embeddingDim, int qHeads, int kvHeads, int headDim, int seqLen, float ropeBase,
                          int ropePositions);

/* the layer with the sparse mask of sentinel_oracle_attention_sparse (the host layer's windowSize / globalTokenCount) */
int sentinel_oracle_layer_sparse(const float* x, const float* wq, const float* wk, const float* wv, const float* wo,
                                 const float* d_y, float* y, float* d_x, float* d_wq, float* d_wk, float* d_wv, float* d_wo,
                                 int embeddingDim, int qHeads, int kvHeads, int headDim, int seqLen, float ropeBase,
                                 int ropePositions, int windowSize, int globalTokenCount);

int sentinel_oracle_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
