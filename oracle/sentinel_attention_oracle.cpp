/*
 * TEST INFRASTRUCTURE ONLY - CPU oracle for Sentinel's causal attention.
 *
 * Restates, in plain C++ on raw arrays, the arithmetic of the reference's host
 * attention path so that fp32 results carry the reference's own summation
 * order.  The shipped library never links or calls this file; only tests/,
 * __graft_entry__.smoke() and bench.py's cpu_baseline leg may use it.
 *
 * Reference sources followed (paths relative to the reference checkout):
 *   sentinel/NeuralNet/Math/Matrix.cpp:11-72,106-148      blocked gemm, transposed packing, OpenMP rule
 *   sentinel/NeuralNet/Activations/Softmax.cpp:10-44       column softmax
 *   sentinel/NeuralNet/Layers/CausalSelfAttention.cpp:90-100   GQA head map, mask rule
 *   sentinel/NeuralNet/Layers/CausalSelfAttention.cpp:122-126  scores = K^T Q, scale, mask
 *   sentinel/NeuralNet/Layers/CausalSelfAttention.cpp:150-152  attended = V P
 *   sentinel/NeuralNet/Layers/CausalSelfAttention.cpp:195-210  softmax backward
 *   sentinel/NeuralNet/Layers/CausalSelfAttention.cpp:232-254  per-head forward
 *   sentinel/NeuralNet/Layers/CausalSelfAttention.cpp:279-353  per-head backward (dense branch)
 *   sentinel/NeuralNet/Cuda/CudaFlashAttention.cu:1260-1264    LSE = max + ln(sum)
 *   sentinel/NeuralNet/Cuda/CudaFlashAttention.cu:576-596      D = rowsum(O * dO)
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   gemm, softmax, forward, backward : bit-compared with the reference's own
 *       compiled CPU sources (oracle/_ref) on committed fixtures, and checked
 *       against float64 brute force, closed forms (Q = 0, constant V, first
 *       query) and central finite differences.
 *   lse, delta : no CPU counterpart in the reference (device-only quantities);
 *       pinned by their definitions in float64 and by closed forms.
 *   causal = 0 : device-API flag with no CPU counterpart; pinned by float64
 *       brute force only.
 *
 * Heads are processed one at a time (forward immediately followed by that
 * head's backward) instead of caching every head's T x T probabilities as the
 * reference layer does; heads are independent, and grouped K/V gradients are
 * still added in increasing query-head order, so results are identical while
 * memory stays at a few T x T matrices.
 */
#include "sentinel_attention_oracle.h"

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstring>
#include <vector>

#if defined(_OPENMP)
#include <omp.h>
#endif

namespace {

constexpr size_t kBlock = 32;  // Matrix.cpp:11

bool insideParallelRegion() {
#if defined(_OPENMP)
    return omp_in_parallel() != 0;
#else
    return true;
#endif
}

// One 32-row band of C += A * B, i-k-j inside 32^3 blocks (Matrix.cpp:24-43).
void gemmRowBand(const float* a, size_t lda, const float* b, size_t ldb, float* c, size_t ldc,
                 size_t rowLo, size_t rowHi, size_t n, size_t kTotal) {
    for (size_t colLo = 0; colLo < n; colLo += kBlock) {
        const size_t colHi = std::min(colLo + kBlock, n);
        for (size_t kLo = 0; kLo < kTotal; kLo += kBlock) {
            const size_t kHi = std::min(kLo + kBlock, kTotal);
            for (size_t i = rowLo; i < rowHi; ++i) {
                float* cRow = c + i * ldc;
                for (size_t kk = kLo; kk < kHi; ++kk) {
                    const float aik = a[i * lda + kk];
                    const float* bRow = b + kk * ldb;
                    for (size_t j = colLo; j < colHi; ++j) cRow[j] += aik * bRow[j];
                }
            }
        }
    }
}

// dst (outRows x outCols) = src^T, src is outCols x outRows (Matrix.cpp:14-22)
void packTranspose(const float* src, size_t srcCols, size_t outRows, size_t outCols, std::vector<float>& dst) {
    dst.resize(outRows * outCols);
    for (size_t r = 0; r < outRows; ++r)
        for (size_t c = 0; c < outCols; ++c) dst[r * outCols + c] = src[c * srcCols + r];
}

struct Scratch {
    std::vector<float> packA, packB;
    std::vector<float> qHead, kHead, vHead, oHead, gHead;  // d x T each
    std::vector<float> scores, probs, dProbs, dScores;     // T x T each, [key][query]
    std::vector<float> dqHead, dkHead, dvHead;
};

// C = op(A) op(B); zero-fill then accumulate (Matrix.cpp:106-148).
void gemm(const float* a, size_t aRows, size_t aCols, const float* b, size_t bRows, size_t bCols, float* c,
          bool transA, bool transB, Scratch& scratch) {
    const size_t m = transA ? aCols : aRows;
    const size_t kTotal = transA ? aRows : aCols;
    const size_t n = transB ? bRows : bCols;
    std::fill(c, c + m * n, 0.0f);

    const float* ap = a;
    size_t lda = aCols;
    if (transA) {
        packTranspose(a, aCols, m, kTotal, scratch.packA);
        ap = scratch.packA.data();
        lda = kTotal;
    }
    const float* bp = b;
    size_t ldb = bCols;
    if (transB) {
        packTranspose(b, bCols, kTotal, n, scratch.packB);
        bp = scratch.packB.data();
        ldb = n;
    }

    const size_t work = m * kTotal * n;
    const long bandCount = static_cast<long>((m + kBlock - 1) / kBlock);
    if (work >= 65536 && !insideParallelRegion()) {  // Matrix.cpp:139-146
#if defined(_OPENMP)
#pragma omp parallel for schedule(static)
#endif
        for (long band = 0; band < bandCount; ++band) {
            const size_t lo = static_cast<size_t>(band) * kBlock;
            gemmRowBand(ap, lda, bp, ldb, c, n, lo, std::min(lo + kBlock, m), n, kTotal);
        }
        return;
    }
    for (long band = 0; band < bandCount; ++band) {
        const size_t lo = static_cast<size_t>(band) * kBlock;
        gemmRowBand(ap, lda, bp, ldb, c, n, lo, std::min(lo + kBlock, m), n, kTotal);
    }
}

// Softmax over rows (classes) for every column (Softmax.cpp:10-44).
void softmaxColumns(const float* logits, float* out, size_t rows, size_t cols) {
    const bool parallel = cols >= 32 && !insideParallelRegion();
    (void)parallel;
#if defined(_OPENMP)
#pragma omp parallel for schedule(static) if (parallel)
#endif
    for (long col = 0; col < static_cast<long>(cols); ++col) {
        float top = logits[col];
        for (size_t r = 1; r < rows; ++r)
            if (logits[r * cols + col] > top) top = logits[r * cols + col];
        float total = 0.0f;
        for (size_t r = 0; r < rows; ++r) {
            const float e = std::exp(logits[r * cols + col] - top);
            out[r * cols + col] = e;
            total += e;
        }
        for (size_t r = 0; r < rows; ++r) out[r * cols + col] /= total;
    }
}

void gatherHead(const float* base, int head, int d, size_t stride, size_t col0, size_t t, std::vector<float>& dst) {
    dst.resize(static_cast<size_t>(d) * t);
    for (int r = 0; r < d; ++r)
        std::memcpy(dst.data() + static_cast<size_t>(r) * t,
                    base + (static_cast<size_t>(head) * d + r) * stride + col0, t * sizeof(float));
}

void scatterHead(float* base, int head, int d, size_t stride, size_t col0, size_t t, const float* src, bool add) {
    for (int r = 0; r < d; ++r) {
        float* row = base + (static_cast<size_t>(head) * d + r) * stride + col0;
        const float* s = src + static_cast<size_t>(r) * t;
        if (add)
            for (size_t c = 0; c < t; ++c) row[c] += s[c];
        else
            std::memcpy(row, s, t * sizeof(float));
    }
}

struct Geometry {
    int qHeads, kvHeads, d;
    size_t stride, t;
    float scale;
    bool causal;
    int window = 0;        // sliding window (<= 0: none)
    int globalTokens = 0;  // keys before this index are visible to every later query
};

// CausalSelfAttention::allowsKey (Layers/CausalSelfAttention.cpp:95-100)
bool allowsKey(long long query, long long key, int window, int globalTokens) {
    if (key > query) return false;
    if (key < globalTokens) return true;
    if (window <= 0) return true;
    return key >= query - window + 1;
}

void onePack(const Geometry& g, size_t col0, const float* q, const float* k, const float* v, float* out, float* lse,
             const float* dOut, float* dq, float* dk, float* dv, Scratch& s) {
    const size_t t = g.t;
    const int d = g.d;
    const int group = g.qHeads / g.kvHeads;  // CausalSelfAttention.cpp:90-93
    s.scores.resize(t * t);
    s.probs.resize(t * t);
    s.oHead.resize(static_cast<size_t>(d) * t);

    if (dOut) {
        // keyGradient / valueGradient start from zero (CausalSelfAttention.cpp:271-276)
        for (int h = 0; h < g.kvHeads; ++h)
            for (int r = 0; r < d; ++r) {
                const size_t off = (static_cast<size_t>(h) * d + r) * g.stride + col0;
                std::fill(dk + off, dk + off + t, 0.0f);
                std::fill(dv + off, dv + off + t, 0.0f);
            }
        s.dProbs.resize(t * t);
        s.dScores.resize(t * t);
        s.dqHead.resize(static_cast<size_t>(d) * t);
        s.dkHead.resize(static_cast<size_t>(d) * t);
        s.dvHead.resize(static_cast<size_t>(d) * t);
    }

    for (int h = 0; h < g.qHeads; ++h) {
        const int kvHead = h / group;
        gatherHead(q, h, d, g.stride, col0, t, s.qHead);
        gatherHead(k, kvHead, d, g.stride, col0, t, s.kHead);
        gatherHead(v, kvHead, d, g.stride, col0, t, s.vHead);

        // scores[key][query] = scale * sum_dim K[dim][key] Q[dim][query], then mask (CausalSelfAttention.cpp:122-126)
        gemm(s.kHead.data(), d, t, s.qHead.data(), d, t, s.scores.data(), true, false, s);
        for (size_t i = 0; i < t * t; ++i) s.scores[i] *= g.scale;
        // applyAttentionMaskInPlace (CausalSelfAttention.cpp:109-120): the dense masked path, which the reference's
        // sparse-compute path (:128-168) reproduces up to summation order
        if (g.causal)
            for (size_t key = 0; key < t; ++key)
                for (size_t query = 0; query < t; ++query)
                    if (!allowsKey(static_cast<long long>(query), static_cast<long long>(key), g.window, g.globalTokens))
                        s.scores[key * t + query] = -1e9f;

        softmaxColumns(s.scores.data(), s.probs.data(), t, t);

        // attended = V P (CausalSelfAttention.cpp:150-152)
        gemm(s.vHead.data(), d, t, s.probs.data(), t, t, s.oHead.data(), false, false, s);
        scatterHead(out, h, d, g.stride, col0, t, s.oHead.data(), false);

        if (lse) {
            // natural-log LSE of the scaled, masked scores, accumulated in double
            for (size_t query = 0; query < t; ++query) {
                float top = s.scores[query];
                for (size_t key = 1; key < t; ++key) top = std::max(top, s.scores[key * t + query]);
                double total = 0.0;
                for (size_t key = 0; key < t; ++key)
                    total += std::exp(static_cast<double>(s.scores[key * t + query]) - static_cast<double>(top));
                lse[static_cast<size_t>(h) * g.stride + col0 + query] = static_cast<float>(top + std::log(total));
            }
        }

        if (!dOut) continue;

        gatherHead(dOut, h, d, g.stride, col0, t, s.gHead);
        // dV = dA P^T ; dP = V^T dA (CausalSelfAttention.cpp:334-335)
        gemm(s.gHead.data(), d, t, s.probs.data(), t, t, s.dvHead.data(), false, true, s);
        gemm(s.vHead.data(), d, t, s.gHead.data(), d, t, s.dProbs.data(), true, false, s);
        // softmax jacobian per query column (CausalSelfAttention.cpp:195-210)
        for (size_t query = 0; query < t; ++query) {
            float dot = 0.0f;
            for (size_t key = 0; key < t; ++key) dot += s.dProbs[key * t + query] * s.probs[key * t + query];
            for (size_t key = 0; key < t; ++key)
                s.dScores[key * t + query] = s.probs[key * t + query] * (s.dProbs[key * t + query] - dot);
        }
        if (g.causal)  // CausalSelfAttention.cpp:338-343
            for (size_t key = 0; key < t; ++key)
                for (size_t query = 0; query < t; ++query)
                    if (!allowsKey(static_cast<long long>(query), static_cast<long long>(key), g.window, g.globalTokens))
                        s.dScores[key * t + query] = 0.0f;
        for (size_t i = 0; i < t * t; ++i) s.dScores[i] *= g.scale;
        // dQ = K dS ; dK = Q dS^T (CausalSelfAttention.cpp:346-347)
        gemm(s.kHead.data(), d, t, s.dScores.data(), t, t, s.dqHead.data(), false, false, s);
        gemm(s.qHead.data(), d, t, s.dScores.data(), t, t, s.dkHead.data(), false, true, s);

        scatterHead(dq, h, d, g.stride, col0, t, s.dqHead.data(), false);
        scatterHead(dk, kvHead, d, g.stride, col0, t, s.dkHead.data(), true);
        scatterHead(dv, kvHead, d, g.stride, col0, t, s.dvHead.data(), true);
    }
}

}  // namespace

extern "C" int sentinel_oracle_attention_sparse(const float* q, const float* k, const float* v, float* out, float* lse,
                                                const float* d_out, float* dq, float* dk, float* dv, int qHeads,
                                                int kvHeads, int headDim, int strideColumns, int colStart, int seqLen,
                                                int packCount, float scale, int causal, int packParallel, int windowSize,
                                                int globalTokenCount) {
    if (!q || !k || !v || !out) return -1;
    if (qHeads <= 0 || kvHeads <= 0 || headDim <= 0 || qHeads % kvHeads != 0) return -1;
    if (seqLen <= 0 || packCount <= 0 || colStart < 0) return -1;
    if (static_cast<long long>(colStart) + static_cast<long long>(packCount) * seqLen > strideColumns) return -1;
    const bool wantBackward = d_out != nullptr;
    if (wantBackward != (dq != nullptr) || wantBackward != (dk != nullptr) || wantBackward != (dv != nullptr)) return -1;

    if (globalTokenCount < 0) return -1;
    if (!causal && (windowSize > 0 || globalTokenCount > 0)) return -1;  // the sparse mask refines the causal one
    Geometry g{qHeads, kvHeads, headDim, static_cast<size_t>(strideColumns), static_cast<size_t>(seqLen), scale, causal != 0,
               windowSize, globalTokenCount};

    if (packParallel && packCount > 1) {
#if defined(_OPENMP)
#pragma omp parallel
#endif
        {
            Scratch scratch;
#if defined(_OPENMP)
#pragma omp for schedule(dynamic, 1)
#endif
            for (int pack = 0; pack < packCount; ++pack)
                onePack(g, static_cast<size_t>(colStart) + static_cast<size_t>(pack) * g.t, q, k, v, out, lse, d_out, dq, dk,
                        dv, scratch);
        }
        return 0;
    }
    Scratch scratch;
    for (int pack = 0; pack < packCount; ++pack)
        onePack(g, static_cast<size_t>(colStart) + static_cast<size_t>(pack) * g.t, q, k, v, out, lse, d_out, dq, dk, dv,
                scratch);
    return 0;
}

extern "C" int sentinel_oracle_attention(const float* q, const float* k, const float* v, float* out, float* lse,
                                         const float* d_out, float* dq, float* dk, float* dv, int qHeads, int kvHeads,
                                         int headDim, int strideColumns, int colStart, int seqLen, int packCount,
                                         float scale, int causal, int packParallel) {
    return sentinel_oracle_attention_sparse(q, k, v, out, lse, d_out, dq, dk, dv, qHeads, kvHeads, headDim, strideColumns,
                                            colStart, seqLen, packCount, scale, causal, packParallel, 0, 0);
}

extern "C" int sentinel_oracle_delta(const float* out, const float* d_out, float* delta, int qHeads, int headDim,
                                     int strideColumns, int colStart, int seqLen, int packCount) {
    if (!out || !d_out || !delta || qHeads <= 0 || headDim <= 0 || seqLen <= 0 || packCount <= 0 || colStart < 0) return -1;
    if (static_cast<long long>(colStart) + static_cast<long long>(packCount) * seqLen > strideColumns) return -1;
    const size_t stride = static_cast<size_t>(strideColumns);
    for (int h = 0; h < qHeads; ++h)
        for (size_t col = static_cast<size_t>(colStart); col < static_cast<size_t>(colStart) + static_cast<size_t>(packCount) * seqLen; ++col) {
            float sum = 0.0f;  // CudaFlashAttention.cu:589-594: dims in increasing order, fp32
            for (int r = 0; r < headDim; ++r) {
                const size_t idx = (static_cast<size_t>(h) * headDim + r) * stride + col;
                sum += out[idx] * d_out[idx];
            }
            delta[static_cast<size_t>(h) * stride + col] = sum;
        }
    return 0;
}

extern "C" int sentinel_oracle_gemm(const float* a, int aRows, int aCols, const float* b, int bRows, int bCols, float* c,
                                    int transposeA, int transposeB) {
    if (!a || !b || !c || aRows <= 0 || aCols <= 0 || bRows <= 0 || bCols <= 0) return -1;
    const int inner = transposeA ? aRows : aCols;
    const int innerB = transposeB ? bCols : bRows;
    if (inner != innerB) return -1;
    Scratch scratch;
    gemm(a, aRows, aCols, b, bRows, bCols, c, transposeA != 0, transposeB != 0, scratch);
    return 0;
}

extern "C" int sentinel_oracle_softmax_columns(const float* logits, float* out, int rows, int cols) {
    if (!logits || !out || rows <= 0 || cols <= 0) return -1;
    softmaxColumns(logits, out, static_cast<size_t>(rows), static_cast<size_t>(cols));
    return 0;
}

// Layers/RotaryEmbedding.cpp:8-29
extern "C" int sentinel_oracle_rope_tables(int headDim, int positions, float base, float* cosTable, float* sinTable) {
    if (headDim <= 0 || headDim % 2 != 0 || positions <= 0 || !(base > 0.0f) || !cosTable || !sinTable) return -1;
    const int pairCount = headDim / 2;
    for (int position = 0; position < positions; ++position) {
        for (int pairIndex = 0; pairIndex < pairCount; ++pairIndex) {
            const float exponent = -2.0f * static_cast<float>(pairIndex) / static_cast<float>(headDim);
            const float angle = static_cast<float>(position) * std::pow(base, exponent);
            const size_t tableIndex = static_cast<size_t>(position) * pairCount + pairIndex;
            cosTable[tableIndex] = std::cos(angle);
            sinTable[tableIndex] = std::sin(angle);
        }
    }
    return 0;
}

// Layers/RotaryEmbedding.cpp:39-81 with the device position rule of Cuda/CudaOps.cu:362-402
extern "C" int sentinel_oracle_rope_rotate(float* tensor, int heads, int headDim, int strideColumns, int colStart,
                                           int columns, int positionOffset, int segmentLength, const float* cosTable,
                                           const float* sinTable, int tablePositions, int inverse) {
    if (!tensor || !cosTable || !sinTable || heads <= 0 || headDim <= 0 || headDim % 2 != 0) return -1;
    if (columns < 0 || colStart < 0 || colStart + columns > strideColumns) return -1;
    if (positionOffset < 0 || segmentLength < 0) return -1;
    if (segmentLength > 0 ? segmentLength > tablePositions : positionOffset + columns > tablePositions) return -1;
    const int pairCount = headDim / 2;
    for (int headIndex = 0; headIndex < heads; ++headIndex) {
        const size_t rowOffset = static_cast<size_t>(headIndex) * headDim;
        for (int column = 0; column < columns; ++column) {
            const int position = segmentLength > 0 ? column % segmentLength : positionOffset + column;
            for (int pairIndex = 0; pairIndex < pairCount; ++pairIndex) {
                float* even = tensor + (rowOffset + 2 * pairIndex) * strideColumns + colStart + column;
                float* odd = even + strideColumns;
                const float cosValue = cosTable[static_cast<size_t>(position) * pairCount + pairIndex];
                const float sinValue = sinTable[static_cast<size_t>(position) * pairCount + pairIndex];
                const float evenValue = *even;
                const float oddValue = *odd;
                if (!inverse) {
                    *even = evenValue * cosValue - oddValue * sinValue;
                    *odd = evenValue * sinValue + oddValue * cosValue;
                } else {
                    *even = evenValue * cosValue + oddValue * sinValue;
                    *odd = -evenValue * sinValue + oddValue * cosValue;
                }
            }
        }
    }
    return 0;
}

// Layers/CausalSelfAttention.cpp:212-264 (forward) and :266-368 (backward); windowSize <= 0 and globalTokenCount 0
// give the full causal mask
extern "C" int sentinel_oracle_layer_sparse(const float* x, const float* wq, const float* wk, const float* wv,
                                            const float* wo, const float* d_y, float* y, float* d_x, float* d_wq,
                                            float* d_wk, float* d_wv, float* d_wo, int embeddingDim, int qHeads, int kvHeads,
                                            int headDim, int seqLen, float ropeBase, int ropePositions, int windowSize,
                                            int globalTokenCount) {
    if (!x || !wq || !wk || !wv || !wo || !y) return -1;
    if (embeddingDim <= 0 || qHeads <= 0 || kvHeads <= 0 || qHeads % kvHeads != 0 || headDim <= 0 || headDim % 2 != 0) return -1;
    if (seqLen <= 0 || seqLen > ropePositions) return -1;
    const bool wantBackward = d_y != nullptr;
    if (wantBackward && (!d_x || !d_wq || !d_wk || !d_wv || !d_wo)) return -1;
    const int e = embeddingDim, t = seqLen, qRows = qHeads * headDim, kvRows = kvHeads * headDim;
    std::vector<float> cosT(static_cast<size_t>(ropePositions) * headDim / 2), sinT(cosT.size());
    if (sentinel_oracle_rope_tables(headDim, ropePositions, ropeBase, cosT.data(), sinT.data()) != 0) return -1;

    std::vector<float> q(static_cast<size_t>(qRows) * t), k(static_cast<size_t>(kvRows) * t), v(k.size()), a(q.size());
    sentinel_oracle_gemm(wq, qRows, e, x, e, t, q.data(), 0, 0);
    sentinel_oracle_gemm(wk, kvRows, e, x, e, t, k.data(), 0, 0);
    sentinel_oracle_gemm(wv, kvRows, e, x, e, t, v.data(), 0, 0);
    sentinel_oracle_rope_rotate(q.data(), qHeads, headDim, t, 0, t, 0, 0, cosT.data(), sinT.data(), ropePositions, 0);
    sentinel_oracle_rope_rotate(k.data(), kvHeads, headDim, t, 0, t, 0, 0, cosT.data(), sinT.data(), ropePositions, 0);
    const float scale = 1.0f / std::sqrt(static_cast<float>(headDim));
    if (!wantBackward) {
        if (sentinel_oracle_attention_sparse(q.data(), k.data(), v.data(), a.data(), nullptr, nullptr, nullptr, nullptr, nullptr,
                                             qHeads, kvHeads, headDim, t, 0, t, 1, scale, 1, 0, windowSize, globalTokenCount) != 0)
            return -1;
        sentinel_oracle_gemm(wo, e, qRows, a.data(), qRows, t, y, 0, 0);
        return 0;
    }
    std::vector<float> dA(q.size()), dq(q.size()), dk(k.size()), dv(k.size()), temp(static_cast<size_t>(e) * t);
    // forward once for A (and Y), then the backward from dA = Wo^T dY
    if (sentinel_oracle_attention_sparse(q.data(), k.data(), v.data(), a.data(), nullptr, nullptr, nullptr, nullptr, nullptr,
                                         qHeads, kvHeads, headDim, t, 0, t, 1, scale, 1, 0, windowSize, globalTokenCount) != 0)
        return -1;
    sentinel_oracle_gemm(wo, e, qRows, a.data(), qRows, t, y, 0, 0);
    sentinel_oracle_gemm(d_y, e, t, a.data(), qRows, t, d_wo, 0, 1);
    sentinel_oracle_gemm(wo, e, qRows, d_y, e, t, dA.data(), 1, 0);
    if (sentinel_oracle_attention_sparse(q.data(), k.data(), v.data(), a.data(), nullptr, dA.data(), dq.data(), dk.data(),
                                         dv.data(), qHeads, kvHeads, headDim, t, 0, t, 1, scale, 1, 0, windowSize,
                                         globalTokenCount) != 0)
        return -1;
    sentinel_oracle_rope_rotate(dq.data(), qHeads, headDim, t, 0, t, 0, 0, cosT.data(), sinT.data(), ropePositions, 1);
    sentinel_oracle_rope_rotate(dk.data(), kvHeads, headDim, t, 0, t, 0, 0, cosT.data(), sinT.data(), ropePositions, 1);
    sentinel_oracle_gemm(dq.data(), qRows, t, x, e, t, d_wq, 0, 1);
    sentinel_oracle_gemm(dk.data(), kvRows, t, x, e, t, d_wk, 0, 1);
    sentinel_oracle_gemm(dv.data(), kvRows, t, x, e, t, d_wv, 0, 1);
    sentinel_oracle_gemm(wq, qRows, e, dq.data(), qRows, t, d_x, 1, 0);
    sentinel_oracle_gemm(wk, kvRows, e, dk.data(), kvRows, t, temp.data(), 1, 0);
    for (size_t i = 0; i < temp.size(); ++i) d_x[i] += temp[i];
    sentinel_oracle_gemm(wv, kvRows, e, dv.data(), kvRows, t, temp.data(), 1, 0);
    for (size_t i = 0; i < temp.size(); ++i) d_x[i] += temp[i];
    return 0;
}

extern "C" int sentinel_oracle_layer(const float* x, const float* wq, const float* wk, const float* wv, const float* wo,
                                     const float* d_y, float* y, float* d_x, float* d_wq, float* d_wk, float* d_wv,
                                     float* d_wo, int embeddingDim, int qHeads, int kvHeads, int headDim, int seqLen,
                                     float ropeBase, int ropePositions) {
    return sentinel_oracle_layer_sparse(x, wq, wk, wv, wo, d_y, y, d_x, d_wq, d_wk, d_wv, d_wo, embeddingDim, qHeads, kvHeads,
                                        headDim, seqLen, ropeBase, ropePositions, 0, 0);
}

extern "C" int sentinel_oracle_max_threads(void) {
#if defined(_OPENMP)
    return omp_get_max_threads();
#else
    return 1;
#endif
}
