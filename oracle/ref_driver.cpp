/*
 * TEST INFRASTRUCTURE ONLY - drives the reference's own compiled CPU attention.
 *
 * Built only where the reference checkout exists (see oracle/Makefile); it
 * includes the reference headers by path and links the reference's own
 * Matrix / Softmax / RotaryEmbedding / CausalSelfAttention / UniformInit
 * objects.  No reference source is copied into this repository.
 *
 * The reference layer (Layers/CausalSelfAttention.hpp:44-88) only accepts an
 * embedding matrix X and projection weights.  To feed it raw Q, K, V the
 * driver stacks X = [Q; K; V] and uses 0/1 selection matrices for W_q, W_k,
 * W_v (exact in fp32), W_o = identity, and overwrites the public RoPE tables
 * with cos = 1, sin = 0 (RotaryEmbedding.hpp:20-21), so that
 *   cache.attended       = O
 *   cache.scores[h]      = scaled, masked scores  (-> LSE)
 *   cache.queryGradient  = dQ, cache.keyGradient = dK, cache.valueGradient = dV
 * come straight out of the reference's forward / backward.
 * The layer always uses scale = 1/sqrt(headDim) and the causal mask.
 */
#include "NeuralNet/Activations/Softmax.hpp"
#include "NeuralNet/Layers/CausalSelfAttention.hpp"
#include "NeuralNet/Layers/RotaryEmbedding.hpp"
#include "NeuralNet/Math/Matrix.hpp"

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <exception>
#include <vector>

namespace {

Matrix selection(int rows, int cols, int colOffset) {
    Matrix w(static_cast<size_t>(rows), static_cast<size_t>(cols), 0.0f);
    for (int r = 0; r < rows; ++r) w.at(static_cast<size_t>(r), static_cast<size_t>(colOffset + r)) = 1.0f;
    return w;
}

void runLayer(const float* q, const float* k, const float* v, float* out, float* lse, const float* dOut, float* dq,
              float* dk, float* dv, int qHeads, int kvHeads, int d, size_t stride, size_t col0, int t, int qHead0,
              int kvHead0, bool accumulateKv, int windowSize = 0, int globalTokenCount = 0, bool preferSparse = true) {
    const int qRows = qHeads * d;
    const int kvRows = kvHeads * d;
    const int embed = qRows + 2 * kvRows;

    RotaryEmbedding rope(d, t);
    std::fill(rope.cosTable.begin(), rope.cosTable.end(), 1.0f);
    std::fill(rope.sinTable.begin(), rope.sinTable.end(), 0.0f);

    CausalSelfAttention layer(selection(qRows, embed, 0), selection(kvRows, embed, qRows),
                              selection(kvRows, embed, qRows + kvRows), selection(qRows, qRows, 0), rope, qHeads,
                              windowSize > 0 ? windowSize : t, globalTokenCount, kvHeads);
    layer.preferSparseCompute = preferSparse;

    Matrix x(static_cast<size_t>(embed), static_cast<size_t>(t), 0.0f);
    for (int r = 0; r < qRows; ++r)
        for (int c = 0; c < t; ++c) x.at(r, c) = q[(static_cast<size_t>(qHead0) * d + r) * stride + col0 + c];
    for (int r = 0; r < kvRows; ++r)
        for (int c = 0; c < t; ++c) {
            x.at(qRows + r, c) = k[(static_cast<size_t>(kvHead0) * d + r) * stride + col0 + c];
            x.at(qRows + kvRows + r, c) = v[(static_cast<size_t>(kvHead0) * d + r) * stride + col0 + c];
        }

    CausalSelfAttentionCache cache;
    layer.forward(x, cache);
    for (int r = 0; r < qRows; ++r)
        for (int c = 0; c < t; ++c) out[(static_cast<size_t>(qHead0) * d + r) * stride + col0 + c] = cache.attended.at(r, c);

    if (lse) {
        for (int h = 0; h < qHeads; ++h) {
            const Matrix& s = cache.scores[static_cast<size_t>(h)];
            for (int query = 0; query < t; ++query) {
                float top = s.at(0, query);
                for (int key = 1; key < t; ++key) top = std::max(top, s.at(key, query));
                double total = 0.0;
                for (int key = 0; key < t; ++key) total += std::exp(static_cast<double>(s.at(key, query)) - static_cast<double>(top));
                lse[static_cast<size_t>(qHead0 + h) * stride + col0 + query] = static_cast<float>(top + std::log(total));
            }
        }
    }
    if (!dOut) return;

    Matrix g(static_cast<size_t>(qRows), static_cast<size_t>(t), 0.0f);
    for (int r = 0; r < qRows; ++r)
        for (int c = 0; c < t; ++c) g.at(r, c) = dOut[(static_cast<size_t>(qHead0) * d + r) * stride + col0 + c];
    Matrix gwq, gwk, gwv, gwo;
    layer.backward(g, cache, gwq, gwk, gwv, gwo);
    for (int r = 0; r < qRows; ++r)
        for (int c = 0; c < t; ++c)
            dq[(static_cast<size_t>(qHead0) * d + r) * stride + col0 + c] = cache.queryGradient.at(r, c);
    for (int r = 0; r < kvRows; ++r)
        for (int c = 0; c < t; ++c) {
            const size_t idx = (static_cast<size_t>(kvHead0) * d + r) * stride + col0 + c;
            if (accumulateKv) {
                dk[idx] += cache.keyGradient.at(r, c);
                dv[idx] += cache.valueGradient.at(r, c);
            } else {
                dk[idx] = cache.keyGradient.at(r, c);
                dv[idx] = cache.valueGradient.at(r, c);
            }
        }
}

}  // namespace

/*
 * Same argument meaning as sentinel_oracle_attention; `scale` must equal
 * 1/sqrt(headDim) and causal must be 1 (the layer has no other mode).
 * perHead = 0: one layer call per pack with all heads (native GQA inside the layer).
 * perHead = 1: one single-head layer call per (pack, query head) to bound memory;
 *              grouped dK / dV are added in increasing query-head order like
 *              addHeadInto (Layers/CausalSelfAttention.cpp:187-193).
 */
extern "C" int sentinel_ref_attention(const float* q, const float* k, const float* v, float* out, float* lse,
                                      const float* d_out, float* dq, float* dk, float* dv, int qHeads, int kvHeads,
                                      int headDim, int strideColumns, int colStart, int seqLen, int packCount, int perHead) {
    try {
        if (qHeads <= 0 || kvHeads <= 0 || qHeads % kvHeads != 0) return -1;
        const size_t stride = static_cast<size_t>(strideColumns);
        for (int pack = 0; pack < packCount; ++pack) {
            const size_t col0 = static_cast<size_t>(colStart) + static_cast<size_t>(pack) * seqLen;
            if (!perHead) {
                runLayer(q, k, v, out, lse, d_out, dq, dk, dv, qHeads, kvHeads, headDim, stride, col0, seqLen, 0, 0, false);
                continue;
            }
            const int group = qHeads / kvHeads;
            if (d_out)
                for (int r = 0; r < kvHeads * headDim; ++r)
                    for (int c = 0; c < seqLen; ++c) {
                        dk[static_cast<size_t>(r) * stride + col0 + c] = 0.0f;
                        dv[static_cast<size_t>(r) * stride + col0 + c] = 0.0f;
                    }
            for (int h = 0; h < qHeads; ++h)
                runLayer(q, k, v, out, lse, d_out, dq, dk, dv, 1, 1, headDim, stride, col0, seqLen, h, h / group, true);
        }
        return 0;
    } catch (const std::exception&) {
        return -2;
    }
}

/*
 * The layer's sparse mask (windowSize, globalTokenCount; Layers/CausalSelfAttention.cpp:95-120), one layer call
 * per pack with all heads.  preferSparse = 0: dense masked path; 1: the sparse-compute path (:128-168).
 */
extern "C" int sentinel_ref_attention_sparse(const float* q, const float* k, const float* v, float* out, float* lse,
                                             const float* d_out, float* dq, float* dk, float* dv, int qHeads, int kvHeads,
                                             int headDim, int strideColumns, int colStart, int seqLen, int packCount,
                                             int windowSize, int globalTokenCount, int preferSparse) {
    try {
        if (qHeads <= 0 || kvHeads <= 0 || qHeads % kvHeads != 0) return -1;
        for (int pack = 0; pack < packCount; ++pack)
            runLayer(q, k, v, out, lse, d_out, dq, dk, dv, qHeads, kvHeads, headDim, static_cast<size_t>(strideColumns),
                     static_cast<size_t>(colStart) + static_cast<size_t>(pack) * seqLen, seqLen, 0, 0, false, windowSize,
                     globalTokenCount, preferSparse != 0);
        return 0;
    } catch (const std::exception&) {
        return -2;
    }
}

extern "C" int sentinel_ref_gemm(const float* a, int aRows, int aCols, const float* b, int bRows, int bCols, float* c,
                                 int transposeA, int transposeB) {
    try {
        Matrix left(static_cast<size_t>(aRows), static_cast<size_t>(aCols));
        Matrix right(static_cast<size_t>(bRows), static_cast<size_t>(bCols));
        std::copy(a, a + left.data.size(), left.data.begin());
        std::copy(b, b + right.data.size(), right.data.begin());
        Matrix result;
        Matrix::gemm(left, right, result, transposeA != 0, transposeB != 0);
        std::copy(result.data.begin(), result.data.end(), c);
        return 0;
    } catch (const std::exception&) {
        return -2;
    }
}

extern "C" int sentinel_ref_softmax_columns(const float* logits, float* out, int rows, int cols) {
    try {
        Matrix in(static_cast<size_t>(rows), static_cast<size_t>(cols));
        std::copy(logits, logits + in.data.size(), in.data.begin());
        Matrix result;
        Softmax::applyInto(in, result);
        std::copy(result.data.begin(), result.data.end(), out);
        return 0;
    } catch (const std::exception&) {
        return -2;
    }
}

// The reference's own RotaryEmbedding (Layers/RotaryEmbedding.cpp): tables and the in-place rotation of a
// rows x columns matrix (column = position; the host layer has no offset / segment rule).
extern "C" int sentinel_ref_rope_tables(int headDim, int positions, float base, float* cosTable, float* sinTable) {
    try {
        const RotaryEmbedding rope(headDim, positions, base);
        std::copy(rope.cosTable.begin(), rope.cosTable.end(), cosTable);
        std::copy(rope.sinTable.begin(), rope.sinTable.end(), sinTable);
        return 0;
    } catch (const std::exception&) {
        return -1;
    }
}

extern "C" int sentinel_ref_rope_rotate(float* tensor, int heads, int headDim, int columns, int positions, float base,
                                        int inverse) {
    try {
        const RotaryEmbedding rope(headDim, positions, base);
        Matrix m(static_cast<size_t>(heads) * headDim, static_cast<size_t>(columns), 0.0f);
        for (size_t r = 0; r < m.rows; ++r)
            for (size_t c = 0; c < m.cols; ++c) m.at(r, c) = tensor[r * m.cols + c];
        if (inverse)
            rope.rotateInverseInPlace(m, heads);
        else
            rope.rotateInPlace(m, heads);
        for (size_t r = 0; r < m.rows; ++r)
            for (size_t c = 0; c < m.cols; ++c) tensor[r * m.cols + c] = m.at(r, c);
        return 0;
    } catch (const std::exception&) {
        return -1;
    }
}

// The reference's attention layer with real weights and its own RoPE tables, full causal mask (windowSize 0):
// forward and, when d_y != NULL, backward. Shapes as in sentinel_oracle_layer.
extern "C" int sentinel_ref_layer(const float* x, const float* wq, const float* wk, const float* wv, const float* wo,
                                  const float* d_y, float* y, float* d_x, float* d_wq, float* d_wk, float* d_wv, float* d_wo,
                                  int embeddingDim, int qHeads, int kvHeads, int headDim, int seqLen, float ropeBase,
                                  int ropePositions) {
    try {
        const size_t e = static_cast<size_t>(embeddingDim), t = static_cast<size_t>(seqLen);
        const size_t qRows = static_cast<size_t>(qHeads) * headDim, kvRows = static_cast<size_t>(kvHeads) * headDim;
        auto load = [](const float* src, size_t rows, size_t cols) {
            Matrix m(rows, cols, 0.0f);
            std::copy(src, src + rows * cols, m.data.begin());
            return m;
        };
        auto store = [](const Matrix& m, float* dst) { std::copy(m.data.begin(), m.data.end(), dst); };
        CausalSelfAttention layer(load(wq, qRows, e), load(wk, kvRows, e), load(wv, kvRows, e), load(wo, e, qRows),
                                  RotaryEmbedding(headDim, ropePositions, ropeBase), qHeads, 0, 0, kvHeads);
        CausalSelfAttentionCache cache;
        store(layer.forward(load(x, e, t), cache), y);
        if (!d_y) return 0;
        Matrix gwq, gwk, gwv, gwo;
        store(layer.backward(load(d_y, e, t), cache, gwq, gwk, gwv, gwo), d_x);
        store(gwq, d_wq);
        store(gwk, d_wk);
        store(gwv, d_wv);
        store(gwo, d_wo);
        return 0;
    } catch (const std::exception&) {
        return -1;
    }
}
