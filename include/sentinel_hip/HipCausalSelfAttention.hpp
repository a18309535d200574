// Header-only C++ attention layer on the device for Sentinel's host code: the caller of the attention core.
//
// HipCausalSelfAttention mirrors the training-path face of class CudaCausalSelfAttention
// (sentinel/NeuralNet/Cuda/CudaCausalSelfAttention.hpp:11-118): the same public weight / table / activation
// members, uploadFrom, forward(input, out, segmentLength) and backward(outputGradient, inputGradient, four weight
// gradients), so that a transformer block written against the CUDA class can hold this one instead. What it does
// (Cuda/CudaCausalSelfAttention.cu:181-253 forward, :345-547 backward, flash branch):
//   Q = Wq X, K = Wk X, V = Wv X        fp32 GEMMs (rocBLAS; the CUDA class uses cuBLASLt), or, with
//                                       HipAmp::preferMixedPrecision, 16-bit operands with fp32 accumulation
//                                       (CudaAmp::preferMixedPrecision, Cuda/CudaMatmul.cu:413)
//   RoPE on Q, K, packs restart at position 0 (segmentLength)
//   flash attention, grouped-query heads read in place (no expandKvHeadsInto / reduceKvHeadGradsInto)
//   Y = Wo A
// and the backward of each step. With 16-bit HipFlashAttention::computeType() the rotation rides on the layout
// conversion (sentinel_hip_flash_fwd_rope / _bwd_rope) and query / key stay unrotated in the cache; with fp32
// arithmetic they are rotated in place like the reference's.
// Generation: HipKvCache mirrors CudaKvCache (Cuda/CudaKvCache.hpp:10-31), prefill / decode mirror
// CudaCausalSelfAttention::prefill / decode (Cuda/CudaCausalSelfAttention.cu:549-575): the rotated K and V columns
// are appended to the cache and the single query of a decode step attends to it with sentinel_hip_decode_attention
// in place of attendCachedQuery's per-head copies and GEMMs (:318-341).
// Layers with a sliding window / global tokens (windowSize, globalTokenCount) run on the same kernels with the
// sparse mask (sentinel_hip_flash_fwd_sparse / _bwd_sparse), where the CUDA class falls back to its dense path.
// With preferFlashAttention = false the layer takes the dense materialising path (Cuda/CudaCausalSelfAttention.cu:255-314
// forward, :445-505 backward): keys x queries scores per (head, pack), probabilities cached for the backward. The CUDA
// class walks the heads one at a time (three head copies, GEMM, scale, mask, softmax, copy, GEMM, head write-back per
// head); here the head blocks of the [(head*d + dim), column] matrices are addressed in place by strided-batched
// GEMMs over all K/V heads at once and one fused scale + mask + softmax launch covers every head and pack.
// Multi-head layers (kvHeadCount == headCount) keep the three projection weights stacked in qkvWeight
// (usesFusedQkv, :19-21, :190-201): one projection GEMM forward, one weight-gradient and one input-gradient GEMM
// backward. queryWeight / keyWeight / valueWeight, query / key / value and the three gradients are row-block views of
// the stacked matrices, so the CUDA class's device-to-device split copies and its syncFusedQkvWeight re-stacking after
// an optimizer step have nothing left to do.
// Link against libsentinel_hip_attn.so, rocBLAS and the HIP runtime.
#ifndef SENTINEL_HIP_HIPCAUSALSELFATTENTION_HPP
#define SENTINEL_HIP_HIPCAUSALSELFATTENTION_HPP

#include "HipAmp.hpp"
#include "HipFlashAttention.hpp"

#include <rocblas/rocblas.h>

#include <cmath>

namespace sentinel_hip_host {

/// C = op(A) op(B) (+ C) on row-major fp32 device matrices; stands for CudaMatrix::multiplyInto and its
/// transposed variants (sentinel/NeuralNet/Cuda/CudaMatmul.hpp), including its mixed-precision branch (HipAmp).
class HipGemm {
public:
    static void multiplyInto(const HipMatrix& a, const HipMatrix& b, HipMatrix& c, bool transposeA = false,
                             bool transposeB = false, bool accumulate = false) {
        const size_t m = transposeA ? a.cols : a.rows;
        const size_t ka = transposeA ? a.rows : a.cols;
        const size_t kb = transposeB ? b.cols : b.rows;
        const size_t n = transposeB ? b.rows : b.cols;
        if (a.empty() || b.empty() || ka != kb) throw std::invalid_argument("HipGemm::multiplyInto shape mismatch");
        if (accumulate) {
            if (c.rows != m || c.cols != n) throw std::invalid_argument("HipGemm::multiplyInto accumulate shape mismatch");
        } else {
            c.ensureSize(m, n);
        }
        const float alpha = 1.0f;
        const float beta = accumulate ? 1.0f : 0.0f;
        rocblas_handle h = handle();
        if (rocblas_set_stream(h, HipFlashAttention::activeStream()) != rocblas_status_success)
            throw std::runtime_error("HipGemm rocblas_set_stream failed");
        // mixed precision first, as CudaMatrix::multiplyInto does (Cuda/CudaMatmul.cu:413): 16-bit copies of both
        // operands, fp32 accumulation; products too small for it and a switched-off HipAmp fall through to fp32
        if (HipAmp::tryMultiply(h, a.buffer.deviceData, a.elementCount(), a.cols, transposeA, b.buffer.deviceData,
                                b.elementCount(), b.cols, transposeB, c.buffer.deviceData, n, m, n, ka, accumulate))
            return;
        // row-major C = op(A) op(B)  <=>  column-major C^T = op(B)^T op(A)^T, each row-major matrix read as its transpose
        const rocblas_status st = rocblas_sgemm(
            h, transposeB ? rocblas_operation_transpose : rocblas_operation_none,
            transposeA ? rocblas_operation_transpose : rocblas_operation_none, static_cast<rocblas_int>(n),
            static_cast<rocblas_int>(m), static_cast<rocblas_int>(ka), &alpha, b.buffer.deviceData,
            static_cast<rocblas_int>(b.cols), a.buffer.deviceData, static_cast<rocblas_int>(a.cols), &beta,
            c.buffer.deviceData, static_cast<rocblas_int>(n));
        if (st != rocblas_status_success) throw std::runtime_error("HipGemm rocblas_sgemm failed");
    }

    /// `batch` products C_i = op(A_i) op(B_i) (+ C_i) on row-major fp32 blocks addressed in place: block i of X starts
    /// at x + i * strideX and its rows are ldX floats apart. op(A) is m x k, op(B) is k x n. Head blocks of the
    /// [(head*d + dim), column] activations are such blocks (stride = d * columns, ld = columns), which is what lets
    /// the dense attention path run without CudaOps::extractHeadInto / writeHead copies.
    static void multiplyBatched(const float* a, size_t lda, long long strideA, bool transposeA, const float* b, size_t ldb,
                                long long strideB, bool transposeB, float* c, size_t ldc, long long strideC, size_t m, size_t n,
                                size_t k, int batch, bool accumulate = false) {
        if (!a || !b || !c || m == 0 || n == 0 || k == 0 || batch <= 0)
            throw std::invalid_argument("HipGemm::multiplyBatched empty operand");
        const float alpha = 1.0f;
        const float beta = accumulate ? 1.0f : 0.0f;
        rocblas_handle h = handle();
        if (rocblas_set_stream(h, HipFlashAttention::activeStream()) != rocblas_status_success)
            throw std::runtime_error("HipGemm rocblas_set_stream failed");
        const rocblas_status st = rocblas_sgemm_strided_batched(
            h, transposeB ? rocblas_operation_transpose : rocblas_operation_none,
            transposeA ? rocblas_operation_transpose : rocblas_operation_none, static_cast<rocblas_int>(n),
            static_cast<rocblas_int>(m), static_cast<rocblas_int>(k), &alpha, b, static_cast<rocblas_int>(ldb), strideB, a,
            static_cast<rocblas_int>(lda), strideA, &beta, c, static_cast<rocblas_int>(ldc), strideC, batch);
        if (st != rocblas_status_success) throw std::runtime_error("HipGemm rocblas_sgemm_strided_batched failed");
    }

private:
    static rocblas_handle handle() {
        static rocblas_handle h = [] {
            rocblas_handle created = nullptr;
            if (rocblas_create_handle(&created) != rocblas_status_success) throw std::runtime_error("HipGemm rocblas_create_handle failed");
            return created;
        }();
        return h;
    }
};

/// What uploadFrom needs of the host layer (Layers/CausalSelfAttention.hpp:44-57): row-major weights
/// (queryWeight (headCount*headDimension) x embeddingDim, key / value (kvHeadCount*headDimension) x embeddingDim,
/// outputWeight embeddingDim x (headCount*headDimension)) and the RoPE parameters.
struct HostAttentionWeights {
    std::vector<float> queryWeight, keyWeight, valueWeight, outputWeight;
    int embeddingDim = 0;
    int headCount = 0;
    int kvHeadCount = 0;  // <= 0: same as headCount
    int headDimension = 0;
    int maximumPositionCount = 0;
    float ropeBase = 10000.0f;
    int windowSize = 0;  // <= 0: full causal
    int globalTokenCount = 0;
};

/// append only device KV cache for one attention layer: key and value are embeddingDim x maximumPositionCount with
/// a used prefix of `length` columns (class CudaKvCache, Cuda/CudaKvCache.hpp:10-31, Cuda/CudaKvCache.cu:9-43)
class HipKvCache {
public:
    HipMatrix key;
    HipMatrix value;
    int length = 0;
    int maximumPositionCount = 0;
    int embeddingDim = 0;

    /// allocate capacity and reset length to zero
    void ensureCapacity(int embeddingDimension, int maximumPositions) {
        if (embeddingDimension <= 0) throw std::invalid_argument("HipKvCache::ensureCapacity embeddingDim must be > 0");
        if (maximumPositions <= 0) throw std::invalid_argument("HipKvCache::ensureCapacity maximumPositionCount must be > 0");
        if (embeddingDim != embeddingDimension || maximumPositionCount != maximumPositions || key.empty() || value.empty()) {
            key.ensureSize(static_cast<size_t>(embeddingDimension), static_cast<size_t>(maximumPositions));
            value.ensureSize(static_cast<size_t>(embeddingDimension), static_cast<size_t>(maximumPositions));
            throwIfHipFailed(hipMemsetAsync(key.buffer.deviceData, 0, key.byteCount(), HipFlashAttention::activeStream()), "HipKvCache zero key");
            throwIfHipFailed(hipMemsetAsync(value.buffer.deviceData, 0, value.byteCount(), HipFlashAttention::activeStream()), "HipKvCache zero value");
        }
        embeddingDim = embeddingDimension;
        maximumPositionCount = maximumPositions;
        length = 0;
    }

    /// set length to zero keep capacity
    void reset() { length = 0; }

    /// append packed key and value columns embeddingDim x stepCount
    void append(const HipMatrix& keyStep, const HipMatrix& valueStep) {
        if (key.empty() || value.empty()) throw std::logic_error("HipKvCache::append capacity not allocated");
        if (keyStep.empty() || valueStep.empty()) throw std::invalid_argument("HipKvCache::append empty step");
        if (keyStep.rows != static_cast<size_t>(embeddingDim) || valueStep.rows != static_cast<size_t>(embeddingDim))
            throw std::invalid_argument("HipKvCache::append embedding dim mismatch");
        if (keyStep.cols != valueStep.cols) throw std::invalid_argument("HipKvCache::append step length mismatch");
        const int stepCount = static_cast<int>(keyStep.cols);
        if (length + stepCount > maximumPositionCount) throw std::invalid_argument("HipKvCache::append exceeds maximumPositionCount");
        writeColumns(key, keyStep);
        writeColumns(value, valueStep);
        length += stepCount;
    }

private:
    // the step's columns land behind the used prefix of every row: a strided 2-D copy
    void writeColumns(HipMatrix& cache, const HipMatrix& step) const {
        throwIfHipFailed(hipMemcpy2DAsync(cache.buffer.deviceData + length, cache.cols * sizeof(float), step.buffer.deviceData,
                                          step.cols * sizeof(float), step.cols * sizeof(float), step.rows,
                                          hipMemcpyDeviceToDevice, HipFlashAttention::activeStream()),
                         "HipKvCache::append copy");
    }
};

/// A layer's weights as HipAmp knows them (CudaAmp::registerMasterWeight calls of the CUDA class,
/// Cuda/CudaCausalSelfAttention.cu:146-151, :164-172). The registrations end with this object, so that no other
/// allocation at a dead weight's address can be served its 16-bit copy.
class MasterWeightRegistrations {
public:
    MasterWeightRegistrations() = default;
    MasterWeightRegistrations(const MasterWeightRegistrations&) = delete;
    MasterWeightRegistrations& operator=(const MasterWeightRegistrations&) = delete;
    MasterWeightRegistrations(MasterWeightRegistrations&& other) noexcept : pointers(std::move(other.pointers)) {
        other.pointers.clear();
    }
    MasterWeightRegistrations& operator=(MasterWeightRegistrations&& other) noexcept {
        if (this != &other) {
            clear();
            pointers = std::move(other.pointers);
            other.pointers.clear();
        }
        return *this;
    }
    ~MasterWeightRegistrations() { clear(); }

    /// register exactly these matrices (empty ones are skipped); earlier registrations of this object end
    void set(std::initializer_list<const HipMatrix*> weights) {
        clear();
        for (const HipMatrix* weight : weights) {
            if (weight == nullptr || weight->empty()) continue;
            HipAmp::registerMasterWeight(weight->buffer.deviceData, weight->elementCount());
            pointers.push_back(weight->buffer.deviceData);
        }
    }
    void clear() {
        for (const float* pointer : pointers) HipAmp::forgetMasterWeight(pointer);
        pointers.clear();
    }

private:
    std::vector<const float*> pointers;
};

class HipCausalSelfAttention {
public:
    HipMatrix queryWeight, keyWeight, valueWeight, outputWeight;
    /// stacked [query; key; value] weights, projections and gradients of a multi-head layer (usesFusedQkv); the split
    /// matrices above and below are then views of their row blocks
    HipMatrix qkvWeight, qkvProjected, qkvGradient, qkvWeightGradient;
    HipMatrix cosTable, sinTable;
    /// the matrices the projection products read, registered with HipAmp: their 16-bit copies are kept until
    /// HipAmp::invalidateMasterWeightHalves() (call it after every optimizer step when preferMixedPrecision is on)
    MasterWeightRegistrations masterWeights;
    int headCount = 0;
    int kvHeadCount = 0;
    int headDimension = 0;
    int pairCount = 0;
    int maximumPositionCount = 0;
    int windowSize = 0;
    int globalTokenCount = 0;
    int activeSegmentLength = 0;
    int activePackCount = 0;
    bool preferFlashAttention = true;
    bool usedFlashAttention = false;

    HipMatrix query, key, value, attended, output;
    HipMatrix inputCache, attendedGradient, queryGradient, keyGradient, valueGradient;
    HipMatrix flashLogSumExp, flashDelta;
    /// mixed-precision projections: the 16-bit copies of the input and of the attended matrix that the forward call's
    /// products read, kept for the weight-gradient products of the backward call (2 bytes per element of each)
    HipDeviceBuffer inputHalf, attendedHalf;
    int keptHalfType = -1;  // SENTINEL_HIP_F16 / _BF16 while both copies match inputCache and attended, else -1
    /// the forward call's 16-bit operands, kept for the backward call like flashLogSumExp (MFMA arithmetic only; costs
    /// 4 bytes per element of query / key / value in device memory per layer; set keepFlashOperands = false to convert
    /// them again in the backward call instead)
    HipFlashAttention::KeptOperands flashOperands;
    bool keepFlashOperands = true;
    HipFlashAttention::KeptOperands* keptOperands() { return keepFlashOperands ? &flashOperands : nullptr; }
    /// dense path: probabilities of every (head, pack), row (head * packs + pack) holds one keys x queries matrix; kept
    /// for the backward like the CUDA class's cachedHeadProbabilities
    HipMatrix probabilities;
    /// dense path backward: probability / score gradients of the heads one batched product covers
    HipMatrix scoreGradient;
    HipDeviceBuffer decodeWorkspace;

    /// upload weights and build the RoPE tables the way RotaryEmbedding does (Layers/RotaryEmbedding.cpp:8-29)
    void uploadFrom(const HostAttentionWeights& host) {
        const char* op = "HipCausalSelfAttention::uploadFrom";
        if (host.embeddingDim <= 0 || host.headCount <= 0 || host.headDimension <= 0 || host.headDimension % 2 != 0)
            throw std::invalid_argument(std::string(op) + " invalid dims");
        const int kv = host.kvHeadCount <= 0 ? host.headCount : host.kvHeadCount;
        if (host.headCount % kv != 0) throw std::invalid_argument(std::string(op) + " headCount must be divisible by kvHeadCount");
        if (host.maximumPositionCount <= 0 || !(host.ropeBase > 0.0f)) throw std::invalid_argument(std::string(op) + " invalid rope");
        headCount = host.headCount;
        kvHeadCount = kv;
        headDimension = host.headDimension;
        pairCount = headDimension / 2;
        maximumPositionCount = host.maximumPositionCount;
        windowSize = host.windowSize;
        globalTokenCount = host.globalTokenCount;
        const size_t e = static_cast<size_t>(host.embeddingDim);
        const size_t qRows = static_cast<size_t>(headCount) * headDimension, kvRows = static_cast<size_t>(kv) * headDimension;
        if (host.queryWeight.size() != qRows * e || host.keyWeight.size() != kvRows * e || host.valueWeight.size() != kvRows * e)
            throw std::invalid_argument(std::string(op) + " key/value rows mismatch kvHeadCount");
        // views of a previous configuration's stacked matrices must not outlive them
        HipMatrix* mayBeViews[] = {&queryWeight, &keyWeight, &valueWeight, &query, &key, &value, &queryGradient, &keyGradient,
                                   &valueGradient};
        for (HipMatrix* m : mayBeViews)
            if (!m->buffer.ownsMemory) *m = HipMatrix();
        if (usesFusedQkv()) {
            qkvWeight.ensureSize(3 * qRows, e);
            queryWeight.viewRows(qkvWeight, 0, qRows);
            keyWeight.viewRows(qkvWeight, qRows, qRows);
            valueWeight.viewRows(qkvWeight, 2 * qRows, qRows);
        } else {
            qkvWeight = HipMatrix();
        }
        queryWeight.upload(host.queryWeight, qRows, e);
        keyWeight.upload(host.keyWeight, kvRows, e);
        valueWeight.upload(host.valueWeight, kvRows, e);
        outputWeight.upload(host.outputWeight, e, qRows);
        std::vector<float> cosHost(static_cast<size_t>(maximumPositionCount) * pairCount), sinHost(cosHost.size());
        for (int position = 0; position < maximumPositionCount; ++position)
            for (int pairIndex = 0; pairIndex < pairCount; ++pairIndex) {
                const float exponent = -2.0f * static_cast<float>(pairIndex) / static_cast<float>(headDimension);
                const float angle = static_cast<float>(position) * std::pow(host.ropeBase, exponent);
                cosHost[static_cast<size_t>(position) * pairCount + pairIndex] = std::cos(angle);
                sinHost[static_cast<size_t>(position) * pairCount + pairIndex] = std::sin(angle);
            }
        cosTable.upload(cosHost, static_cast<size_t>(maximumPositionCount), static_cast<size_t>(pairCount));
        sinTable.upload(sinHost, static_cast<size_t>(maximumPositionCount), static_cast<size_t>(pairCount));
        registerMasterWeights();
    }

    /// (re-)register the weights the products read: the stacked matrix of a multi-head layer, else the three split ones,
    /// and the output weight. Registering marks their 16-bit copies stale (CudaAmp::registerMasterWeight).
    void registerMasterWeights() {
        if (usesFusedQkv() && !qkvWeight.empty())
            masterWeights.set({&qkvWeight, &outputWeight});
        else
            masterWeights.set({&queryWeight, &keyWeight, &valueWeight, &outputWeight});
    }

    static HipCausalSelfAttention createFrom(const HostAttentionWeights& host) {
        HipCausalSelfAttention layer;
        layer.uploadFrom(host);
        return layer;
    }

    /// one stacked projection for multi-head layers (CudaCausalSelfAttention::usesFusedQkv, Cuda/CudaCausalSelfAttention.cu:19-21)
    bool usesFusedQkv() const { return kvHeadCount > 0 && kvHeadCount == headCount; }

    /// CudaCausalSelfAttention::syncFusedQkvWeight (:155-173) re-stacks the split weights after the optimizer changed
    /// them. Here the split weights are views of the stacked matrix, so an update of either is an update of both and
    /// there is nothing to copy; only split weights that were replaced by matrices of their own are stacked again.
    void syncFusedQkvWeight() {
        if (!usesFusedQkv()) {
            if (!qkvWeight.empty()) {
                qkvWeight = HipMatrix();
                registerMasterWeights();
            }
            return;
        }
        if (queryWeight.empty() || keyWeight.empty() || valueWeight.empty()) return;
        if (queryWeight.cols != keyWeight.cols || queryWeight.cols != valueWeight.cols)
            throw std::invalid_argument("HipCausalSelfAttention::syncFusedQkvWeight embed mismatch");
        if (queryWeight.rows != keyWeight.rows || queryWeight.rows != valueWeight.rows)
            throw std::invalid_argument("HipCausalSelfAttention::syncFusedQkvWeight projection rows mismatch");
        const size_t rows = queryWeight.rows;
        const bool stacked = !qkvWeight.empty() && qkvWeight.rows == 3 * rows && qkvWeight.cols == queryWeight.cols &&
                             queryWeight.buffer.deviceData == qkvWeight.buffer.deviceData &&
                             keyWeight.buffer.deviceData == qkvWeight.buffer.deviceData + rows * qkvWeight.cols &&
                             valueWeight.buffer.deviceData == qkvWeight.buffer.deviceData + 2 * rows * qkvWeight.cols;
        if (stacked) return;
        HipMatrix fresh;
        fresh.ensureSize(3 * rows, queryWeight.cols);
        HipMatrix* parts[3] = {&queryWeight, &keyWeight, &valueWeight};
        for (int i = 0; i < 3; ++i)
            throwIfHipFailed(hipMemcpyAsync(fresh.buffer.deviceData + i * rows * fresh.cols, parts[i]->buffer.deviceData,
                                            parts[i]->byteCount(), hipMemcpyDeviceToDevice, HipFlashAttention::activeStream()),
                             "HipCausalSelfAttention::syncFusedQkvWeight copy");
        throwIfHipFailed(hipStreamSynchronize(HipFlashAttention::activeStream()), "HipCausalSelfAttention::syncFusedQkvWeight");
        qkvWeight = std::move(fresh);
        for (int i = 0; i < 3; ++i) parts[i]->viewRows(qkvWeight, i * rows, rows);
        registerMasterWeights();
    }

    /// release dense-only scratch (CudaCausalSelfAttention::releaseDenseAttentionScratch, :59-77)
    void releaseDenseAttentionScratch() {
        probabilities = HipMatrix();
        scoreGradient = HipMatrix();
    }
    /// release flash-only scratch (CudaCausalSelfAttention::releaseFlashAttentionScratch, :79-86)
    void releaseFlashAttentionScratch() {
        flashLogSumExp = HipMatrix();
        flashDelta = HipMatrix();
        flashOperands.release();
    }
    /// free the activations after a forward, weights kept (CudaCausalSelfAttention::releaseActivationScratch, :88-108)
    void releaseActivationScratch() {
        releaseFlashAttentionScratch();
        releaseDenseAttentionScratch();
        HipMatrix* all[] = {&query, &key, &value, &queryGradient, &keyGradient, &valueGradient, &qkvProjected, &qkvGradient,
                            &attended, &output, &inputCache, &attendedGradient};
        for (HipMatrix* m : all) *m = HipMatrix();
        inputHalf.free();
        attendedHalf.free();
        keptHalfType = -1;
    }

    /// CudaCausalSelfAttention::canUseFlashAttention (Cuda/CudaCausalSelfAttention.cu:46-57) without the
    /// multiple-of-4 rules and without the full-causal-only rule, neither of which these kernels need
    bool canUseFlashAttention(int sequenceLength) const {
        (void)sequenceLength;
        if (!preferFlashAttention) return false;
        if (headDimension <= 0 || headDimension > HipFlashAttention::maxHeadDimension) return false;
        return true;
    }

    /// the sparse mask is in force for sequences longer than the window (CausalSelfAttention::usesSparseCompute's
    /// rule, Layers/CausalSelfAttention.cpp:102-107; shorter ones see the plain causal mask)
    bool usesSparseMask(int sequenceLength) const { return windowSize > 0 && windowSize < sequenceLength; }

    /// causal multi head attention writing into out; input is embeddingDim x columns, packs of segmentLength columns
    void forward(const HipMatrix& input, HipMatrix& out, int segmentLength = 0) {
        const char* op = "HipCausalSelfAttention::forward";
        if (input.empty()) throw std::invalid_argument(std::string(op) + " empty input");
        if (queryWeight.empty()) throw std::logic_error(std::string(op) + " called before uploadFrom");
        if (queryWeight.cols != input.rows) throw std::invalid_argument(std::string(op) + " embedding dim mismatch");
        const int columns = static_cast<int>(input.cols);
        if (segmentLength <= 0) segmentLength = columns;
        if (columns % segmentLength != 0) throw std::invalid_argument(std::string(op) + " columns must be a multiple of segmentLength");
        if (segmentLength > maximumPositionCount) throw std::invalid_argument(std::string(op) + " segmentLength exceeds RoPE table");
        activeSegmentLength = segmentLength;
        activePackCount = columns / segmentLength;
        usedFlashAttention = canUseFlashAttention(segmentLength);
        HipAmp::ActivationCastScope castOnce;  // no cast buffer below is rewritten once a product has read it
        keptHalfType = -1;
        const bool keepHalves = HipAmp::wouldMultiplyMixed(queryWeight.rows, input.cols, input.rows) &&
                                HipAmp::wouldMultiplyMixed(outputWeight.rows, input.cols, outputWeight.cols);
        if (keepHalves) {
            const int type = HipAmp::persistActivationHalf(input.buffer.deviceData, input.elementCount(), inputHalf);
            castOnce.adopt(input.buffer.deviceData, input.elementCount(), inputHalf.deviceData, type);
        }

        inputCache.ensureSize(input.rows, input.cols);
        throwIfHipFailed(hipMemcpyAsync(inputCache.buffer.deviceData, input.buffer.deviceData, input.byteCount(),
                                        hipMemcpyDeviceToDevice, HipFlashAttention::activeStream()),
                         "HipCausalSelfAttention::forward input copy");
        project(input);
        const float scale = 1.0f / std::sqrt(static_cast<float>(headDimension));
        const bool sparse = usesSparseMask(segmentLength);
        if (!usedFlashAttention) {
            releaseFlashAttentionScratch();
            HipOps::rotaryRotateInPlace(query, headCount, headDimension, pairCount, cosTable, sinTable, 0, segmentLength);
            HipOps::rotaryRotateInPlace(key, kvHeadCount, headDimension, pairCount, cosTable, sinTable, 0, segmentLength);
            attendDense(segmentLength, activePackCount);
        } else if (fusedRotation()) {
            releaseDenseAttentionScratch();
            if (sparse)
                HipFlashAttention::forwardMultiHeadSparse(query, key, value, attended, flashLogSumExp, &cosTable, &sinTable, 0,
                                                          windowSize, globalTokenCount, headCount, headDimension, scale, 0,
                                                          segmentLength, activePackCount, kvHeadCount, keptOperands());
            else
                HipFlashAttention::forwardMultiHeadRope(query, key, value, attended, flashLogSumExp, cosTable, sinTable, 0,
                                                        headCount, headDimension, scale, true, 0, segmentLength,
                                                        activePackCount, kvHeadCount, keptOperands());
        } else {
            releaseDenseAttentionScratch();
            HipOps::rotaryRotateInPlace(query, headCount, headDimension, pairCount, cosTable, sinTable, 0, segmentLength);
            HipOps::rotaryRotateInPlace(key, kvHeadCount, headDimension, pairCount, cosTable, sinTable, 0, segmentLength);
            if (sparse)
                HipFlashAttention::forwardMultiHeadSparse(query, key, value, attended, flashLogSumExp, nullptr, nullptr, 0,
                                                          windowSize, globalTokenCount, headCount, headDimension, scale, 0,
                                                          segmentLength, activePackCount, kvHeadCount, keptOperands());
            else
                HipFlashAttention::forwardMultiHead(query, key, value, attended, flashLogSumExp, headCount, headDimension, scale,
                                                    true, 0, segmentLength, activePackCount, kvHeadCount, keptOperands());
        }
        if (keepHalves) {
            keptHalfType = HipAmp::persistActivationHalf(attended.buffer.deviceData, attended.elementCount(), attendedHalf);
            castOnce.adopt(attended.buffer.deviceData, attended.elementCount(), attendedHalf.deviceData, keptHalfType);
        }
        HipGemm::multiplyInto(outputWeight, attended, out);
    }

    /// backprop through the layer; weight gradients are overwritten (summed over all columns of the batch).
    /// materializeSplitWeightGrads = false leaves the stacked qkvWeightGradient only (multi-head layers), as in
    /// CudaCausalSelfAttention::backward (Cuda/CudaCausalSelfAttention.cu:357-365, :519-529).
    void backward(const HipMatrix& outputGradient, HipMatrix& inputGradient, HipMatrix& queryWeightGradient,
                  HipMatrix& keyWeightGradient, HipMatrix& valueWeightGradient, HipMatrix& outputWeightGradient,
                  bool materializeSplitWeightGrads = true) {
        const char* op = "HipCausalSelfAttention::backward";
        if (inputCache.empty()) throw std::logic_error(std::string(op) + " called before forward");
        if (outputGradient.rows != outputWeight.rows || outputGradient.cols != attended.cols)
            throw std::invalid_argument(std::string(op) + " output gradient shape mismatch");
        if (usedFlashAttention) {
            if (flashLogSumExp.rows != static_cast<size_t>(headCount) || flashLogSumExp.cols != query.cols)
                throw std::invalid_argument(std::string(op) + " flash logSumExp shape mismatch");
        } else if (probabilities.rows != static_cast<size_t>(headCount) * activePackCount) {
            throw std::invalid_argument(std::string(op) + " head cache size mismatch");
        }
        // outputGradient, the stacked / split projection gradients and inputCache feed two or three products each
        HipAmp::ActivationCastScope castOnce;
        if (keptHalfType >= 0) {  // the forward call's 16-bit copies of the input and of the attended matrix
            castOnce.adopt(inputCache.buffer.deviceData, inputCache.elementCount(), inputHalf.deviceData, keptHalfType);
            castOnce.adopt(attended.buffer.deviceData, attended.elementCount(), attendedHalf.deviceData, keptHalfType);
        }
        HipGemm::multiplyInto(outputGradient, attended, outputWeightGradient, false, true);
        HipGemm::multiplyInto(outputWeight, outputGradient, attendedGradient, true, false);
        if (usesFusedQkv()) {
            qkvGradient.ensureSize(3 * query.rows, query.cols);
            queryGradient.viewRows(qkvGradient, 0, query.rows);
            keyGradient.viewRows(qkvGradient, query.rows, query.rows);
            valueGradient.viewRows(qkvGradient, 2 * query.rows, query.rows);
        }
        const float scale = 1.0f / std::sqrt(static_cast<float>(headDimension));
        const bool sparse = usesSparseMask(activeSegmentLength);
        if (!usedFlashAttention) {
            backwardDense(activeSegmentLength, activePackCount);
            HipOps::rotaryRotateInverseInPlace(queryGradient, headCount, headDimension, pairCount, cosTable, sinTable, 0,
                                               activeSegmentLength);
            HipOps::rotaryRotateInverseInPlace(keyGradient, kvHeadCount, headDimension, pairCount, cosTable, sinTable, 0,
                                               activeSegmentLength);
        } else if (fusedRotation()) {
            if (sparse)
                HipFlashAttention::backwardMultiHeadSparse(query, key, value, attended, flashLogSumExp, attendedGradient,
                                                           queryGradient, keyGradient, valueGradient, flashDelta, &cosTable,
                                                           &sinTable, 0, windowSize, globalTokenCount, headCount, headDimension,
                                                           scale, 0, activeSegmentLength, activePackCount, kvHeadCount, keptOperands());
            else
                HipFlashAttention::backwardMultiHeadRope(query, key, value, attended, flashLogSumExp, attendedGradient,
                                                         queryGradient, keyGradient, valueGradient, flashDelta, cosTable,
                                                         sinTable, 0, headCount, headDimension, scale, true, 0,
                                                         activeSegmentLength, activePackCount, kvHeadCount, keptOperands());
        } else {
            if (sparse)
                HipFlashAttention::backwardMultiHeadSparse(query, key, value, attended, flashLogSumExp, attendedGradient,
                                                           queryGradient, keyGradient, valueGradient, flashDelta, nullptr,
                                                           nullptr, 0, windowSize, globalTokenCount, headCount, headDimension,
                                                           scale, 0, activeSegmentLength, activePackCount, kvHeadCount, keptOperands());
            else
                HipFlashAttention::backwardMultiHead(query, key, value, attended, flashLogSumExp, attendedGradient,
                                                     queryGradient, keyGradient, valueGradient, flashDelta, headCount,
                                                     headDimension, scale, true, 0, activeSegmentLength, activePackCount,
                                                     kvHeadCount, keptOperands());
            HipOps::rotaryRotateInverseInPlace(queryGradient, headCount, headDimension, pairCount, cosTable, sinTable, 0,
                                               activeSegmentLength);
            HipOps::rotaryRotateInverseInPlace(keyGradient, kvHeadCount, headDimension, pairCount, cosTable, sinTable, 0,
                                               activeSegmentLength);
        }
        if (usesFusedQkv()) {
            if (queryGradient.buffer.deviceData != qkvGradient.buffer.deviceData)
                throw std::logic_error(std::string(op) + " gradient views were replaced");
            // stacked [dQ; dK; dV]: one weight-gradient product and one input-gradient product (:507-530)
            HipGemm::multiplyInto(qkvGradient, inputCache, qkvWeightGradient, false, true);
            if (materializeSplitWeightGrads) {
                HipMatrix* parts[3] = {&queryWeightGradient, &keyWeightGradient, &valueWeightGradient};
                for (int i = 0; i < 3; ++i) {
                    parts[i]->ensureSize(queryWeight.rows, queryWeight.cols);
                    throwIfHipFailed(hipMemcpyAsync(parts[i]->buffer.deviceData,
                                                    qkvWeightGradient.buffer.deviceData + i * queryWeight.elementCount(),
                                                    queryWeight.byteCount(), hipMemcpyDeviceToDevice,
                                                    HipFlashAttention::activeStream()),
                                     "HipCausalSelfAttention::backward weight gradient split");
                }
            }
            HipGemm::multiplyInto(qkvWeight, qkvGradient, inputGradient, true, false);
        } else {
            if (materializeSplitWeightGrads) {
                HipGemm::multiplyInto(queryGradient, inputCache, queryWeightGradient, false, true);
                HipGemm::multiplyInto(keyGradient, inputCache, keyWeightGradient, false, true);
                HipGemm::multiplyInto(valueGradient, inputCache, valueWeightGradient, false, true);
            }
            HipGemm::multiplyInto(queryWeight, queryGradient, inputGradient, true, false);
            HipGemm::multiplyInto(keyWeight, keyGradient, inputGradient, true, false, true);
            HipGemm::multiplyInto(valueWeight, valueGradient, inputGradient, true, false, true);
        }
    }

    /// reset cache then run full sequence attention and append rotated KV
    void prefill(const HipMatrix& input, HipKvCache& cache, HipMatrix& out) {
        const char* op = "HipCausalSelfAttention::prefill";
        if (input.empty()) throw std::invalid_argument(std::string(op) + " empty input");
        if (queryWeight.empty()) throw std::logic_error(std::string(op) + " weights not uploaded");
        if (queryWeight.cols != input.rows) throw std::invalid_argument(std::string(op) + " embedding dim mismatch");
        if (static_cast<int>(input.cols) > maximumPositionCount)
            throw std::invalid_argument(std::string(op) + " sequence longer than maximumPositionCount");
        cache.ensureCapacity(static_cast<int>(keyWeight.rows), maximumPositionCount);
        projectAndRotate(input, 0);
        cache.append(key, value);
        const float scale = 1.0f / std::sqrt(static_cast<float>(headDimension));
        if (!canUseFlashAttention(static_cast<int>(input.cols)))
            attendDense(static_cast<int>(input.cols), 1);
        else if (usesSparseMask(static_cast<int>(input.cols)))
            HipFlashAttention::forwardMultiHeadSparse(query, key, value, attended, flashLogSumExp, nullptr, nullptr, 0, windowSize,
                                                      globalTokenCount, headCount, headDimension, scale, 0,
                                                      static_cast<int>(input.cols), 1, kvHeadCount);
        else
            HipFlashAttention::forwardMultiHead(query, key, value, attended, flashLogSumExp, headCount, headDimension, scale, true,
                                                0, static_cast<int>(input.cols), 1, kvHeadCount);
        HipGemm::multiplyInto(outputWeight, attended, out);
    }

    /// single token attention against append only KV cache
    void decode(const HipMatrix& input, HipKvCache& cache, HipMatrix& out) {
        const char* op = "HipCausalSelfAttention::decode";
        if (input.empty()) throw std::invalid_argument(std::string(op) + " empty input");
        if (input.cols != 1) throw std::invalid_argument(std::string(op) + " expects a single token column");
        if (queryWeight.empty()) throw std::logic_error(std::string(op) + " weights not uploaded");
        if (queryWeight.cols != input.rows) throw std::invalid_argument(std::string(op) + " embedding dim mismatch");
        if (cache.key.empty() || cache.value.empty()) throw std::logic_error(std::string(op) + " cache not allocated");
        if (cache.length >= cache.maximumPositionCount) throw std::invalid_argument(std::string(op) + " cache full");
        if (cache.length >= maximumPositionCount) throw std::invalid_argument(std::string(op) + " position exceeds RoPE table");
        projectAndRotate(input, cache.length);
        cache.append(key, value);
        attendCachedQuery(cache, out);
    }

private:
    // Q, K, V projections of the input columns: one stacked product whose row blocks query / key / value then view
    // (multi-head layers), three products otherwise (CudaCausalSelfAttention::projectAndRotate,
    // Cuda/CudaCausalSelfAttention.cu:181-208, without its three split copies)
    void project(const HipMatrix& input) {
        // query / key / value get new contents: 16-bit copies of the old ones must not serve a later backward call (the
        // training forward refills them right after this; prefill and decode do not)
        flashOperands.invalidate();
        keptHalfType = -1;  // likewise the kept 16-bit copies of input and attended; forward() sets it again
        if (usesFusedQkv()) {
            syncFusedQkvWeight();
            HipGemm::multiplyInto(qkvWeight, input, qkvProjected);
            query.viewRows(qkvProjected, 0, queryWeight.rows);
            key.viewRows(qkvProjected, queryWeight.rows, queryWeight.rows);
            value.viewRows(qkvProjected, 2 * queryWeight.rows, queryWeight.rows);
        } else {
            HipGemm::multiplyInto(queryWeight, input, query);
            HipGemm::multiplyInto(keyWeight, input, key);
            HipGemm::multiplyInto(valueWeight, input, value);
        }
    }

    // projections, then Q and K rotated in place for positions offset, offset + 1, ...
    void projectAndRotate(const HipMatrix& input, int positionOffset) {
        project(input);
        HipOps::rotaryRotateInPlace(query, headCount, headDimension, pairCount, cosTable, sinTable, positionOffset);
        HipOps::rotaryRotateInPlace(key, kvHeadCount, headDimension, pairCount, cosTable, sinTable, positionOffset);
    }

    // Dense forward (Cuda/CudaCausalSelfAttention.cu:255-314): P = softmax(mask(scale * K^T Q)) per (head, pack), kept in
    // `probabilities`; attended = V P. Head h of query head group j of K/V head v is h = v * group + j: for a fixed
    // (pack, j) the blocks of the K/V heads are a constant stride apart in every operand, one batched product each.
    void attendDense(int segmentLength, int packCount) {
        const size_t t = static_cast<size_t>(segmentLength), cols = query.cols, d = static_cast<size_t>(headDimension);
        const size_t tt = t * t;
        const int group = headCount / kvHeadCount;
        const float scale = 1.0f / std::sqrt(static_cast<float>(headDimension));
        probabilities.ensureSize(static_cast<size_t>(headCount) * packCount, tt);
        attended.ensureSize(query.rows, cols);
        float* p = probabilities.buffer.deviceData;
        const long long kvStride = static_cast<long long>(d * cols), qStride = kvStride * group;
        const long long pStride = static_cast<long long>(tt) * packCount * group;
        for (int pack = 0; pack < packCount; ++pack)
            for (int j = 0; j < group; ++j) {
                const size_t c0 = static_cast<size_t>(pack) * t;
                HipGemm::multiplyBatched(key.buffer.deviceData + c0, cols, kvStride, true,
                                         query.buffer.deviceData + j * d * cols + c0, cols, qStride, false,
                                         p + (static_cast<size_t>(j) * packCount + pack) * tt, t, pStride, t, t, d, kvHeadCount);
            }
        HipOps::maskedSoftmaxInPlace(p, headCount * packCount, static_cast<long long>(tt), segmentLength, segmentLength, scale,
                                     windowSize, globalTokenCount);
        for (int pack = 0; pack < packCount; ++pack)
            for (int j = 0; j < group; ++j) {
                const size_t c0 = static_cast<size_t>(pack) * t;
                HipGemm::multiplyBatched(value.buffer.deviceData + c0, cols, kvStride, false,
                                         p + (static_cast<size_t>(j) * packCount + pack) * tt, t, pStride, false,
                                         attended.buffer.deviceData + j * d * cols + c0, cols, qStride, d, t, t, kvHeadCount);
            }
    }

    // Dense backward (:445-505) from the cached probabilities: per (pack, j) and batched over the K/V heads
    //   dV += dA P^T,  dP = V^T dA,  dS = scale * P (dP - colsum(dP P)) masked,  dQ = K dS,  dK += Q dS^T
    // (+= over the query heads j of a K/V head: the first j overwrites, so no zero pass is needed).
    void backwardDense(int segmentLength, int packCount) {
        const size_t t = static_cast<size_t>(segmentLength), cols = query.cols, d = static_cast<size_t>(headDimension);
        const size_t tt = t * t;
        const int group = headCount / kvHeadCount;
        const float scale = 1.0f / std::sqrt(static_cast<float>(headDimension));
        queryGradient.ensureSize(query.rows, cols);
        keyGradient.ensureSize(key.rows, cols);
        valueGradient.ensureSize(value.rows, cols);
        scoreGradient.ensureSize(static_cast<size_t>(kvHeadCount), tt);
        float* ds = scoreGradient.buffer.deviceData;
        const long long kvStride = static_cast<long long>(d * cols), qStride = kvStride * group;
        const long long pStride = static_cast<long long>(tt) * packCount * group, dsStride = static_cast<long long>(tt);
        for (int pack = 0; pack < packCount; ++pack)
            for (int j = 0; j < group; ++j) {
                const size_t c0 = static_cast<size_t>(pack) * t;
                const float* p = probabilities.buffer.deviceData + (static_cast<size_t>(j) * packCount + pack) * tt;
                const float* dA = attendedGradient.buffer.deviceData + j * d * cols + c0;
                const float* q = query.buffer.deviceData + j * d * cols + c0;
                HipGemm::multiplyBatched(dA, cols, qStride, false, p, t, pStride, true, valueGradient.buffer.deviceData + c0, cols,
                                         kvStride, d, t, t, kvHeadCount, j > 0);
                HipGemm::multiplyBatched(value.buffer.deviceData + c0, cols, kvStride, true, dA, cols, qStride, false, ds, t,
                                         dsStride, t, t, d, kvHeadCount);
                HipOps::maskedSoftmaxBackwardInPlace(p, pStride, ds, dsStride, kvHeadCount, segmentLength, segmentLength, scale,
                                                     windowSize, globalTokenCount);
                HipGemm::multiplyBatched(key.buffer.deviceData + c0, cols, kvStride, false, ds, t, dsStride, false,
                                         queryGradient.buffer.deviceData + j * d * cols + c0, cols, qStride, d, t, t, kvHeadCount);
                HipGemm::multiplyBatched(q, cols, qStride, false, ds, t, dsStride, true, keyGradient.buffer.deviceData + c0, cols,
                                         kvStride, d, t, t, kvHeadCount, j > 0);
            }
    }

    void attendCachedQuery(const HipKvCache& cache, HipMatrix& out) {
        const float scale = 1.0f / std::sqrt(static_cast<float>(headDimension));
        attended.ensureSize(query.rows, 1);
        const size_t need = sentinel_hip_decode_workspace_bytes(headCount, headDimension, cache.length);
        decodeWorkspace.ensureCapacity(need);
        const int code = sentinel_hip_decode_attention(query.buffer.deviceData, cache.key.buffer.deviceData,
                                                       cache.value.buffer.deviceData, attended.buffer.deviceData, headCount,
                                                       kvHeadCount, headDimension, cache.maximumPositionCount, cache.length, scale,
                                                       windowSize, globalTokenCount, decodeWorkspace.deviceData, need,
                                                       HipFlashAttention::activeStream());
        if (code != SENTINEL_HIP_OK) {
            std::string detail = sentinel_hip_last_error();
            if (detail.empty()) detail = sentinel_hip_strerror(code);
            if (code == SENTINEL_HIP_RUNTIME) throw std::runtime_error(detail);
            throw std::invalid_argument(detail);
        }
        HipGemm::multiplyInto(outputWeight, attended, out);
    }

    // the rotation rides on the fp32 <-> 16-bit conversion when there is one
    bool fusedRotation() const {
        const int compute = HipFlashAttention::computeType();
        return (compute == SENTINEL_HIP_COMPUTE_BF16 || compute == SENTINEL_HIP_COMPUTE_F16) &&
               headDimension % 8 == 0 && headDimension <= 128;
    }
};

}  // namespace sentinel_hip_host
#endif
