// Header-only C++ face of the HIP attention library for Sentinel's host code.
//
// HipMatrix mirrors the parts of CudaMatrix the attention dispatch touches
// (sentinel/NeuralNet/Cuda/CudaMatmul.hpp:100-171: rows, cols, buffer.deviceData, ensureSize, upload,
// download) and HipFlashAttention mirrors class CudaFlashAttention
// (sentinel/NeuralNet/Cuda/CudaFlashAttention.hpp:12-41): same static methods, argument order, defaults,
// output resizing (CudaFlashAttention.cu:1555-1556, :1633-1640) and exception types
// (std::invalid_argument for shape / window errors, std::runtime_error for device errors).
// Extra trailing argument kvHeadCount (0 = same as headCount) exposes native grouped-query attention.
// Link against libsentinel_hip_attn.so and the HIP runtime.
#ifndef SENTINEL_HIP_HIPFLASHATTENTION_HPP
#define SENTINEL_HIP_HIPFLASHATTENTION_HPP

#include "../sentinel_hip_attn.h"

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <stdexcept>
#include <string>
#include <vector>

namespace sentinel_hip_host {

inline void throwIfHipFailed(hipError_t status, const char* what) {
    if (status != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(status));
}

/// reusable device float buffer, grows only when capacity is too small; it can also stand for a range of another
/// buffer's memory (alias), which it then never frees
class HipDeviceBuffer {
public:
    float* deviceData = nullptr;
    size_t capacityBytes = 0;
    bool ownsMemory = true;

    HipDeviceBuffer() = default;
    ~HipDeviceBuffer() { this->free(); }
    HipDeviceBuffer(const HipDeviceBuffer&) = delete;
    HipDeviceBuffer& operator=(const HipDeviceBuffer&) = delete;
    HipDeviceBuffer(HipDeviceBuffer&& other) noexcept
        : deviceData(other.deviceData), capacityBytes(other.capacityBytes), ownsMemory(other.ownsMemory) {
        other.deviceData = nullptr;
        other.capacityBytes = 0;
        other.ownsMemory = true;
    }
    HipDeviceBuffer& operator=(HipDeviceBuffer&& other) noexcept {
        if (this != &other) {
            this->free();
            deviceData = other.deviceData;
            capacityBytes = other.capacityBytes;
            ownsMemory = other.ownsMemory;
            other.deviceData = nullptr;
            other.capacityBytes = 0;
            other.ownsMemory = true;
        }
        return *this;
    }
    void ensureCapacity(size_t requiredBytes) {
        if (requiredBytes <= capacityBytes) return;
        this->free();
        throwIfHipFailed(hipMalloc(reinterpret_cast<void**>(&deviceData), requiredBytes), "HipDeviceBuffer hipMalloc");
        capacityBytes = requiredBytes;
    }
    /// stand for `bytes` of memory that someone else owns and keeps alive
    void alias(float* memory, size_t bytes) {
        this->free();
        deviceData = memory;
        capacityBytes = bytes;
        ownsMemory = false;
    }
    void free() {
        if (deviceData && ownsMemory) (void)hipFree(deviceData);
        deviceData = nullptr;
        capacityBytes = 0;
        ownsMemory = true;
    }
};

/// row major float matrix that lives on the device
class HipMatrix {
public:
    size_t rows = 0;
    size_t cols = 0;
    HipDeviceBuffer buffer;

    HipMatrix() = default;
    HipMatrix(HipMatrix&&) noexcept = default;
    HipMatrix& operator=(HipMatrix&&) noexcept = default;

    bool empty() const { return rows == 0 || cols == 0; }
    size_t elementCount() const { return rows * cols; }
    size_t byteCount() const { return rows * cols * sizeof(float); }
    void ensureSize(size_t rowCount, size_t columnCount) {
        rows = rowCount;
        cols = columnCount;
        buffer.ensureCapacity(byteCount());
    }
    void upload(const std::vector<float>& host, size_t rowCount, size_t columnCount) {
        if (host.size() != rowCount * columnCount) throw std::invalid_argument("HipMatrix::upload size mismatch");
        ensureSize(rowCount, columnCount);
        throwIfHipFailed(hipMemcpy(buffer.deviceData, host.data(), byteCount(), hipMemcpyHostToDevice), "HipMatrix::upload");
    }
    std::vector<float> download() const {
        std::vector<float> host(elementCount());
        throwIfHipFailed(hipDeviceSynchronize(), "HipMatrix::download sync");
        throwIfHipFailed(hipMemcpy(host.data(), buffer.deviceData, byteCount(), hipMemcpyDeviceToHost), "HipMatrix::download");
        return host;
    }
    void fill(float value) { upload(std::vector<float>(elementCount(), value), rows, cols); }
    /// become rows [firstRow, firstRow + rowCount) of `whole` without a copy: a block of rows of a row-major matrix is
    /// itself a row-major matrix. `whole` must outlive the view and keep its size.
    void viewRows(HipMatrix& whole, size_t firstRow, size_t rowCount) {
        if (firstRow + rowCount > whole.rows) throw std::invalid_argument("HipMatrix::viewRows outside the matrix");
        rows = rowCount;
        cols = whole.cols;
        buffer.alias(whole.buffer.deviceData + firstRow * whole.cols, byteCount());
    }
};

class HipFlashAttention {
public:
    static constexpr int queryTileSize = 128;
    static constexpr int keyTileSize = 64;
    static constexpr int maxHeadDimension = 128;

    /// arithmetic for the matrix products: SENTINEL_HIP_COMPUTE_AUTO (exact fp32 for these fp32 matrices),
    /// SENTINEL_HIP_COMPUTE_BF16 or SENTINEL_HIP_COMPUTE_F16 (MFMA; head_dim a multiple of 8, padded to 64 / 128 inside)
    static int& computeType() {
        static int value = SENTINEL_HIP_COMPUTE_AUTO;
        return value;
    }

    /// process-wide launch stream (stands for CudaMatmul::activeStream, CudaMatmul.cu:493-506)
    static hipStream_t& activeStream() {
        static hipStream_t stream = nullptr;
        return stream;
    }

    /// The 16-bit copies of query, key, value and out that a forward call with MFMA arithmetic makes anyway, kept for the
    /// backward call of the same tensors (SENTINEL_HIP_WORKSPACE_KEEP / _REUSE), the way CudaCausalSelfAttention keeps
    /// flashLogSumExp between its two calls (Cuda/CudaCausalSelfAttention.cu:237-249, :421-438): the backward call then
    /// converts outGradient only. One per layer; pass it to the forward and to the backward call. A backward call whose
    /// matrices (query, key, value, out by device address), shape, mask, arithmetic or rotation differ from the forward
    /// call that filled it converts everything again. What cannot be seen from here is a matrix that was overwritten in
    /// place between the two calls: whoever does that calls invalidate().
    struct KeptOperands {
        HipDeviceBuffer workspace;
        bool filled = false;
        const void* query = nullptr;
        const void* key = nullptr;
        const void* value = nullptr;
        const void* out = nullptr;
        const void* tables = nullptr;
        int geometry[12] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        /// the matrices the copies were made from have new contents: the next backward call converts them again
        void invalidate() { filled = false; }
        void release() {
            workspace.free();
            filled = false;
        }
    };

    static void forward(const HipMatrix& query, const HipMatrix& key, const HipMatrix& value, HipMatrix& out,
                        HipMatrix& logSumExp, float scale, bool causal = true) {
        forwardMultiHead(query, key, value, out, logSumExp, 1, static_cast<int>(query.rows), scale, causal, 0,
                         static_cast<int>(query.cols));
    }

    static void forwardMultiHead(const HipMatrix& query, const HipMatrix& key, const HipMatrix& value, HipMatrix& out,
                                 HipMatrix& logSumExp, int headCount, int headDimension, float scale, bool causal = true,
                                 int columnStart = 0, int columnCount = 0, int packCount = 1, int kvHeadCount = 0,
                                 KeptOperands* kept = nullptr) {
        const char* op = "HipFlashAttention::forwardMultiHead";
        const int kvHeads = validateMultiHeadShape(query, key, value, headCount, headDimension, kvHeadCount, op);
        if (!sentinel_hip_device_available()) throw std::runtime_error(std::string(op) + " no HIP device");
        out.ensureSize(query.rows, query.cols);
        logSumExp.ensureSize(static_cast<size_t>(headCount), query.cols);
        void* ws = nullptr;
        int layoutFlags = 0;
        const size_t wsBytes = workspaceFor(headCount, kvHeads, headDimension, query, key, value, out, causal, columnStart, columnCount,
                                            packCount, false, ws, kept, nullptr, 0, 0, 0, layoutFlags);
        check(sentinel_hip_flash_fwd(query.buffer.deviceData, key.buffer.deviceData, value.buffer.deviceData,
                                     out.buffer.deviceData, logSumExp.buffer.deviceData, SENTINEL_HIP_F32, computeType(),
                                     SENTINEL_HIP_LAYOUT_COLUMNS | layoutFlags, headCount, kvHeads, headDimension,
                                     static_cast<int>(query.cols), columnStart, columnCount, packCount, scale, causal ? 1 : 0,
                                     ws, wsBytes, activeStream()));
    }

    static void backward(const HipMatrix& query, const HipMatrix& key, const HipMatrix& value, const HipMatrix& out,
                         const HipMatrix& logSumExp, const HipMatrix& outGradient, HipMatrix& queryGradient,
                         HipMatrix& keyGradient, HipMatrix& valueGradient, float scale, bool causal = true) {
        HipMatrix deltaWorkspace;
        backwardMultiHead(query, key, value, out, logSumExp, outGradient, queryGradient, keyGradient, valueGradient,
                          deltaWorkspace, 1, static_cast<int>(query.rows), scale, causal, 0, static_cast<int>(query.cols));
        throwIfHipFailed(hipStreamSynchronize(activeStream()), "HipFlashAttention::backward");  // deltaWorkspace dies here
    }

    static void backwardMultiHead(const HipMatrix& query, const HipMatrix& key, const HipMatrix& value, const HipMatrix& out,
                                  const HipMatrix& logSumExp, const HipMatrix& outGradient, HipMatrix& queryGradient,
                                  HipMatrix& keyGradient, HipMatrix& valueGradient, HipMatrix& deltaWorkspace, int headCount,
                                  int headDimension, float scale, bool causal = true, int columnStart = 0,
                                  int columnCount = 0, int packCount = 1, int kvHeadCount = 0, KeptOperands* kept = nullptr) {
        const char* op = "HipFlashAttention::backwardMultiHead";
        const int kvHeads = validateMultiHeadShape(query, key, value, headCount, headDimension, kvHeadCount, op);
        if (out.rows != query.rows || out.cols != query.cols) throw std::invalid_argument(std::string(op) + " out shape mismatch");
        if (outGradient.rows != query.rows || outGradient.cols != query.cols)
            throw std::invalid_argument(std::string(op) + " outGradient shape mismatch");
        if (logSumExp.rows != static_cast<size_t>(headCount) || logSumExp.cols != query.cols)
            throw std::invalid_argument(std::string(op) + " logSumExp shape mismatch");
        if (!sentinel_hip_device_available()) throw std::runtime_error(std::string(op) + " no HIP device");
        if (packCount <= 0) packCount = 1;
        int resolvedCount = columnCount > 0 ? columnCount : static_cast<int>(query.cols) - columnStart;
        if (columnStart < 0 || resolvedCount <= 0 || columnStart + resolvedCount > static_cast<int>(query.cols))
            throw std::invalid_argument("HipFlashAttention invalid column window");
        queryGradient.ensureSize(query.rows, query.cols);
        keyGradient.ensureSize(key.rows, key.cols);
        valueGradient.ensureSize(value.rows, value.cols);
        deltaWorkspace.ensureSize(static_cast<size_t>(headCount), static_cast<size_t>(packCount) * static_cast<size_t>(resolvedCount));
        void* ws = nullptr;
        int layoutFlags = 0;
        const size_t wsBytes = workspaceFor(headCount, kvHeads, headDimension, query, key, value, out, causal, columnStart, columnCount,
                                            packCount, true, ws, kept, nullptr, 0, 0, 0, layoutFlags);
        check(sentinel_hip_flash_bwd(query.buffer.deviceData, key.buffer.deviceData, value.buffer.deviceData,
                                     out.buffer.deviceData, logSumExp.buffer.deviceData, outGradient.buffer.deviceData,
                                     queryGradient.buffer.deviceData, keyGradient.buffer.deviceData,
                                     valueGradient.buffer.deviceData, deltaWorkspace.buffer.deviceData, SENTINEL_HIP_F32,
                                     computeType(), SENTINEL_HIP_LAYOUT_COLUMNS | layoutFlags, headCount, kvHeads, headDimension,
                                     static_cast<int>(query.cols), columnStart, columnCount, packCount, scale, causal ? 1 : 0,
                                     ws, wsBytes, activeStream()));
    }

    /// forwardMultiHead on unrotated query / key: the rotary embedding (tables rows = positions, cols = headDimension / 2)
    /// is applied on the way into the kernels. Exists for 16-bit computeType() (see sentinel_hip_flash_fwd_rope).
    static void forwardMultiHeadRope(const HipMatrix& query, const HipMatrix& key, const HipMatrix& value, HipMatrix& out,
                                     HipMatrix& logSumExp, const HipMatrix& cosTable, const HipMatrix& sinTable,
                                     int positionOffset, int headCount, int headDimension, float scale, bool causal = true,
                                     int columnStart = 0, int columnCount = 0, int packCount = 1, int kvHeadCount = 0,
                                 KeptOperands* kept = nullptr) {
        const char* op = "HipFlashAttention::forwardMultiHeadRope";
        const int kvHeads = validateMultiHeadShape(query, key, value, headCount, headDimension, kvHeadCount, op);
        if (cosTable.empty() || sinTable.empty()) throw std::invalid_argument(std::string(op) + " empty tables");
        if (!sentinel_hip_device_available()) throw std::runtime_error(std::string(op) + " no HIP device");
        out.ensureSize(query.rows, query.cols);
        logSumExp.ensureSize(static_cast<size_t>(headCount), query.cols);
        void* ws = nullptr;
        int layoutFlags = 0;
        const size_t wsBytes = workspaceFor(headCount, kvHeads, headDimension, query, key, value, out, causal, columnStart, columnCount,
                                            packCount, false, ws, kept, cosTable.buffer.deviceData, 0, 0, positionOffset, layoutFlags);
        check(sentinel_hip_flash_fwd_rope(query.buffer.deviceData, key.buffer.deviceData, value.buffer.deviceData,
                                          out.buffer.deviceData, logSumExp.buffer.deviceData, cosTable.buffer.deviceData,
                                          sinTable.buffer.deviceData, static_cast<int>(cosTable.rows), positionOffset,
                                          SENTINEL_HIP_F32, computeType(), SENTINEL_HIP_LAYOUT_COLUMNS | layoutFlags, headCount, kvHeads,
                                          headDimension, static_cast<int>(query.cols), columnStart, columnCount, packCount,
                                          scale, causal ? 1 : 0, ws, wsBytes, activeStream()));
    }

    /// backwardMultiHead on unrotated query / key; queryGradient / keyGradient come back rotated back.
    static void backwardMultiHeadRope(const HipMatrix& query, const HipMatrix& key, const HipMatrix& value, const HipMatrix& out,
                                      const HipMatrix& logSumExp, const HipMatrix& outGradient, HipMatrix& queryGradient,
                                      HipMatrix& keyGradient, HipMatrix& valueGradient, HipMatrix& deltaWorkspace,
                                      const HipMatrix& cosTable, const HipMatrix& sinTable, int positionOffset, int headCount,
                                      int headDimension, float scale, bool causal = true, int columnStart = 0,
                                      int columnCount = 0, int packCount = 1, int kvHeadCount = 0, KeptOperands* kept = nullptr) {
        const char* op = "HipFlashAttention::backwardMultiHeadRope";
        const int kvHeads = validateMultiHeadShape(query, key, value, headCount, headDimension, kvHeadCount, op);
        if (out.rows != query.rows || out.cols != query.cols) throw std::invalid_argument(std::string(op) + " out shape mismatch");
        if (outGradient.rows != query.rows || outGradient.cols != query.cols)
            throw std::invalid_argument(std::string(op) + " outGradient shape mismatch");
        if (logSumExp.rows != static_cast<size_t>(headCount) || logSumExp.cols != query.cols)
            throw std::invalid_argument(std::string(op) + " logSumExp shape mismatch");
        if (cosTable.empty() || sinTable.empty()) throw std::invalid_argument(std::string(op) + " empty tables");
        if (!sentinel_hip_device_available()) throw std::runtime_error(std::string(op) + " no HIP device");
        if (packCount <= 0) packCount = 1;
        const int resolvedCount = columnCount > 0 ? columnCount : static_cast<int>(query.cols) - columnStart;
        if (columnStart < 0 || resolvedCount <= 0 || columnStart + resolvedCount > static_cast<int>(query.cols))
            throw std::invalid_argument("HipFlashAttention invalid column window");
        queryGradient.ensureSize(query.rows, query.cols);
        keyGradient.ensureSize(key.rows, key.cols);
        valueGradient.ensureSize(value.rows, value.cols);
        deltaWorkspace.ensureSize(static_cast<size_t>(headCount), static_cast<size_t>(packCount) * static_cast<size_t>(resolvedCount));
        void* ws = nullptr;
        int layoutFlags = 0;
        const size_t wsBytes = workspaceFor(headCount, kvHeads, headDimension, query, key, value, out, causal, columnStart, columnCount,
                                            packCount, true, ws, kept, cosTable.buffer.deviceData, 0, 0, positionOffset, layoutFlags);
        check(sentinel_hip_flash_bwd_rope(query.buffer.deviceData, key.buffer.deviceData, value.buffer.deviceData,
                                          out.buffer.deviceData, logSumExp.buffer.deviceData, outGradient.buffer.deviceData,
                                          queryGradient.buffer.deviceData, keyGradient.buffer.deviceData,
                                          valueGradient.buffer.deviceData, deltaWorkspace.buffer.deviceData,
                                          cosTable.buffer.deviceData, sinTable.buffer.deviceData,
                                          static_cast<int>(cosTable.rows), positionOffset, SENTINEL_HIP_F32, computeType(),
                                          SENTINEL_HIP_LAYOUT_COLUMNS | layoutFlags, headCount, kvHeads, headDimension,
                                          static_cast<int>(query.cols), columnStart, columnCount, packCount, scale,
                                          causal ? 1 : 0, ws, wsBytes, activeStream()));
    }

    /// forwardMultiHead under the attention layer's sparse mask (windowSize, globalTokenCount of
    /// CausalSelfAttention::allowsKey, Layers/CausalSelfAttention.cpp:95-100), which the CUDA layer can only run on
    /// its dense path. cosTable / sinTable may be null: no rotation; otherwise as forwardMultiHeadRope.
    static void forwardMultiHeadSparse(const HipMatrix& query, const HipMatrix& key, const HipMatrix& value, HipMatrix& out,
                                       HipMatrix& logSumExp, const HipMatrix* cosTable, const HipMatrix* sinTable,
                                       int positionOffset, int windowSize, int globalTokenCount, int headCount,
                                       int headDimension, float scale, int columnStart = 0, int columnCount = 0,
                                       int packCount = 1, int kvHeadCount = 0, KeptOperands* kept = nullptr) {
        const char* op = "HipFlashAttention::forwardMultiHeadSparse";
        const int kvHeads = validateMultiHeadShape(query, key, value, headCount, headDimension, kvHeadCount, op);
        if ((cosTable == nullptr) != (sinTable == nullptr)) throw std::invalid_argument(std::string(op) + " empty tables");
        if (cosTable && (cosTable->empty() || sinTable->empty())) throw std::invalid_argument(std::string(op) + " empty tables");
        if (!sentinel_hip_device_available()) throw std::runtime_error(std::string(op) + " no HIP device");
        out.ensureSize(query.rows, query.cols);
        logSumExp.ensureSize(static_cast<size_t>(headCount), query.cols);
        void* ws = nullptr;
        int layoutFlags = 0;
        const size_t wsBytes = workspaceFor(headCount, kvHeads, headDimension, query, key, value, out, true, columnStart, columnCount,
                                            packCount, false, ws, kept, cosTable ? cosTable->buffer.deviceData : nullptr, windowSize,
                                            globalTokenCount, positionOffset, layoutFlags);
        check(sentinel_hip_flash_fwd_sparse(query.buffer.deviceData, key.buffer.deviceData, value.buffer.deviceData,
                                            out.buffer.deviceData, logSumExp.buffer.deviceData,
                                            cosTable ? cosTable->buffer.deviceData : nullptr,
                                            sinTable ? sinTable->buffer.deviceData : nullptr,
                                            cosTable ? static_cast<int>(cosTable->rows) : 0, positionOffset, windowSize,
                                            globalTokenCount, SENTINEL_HIP_F32, computeType(), SENTINEL_HIP_LAYOUT_COLUMNS | layoutFlags,
                                            headCount, kvHeads, headDimension, static_cast<int>(query.cols), columnStart,
                                            columnCount, packCount, scale, 1, ws, wsBytes, activeStream()));
    }

    /// backwardMultiHead under the same mask; with tables, queryGradient / keyGradient come back rotated back.
    static void backwardMultiHeadSparse(const HipMatrix& query, const HipMatrix& key, const HipMatrix& value,
                                        const HipMatrix& out, const HipMatrix& logSumExp, const HipMatrix& outGradient,
                                        HipMatrix& queryGradient, HipMatrix& keyGradient, HipMatrix& valueGradient,
                                        HipMatrix& deltaWorkspace, const HipMatrix* cosTable, const HipMatrix* sinTable,
                                        int positionOffset, int windowSize, int globalTokenCount, int headCount,
                                        int headDimension, float scale, int columnStart = 0, int columnCount = 0,
                                        int packCount = 1, int kvHeadCount = 0, KeptOperands* kept = nullptr) {
        const char* op = "HipFlashAttention::backwardMultiHeadSparse";
        const int kvHeads = validateMultiHeadShape(query, key, value, headCount, headDimension, kvHeadCount, op);
        if (out.rows != query.rows || out.cols != query.cols) throw std::invalid_argument(std::string(op) + " out shape mismatch");
        if (outGradient.rows != query.rows || outGradient.cols != query.cols)
            throw std::invalid_argument(std::string(op) + " outGradient shape mismatch");
        if (logSumExp.rows != static_cast<size_t>(headCount) || logSumExp.cols != query.cols)
            throw std::invalid_argument(std::string(op) + " logSumExp shape mismatch");
        if ((cosTable == nullptr) != (sinTable == nullptr)) throw std::invalid_argument(std::string(op) + " empty tables");
        if (cosTable && (cosTable->empty() || sinTable->empty())) throw std::invalid_argument(std::string(op) + " empty tables");
        if (!sentinel_hip_device_available()) throw std::runtime_error(std::string(op) + " no HIP device");
        if (packCount <= 0) packCount = 1;
        const int resolvedCount = columnCount > 0 ? columnCount : static_cast<int>(query.cols) - columnStart;
        if (columnStart < 0 || resolvedCount <= 0 || columnStart + resolvedCount > static_cast<int>(query.cols))
            throw std::invalid_argument("HipFlashAttention invalid column window");
        queryGradient.ensureSize(query.rows, query.cols);
        keyGradient.ensureSize(key.rows, key.cols);
        valueGradient.ensureSize(value.rows, value.cols);
        deltaWorkspace.ensureSize(static_cast<size_t>(headCount), static_cast<size_t>(packCount) * static_cast<size_t>(resolvedCount));
        void* ws = nullptr;
        int layoutFlags = 0;
        const size_t wsBytes = workspaceFor(headCount, kvHeads, headDimension, query, key, value, out, true, columnStart, columnCount,
                                            packCount, true, ws, kept, cosTable ? cosTable->buffer.deviceData : nullptr, windowSize,
                                            globalTokenCount, positionOffset, layoutFlags);
        check(sentinel_hip_flash_bwd_sparse(query.buffer.deviceData, key.buffer.deviceData, value.buffer.deviceData,
                                            out.buffer.deviceData, logSumExp.buffer.deviceData, outGradient.buffer.deviceData,
                                            queryGradient.buffer.deviceData, keyGradient.buffer.deviceData,
                                            valueGradient.buffer.deviceData, deltaWorkspace.buffer.deviceData,
                                            cosTable ? cosTable->buffer.deviceData : nullptr,
                                            sinTable ? sinTable->buffer.deviceData : nullptr,
                                            cosTable ? static_cast<int>(cosTable->rows) : 0, positionOffset, windowSize,
                                            globalTokenCount, SENTINEL_HIP_F32, computeType(), SENTINEL_HIP_LAYOUT_COLUMNS | layoutFlags,
                                            headCount, kvHeads, headDimension, static_cast<int>(query.cols), columnStart,
                                            columnCount, packCount, scale, 1, ws, wsBytes, activeStream()));
    }

private:
    // validateMultiHeadShape (CudaFlashAttention.cu:1458-1471), K/V rows rule widened to grouped heads
    static int validateMultiHeadShape(const HipMatrix& query, const HipMatrix& key, const HipMatrix& value, int headCount,
                                      int headDimension, int kvHeadCount, const char* op) {
        const std::string name(op);
        if (query.empty() || key.empty() || value.empty()) throw std::invalid_argument(name + " empty input");
        if (headCount <= 0 || headDimension <= 0) throw std::invalid_argument(name + " invalid head geometry");
        if (headDimension > maxHeadDimension) throw std::invalid_argument(name + " headDim exceeds maxHeadDimension");
        const int kvHeads = kvHeadCount <= 0 ? headCount : kvHeadCount;
        if (headCount % kvHeads != 0) throw std::invalid_argument(name + " headCount must be divisible by kvHeadCount");
        if (query.rows != static_cast<size_t>(headCount) * static_cast<size_t>(headDimension))
            throw std::invalid_argument(name + " query rows mismatch headCount*headDim");
        if (key.rows != static_cast<size_t>(kvHeads) * static_cast<size_t>(headDimension) || value.rows != key.rows)
            throw std::invalid_argument(name + " key/value rows mismatch");
        if (query.cols != key.cols || query.cols != value.cols) throw std::invalid_argument(name + " sequenceLength mismatch");
        return kvHeads;
    }

    // Scratch for MFMA arithmetic on Sentinel's layout: the caller's KeptOperands where given (sized for the backward
    // call, filled by the forward call, reused by a backward call of the same shape), else one process-wide buffer that
    // only grows (its first growth allocates, so warm it up before capturing a graph).  `layoutFlags` comes back with
    // the workspace flag to OR into the layout argument.
    static size_t workspaceFor(int headCount, int kvHeads, int headDimension, const HipMatrix& query, const HipMatrix& key,
                               const HipMatrix& value, const HipMatrix& out, bool causal, int columnStart, int columnCount,
                               int packCount, bool backward, void*& ws, KeptOperands* kept,
                               const void* tables, int windowSize, int globalTokenCount, int positionOffset,
                               int& layoutFlags) {
        static HipDeviceBuffer scratch;
        layoutFlags = 0;
        const int resolved = columnCount > 0 ? columnCount : static_cast<int>(query.cols) - columnStart;
        auto bytesFor = [&](bool forBackward) {
            return sentinel_hip_flash_workspace_bytes(SENTINEL_HIP_F32, computeType(), SENTINEL_HIP_LAYOUT_COLUMNS, headCount,
                                                      kvHeads, headDimension, resolved > 0 ? resolved : 1,
                                                      packCount > 0 ? packCount : 1, forBackward ? 1 : 0);
        };
        if (kept) {
            const int geometry[12] = {headCount,   kvHeads,       headDimension, static_cast<int>(query.cols), columnStart, columnCount,
                                      packCount,   computeType(), windowSize,    globalTokenCount,             positionOffset,
                                      causal ? 1 : 0};
            const size_t keptBytes = bytesFor(true);
            if (keptBytes == 0) {
                kept->filled = false;  // exact fp32 arithmetic converts nothing
            } else if (!backward) {
                kept->workspace.ensureCapacity(keptBytes);
                kept->filled = true;
                kept->query = query.buffer.deviceData;
                kept->key = key.buffer.deviceData;
                kept->value = value.buffer.deviceData;
                kept->out = out.buffer.deviceData;  // (the forward call has sized it before asking for the workspace)
                kept->tables = tables;
                for (int i = 0; i < 12; ++i) kept->geometry[i] = geometry[i];
                layoutFlags = SENTINEL_HIP_WORKSPACE_KEEP;
                ws = kept->workspace.deviceData;
                return keptBytes;
            } else if (kept->filled && kept->workspace.capacityBytes >= keptBytes && kept->query == query.buffer.deviceData &&
                       kept->key == key.buffer.deviceData && kept->value == value.buffer.deviceData &&
                       kept->out == out.buffer.deviceData && kept->tables == tables) {
                bool same = true;
                for (int i = 0; i < 12; ++i) same = same && kept->geometry[i] == geometry[i];
                if (same) {
                    layoutFlags = SENTINEL_HIP_WORKSPACE_REUSE;
                    ws = kept->workspace.deviceData;
                    return keptBytes;
                }
            }
        }
        const size_t need = bytesFor(backward);
        if (need == 0) return 0;
        scratch.ensureCapacity(need);
        ws = scratch.deviceData;
        return need;
    }

    static void check(int code) {
        if (code == SENTINEL_HIP_OK) return;
        std::string detail = sentinel_hip_last_error();
        if (detail.empty()) detail = sentinel_hip_strerror(code);
        if (code == SENTINEL_HIP_RUNTIME) throw std::runtime_error(detail);
        throw std::invalid_argument(detail);
    }
};

/// The rotary-embedding pair of Sentinel's CudaOps (sentinel/NeuralNet/Cuda/CudaOps.hpp:155-159): same names,
/// argument order, defaults and exceptions (Cuda/CudaOps.cu:1318-1360). Tables are rows = positions,
/// cols = pairCount, as CudaCausalSelfAttention keeps them.
class HipOps {
public:
    static void rotaryRotateInPlace(HipMatrix& tensor, int headCount, int headDimension, int pairCount,
                                    const HipMatrix& cosTable, const HipMatrix& sinTable, int positionOffset = 0,
                                    int segmentLength = 0) {
        rotate("HipOps::rotaryRotateInPlace", tensor, headCount, headDimension, pairCount, cosTable, sinTable,
               positionOffset, segmentLength, 0);
    }
    static void rotaryRotateInverseInPlace(HipMatrix& tensor, int headCount, int headDimension, int pairCount,
                                           const HipMatrix& cosTable, const HipMatrix& sinTable, int positionOffset = 0,
                                           int segmentLength = 0) {
        rotate("HipOps::rotaryRotateInverseInPlace", tensor, headCount, headDimension, pairCount, cosTable, sinTable,
               positionOffset, segmentLength, 1);
    }

    /// CudaOps::scaleInPlace + applySparseAttentionMaskInPlace + softmaxInto (Cuda/CudaOps.hpp:141-147) for `batch`
    /// keys x queries score matrices, `batchStride` floats apart, in place and in one launch
    static void maskedSoftmaxInPlace(float* scores, int batch, long long batchStride, int keyCount, int queryCount, float scale,
                                     int windowSize, int globalTokenCount, int queryPositionStart = 0, int segmentLength = 0) {
        throwUnlessOk(sentinel_hip_dense_softmax_fwd(scores, batch, batchStride, keyCount, queryCount, queryPositionStart,
                                                     windowSize, globalTokenCount, segmentLength, scale,
                                                     HipFlashAttention::activeStream()));
    }
    /// CudaOps::softmaxBackwardInto + zeroForbiddenScoreGradientsInPlace + scaleInPlace (Cuda/CudaOps.hpp:150-153): the
    /// score gradient replaces the probability gradient
    static void maskedSoftmaxBackwardInPlace(const float* probabilities, long long probabilityBatchStride, float* gradient,
                                             long long gradientBatchStride, int batch, int keyCount, int queryCount, float scale,
                                             int windowSize, int globalTokenCount, int queryPositionStart = 0,
                                             int segmentLength = 0) {
        throwUnlessOk(sentinel_hip_dense_softmax_bwd(probabilities, probabilityBatchStride, gradient, gradientBatchStride, batch,
                                                     keyCount, queryCount, queryPositionStart, windowSize, globalTokenCount,
                                                     segmentLength, scale, HipFlashAttention::activeStream()));
    }

private:
    static void throwUnlessOk(int code) {
        if (code == SENTINEL_HIP_OK) return;
        std::string detail = sentinel_hip_last_error();
        if (detail.empty()) detail = sentinel_hip_strerror(code);
        if (code == SENTINEL_HIP_RUNTIME) throw std::runtime_error(detail);
        throw std::invalid_argument(detail);
    }
    static void rotate(const char* op, HipMatrix& tensor, int headCount, int headDimension, int pairCount,
                       const HipMatrix& cosTable, const HipMatrix& sinTable, int positionOffset, int segmentLength,
                       int inverse) {
        const std::string name(op);
        if (tensor.empty()) throw std::invalid_argument(name + " empty tensor");
        if (headCount <= 0 || headDimension <= 0 || pairCount <= 0 || 2 * pairCount != headDimension)
            throw std::invalid_argument(name + " invalid rope dims");
        if (static_cast<int>(tensor.rows) != headCount * headDimension) throw std::invalid_argument(name + " embedding dim mismatch");
        if (cosTable.empty() || sinTable.empty()) throw std::invalid_argument(name + " empty tables");
        if (cosTable.cols != static_cast<size_t>(pairCount) || sinTable.cols != cosTable.cols || sinTable.rows != cosTable.rows)
            throw std::invalid_argument(name + " table shape mismatch");
        if (!sentinel_hip_device_available()) throw std::runtime_error(name + " no HIP device");
        const int code = sentinel_hip_rope_rotate(tensor.buffer.deviceData, headCount, headDimension,
                                                  static_cast<int>(tensor.cols), 0, static_cast<int>(tensor.cols),
                                                  positionOffset, segmentLength, cosTable.buffer.deviceData,
                                                  sinTable.buffer.deviceData, static_cast<int>(cosTable.rows), inverse,
                                                  HipFlashAttention::activeStream());
        if (code == SENTINEL_HIP_OK) return;
        std::string detail = sentinel_hip_last_error();
        if (detail.empty()) detail = sentinel_hip_strerror(code);
        if (code == SENTINEL_HIP_RUNTIME) throw std::runtime_error(detail);
        throw std::invalid_argument(detail);
    }
};

}  // namespace sentinel_hip_host
#endif
