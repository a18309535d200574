// Mixed-precision GEMMs for the attention layer's projections: fp32 matrices in, 16-bit operand copies on the
// matrix cores, fp32 accumulation, fp32 result.
//
// HipAmp mirrors the part of class CudaAmp (sentinel/NeuralNet/Cuda/CudaAmp.hpp:54-190) that
// CudaMatrix::multiplyInto goes through (Cuda/CudaMatmul.cu:413, :437): the process-wide preferMixedPrecision switch,
// the registry of fp32 master weights whose 16-bit copies stay valid until the optimizer has stepped
// (registerMasterWeight / invalidateMasterWeightHalves / clearMasterWeights, Cuda/CudaAmp.cu:140-157, :303-309,
// :326-336), the operand casts (castFloatBufferToHalf, :523-527) and the eligibility rule of
// launchCublasLtMatmulFp16 (:892-896: contraction >= 256, rows and columns >= 32; smaller products stay fp32).
// Differences, on purpose:
//  * operandType(): SENTINEL_HIP_F16 like the reference, or SENTINEL_HIP_BF16, which runs at the same matrix rate on
//    gfx950, has fp32's exponent range and so needs no loss scaling;
//  * activations are cast again for every product unless the caller opens an ActivationCastScope: the reference keeps
//    four casts keyed by source address alone (getOrCastActivationHalf, Cuda/CudaAmp.cu:55-79), which a buffer
//    rewritten in place defeats; inside a scope (the layer opens one per forward / backward call, during which no
//    cast buffer is rewritten) a tensor that feeds several products is cast once, and the layer keeps the 16-bit copies
//    of its input and of the attended matrix from the forward call for the backward call's weight-gradient products
//    (persistActivationHalf, as the reference does for its cached inputs, Cuda/CudaAmp.cu:862-869);
//  * forgetMasterWeight(): a layer that dies takes its registrations with it, so that another allocation at the same
//    address can never be served a dead weight's copy;
//  * products that accumulate into the result (beta = 1) take the 16-bit path too.
// The GEMM is rocBLAS's rocblas_gemm_ex (16-bit A and B, fp32 C, fp32 accumulation), where the reference calls
// cuBLASLt (launchCublasLtMatmulFp16Halves, Cuda/CudaAmp.cu:589-851).
#ifndef SENTINEL_HIP_HIPAMP_HPP
#define SENTINEL_HIP_HIPAMP_HPP

#include "HipFlashAttention.hpp"

#include <rocblas/rocblas.h>

#include <cstdint>

namespace sentinel_hip_host {

class HipAmp {
public:
    /// when true HipGemm::multiplyInto prefers the 16-bit matrix-core GEMM (CudaAmp::preferMixedPrecision)
    static bool& preferMixedPrecision() {
        static bool value = false;
        return value;
    }

    /// element type of the operand copies: SENTINEL_HIP_F16 (the reference's) or SENTINEL_HIP_BF16
    static int& operandType() {
        static int value = SENTINEL_HIP_F16;
        return value;
    }

    /// products that took the 16-bit path since the process started (tests and benches read it to see which path ran)
    static unsigned long long& mixedProductCount() {
        static unsigned long long value = 0;
        return value;
    }

    /// operand casts launched since the process started (weights and activations)
    static unsigned long long& castCount() {
        static unsigned long long value = 0;
        return value;
    }

    /// CudaAmp::registerMasterWeight: the 16-bit copy of this fp32 weight is made on first use and kept until
    /// invalidateMasterWeightHalves; registering again marks the copy stale
    static void registerMasterWeight(const float* deviceData, size_t elementCount) {
        if (deviceData == nullptr || elementCount == 0) return;
        for (MasterWeightHalf& entry : masterWeights()) {
            if (entry.deviceData == deviceData) {
                entry.elementCount = elementCount;
                entry.valid = false;
                return;
            }
        }
        masterWeights().emplace_back();
        masterWeights().back().deviceData = deviceData;
        masterWeights().back().elementCount = elementCount;
    }

    /// drop one registration and its copy (the buffer is about to be freed or to hold something else)
    static void forgetMasterWeight(const float* deviceData) {
        if (deviceData == nullptr) return;
        std::vector<MasterWeightHalf>& all = masterWeights();
        for (size_t i = 0; i < all.size(); ++i)
            if (all[i].deviceData == deviceData) {
                all[i] = std::move(all.back());
                all.pop_back();
                return;
            }
    }

    /// CudaAmp::invalidateMasterWeightHalves: call after the optimizer changed the weights
    static void invalidateMasterWeightHalves() {
        for (MasterWeightHalf& entry : masterWeights()) entry.valid = false;
    }

    /// CudaAmp::clearMasterWeights
    static void clearMasterWeights() {
        masterWeights().clear();
        clearActivationSlots();
    }

    /// Between construction and destruction a tensor that feeds several products is cast once. Open one only around
    /// code that does not rewrite a buffer after a product has read it (scopes do not nest: the inner one's end also
    /// ends the outer one's reuse, which costs casts, never correctness).
    class ActivationCastScope {
    public:
        ActivationCastScope() {
            clearActivationSlots();
            adoptedCopies().clear();
            scopeOpen() = true;
        }
        ~ActivationCastScope() {
            scopeOpen() = false;
            clearActivationSlots();
            adoptedCopies().clear();
        }
        ActivationCastScope(const ActivationCastScope&) = delete;
        ActivationCastScope& operator=(const ActivationCastScope&) = delete;

        /// until the scope ends, products that read `source` (elementCount fp32 values) take this 16-bit copy of it, which
        /// the caller made (persistActivationHalf) and keeps alive and current
        void adopt(const float* source, size_t elementCount, const void* half, int type) {
            if (source == nullptr || half == nullptr || elementCount == 0) return;
            adoptedCopies().push_back(AdoptedCopy{source, elementCount, half, type});
        }
    };

    /// CudaAmp::persistActivationHalf (Cuda/CudaAmp.cu:862-869): a 16-bit copy of an activation in a buffer of the
    /// caller's, e.g. kept from the forward call for the weight-gradient products of the backward call; returns the type
    /// it was cast to (operandType() at the time)
    static int persistActivationHalf(const float* source, size_t elementCount, HipDeviceBuffer& destination) {
        const int type = operandType();
        if (type != SENTINEL_HIP_F16 && type != SENTINEL_HIP_BF16)
            throw std::invalid_argument("HipAmp::operandType must be SENTINEL_HIP_F16 or SENTINEL_HIP_BF16");
        cast(source, elementCount, type, destination);
        return type;
    }

    /// the size rule of tryMultiply (CudaAmp::launchCublasLtMatmulFp16, Cuda/CudaAmp.cu:896) and the switch
    static bool wouldMultiplyMixed(size_t m, size_t n, size_t k) {
        return preferMixedPrecision() && k >= 256 && m >= 32 && n >= 32;
    }

    /// C (+)= op(A) op(B) on row-major fp32 matrices through 16-bit copies of A and B; false (nothing done) when the
    /// switch is off or the product is too small for it, the caller then multiplies in fp32. lda / ldb / ldc: floats
    /// between rows; aElements / bElements: whole operands (contiguous).
    static bool tryMultiply(rocblas_handle handle, const float* a, size_t aElements, size_t lda, bool transposeA, const float* b,
                            size_t bElements, size_t ldb, bool transposeB, float* c, size_t ldc, size_t m, size_t n, size_t k,
                            bool accumulate) {
        if (!wouldMultiplyMixed(m, n, k)) return false;
        const int type = operandType();
        if (type != SENTINEL_HIP_F16 && type != SENTINEL_HIP_BF16)
            throw std::invalid_argument("HipAmp::operandType must be SENTINEL_HIP_F16 or SENTINEL_HIP_BF16");
        const void* a16 = operand16(a, aElements, type);
        const void* b16 = operand16(b, bElements, type);
        const rocblas_datatype in = type == SENTINEL_HIP_F16 ? rocblas_datatype_f16_r : rocblas_datatype_bf16_r;
        const float alpha = 1.0f;
        const float beta = accumulate ? 1.0f : 0.0f;
        // row-major C = op(A) op(B)  <=>  column-major C^T = op(B)^T op(A)^T, each row-major matrix read as its transpose
        const rocblas_status st = rocblas_gemm_ex(
            handle, transposeB ? rocblas_operation_transpose : rocblas_operation_none,
            transposeA ? rocblas_operation_transpose : rocblas_operation_none, static_cast<rocblas_int>(n),
            static_cast<rocblas_int>(m), static_cast<rocblas_int>(k), &alpha, b16, in, static_cast<rocblas_int>(ldb), a16, in,
            static_cast<rocblas_int>(lda), &beta, c, rocblas_datatype_f32_r, static_cast<rocblas_int>(ldc), c,
            rocblas_datatype_f32_r, static_cast<rocblas_int>(ldc), rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
        if (st != rocblas_status_success) throw std::runtime_error("HipAmp rocblas_gemm_ex failed");
        ++mixedProductCount();
        return true;
    }

    /// 16-bit copy of a registered master weight (made now if stale), nullptr for anything else
    /// (CudaAmp::masterWeightHalfOrNull, Cuda/CudaAmp.cu:338-355)
    static const void* masterWeightHalfOrNull(const float* deviceData, size_t elementCount, int type) {
        if (deviceData == nullptr || elementCount == 0) return nullptr;
        for (MasterWeightHalf& entry : masterWeights()) {
            if (entry.deviceData != deviceData || entry.elementCount != elementCount) continue;
            if (!entry.valid || entry.type != type) {
                cast(deviceData, elementCount, type, entry.half);
                entry.type = type;
                entry.valid = true;
            }
            return entry.half.deviceData;
        }
        return nullptr;
    }

private:
    struct MasterWeightHalf {
        const float* deviceData = nullptr;
        size_t elementCount = 0;
        HipDeviceBuffer half;
        int type = -1;
        bool valid = false;
    };
    struct ActivationSlot {
        const float* source = nullptr;
        size_t elementCount = 0;
        int type = -1;
        HipDeviceBuffer half;
        unsigned long long lastUsed = 0;
    };
    static constexpr int activationSlotCount = 4;
    struct AdoptedCopy {
        const float* source;
        size_t elementCount;
        const void* half;
        int type;
    };
    static std::vector<AdoptedCopy>& adoptedCopies() {
        static std::vector<AdoptedCopy>* all = new std::vector<AdoptedCopy>();
        return *all;
    }

    static std::vector<MasterWeightHalf>& masterWeights() {
        // never destroyed: objects that forget their registrations in their destructors may outlive any static
        static std::vector<MasterWeightHalf>* all = new std::vector<MasterWeightHalf>();
        return *all;
    }
    static ActivationSlot* activationSlots() {
        static ActivationSlot slots[activationSlotCount];
        return slots;
    }
    static bool& scopeOpen() {
        static bool open = false;
        return open;
    }
    static void clearActivationSlots() {
        ActivationSlot* slots = activationSlots();
        for (int i = 0; i < activationSlotCount; ++i) {
            slots[i].source = nullptr;
            slots[i].elementCount = 0;
            slots[i].lastUsed = 0;
        }
    }

    static void cast(const float* source, size_t elementCount, int type, HipDeviceBuffer& destination) {
        ++castCount();
        destination.ensureCapacity(elementCount * 2);
        const int code = sentinel_hip_cast_to_16bit(source, destination.deviceData, elementCount, type,
                                                    HipFlashAttention::activeStream());
        if (code == SENTINEL_HIP_OK) return;
        const std::string message = std::string("HipAmp cast: ") + sentinel_hip_last_error();
        if (code == SENTINEL_HIP_RUNTIME) throw std::runtime_error(message);
        throw std::invalid_argument(message);
    }

    /// the 16-bit copy a product reads for this operand: a master weight's, else an activation slot's (the least recently
    /// used of four, as in the reference; found again only inside an ActivationCastScope). The products of one stream
    /// run in order, so a slot can be filled again as soon as the product that read it has been launched.
    static const void* operand16(const float* source, size_t elementCount, int type) {
        if (const void* weight = masterWeightHalfOrNull(source, elementCount, type)) return weight;
        for (const AdoptedCopy& copy : adoptedCopies())
            if (copy.source == source && copy.elementCount == elementCount && copy.type == type) return copy.half;
        static unsigned long long useCounter = 1;
        ActivationSlot* slots = activationSlots();
        if (scopeOpen())
            for (int i = 0; i < activationSlotCount; ++i)
                if (slots[i].source == source && slots[i].elementCount == elementCount && slots[i].type == type &&
                    slots[i].half.deviceData != nullptr) {
                    slots[i].lastUsed = ++useCounter;
                    return slots[i].half.deviceData;
                }
        int victim = 0;
        for (int i = 1; i < activationSlotCount; ++i)
            if (slots[i].lastUsed < slots[victim].lastUsed) victim = i;
        ActivationSlot& slot = slots[victim];
        slot.source = nullptr;  // not a valid copy of anything while the cast can still throw
        cast(source, elementCount, type, slot.half);
        slot.source = source;
        slot.elementCount = elementCount;
        slot.type = type;
        slot.lastUsed = ++useCounter;
        return slot.half.deviceData;
    }
};

}  // namespace sentinel_hip_host
#endif
