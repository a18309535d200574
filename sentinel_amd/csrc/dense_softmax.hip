// Masked column softmax and its backward for the dense (materialising) attention path of the layer.
//
// The layer's fallback when flash attention is switched off keeps one keys x queries fp32 score matrix per
// (head, pack): S = K^T Q from a library GEMM, then probabilities P in place, then A = V P.  The reference does this
// with one launch per step and head (CudaOps::scaleInPlace, applySparseAttentionMaskInPlace, softmaxInto;
// backward: softmaxBackwardInto, zeroForbiddenScoreGradientsInPlace, scaleInPlace;
// sentinel/NeuralNet/Cuda/CudaOps.cu:249-344, called from Cuda/CudaCausalSelfAttention.cu:272-275 and :455-457).
// Here one launch covers every matrix of a batch and fuses the three steps: the matrix is read twice and written once
// (backward: two reads of P and dP, one write), 12 B per element against 28 B for the separate passes.
//
// Layout: element (key, query) of matrix b at base[b * batch_stride + key * query_count + query].  The softmax runs
// down a column (over keys), so consecutive lanes take consecutive queries (coalesced rows) and a workgroup's four
// wavefronts split the keys of its 64 columns; the three column statistics meet in LDS.
#include "flash_common.h"

namespace sentinel_hip {
namespace {

constexpr int kColumns = 64;  // queries per workgroup = lanes of a wavefront
constexpr int kSlices = 4;    // wavefronts per workgroup, each takes every fourth key
constexpr float kMaskedScore = -1.0e9f;  // the value the reference writes over forbidden pairs (CudaOps.cu:285)

// CudaOps::runApplySparseAttentionMaskInPlace's predicate (CudaOps.cu:257-283)
__device__ __forceinline__ bool allowed_pair(int key, int query, int query_position_start, int window, int global_tokens,
                                             int segment_length) {
    int key_pos = key, query_pos = query_position_start + query;
    if (segment_length > 0) {
        if (key / segment_length != query / segment_length) return false;
        key_pos = key % segment_length;
        query_pos = query % segment_length;
    }
    if (key_pos > query_pos) return false;
    return key_pos < global_tokens || window <= 0 || key_pos >= query_pos - window + 1;
}

__global__ __launch_bounds__(kColumns* kSlices) void dense_softmax_fwd_kernel(float* scores, long long batch_stride,
                                                                               int key_count, int query_count,
                                                                               int query_position_start, int window,
                                                                               int global_tokens, int segment_length,
                                                                               float scale) {
    __shared__ float stat[kSlices][kColumns];
    const int lane = threadIdx.x % kColumns;
    const int slice = threadIdx.x / kColumns;
    const int query = blockIdx.x * kColumns + lane;
    const bool live = query < query_count;
    float* column = scores + (long long)blockIdx.y * batch_stride + (live ? query : 0);
    auto masked_score = [&](int key) {
        const float s = column[(long long)key * query_count] * scale;
        return allowed_pair(key, query, query_position_start, window, global_tokens, segment_length) ? s : kMaskedScore;
    };
    auto combine = [&](float mine, bool take_max) {
        stat[slice][lane] = mine;
        __syncthreads();
        float all = stat[0][lane];
        for (int s = 1; s < kSlices; ++s) all = take_max ? fmaxf(all, stat[s][lane]) : all + stat[s][lane];
        __syncthreads();
        return all;
    };
    float top = -__builtin_inff();
    if (live)
        for (int key = slice; key < key_count; key += kSlices) top = fmaxf(top, masked_score(key));
    top = combine(top, true);
    float sum = 0.0f;
    if (live)
        for (int key = slice; key < key_count; key += kSlices) {
            const float e = expf(masked_score(key) - top);
            column[(long long)key * query_count] = e;
            sum += e;
        }
    sum = combine(sum, false);
    const float inverse = 1.0f / sum;
    if (live)
        for (int key = slice; key < key_count; key += kSlices) column[(long long)key * query_count] *= inverse;
}

// score_gradient = scale * P * (dP - sum_keys dP * P), zero on forbidden pairs; written over dP
__global__ __launch_bounds__(kColumns* kSlices) void dense_softmax_bwd_kernel(const float* probabilities,
                                                                               long long probability_batch_stride,
                                                                               float* gradient, long long gradient_batch_stride,
                                                                               int key_count, int query_count,
                                                                               int query_position_start, int window,
                                                                               int global_tokens, int segment_length,
                                                                               float scale) {
    __shared__ float stat[kSlices][kColumns];
    const int lane = threadIdx.x % kColumns;
    const int slice = threadIdx.x / kColumns;
    const int query = blockIdx.x * kColumns + lane;
    const bool live = query < query_count;
    const float* p = probabilities + (long long)blockIdx.y * probability_batch_stride + (live ? query : 0);
    float* g = gradient + (long long)blockIdx.y * gradient_batch_stride + (live ? query : 0);
    float dot = 0.0f;
    if (live)
        for (int key = slice; key < key_count; key += kSlices) dot += g[(long long)key * query_count] * p[(long long)key * query_count];
    stat[slice][lane] = dot;
    __syncthreads();
    dot = stat[0][lane];
    for (int s = 1; s < kSlices; ++s) dot += stat[s][lane];
    if (live)
        for (int key = slice; key < key_count; key += kSlices) {
            const long long at = (long long)key * query_count;
            const bool allowed = allowed_pair(key, query, query_position_start, window, global_tokens, segment_length);
            g[at] = allowed ? p[at] * (g[at] - dot) * scale : 0.0f;
        }
}

}  // namespace

hipError_t launch_dense_softmax_fwd(float* scores, int batch, long long batch_stride, int key_count, int query_count,
                                    int query_position_start, int window, int global_tokens, int segment_length, float scale,
                                    hipStream_t stream) {
    const dim3 grid((query_count + kColumns - 1) / kColumns, batch);
    KernelTimer timer("dense_softmax_fwd", stream);
    hipLaunchKernelGGL(dense_softmax_fwd_kernel, grid, dim3(kColumns * kSlices), 0, stream, scores, batch_stride, key_count,
                       query_count, query_position_start, window, global_tokens, segment_length, scale);
    return hipGetLastError();
}

hipError_t launch_dense_softmax_bwd(const float* probabilities, long long probability_batch_stride, float* gradient,
                                    long long gradient_batch_stride, int batch, int key_count, int query_count,
                                    int query_position_start, int window, int global_tokens, int segment_length, float scale,
                                    hipStream_t stream) {
    const dim3 grid((query_count + kColumns - 1) / kColumns, batch);
    KernelTimer timer("dense_softmax_bwd", stream);
    hipLaunchKernelGGL(dense_softmax_bwd_kernel, grid, dim3(kColumns * kSlices), 0, stream, probabilities,
                       probability_batch_stride, gradient, gradient_batch_stride, key_count, query_count, query_position_start,
                       window, global_tokens, segment_length, scale);
    return hipGetLastError();
}

}  // namespace sentinel_hip
