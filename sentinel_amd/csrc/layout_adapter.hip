// Layout / type adapter between Sentinel's device layout and the MFMA kernels' layout.
//
// Sentinel keeps activations as fp32 matrices [(head * head_dim + dim), column]
// (sentinel/NeuralNet/Cuda/CudaFlashAttention.cu:129-135): the head dimension, which every attention
// product contracts over, is strided by the column count.  The MFMA kernels want [B, H, T, d] 16-bit
// with d contiguous.  These kernels transpose 64 x 64 tiles through LDS so that both the fp32 side
// (token-contiguous) and the 16-bit side (d-contiguous) are accessed with coalesced rows.
// `src` / `dst` on the column side are already advanced to the first column of pack 0.
#include "flash_common.h"
#include "mfma_tile.h"

namespace sentinel_hip {
namespace {

constexpr int kTile = 64;

template <typename E>
__global__ __launch_bounds__(256) void columns_to_bhtd_kernel(const float* __restrict__ src, unsigned short* __restrict__ dst,
                                                               int heads, int d, long long stride, int T) {
    __shared__ float tile[kTile][kTile + 1];
    const int t0 = blockIdx.x * kTile;
    const int c0 = blockIdx.y * kTile;
    const int b = blockIdx.z / heads;
    const int h = blockIdx.z % heads;
    const int tid = threadIdx.x;
    for (int i = 0; i < kTile * kTile / 256; ++i) {
        const int c = i * 4 + tid / kTile;
        const int t = tid % kTile;
        float x = 0.0f;
        if (t0 + t < T && c0 + c < d) x = src[((long long)h * d + c0 + c) * stride + (long long)b * T + t0 + t];
        tile[c][t] = x;
    }
    __syncthreads();
    for (int i = 0; i < kTile * kTile / 512; ++i) {
        const int t = i * 8 + tid / 32;
        const int c = (tid % 32) * 2;
        if (t0 + t < T && c0 + c < d) {
            const unsigned w = E::pack2(tile[c][t], tile[c + 1][t]);
            *reinterpret_cast<unsigned*>(dst + (((long long)b * heads + h) * T + t0 + t) * d + c0 + c) = w;
        }
    }
}

template <typename E>
__global__ __launch_bounds__(256) void bhtd_to_columns_kernel(const unsigned short* __restrict__ src, float* __restrict__ dst,
                                                               int heads, int d, long long stride, int T) {
    __shared__ float tile[kTile][kTile + 1];
    const int t0 = blockIdx.x * kTile;
    const int c0 = blockIdx.y * kTile;
    const int b = blockIdx.z / heads;
    const int h = blockIdx.z % heads;
    const int tid = threadIdx.x;
    for (int i = 0; i < kTile * kTile / 512; ++i) {
        const int t = i * 8 + tid / 32;
        const int c = (tid % 32) * 2;
        if (t0 + t < T && c0 + c < d) {
            const unsigned w = *reinterpret_cast<const unsigned*>(src + (((long long)b * heads + h) * T + t0 + t) * d + c0 + c);
            tile[c][t] = E::lo(w);
            tile[c + 1][t] = E::hi(w);
        }
    }
    __syncthreads();
    for (int i = 0; i < kTile * kTile / 256; ++i) {
        const int c = i * 4 + tid / kTile;
        const int t = tid % kTile;
        if (t0 + t < T && c0 + c < d) dst[((long long)h * d + c0 + c) * stride + (long long)b * T + t0 + t] = tile[c][t];
    }
}

}  // namespace

hipError_t launch_columns_to_bhtd(Elem type, const float* src, void* dst, int heads, int head_dim, int stride_columns,
                                  int seq_len, int packs, hipStream_t stream) {
    const dim3 grid((seq_len + kTile - 1) / kTile, (head_dim + kTile - 1) / kTile, packs * heads);
    auto out = static_cast<unsigned short*>(dst);
    KernelTimer timer("columns_to_bhtd", stream);
    if (type == Elem::BF16)
        hipLaunchKernelGGL(columns_to_bhtd_kernel<Bf16>, grid, dim3(256), 0, stream, src, out, heads, head_dim,
                           (long long)stride_columns, seq_len);
    else if (type == Elem::F16)
        hipLaunchKernelGGL(columns_to_bhtd_kernel<Fp16>, grid, dim3(256), 0, stream, src, out, heads, head_dim,
                           (long long)stride_columns, seq_len);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_bhtd_to_columns(Elem type, const void* src, float* dst, int heads, int head_dim, int stride_columns,
                                  int seq_len, int packs, hipStream_t stream) {
    const dim3 grid((seq_len + kTile - 1) / kTile, (head_dim + kTile - 1) / kTile, packs * heads);
    auto in = static_cast<const unsigned short*>(src);
    KernelTimer timer("bhtd_to_columns", stream);
    if (type == Elem::BF16)
        hipLaunchKernelGGL(bhtd_to_columns_kernel<Bf16>, grid, dim3(256), 0, stream, in, dst, heads, head_dim,
                           (long long)stride_columns, seq_len);
    else if (type == Elem::F16)
        hipLaunchKernelGGL(bhtd_to_columns_kernel<Fp16>, grid, dim3(256), 0, stream, in, dst, heads, head_dim,
                           (long long)stride_columns, seq_len);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

}  // namespace sentinel_hip
