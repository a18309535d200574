// Layout / type adapter between Sentinel's device layout and the MFMA kernels' layout.
//
// Sentinel keeps activations as fp32 matrices [(head * head_dim + dim), column]
// (sentinel/NeuralNet/Cuda/CudaFlashAttention.cu:129-135): the head dimension, which every attention
// product contracts over, is strided by the column count.  The MFMA kernels want [B, H, T, d] 16-bit
// with d contiguous.  These kernels transpose 64 x 64 tiles through LDS so that both the fp32 side
// (token-contiguous) and the 16-bit side (d-contiguous) are accessed with coalesced rows.
// `src` / `dst` on the column side are already advanced to the first column of pack 0.
//
// The rotary embedding that Sentinel applies to Q and K just before attention, and its inverse on dQ and dK
// just after (CudaOps::rotaryRotateInPlace / rotaryRotateInverseInPlace, Cuda/CudaOps.cu:362-402, called at
// Cuda/CudaCausalSelfAttention.cu:206-207 and :508-509), can ride on these passes: a pair (even, odd) of head
// dims is exactly the pair of values one thread packs / unpacks, so the rotation costs two table reads and no
// extra trip through memory.  The rotation is done in fp32 without fused multiply-adds, so it rounds like the
// reference's; the result is then rounded once to 16 bit.
#include "flash_common.h"
#include "mfma_tile.h"

namespace sentinel_hip {
namespace {

constexpr int kTile = 64;

// (even, odd) -> rotated pair; INVERSE rotates back (the transpose of the rotation)
template <bool INVERSE>
__device__ __forceinline__ void rotate_pair(float& even, float& odd, float c, float s) {
#pragma clang fp contract(off)
    const float e = even;
    const float o = odd;
    if (!INVERSE) {
        even = e * c - o * s;
        odd = e * s + o * c;
    } else {
        even = e * c + o * s;
        odd = -e * s + o * c;
    }
}

template <typename E>
__global__ __launch_bounds__(256) void columns_to_bhtd_kernel(const float* __restrict__ src, unsigned short* __restrict__ dst,
                                                               int heads, int d, long long stride, int T, RopeTables rope) {
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
            float even = tile[c][t];
            float odd = tile[c + 1][t];
            if (rope.cos) {
                const long long at = (long long)(rope.offset + t0 + t) * (d / 2) + (c0 + c) / 2;
                rotate_pair<false>(even, odd, rope.cos[at], rope.sin[at]);
            }
            *reinterpret_cast<unsigned*>(dst + (((long long)b * heads + h) * T + t0 + t) * d + c0 + c) = E::pack2(even, odd);
        }
    }
}

template <typename E>
__global__ __launch_bounds__(256) void bhtd_to_columns_kernel(const unsigned short* __restrict__ src, float* __restrict__ dst,
                                                               int heads, int d, long long stride, int T, RopeTables rope) {
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
            float even = E::lo(w);
            float odd = E::hi(w);
            if (rope.cos) {
                const long long at = (long long)(rope.offset + t0 + t) * (d / 2) + (c0 + c) / 2;
                rotate_pair<true>(even, odd, rope.cos[at], rope.sin[at]);
            }
            tile[c][t] = even;
            tile[c + 1][t] = odd;
        }
    }
    __syncthreads();
    for (int i = 0; i < kTile * kTile / 256; ++i) {
        const int c = i * 4 + tid / kTile;
        const int t = tid % kTile;
        if (t0 + t < T && c0 + c < d) dst[((long long)h * d + c0 + c) * stride + (long long)b * T + t0 + t] = tile[c][t];
    }
}

// In-place rotation of fp32 column-layout rows: the replacement of CudaOpsRotaryRotateEntry /
// CudaOpsRotaryRotateInverseEntry (Cuda/CudaOps.cu:362-402).  One thread per (pair row, column): both the tensor
// rows and (within a pair row) nothing else is strided; the table is read once per element and stays in L2.
template <bool INVERSE>
__global__ __launch_bounds__(256) void rope_rotate_f32_kernel(float* __restrict__ tensor, int pair_rows, int pairs,
                                                               long long stride, int columns, int position_offset,
                                                               int segment_length, const float* __restrict__ cos_table,
                                                               const float* __restrict__ sin_table) {
    const int column = blockIdx.x * 256 + threadIdx.x;
    const int pair_row = blockIdx.y;  // head * pairs + pair
    if (column >= columns || pair_row >= pair_rows) return;
    const int position = segment_length > 0 ? column % segment_length : position_offset + column;
    const long long at = (long long)position * pairs + pair_row % pairs;
    float* even_at = tensor + (long long)(2 * pair_row) * stride + column;
    float even = even_at[0];
    float odd = even_at[stride];
    rotate_pair<INVERSE>(even, odd, cos_table[at], sin_table[at]);
    even_at[0] = even;
    even_at[stride] = odd;
}

}  // namespace

hipError_t launch_rope_rotate_f32(float* tensor, int heads, int head_dim, int stride_columns, int columns,
                                  int position_offset, int segment_length, const float* cos, const float* sin, bool inverse,
                                  hipStream_t stream) {
    const int pairs = head_dim / 2;
    const dim3 grid((columns + 255) / 256, heads * pairs);
    KernelTimer timer("rope_rotate_f32", stream);
    if (inverse)
        hipLaunchKernelGGL(rope_rotate_f32_kernel<true>, grid, dim3(256), 0, stream, tensor, heads * pairs, pairs,
                           (long long)stride_columns, columns, position_offset, segment_length, cos, sin);
    else
        hipLaunchKernelGGL(rope_rotate_f32_kernel<false>, grid, dim3(256), 0, stream, tensor, heads * pairs, pairs,
                           (long long)stride_columns, columns, position_offset, segment_length, cos, sin);
    return hipGetLastError();
}

hipError_t launch_columns_to_bhtd(Elem type, const float* src, void* dst, int heads, int head_dim, int stride_columns,
                                  int seq_len, int packs, RopeTables rope, hipStream_t stream) {
    const dim3 grid((seq_len + kTile - 1) / kTile, (head_dim + kTile - 1) / kTile, packs * heads);
    auto out = static_cast<unsigned short*>(dst);
    KernelTimer timer("columns_to_bhtd", stream);
    if (type == Elem::BF16)
        hipLaunchKernelGGL(columns_to_bhtd_kernel<Bf16>, grid, dim3(256), 0, stream, src, out, heads, head_dim,
                           (long long)stride_columns, seq_len, rope);
    else if (type == Elem::F16)
        hipLaunchKernelGGL(columns_to_bhtd_kernel<Fp16>, grid, dim3(256), 0, stream, src, out, heads, head_dim,
                           (long long)stride_columns, seq_len, rope);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_bhtd_to_columns(Elem type, const void* src, float* dst, int heads, int head_dim, int stride_columns,
                                  int seq_len, int packs, RopeTables rope, hipStream_t stream) {
    const dim3 grid((seq_len + kTile - 1) / kTile, (head_dim + kTile - 1) / kTile, packs * heads);
    auto in = static_cast<const unsigned short*>(src);
    KernelTimer timer("bhtd_to_columns", stream);
    if (type == Elem::BF16)
        hipLaunchKernelGGL(bhtd_to_columns_kernel<Bf16>, grid, dim3(256), 0, stream, in, dst, heads, head_dim,
                           (long long)stride_columns, seq_len, rope);
    else if (type == Elem::F16)
        hipLaunchKernelGGL(bhtd_to_columns_kernel<Fp16>, grid, dim3(256), 0, stream, in, dst, heads, head_dim,
                           (long long)stride_columns, seq_len, rope);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

}  // namespace sentinel_hip
