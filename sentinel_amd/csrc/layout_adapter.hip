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

// Tile = 64 head dims x 64 tokens, kept in LDS as tile[dim][token] with a row stride of 65 floats: the
// token-major side (fp32, 4 tokens per thread) and the dim-major side (16 bit, 8 dims = 16 bytes per thread)
// both touch 64 different banks per wavefront access.  VEC4: the fp32 rows can be accessed as aligned float4
// (pointer, stride and sequence length all multiples of 4 floats); otherwise the same code runs on scalars.
// The 16-bit side may be wider than the fp32 side (d_out > d, both multiples of 8): head dims the MFMA kernels have no
// tiling for are padded with zeros to the next one they have, which changes no product.
// Up to kMaxConvertJobs tensors of one call (Q, K, V; or Q, O, K, V, dO) go through one launch: at the sequence lengths
// Sentinel trains with a conversion takes about as long as its launch, and three to five of them were 40 % of a step.
// grid.z runs over the (pack, head) pairs of all jobs one after the other; z_end is the running total.
template <typename E, bool VEC4>
__global__ __launch_bounds__(256) void columns_to_bhtd_kernel(ConvertJobs jobs, int d, int d_out, long long stride, int T,
                                                               RopeTables tables) {
    __shared__ float tile[kTile][kTile + 1];
    const int t0 = blockIdx.x * kTile;
    const int c0 = blockIdx.y * kTile;
    int job = 0, z = blockIdx.z;
    while (job + 1 < jobs.count && (int)blockIdx.z >= jobs.job[job].z_end) ++job;
    if (job > 0) z -= jobs.job[job - 1].z_end;
    const float* __restrict__ src = jobs.job[job].src;
    unsigned short* __restrict__ dst = jobs.job[job].dst;
    const int heads = jobs.job[job].heads;
    RopeTables rope = tables;
    if (!jobs.job[job].rotate) rope.cos = nullptr;
    const int b = z / heads;
    const int h = z % heads;
    const int tid = threadIdx.x;
    {
        const int t4 = (tid % 16) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = i * 16 + tid / 16;
            float x[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if (c0 + c < d) {
                const float* at = src + ((long long)h * d + c0 + c) * stride + (long long)b * T + t0 + t4;
                if (VEC4) {
                    if (t0 + t4 < T) {
                        const float4 v = *reinterpret_cast<const float4*>(at);
                        x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (t0 + t4 + e < T) x[e] = at[e];
                }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) tile[c][t4 + e] = x[e];
        }
    }
    __syncthreads();
    const int c8 = (tid % 8) * 8;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int t = i * 32 + tid / 8;
        if (t0 + t < T && c0 + c8 < d_out) {  // head dims [d, d_out) are written as zeros (the load phase left them zero)
            float x[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = tile[c8 + e][t];
            if (rope.cos && c0 + c8 < d) {
                const long long at = (long long)(rope.offset + t0 + t) * (d / 2) + (c0 + c8) / 2;
                const float4 c = *reinterpret_cast<const float4*>(rope.cos + at);
                const float4 sn = *reinterpret_cast<const float4*>(rope.sin + at);
                rotate_pair<false>(x[0], x[1], c.x, sn.x);
                rotate_pair<false>(x[2], x[3], c.y, sn.y);
                rotate_pair<false>(x[4], x[5], c.z, sn.z);
                rotate_pair<false>(x[6], x[7], c.w, sn.w);
            }
            u32x4 w;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = E::pack2(x[2 * e], x[2 * e + 1]);
            *reinterpret_cast<u32x4*>(dst + (((long long)b * heads + h) * T + t0 + t) * d_out + c0 + c8) = w;
        }
    }
}

template <typename E, bool VEC4>
__global__ __launch_bounds__(256) void bhtd_to_columns_kernel(const unsigned short* __restrict__ src, float* __restrict__ dst,
                                                               int heads, int d, int d_in, long long stride, int T,
                                                               RopeTables rope) {
    __shared__ float tile[kTile][kTile + 1];
    const int t0 = blockIdx.x * kTile;
    const int c0 = blockIdx.y * kTile;
    const int b = blockIdx.z / heads;
    const int h = blockIdx.z % heads;
    const int tid = threadIdx.x;
    const int c8 = (tid % 8) * 8;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int t = i * 32 + tid / 8;
        if (t0 + t < T && c0 + c8 < d) {
            const u32x4 w = *reinterpret_cast<const u32x4*>(src + (((long long)b * heads + h) * T + t0 + t) * d_in + c0 + c8);
            float x[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                x[2 * e] = E::lo(w[e]);
                x[2 * e + 1] = E::hi(w[e]);
            }
            if (rope.cos) {
                const long long at = (long long)(rope.offset + t0 + t) * (d / 2) + (c0 + c8) / 2;
                const float4 c = *reinterpret_cast<const float4*>(rope.cos + at);
                const float4 sn = *reinterpret_cast<const float4*>(rope.sin + at);
                rotate_pair<true>(x[0], x[1], c.x, sn.x);
                rotate_pair<true>(x[2], x[3], c.y, sn.y);
                rotate_pair<true>(x[4], x[5], c.z, sn.z);
                rotate_pair<true>(x[6], x[7], c.w, sn.w);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) tile[c8 + e][t] = x[e];
        }
    }
    __syncthreads();
    const int t4 = (tid % 16) * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = i * 16 + tid / 16;
        if (c0 + c >= d) continue;
        float* at = dst + ((long long)h * d + c0 + c) * stride + (long long)b * T + t0 + t4;
        if (VEC4) {
            if (t0 + t4 < T) *reinterpret_cast<float4*>(at) = make_float4(tile[c][t4], tile[c][t4 + 1], tile[c][t4 + 2], tile[c][t4 + 3]);
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (t0 + t4 + e < T) at[e] = tile[c][t4 + e];
        }
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

// Flat fp32 -> 16-bit cast (round to nearest even; fp16 values beyond its range become infinities, like the conversion
// instruction gives them): the operands of the layer's mixed-precision projection GEMMs.  WIDE: both pointers 16-byte
// aligned, eight values per thread and trip (two 16-byte loads, one 16-byte store); the count's last values, fewer than
// eight, go one per thread through the first workgroup.
template <typename E, bool WIDE>
__global__ __launch_bounds__(256) void cast_f32_to_16bit_kernel(const float* __restrict__ src,
                                                                 unsigned short* __restrict__ dst, size_t count) {
    const size_t first = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t step = (size_t)gridDim.x * 256;
    if (WIDE) {
        const size_t groups = count / 8;
        for (size_t i = first; i < groups; i += step) {
            const float4 a = reinterpret_cast<const float4*>(src)[2 * i];
            const float4 b = reinterpret_cast<const float4*>(src)[2 * i + 1];
            const u32x4 r = {E::pack2(a.x, a.y), E::pack2(a.z, a.w), E::pack2(b.x, b.y), E::pack2(b.z, b.w)};
            reinterpret_cast<u32x4*>(dst)[i] = r;
        }
        const size_t at = groups * 8 + first;
        if (first < 8 && at < count) dst[at] = (unsigned short)(E::pack2(src[at], 0.0f) & 0xffffu);
    } else {
        for (size_t i = first; i < count; i += step) dst[i] = (unsigned short)(E::pack2(src[i], 0.0f) & 0xffffu);
    }
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

// fp32 rows can be read / written as aligned float4
static bool rows_vec4(const void* base, int stride_columns, int seq_len) {
    return (reinterpret_cast<uintptr_t>(base) & 15u) == 0 && stride_columns % 4 == 0 && seq_len % 4 == 0;
}

hipError_t launch_columns_to_bhtd_jobs(Elem type, ConvertJobs jobs, int head_dim, int stride_columns, int seq_len, int packs,
                                       RopeTables rope, hipStream_t stream, int padded_dim) {
    if (padded_dim <= 0) padded_dim = head_dim;
    if (jobs.count <= 0 || jobs.count > kMaxConvertJobs || head_dim % 8 != 0 || padded_dim % 8 != 0 || padded_dim < head_dim)
        return hipErrorInvalidValue;
    bool v4 = true;
    long long z = 0;
    for (int i = 0; i < jobs.count; ++i) {
        v4 = v4 && rows_vec4(jobs.job[i].src, stride_columns, seq_len);
        z += (long long)packs * jobs.job[i].heads;
        jobs.job[i].z_end = (int)z;
    }
    if (z > 65535) {  // more (pack, head) pairs than a grid has rows: one launch per tensor
        for (int i = 0; i < jobs.count; ++i) {
            ConvertJobs one;
            one.count = 1;
            one.job[0] = jobs.job[i];
            if ((long long)packs * one.job[0].heads > 65535) return hipErrorInvalidValue;
            const hipError_t err = launch_columns_to_bhtd_jobs(type, one, head_dim, stride_columns, seq_len, packs, rope, stream,
                                                               padded_dim);
            if (err != hipSuccess) return err;
        }
        return hipSuccess;
    }
    const dim3 grid((seq_len + kTile - 1) / kTile, (padded_dim + kTile - 1) / kTile, (unsigned)z);
    KernelTimer timer("columns_to_bhtd", stream);
#define SENTINEL_LAUNCH(E, V) \
    hipLaunchKernelGGL((columns_to_bhtd_kernel<E, V>), grid, dim3(256), 0, stream, jobs, head_dim, padded_dim, \
                       (long long)stride_columns, seq_len, rope)
    if (type == Elem::BF16) {
        if (v4) SENTINEL_LAUNCH(Bf16, true); else SENTINEL_LAUNCH(Bf16, false);
    } else if (type == Elem::F16) {
        if (v4) SENTINEL_LAUNCH(Fp16, true); else SENTINEL_LAUNCH(Fp16, false);
    } else {
        return hipErrorInvalidValue;
    }
#undef SENTINEL_LAUNCH
    return hipGetLastError();
}

hipError_t launch_columns_to_bhtd(Elem type, const float* src, void* dst, int heads, int head_dim, int stride_columns,
                                  int seq_len, int packs, RopeTables rope, hipStream_t stream, int padded_dim) {
    ConvertJobs jobs;
    jobs.count = 1;
    jobs.job[0] = ConvertJob{src, static_cast<unsigned short*>(dst), heads, rope.cos != nullptr, 0};
    return launch_columns_to_bhtd_jobs(type, jobs, head_dim, stride_columns, seq_len, packs, rope, stream, padded_dim);
}

hipError_t launch_bhtd_to_columns(Elem type, const void* src, float* dst, int heads, int head_dim, int stride_columns,
                                  int seq_len, int packs, RopeTables rope, hipStream_t stream, int padded_dim) {
    if (padded_dim <= 0) padded_dim = head_dim;
    const dim3 grid((seq_len + kTile - 1) / kTile, (head_dim + kTile - 1) / kTile, packs * heads);
    auto in = static_cast<const unsigned short*>(src);
    if (head_dim % 8 != 0 || padded_dim % 8 != 0 || padded_dim < head_dim) return hipErrorInvalidValue;
    const bool v4 = rows_vec4(dst, stride_columns, seq_len);
    KernelTimer timer("bhtd_to_columns", stream);
#define SENTINEL_LAUNCH(E, V) \
    hipLaunchKernelGGL((bhtd_to_columns_kernel<E, V>), grid, dim3(256), 0, stream, in, dst, heads, head_dim, padded_dim, \
                       (long long)stride_columns, seq_len, rope)
    if (type == Elem::BF16) {
        if (v4) SENTINEL_LAUNCH(Bf16, true); else SENTINEL_LAUNCH(Bf16, false);
    } else if (type == Elem::F16) {
        if (v4) SENTINEL_LAUNCH(Fp16, true); else SENTINEL_LAUNCH(Fp16, false);
    } else {
        return hipErrorInvalidValue;
    }
#undef SENTINEL_LAUNCH
    return hipGetLastError();
}

hipError_t launch_cast_f32_to_16bit(Elem type, const float* src, void* dst, size_t count, hipStream_t stream) {
    if (count == 0) return hipSuccess;
    const bool wide = ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) == 0;
    const size_t per_thread = wide ? 8 : 1;
    const size_t wanted = (count + 256 * per_thread - 1) / (256 * per_thread);
    const dim3 grid((unsigned)(wanted < 8192 ? wanted : 8192));  // grid-stride beyond 16 M values
    auto out = static_cast<unsigned short*>(dst);
    KernelTimer timer("cast_f32_to_16bit", stream);
#define SENTINEL_LAUNCH(E, W) hipLaunchKernelGGL((cast_f32_to_16bit_kernel<E, W>), grid, dim3(256), 0, stream, src, out, count)
    if (type == Elem::BF16) {
        if (wide) SENTINEL_LAUNCH(Bf16, true); else SENTINEL_LAUNCH(Bf16, false);
    } else if (type == Elem::F16) {
        if (wide) SENTINEL_LAUNCH(Fp16, true); else SENTINEL_LAUNCH(Fp16, false);
    } else {
        return hipErrorInvalidValue;
    }
#undef SENTINEL_LAUNCH
    return hipGetLastError();
}

}  // namespace sentinel_hip
