// Single-query attention against an append-only K/V cache (the generation step).
//
// Replaces CudaCausalSelfAttention::attendCachedQuery (sentinel/NeuralNet/Cuda/CudaCausalSelfAttention.cu:318-341):
// there, per head, the cached K and V heads are copied out, a (length x 1) score GEMM, scale, mask, softmax and a
// (d x length)(length x 1) GEMM follow: 2 copies + 5 launches per head.  Here one launch reads the cache once:
// the cache stays in Sentinel's layout, fp32 [(head * d + dim), position] with `stride` positions per row
// (CudaKvCache, Cuda/CudaKvCache.hpp), which is position-contiguous, so lanes run along positions and every load is
// a coalesced row segment.  The work is HBM-bound (2 * kv_heads * d * length * 4 bytes for O(length * d) FLOPs)
// and, for the cache sizes of one sequence, latency-bound: the whole cache is a few dozen MB, so what counts is
// how many independent loads are in flight.  The key axis is split over workgroups (flash-decoding) and the head
// dims over the four wavefronts of a workgroup: a workgroup handles one K/V head, kChunk positions and all query
// heads of the group (grouped-query heads share the K/V reads), and leaves an unnormalised partial
// (max, sum, acc[d]) in the workspace; a second small kernel merges the partials.
#include "flash_common.h"

#include <algorithm>
#include <mutex>

namespace sentinel_hip {

// Scratch of the entry point that allocates nothing (sentinel_hip_decode_attention_static): the partial
// (max, sum, acc[d]) records of decode_partial_kernel, in device memory that exists from the moment the code object is
// loaded.  Every device the library runs on holds its own copy of the array, at its own address, until the process
// ends.  In host code the array's name is only a handle for hipGetSymbolAddress: kernels get the address it returns.
static __device__ __align__(256) float decode_static_scratch[kDecodeStaticScratchBytes / sizeof(float)];

hipError_t decode_static_scratch_address(float** address) {
    constexpr int kMaxDevices = 64;
    static std::mutex mutex;
    static float* per_device[kMaxDevices] = {};
    int device = 0;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return err;
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mutex);
    if (!per_device[device]) {  // first call on this device, with it current: ask the runtime where its copy lives
        void* found = nullptr;
        err = hipGetSymbolAddress(&found, HIP_SYMBOL(decode_static_scratch));
        if (err != hipSuccess) return err;
        if (!found) return hipErrorInvalidSymbol;
        per_device[device] = static_cast<float*>(found);
    }
    *address = per_device[device];
    return hipSuccess;
}

namespace {

constexpr int kDecodeThreads = 256;
constexpr int kChunk = 256;       // cache positions per workgroup: 64 lanes x 4 positions
constexpr int kSmallChunk = 64;   // ... x 1 position for short caches, where 256 would leave most of the chip idle
constexpr int kSmallLength = 8192;
constexpr int kWavesPerBlock = kDecodeThreads / 64;
constexpr int kLoadRows = 8;  // cache rows whose loads a wavefront issues together

template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float row_total(float x, int row) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), row * 16));
}
__device__ __forceinline__ float wave_sum(float x) {
    x += dpp_move<0xB1>(x);   // quad_perm [1,0,3,2]
    x += dpp_move<0x4E>(x);   // quad_perm [2,3,0,1]
    x += dpp_move<0x141>(x);  // row_half_mirror
    x += dpp_move<0x140>(x);  // row_mirror
    return (row_total(x, 0) + row_total(x, 1)) + (row_total(x, 2) + row_total(x, 3));
}
__device__ __forceinline__ float wave_max(float x) {
    x = fmaxf(x, dpp_move<0xB1>(x));
    x = fmaxf(x, dpp_move<0x4E>(x));
    x = fmaxf(x, dpp_move<0x141>(x));
    x = fmaxf(x, dpp_move<0x140>(x));
    return fmaxf(fmaxf(row_total(x, 0), row_total(x, 1)), fmaxf(row_total(x, 2), row_total(x, 3)));
}

// Sums N per-lane values across the wavefront at once: on return lane L holds the wavefront total of x[L % N].
// A reduce-scatter: each step halves the number of live values, lanes whose bit is clear keep the lower half of
// the values, the others the upper half (v_permlane32_swap / v_permlane16_swap across rows, row shifts inside a
// row of 16 lanes).  126 instructions for 64 sums, and the results leave as one full-width store, where 64
// separate reductions cost a few dozen instructions and a single-lane store each.  Fewer values (N < 64) leave
// lane bits over, which are summed out at the end.
__device__ __forceinline__ void swap_rows32(float& a, float& b) {  // upper 32 lanes of a <-> lower 32 lanes of b
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap_rows16(float& a, float& b) {  // odd rows of a <-> even rows of b
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
template <int SHIFT>
__device__ __forceinline__ float fold_in_row(float lower, float upper, bool take_upper) {
    // lanes with the bit clear: lower(l) + lower(l + SHIFT); lanes with it set: upper(l) + upper(l - SHIFT)
    const float a = lower + dpp_move<0x100 + SHIFT>(lower);  // row_shl: lane l reads lane l + SHIFT
    const float b = upper + dpp_move<0x110 + SHIFT>(upper);  // row_shr: lane l reads lane l - SHIFT
    return take_upper ? b : a;
}
// N = 8, 16, 32 or 64 values: lane L ends with the wavefront total of x[L % N]
template <int N>
__device__ __forceinline__ float reduce_scatter(float (&x)[N], int lane) {
    if constexpr (N == 64) {
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            swap_rows32(x[i], x[i + 32]);
            x[i] += x[i + 32];
        }
    }
    if constexpr (N >= 32) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            swap_rows16(x[i], x[i + 16]);
            x[i] += x[i + 16];
        }
    }
    if constexpr (N >= 16) {
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = fold_in_row<8>(x[i], x[i + 8], lane & 8);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) x[i] = fold_in_row<4>(x[i], x[i + 4], lane & 4);
#pragma unroll
    for (int i = 0; i < 2; ++i) x[i] = fold_in_row<2>(x[i], x[i + 2], lane & 2);
    float v = fold_in_row<1>(x[0], x[1], lane & 1);
    // lane bits that select no value: plain all-reduce across them
    if constexpr (N <= 8) v += dpp_move<0x128>(v);  // row_ror:8
    if constexpr (N <= 16) {
        float even = v, odd = v;
        swap_rows16(even, odd);  // even = rows (0, 0, 2, 2), odd = rows (1, 1, 3, 3)
        v = even + odd;
    }
    if constexpr (N <= 32) {
        float low = v, high = v;
        swap_rows32(low, high);  // low = lanes 0..31 twice, high = lanes 32..63 twice
        v = low + high;
    }
    return v;
}

// PPL cache positions of one row for this lane: positions first + {0,1,2,3} (VEC4: one aligned 16-byte load) or
// first + 64 * {0 .. PPL-1} (scalar loads, 256-byte row segments per wavefront); positions >= length read as 0
template <bool VEC4, int PPL>
__device__ __forceinline__ void load_positions(const float* row, int first, int length, float (&x)[PPL]) {
    if constexpr (VEC4) {
        static_assert(PPL == 4, "one 16-byte load per lane");
        if (first < length) {  // the row has a multiple of 4 positions, so the whole group is inside the allocation
            const float4 v = *reinterpret_cast<const float4*>(row + first);
            // positions past the used prefix hold whatever was there before: never let them into the arithmetic
            x[0] = v.x;
            x[1] = first + 1 < length ? v.y : 0.0f;
            x[2] = first + 2 < length ? v.z : 0.0f;
            x[3] = first + 3 < length ? v.w : 0.0f;
        } else {
            x[0] = x[1] = x[2] = x[3] = 0.0f;
        }
    } else {
#pragma unroll
        for (int i = 0; i < PPL; ++i) x[i] = first + 64 * i < length ? row[first + 64 * i] : 0.0f;
    }
}

// A workgroup owns kChunk positions of one K/V head; wavefront w owns head dims [w * d/4, (w + 1) * d/4).
// Scores: every wavefront forms the partial dot products of its dims for the four positions of each lane and the
// G query heads of the group (q comes through scalar loads: it is wavefront-uniform), the four partial sums meet
// in LDS, and every wavefront then holds the full scores and derives the same softmax statistics.  Output:
// acc[c] = sum_positions p * V[c][position] for the wavefront's own dims, kLoadRows x G sums reduced together.
// partial layout per (chunk, query head): [0] = max of the scaled scores, [1] = sum of exp, [2 .. 2 + d) = acc
template <int G, bool VEC4, int PPL>
__global__ __launch_bounds__(kDecodeThreads) void decode_partial_kernel(const float* __restrict__ query,
                                                                       const float* __restrict__ key_cache,
                                                                       const float* __restrict__ value_cache,
                                                                       float* __restrict__ partial, int kv_heads, int d,
                                                                       long long stride, int length, float scale,
                                                                       int global_tokens, int window_lo, int global_chunks,
                                                                       int window_chunk) {
    __shared__ float exchange[kWavesPerBlock][G * PPL][64];
    const int lane = threadIdx.x % 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    // Sparse mask of the layer (the query is position length - 1): visible are the global tokens [0, global_tokens)
    // and the window [window_lo, length).  Only chunks that hold a visible position are launched: the first
    // global_chunks ones and those from window_chunk on; partials are numbered by workgroup.
    const int slot = blockIdx.x;
    const int chunk = slot < global_chunks ? slot : slot - global_chunks + window_chunk;
    const int kvh = blockIdx.y;
    const int q_heads = kv_heads * G;
    const int first = chunk * (64 * PPL) + (VEC4 ? 4 * lane : lane);
    const int rows = d / kWavesPerBlock;
    const int r0 = wave * rows, r1 = r0 + rows;

    float s[PPL][G];
#pragma unroll
    for (int i = 0; i < PPL; ++i)
#pragma unroll
        for (int g = 0; g < G; ++g) s[i][g] = 0.0f;
    const float* krow = key_cache + (long long)kvh * d * stride;
    const float* qrow = query + (long long)kvh * G * d;
    for (int c0 = r0; c0 < r1; c0 += kLoadRows) {
        float kv[kLoadRows][PPL];
#pragma unroll
        for (int u = 0; u < kLoadRows; ++u) {
            if (c0 + u < r1) {  // wavefront-uniform
                load_positions<VEC4, PPL>(krow + (long long)(c0 + u) * stride, first, length, kv[u]);
            } else {
                for (int i = 0; i < PPL; ++i) kv[u][i] = 0.0f;
            }
        }
#pragma unroll
        for (int u = 0; u < kLoadRows; ++u)
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const float qc = c0 + u < r1 ? qrow[g * d + c0 + u] : 0.0f;
#pragma unroll
                for (int i = 0; i < PPL; ++i) s[i][g] = __builtin_fmaf(qc, kv[u][i], s[i][g]);
            }
    }
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int i = 0; i < PPL; ++i) exchange[wave][g * PPL + i][lane] = s[i][g];
    __syncthreads();
    float p[PPL][G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float m = -__builtin_inff();
#pragma unroll
        for (int i = 0; i < PPL; ++i) {
            // the same order of additions in every wavefront: all four derive identical statistics
            const float dot = (exchange[0][g * PPL + i][lane] + exchange[1][g * PPL + i][lane]) +
                              (exchange[2][g * PPL + i][lane] + exchange[3][g * PPL + i][lane]);
            const int j = first + (VEC4 ? i : 64 * i);
            s[i][g] = (j < length && (j < global_tokens || j >= window_lo)) ? dot * scale : -__builtin_inff();
            m = fmaxf(m, s[i][g]);
        }
        m = wave_max(m);  // finite: the chunk holds at least one visible position
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < PPL; ++i) {
            p[i][g] = __expf(s[i][g] - m);
            sum += p[i][g];
        }
        sum = wave_sum(sum);
        if (wave == 0 && lane == 0) {
            float* out = partial + ((long long)slot * q_heads + kvh * G + g) * (d + 2);
            out[0] = m;
            out[1] = sum;
        }
    }
    const float* vrow = value_cache + (long long)kvh * d * stride;
    for (int c0 = r0; c0 < r1; c0 += kLoadRows) {
        float vv[kLoadRows][PPL];
#pragma unroll
        for (int u = 0; u < kLoadRows; ++u) {
            if (c0 + u < r1) {
                load_positions<VEC4, PPL>(vrow + (long long)(c0 + u) * stride, first, length, vv[u]);
            } else {
                for (int i = 0; i < PPL; ++i) vv[u][i] = 0.0f;
            }
        }
        float x[kLoadRows * G];
#pragma unroll
        for (int u = 0; u < kLoadRows; ++u)
#pragma unroll
            for (int g = 0; g < G; ++g) {
                float acc = 0.0f;
#pragma unroll
                for (int i = 0; i < PPL; ++i) acc = __builtin_fmaf(p[i][g], vv[u][i], acc);  // p = 0 past the end
                x[u * G + g] = acc;
            }
        // lane L now holds the total with index L % (kLoadRows * G) = (row in batch) * G + head
        const float total = reduce_scatter<kLoadRows * G>(x, lane);
        const int c = c0 + lane / G;
        if (lane < kLoadRows * G && c < r1) partial[((long long)slot * q_heads + kvh * G + lane % G) * (d + 2) + 2 + c] = total;
    }
}

// out[h][c] = sum_chunks e^(m - M) acc[c] / sum_chunks e^(m - M) l.  One workgroup per (head, 32 head dims):
// 8 slices of the chunk list x 32 dims, the slices meet in LDS.
__global__ __launch_bounds__(256) void decode_merge_kernel(const float* __restrict__ partial, float* __restrict__ out,
                                                           int q_heads, int d, int chunks) {
    __shared__ float tops[4];
    __shared__ float denoms[4];
    __shared__ float sums[8][32];
    const int h = blockIdx.x;
    const int lane = threadIdx.x % 64;
    const int wave = threadIdx.x / 64;
    const long long step = (long long)q_heads * (d + 2);
    const float* base = partial + (long long)h * (d + 2);
    float top = -__builtin_inff();
    for (int s = threadIdx.x; s < chunks; s += 256) top = fmaxf(top, base[s * step]);
    top = wave_max(top);
    if (lane == 0) tops[wave] = top;
    __syncthreads();
    top = fmaxf(fmaxf(tops[0], tops[1]), fmaxf(tops[2], tops[3]));
    float denom = 0.0f;
    for (int s = threadIdx.x; s < chunks; s += 256) denom += __expf(base[s * step] - top) * base[s * step + 1];
    denom = wave_sum(denom);
    if (lane == 0) denoms[wave] = denom;
    const int col = blockIdx.y * 32 + threadIdx.x % 32;
    const int slice = threadIdx.x / 32;
    float acc = 0.0f;
    if (col < d) {
#pragma unroll 4
        for (int s = slice; s < chunks; s += 8) acc += __expf(base[s * step] - top) * base[s * step + 2 + col];
    }
    sums[slice][threadIdx.x % 32] = acc;
    __syncthreads();
    if (slice == 0 && col < d) {
        const int c = threadIdx.x;
        const float total = ((sums[0][c] + sums[1][c]) + (sums[2][c] + sums[3][c])) + ((sums[4][c] + sums[5][c]) + (sums[6][c] + sums[7][c]));
        out[(long long)h * d + col] = total / ((denoms[0] + denoms[1]) + (denoms[2] + denoms[3]));
    }
}

}  // namespace

static int decode_chunk(int length) { return length <= kSmallLength ? kSmallChunk : kChunk; }

size_t decode_workspace_bytes(int q_heads, int head_dim, int length) {
    const int chunk = decode_chunk(length);
    const size_t chunks = (static_cast<size_t>(length) + chunk - 1) / chunk;
    return chunks * static_cast<size_t>(q_heads) * (head_dim + 2) * sizeof(float);
}

hipError_t launch_decode_attention(const float* query, const float* key_cache, const float* value_cache, float* out,
                                   int q_heads, int kv_heads, int head_dim, int stride, int length, float scale,
                                   int window, int global_tokens, float* workspace, hipStream_t stream) {
    const int chunk = decode_chunk(length);
    const int all_chunks = (length + chunk - 1) / chunk;
    // window <= 0 or >= length: every position is visible
    const bool sparse = window > 0 && window < length;
    const int window_lo = sparse ? length - window : 0;
    if (!sparse) global_tokens = 0;
    const int global_chunks = sparse ? (std::min(global_tokens, window_lo) + chunk - 1) / chunk : 0;
    const int window_chunk = std::max(global_chunks, window_lo / chunk);
    const int chunks = global_chunks + (all_chunks - window_chunk);
    const int group = q_heads / kv_heads;
    if (head_dim % 8 != 0) return hipErrorInvalidValue;
    const dim3 grid(chunks, kv_heads);
    // aligned 16-byte row loads need every row start 16-byte aligned
    const bool v4 = stride % 4 == 0 && ((reinterpret_cast<uintptr_t>(key_cache) | reinterpret_cast<uintptr_t>(value_cache)) & 15u) == 0;
    {
        KernelTimer timer("decode_partial", stream);
#define SENTINEL_DECODE(G)                                                                                                   \
    do {                                                                                                                     \
        if (chunk == kSmallChunk)                                                                                            \
            hipLaunchKernelGGL((decode_partial_kernel<G, false, 1>), grid, dim3(kDecodeThreads), 0, stream, query,           \
                               key_cache, value_cache, workspace, kv_heads, head_dim, (long long)stride, length, scale,      \
                               global_tokens, window_lo, global_chunks, window_chunk);                                       \
        else if (v4)                                                                                                         \
            hipLaunchKernelGGL((decode_partial_kernel<G, true, 4>), grid, dim3(kDecodeThreads), 0, stream, query,            \
                               key_cache, value_cache, workspace, kv_heads, head_dim, (long long)stride, length, scale,      \
                               global_tokens, window_lo, global_chunks, window_chunk);                                       \
        else                                                                                                                 \
            hipLaunchKernelGGL((decode_partial_kernel<G, false, 4>), grid, dim3(kDecodeThreads), 0, stream, query,           \
                               key_cache, value_cache, workspace, kv_heads, head_dim, (long long)stride, length, scale,      \
                               global_tokens, window_lo, global_chunks, window_chunk);                                       \
    } while (0)
        if (group == 1) SENTINEL_DECODE(1);
        else if (group == 2) SENTINEL_DECODE(2);
        else if (group == 4) SENTINEL_DECODE(4);
        else if (group == 8) SENTINEL_DECODE(8);
        else return hipErrorInvalidValue;
#undef SENTINEL_DECODE
        const hipError_t err = hipGetLastError();
        if (err != hipSuccess) return err;
    }
    KernelTimer timer("decode_merge", stream);
    hipLaunchKernelGGL(decode_merge_kernel, dim3(q_heads, (head_dim + 31) / 32), dim3(256), 0, stream, workspace, out, q_heads,
                       head_dim, chunks);
    return hipGetLastError();
}

}  // namespace sentinel_hip
