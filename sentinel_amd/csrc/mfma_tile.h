// Device helpers shared by the MFMA attention kernels (gfx950): operand types, the 32x32x16 matrix
// instruction, LDS tile staging and the cross-half wavefront exchange.
//
// Register / lane conventions used throughout (wave64, lane = 32 * g + n):
//   v_mfma_f32_32x32x16 computes D[32x32] += A[32x16] * B[16x32].
//   A operand: lane holds row n of A, contraction indices 8g .. 8g+7      (8 x 16-bit = one 128-bit read)
//   B operand: lane holds column n of B, contraction indices 8g .. 8g+7
//   D result : lane holds column n, register i (0..15) is row 8*(i/4) + 4*g + (i%4)
// Every score-like product is computed "transposed" (rows = keys, columns = queries, or the other way
// round in the key-outer kernel) so that one lane owns one softmax row: reductions over a row are
// in-register plus a single exchange between lane and lane+32.
//
// To turn a D result straight into the B operand of the next product (contraction over its rows), the
// rows are loaded in the order row_perm(): D row index m then carries matrix row
//   16*(m/16) + 8*((m/4)%2) + 4*((m/8)%2) + m%4,
// which makes registers 0..7 of lane-half g hold rows 8g..8g+7 and registers 8..15 rows 16+8g..16+8g+7:
// exactly the "contraction indices 8g..8g+7" packing of a B operand, for two consecutive k-steps.
#ifndef SENTINEL_HIP_MFMA_TILE_H
#define SENTINEL_HIP_MFMA_TILE_H

#include <hip/hip_runtime.h>

namespace sentinel_hip {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

struct Bf16 {
    typedef unsigned short storage;
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                       0, 0, 0);
    }
    static __device__ __forceinline__ unsigned pack2(float lo, float hi) {
        bf16x2_t r = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
        return __builtin_bit_cast(unsigned, r);
    }
    static __device__ __forceinline__ float lo(unsigned p) { return __builtin_bit_cast(float, p << 16); }
    static __device__ __forceinline__ float hi(unsigned p) { return __builtin_bit_cast(float, p & 0xffff0000u); }
};

struct Fp16 {
    typedef unsigned short storage;
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0,
                                                      0, 0);
    }
    static __device__ __forceinline__ unsigned pack2(float lo, float hi) {
        f16x2_t r = {static_cast<_Float16>(lo), static_cast<_Float16>(hi)};
        return __builtin_bit_cast(unsigned, r);
    }
    static __device__ __forceinline__ float lo(unsigned p) {
        return static_cast<float>(__builtin_bit_cast(f16x2_t, p)[0]);
    }
    static __device__ __forceinline__ float hi(unsigned p) {
        return static_cast<float>(__builtin_bit_cast(f16x2_t, p)[1]);
    }
};

// Matrix row carried by D row index m (see the header comment).
__device__ __forceinline__ int row_perm(int m) {
    return (m & 16) | (((m >> 2) & 1) << 3) | (((m >> 3) & 1) << 2) | (m & 3);
}

// Row (within a 32-row block) held by D register i of lane-half g when the rows were loaded through row_perm.
__device__ __forceinline__ int perm_row_of_reg(int i, int g) { return ((i >> 3) << 4) | (g << 3) | (i & 7); }

// Plain D layout row of register i.
__device__ __forceinline__ int plain_row_of_reg(int i, int g) { return ((i >> 2) << 3) | (g << 2) | (i & 3); }

// max / sum across the two lane halves (lane n <-> lane n+32); every lane gets the combined value.
// v_permlane32_swap exchanges the upper half of its first operand with the lower half of its second:
// starting from two copies of x, the first ends up holding lane n's x in lanes n and n+32, the second
// lane n+32's x in both.  Written as inline assembly because the compiler builtin returns its first
// result twice; the s_nop covers the VALU-write -> permlane-read wait states the assembler cannot see.
__device__ __forceinline__ void half_exchange(float x, float& from_low, float& from_high) {
    float a = x;
    float b = x;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    from_low = a;
    from_high = b;
}
__device__ __forceinline__ float half_max(float x) {
    float lo, hi;
    half_exchange(x, lo, hi);
    return fmaxf(lo, hi);
}
__device__ __forceinline__ float half_sum(float x) {
    float lo, hi;
    half_exchange(x, lo, hi);
    return lo + hi;
}

__device__ __forceinline__ u32x4 lds_read128(const unsigned short* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ void lds_write128(unsigned short* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }

// ---------------------------------------------------------------------------------------------
// Row-major tile: ROWS x D 16-bit elements of a [.., T, D] tensor -> registers -> LDS[row][D + 8].
// The 8-element pad makes the 128-bit operand reads of 16 consecutive rows hit 64 distinct banks.
// ---------------------------------------------------------------------------------------------
template <int ROWS, int D, int THREADS>
struct RowTile {
    static constexpr int kStride = D + 8;
    static constexpr int kChunksPerRow = D / 8;
    static constexpr int kIters = ROWS * kChunksPerRow / THREADS;
    static_assert(ROWS * kChunksPerRow % THREADS == 0, "tile must divide evenly over the workgroup");
    u32x4 regs[kIters];

    // rows >= row_limit are zero-filled
    __device__ __forceinline__ void load(const unsigned short* base, int row0, int row_limit, int tid) {
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
            const int id = it * THREADS + tid;
            const int r = id / kChunksPerRow;
            const int cc = id % kChunksPerRow;
            const int row = row0 + r;
            u32x4 x = {0u, 0u, 0u, 0u};
            if (row < row_limit) x = *reinterpret_cast<const u32x4*>(base + (long long)row * D + cc * 8);
            regs[it] = x;
        }
    }
    __device__ __forceinline__ void store(unsigned short* lds, int tid) const {
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
            const int id = it * THREADS + tid;
            const int r = id / kChunksPerRow;
            const int cc = id % kChunksPerRow;
            lds_write128(lds + r * kStride + cc * 8, regs[it]);
        }
    }
};

// ---------------------------------------------------------------------------------------------
// Transposed tile: ROWS x D elements of a [.., T, D] tensor -> LDS[c][ROWS + 8] (token-contiguous),
// the orientation needed when the contraction runs over tokens.  Each thread reads two adjacent
// columns of eight consecutive rows (one dword per row, a full wavefront covers whole rows) and
// regroups them in registers into two 8-token runs.
// ---------------------------------------------------------------------------------------------
template <int ROWS, int D, int THREADS>
struct TransposedTile {
    static constexpr int kStride = ROWS + 8;
    static constexpr int kColPairs = D / 2;
    static constexpr int kGroupsPerPass = THREADS / kColPairs;
    static constexpr int kIters = (ROWS / 8) / kGroupsPerPass;
    static_assert((ROWS / 8) % kGroupsPerPass == 0 && kIters >= 1, "tile must divide evenly over the workgroup");
    unsigned regs[kIters][8];

    __device__ __forceinline__ void load(const unsigned short* base, int row0, int row_limit, int tid) {
        const int c2 = tid % kColPairs;
        const int kg = tid / kColPairs;
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int row = row0 + (it * kGroupsPerPass + kg) * 8 + e;
                unsigned x = 0u;
                if (row < row_limit) x = *reinterpret_cast<const unsigned*>(base + (long long)row * D + 2 * c2);
                regs[it][e] = x;
            }
        }
    }
    __device__ __forceinline__ void store(unsigned short* lds, int tid) const {
        const int c2 = tid % kColPairs;
        const int kg = tid / kColPairs;
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
            u32x4 even, odd;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // {S0 = later token, S1 = earlier token}: bytes 0-3 come from S1, 4-7 from S0
                even[j] = __builtin_amdgcn_perm(regs[it][2 * j + 1], regs[it][2 * j], 0x05040100u);
                odd[j] = __builtin_amdgcn_perm(regs[it][2 * j + 1], regs[it][2 * j], 0x07060302u);
            }
            const int tok = (it * kGroupsPerPass + kg) * 8;
            lds_write128(lds + (2 * c2) * kStride + tok, even);
            lds_write128(lds + (2 * c2 + 1) * kStride + tok, odd);
        }
    }
};

}  // namespace sentinel_hip
#endif
