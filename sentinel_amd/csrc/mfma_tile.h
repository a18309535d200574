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
// rows of the first product are loaded in the order row_perm(): D row index m then carries matrix row
// row_perm(m), chosen so that registers 0..7 of lane-half g hold rows 2g + {0,4,8,12,1,5,9,13} and registers
// 8..15 the same rows + 16: the packing of a B operand for two consecutive k-steps whose contraction
// index (g, e) stands for row 2g + rho(e), rho = {0,4,8,12,1,5,9,13}.  The matching A operand of the
// second product is read with two transposing LDS reads, each fetching four rows that lie four apart
// (lds_read_transposed).  Rows four apart is what makes the 32 lanes that the LDS serves per cycle hit 64
// different banks, with the 8-element row pad that also suits the 128-bit row reads (which only need the
// 16 rows of a lane group to be 16 different rows) as well as with the XOR-swizzled unpadded layout.
#ifndef SENTINEL_HIP_MFMA_TILE_H
#define SENTINEL_HIP_MFMA_TILE_H

#include <hip/hip_runtime.h>

#include "grid_plan.h"

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

// Matrix row carried by D row index m = 8a + 4g + r (see the header comment): 16*(a/2) + 4r + 2g + a%2.
__device__ __forceinline__ int row_perm(int m) {
    return (m & 16) | ((m & 3) << 2) | (((m >> 2) & 1) << 1) | ((m >> 3) & 1);
}

// Row (within a 32-row block) held by D register i of lane-half g when the rows were loaded through row_perm.
__device__ __forceinline__ int perm_row_of_reg(int i, int g) {
    return ((i >> 3) << 4) | ((i & 3) << 2) | (g << 1) | ((i >> 2) & 1);
}

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

// Makes a register value opaque at this point of the program: a global load feeding it must have been
// issued and waited for before here.  Used on operand fragments that are loaded once and consumed inside
// a loop: without it the compiler sinks the loads next to the loop and then guards their first use with
// vmcnt waits that, on every later trip, drain the prefetch loads issued at the top of the same trip.
__device__ __forceinline__ void pin_loaded(u32x4& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ void pin_loaded(float& x) { asm volatile("" : "+v"(x)); }

__device__ __forceinline__ u32x4 lds_read128(const unsigned short* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ void lds_write128(unsigned short* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }

// ---------------------------------------------------------------------------------------------
// Global -> LDS staging of a ROWS x D tile of 16-bit elements out of a row-major [T, D] head.
//
// Loads are raw buffer loads: the resource describes exactly one head (T * D * 2 bytes), the per-thread
// byte offset inside a tile is a loop-invariant VGPR and the tile's position is one SGPR, so walking the
// sequence costs no vector address arithmetic and rows past T come back as zeros from the hardware's
// range check (no branches).  LDS rows are padded by PAD elements.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_head_rsrc(const unsigned short* base, long long bytes) {
    const int limit = bytes > 0x7fffffffLL ? 0x7fffffff : (int)bytes;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned short*>(base), 0, limit, 0x00020000);
}

template <int ROWS, int D, int THREADS, int PAD>
struct RowTile {
    static constexpr int kStride = D + PAD;
    static constexpr int kChunksPerRow = D / 8;
    static constexpr int kIters = ROWS * kChunksPerRow / THREADS;
    static constexpr int kRowsPerIter = THREADS / kChunksPerRow;
    static_assert(ROWS * kChunksPerRow % THREADS == 0, "tile must divide evenly over the workgroup");
    u32x4 regs[kIters];

    // byte offset of this thread's first chunk inside a tile / element offset of its LDS slot
    static __device__ __forceinline__ int global_offset(int tid) { return ((tid / kChunksPerRow) * D + (tid % kChunksPerRow) * 8) * 2; }
    static __device__ __forceinline__ int lds_offset(int tid) { return (tid / kChunksPerRow) * kStride + (tid % kChunksPerRow) * 8; }

    // tile_bytes = first row of the tile * D * 2 (wavefront-uniform)
    __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t rsrc, int thread_offset, int tile_bytes) {
#pragma unroll
        for (int it = 0; it < kIters; ++it)
            regs[it] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, thread_offset + it * kRowsPerIter * D * 2, tile_bytes, 0);
    }
    __device__ __forceinline__ void store(unsigned short* lds, int thread_lds_offset) const {
#pragma unroll
        for (int it = 0; it < kIters; ++it) lds_write128(lds + thread_lds_offset + it * kRowsPerIter * kStride, regs[it]);
    }
};

// ---------------------------------------------------------------------------------------------
// A operand whose contraction runs over the ROWS (tokens) of a row-major LDS tile: the transposed view
// tile^T[col][token], read with ds_read_b64_tr_b16.  Within a 16-lane group that instruction returns to
// lane i the 4 x 16-bit values {element i%4 of the 8 bytes addressed by lane 4j + i/4, j = 0..3}; with
// lane i addressing tile[t0 + 4*(i/4)][c0 + 4*(i%4) ..] lane i therefore receives
// tile[t0 + {0,4,8,12}][c0 + i]: four tokens of one column; a second read one row further gives the
// next four.  Together: contraction elements e = 0..7 of this lane-half = tokens t0 + rho(e).
//   lane groups: lanes 0-15 -> columns c0..c0+15, lanes 16-31 -> c0+16..c0+31 (operand rows n = lane % 32),
//   lanes 32-63 the same columns for the second half of the contraction (tokens + 2).
// ---------------------------------------------------------------------------------------------
typedef short s16x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int transposed_read_offset(int lane, int stride) {
    const int i = lane & 15;
    const int column_block = (lane >> 4) & 1;
    const int gh = lane >> 5;
    return (gh * 2 + 4 * (i >> 2)) * stride + column_block * 16 + 4 * (i & 3);
}

// tile_at = tile + transposed_read_offset + t0 * stride + c0
__device__ __forceinline__ u32x4 lds_read_transposed(const unsigned short* tile_at, int stride) {
    typedef s16x4_t __attribute__((address_space(3))) * lds_ptr;
    const s16x4_t even = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(tile_at));           // tokens rho(0..3)
    const s16x4_t odd = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(tile_at + stride));  // tokens rho(4..7)
    const u32x2 a = __builtin_bit_cast(u32x2, even);
    const u32x2 b = __builtin_bit_cast(u32x2, odd);
    u32x4 r = {a[0], a[1], b[0], b[1]};
    return r;
}

// ---------------------------------------------------------------------------------------------
// Global -> LDS without passing through registers (buffer_load ... lds): each lane's 16 bytes land at
// tile + 16 * (chunk index) in issue order, so the tile is unpadded; bank conflicts are avoided by an XOR
// swizzle instead: the 16-byte chunk c of row r is kept at chunk position c ^ (r mod chunks_per_row),
// which is applied on the global side (each lane fetches the chunk that belongs at its position).
// Both operand read patterns stay conflict-free: 16 different rows (mod 16) of one logical chunk hit 16
// different positions, and the four rows (four apart) times four chunks of a transposed read likewise.
// ---------------------------------------------------------------------------------------------
template <int ROWS, int D, int THREADS>
struct DirectTile {
    static constexpr int kChunksPerRow = D / 8;
    static constexpr int kMask = kChunksPerRow - 1;
    static constexpr int kIters = ROWS * kChunksPerRow / THREADS;
    static constexpr int kRowsPerIter = THREADS / kChunksPerRow;
    static constexpr int kElems = ROWS * D;
    static_assert(ROWS * kChunksPerRow % THREADS == 0 && kRowsPerIter % kChunksPerRow == 0, "tile / swizzle period mismatch");

    // byte offset (inside a tile of the head) of the chunk this thread fetches in pass 0
    static __device__ __forceinline__ int global_offset(int tid) {
        const int row = tid / kChunksPerRow;
        const int pos = tid % kChunksPerRow;
        return (row * D + ((pos ^ (row & kMask)) << 3)) * 2;
    }
    // tile_bytes = first row of the tile * D * 2; wave = wavefront index in the workgroup (both uniform)
    static __device__ __forceinline__ void issue(__amdgpu_buffer_rsrc_t rsrc, unsigned short* lds_tile, int thread_offset,
                                                 int tile_bytes, int wave) {
        typedef __attribute__((address_space(3))) void* lds_void;
#pragma unroll
        for (int it = 0; it < kIters; ++it)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void)(lds_tile + (it * THREADS + wave * 64) * 8), 16,
                                                     thread_offset + it * kRowsPerIter * D * 2, tile_bytes, 0, 0);
    }
    // element offset of this lane's 128-bit operand read of row `row` (k-step 0): xor (ks << 4) selects k-step ks
    static __device__ __forceinline__ int row_read_base(int row, int gh) { return row * D + ((gh ^ (row & kMask)) << 3); }
    // element offsets of this lane's two transposed reads (tokens rho(0..3) / rho(4..7)) for token block 0, column block 0:
    // add t0 * D for the token block (t0 a multiple of 16), xor (cb << 5) for column block cb
    static __device__ __forceinline__ int transposed_read_base(int lane, int odd) {
        const int i = lane & 15;
        const int r = (lane >> 5) * 2 + 4 * (i >> 2) + odd;
        const int chunk = ((lane >> 4) & 1) * 2 + ((i & 3) >> 1);
        return r * D + ((chunk ^ (r & kMask)) << 3) + 4 * (i & 1);
    }
};

__device__ __forceinline__ u32x4 lds_read_transposed_pair(const unsigned short* even_at, const unsigned short* odd_at) {
    typedef s16x4_t __attribute__((address_space(3))) * lds_ptr;
    const s16x4_t even = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(even_at));
    const s16x4_t odd = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(odd_at));
    const u32x2 a = __builtin_bit_cast(u32x2, even);
    const u32x2 b = __builtin_bit_cast(u32x2, odd);
    u32x4 r = {a[0], a[1], b[0], b[1]};
    return r;
}


// Two workgroups share a compute unit, one wavefront of each per SIMD, and the hardware issues the older wavefront first
// whenever both are ready: the workgroup that arrived first runs about 1.6 times as fast as the other and finishes its
// tiles early, after which the compute unit is half empty.  Taking turns at the higher priority (the turn changes every
// 2^13 ticks of the constant 100 MHz clock, 82 us; which of the two starts is decided by the wavefront's slot on its SIMD)
// evens the two out, so all workgroups of the persistent grid finish together.
__device__ __forceinline__ unsigned priority_turn_class() {
    return __builtin_amdgcn_s_getreg((3 << 11) | 4) & 1u;  // HW_ID.wave_id, bit 0
}
__device__ __forceinline__ void take_priority_turn(unsigned realtime, unsigned turn_class) {
    if (((realtime >> 13) ^ turn_class) & 1u)
        __builtin_amdgcn_s_setprio(1);
    else
        __builtin_amdgcn_s_setprio(0);
}

// Writes a wavefront's 32 x D block of 16-bit results to 32 consecutive global rows of D elements.  The block is held as
// transposed accumulators: lane (n, gh) owns row n, elements cb*32 + a*8 + gh*4 + [0, 4) in acc[cb][a*4 + ...].  Stored
// straight from there, one instruction would write 16 bytes to each of 32 rows (64 partial-line requests); passing
// through a wavefront-private LDS area (ROWS_PER_PASS * D elements) turns that into whole 16 * D-byte runs per
// instruction.  16-byte
// pieces of a row are XOR-swizzled with the row number to spread the column-wise writes over the banks.  LDS
// instructions of one wavefront execute in order, so no wait is needed between the writes and the reads.
// PIN_ADDRESSES keeps the per-lane address arithmetic at the call site: hoisted over the caller's loops it costs about
// twenty registers there, which the kernels that already use all 256 pay for with spills.
// OPERAND_ORDER: block row r is not matrix row r but, inside its group of 16, row 2 (r / 8) + rho(r % 8), the order in
// which a B operand holds contraction indices (see the header comment).
template <class E, int D, bool PIN_ADDRESSES = true, int ROWS_PER_PASS = 32, bool OPERAND_ORDER = false>
__device__ __forceinline__ void store_rows_via_lds(const f32x16 (&acc)[D / 32], float factor, unsigned short* lds,
                                                   unsigned short* dst, int valid_rows, int lane) {
    constexpr int PIECES = D / 8;          // 16-byte pieces per row
    constexpr int ROWS_PER_STORE = 64 / PIECES;
    static_assert(32 % ROWS_PER_PASS == 0 && ROWS_PER_PASS % ROWS_PER_STORE == 0, "pass / store shape mismatch");
    if (PIN_ADDRESSES) asm volatile("" : "+v"(lane));
    const int n = lane % 32;
    const int gh = lane / 32;
    unsigned char* base = reinterpret_cast<unsigned char*>(lds);
    const int p = lane % PIECES;
    // with ROWS_PER_PASS < 32 the area holds ROWS_PER_PASS * D elements and the block goes through it in several passes
#pragma unroll
    for (int pass = 0; pass < 32 / ROWS_PER_PASS; ++pass) {
        if (ROWS_PER_PASS == 32 || n / ROWS_PER_PASS == pass) {
            const int row = n % ROWS_PER_PASS;
#pragma unroll
            for (int cb = 0; cb < D / 32; ++cb)
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    u32x2 w;
                    w[0] = E::pack2(acc[cb][a * 4 + 0] * factor, acc[cb][a * 4 + 1] * factor);
                    w[1] = E::pack2(acc[cb][a * 4 + 2] * factor, acc[cb][a * 4 + 3] * factor);
                    const int piece = cb * 4 + a;
                    *reinterpret_cast<u32x2*>(base + row * (D * 2) + ((piece ^ (row & (PIECES - 1))) << 4) + gh * 8) = w;
                }
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < ROWS_PER_PASS / ROWS_PER_STORE; ++i) {
            const int r = i * ROWS_PER_STORE + lane / PIECES;
            const u32x4 val = *reinterpret_cast<const u32x4*>(base + r * (D * 2) + ((p ^ (r & (PIECES - 1))) << 4));
            int out_row = pass * ROWS_PER_PASS + r;
            if (OPERAND_ORDER) out_row = (out_row & ~15) | (((out_row >> 3) & 1) << 1) | ((out_row & 3) << 2) | ((out_row >> 2) & 1);
            if (out_row < valid_rows) *reinterpret_cast<u32x4*>(dst + (long long)out_row * D + p * 8) = val;
        }
        __builtin_amdgcn_wave_barrier();
    }
}

// Writes a wavefront's 32 x D block of fp32 results into a column-layout matrix [(head * D + dim), column] (see
// ColumnSink).  The block is held as transposed accumulators: lane (n, gh) owns token n, head dims
// cb*32 + a*8 + gh*4 + [0, 4) in acc[cb][a*4 + ...]; one store instruction writes one head dim of 32 consecutive tokens
// (128 contiguous bytes) for each lane half.  `head_rows` points at (dim 0 of the head, the block's first token).
// Buffer stores: the per-lane part of the address (token, lane half) is one register for all 16 * D / 32 stores, the head
// dim's row is a scalar offset; D * stride * 4 must stay below 2^31 (the host checks).
// ROTATE: each (even, odd) pair of head dims is rotated back by the angle of its token's position (table row
// `position0 + n`), in fp32 without fused multiply-adds, exactly as the conversion pass bhtd_to_columns does.
// valid_dims: head dims the matrix has per head (a multiple of 8, <= D): the kernels' padding dims are not written, and
// the rotary tables have valid_dims / 2 entries per position.
template <int D, bool ROTATE>
__device__ __forceinline__ void store_columns_f32(const f32x16 (&acc)[D / 32], float factor, float* head_rows, int stride,
                                                  int valid_rows, int valid_dims, int lane, const float* cos_table,
                                                  const float* sin_table, int position0, int table_rows_left) {
#pragma clang fp contract(off)
    asm volatile("" : "+v"(lane));  // keeps the per-lane address arithmetic here instead of hoisted over the caller's loops
    const int n = lane % 32;
    const int gh = lane / 32;
    if (n >= valid_rows) return;
    const __amdgpu_buffer_rsrc_t rows = __builtin_amdgcn_make_buffer_rsrc(head_rows, 0, 0x7fffffff, 0x00020000);
    const int lane_bytes = (gh * 4 * stride + n) * 4;
    __amdgpu_buffer_rsrc_t cos_rows = rows, sin_rows = rows;
    int table_bytes = 0;
    if (ROTATE) {
        // the tables' rows from position0 on, with their true extent
        const long long extent = (long long)table_rows_left * (valid_dims / 2) * 4;
        const int records = extent > 0x7fffffffLL ? 0x7fffffff : (int)extent;
        cos_rows = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(cos_table) + (long long)position0 * (valid_dims / 2), 0,
                                                     records, 0x00020000);
        sin_rows = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(sin_table) + (long long)position0 * (valid_dims / 2), 0,
                                                     records, 0x00020000);
        table_bytes = n * (valid_dims / 2) * 4;
    }
#pragma unroll
    for (int cb = 0; cb < D / 32; ++cb)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int dim = cb * 32 + a * 8;  // + gh * 4 through the lane's offset
            if (dim >= valid_dims) continue;  // (wavefront-uniform)
            float x[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) x[j] = acc[cb][a * 4 + j] * factor;
            if (ROTATE) {
                // (one aligned 128-bit load per table = the four pairs of these eight head dims, of which a lane uses the
                //  first or the second two: the 64-bit buffer load builtin of this toolchain fetches one word only)
                const u32x4 cw = __builtin_amdgcn_raw_buffer_load_b128(cos_rows, table_bytes, (dim / 2) * 4, 0);
                const u32x4 sw = __builtin_amdgcn_raw_buffer_load_b128(sin_rows, table_bytes, (dim / 2) * 4, 0);
                const float c0 = __builtin_bit_cast(float, gh ? cw[2] : cw[0]), c1 = __builtin_bit_cast(float, gh ? cw[3] : cw[1]);
                const float s0 = __builtin_bit_cast(float, gh ? sw[2] : sw[0]), s1 = __builtin_bit_cast(float, gh ? sw[3] : sw[1]);
                const float e0 = x[0], o0 = x[1], e1 = x[2], o1 = x[3];
                x[0] = e0 * c0 + o0 * s0;
                x[1] = -e0 * s0 + o0 * c0;
                x[2] = e1 * c1 + o1 * s1;
                x[3] = -e1 * s1 + o1 * c1;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, x[j]), rows, lane_bytes, (dim + j) * stride * 4, 0);
        }
}

// Workgroups the device runs at once, per XCD: occupancy of the kernel times the compute units of an XCD.
template <typename Kernel>
inline int resident_workgroups_per_xcd(Kernel kernel, int threads, size_t dynamic_lds) {
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, dynamic_lds) != hipSuccess || per_cu <= 0) per_cu = 1;
    int device = 0;
    int cus = 0;
    if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess ||
        cus <= 0)
        cus = 256;
    return per_cu * ((cus + kXcds - 1) / kXcds);
}

}  // namespace sentinel_hip
#endif
