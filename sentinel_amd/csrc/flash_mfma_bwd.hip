// Causal flash-attention backward on gfx950 matrix cores (bf16 / fp16 operands, fp32 accumulation).
//
// Replaces CudaFlashAttentionDeltaEntry + CudaFlashAttentionBackwardQueryWmma64Entry
// (sentinel/NeuralNet/Cuda/CudaFlashAttention.cu:576-596, :1269-1456).  Same mathematics
//     P = exp(S - LSE),  dP = dO V^T,  dS = P o (dP - D) * scale,
//     dV = P^T dO,  dK = dS^T Q,  dQ = dS K,          D = rowsum(dO o O)
// but no atomics and no pre-zeroed outputs: the work is split into
//   dkdv_split_kernel   key-outer: a workgroup owns 128 keys of one K/V head; per 32-key block one wavefront
//                       keeps K (as B operand) and dV^T, a second one V and dK^T, and the query tiles of
//                       every query head of the group stream through LDS (grouped-query gradients are summed
//                       in registers, replacing reduceKvHeadGradsInto, CudaCausalSelfAttention.cu:36-44);
//   dq_mfma_kernel      query-outer: a workgroup owns 128 queries, keeps Q, dO (as B operands) and dQ^T in
//                       registers and streams K / V tiles through LDS (recomputing S and dP); it runs first and
//                       also forms D from the dO rows it holds and the O rows, leaving it for the other kernel.
// Tiles sit row-major in LDS; the products that contract over tokens (dV, dK, dQ) read their A operand out
// of the same tiles with transposing LDS reads, so nothing is staged twice.
// In both kernels the score-like tiles are produced so that one lane owns one key (dK/dV kernel) or one
// query (dQ kernel) and their registers are, after type conversion, directly the B operand of the
// following product (see mfma_tile.h).
// Without the sparse mask the grids are persistent (as many workgroups as the device runs at once, each walking the key
// or query tiles of its XCD in snake order); result rows leave through LDS as whole rows (store_rows_via_lds).
#include "flash_common.h"
#include "mfma_tile.h"


#include <type_traits>

namespace sentinel_hip {
namespace {

constexpr int kBwdThreads = 256;

// instruction classes of __builtin_amdgcn_sched_group_barrier
constexpr int kSchedValu = 0x402;  // VALU and transcendental
constexpr int kSchedMfma = 0x008;
constexpr int kSchedDsRead = 0x100;

// A wavefront's 32 x D block of a gradient goes to the caller's fp32 column matrix (rotated back where the sink carries
// rotary tables); `head` is the tensor's head index, `token0` the block's first token inside pack `pack`.
template <int D>
__device__ __forceinline__ void store_block_to_sink(const f32x16 (&acc)[D / 32], float factor, const ColumnSink& sink, int head,
                                                    int pack, int token0, int seq_len, int lane) {
    float* head_rows = sink.base + (long long)head * sink.head_dim * sink.stride + (long long)pack * seq_len + token0;
    if (sink.inverse_rope.cos)
        store_columns_f32<D, true>(acc, factor, head_rows, (int)sink.stride, seq_len - token0, sink.head_dim, lane,
                                   sink.inverse_rope.cos, sink.inverse_rope.sin, sink.inverse_rope.offset + token0,
                                   sink.inverse_rope.positions - (sink.inverse_rope.offset + token0));
    else
        store_columns_f32<D, false>(acc, factor, head_rows, (int)sink.stride, seq_len - token0, sink.head_dim, lane, nullptr,
                                    nullptr, 0, 0);
}
constexpr int kOperandLead = 4;

// ------------------------------------------------------------------------------------------------
// dQ: query-outer
// ------------------------------------------------------------------------------------------------
constexpr int kDqQueryTile = 128;
constexpr int kDqKeyTile = 64;

// COLUMNS: dQ goes to the caller's fp32 column matrix (dq_columns) instead of the 16-bit tensor; a compile-time switch,
// because with the choice made at run time the 16-bit version lost 1.5 - 2 %.
template <typename E, int D, bool CAUSAL, bool WINDOW, bool COLUMNS = false>
__global__ __launch_bounds__(kBwdThreads, D <= 64 ? 3 : 2) void dq_mfma_kernel(const unsigned short* __restrict__ q,
                                                                  const unsigned short* __restrict__ k,
                                                                  const unsigned short* __restrict__ v,
                                                                  const unsigned short* __restrict__ out,
                                                                  const unsigned short* __restrict__ d_out,
                                                                  const float* __restrict__ lse,
                                                                  float* __restrict__ delta,
                                                                  unsigned short* __restrict__ dq, RowMap lm, AttnGeom g,
                                                                  int q_tiles, int total_tiles, int tiles_per_xcd, int deal,
                                                                  ColumnSink dq_columns) {
    constexpr int KT = kDqKeyTile;
    typedef DirectTile<KT, D, kBwdThreads> Tile;
    constexpr int KSTEPS = D / 16;
    constexpr int CB = D / 32;

    // two stages of (K, V) tiles; separate arrays so that loads into one stage are known not to alias reads of the other
    __shared__ __attribute__((aligned(16))) unsigned short k_lds0[Tile::kElems];
    __shared__ __attribute__((aligned(16))) unsigned short v_lds0[Tile::kElems];
    __shared__ __attribute__((aligned(16))) unsigned short k_lds1[Tile::kElems];
    __shared__ __attribute__((aligned(16))) unsigned short v_lds1[Tile::kElems];

    const int T = g.seq_len;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);  // wavefront-uniform by construction; tell the compiler
    const int lane = tid % 64;
    const int n = lane % 32;
    const int gh = lane / 32;

    // Persistent workgroups: as many as the device runs at once, each walking several query tiles.  Each XCD owns a
    // contiguous range of tiles (head-major, longest query tile of a head first: the tiles of one head stream the same
    // K / V through one L2); tile_of_slot hands them out in the order the host chose (plan_persistent_grid): by default
    // round r hands the XCD's tiles [r S, (r + 1) S) to its S workgroups, forwards in even rounds and backwards in odd
    // ones, so long and short tiles alternate.
    const unsigned turn_class = priority_turn_class();
    const int xcd = (int)blockIdx.x % kXcds;
    const int slot = (int)blockIdx.x / kXcds;
    const int slots = (int)gridDim.x / kXcds;
    for (int round = 0;; ++round) {
    const int local_tile = tile_of_slot(slot, slots, round, tiles_per_xcd, q_tiles, deal);
    const int tile_id = xcd * tiles_per_xcd + local_tile;
    if (local_tile >= tiles_per_xcd || tile_id >= total_tiles) break;
    const int bh = tile_id / q_tiles;
    const int qt = q_tiles - 1 - tile_id % q_tiles;
    const int b = bh / g.q_heads;
    const int h = bh % g.q_heads;
    const int kvh = h / (g.q_heads / g.kv_heads);

    const long long q_head = ((long long)b * g.q_heads + h) * T * D;
    const unsigned short* kb = k + ((long long)b * g.kv_heads + kvh) * T * D;
    const unsigned short* vb = v + ((long long)b * g.kv_heads + kvh) * T * D;

    const int q0w = qt * kDqQueryTile + wave * 32;
    const int qrow = q0w + n;
    const int qload = qrow < T ? qrow : T - 1;

    u32x4 qf[KSTEPS];
    u32x4 gf[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        qf[ks] = *reinterpret_cast<const u32x4*>(q + q_head + (long long)qload * D + ks * 16 + gh * 8);
        gf[ks] = *reinterpret_cast<const u32x4*>(d_out + q_head + (long long)qload * D + ks * 16 + gh * 8);
    }
    const float c2 = g.scale * kLog2e;
    const float lse2_raw = lse[b * lm.pack_stride + h * lm.head_stride + qload];
    // D = sum_c dO * O of this lane's query: the lane holds half of the row's dO (8 dims per k-step), the other
    // half sits 32 lanes away.  Computed here (the dO row is in registers anyway) and left in `delta` for the
    // dK/dV kernel, which runs after this one: no separate pass over O and dO.
    float dl;
    {
        float part = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            const u32x4 o = *reinterpret_cast<const u32x4*>(out + q_head + (long long)qload * D + ks * 16 + gh * 8);
#pragma unroll
            for (int e = 0; e < 4; ++e) part += E::lo(o[e]) * E::lo(gf[ks][e]) + E::hi(o[e]) * E::hi(gf[ks][e]);
        }
        dl = half_sum(part);
        if (gh == 0 && qrow < T) delta[(long long)h * g.packs * T + (long long)b * T + qrow] = dl;
    }

    const int q_hi = min(T, (qt + 1) * kDqQueryTile);
    const int kv_tiles = CAUSAL ? (q_hi + KT - 1) / KT : (T + KT - 1) / KT;
    // WINDOW (Sentinel's sliding window + global tokens on top of the causal mask): the key tiles this query tile
    // sees are those holding global tokens, [0, g_tiles), and those from the window of its first query up to the
    // diagonal, [w_first, kv_tiles); trip `it` works on tile_of(it)
    static_assert(CAUSAL || !WINDOW, "the sparse mask refines the causal one");
    int g_tiles = 0, w_first = 0;
    if (WINDOW) {
        g_tiles = min(kv_tiles, (g.global_tokens + KT - 1) / KT);
        w_first = max(g_tiles, max(0, qt * kDqQueryTile - g.window + 1) / KT);
    }
    const int n_trips = WINDOW ? g_tiles + (kv_tiles - w_first) : kv_tiles;
    auto tile_of = [&](int it) { return WINDOW ? (it < g_tiles ? it : it - g_tiles + w_first) : it; };

    const __amdgpu_buffer_rsrc_t k_rsrc = make_head_rsrc(kb, (long long)T * D * 2);
    const __amdgpu_buffer_rsrc_t v_rsrc = make_head_rsrc(vb, (long long)T * D * 2);
    const int ld_off = Tile::global_offset(tid);
    Tile::issue(k_rsrc, k_lds0, ld_off, tile_of(0) * KT * D * 2, wave);
    Tile::issue(v_rsrc, v_lds0, ld_off, tile_of(0) * KT * D * 2, wave);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        pin_loaded(qf[ks]);
        pin_loaded(gf[ks]);
    }
    float lse2 = lse2_raw * kLog2e;
    pin_loaded(lse2);
    pin_loaded(dl);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the first tiles have landed in LDS
    __syncthreads();

    f32x16 acc[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[cb][i] = 0.0f;

    const int mask_base = (CAUSAL ? min(qrow, T - 1) : T - 1) - 2 * gh;  // last live key of this lane's query, minus the lane half's row offset
    // sparse mask: a key is dead when it is no global token and lies window or more before the query, i.e. when
    // global_base <= key - 2 gh <= window_base
    const int global_base = g.global_tokens - 2 * gh;
    const int window_base = qrow - g.window - 2 * gh;
    const int k_off = Tile::row_read_base(row_perm(n), gh);
    const int t_even = Tile::transposed_read_base(lane, 0);
    const int t_odd = Tile::transposed_read_base(lane, 1);

    // one trip over tile j held in (kt, vt); the next tile streams into (kt_next, vt_next) meanwhile.
    // MASKED trips compare key against query per element; the others run the bare softmax-backward arithmetic.
    // head_dim 64 (bound by the vector ALU, registers to spare): the dP chains start from -D held in sixteen registers, which
    // saves the subtraction per element; head_dim 128 has no registers for that and subtracts
    constexpr bool FOLD_DELTA = D <= 64 && !WINDOW;  // (the sparse-mask variant would drop to two wavefronts per SIMD)
    f32x16 dp_start;
#pragma unroll
    for (int i = 0; i < 16; ++i) dp_start[i] = FOLD_DELTA ? -dl : 0.0f;
    auto tile_trip = [&](auto masked_tag, int j, const unsigned short* kt, const unsigned short* vt, unsigned short* kt_next,
                         unsigned short* vt_next) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        const bool more = j + 1 < n_trips;
        if (more) {
            Tile::issue(k_rsrc, kt_next, ld_off, tile_of(j + 1) * KT * D * 2, wave);
            Tile::issue(v_rsrc, vt_next, ld_off, tile_of(j + 1) * KT * D * 2, wave);
        }
        const int key0 = tile_of(j) * KT;
        // wavefront-uniform: the whole tile lies above this wavefront's diagonal, or holds no global token and
        // lies below the window of this wavefront's first query
        const bool skip = MASKED && CAUSAL &&
                          (key0 > q0w + 31 || (WINDOW && key0 >= g.global_tokens && key0 + KT - 1 < q0w - g.window + 1));
        if (!skip) {
            // two 32-key halves one after the other keeps the live score registers to one half
#pragma unroll
            for (int kbk = 0; kbk < 2; ++kbk) {
                f32x16 s;
                f32x16 dp;
#pragma unroll
                for (int i = 0; i < 16; ++i) s[i] = 0.0f;
                // program order = issue order wanted within each instruction class; the interleave of the classes
                // is laid down by the scheduling groups at the end of the half
                u32x4 ak[KSTEPS];
                u32x4 av[KSTEPS];
#pragma unroll
                for (int ks = 0; ks < KSTEPS; ++ks) ak[ks] = lds_read128(kt + kbk * 32 * D + (k_off ^ (ks << 4)));
#pragma unroll
                for (int ks = 0; ks < KSTEPS; ++ks) av[ks] = lds_read128(vt + kbk * 32 * D + (k_off ^ (ks << 4)));
#pragma unroll
                for (int ks = 0; ks < KSTEPS; ++ks) s = E::mfma(ak[ks], qf[ks], s);
#pragma unroll
                for (int ks = 0; ks < KSTEPS; ++ks) dp = E::mfma(av[ks], gf[ks], ks == 0 ? dp_start : dp);

                u32x4 kt_frag[2][CB];
#pragma unroll
                for (int half = 0; half < 2; ++half)
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) {
                        const int t0 = (kbk * 32 + half * 16) * D;
                        kt_frag[half][cb] =
                            lds_read_transposed_pair(kt + t0 + (t_even ^ (cb << 5)), kt + t0 + (t_odd ^ (cb << 5)));
                    }
                float p[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    p[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i], c2, -lse2));
                    // dead iff key0 + 32 kbk + (row of register i in lane half 0) + 2 gh > last live key
                    if (MASKED && perm_row_of_reg(i, 0) > mask_base - key0 - kbk * 32) p[i] = 0.0f;
                    if (MASKED && WINDOW && perm_row_of_reg(i, 0) >= global_base - key0 - kbk * 32 &&
                        perm_row_of_reg(i, 0) <= window_base - key0 - kbk * 32)
                        p[i] = 0.0f;
                }
                u32x4 dsf[2];
#pragma unroll
                for (int half = 0; half < 2; ++half)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int i = half * 8 + 2 * e;
                        dsf[half][e] = FOLD_DELTA ? E::pack2(p[i] * dp[i], p[i + 1] * dp[i + 1])
                                                  : E::pack2(p[i] * (dp[i] - dl), p[i + 1] * (dp[i + 1] - dl));
                    }
#pragma unroll
                for (int half = 0; half < 2; ++half) {
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) acc[cb] = E::mfma(kt_frag[half][cb], dsf[half], acc[cb]);
                }
                {
                    // S chain with its operand reads kOperandLead ahead, then the dP chain overlapped with exp(S) and
                    // the transposed reads of the dQ operands, then the rest of the arithmetic, then the dQ chain
                    __builtin_amdgcn_sched_group_barrier(kSchedDsRead, kOperandLead, 0);
#pragma unroll
                    for (int i = 0; i < 2 * KSTEPS - kOperandLead; ++i) {
                        __builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(kSchedDsRead, 1, 0);
                        if (i >= KSTEPS + 1) __builtin_amdgcn_sched_group_barrier(kSchedValu, 5, 0);
                    }
#pragma unroll
                    for (int i = 0; i < kOperandLead; ++i) {
                        __builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(kSchedDsRead, 2, 0);
                        __builtin_amdgcn_sched_group_barrier(kSchedValu, 5, 0);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        const unsigned now = WINDOW ? 0u : (unsigned)__builtin_amdgcn_s_memrealtime();
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this thread's share of the next tile is in LDS
        __syncthreads();
        if (!WINDOW) take_priority_turn(now, turn_class);  // the persistent grid only: see take_priority_turn
    };

    // Trips [bare_begin, bare_end) need no mask for any wavefront: their tiles end at or before the first query of the
    // workgroup and, under the sparse mask, start inside the window of its last query (the trips before them hold the
    // global tokens and the window's far edge, the ones after them the diagonal).  Both bounds are even so that every
    // run of trips starts on LDS stage 0.
    int bare_begin = 0;
    int bare_end = (CAUSAL ? min(kv_tiles, qt * (kDqQueryTile / KT)) : T / KT) & ~1;
    if (WINDOW) {
        const int q_last = q_hi - 1;
        const int inside = max(w_first, (max(0, q_last - g.window + 1) + KT - 1) / KT);  // first tile inside every window
        bare_begin = (g_tiles + inside - w_first + 1) & ~1;
        bare_end = (g_tiles + min(kv_tiles, qt * (kDqQueryTile / KT)) - w_first) & ~1;
        if (bare_end <= bare_begin) bare_begin = bare_end = 0;
        for (int j = 0; j < bare_begin; j += 2) {
            tile_trip(std::true_type{}, j, k_lds0, v_lds0, k_lds1, v_lds1);
            tile_trip(std::true_type{}, j + 1, k_lds1, v_lds1, k_lds0, v_lds0);
        }
    }
    for (int j = bare_begin; j < bare_end; j += 2) {
        tile_trip(std::false_type{}, j, k_lds0, v_lds0, k_lds1, v_lds1);
        tile_trip(std::false_type{}, j + 1, k_lds1, v_lds1, k_lds0, v_lds0);
    }
    for (int j = bare_end; j < n_trips; j += 2) {
        tile_trip(std::true_type{}, j, k_lds0, v_lds0, k_lds1, v_lds1);
        if (j + 1 < n_trips) tile_trip(std::true_type{}, j + 1, k_lds1, v_lds1, k_lds0, v_lds0);
    }

    // dQ rows leave through the second LDS stage, which no wavefront reads or fills any more: the last trip ended with
    // a barrier, and the next tile's first loads go to stage 0 and are followed by a barrier before stage 1 is filled
    if constexpr (COLUMNS)
        store_block_to_sink<D>(acc, g.scale, dq_columns, h, b, q0w, T, lane);
    else
        store_rows_via_lds<E, D>(acc, g.scale, (wave < 2 ? k_lds1 : v_lds1) + (wave & 1) * (32 * D),
                                 dq + q_head + (long long)q0w * D, T - q0w, lane);
    }  // next tile of this workgroup (the last trip ended with a barrier: the LDS stages are free)
}

constexpr int kDkvKeyTile = 128;
// sparse mask without global tokens: windows up to this many keys run the split dK/dV kernel on the persistent grid
constexpr int kMaxPersistentWindow = 512;
constexpr int kDkvQueryTile = 64;

// ------------------------------------------------------------------------------------------------
// dK, dV with the work of a 32-key block split over two wavefronts (512 threads, two wavefronts per SIMD):
//   score wavefront (waves 0..3):  S = Q K^T, P = exp2(S c - lse2), publishes P (16-bit) in LDS, dV^T += dO^T P
//   grad  wavefront (waves 4..7):  dP - D = dO V^T - D (accumulator starts at -D), dS = P o (dP - D), dK^T += Q^T dS
// The grad wavefronts run one stage behind the score wavefronts, so that P is always complete when it is
// read and one workgroup barrier per stage is all the synchronisation there is: three tile stages rotate
// (being filled / scored / back-propagated) and two P buffers alternate.  Each wavefront holds one operand
// (K or V, 32 keys) and one accumulator (dV^T or dK^T) in registers: half the registers of doing both, which
// is what lets two wavefronts share a SIMD and overlap one's exponentials with the other's matrix products.
// ------------------------------------------------------------------------------------------------
constexpr int kDkvSplitThreads = 512;

template <int D>
struct DkvSplitStage {
    static constexpr int QT = kDkvQueryTile;
    static constexpr int QS = D + 8;
    unsigned short q[QT * QS];
    unsigned short g[QT * QS];
    float nls[QT];  // -LSE / scale, in operand order (see stage_slot)
    float ndl[QT];  // -D, same order
};

template <int D>
struct DkvSplitLds {
    DkvSplitStage<D> stage[3];
    u32x4 p[2][4][2][2][64];  // [buffer][key block][32-query block][16-query half][lane]
};

// Position of query row r of a stage in the nls / ndl arrays: rows are kept in the order the score registers
// of a lane hold them (the inverse of perm_row_of_reg: 16 * (r / 16) + 8 g + 4 a + j for r = 16 c + 4 j + 2 g + a),
// so four 128-bit reads fill the 16 per-lane values in register order.
__device__ __forceinline__ int stage_slot(int r) {
    return (r & ~15) | (((r >> 1) & 1) << 3) | ((r & 1) << 2) | ((r >> 2) & 3);
}

// ------------------------------------------------------------------------------------------------
// dK, dV for head dims up to 64: one wavefront per 32-key block holds K, V (as B operands) and both
// accumulators and still leaves room for two wavefronts per SIMD, so the work is not split over roles.
// ------------------------------------------------------------------------------------------------
template <int D>
struct DkvLds {
    static constexpr int QT = kDkvQueryTile;
    static constexpr int kPad = 8;  // row pad (elements): conflict-free for the 128-bit row reads and the transposed reads
    static constexpr int QS = D + kPad;
    unsigned short q[QT * QS];
    unsigned short g[QT * QS];
    float lse2[QT];
    float dl[QT];  // -D of the stage's queries
};

// Stage ranges of one query head for a wavefront whose 32 keys start at k0w, under the causal mask and, with
// WINDOW, Sentinel's sparse mask: stages [first, causal_end) cross the causal diagonal, stages [upper_begin, end)
// hold queries that lie window or more behind one of the wavefront's keys outside the global range; both kinds
// take the masked code, what lies between runs bare.
struct DkvMaskedRanges {
    int causal_end;
    int upper_begin;
};
template <bool CAUSAL, bool WINDOW>
__device__ __forceinline__ DkvMaskedRanges dkv_masked_ranges(const AttnGeom& g, int k0w, int first, int end, int q_first,
                                                             int n_qt) {
    constexpr int QT = 64;
    DkvMaskedRanges r;
    r.causal_end = first;
    r.upper_begin = end;
    if (k0w + 31 >= g.seq_len) {  // keys past the end of the sequence: every stage masks them
        r.causal_end = end;
        return r;
    }
    if (CAUSAL) r.causal_end = min(end, first + max(0, (k0w + 31 + QT - 1) / QT - q_first));
    if (WINDOW) {
        const int kmin = max(k0w, g.global_tokens);  // first key of the wavefront the window applies to
        if (kmin <= k0w + 31) r.upper_begin = max(r.causal_end, first + min(n_qt, max(0, (kmin + g.window) / QT - q_first)));
    }
    return r;
}

// Query tiles a key tile of 128 keys starting at k0 meets: from its causal diagonal to the end of the sequence, or,
// with the sparse mask and no global token in the tile, to the last query whose window still reaches the tile.
template <bool CAUSAL, bool WINDOW>
__device__ __forceinline__ int dkv_query_tiles(const AttnGeom& g, int k0, int q_first) {
    constexpr int QT = 64;
    const int q_tiles_all = (g.seq_len + QT - 1) / QT;
    if (WINDOW && k0 >= g.global_tokens) {
        const long long last_query = (long long)k0 + 127 + g.window - 1;
        if (last_query < g.seq_len) return (int)(last_query / QT) + 1 - q_first;
    }
    return q_tiles_all - q_first;
}

// Tile `local` of XCD `xcd` -> (K/V head, key tile).  Workgroup ids are dealt round-robin to the 8 XCDs; each XCD gets a contiguous
// set of heads and walks them head after head, key tiles in increasing order: the key tiles of one head run side by
// side on the XCD and share that head's Q / dO stream in its L2 (HBM reads stay at the algorithmic bytes; a tile-major
// order over the heads was 2 % faster and read five times as much).  Under the causal mask the first key tiles of a
// head see the most queries, so each head starts with its longest work.  Key tiles that hold global tokens of the
// sparse mask (`front_tiles` of them per head) meet every query tile and are far longer than the windowed ones:
// those are dealt first, for all heads of the XCD, so that they start together at the head of the grid.
__device__ __forceinline__ bool dkv_tile_of_workgroup(int xcd, int local, int per_xcd, int k_tiles, int total_tiles,
                                                      int front_tiles, int& bkv, int& ktile) {
    const int heads = total_tiles / k_tiles;
    if (front_tiles > 0 && heads % kXcds == 0) {
        const int heads_per_xcd = heads / kXcds;
        const int front = front_tiles * heads_per_xcd;
        if (local < front) {
            ktile = local / heads_per_xcd;
            bkv = xcd * heads_per_xcd + local % heads_per_xcd;
        } else {
            const int rest = local - front;
            const int tail_tiles = k_tiles - front_tiles;
            bkv = xcd * heads_per_xcd + rest / tail_tiles;
            ktile = front_tiles + rest % tail_tiles;
        }
        return local < per_xcd && bkv < heads;
    }
    const int tile_id = xcd * per_xcd + local;
    bkv = tile_id / k_tiles;
    ktile = tile_id % k_tiles;
    return tile_id < total_tiles;
}

// COLUMNS: dK and dV go to the caller's fp32 column matrices (dk_columns, dv_columns) instead of the 16-bit tensors.  A
// compile-time switch: with the choice made at run time the register allocation of the whole kernel changed and the
// 16-bit version lost 5 - 7 %.
template <typename E, int D, bool CAUSAL, bool WINDOW, bool COLUMNS = false>
__global__ __launch_bounds__(kBwdThreads, 2) void dkdv_mfma_kernel(
    const unsigned short* __restrict__ q, const unsigned short* __restrict__ k, const unsigned short* __restrict__ v,
    const unsigned short* __restrict__ d_out, const float* __restrict__ lse, const float* __restrict__ delta,
    unsigned short* __restrict__ dk, unsigned short* __restrict__ dv, RowMap lm, AttnGeom g, int k_tiles,
    int total_tiles, int tiles_per_xcd, int deal, ColumnSink dk_columns, ColumnSink dv_columns) {
    constexpr int QT = kDkvQueryTile;
    typedef RowTile<QT, D, kBwdThreads, DkvLds<D>::kPad> RTile;
    constexpr int QS = RTile::kStride;
    static_assert(QS == DkvLds<D>::QS, "LDS layout mismatch");
    constexpr int KSTEPS = D / 16;
    constexpr int CB = D / 32;

    extern __shared__ __attribute__((aligned(16))) unsigned char dkv_smem[];
    DkvLds<D>* lds = reinterpret_cast<DkvLds<D>*>(dkv_smem);  // two stages

    const int group = g.q_heads / g.kv_heads;
    const int T = g.seq_len;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);  // wavefront-uniform by construction; tell the compiler
    const int lane = tid % 64;
    const int n = lane % 32;
    const int gh = lane / 32;

    // persistent workgroups walking the XCD's key tiles in the order the host chose (tile_of_slot; see dq_mfma_kernel)
    const int front_tiles = WINDOW ? min(k_tiles - 1, (g.global_tokens + kDkvKeyTile - 1) / kDkvKeyTile) : 0;
    const unsigned turn_class = priority_turn_class();
    const int xcd = (int)blockIdx.x % kXcds;
    const int slot = (int)blockIdx.x / kXcds;
    const int slots = (int)gridDim.x / kXcds;
    for (int round = 0;; ++round) {
    const int local_tile = tile_of_slot(slot, slots, round, tiles_per_xcd, k_tiles, deal);
    int bkv, ktile;
    if (local_tile >= tiles_per_xcd ||
        !dkv_tile_of_workgroup(xcd, local_tile, tiles_per_xcd, k_tiles, total_tiles, front_tiles, bkv, ktile))
        break;
    const int b = bkv / g.kv_heads;
    const int kvh = bkv % g.kv_heads;

    const long long kv_head = ((long long)b * g.kv_heads + kvh) * T * D;
    const int k0w = ktile * kDkvKeyTile + wave * 32;
    const int key = k0w + n;
    const int kload = key < T ? key : T - 1;
    const bool key_dead = key >= T;

    // K^T and V^T as B operands: column = key, contraction over head dims
    u32x4 kf[KSTEPS];
    u32x4 vf[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        kf[ks] = *reinterpret_cast<const u32x4*>(k + kv_head + (long long)kload * D + ks * 16 + gh * 8);
        vf[ks] = *reinterpret_cast<const u32x4*>(v + kv_head + (long long)kload * D + ks * 16 + gh * 8);
    }
    const float c2 = g.scale * kLog2e;

    static_assert(QT == 64 && kDkvKeyTile == 128, "dkv_query_tiles / dkv_masked_ranges assume these tiles");
    const int q_first = CAUSAL ? (ktile * kDkvKeyTile) / QT : 0;
    const int n_qt = dkv_query_tiles<CAUSAL, WINDOW>(g, ktile * kDkvKeyTile, q_first);
    const int n_iter = group * n_qt;

    f32x16 dk_acc[CB];
    f32x16 dv_acc[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            dk_acc[cb][i] = 0.0f;
            dv_acc[cb][i] = 0.0f;
        }

    RTile qtile;
    RTile gtile;
    float row_val = 0.0f;  // threads 0..63: lse; threads 64..127: delta
    const int ld_off = RTile::global_offset(tid);
    const int st_off = RTile::lds_offset(tid);

    // threads 0..63 fetch lse, 64..127 delta of the stage's queries (the upper half of the workgroup repeats
    // them); the row load is issued before the tile loads so that waiting for it never waits for those
    const int row_slot = tid % QT;
    const bool row_is_delta = (tid / QT) & 1;
    auto load_stage = [&](int it) {
        const int h = kvh * group + it / n_qt;
        const int q0 = (q_first + it % n_qt) * QT;
        const long long q_head = ((long long)b * g.q_heads + h) * T * D;
        const int t = min(q0 + row_slot, T - 1);
        const float* row_src = row_is_delta ? delta + (long long)h * g.packs * T + (long long)b * T
                                            : lse + b * lm.pack_stride + h * lm.head_stride;
        row_val = row_src[t];
        const __amdgpu_buffer_rsrc_t q_rsrc = make_head_rsrc(q + q_head, (long long)T * D * 2);
        const __amdgpu_buffer_rsrc_t g_rsrc = make_head_rsrc(d_out + q_head, (long long)T * D * 2);
        qtile.load(q_rsrc, ld_off, q0 * D * 2);
        gtile.load(g_rsrc, ld_off, q0 * D * 2);
    };
    auto store_stage = [&](DkvLds<D>& st, int it) {
        qtile.store(st.q, st_off);
        gtile.store(st.g, st_off);
        const int q0 = (q_first + it % n_qt) * QT;
        const bool live = q0 + row_slot < T;
        if (tid < QT)
            st.lse2[stage_slot(row_slot)] = live ? row_val * kLog2e : __builtin_inff();  // exp2(s - inf) = 0 for padded queries
        else if (tid < 2 * QT)
            st.dl[stage_slot(row_slot)] = live ? -row_val : 0.0f;  // -D: what the dP chains start from
    };

    // n_iter >= 1 always (the key tile's own queries)
    load_stage(0);
    store_stage(lds[0], 0);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        pin_loaded(kf[ks]);
        pin_loaded(vf[ks]);
    }
    __syncthreads();

    const int r_off = row_perm(n) * QS + gh * 8;
    const int t_off = transposed_read_offset(lane, QS);

    // P and dS of one 32-query block from its S and dP tiles (this lane: one key, 16 queries), rounded and
    // packed as the B operands of the dV / dK products.  MASKED is only instantiated for stages that touch
    // the causal diagonal or the end of the sequence, so the common case carries no compare / select.
    auto softmax_backward = [&](auto masked_tag, const f32x16& s, const f32x16& dp, const DkvLds<D>& st, int qb, int q0b,
                                u32x4 (&pf)[2], u32x4 (&dsf)[2]) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        // lse of the 16 queries this lane holds, in register order (the array is kept in that order); dp arrives as dP - D
        float l2[16];
#pragma unroll
        for (int part = 0; part < 4; ++part) {
            const int base = qb * 32 + (part >> 1) * 16 + gh * 8 + (part & 1) * 4;
            const float4 a = *reinterpret_cast<const float4*>(&st.lse2[base]);
            l2[part * 4] = a.x; l2[part * 4 + 1] = a.y; l2[part * 4 + 2] = a.z; l2[part * 4 + 3] = a.w;
        }
#pragma unroll
        for (int half = 0; half < 2; ++half) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float p2[2];
                float ds2[2];
#pragma unroll
                for (int w = 0; w < 2; ++w) {
                    const int i = half * 8 + 2 * e + w;
                    // a dead pair gets exponent -inf (p = 0 exactly).  The empty asm makes the value opaque: without it the
                    // select is compiled into a branch around the arithmetic that feeds it, per element
                    float exponent = __builtin_fmaf(s[i], c2, -l2[i]);
                    if (MASKED) {
                        asm("" : "+v"(exponent));
                        const int query = q0b + perm_row_of_reg(i, gh);
                        if ((CAUSAL && key > query) || key_dead || (WINDOW && outside_window(g, query, key)))
                            exponent = -__builtin_inff();
                    }
                    const float p = __builtin_amdgcn_exp2f(exponent);
                    p2[w] = p;
                    ds2[w] = p * dp[i];
                }
                pf[half][e] = E::pack2(p2[0], p2[1]);
                dsf[half][e] = E::pack2(ds2[0], ds2[1]);
            }
        }
    };

    // One stage = NB 32-query blocks.  Blocks entirely above the diagonal are not skipped (a few per
    // workgroup): they are masked to zero instead, which keeps the stage body free of branches.
    auto process_stage = [&](auto masked_tag, const DkvLds<D>& st, int q0) {
        constexpr int NB = QT / 32;
        f32x16 s[2];
        f32x16 dp[2];
        u32x4 pf[2][2];
        u32x4 dsf[2][2];
        auto scores = [&](int blk) {  // S and dP - D of block blk: the dP chain starts from -D of the lane's 16 queries
#pragma unroll
            for (int i = 0; i < 16; ++i) s[blk & 1][i] = 0.0f;
#pragma unroll
            for (int part = 0; part < 4; ++part) {
                const float4 d4 = *reinterpret_cast<const float4*>(&st.dl[blk * 32 + (part >> 1) * 16 + gh * 8 + (part & 1) * 4]);
                dp[blk & 1][part * 4] = d4.x; dp[blk & 1][part * 4 + 1] = d4.y;
                dp[blk & 1][part * 4 + 2] = d4.z; dp[blk & 1][part * 4 + 3] = d4.w;
            }
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                s[blk & 1] = E::mfma(lds_read128(&st.q[blk * 32 * QS + r_off + ks * 16]), kf[ks], s[blk & 1]);
                dp[blk & 1] = E::mfma(lds_read128(&st.g[blk * 32 * QS + r_off + ks * 16]), vf[ks], dp[blk & 1]);
            }
        };
        auto gradients = [&](int blk) {  // dV += dO^T P, dK += Q^T dS of block blk
#pragma unroll
            for (int c2i = 0; c2i < 2; ++c2i)
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                    const u32x4 tg = lds_read_transposed(&st.g[t_off + (blk * 32 + c2i * 16) * QS + cb * 32], QS);
                    dv_acc[cb] = E::mfma(tg, pf[blk & 1][c2i], dv_acc[cb]);
                    const u32x4 tq = lds_read_transposed(&st.q[t_off + (blk * 32 + c2i * 16) * QS + cb * 32], QS);
                    dk_acc[cb] = E::mfma(tq, dsf[blk & 1][c2i], dk_acc[cb]);
                }
        };
#pragma unroll
        for (int blk = 0; blk < NB; ++blk) {
            scores(blk);
            softmax_backward(masked_tag, s[blk & 1], dp[blk & 1], st, blk, q0 + blk * 32, pf[blk & 1], dsf[blk & 1]);
            gradients(blk);
        }
    };

    // one trip of the stage loop: prefetch the next stage, work on this one, publish the next one
    auto stage_trip = [&](auto masked_tag, int it) {
        const bool more = it + 1 < n_iter;
        if (more) load_stage(it + 1);
        process_stage(masked_tag, lds[it & 1], (q_first + it % n_qt) * QT);
        if (more) store_stage(lds[(it + 1) & 1], it + 1);
        const unsigned now = WINDOW ? 0u : (unsigned)__builtin_amdgcn_s_memrealtime();
        __syncthreads();
        if (!WINDOW) take_priority_turn(now, turn_class);  // the persistent grid only: see take_priority_turn
    };

    // Per query head of the group: the leading stages that touch this wavefront's causal diagonal (all stages if
    // the key tile runs past the end of the sequence) take the masked code, the rest the unmasked code.  Two
    // loops one after the other rather than a branch inside one loop, so the accumulators have one home.
    {
        int it = 0;
        for (int gi = 0; gi < group; ++gi) {
            const int head_end = (gi + 1) * n_qt;
            const DkvMaskedRanges r = dkv_masked_ranges<CAUSAL, WINDOW>(g, k0w, it, head_end, q_first, n_qt);
            for (; it < r.causal_end; ++it) stage_trip(std::true_type{}, it);
            for (; it < r.upper_begin; ++it) stage_trip(std::false_type{}, it);
            if (WINDOW)
                for (; it < head_end; ++it) stage_trip(std::true_type{}, it);
        }
    }

    {
        // dK and dV rows leave through the second LDS stage (free: every trip ended with a barrier, and the next key
        // tile fills stage 0 and passes a barrier before it touches stage 1), one after the other through the same area
        static_assert(sizeof(DkvLds<D>) >= 4 * 32 * D * 2, "second stage too small to stage the result rows");
        unsigned short* area = reinterpret_cast<unsigned short*>(&lds[1]) + wave * (32 * D);
        if constexpr (COLUMNS) {
            store_block_to_sink<D>(dk_acc, g.scale, dk_columns, kvh, b, k0w, T, lane);
            store_block_to_sink<D>(dv_acc, 1.0f, dv_columns, kvh, b, k0w, T, lane);
        } else {
            store_rows_via_lds<E, D>(dk_acc, g.scale, area, dk + kv_head + (long long)k0w * D, T - k0w, lane);
            __builtin_amdgcn_wave_barrier();
            store_rows_via_lds<E, D>(dv_acc, 1.0f, area, dv + kv_head + (long long)k0w * D, T - k0w, lane);
        }
    }
    }  // next key tile of this workgroup (every stage trip ended with a barrier: the LDS stages are free)
}

// COLUMNS: as in dkdv_mfma_kernel
template <typename E, int D, bool CAUSAL, bool WINDOW, bool COLUMNS = false>
__global__ __launch_bounds__(kDkvSplitThreads) void dkdv_split_kernel(
    const unsigned short* __restrict__ q, const unsigned short* __restrict__ k, const unsigned short* __restrict__ v,
    const unsigned short* __restrict__ d_out, const float* __restrict__ lse, const float* __restrict__ delta,
    unsigned short* __restrict__ dk, unsigned short* __restrict__ dv, RowMap lm, AttnGeom g, int k_tiles,
    int total_tiles, int tiles_per_xcd, int deal, ColumnSink dk_columns, ColumnSink dv_columns) {
    constexpr int QT = kDkvQueryTile;
    // the query / dO tiles of a stage are staged by the score wavefronts alone (threads 0..255): they have about a
    // quarter of a stage to spare, the grad wavefronts are the critical path
    typedef RowTile<QT, D, kDkvSplitThreads / 2, 8> RTile;
    constexpr int QS = RTile::kStride;
    static_assert(QS == DkvSplitStage<D>::QS, "LDS layout mismatch");
    constexpr int KSTEPS = D / 16;
    constexpr int CB = D / 32;

    extern __shared__ __attribute__((aligned(16))) unsigned char dkv_smem[];
    DkvSplitLds<D>& lds = *reinterpret_cast<DkvSplitLds<D>*>(dkv_smem);

    const int group = g.q_heads / g.kv_heads;
    const int T = g.seq_len;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const bool grad_role = wave >= 4;
    const int kblock = wave & 3;
    const int lane = tid % 64;
    const int n = lane % 32;
    const int gh = lane / 32;

    // persistent workgroups walking the XCD's key tiles in the order the host chose (tile_of_slot; see dq_mfma_kernel)
    const int front_tiles = WINDOW ? min(k_tiles - 1, (g.global_tokens + kDkvKeyTile - 1) / kDkvKeyTile) : 0;
    const int xcd = (int)blockIdx.x % kXcds;
    const int slot = (int)blockIdx.x / kXcds;
    const int slots = (int)gridDim.x / kXcds;
    for (int round = 0;; ++round) {
    const int local_tile = tile_of_slot(slot, slots, round, tiles_per_xcd, k_tiles, deal);
    int bkv, ktile;
    if (local_tile >= tiles_per_xcd ||
        !dkv_tile_of_workgroup(xcd, local_tile, tiles_per_xcd, k_tiles, total_tiles, front_tiles, bkv, ktile))
        break;
    const int b = bkv / g.kv_heads;
    const int kvh = bkv % g.kv_heads;

    const long long kv_head = ((long long)b * g.kv_heads + kvh) * T * D;
    const int k0w = ktile * kDkvKeyTile + kblock * 32;
    const int key = k0w + n;
    const int kload = key < T ? key : T - 1;
    const bool key_dead = key >= T;

    // this wavefront's B operand: K^T (score role) or V^T (grad role); column = key, contraction over head dims
    u32x4 of[KSTEPS];
    {
        const unsigned short* src = (grad_role ? v : k) + kv_head + (long long)kload * D + gh * 8;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) of[ks] = *reinterpret_cast<const u32x4*>(src + ks * 16);
    }
    const float c2 = g.scale * kLog2e;

    static_assert(QT == 64 && kDkvKeyTile == 128, "dkv_query_tiles / dkv_masked_ranges assume these tiles");
    const int q_first = CAUSAL ? (ktile * kDkvKeyTile) / QT : 0;
    const int n_qt = dkv_query_tiles<CAUSAL, WINDOW>(g, ktile * kDkvKeyTile, q_first);
    const int n_iter = group * n_qt;

    f32x16 acc[CB];  // dV^T (score role) or dK^T (grad role)
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[cb][i] = 0.0f;

    RTile qtile;
    RTile gtile;
    float row_val = 0.0f;  // threads 0..63: lse; threads 64..127: delta
    const int ld_off = RTile::global_offset(tid);
    const int st_off = RTile::lds_offset(tid);
    const int row_slot = tid % QT;
    const bool row_is_delta = (tid / QT) & 1;
    const bool row_thread = tid < 2 * QT;
    const float neg_inv_scale = -1.0f / g.scale;

    auto load_stage = [&](int it) {
        const int h = kvh * group + it / n_qt;
        const int q0 = (q_first + it % n_qt) * QT;
        const long long q_head = ((long long)b * g.q_heads + h) * T * D;
        {   // every thread loads a row value (no branch); only the first 128 publish theirs
            const int t = min(q0 + row_slot, T - 1);
            const float* row_src = row_is_delta ? delta + (long long)h * g.packs * T + (long long)b * T
                                                : lse + b * lm.pack_stride + h * lm.head_stride;
            row_val = row_src[t];
        }
        const __amdgpu_buffer_rsrc_t q_rsrc = make_head_rsrc(q + q_head, (long long)T * D * 2);
        const __amdgpu_buffer_rsrc_t g_rsrc = make_head_rsrc(d_out + q_head, (long long)T * D * 2);
        qtile.load(q_rsrc, ld_off, q0 * D * 2);
        gtile.load(g_rsrc, ld_off, q0 * D * 2);
    };
    // Row values are published as accumulator start values: -lse / scale for the S chain (so that
    // P = exp2(c * S) needs no subtraction) and -D for the dP chain.  -inf makes P = 0 for padded queries.
    auto store_stage = [&](DkvSplitStage<D>& st, int it) {
        qtile.store(st.q, st_off);
        gtile.store(st.g, st_off);
        // Every thread publishes its row value (threads 128.. repeat the values of threads 0..127): with a branch
        // around the store the compiler sinks the load into it, to the end of the trip, where its latency holds up
        // the workgroup barrier.
        const int q0 = (q_first + it % n_qt) * QT;
        const bool live = q0 + row_slot < T;
        float* slot = (row_is_delta ? st.ndl : st.nls) + stage_slot(row_slot);
        *slot = row_is_delta ? (live ? -row_val : 0.0f) : (live ? row_val * neg_inv_scale : -__builtin_inff());
    };

    if (!grad_role) {
        load_stage(0);
        store_stage(lds.stage[0], 0);
    }
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) pin_loaded(of[ks]);
    __syncthreads();

    // LDS addressing: one opaque per-lane byte offset per access pattern and stage, everything else is a
    // compile-time constant that folds into the instruction's offset field.
    constexpr int kStageBytes = (int)sizeof(DkvSplitStage<D>);
    constexpr int kGOff = QT * QS;                    // elements from q to g
    constexpr int kNlsBytes = 2 * QT * QS * 2;        // bytes from the stage start to nls
    constexpr int kNdlBytes = kNlsBytes + QT * 4;
    constexpr int kPBase = 3 * kStageBytes;           // bytes from the LDS start to p
    constexpr int kPBufBytes = 4 * 2 * 2 * 64 * 16;
    const int r_lane = (row_perm(n) * QS + gh * 8) * 2;
    const int t_lane = transposed_read_offset(lane, QS) * 2;
    const int v_lane = gh * 32;
    const int p_lane = kPBase + kblock * (2 * 2 * 64 * 16) + lane * 16;
    auto opaque = [](int x) {
        asm volatile("" : "+v"(x));
        return x;
    };
    auto tile_at = [&](int byte_off) { return reinterpret_cast<const unsigned short*>(dkv_smem + byte_off); };

    // the 16 per-lane row values of a 32-query block, in register order
    auto row_values = [&](int arr_off, int blk, f32x16& out) {
        const float* arr = reinterpret_cast<const float*>(dkv_smem + arr_off);
#pragma unroll
        for (int part = 0; part < 4; ++part) {
            const float4 a = *reinterpret_cast<const float4*>(&arr[blk * 32 + (part >> 1) * 16 + (part & 1) * 4]);
            out[part * 4 + 0] = a.x;
            out[part * 4 + 1] = a.y;
            out[part * 4 + 2] = a.z;
            out[part * 4 + 3] = a.w;
        }
    };

    // Operand fetches run one phase ahead of the matrix chain that consumes them: the LDS round trip is
    // then hidden behind the previous chain or the softmax arithmetic instead of stalling every instruction.
    auto fence = [] { __builtin_amdgcn_sched_barrier(0); };
    auto read_rows = [&](const unsigned short* at, u32x4 (&frag)[KSTEPS]) {
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) frag[ks] = lds_read128(at + ks * 16);
    };
    auto read_cols = [&](const unsigned short* at, u32x4 (&frag)[2][CB]) {  // token block of 32 at `at`
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) frag[half][cb] = lds_read_transposed(at + half * 16 * QS + cb * 32, QS);
    };
    // The next stage's global loads are issued just ahead of the last matrix chain of a trip (no LDS access
    // follows them in the trip) and published to LDS behind it; then every wavefront meets at the barrier.
    // Past the last stage the fetch repeats that stage into the (then unused) next buffer: no branch in a trip.
    auto prefetch = [&](int it) { load_stage(min(it + 1, n_iter - 1)); };
    auto last_chain = [&](int it, auto&& chain) {
        const int next = min(it + 1, n_iter - 1);
        chain();
        store_stage(lds.stage[(it + 1) % 3], next);
        __syncthreads();
    };
    auto last_chain_grad = [&](auto&& chain) {
        chain();
        __syncthreads();
    };

    // score role, trip `it`: P of both 32-query blocks of stage `it` -> LDS, dV^T += dO^T P
    auto score_trip = [&](auto masked_tag, int it) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        const int stage = it % 3;
        const int q0 = (q_first + it % n_qt) * QT;
        const unsigned short* rows = tile_at(opaque(stage * kStageBytes + r_lane));
        const unsigned short* cols = tile_at(opaque(stage * kStageBytes + t_lane));
        const int nls_off = opaque(stage * kStageBytes + kNlsBytes + v_lane);
        u32x4* pout = reinterpret_cast<u32x4*>(dkv_smem + opaque(p_lane + (it & 1) * kPBufBytes));
        // key - query of register i, block blk is mask_rel - (32 blk + row of register i in lane half 0): one
        // per-lane value compared against compile-time constants; a key past the end masks everything
        const int mask_rel = key_dead ? 0x7fffffff : (CAUSAL ? key - q0 - gh * 2 : -0x7fffffff);
        // sparse mask: a key outside the global range is dead for queries window or more behind it, i.e. from
        // 32 blk + row = mask_rel + window on
        const int window_rel = (WINDOW && !key_dead && key >= g.global_tokens) ? mask_rel + g.window : 0x7fffffff;
        u32x4 qrow[KSTEPS];
        u32x4 gcol[2][CB];
        f32x16 s;
        row_values(nls_off, 0, s);  // first: the chain's first instruction needs the accumulator start and one operand only
        read_rows(rows, qrow);
        fence();
#pragma unroll
        for (int blk = 0; blk < QT / 32; ++blk) {
            // S chain (accumulator starts at -lse / scale); the dO^T operands of the dV chain are fetched meanwhile
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) s = E::mfma(qrow[ks], of[ks], s);
            read_cols(cols + kGOff + blk * 32 * QS, gcol);
            // the next stage's global loads go out behind the first chain of the trip: their address arithmetic runs
            // under it and their latency under the rest of the trip
            if (blk == 0) prefetch(it);
            fence();
            u32x4 pf[2];
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float p2[2];
#pragma unroll
                    for (int w = 0; w < 2; ++w) {
                        const int i = half * 8 + 2 * e + w;
                        float p = __builtin_amdgcn_exp2f(s[i] * c2);
                        if (MASKED && mask_rel > blk * 32 + perm_row_of_reg(i, 0)) p = 0.0f;
                        if (MASKED && WINDOW && window_rel <= blk * 32 + perm_row_of_reg(i, 0)) p = 0.0f;
                        p2[w] = p;
                    }
                    pf[half][e] = E::pack2(p2[0], p2[1]);
                }
            pout[(blk * 2 + 0) * 64] = pf[0];
            pout[(blk * 2 + 1) * 64] = pf[1];
            auto dv_chain = [&] {
#pragma unroll
                for (int half = 0; half < 2; ++half)
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) acc[cb] = E::mfma(gcol[half][cb], pf[half], acc[cb]);
            };
            if (blk + 1 < QT / 32) {  // next block's Q rows and row values: in flight during the dV chain
                read_rows(rows + (blk + 1) * 32 * QS, qrow);
                row_values(nls_off, blk + 1, s);
                fence();
                dv_chain();
                fence();
            } else {
                fence();
                last_chain(it, dv_chain);
            }
        }
    };

    // grad role, trip `it`: stage it - 1, dS = P o (dP - D), dK^T += Q^T dS
    auto grad_trip = [&](int it) {
        const int stage = (it - 1) % 3;
        const unsigned short* rows = tile_at(opaque(stage * kStageBytes + r_lane));
        const unsigned short* cols = tile_at(opaque(stage * kStageBytes + t_lane));
        const int ndl_off = opaque(stage * kStageBytes + kNdlBytes + v_lane);
        const u32x4* pin = reinterpret_cast<const u32x4*>(dkv_smem + opaque(p_lane + ((it - 1) & 1) * kPBufBytes));
        u32x4 grow[KSTEPS];
        u32x4 qcol[2][CB];
        f32x16 dp;
        row_values(ndl_off, 0, dp);
        read_rows(rows + kGOff, grow);
        fence();
#pragma unroll
        for (int blk = 0; blk < QT / 32; ++blk) {
            // dP chain (accumulator starts at -D); P and the Q^T operands of the dK chain are fetched meanwhile
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) dp = E::mfma(grow[ks], of[ks], dp);
            const u32x4 pf0 = pin[(blk * 2 + 0) * 64];
            const u32x4 pf1 = pin[(blk * 2 + 1) * 64];
            read_cols(cols + blk * 32 * QS, qcol);
            fence();
            u32x4 dsf[2];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                dsf[0][e] = E::pack2(E::lo(pf0[e]) * dp[2 * e], E::hi(pf0[e]) * dp[2 * e + 1]);
                dsf[1][e] = E::pack2(E::lo(pf1[e]) * dp[8 + 2 * e], E::hi(pf1[e]) * dp[8 + 2 * e + 1]);
            }
            auto dk_chain = [&] {
#pragma unroll
                for (int half = 0; half < 2; ++half)
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) acc[cb] = E::mfma(qcol[half][cb], dsf[half], acc[cb]);
            };
            if (blk + 1 < QT / 32) {
                read_rows(rows + kGOff + (blk + 1) * 32 * QS, grow);
                row_values(ndl_off, blk + 1, dp);
                fence();
                dk_chain();
                fence();
            } else {
                fence();
                last_chain_grad(dk_chain);
            }
        }
    };

    // Trip i: the score wavefronts work on stage i, the grad wavefronts on stage i - 1 (trip 0 / trip n_iter
    // are idle for the grad / score role).  Masked and unmasked score trips sit in loops of their own.
    if (!grad_role) {
        int it = 0;
        for (int gi = 0; gi < group; ++gi) {
            const int head_end = (gi + 1) * n_qt;
            const DkvMaskedRanges r = dkv_masked_ranges<CAUSAL, WINDOW>(g, k0w, it, head_end, q_first, n_qt);
            for (; it < r.causal_end; ++it) score_trip(std::true_type{}, it);
            for (; it < r.upper_begin; ++it) score_trip(std::false_type{}, it);
            if (WINDOW)
                for (; it < head_end; ++it) score_trip(std::true_type{}, it);
        }
        // Last trip of the tile: the grad wavefronts work on the last stage, the score wavefronts have none left and
        // store dV meanwhile.  The stage buffers are still in use; the rows pass through the P buffer this trip would
        // have filled, 4 KB per wavefront, 16 rows at a time.
        static_assert(kPBufBytes >= 4 * 16 * D * 2, "P buffer too small to stage the dV rows");
        if constexpr (COLUMNS)
            store_block_to_sink<D>(acc, 1.0f, dv_columns, kvh, b, k0w, T, lane);
        else
            store_rows_via_lds<E, D, true, 16>(
                acc, 1.0f, reinterpret_cast<unsigned short*>(dkv_smem + kPBase + (n_iter & 1) * kPBufBytes) + kblock * (16 * D),
                dv + kv_head + (long long)k0w * D, T - k0w, lane);
        __syncthreads();
    } else {
        __syncthreads();  // trip 0: the score wavefronts work on stage 0 and publish stage 1
        for (int it = 1; it <= n_iter; ++it) grad_trip(it);
    }

    if (grad_role) {
        // dK rows leave through stages 1 and 2 of the LDS: both roles have passed the last barrier of the tile, and the
        // next key tile fills stage 0 and passes a barrier before it touches the others
        static_assert(2 * sizeof(DkvSplitStage<D>) >= 4 * 32 * D * 2, "stages 1 and 2 too small to stage the dK rows");
        unsigned short* area = reinterpret_cast<unsigned short*>(dkv_smem + sizeof(DkvSplitStage<D>)) + kblock * (32 * D);
        if constexpr (COLUMNS)
            store_block_to_sink<D>(acc, g.scale, dk_columns, kvh, b, k0w, T, lane);
        else
            store_rows_via_lds<E, D>(acc, g.scale, area, dk + kv_head + (long long)k0w * D, T - k0w, lane);
    }
    }  // next key tile of this workgroup (both roles have passed the last barrier of the tile: the LDS is free)
}

template <typename E, int D>
hipError_t run_bwd(const void* q, const void* k, const void* v, const void* out, const float* lse, RowMap lm,
                   const void* d_out, void* dq, void* dk, void* dv, float* delta, AttnGeom g,
                   hipStream_t stream, ColumnSink dq_columns, ColumnSink dk_columns, ColumnSink dv_columns) {
    auto qp = static_cast<const unsigned short*>(q);
    auto kp = static_cast<const unsigned short*>(k);
    auto vp = static_cast<const unsigned short*>(v);
    auto op = static_cast<const unsigned short*>(out);
    auto gp = static_cast<const unsigned short*>(d_out);
    auto dqp = static_cast<unsigned short*>(dq);
    auto dkp = static_cast<unsigned short*>(dk);
    auto dvp = static_cast<unsigned short*>(dv);
    const int T = g.seq_len;
    hipError_t err;
    // dQ first: it also leaves D = rowsum(dO o O) in `delta` for the dK/dV kernel
    {
        const int q_tiles = (T + kDqQueryTile - 1) / kDqQueryTile;
        const int total = g.packs * g.q_heads * q_tiles;
        const int tiles_per_xcd = (total + kXcds - 1) / kXcds;
        const long long streamed = 2ll * T * D * 2;  // K and V of a head
        auto launch = [&](auto kernel) {
            static const int resident = resident_workgroups_per_xcd(kernel, kBwdThreads, 0);  // per kernel instantiation
            // under the sparse mask tile lengths no longer grow with the tile index, and one workgroup per tile handed out
            // as slots free up is 6 - 13 % faster than the fixed snake assignment
            const GridPlan plan = g.window > 0 ? GridPlan{tiles_per_xcd, 0}
                                               : plan_persistent_grid(total, q_tiles, resident, g.causal != 0, streamed);
            KernelTimer timer("dq_mfma", stream);
            hipLaunchKernelGGL(kernel, dim3(kXcds * plan.slots), dim3(kBwdThreads), 0, stream, qp, kp, vp, op, gp, lse, delta, dqp,
                               lm, g, q_tiles, total, tiles_per_xcd, plan.deal, dq_columns);
        };
        const bool columns = dq_columns.base != nullptr;
        if (g.window > 0)
            columns ? launch(dq_mfma_kernel<E, D, true, true, true>) : launch(dq_mfma_kernel<E, D, true, true>);
        else if (g.causal)
            columns ? launch(dq_mfma_kernel<E, D, true, false, true>) : launch(dq_mfma_kernel<E, D, true, false>);
        else
            columns ? launch(dq_mfma_kernel<E, D, false, false, true>) : launch(dq_mfma_kernel<E, D, false, false>);
        err = hipGetLastError();
        if (err != hipSuccess) return err;
    }
    // dK, dV
    const int k_tiles = (T + kDkvKeyTile - 1) / kDkvKeyTile;
    const int total = g.packs * g.kv_heads * k_tiles;
    const int tiles_per_xcd = (total + kXcds - 1) / kXcds;
    const long long streamed = 2ll * (g.q_heads / g.kv_heads) * T * D * 2;  // Q and dO of the heads that share a K / V head
    if constexpr (D <= 64) {
        const size_t smem = 2 * sizeof(DkvLds<D>);
        auto launch = [&](auto kernel) {
            static const int resident = resident_workgroups_per_xcd(kernel, kBwdThreads, smem);  // per kernel instantiation
            // under the sparse mask the key tiles are short and of two very different lengths: one workgroup per tile,
            // dispatched in order (long ones first), balances better than a fixed assignment (at head_dim 64 the persistent
            // grid measured the same for short windows without global tokens and worse for every other mask)
            const GridPlan plan = g.window > 0 ? GridPlan{tiles_per_xcd, 0}
                                               : plan_persistent_grid(total, k_tiles, resident, g.causal != 0, streamed);
            KernelTimer timer("dkdv_mfma", stream);
            hipLaunchKernelGGL(kernel, dim3(kXcds * plan.slots), dim3(kBwdThreads), smem, stream, qp, kp, vp, gp, lse, delta, dkp,
                               dvp, lm, g, k_tiles, total, tiles_per_xcd, plan.deal, dk_columns, dv_columns);
        };
        // both gradients go the same way: the column-layout caller passes both sinks, every other caller none
        const bool columns = dk_columns.base && dv_columns.base;
        if (columns != (dk_columns.base || dv_columns.base)) return hipErrorInvalidValue;
        if (g.window > 0)
            columns ? launch(dkdv_mfma_kernel<E, D, true, true, true>) : launch(dkdv_mfma_kernel<E, D, true, true>);
        else if (g.causal)
            columns ? launch(dkdv_mfma_kernel<E, D, true, false, true>) : launch(dkdv_mfma_kernel<E, D, true, false>);
        else
            columns ? launch(dkdv_mfma_kernel<E, D, false, false, true>) : launch(dkdv_mfma_kernel<E, D, false, false>);
        err = hipGetLastError();
    } else {
        const size_t smem = sizeof(DkvSplitLds<D>);
        auto launch = [&](auto kernel) -> hipError_t {
            // one-time per kernel instantiation: opt in to more than 64 KiB of LDS, then ask how many workgroups fit
            static const hipError_t raised = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                                 hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
            if (raised != hipSuccess) return raised;
            static const int resident = resident_workgroups_per_xcd(kernel, kDkvSplitThreads, smem);
            // under the sparse mask the key tiles are short and, with global tokens, of two very different lengths: one
            // workgroup per tile, dispatched in order (long ones first), balances better than a fixed assignment; without
            // global tokens and with a window of a few stages all tiles are alike and the persistent grid (snake) saves
            // the workgroup launches (measured at d = 128, T = 4096: window 128 0.267 -> 0.238 ms, window 512
            // 0.405 -> 0.395 ms, window 2048 0.870 -> 0.925 ms; T = 2048: window 256 0.172 -> 0.152 ms)
            const bool alike = g.window > 0 && g.window <= kMaxPersistentWindow && g.global_tokens == 0 && tiles_per_xcd > resident;
            const GridPlan plan = g.window > 0 ? GridPlan{alike ? resident : tiles_per_xcd, 0}
                                               : plan_persistent_grid(total, k_tiles, resident, g.causal != 0, streamed);
            KernelTimer timer("dkdv_mfma", stream);
            hipLaunchKernelGGL(kernel, dim3(kXcds * plan.slots), dim3(kDkvSplitThreads), smem, stream, qp, kp, vp, gp, lse, delta, dkp,
                               dvp, lm, g, k_tiles, total, tiles_per_xcd, plan.deal, dk_columns, dv_columns);
            return hipGetLastError();
        };
        const bool columns = dk_columns.base && dv_columns.base;
        if (columns != (dk_columns.base || dv_columns.base)) return hipErrorInvalidValue;
        if (g.window > 0)
            err = columns ? launch(dkdv_split_kernel<E, D, true, true, true>) : launch(dkdv_split_kernel<E, D, true, true>);
        else if (g.causal)
            err = columns ? launch(dkdv_split_kernel<E, D, true, false, true>) : launch(dkdv_split_kernel<E, D, true, false>);
        else
            err = columns ? launch(dkdv_split_kernel<E, D, false, false, true>) : launch(dkdv_split_kernel<E, D, false, false>);
    }
    return err;
}

}  // namespace

hipError_t launch_bwd_mfma(Elem type, const void* q, const void* k, const void* v, const void* out, const float* lse,
                           RowMap lm, const void* d_out, void* dq, void* dk, void* dv, float* delta, AttnGeom g,
                           hipStream_t stream, ColumnSink dq_columns, ColumnSink dk_columns, ColumnSink dv_columns) {
    if (type == Elem::BF16) {
        if (g.head_dim == 64) return run_bwd<Bf16, 64>(q, k, v, out, lse, lm, d_out, dq, dk, dv, delta, g, stream, dq_columns, dk_columns,
                                                              dv_columns);
        if (g.head_dim == 128) return run_bwd<Bf16, 128>(q, k, v, out, lse, lm, d_out, dq, dk, dv, delta, g, stream, dq_columns, dk_columns,
                                                              dv_columns);
    } else if (type == Elem::F16) {
        if (g.head_dim == 64) return run_bwd<Fp16, 64>(q, k, v, out, lse, lm, d_out, dq, dk, dv, delta, g, stream, dq_columns, dk_columns,
                                                              dv_columns);
        if (g.head_dim == 128) return run_bwd<Fp16, 128>(q, k, v, out, lse, lm, d_out, dq, dk, dv, delta, g, stream, dq_columns, dk_columns,
                                                              dv_columns);
    }
    return hipErrorInvalidValue;
}

}  // namespace sentinel_hip
