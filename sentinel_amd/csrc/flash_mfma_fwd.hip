// Causal flash-attention forward on gfx950 matrix cores (bf16 / fp16 operands, fp32 accumulation).
//
// Replaces CudaFlashAttentionForwardWmma64Entry (sentinel/NeuralNet/Cuda/CudaFlashAttention.cu:1105-1266):
// same result (O and per-query LSE = max + ln(sum), natural log of the scaled scores), different design:
//   * tensors are [B, H, T, D] 16-bit, so every global access is a coalesced 128-bit buffer load with
//     a loop-invariant vector offset (the hardware range check zero-fills rows past T); nothing is
//     converted or gathered per tile;
//   * a workgroup of 4 wavefronts owns 128 queries (32 per wavefront) and walks 64-key tiles;
//     Q stays in registers for the whole query tile, K and V tiles are double-buffered in LDS (row-major,
//     XOR-swizzled) and the next tile streams straight into LDS (buffer_load ... lds) while the current one
//     is multiplied;
//   * S^T = K Q^T, so a lane owns one query: the online-softmax max / sum are in-register plus one
//     v_permlane32_swap, and P^T feeds the P V product from registers (no LDS round trip); V^T is read
//     out of the row-major V tile with transposing LDS reads;
//   * the running maximum is only raised (and O rescaled) when a row's maximum grows by more than 2^8,
//     which is exact and keeps P within the 16-bit range;
//   * key tiles above the diagonal are skipped; only tiles that cross it are masked; with Sentinel's sparse mask
//     (sliding window + global tokens, WINDOW) the key tiles below every window of the query tile are skipped too;
//   * grouped-query attention reads the shared K/V head in place;
//   * the grid is persistent (as many workgroups as the device runs at once, each walking several query tiles), the two
//     workgroups of a compute unit take turns at the higher wave priority, and the O rows leave through LDS as whole rows.
#include "flash_common.h"
#include "mfma_tile.h"

namespace sentinel_hip {
namespace {

constexpr int kFwdThreads = 256;
constexpr int kFwdQueryTile = 128;
// instruction classes of __builtin_amdgcn_sched_group_barrier
constexpr int kSchedMfma = 0x008;
constexpr int kSchedDsRead = 0x100;
constexpr int kSchedVmem = 0x010;
constexpr int kOperandLead = 4;

constexpr int kFwdKeyTile = 64;

template <typename E, int D, bool CAUSAL, bool WINDOW>
__global__ __launch_bounds__(kFwdThreads, D <= 64 ? 3 : 2) void fwd_mfma_kernel(const unsigned short* __restrict__ q,
                                                                   const unsigned short* __restrict__ k,
                                                                   const unsigned short* __restrict__ v,
                                                                   unsigned short* __restrict__ out,
                                                                   float* __restrict__ lse, RowMap lm, AttnGeom g,
                                                                   int q_tiles, int total_tiles, int tiles_per_xcd, int deal,
                                                                   ColumnSink out_columns) {
    constexpr int KT = kFwdKeyTile;
    typedef DirectTile<KT, D, kFwdThreads> Tile;
    constexpr int KSTEPS = D / 16;  // k-steps of the S^T product
    constexpr int CB = D / 32;      // 32-row blocks of O^T

    // two stages of (K, V) tiles; separate arrays so that the loads streaming into one stage are known not to
    // alias the operand reads of the other (one array indexed by stage makes the compiler wait for the loads
    // before every LDS read)
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

    // Persistent workgroups: the grid holds as many workgroups as the device runs at once and each walks several
    // query tiles (launching a workgroup costs about 5 us of its slot, a sixth of an average tile at T = 4096).
    // Workgroup ids are dealt round-robin to the 8 XCDs; each XCD owns a contiguous range of tiles (head-major,
    // longest query tile of a head first), so the query tiles of one head, which stream the same K / V, share one
    // L2.  tile_of_slot hands them out in the order the host chose (plan_persistent_grid), so that every workgroup and
    // every compute unit ends up with about the same work.
    const unsigned turn_class = priority_turn_class();
    const int xcd = (int)blockIdx.x % kXcds;
    const int slot = (int)blockIdx.x / kXcds;
    const int slots = (int)gridDim.x / kXcds;
    for (int round = 0;; ++round) {
    // (under the sparse mask one workgroup per tile is launched, more than run at once, and tile lengths do not follow
    //  the tile index: plain order)
    const int local_tile = WINDOW ? round * slots + slot
                                  : __builtin_amdgcn_readfirstlane(tile_of_slot(slot, slots, round, tiles_per_xcd, q_tiles, deal));
    const int tile_id = xcd * tiles_per_xcd + local_tile;
    if (local_tile >= tiles_per_xcd || tile_id >= total_tiles) break;
    const int bh = tile_id / q_tiles;
    const int qt = q_tiles - 1 - tile_id % q_tiles;  // longest first within a head
    const int b = bh / g.q_heads;
    const int h = bh % g.q_heads;
    const int kvh = h / (g.q_heads / g.kv_heads);

    const unsigned short* qb = q + ((long long)b * g.q_heads + h) * T * D;
    const unsigned short* kb = k + ((long long)b * g.kv_heads + kvh) * T * D;
    const unsigned short* vb = v + ((long long)b * g.kv_heads + kvh) * T * D;

    const int q0w = qt * kFwdQueryTile + wave * 32;  // first query of this wavefront
    const int qrow = q0w + n;
    const int qload = qrow < T ? qrow : T - 1;

    // Q^T as B operand: column = query, contraction over head dims
    u32x4 qf[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
        qf[ks] = *reinterpret_cast<const u32x4*>(qb + (long long)qload * D + ks * 16 + gh * 8);

    const int q_hi = min(T, (qt + 1) * kFwdQueryTile);        // one past the last query of the tile
    const int kv_tiles = CAUSAL ? (q_hi + KT - 1) / KT : (T + KT - 1) / KT;
    // WINDOW: the key tiles this query tile sees are the ones holding global tokens, [0, g_tiles), and those from
    // the window of its first query up to the diagonal, [w_first, kv_tiles); trip `it` works on tile_of(it)
    static_assert(CAUSAL || !WINDOW, "the sparse mask refines the causal one");
    int g_tiles = 0, w_first = 0;
    if (WINDOW) {
        g_tiles = min(kv_tiles, (g.global_tokens + KT - 1) / KT);
        w_first = max(g_tiles, max(0, qt * kFwdQueryTile - g.window + 1) / KT);
    }
    const int n_trips = WINDOW ? g_tiles + (kv_tiles - w_first) : kv_tiles;
    auto tile_of = [&](int it) { return WINDOW ? (it < g_tiles ? it : it - g_tiles + w_first) : it; };

    const __amdgpu_buffer_rsrc_t k_rsrc = make_head_rsrc(kb, (long long)T * D * 2);
    const __amdgpu_buffer_rsrc_t v_rsrc = make_head_rsrc(vb, (long long)T * D * 2);
    const int ld_off = Tile::global_offset(tid);
    Tile::issue(k_rsrc, k_lds0, ld_off, tile_of(0) * KT * D * 2, wave);
    Tile::issue(v_rsrc, v_lds0, ld_off, tile_of(0) * KT * D * 2, wave);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) pin_loaded(qf[ks]);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the first tiles have landed in LDS
    __syncthreads();

    f32x16 acc[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[cb][i] = 0.0f;
    // Under the sparse mask a row can meet a tile in which all its keys are masked before it meets a visible key:
    // a finite floor keeps exp2(-inf - m) = 0 there instead of exp2(-inf + inf)
    float m_run = WINDOW ? -1e30f : -__builtin_inff();
    float l_run = 0.0f;  // this lane's half of the row sum
    const float c2 = g.scale * kLog2e;

    const int k_off = Tile::row_read_base(row_perm(n), gh);  // K operand read: row carried by D row n
    const int t_even = Tile::transposed_read_base(lane, 0);  // V^T operand reads out of the row-major V tile
    const int t_odd = Tile::transposed_read_base(lane, 1);
    const float raise_after = 8.0f;                // log2 units a row maximum may grow before O is rescaled

    // one trip over the tile held in (k_cur, v_cur); the next tile streams into (k_next, v_next) meanwhile
    auto tile_trip = [&](int j, const unsigned short* k_cur, const unsigned short* v_cur, unsigned short* k_next,
                         unsigned short* v_next) __attribute__((always_inline)) {
        // the next tile's requests go out between the matrix instructions of the score chains (a wavefront is held for
        // 40 - 60 cycles per request, which then passes while its own matrix instructions run); the last trip fetches
        // its own tile once more, which nobody reads
        const int next_bytes = tile_of(j + 1 < n_trips ? j + 1 : j) * KT * D * 2;
        // (under the sparse mask a wavefront may skip trips in mid-tile; there the requests go out first, as a block)
        constexpr bool SPREAD = !WINDOW;
        if (!SPREAD && j + 1 < n_trips) {
            Tile::issue(k_rsrc, k_next, ld_off, next_bytes, wave);
            Tile::issue(v_rsrc, v_next, ld_off, next_bytes, wave);
        }

        const int key0 = tile_of(j) * KT;
        // wavefront-uniform: the whole tile lies above this wavefront's diagonal, or holds no global token and
        // lies below the window of this wavefront's first query
        const bool skip = (CAUSAL && key0 > q0w + 31) ||
                          (WINDOW && key0 >= g.global_tokens && key0 + KT - 1 < q0w - g.window + 1);
        if (!skip) {
            // S^T chains with their K operands read kOperandLead instructions ahead; the V^T operands of the first
            // half of the PV product are fetched behind them and land during the softmax arithmetic
            f32x16 s[2];
            u32x4 kfrag[2][KSTEPS];
            u32x4 vfrag[4][CB];
#pragma unroll
            for (int kbk = 0; kbk < 2; ++kbk)
#pragma unroll
                for (int ks = 0; ks < KSTEPS; ++ks) kfrag[kbk][ks] = lds_read128(k_cur + kbk * 32 * D + (k_off ^ (ks << 4)));
#pragma unroll
            for (int kbk = 0; kbk < 2; ++kbk) {
#pragma unroll
                for (int i = 0; i < 16; ++i) s[kbk][i] = 0.0f;
#pragma unroll
                for (int ks = 0; ks < KSTEPS; ++ks) s[kbk] = E::mfma(kfrag[kbk][ks], qf[ks], s[kbk]);
            }
            if (SPREAD) {
                Tile::issue(k_rsrc, k_next, ld_off, next_bytes, wave);
                Tile::issue(v_rsrc, v_next, ld_off, next_bytes, wave);
            }
#pragma unroll
            for (int c4 = 0; c4 < 2; ++c4)
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
                    vfrag[c4][cb] = lds_read_transposed_pair(v_cur + c4 * 16 * D + (t_even ^ (cb << 5)),
                                                             v_cur + c4 * 16 * D + (t_odd ^ (cb << 5)));
            static_assert(2 * Tile::kIters == KSTEPS, "one request per two matrix instructions of the score chains");
            __builtin_amdgcn_sched_group_barrier(kSchedDsRead, kOperandLead, 0);
#pragma unroll
            for (int i = 0; i < 2 * KSTEPS - kOperandLead; ++i) {
                __builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
                __builtin_amdgcn_sched_group_barrier(kSchedDsRead, 1, 0);
                if (SPREAD && (i & 1)) __builtin_amdgcn_sched_group_barrier(kSchedVmem, 1, 0);
            }
#pragma unroll
            for (int i = 0; i < kOperandLead; ++i) {
                __builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
                __builtin_amdgcn_sched_group_barrier(kSchedDsRead, 4 * CB / kOperandLead, 0);
                if (SPREAD && (i & 1)) __builtin_amdgcn_sched_group_barrier(kSchedVmem, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);

            // also when the tile's first key outside the global range lies below the window of the wavefront's last query
            const bool need_mask = (CAUSAL && key0 + KT - 1 > q0w) || (!CAUSAL && key0 + KT > T) ||
                                   (WINDOW && key0 + KT > g.global_tokens && max(key0, g.global_tokens) < q0w + 32 - g.window);
            if (need_mask) {
#pragma unroll
                for (int kbk = 0; kbk < 2; ++kbk)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int key = key0 + kbk * 32 + perm_row_of_reg(i, gh);
                        const bool dead = CAUSAL ? (key > qrow || (WINDOW && outside_window(g, qrow, key))) : key >= T;
                        if (dead) s[kbk][i] = -__builtin_inff();
                    }
            }

            float mx = s[0][0];
#pragma unroll
            for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s[0][i]);
#pragma unroll
            for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[1][i]);
            mx = half_max(mx);
            // raise the reference maximum only when some row outgrew it by more than 2^raise_after
            if (__any((mx - m_run) * c2 > raise_after)) {
                const float m_new = fmaxf(m_run, mx);
                const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c2);
                l_run *= alpha;
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[cb][i] *= alpha;
                m_run = m_new;
            }
            const float mc = m_run * c2;

            float psum = 0.0f;
            u32x4 pf[4];  // P^T as B operand, four 16-key k-steps
#pragma unroll
            for (int kbk = 0; kbk < 2; ++kbk) {
#pragma unroll
                for (int half = 0; half < 2; ++half) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kbk][half * 8 + 2 * e], c2, -mc));
                        const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kbk][half * 8 + 2 * e + 1], c2, -mc));
                        psum += p0 + p1;
                        pf[kbk * 2 + half][e] = E::pack2(p0, p1);
                    }
                }
            }
            l_run += psum;

            __builtin_amdgcn_sched_barrier(0);
            // PV: the first half runs on the operands fetched above while the second half's are read
#pragma unroll
            for (int c4 = 2; c4 < 4; ++c4)
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
                    vfrag[c4][cb] = lds_read_transposed_pair(v_cur + c4 * 16 * D + (t_even ^ (cb << 5)),
                                                             v_cur + c4 * 16 * D + (t_odd ^ (cb << 5)));
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4)
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) acc[cb] = E::mfma(vfrag[c4][cb], pf[c4], acc[cb]);
#pragma unroll
            for (int i = 0; i < 2 * CB; ++i) {
                __builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
                __builtin_amdgcn_sched_group_barrier(kSchedDsRead, 2, 0);
            }
            __builtin_amdgcn_sched_group_barrier(kSchedMfma, 2 * CB, 0);
            __builtin_amdgcn_sched_barrier(0);
        }  // (under the plain causal mask a wavefront skips only the last trip of its tile, after which nothing is read)

        // priority turns: for the persistent grid with two workgroups per compute unit (head_dim 128) only
        constexpr bool TURNS = !WINDOW && D > 64;
        const unsigned now = TURNS ? (unsigned)__builtin_amdgcn_s_memrealtime() : 0u;
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this thread's share of the next tile is in LDS
        __syncthreads();
        if (TURNS) take_priority_turn(now, turn_class);
    };
    for (int j = 0; j < n_trips; j += 2) {
        tile_trip(j, k_lds0, v_lds0, k_lds1, v_lds1);
        if (j + 1 < n_trips) tile_trip(j + 1, k_lds1, v_lds1, k_lds0, v_lds0);
    }

    const float l_tot = half_sum(l_run);
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    // O rows leave through the second LDS stage, which no wavefront reads or fills any more: the last trip ended with a
    // barrier, and the next tile's first loads go to stage 0 and are followed by a barrier before stage 1 is filled
    store_rows_via_lds<E, D, false>(acc, inv, (wave < 2 ? k_lds1 : v_lds1) + (wave & 1) * (32 * D),
                             out + ((long long)b * g.q_heads + h) * T * D + (long long)q0w * D, T - q0w, lane);
    // the caller's fp32 column matrix, if it keeps O that way: straight from the accumulators, unrounded
    if (out_columns.base)
        store_columns_f32<D, false>(acc, inv,
                                    out_columns.base + (long long)h * out_columns.head_dim * out_columns.stride + (long long)b * T + q0w,
                                    (int)out_columns.stride, T - q0w, out_columns.head_dim, lane, nullptr, nullptr, 0, 0);
    if (qrow < T && gh == 0)
        lse[b * lm.pack_stride + h * lm.head_stride + qrow] = m_run * g.scale + (l_tot > 0.0f ? __logf(l_tot) : 0.0f);
    }  // next tile of this workgroup (the last trip ended with a barrier: the LDS stages are free)
}

template <typename E, int D>
hipError_t run_fwd(const void* q, const void* k, const void* v, void* out, float* lse, RowMap lm, AttnGeom g,
                   hipStream_t stream, ColumnSink out_columns) {
    const int q_tiles = (g.seq_len + kFwdQueryTile - 1) / kFwdQueryTile;
    const int total = g.packs * g.q_heads * q_tiles;
    const int tiles_per_xcd = (total + kXcds - 1) / kXcds;
    const long long streamed = 2ll * g.seq_len * D * 2;  // K and V of a head
    auto qp = static_cast<const unsigned short*>(q);
    auto kp = static_cast<const unsigned short*>(k);
    auto vp = static_cast<const unsigned short*>(v);
    auto op = static_cast<unsigned short*>(out);
    auto launch = [&](auto kernel) {
        static const int resident = resident_workgroups_per_xcd(kernel, kFwdThreads, 0);  // per kernel instantiation
        // under the sparse mask tile lengths no longer grow with the tile index, and one workgroup per tile handed out
        // as slots free up is 6 - 13 % faster than a fixed assignment; only where a tile is a few trips long (windows up
        // to two query tiles) the 5 us a workgroup costs to launch weigh more, and the persistent grid, tiles in plain
        // order, is 5 % faster (measured at d = 128, T = 4096: window 128 0.174 -> 0.166 ms, window 512 0.239 -> 0.249 ms;
        // T = 2048: window 64 0.085 -> 0.078 ms, window 256 0.109 -> 0.103 ms; no difference at d = 64)
        const bool short_window = g.window > 0 && g.window <= 2 * kFwdQueryTile && tiles_per_xcd > resident;
        const GridPlan plan = g.window > 0 ? GridPlan{short_window ? resident : tiles_per_xcd, 0}
                                           : plan_persistent_grid(total, q_tiles, resident, g.causal != 0, streamed);
        KernelTimer timer("fwd_mfma", stream);
        hipLaunchKernelGGL(kernel, dim3(kXcds * plan.slots), dim3(kFwdThreads), 0, stream, qp, kp, vp, op, lse, lm, g, q_tiles,
                           total, tiles_per_xcd, plan.deal, out_columns);
    };
    if (g.window > 0)
        launch(fwd_mfma_kernel<E, D, true, true>);
    else if (g.causal)
        launch(fwd_mfma_kernel<E, D, true, false>);
    else
        launch(fwd_mfma_kernel<E, D, false, false>);
    return hipGetLastError();
}

}  // namespace

bool mfma_supported(int head_dim) { return head_dim == 64 || head_dim == 128; }

hipError_t launch_fwd_mfma(Elem type, const void* q, const void* k, const void* v, void* out, float* lse, RowMap lm,
                           AttnGeom g, hipStream_t stream, ColumnSink out_columns) {
    if (type == Elem::BF16) {
        if (g.head_dim == 64) return run_fwd<Bf16, 64>(q, k, v, out, lse, lm, g, stream, out_columns);
        if (g.head_dim == 128) return run_fwd<Bf16, 128>(q, k, v, out, lse, lm, g, stream, out_columns);
    } else if (type == Elem::F16) {
        if (g.head_dim == 64) return run_fwd<Fp16, 64>(q, k, v, out, lse, lm, g, stream, out_columns);
        if (g.head_dim == 128) return run_fwd<Fp16, 128>(q, k, v, out, lse, lm, g, stream, out_columns);
    }
    return hipErrorInvalidValue;
}

}  // namespace sentinel_hip
