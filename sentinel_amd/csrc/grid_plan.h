// Tile assignment of the persistent attention kernels: which tile a workgroup takes in which round (tile_of_slot, used by
// the kernels and by the host) and the host's choice between the two orders (plan_persistent_grid).  Plain C++: the
// kernels include it through mfma_tile.h, host-only checks build it with any C++ compiler.
#ifndef SENTINEL_HIP_GRID_PLAN_H
#define SENTINEL_HIP_GRID_PLAN_H

#include <mutex>

#if defined(__HIPCC__)
#define SENTINEL_HIP_HOST_DEVICE __host__ __device__
#else
#define SENTINEL_HIP_HOST_DEVICE
#endif

namespace sentinel_hip {

// The device is built from kXcds accelerator dies (XCDs), each with its own L2; the hardware deals workgroup ids
// round-robin to them, so workgroup id % kXcds names the die a workgroup runs on.
constexpr int kXcds = 8;

// Which tile of its XCD a workgroup of a persistent grid takes in `round`.  The XCD's tiles are numbered head-major,
// the longest tile of a head first (the last query tile, or the first key tile, under the causal mask);
// `slot` = workgroup id / kXcds of `slots`.
// * Snake (deal == 0): round r hands tiles [r S, (r + 1) S) to the S workgroups, forwards in even rounds and backwards
//   in odd ones, so long and short tiles alternate for every workgroup and the tiles of a head stay neighbours (they
//   share that head's streamed operands in the XCD's L2).
// * Dealt (deal != 0; the host asks for it on small problems, see plan_persistent_grid): the hardware places workgroups
//   s, s + 32, s + 64 .. of an XCD on the same compute unit (32 per XCD), and with head-major numbering those are tiles
//   of the same length whenever the tiles per head divide 32: one compute unit would get only the longest tiles, another
//   only the shortest (a factor of 8 at 8 tiles per head).  The tiles are taken length-major instead (all longest
//   first) and dealt to the compute units like cards, 32 per pass, forwards in even passes and backwards in odd ones;
//   the passes of a round go to the compute unit's workgroups in turn, in reversed order in odd rounds (the workgroup
//   that got the shorter tile of a round takes the longer one of the next).
// Returns the head-major tile index inside the XCD (>= tiles_per_xcd: nothing left for this workgroup).
constexpr int kCusPerXcd = 32;
SENTINEL_HIP_HOST_DEVICE inline __attribute__((always_inline)) int tile_of_slot(int slot, int slots, int round, int tiles_per_xcd, int tiles_per_head, int deal) {
    if (deal) {
        const int passes = slots / kCusPerXcd;
        const int turn = slot / kCusPerXcd, cu = slot % kCusPerXcd;
        const int pass = round * passes + ((round & 1) ? passes - 1 - turn : turn);
        const int sorted = pass * kCusPerXcd + ((pass & 1) ? kCusPerXcd - 1 - cu : cu);  // position in length-major order
        if (sorted >= tiles_per_xcd) return tiles_per_xcd;
        // position `sorted` of the length-major order = tile `rank` (0: longest) of head sorted - rank * heads; scalar
        // loops over the few tiles of a head instead of two divisions by run-time values (whose temporaries cost the
        // 256-register kernels a spill)
        int heads = 0;
        for (int t = 0; t < tiles_per_xcd; t += tiles_per_head) ++heads;
        int rank = 0, first = 0;
        while (first + heads <= sorted) {
            first += heads;
            ++rank;
        }
        return (sorted - first) * tiles_per_head + rank;
    }
    return round * slots + ((round & 1) ? slots - 1 - slot : slot);
}

// Grid of a persistent kernel over `total_tiles` tiles (an eighth per XCD, rounded up), `tiles_per_head` of them per head, `resident` workgroups
// running at once per XCD; `streamed_bytes_per_head` = the operands every tile of a head streams (K and V, or Q and dO).
// Chooses between the head-major snake and the length-major deal of tile_of_slot:
// * the deal gives up the reuse of a head's streamed operands between neighbouring workgroups, so it is considered only
//   while the XCD's heads together stream at most 8 MB (twice its L2; measured: up to there the order of the tiles does
//   not change a kernel's time, at 16 MB and more the deal costs 2 - 35 %);
// * of the two, the plan whose busiest compute unit has less work wins (tile of rank r of a head counted as
//   tiles_per_head - r steps plus one for its prologue), the snake on a tie or a gain under 3 %: it is already even
//   when a whole, even number of rounds pairs every long tile with a short one.
// A dealt grid is a whole number of passes of 32 workgroups per XCD; the spare workgroups find nothing and leave.
struct GridPlan {
    int slots;  // workgroups per XCD
    int deal;   // argument of tile_of_slot
};
inline long long busiest_compute_unit(int slots, int tiles_per_xcd, int tiles_per_head, int deal) {
    long long load[kCusPerXcd] = {};
    for (int round = 0; round * slots < tiles_per_xcd; ++round)
        for (int slot = 0; slot < slots; ++slot) {
            const int tile = tile_of_slot(slot, slots, round, tiles_per_xcd, tiles_per_head, deal);
            if (tile < tiles_per_xcd) load[slot % kCusPerXcd] += tiles_per_head - tile % tiles_per_head + 1;
        }
    long long most = 0;
    for (long long l : load) most = l > most ? l : most;
    return most;
}
inline GridPlan plan_persistent_grid(int total_tiles, int tiles_per_head, int resident, bool lengths_differ,
                                     long long streamed_bytes_per_head) {
    constexpr long long kDealFootprintLimit = 8ll << 20;
    const int tiles_per_xcd = (total_tiles + kXcds - 1) / kXcds;
    const GridPlan snake{tiles_per_xcd < resident ? tiles_per_xcd : resident, 0};
    // (every XCD must hold the same whole number of heads: the kernels leave their loop at the first tile past the end
    //  of the problem, and only the snake meets those last; with one tile per head all tiles are alike and there is
    //  nothing to deal)
    if (!lengths_differ || tiles_per_head <= 1 || resident % kCusPerXcd != 0 || tiles_per_xcd % tiles_per_head != 0 ||
        total_tiles != kXcds * tiles_per_xcd)
        return snake;
    if (tiles_per_xcd / tiles_per_head * streamed_bytes_per_head > kDealFootprintLimit) return snake;
    // Comparing the two orders walks every tile of an XCD twice (tens of microseconds for thousands of short tiles, as much
    // as the kernel it plans): a training step asks for the same few plans over and over, so the answers are remembered.
    struct Known {
        int total_tiles, tiles_per_head, resident;
        GridPlan plan;
    };
    constexpr int kKnown = 16;
    static Known known[kKnown];
    static int known_count = 0, next_slot = 0;
    static std::mutex guard;
    {
        std::lock_guard<std::mutex> lock(guard);
        for (int i = 0; i < known_count; ++i)
            if (known[i].total_tiles == total_tiles && known[i].tiles_per_head == tiles_per_head && known[i].resident == resident)
                return known[i].plan;
    }
    const int passes = (tiles_per_xcd + kCusPerXcd - 1) / kCusPerXcd * kCusPerXcd;
    const GridPlan dealt{passes < resident ? passes : resident, 1};
    const long long snake_most = busiest_compute_unit(snake.slots, tiles_per_xcd, tiles_per_head, 0);
    const long long dealt_most = busiest_compute_unit(dealt.slots, tiles_per_xcd, tiles_per_head, 1);
    const GridPlan plan = dealt_most * 100 < snake_most * 97 ? dealt : snake;
    {
        std::lock_guard<std::mutex> lock(guard);
        known[next_slot] = Known{total_tiles, tiles_per_head, resident, plan};
        next_slot = (next_slot + 1) % kKnown;
        if (known_count < kKnown) ++known_count;
    }
    return plan;
}

}  // namespace sentinel_hip
#endif
