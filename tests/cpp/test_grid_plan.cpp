// Host-side check of the persistent grids' tile assignment (sentinel_amd/csrc/grid_plan.h: tile_of_slot,
// plan_persistent_grid).  Plain C++, needs neither a GPU nor the HIP compiler: it runs the index arithmetic the kernels use.
#include "../../sentinel_amd/csrc/grid_plan.h"

#include <cstdio>
#include <vector>

using namespace sentinel_hip;

static int failures = 0;
#define EXPECT(cond, ...)                 \
    do {                                  \
        if (!(cond)) {                    \
            ++failures;                   \
            std::printf("FAIL " __VA_ARGS__); \
            std::printf("\n");            \
        }                                 \
    } while (0)

// every tile of the XCD goes to exactly one (round, workgroup), and a workgroup that finds nothing finds nothing later
static void check_cover(int slots, int tiles_per_xcd, int tiles_per_head, int deal) {
    std::vector<int> seen(tiles_per_xcd, 0);
    for (int slot = 0; slot < slots; ++slot) {
        bool done = false;
        for (int round = 0; round * slots < tiles_per_xcd + slots; ++round) {
            const int tile = tile_of_slot(slot, slots, round, tiles_per_xcd, tiles_per_head, deal);
            if (tile >= tiles_per_xcd) {
                done = true;  // the kernels leave their loop here
                continue;
            }
            EXPECT(tile >= 0, "negative tile");
            EXPECT(!done, "slots %d tiles %d per head %d deal %d: slot %d gets tile %d after an empty round", slots, tiles_per_xcd,
                   tiles_per_head, deal, slot, tile);
            if (tile >= 0) ++seen[tile];
        }
    }
    for (int t = 0; t < tiles_per_xcd; ++t)
        EXPECT(seen[t] == 1, "slots %d tiles %d per head %d deal %d: tile %d taken %d times", slots, tiles_per_xcd, tiles_per_head,
               deal, t, seen[t]);
}

int main() {
    for (int tiles_per_head : {1, 2, 3, 4, 8, 16, 32, 33, 128})
        for (int heads : {1, 2, 3, 12, 16, 48})
            for (int resident : {32, 64, 96}) {
                const int tiles = tiles_per_head * heads;
                const GridPlan plan = plan_persistent_grid(kXcds * tiles, tiles_per_head, resident, true, 1 << 16);
                EXPECT(plan.slots > 0 && plan.slots <= resident, "plan slots %d of %d", plan.slots, resident);
                EXPECT(!plan.deal || plan.slots % kCusPerXcd == 0, "a dealt grid is whole passes");
                check_cover(plan.slots, tiles, tiles_per_head, plan.deal);
                // both orders cover, whichever the plan chose
                check_cover(tiles < resident ? tiles : resident, tiles, tiles_per_head, 0);
                const int passes = (tiles + kCusPerXcd - 1) / kCusPerXcd * kCusPerXcd;
                check_cover(passes < resident ? passes : resident, tiles, tiles_per_head, 1);
            }
    // GPT-2-small shape (8 x 12 heads, T 1024, 128-row tiles): 96 tiles per XCD, 8 per head, 96 resident workgroups.  The
    // snake hands a compute unit three tiles of one length (27 units of work on the busiest against 18 dealt).
    const GridPlan small = plan_persistent_grid(8 * 96, 8, 96, true, 2ll * 1024 * 64 * 2);
    EXPECT(small.deal == 1 && small.slots == 96, "GPT-2-small shape should be dealt: slots %d deal %d", small.slots, small.deal);
    EXPECT(busiest_compute_unit(96, 96, 8, 0) == 27 && busiest_compute_unit(96, 96, 8, 1) == 18, "busiest-unit estimate");
    // two full rounds pair long with short tiles: the snake is already even and stays
    EXPECT(plan_persistent_grid(8 * 192, 4, 96, true, 2ll * 512 * 64 * 2).deal == 0, "an even number of rounds keeps the snake");
    // equal tile lengths (no causal mask), heads cut by the XCD boundary, or operands beyond the footprint limit: snake
    EXPECT(plan_persistent_grid(8 * 96, 8, 96, false, 1 << 16).deal == 0, "equal lengths keep the snake");
    EXPECT(plan_persistent_grid(8 * 100, 8, 96, true, 1 << 16).deal == 0, "partial heads keep the snake");
    // 95 heads of 4 tiles: 48 tiles per XCD are 12 whole heads, but the last XCD holds 11 (its dealt order would meet the
    // missing head's tiles before real ones)
    EXPECT(plan_persistent_grid(95 * 4, 4, 32, true, 1 << 16).deal == 0, "a short last XCD keeps the snake");
    EXPECT(plan_persistent_grid(96 * 4, 4, 32, true, 1 << 16).slots == 32, "slots");
    EXPECT(plan_persistent_grid(8 * 512, 32, 64, true, 2ll * 4096 * 128 * 2).deal == 0, "32 MB of K / V per XCD keeps the snake");
    std::printf(failures ? "%d failures\n" : "grid plan ok\n", failures);
    return failures ? 1 : 0;
}
