// Host-side test of the work split shared by the tiled matrix-core kernels
// (riftco-transformer_amd/csrc/tile_plan.hpp).  No device needed: the plan is
// plain arithmetic that kernels and launchers evaluate alike.
//
// For every (tile count, steps per tile) in a sweep it checks that
//   * whole tiles plus unit-dealt tiles are all the tiles,
//   * the runs are contiguous, cover every (tile, step) unit exactly once and
//     never exceed one tile's worth of steps (so a run touches <= 2 tiles),
//   * owner() inverts begin(),
//   * the workgroups that hold parts of a tile are exactly
//     owner(first unit) .. owner(last unit), and slot() gives each of them a
//     slot of its own (0 for the first tile of its run, 1 for the second).

#include "../../riftco-transformer_amd/csrc/tile_plan.hpp"

#include <cstdio>
#include <cstdlib>
#include <set>
#include <vector>

namespace {

int failures = 0;

void require(bool condition, const char* what, unsigned tiles,
             unsigned steps) {
    if (!condition) {
        std::fprintf(stderr, "tile plan: %s (tiles %u, steps %u)\n", what,
                     tiles, steps);
        ++failures;
    }
}

void check(unsigned tiles, unsigned steps) {
    rthip::TilePlan plan{};
    plan.tiles_n = 7;
    plan.steps = steps;
    const unsigned groups = rthip::plan_tiles(
        plan, tiles, 128 * 128 * sizeof(float), std::size_t{64} << 20);
    if (groups == 0) {
        require(plan.whole_tiles == tiles, "every tile whole", tiles, steps);
        return;
    }
    const unsigned dealt = tiles - plan.whole_tiles;
    require(dealt > 0 && dealt < rthip::kPlanPlaces && dealt < groups,
            "leftover tiles only, more runs than tiles", tiles, steps);
    require(plan.whole_tiles % rthip::kPlanPlaces == 0,
            "whole tiles fill the device evenly", tiles, steps);
    require(groups <= rthip::kPlanPlaces, "no more runs than places", tiles,
            steps);
    const unsigned units = dealt * steps;
    require(plan.begin(0) == 0 && plan.begin(groups) == units,
            "runs cover all units", tiles, steps);
    std::vector<std::set<unsigned>> holders(dealt);
    for (unsigned group = 0; group < groups; ++group) {
        const unsigned begin = plan.begin(group);
        const unsigned end = plan.begin(group + 1);
        require(end > begin && end - begin <= steps, "run length", tiles,
                steps);
        require(end - begin >= rthip::kPlanMinimumRunSteps ||
                    groups == rthip::kPlanPlaces,
                "runs are not shorter than the minimum", tiles, steps);
        require(plan.owner(begin) == group && plan.owner(end - 1) == group,
                "owner inverts begin", tiles, steps);
        const unsigned first_tile = begin / steps;
        const unsigned last_tile = (end - 1) / steps;
        require(last_tile - first_tile <= 1, "a run touches two tiles at most",
                tiles, steps);
        for (unsigned tile = first_tile; tile <= last_tile; ++tile) {
            holders[tile].insert(group);
            require(plan.slot(group, tile) ==
                        group * 2 + (tile == first_tile ? 0U : 1U),
                    "slot numbering", tiles, steps);
        }
    }
    for (unsigned tile = 0; tile < dealt; ++tile) {
        const unsigned first = plan.owner(tile * steps);
        const unsigned last = plan.owner(tile * steps + steps - 1);
        require(holders[tile].size() == last - first + 1 &&
                    *holders[tile].begin() == first &&
                    *holders[tile].rbegin() == last,
                "holders of a tile are a contiguous range of runs", tiles,
                steps);
    }
}

}  // namespace

int main() {
    // the shapes of the benchmark: 2048 x 11008 and 2048 x 4096 outputs
    {
        rthip::TilePlan plan{};
        plan.tiles_n = 86;
        plan.steps = 128;
        const unsigned groups = rthip::plan_tiles(
            plan, 1376, 128 * 128 * sizeof(float), std::size_t{64} << 20);
        require(groups == 512 && plan.whole_tiles == 1024 &&
                    plan.quotient == 88 && plan.remainder == 0,
                "1376 tiles: 1024 whole, 352 in 512 runs of 88 steps", 1376,
                128);
        plan.tiles_n = 32;
        require(rthip::plan_tiles(plan, 512, 128 * 128 * sizeof(float),
                                  std::size_t{64} << 20) == 0,
                "512 tiles: all whole", 512, 128);
    }
    for (unsigned tiles = 1; tiles <= 1600; tiles += (tiles < 40 ? 1 : 7)) {
        for (unsigned steps : {1U, 8U, 15U, 16U, 17U, 33U, 128U, 344U}) {
            check(tiles, steps);
        }
    }
    // too little workspace: no dealing
    {
        rthip::TilePlan plan{};
        plan.tiles_n = 4;
        plan.steps = 64;
        require(rthip::plan_tiles(plan, 100, 128 * 128 * sizeof(float),
                                  std::size_t{1} << 20) == 0,
                "partial tiles must fit the workspace", 100, 64);
    }
    if (failures != 0) {
        return 1;
    }
    std::printf("tile plan tests passed\n");
    return 0;
}
