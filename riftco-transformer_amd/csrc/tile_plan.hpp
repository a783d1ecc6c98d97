// How the tiled matrix-core kernels (nf4_mfma.hip, dense_matmul.hip) cover an
// output whose tile count does not fill the device evenly.
//
// Tiles are numbered row-major (tile / tiles_n is the tile row).  The first
// `whole_tiles` workgroups of a launch take one whole tile each.  The tiles
// after those are cut along the contraction into (tile, step) units -- one
// contraction step of one tile, tile-major -- which are dealt to the remaining
// workgroups in contiguous runs: the first `remainder` of them take
// quotient + 1 units, the others quotient.  A run never exceeds one tile's
// worth of steps, so it touches at most two tiles; a run that covers a whole
// tile writes the output as usual, the others write partial tiles to a
// workspace (slot 2 g for the first tile of workgroup g's run, 2 g + 1 for the
// second) and a second kernel adds the parts of each tile in ascending
// workgroup order.  Whole-tile workgroups come first in the grid and the
// shorter runs last, which is also the order in which the device starts them.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>

namespace rthip {

struct TilePlan {
    unsigned tiles_n;      // output tiles per tile row (of this launch)
    unsigned whole_tiles;  // tiles computed by one workgroup each
    unsigned steps;        // contraction steps per tile
    unsigned quotient;
    unsigned remainder;
    // A launch may cover only the tile columns [first_tile_n, first_tile_n +
    // tiles_n) of the output.
    unsigned first_tile_n = 0;

    __host__ __device__ unsigned tile_row(unsigned tile) const {
        return tile / tiles_n;
    }
    __host__ __device__ unsigned tile_column(unsigned tile) const {
        return first_tile_n + tile % tiles_n;
    }

    __host__ __device__ unsigned begin(unsigned group) const {
        return group * quotient + (group < remainder ? group : remainder);
    }
    __host__ __device__ unsigned owner(unsigned unit) const {
        const unsigned boundary = remainder * (quotient + 1);
        return unit < boundary ? unit / (quotient + 1)
                               : remainder + (unit - boundary) / quotient;
    }
    // Slot of workgroup `group`'s part of unit-dealt tile `dealt_tile`.
    __host__ __device__ unsigned slot(unsigned group,
                                      unsigned dealt_tile) const {
        return group * 2 + (dealt_tile == begin(group) / steps ? 0U : 1U);
    }
};

// Workgroups of 256 threads the device holds at once: two per compute unit
// (`places` of plan_tiles unless the caller's workgroups are another size).
constexpr unsigned kPlanPlaces = 512;
// A run is at least this many steps, and unit dealing is not worth a second
// kernel when the leftover tiles nearly fill the device anyway.
constexpr unsigned kPlanMinimumRunSteps = 8;

// Decides the split for `tiles` tiles of `plan.steps` steps each (tiles_n and
// steps already set).  Returns the number of unit-dealt workgroups; zero means
// every tile is computed whole.  slot_bytes: size of one partial tile;
// workspace_bytes: room for the partial tiles.
inline unsigned plan_tiles(TilePlan& plan, unsigned tiles,
                           std::size_t slot_bytes,
                           std::size_t workspace_bytes,
                           unsigned places = kPlanPlaces) {
    plan.whole_tiles = tiles;
    plan.quotient = 0;
    plan.remainder = 0;
    const unsigned leftover = tiles % places;
    if (leftover == 0 || leftover * 10 >= places * 9 ||
        plan.steps < 2 * kPlanMinimumRunSteps ||
        static_cast<std::size_t>(places) * 2 * slot_bytes >
            workspace_bytes) {
        return 0;
    }
    const unsigned units = leftover * plan.steps;
    unsigned groups = units / kPlanMinimumRunSteps;
    if (groups > places) {
        groups = places;
    }
    if (groups <= leftover) {
        return 0;  // runs of a whole tile: nothing to deal
    }
    plan.whole_tiles = tiles - leftover;
    plan.quotient = units / groups;
    plan.remainder = units % groups;
    return groups;
}

}  // namespace rthip
