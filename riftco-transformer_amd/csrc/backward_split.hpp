// How the small-batch input backward (nf4_small_backward.hip) cuts its work:
// column tiles of 128 outputs times chunks of weight rows.  Plain host
// arithmetic, shared by the launcher and a host-side test.
#pragma once

#include <cstddef>

namespace rthip {

constexpr int kTileColumns = 128;     // output columns of a workgroup
constexpr unsigned kWalkRows = 128;   // weight rows a workgroup walks per step
constexpr unsigned kMaxChunks = 16;   // partial sums the second kernel adds
constexpr unsigned kComputeUnits = 256;

struct BackwardSplit {
    unsigned column_tiles;   // ceil(I / 128)
    unsigned chunks;         // pieces of the weight rows
    unsigned chunk_rows;     // rows per piece, a multiple of 128
    unsigned units_per_xcd;  // ceil(column_tiles * chunks / 8)
};

// One workgroup fits per compute unit, so the kernel takes
// ceil(units / 256) rounds of a chunk's length each; among the chunk counts
// whose partial sums fit the workspace the one with the least
// rounds x chunk length wins (ties: fewer chunks; every further chunk is
// charged the cost of writing and adding one more partial sum).
inline BackwardSplit split_weight_rows(std::size_t rows,
                                       std::size_t input_width,
                                       std::size_t output_width,
                                       std::size_t workspace_bytes) {
    BackwardSplit best{};
    const unsigned column_tiles = static_cast<unsigned>(
        (input_width + kTileColumns - 1) / kTileColumns);
    double best_cost = 0.0;
    for (unsigned chunks = 1; chunks <= kMaxChunks; ++chunks) {
        const unsigned chunk_rows = static_cast<unsigned>(
            ((output_width + chunks - 1) / chunks + kWalkRows - 1) /
            kWalkRows * kWalkRows);
        const unsigned actual = static_cast<unsigned>(
            (output_width + chunk_rows - 1) / chunk_rows);
        if (actual != chunks) {
            continue;  // the same split as a smaller count
        }
        if (chunks > 1 && static_cast<std::size_t>(chunks) * rows *
                                  input_width * sizeof(float) >
                              workspace_bytes) {
            break;
        }
        const unsigned units = column_tiles * chunks;
        const unsigned rounds = (units + kComputeUnits - 1) / kComputeUnits;
        const double cost =
            static_cast<double>(rounds) * chunk_rows + 8.0 * (chunks - 1);
        if (best.chunks == 0 || cost < best_cost) {
            best_cost = cost;
            best.column_tiles = column_tiles;
            best.chunks = chunks;
            best.chunk_rows = chunk_rows;
            best.units_per_xcd = (units + 7) / 8;
        }
    }
    return best;
}

}  // namespace rthip
