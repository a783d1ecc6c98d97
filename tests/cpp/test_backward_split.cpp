// Host-side test of the work split of the small-batch input backward
// (riftco-transformer_amd/csrc/backward_split.hpp).  No device needed.
//
// For a sweep of shapes it checks that the chunks are whole walk steps, cover
// every weight row exactly once, that their partial sums fit the workspace,
// that every (tile, chunk) unit gets a workgroup, and that no admissible
// chunk count would take fewer rounds x rows.

#include "../../riftco-transformer_amd/csrc/backward_split.hpp"

#include <cstdio>
#include <initializer_list>

namespace {

int failures = 0;

void require(bool condition, const char* what, std::size_t rows,
             std::size_t input_width, std::size_t output_width) {
    if (!condition) {
        std::fprintf(stderr, "backward split: %s (rows %zu, I %zu, O %zu)\n",
                     what, rows, input_width, output_width);
        ++failures;
    }
}

void check(std::size_t rows, std::size_t input_width,
           std::size_t output_width, std::size_t workspace) {
    using namespace rthip;
    const BackwardSplit split =
        split_weight_rows(rows, input_width, output_width, workspace);
    const auto bad = [&](const char* what) {
        require(false, what, rows, input_width, output_width);
    };
    if (split.chunks < 1 || split.chunks > kMaxChunks) {
        bad("chunk count in range");
        return;
    }
    if (split.chunk_rows == 0 || split.chunk_rows % kWalkRows != 0) {
        bad("chunks are whole walk steps");
    }
    // chunks 0 .. chunks - 1 cover [0, output_width) and none is empty
    if (static_cast<std::size_t>(split.chunks) * split.chunk_rows <
            output_width ||
        static_cast<std::size_t>(split.chunks - 1) * split.chunk_rows >=
            output_width) {
        bad("chunks cover every weight row, none is empty");
    }
    if (split.column_tiles * static_cast<std::size_t>(kTileColumns) <
            input_width ||
        (split.column_tiles - 1) * static_cast<std::size_t>(kTileColumns) >=
            input_width) {
        bad("column tiles cover the row width");
    }
    if (split.units_per_xcd * 8U < split.column_tiles * split.chunks ||
        (split.units_per_xcd - 1) * 8U >= split.column_tiles * split.chunks) {
        bad("one workgroup per unit, at most seven idle");
    }
    if (split.chunks > 1 && static_cast<std::size_t>(split.chunks) * rows *
                                    input_width * sizeof(float) >
                                workspace) {
        bad("partial sums fit the workspace");
    }
    // no admissible split is cheaper under the same measure
    const auto cost = [&](unsigned chunks, unsigned chunk_rows) {
        const unsigned units = split.column_tiles * chunks;
        const unsigned rounds = (units + kComputeUnits - 1) / kComputeUnits;
        return static_cast<double>(rounds) * chunk_rows + 8.0 * (chunks - 1);
    };
    const double chosen = cost(split.chunks, split.chunk_rows);
    for (unsigned chunks = 1; chunks <= kMaxChunks; ++chunks) {
        const unsigned chunk_rows = static_cast<unsigned>(
            ((output_width + chunks - 1) / chunks + kWalkRows - 1) /
            kWalkRows * kWalkRows);
        if ((output_width + chunk_rows - 1) / chunk_rows != chunks) {
            continue;
        }
        if (chunks > 1 && static_cast<std::size_t>(chunks) * rows *
                                  input_width * sizeof(float) >
                              workspace) {
            break;
        }
        if (cost(chunks, chunk_rows) < chosen) {
            bad("a cheaper split exists");
        }
    }
}

}  // namespace

int main() {
    const std::size_t workspace = std::size_t{64} << 20;
    const std::size_t widths[] = {8,    40,   128,  136,   1000, 1024,
                                  4096, 4104, 11008, 16384, 131072};
    const std::size_t heights[] = {4,    20,   128,  132,  1000,
                                   4096, 11008, 32000, 100000};
    for (const std::size_t rows : {std::size_t{1}, std::size_t{16},
                                   std::size_t{33}, std::size_t{64}}) {
        for (const std::size_t input_width : widths) {
            for (const std::size_t output_width : heights) {
                check(rows, input_width, output_width, workspace);
                check(rows, input_width, output_width, std::size_t{1} << 20);
            }
        }
    }
    // the two transformer shapes: as many units as compute units, and three
    // short rounds instead of one long one
    const rthip::BackwardSplit gate =
        rthip::split_weight_rows(16, 4096, 11008, workspace);
    require(gate.column_tiles == 32 && gate.chunks == 8 &&
                gate.chunk_rows == 1408,
            "11008 x 4096 is cut into 8 chunks of 1408 rows", 16, 4096, 11008);
    const rthip::BackwardSplit down =
        rthip::split_weight_rows(16, 11008, 4096, workspace);
    require(down.column_tiles == 86 && down.chunks == 8 &&
                down.chunk_rows == 512,
            "4096 x 11008 is cut into 8 chunks of 512 rows", 16, 11008, 4096);
    if (failures != 0) {
        std::fprintf(stderr, "%d backward split checks failed\n", failures);
        return 1;
    }
    std::printf("backward split tests passed\n");
    return 0;
}
