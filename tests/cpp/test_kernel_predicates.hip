// TEST INFRASTRUCTURE: the kernels' shape predicates (csrc/kernels.hpp), which
// decide on the host what a launch may assume.  Links librthip.so and calls the
// *_supports functions with made-up addresses; nothing is launched, no device
// is needed.
#include "kernels.hpp"

#include <cstdint>
#include <cstdio>
#include <cstdlib>

namespace {

using rthip::LinearProblem;

int failures = 0;
void expect(bool condition, const char* what) {
    if (!condition) {
        std::printf("FAILED: %s\n", what);
        ++failures;
    }
}

// Addresses are only inspected for alignment.
template <typename T>
T* address(std::uintptr_t value) {
    return reinterpret_cast<T*>(value);
}

LinearProblem problem(std::size_t rows, std::size_t input_width,
                      std::size_t output_width, unsigned block_shift = 6) {
    LinearProblem p{};
    p.activations = address<const float>(0x10000);
    p.weight.codes = address<const std::uint8_t>(0x20000);
    p.weight.primary_scales = address<const void>(0x30000);
    p.weight.secondary_scales = nullptr;
    p.weight.encoding = 0;
    p.bias = nullptr;
    p.result = address<float>(0x40000);
    p.rows = rows;
    p.input_width = input_width;
    p.output_width = output_width;
    p.block_shift = block_shift;
    return p;
}

LinearProblem with_adapter(LinearProblem p) {
    p.lora.reduced = address<const float>(0x50000);
    p.lora.b = address<const float>(0x60000);
    p.lora.rank = 16;
    p.lora.scale = 1.0F;
    return p;
}

// With an adapter term the partial sums of the small-batch input backward
// always pass through the 64 MiB stream workspace (or the caller's scratch):
// rows * input_width * 4 bytes must fit, or another family has to serve.
void test_adapter_partial_sums_fit_the_workspace() {
    const std::size_t limit = rthip::kStreamWorkspaceBytes / sizeof(float);
    // 64 rows x 262144 columns = exactly 64 MiB of partial sums
    expect(rthip::small_input_backward_supports(
               with_adapter(problem(64, limit / 64, 64))),
           "small backward, adapter, partial sums of exactly 64 MiB");
    expect(!rthip::small_input_backward_supports(
               with_adapter(problem(64, limit / 64 + 8, 64))),
           "small backward, adapter, partial sums above 64 MiB are refused");
    expect(rthip::small_input_backward_supports(
               problem(64, limit / 64 + 8, 64)),
           "small backward without adapter is not bound by the workspace");
    // the caller's scratch replaces the workspace in the bound
    LinearProblem scratch = with_adapter(problem(16, 4096, 4096));
    scratch.scratch = address<float>(0x70000);
    scratch.scratch_bytes = 16 * 4096 * sizeof(float);
    expect(rthip::small_input_backward_supports(scratch),
           "small backward, adapter, scratch of exactly the partial sums");
    scratch.scratch_bytes -= 4;
    expect(!rthip::small_input_backward_supports(scratch),
           "small backward, adapter, scratch four bytes short");

    expect(rthip::stream_input_backward_supports(
               with_adapter(problem(4, limit / 4, 64))),
           "streaming backward, adapter, partial sums of exactly 64 MiB");
    expect(!rthip::stream_input_backward_supports(
               with_adapter(problem(4, limit / 4 + 64, 64))),
           "streaming backward, adapter, above 64 MiB is refused");
    expect(rthip::stream_input_backward_supports(
               problem(4, limit / 4 + 64, 64)),
           "streaming backward without adapter is not bound by the workspace");
}

void test_decode_kernel_shapes() {
    expect(rthip::gemv1_forward_supports(problem(1, 4096, 4096)), "q_proj");
    expect(rthip::gemv1_forward_supports(problem(4, 11008, 4096)),
           "down_proj, four rows");
    expect(rthip::gemv1_forward_supports(problem(1, 12288, 64)),
           "three stripes of 4096");
    expect(!rthip::gemv1_forward_supports(problem(1, 12352, 64)),
           "rows wider than three stripes");
    expect(!rthip::gemv1_forward_supports(problem(5, 4096, 4096)), "five rows");
    expect(!rthip::gemv1_forward_supports(problem(1, 4096, 4100)),
           "an output width that is no multiple of eight");
    expect(!rthip::gemv1_forward_supports(problem(1, 4096, 4096, 5)),
           "block size 32");
    expect(!rthip::gemv1_forward_supports(problem(1, 4128, 64)),
           "a row width that is no multiple of the block size");
    LinearProblem odd = problem(1, 4096, 4096);
    odd.weight.codes = address<const std::uint8_t>(0x20002);
    expect(!rthip::gemv1_forward_supports(odd), "codes not 4-byte aligned");
    odd = problem(1, 4096, 4096);
    odd.activations = address<const float>(0x10008);
    expect(!rthip::gemv1_forward_supports(odd), "x not 16-byte aligned");
    // what it leaves, the older kernel takes
    expect(rthip::gemv_forward_supports(problem(1, 28672, 8192)),
           "a row of 28672 weights goes to the older kernel");
    expect(rthip::gemv_forward_supports(problem(1, 4096, 4100)),
           "so does an odd output width");
}

void test_tiled_kernel_shapes() {
    expect(rthip::mfma_forward_supports(problem(2048, 4096, 11008)), "prefill");
    expect(!rthip::mfma_forward_supports(problem(2048, 4080, 11008)),
           "contraction not a multiple of 32");
    expect(rthip::mfma_input_backward_supports(problem(2048, 4096, 11008)),
           "prefill backward");
    expect(!rthip::mfma_input_backward_supports(problem(2048, 4096, 11000)),
           "backward contraction not a multiple of 32");
    // buffer loads: 32-bit flat weight indices, a tile's rows of the
    // activations within 32-bit byte offsets
    expect(rthip::mfma_forward_supports(problem(128, 32768, 65536)),
           "2^31 weights");
    expect(!rthip::mfma_forward_supports(problem(128, 65536, 65536)),
           "2^32 weights");
    expect(!rthip::mfma_forward_supports(problem(128, 1U << 22, 32)),
           "a row of 2^22 activations");
    // 256-row tiles take the tile columns that fill the 256 compute units in
    // whole rounds (a multiple of 256 / gcd(256, tile rows)), if that is at
    // least half of them and the last tile row is more than half full
    const auto tall = rthip::mfma_forward_tall_tile_columns;
    expect(tall(2048, 4096) == 32, "8 x 32 tall tiles: one launch");
    expect(tall(2048, 11008) == 64, "8 x 64 of 86 tile columns");
    expect(tall(4096, 11008) == 80, "16 x 80 of 86");
    expect(tall(1024, 11008) == 64, "4 x 64 of 86");
    expect(tall(512, 11008) == 0, "2 tile rows: 128 columns per round");
    expect(tall(2048, 4224) == 32, "32 of 33");
    expect(tall(2048, 2048) == 0, "16 tile columns: no whole round");
    expect(tall(2048, 12288 + 64) == 96, "a ragged last column stays square");
    expect(tall(255, 4096) == 0, "fewer rows than a tall tile");
    expect(tall(2048 + 100, 4096) == 0, "last tile row under half full");
    expect(tall(2048 + 129, 11008 * 4) == 256, "9 tile rows: 256 per round");
}

}  // namespace

int main() {
    test_adapter_partial_sums_fit_the_workspace();
    test_decode_kernel_shapes();
    test_tiled_kernel_shapes();
    if (failures != 0) {
        std::printf("%d kernel predicate check(s) failed\n", failures);
        return 1;
    }
    std::printf("kernel predicate tests passed\n");
    return 0;
}
