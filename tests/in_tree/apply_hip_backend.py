"""TEST INFRASTRUCTURE, build container only: proves the drop-in at the
reference's own registry, with the reference's own tests.

    python tests/in_tree/apply_hip_backend.py [--keep]

What it does, in a scratch directory outside this repository:

1. copies the reference's `include/`, `src/core/`, `src/nn/`, `src/optim/`,
   `src/model/`, `src/c_api/` and five of its tests
   from /root/reference -- nothing of the reference enters this repository;
2. applies the edits a maintainer would make to add the backend, each written
   here as "find this short anchor, put that text beside it":
     * `Hip = 4` appended to ExecutionBackend
       (include/riftco_transformer/core/backend.hpp:13-18),
     * `hip_backend_adapter()` declared beside `tpu_backend_adapter()`
       (src/core/backend/adapter.hpp) and returned by the registry's switch
       (src/core/backend/registry.cpp:127-141),
     * the validated-once change of the dispatcher: an optional
       `ScaleValidationMemo` interface next to QuantizedWeightStorage
       (src/core/backend/nn/quantized_linear/storage.hpp) and, in
       require_weight_storage (dispatch.cpp:203-242), the O(#blocks) scale
       scan skipped for storage that says it has been scanned -- the block
       count is still compared on every call, with the same exception and
       message,
     * `ExecutionBackend::Hip` added to the accelerator loop of
       test_quantized_linear_backend.cpp (:502-513) with a
       RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP gate (:455-470), and to the
       identity, diagnostic and thread-local checks of test_backend.cpp
       (:172-240, :333-353, :355-395),
     * `Linear::forward` (src/nn/linear.cpp:147-172) sends a layer that holds
       a packed weight and a low-rank adapter on the hip backend through ONE
       custom-gradient node (FUSED_LINEAR below, the file a maintainer would
       add as src/nn/hip_fused_linear.cpp): bias, adapter and packed product
       in one dispatch forward, dx / dA / dB in one call backward,
     * `RT_BACKEND_HIP ((rt_backend)4)` in the C ABI
       (include/riftco_transformer/c_api.h:51-55) and its two switch cases
       in src/c_api/bridge.cpp:5-56,
     * the reference's nn and quantization tests learn about hip WITHOUT any
       of their text entering this repository: in the scratch copies of
       tests/nn/test_quantized_linear.cpp and tests/core/test_quantization.cpp
       every `ExecutionBackend::Metal` becomes `ExecutionBackend::Hip` (their
       "if the accelerator is available" blocks: polymorphic Module::to,
       :269-318, and byte-preserving transfer, :400-435), and the two
       CPU-only tests of the former (autograd graph of 2 nodes / 20 elements
       and VJP, :140-183; packed bytes unchanged across an Adam step and the
       merged export, :185-267) are duplicated with `Cpu` replaced by `Hip`
       and run when the backend is available,
     * the same for the model: in the scratch copy of
       tests/model/test_qlora_model.cpp the polymorphic transfer of the
       decoder-only model (:276-323) names hip, and the training test
       (:136-274: quantize, attach adapters, one step of cross entropy,
       backward and paged Adam, merged export) is duplicated with the
       quantized model moved to hip before its adapters go to the optimizer;
3. compiles the edited files and this repository's adapter sources
   (hip_adapter.cpp with -DRIFTCO_TRANSFORMER_IN_TREE, hip_runtime.cpp,
   packed_state.cpp) with g++ and links them with the objects of the
   unedited reference sources that oracle/Makefile already built
   (oracle/_ref/obj: tensor, quantization, backend, autograd and the few
   nn/ files of a Linear) and with the reference's optimizer, remaining nn/
   files and decoder-only model, compiled here as they are;
4. leaves the test programs (the accelerator test twice: as it is, and with
   the RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP gate on; the nn, quantization
   and model tests; tests/in_tree/test_c_api_identity.cpp, this repository's own few
   lines over the edited bridge) in tests/in_tree/build/ (git-ignored; they
   travel to the GPU box, where tests/test_in_tree.py runs them against the
   real librthip.so).

tests/test_in_tree.py runs this script and then the programs against the
host-only test runtime (tests/fakes/fake_rthip.cpp).
"""
import argparse
import os
import shutil
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REFERENCE = os.environ.get("REFERENCE", "/root/reference")
BACKEND = os.path.join(ROOT, "riftco-transformer_amd", "backend")
REF_OBJECTS = os.path.join(ROOT, "oracle", "_ref", "obj", "src")
BUILD = os.path.join(HERE, "build")

# Reference sources that the edits touch (recompiled from the scratch copy;
# their objects under oracle/_ref/obj are left out of the link) ...
EDITED_SOURCES = [
    "src/core/backend/registry.cpp",
    "src/core/backend/nn/quantized_linear/dispatch.cpp",
    "src/nn/linear.cpp",
]
# ... reference sources that are compiled as they are, beyond the objects
# oracle/Makefile built (the nn tests need the optimizer, the model test the
# decoder-only model and the layers under it) ...
EXTRA_SOURCES = [
    "src/optim/adam.cpp",
    "src/nn/activations.cpp",
    "src/nn/embedding.cpp",
    "src/nn/layer_norm.cpp",
    "src/nn/loss.cpp",
    "src/nn/rms_norm.cpp",
    "src/model/causal_self_attention.cpp",
    "src/model/decoder_only_transformer.cpp",
    "src/model/feed_forward.cpp",
    "src/model/transformer_block.cpp",
]
# ... and the file the Linear edit adds
ADDED_SOURCES = {"src/nn/hip_fused_linear.cpp": None}  # text: FUSED_LINEAR
# program -> (source, extra compiler flags)
TESTS = {
    "quantized_linear_backend_tests":
        ("tests/core/backend/test_quantized_linear_backend.cpp", []),
    # the hardware gate: an unavailable hip backend is a failure
    "quantized_linear_backend_tests_hip_required":
        ("tests/core/backend/test_quantized_linear_backend.cpp",
         ["-DRIFTCO_TRANSFORMER_TEST_REQUIRE_HIP=1"]),
    "backend_tests": ("tests/core/backend/test_backend.cpp", []),
    "quantized_linear_tests": ("tests/nn/test_quantized_linear.cpp", []),
    "quantization_tests": ("tests/core/test_quantization.cpp", []),
    "qlora_model_tests": ("tests/model/test_qlora_model.cpp", []),
}
# this repository's own programs over the edited tree: the C ABI bridge, and
# the fused Linear against the reference's composition on the CPU backend
C_API_TEST = os.path.join(HERE, "test_c_api_identity.cpp")
OWN_TESTS = {"fused_linear_tests": os.path.join(HERE, "test_fused_linear.cpp")}


class Edit:
    """Insert `text` after (or before, or instead of) the only occurrence of
    `anchor` in `path`."""

    def __init__(self, path, anchor, text, where="after", count=1):
        self.path, self.anchor, self.text = path, anchor, text
        self.where, self.count = where, count

    def apply(self, tree):
        path = os.path.join(tree, self.path)
        with open(path) as handle:
            source = handle.read()
        found = source.count(self.anchor)
        if found != self.count:
            raise SystemExit(
                f"{self.path}: expected {self.count} occurrence(s) of "
                f"{self.anchor!r}, found {found}: the reference has changed")
        if self.where == "after":
            replacement = self.anchor + self.text
        elif self.where == "before":
            replacement = self.text + self.anchor
        else:
            replacement = self.text
        with open(path, "w") as handle:
            handle.write(source.replace(self.anchor, replacement))


MEMO_INTERFACE = """
// Optional extension of immutable weight storage: remembers that the
// O(#blocks) scan of its scale values has passed once.
#define RIFTCO_TRANSFORMER_HAS_SCALE_VALIDATION_MEMO 1
class ScaleValidationMemo {
public:
    virtual ~ScaleValidationMemo() = default;
    [[nodiscard]] virtual bool scales_validated() const noexcept = 0;
    virtual void mark_scales_validated() const noexcept = 0;
};

"""

MEMO_USE = """    const auto* memo = dynamic_cast<const ScaleValidationMemo*>(&weight);
    if (memo != nullptr && memo->scales_validated()) {
        // scanned before and immutable since: only the count can disagree
        if (scales.scale_count() != expected_scales) {
            throw std::invalid_argument(
                scales.encoding == Nf4ScaleEncoding::Float32
                    ? "legacy NF4 scale storage has an invalid representation"
                    : "double-quantized NF4 scale storage has an invalid "
                      "representation"
            );
        }
    } else {
        require_scale_storage(scales, expected_scales);
        if (memo != nullptr) {
            memo->mark_scales_validated();
        }
    }
"""

FUSED_LINEAR = r"""// Linear::forward for a layer that holds a packed NF4 weight and a low-rank
// adapter, on the hip backend: one custom-gradient node around the adapter's
// fused calls instead of quantized_linear + broadcast + add + two matmuls +
// scale (src/nn/linear.cpp:147-172, src/nn/low_rank_adapter.cpp:126-151).
#include "riftco_transformer/core/autograd.hpp"
#include "riftco_transformer/core/quantized_weight.hpp"
#include "riftco_transformer/core/tensor_ops.hpp"
#include "riftco_transformer/nn/low_rank_adapter.hpp"
#include "riftco_transformer/nn/parameter.hpp"

#include "core/backend/adapter.hpp"
#include "core/backend/adapters/hip/hip_adapter.hpp"

#include <utility>
#include <vector>

namespace riftco_transformer {

Variable hip_fused_quantized_linear(
    const Variable& input,
    const QuantizedWeight& weight,
    const Parameter* bias,
    const LowRankAdapter& lora
) {
    const std::size_t input_width = weight.shape()[1];
    const std::size_t output_width = weight.shape()[0];
    const std::size_t rows = input.value().numel() / input_width;
    const ExecutionBackend backend = input.value().backend();
    const backend_detail::QuantizedLinearDimensions dimensions{
        rows, input_width, output_width, weight.block_size()};
    Tensor::Shape output_shape = input.value().shape();
    output_shape.back() = output_width;
    Tensor output(output_shape, backend);
    Tensor reduced({rows, lora.rank()}, backend);
    backend_detail::hip_quantized_linear_adapter_forward({
        backend_detail::tensor_storage(input.value()),
        backend_detail::quantized_weight_storage(weight),
        bias != nullptr ? &backend_detail::tensor_storage(bias->value())
                        : nullptr,
        backend_detail::tensor_storage(lora.a().value()),
        backend_detail::tensor_storage(lora.b().value()),
        lora.rank(),
        lora.scale(),
        backend_detail::tensor_storage(reduced),
        backend_detail::tensor_storage(output),
        dimensions,
    });

    std::vector<Variable> dependencies{
        input, lora.a().variable(), lora.b().variable()};
    if (bias != nullptr) {
        dependencies.push_back(bias->variable());
    }
    return custom_gradient(
        std::move(output),
        dependencies,
        [weight, dimensions, backend, has_bias = bias != nullptr,
         input_value = input.value(), reduced = std::move(reduced),
         a = lora.a().value(), b = lora.b().value(), rank = lora.rank(),
         scale = lora.scale()](const Tensor& upstream) {
            Tensor input_gradient(input_value.shape(), backend);
            Tensor a_gradient(a.shape(), backend);
            Tensor b_gradient(b.shape(), backend);
            backend_detail::hip_quantized_linear_adapter_backward({
                backend_detail::tensor_storage(upstream),
                backend_detail::tensor_storage(input_value),
                backend_detail::tensor_storage(reduced),
                backend_detail::quantized_weight_storage(weight),
                backend_detail::tensor_storage(a),
                backend_detail::tensor_storage(b),
                rank,
                scale,
                backend_detail::tensor_storage(input_gradient),
                backend_detail::tensor_storage(a_gradient),
                backend_detail::tensor_storage(b_gradient),
                dimensions,
            });
            std::vector<Tensor> gradients;
            gradients.push_back(std::move(input_gradient));
            gradients.push_back(std::move(a_gradient));
            gradients.push_back(std::move(b_gradient));
            if (has_bias) {
                gradients.push_back(tensor_ops::sum_to_shape(
                    upstream, {dimensions.output_width}));
            }
            return gradients;
        }
    );
}

}  // namespace riftco_transformer
"""
ADDED_SOURCES["src/nn/hip_fused_linear.cpp"] = FUSED_LINEAR

FUSED_LINEAR_DECLARATION = """
namespace riftco_transformer {
// src/nn/hip_fused_linear.cpp
[[nodiscard]] Variable hip_fused_quantized_linear(
    const Variable& input, const QuantizedWeight& weight,
    const Parameter* bias, const LowRankAdapter& lora);
}  // namespace riftco_transformer
"""

FUSED_LINEAR_USE = """    if (has_quantized_weight() && has_lora() &&
        input.value().backend() == ExecutionBackend::Hip) {
        // bias, adapter and packed product in one dispatch, one graph node
        return hip_fused_quantized_linear(
            input, *quantized_weight_, has_bias() ? &bias_ : nullptr, *lora_);
    }

"""

EDITS = [
    # 1. identity
    Edit("include/riftco_transformer/core/backend.hpp", "    Tpu = 3,\n",
         "    Hip = 4,\n"),
    # 2. registry
    Edit("src/core/backend/adapter.hpp",
         "tpu_backend_adapter() noexcept;\n",
         "\n// The AMD MI355X (gfx950) adapter: adapters/hip/hip_adapter.cpp, or\n"
         "// adapters/hip/stub.cpp when the backend is not built.\n"
         "[[nodiscard]] const BackendAdapter& hip_backend_adapter() noexcept;\n"),
    Edit("src/core/backend/registry.cpp",
         "            return &tpu_backend_adapter();\n",
         "        case ExecutionBackend::Hip:\n"
         "            return &hip_backend_adapter();\n"),
    # 3. the dispatcher reads an immutable weight's scales once
    Edit("src/core/backend/nn/quantized_linear/storage.hpp",
         "// Immutable backend-owned storage for one packed NF4 weight.",
         MEMO_INTERFACE, where="before"),
    Edit("src/core/backend/nn/quantized_linear/dispatch.cpp",
         "    require_scale_storage(scales, expected_scales);\n",
         MEMO_USE, where="instead"),
    # 4. the reference's tests learn about the new backend
    Edit("tests/core/backend/test_quantized_linear_backend.cpp",
         "constexpr std::size_t kEdgeWidth = 33;\n",
         "#ifndef RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP\n"
         "#define RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP 0\n#endif\n",
         where="before"),
    Edit("tests/core/backend/test_quantized_linear_backend.cpp",
         "    case ExecutionBackend::Cpu:\n        return false;\n",
         "    case ExecutionBackend::Hip:\n"
         "        return RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP != 0;\n"),
    Edit("tests/core/backend/test_quantized_linear_backend.cpp",
         "std::array<ExecutionBackend, 3> accelerators{\n",
         "std::array<ExecutionBackend, 4> accelerators{\n"
         "            ExecutionBackend::Hip,\n", where="instead"),
    Edit("tests/core/backend/test_backend.cpp",
         "        \"TPU execution backend name\"\n    );\n",
         "    require(\n"
         "        static_cast<std::uint8_t>(ExecutionBackend::Hip) == 4,\n"
         "        \"HIP execution backend numeric identity\"\n    );\n"
         "    require(\n"
         "        riftco_transformer::execution_backend_name(\n"
         "            ExecutionBackend::Hip\n"
         "        ) == std::string_view(\"hip\"),\n"
         "        \"HIP execution backend name\"\n    );\n"),
    Edit("tests/core/backend/test_backend.cpp",
         "    constexpr std::array optional_backends{\n",
         "        ExecutionBackend::Hip,\n"),
    # 5. the fused Linear
    Edit("src/nn/linear.cpp", "namespace riftco_transformer {\n",
         FUSED_LINEAR_DECLARATION, where="before"),
    Edit("src/nn/linear.cpp",
         "    Tensor::Shape output_shape = input.value().shape();\n"
         "    output_shape.back() = output_width();\n",
         FUSED_LINEAR_USE, where="before"),
    # 6. the C ABI's backend identity
    Edit("include/riftco_transformer/c_api.h",
         "#define RT_BACKEND_TPU ((rt_backend)3)\n",
         "#define RT_BACKEND_HIP ((rt_backend)4)\n"),
    Edit("src/c_api/bridge.cpp",
         "            result = riftco_transformer::ExecutionBackend::Tpu;\n"
         "            break;\n",
         "        case RT_BACKEND_HIP:\n"
         "            result = riftco_transformer::ExecutionBackend::Hip;\n"
         "            break;\n"),
    Edit("src/c_api/bridge.cpp",
         "            return RT_BACKEND_TPU;\n",
         "        case riftco_transformer::ExecutionBackend::Hip:\n"
         "            return RT_BACKEND_HIP;\n"),
    Edit("tests/core/backend/test_backend.cpp",
         "        test_scoped_selection_restores_previous_backend();\n",
         "        test_selection_is_thread_local_if_available(\n"
         "            ExecutionBackend::Hip,\n            \"HIP\"\n        );\n",
         where="before"),
]


def copy_reference(tree):
    for part in ("include", os.path.join("src", "core"),
                 os.path.join("src", "nn"), os.path.join("src", "optim"),
                 os.path.join("src", "model"), os.path.join("src", "c_api")):
        shutil.copytree(os.path.join(REFERENCE, part),
                        os.path.join(tree, part))
    for source, _ in TESTS.values():
        target = os.path.join(tree, source)
        os.makedirs(os.path.dirname(target), exist_ok=True)
        shutil.copy(os.path.join(REFERENCE, source), target)
    for source, text in ADDED_SOURCES.items():
        with open(os.path.join(tree, source), "w") as handle:
            handle.write(text)
    # the adapter's public header where the reference's sources look for it
    home = os.path.join(tree, "src", "core", "backend", "adapters", "hip")
    os.makedirs(home, exist_ok=True)
    for name in ("hip_adapter.hpp", "interface.hpp"):
        shutil.copy(os.path.join(BACKEND, name), os.path.join(home, name))


def rewrite(tree, path, transform):
    path = os.path.join(tree, path)
    with open(path) as handle:
        source = handle.read()
    with open(path, "w") as handle:
        handle.write(transform(source))


def function_text(source, name, path):
    """The text of `void name() { ... }` at namespace scope: from its first
    line to the first line that holds only the closing brace."""
    head = f"void {name}() {{\n"
    if source.count(head) != 1:
        raise SystemExit(f"{path}: expected one definition of {name}(): "
                         "the reference has changed")
    start = source.index(head)
    end = source.index("\n}\n", start) + 3
    return source[start:end]


def accelerator_becomes_hip(source, path, expected):
    """The tests' "if the accelerator is available" blocks name Metal: in the
    scratch copy they name hip."""
    if source.count("ExecutionBackend::Metal") != expected:
        raise SystemExit(f"{path}: expected {expected} mentions of "
                         "ExecutionBackend::Metal: the reference has changed")
    return source.replace("ExecutionBackend::Metal", "ExecutionBackend::Hip")


NN_TEST = "tests/nn/test_quantized_linear.cpp"
# tests that the reference runs on the CPU backend only, repeated on hip
NN_TESTS_ON_HIP = ["test_forward_backward_and_graph_memory",
                   "test_linear_qlora_composition_and_export"]


def nn_test_on_hip(source):
    source = accelerator_becomes_hip(source, NN_TEST, 7)
    copies, calls = [], []
    for name in NN_TESTS_ON_HIP:
        text = function_text(source, name, NN_TEST)
        if "ExecutionBackend::Cpu" not in text:
            raise SystemExit(f"{NN_TEST}: {name} names no backend")
        copies.append(text.replace(f"void {name}()", f"void {name}_on_hip()")
                      .replace("ExecutionBackend::Cpu",
                               "ExecutionBackend::Hip"))
        calls.append(f"            {name}_on_hip();\n")
    close = "}  // namespace\n\nint main() {\n"
    first_call = f"        {NN_TESTS_ON_HIP[0]}();\n"
    if source.count(close) != 1 or source.count(first_call) != 1:
        raise SystemExit(f"{NN_TEST}: main() has changed")
    source = source.replace(close, "\n".join(copies) + "\n" + close)
    return source.replace(
        first_call,
        first_call +
        "        if (riftco_transformer::execution_backend_available(\n"
        "                ExecutionBackend::Hip)) {\n" + "".join(calls) +
        "            std::cout << \"quantized Linear tests ran on hip\\n\";\n"
        "        }\n")


QUANTIZATION_TEST = "tests/core/test_quantization.cpp"


def quantization_test_on_hip(source):
    return accelerator_becomes_hip(source, QUANTIZATION_TEST, 6)


MODEL_TEST = "tests/model/test_qlora_model.cpp"


# the training test of the reference runs on the CPU backend: repeated with
# the quantized model moved to hip before its adapters are handed to Adam
MODEL_TRAINING_TEST = "test_model_qlora_training_and_fp32_export"
MODEL_TRANSFER_TEST = "test_polymorphic_model_transfer_if_metal_available"


def model_test_on_hip(source):
    source = accelerator_becomes_hip(source, MODEL_TEST, 4)
    transfer = function_text(source, MODEL_TRANSFER_TEST, MODEL_TEST)
    source = source.replace(
        transfer,
        transfer[:-3] +
        "\n    std::cout << \"QLoRA model moved to hip and back\\n\";\n}\n")
    training = function_text(source, MODEL_TRAINING_TEST, MODEL_TEST)
    attached = "    });\n    ParameterList adapters = model.lora_parameters();\n"
    if training.count(attached) != 1:
        raise SystemExit(f"{MODEL_TEST}: {MODEL_TRAINING_TEST} has changed")
    on_hip = training.replace(
        f"void {MODEL_TRAINING_TEST}()", f"void {MODEL_TRAINING_TEST}_on_hip()"
    ).replace(
        attached,
        "    });\n"
        "    static_cast<riftco_transformer::Module&>(model).to(\n"
        "        riftco_transformer::ExecutionBackend::Hip);\n"
        "    require(\n"
        "        model.backend() == riftco_transformer::ExecutionBackend::Hip,\n"
        "        \"the quantized model trains on hip\"\n"
        "    );\n"
        "    ParameterList adapters = model.lora_parameters();\n")
    close = "}  // namespace\n\nint main() {\n"
    first_call = f"        {MODEL_TRAINING_TEST}();\n"
    if source.count(close) != 1 or source.count(first_call) != 1:
        raise SystemExit(f"{MODEL_TEST}: main() has changed")
    source = source.replace(close, on_hip + "\n" + close)
    return source.replace(
        first_call,
        first_call +
        "        if (riftco_transformer::execution_backend_available(\n"
        "                riftco_transformer::ExecutionBackend::Hip)) {\n"
        f"            {MODEL_TRAINING_TEST}_on_hip();\n"
        "            std::cout << \"QLoRA model trained on hip\\n\";\n"
        "        }\n")


def compile_one(job):
    source, target, flags = job
    os.makedirs(os.path.dirname(target), exist_ok=True)
    subprocess.run(["g++", "-O1", "-std=c++20", "-fPIC", "-w",
                    "-ffp-contract=off"] + flags + ["-c", "-o", target,
                                                    source], check=True)
    return target


def reference_objects():
    """Objects of the unedited reference sources (built by oracle/Makefile)."""
    skip = {os.path.splitext(os.path.relpath(source, "src"))[0] + ".o"
            for source in EDITED_SOURCES}
    found = []
    for directory, _, names in os.walk(REF_OBJECTS):
        for name in names:
            path = os.path.join(directory, name)
            if name.endswith(".o") and \
                    os.path.relpath(path, REF_OBJECTS) not in skip:
                found.append(path)
    return sorted(found)


def build(tree):
    includes = ["-I" + os.path.join(tree, "include"),
                "-I" + os.path.join(tree, "src")]
    objects = os.path.join(tree, "obj")
    jobs = []
    for source in EDITED_SOURCES + EXTRA_SOURCES:
        jobs.append((os.path.join(tree, source),
                     os.path.join(objects, source + ".o"), includes))
    for source in sorted(ADDED_SOURCES):
        jobs.append((os.path.join(tree, source),
                     os.path.join(objects, source + ".o"),
                     includes + ["-DRIFTCO_TRANSFORMER_IN_TREE"]))
    for name in ("hip_adapter.cpp", "hip_runtime.cpp", "packed_state.cpp"):
        jobs.append((os.path.join(BACKEND, name),
                     os.path.join(objects, "hip", name + ".o"),
                     includes + ["-DRIFTCO_TRANSFORMER_IN_TREE"]))
    for name, (source, flags) in TESTS.items():
        jobs.append((os.path.join(tree, source),
                     os.path.join(objects, name + ".o"), includes + flags))
    for name, source in OWN_TESTS.items():
        jobs.append((source, os.path.join(objects, name + ".o"), includes))
    library_count = len(jobs) - len(TESTS) - len(OWN_TESTS)
    # the C ABI bridge pulls in every handle type of the reference: its two
    # backend functions are linked alone (sections, then --gc-sections)
    bridge = includes + ["-I" + os.path.join(tree, "src", "c_api"),
                         "-ffunction-sections", "-fdata-sections"]
    jobs.append((os.path.join(tree, "src", "c_api", "bridge.cpp"),
                 os.path.join(objects, "c_api", "bridge.o"), bridge))
    jobs.append((C_API_TEST, os.path.join(objects, "c_api", "test.o"),
                 bridge))
    with ThreadPoolExecutor(max_workers=8) as pool:
        built = list(pool.map(compile_one, jobs))
    library = built[:library_count]
    os.makedirs(BUILD, exist_ok=True)
    subprocess.run(
        ["g++", "-Wl,--gc-sections", "-o",
         os.path.join(BUILD, "c_api_identity_tests")] + built[-2:] + library +
        reference_objects() + ["-ldl", "-lpthread"], check=True)
    for name in list(TESTS) + list(OWN_TESTS):
        subprocess.run(
            ["g++", "-o", os.path.join(BUILD, name),
             os.path.join(objects, name + ".o")] + library +
            reference_objects() + ["-ldl", "-lpthread"], check=True)


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--keep", action="store_true",
                        help="keep the scratch tree and print its path")
    arguments = parser.parse_args()
    if not os.path.isdir(os.path.join(REFERENCE, "src", "core")):
        raise SystemExit(f"{REFERENCE} is not present")
    if not os.path.isdir(REF_OBJECTS):
        raise SystemExit("oracle/_ref/obj is missing: run `make -C oracle _ref`")
    tree = tempfile.mkdtemp(prefix="riftco_in_tree_")
    try:
        copy_reference(tree)
        for edit in EDITS:
            edit.apply(tree)
        rewrite(tree, NN_TEST, nn_test_on_hip)
        rewrite(tree, QUANTIZATION_TEST, quantization_test_on_hip)
        rewrite(tree, MODEL_TEST, model_test_on_hip)
        build(tree)
    finally:
        if arguments.keep:
            print("scratch tree kept at", tree)
        else:
            shutil.rmtree(tree, ignore_errors=True)
    print("built", ", ".join(sorted(list(TESTS) + list(OWN_TESTS) +
                                   ["c_api_identity_tests"])),
          "in", BUILD)


if __name__ == "__main__":
    sys.exit(main())
