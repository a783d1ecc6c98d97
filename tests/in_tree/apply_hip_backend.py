"""TEST INFRASTRUCTURE, build container only: proves the drop-in at the
reference's own registry, with the reference's own tests.

    python tests/in_tree/apply_hip_backend.py [--keep]

What it does, in a scratch directory outside this repository:

1. copies the reference's `include/`, `src/core/` and two of its tests
   (tests/core/backend/test_quantized_linear_backend.cpp, test_backend.cpp)
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
       (:172-240, :333-353, :355-395);
3. compiles the edited files and this repository's adapter sources
   (hip_adapter.cpp with -DRIFTCO_TRANSFORMER_IN_TREE, hip_runtime.cpp,
   packed_state.cpp) with g++ and links them with the objects of the
   unedited reference sources that oracle/Makefile already built
   (oracle/_ref/obj: tensor, quantization, backend, autograd and the few
   nn/ files of a Linear);
4. leaves the test programs (the accelerator test twice: as it is, and with
   the RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP gate on) in tests/in_tree/build/ (git-ignored; they
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
]
# program -> (source, extra compiler flags)
TESTS = {
    "quantized_linear_backend_tests":
        ("tests/core/backend/test_quantized_linear_backend.cpp", []),
    # the hardware gate: an unavailable hip backend is a failure
    "quantized_linear_backend_tests_hip_required":
        ("tests/core/backend/test_quantized_linear_backend.cpp",
         ["-DRIFTCO_TRANSFORMER_TEST_REQUIRE_HIP=1"]),
    "backend_tests": ("tests/core/backend/test_backend.cpp", []),
}


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
    Edit("tests/core/backend/test_backend.cpp",
         "        test_scoped_selection_restores_previous_backend();\n",
         "        test_selection_is_thread_local_if_available(\n"
         "            ExecutionBackend::Hip,\n            \"HIP\"\n        );\n",
         where="before"),
]


def copy_reference(tree):
    for part in ("include", os.path.join("src", "core")):
        shutil.copytree(os.path.join(REFERENCE, part),
                        os.path.join(tree, part))
    for source, _ in TESTS.values():
        target = os.path.join(tree, source)
        os.makedirs(os.path.dirname(target), exist_ok=True)
        shutil.copy(os.path.join(REFERENCE, source), target)


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
    for source in EDITED_SOURCES:
        jobs.append((os.path.join(tree, source),
                     os.path.join(objects, source + ".o"), includes))
    for name in ("hip_adapter.cpp", "hip_runtime.cpp", "packed_state.cpp"):
        jobs.append((os.path.join(BACKEND, name),
                     os.path.join(objects, "hip", name + ".o"),
                     includes + ["-DRIFTCO_TRANSFORMER_IN_TREE"]))
    for name, (source, flags) in TESTS.items():
        jobs.append((os.path.join(tree, source),
                     os.path.join(objects, name + ".o"), includes + flags))
    with ThreadPoolExecutor(max_workers=8) as pool:
        built = list(pool.map(compile_one, jobs))
    library = [path for path in built
               if os.path.basename(path)[:-2] not in TESTS]
    os.makedirs(BUILD, exist_ok=True)
    for name in TESTS:
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
        build(tree)
    finally:
        if arguments.keep:
            print("scratch tree kept at", tree)
        else:
            shutil.rmtree(tree, ignore_errors=True)
    print("built", ", ".join(sorted(TESTS)), "in", BUILD)


if __name__ == "__main__":
    sys.exit(main())
