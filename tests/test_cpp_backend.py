"""Runs the C++ tests of the `hip` backend adapter (tests/cpp).

Without a GPU the adapter is exercised against the host-only test runtime
(tests/fakes/fake_rthip.cpp, a stand-in for librthip.so that computes with the
CPU oracle): storage accounting, byte-preserving transfer, dispatcher
validation, error mapping and the unavailable paths.  With a GPU the same
binary runs against the real library, with test plugins refused.

The binaries are built beforehand by `make -C tests/cpp` (which
__graft_entry__.build() runs); a missing binary is a failure, not a skip.
"""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BUILD = os.path.join(HERE, "cpp", "build")
BINARY = os.path.join(BUILD, "test_hip_backend")
FAKE = os.path.join(BUILD, "librthip_fake.so")
CONFORMANCE = os.path.join(BUILD, "test_in_tree_conformance")


def run(arguments=(), **environment):
    env = {k: v for k, v in os.environ.items()
           if not k.startswith(("RIFTCO_TRANSFORMER_", "FAKE_RTHIP_"))}
    env["RIFTCO_TRANSFORMER_TEST_GOLDEN"] = os.path.join(HERE, "golden")
    env.update(environment)
    assert os.path.exists(BINARY), \
        "tests/cpp/build/test_hip_backend is not built (make -C tests/cpp)"
    return subprocess.run([BINARY, *arguments], env=env, capture_output=True,
                          text=True, timeout=300)


def expect_pass(result, fragment="hip backend tests passed"):
    assert result.returncode == 0, result.stdout + result.stderr
    assert fragment in result.stdout


def test_adapter_on_the_host_only_runtime():
    expect_pass(run(RIFTCO_TRANSFORMER_HIP_LIBRARY=FAKE,
                    RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP="1",
                    FAKE_RTHIP_CAN_FAIL="1"))


@pytest.mark.parametrize("options", [
    {"RIFTCO_TRANSFORMER_HIP_POOL": "0"},
    {"RIFTCO_TRANSFORMER_HIP_ASYNC": "1"},
    {"RIFTCO_TRANSFORMER_HIP_POOL": "0", "RIFTCO_TRANSFORMER_HIP_ASYNC": "1"},
    {"RIFTCO_TRANSFORMER_HIP_MERGE": "0"},
    {"RIFTCO_TRANSFORMER_HIP_POOL": "0", "RIFTCO_TRANSFORMER_HIP_MERGE": "0"},
    {"RIFTCO_TRANSFORMER_HIP_ASYNC": "1", "RIFTCO_TRANSFORMER_HIP_MERGE": "0"},
])
def test_adapter_options_on_the_host_only_runtime(options):
    """Without the buffer pool, without the per-operation synchronise, and
    with decode-sized forwards that share an input merged into one launch."""
    expect_pass(run(RIFTCO_TRANSFORMER_HIP_LIBRARY=FAKE,
                    RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP="1", **options))


SANITIZER_ENVIRONMENT = {
    # the harness preloads a library of its own; ASan only insists on being
    # first in the list, which has no bearing on what is checked here
    "ASAN_OPTIONS": "verify_asan_link_order=0:detect_leaks=1:"
                    "abort_on_error=0:exitcode=23",
    "UBSAN_OPTIONS": "halt_on_error=1:print_stacktrace=1:exitcode=23",
    "TSAN_OPTIONS": "halt_on_error=1:exitcode=23",
}


def run_sanitized(program, runtime, **environment):
    binary = os.path.join(BUILD, program)
    library = os.path.join(BUILD, runtime)
    assert os.path.exists(binary) and os.path.exists(library), \
        f"{program} is not built (make -C tests/cpp sanitize)"
    env = {k: v for k, v in os.environ.items()
           if not k.startswith(("RIFTCO_TRANSFORMER_", "FAKE_RTHIP_"))}
    env.update(SANITIZER_ENVIRONMENT)
    env["RIFTCO_TRANSFORMER_TEST_GOLDEN"] = os.path.join(HERE, "golden")
    env["RIFTCO_TRANSFORMER_HIP_LIBRARY"] = library
    env["RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP"] = "1"
    env.update(environment)
    return subprocess.run([binary], env=env, capture_output=True, text=True,
                          timeout=600)


@pytest.mark.parametrize("options", [
    {"FAKE_RTHIP_CAN_FAIL": "1"},
    {"RIFTCO_TRANSFORMER_HIP_POOL": "0"},
    {"RIFTCO_TRANSFORMER_HIP_ASYNC": "1"},
    {"RIFTCO_TRANSFORMER_HIP_MERGE": "0"},
    {"FAKE_RTHIP_NO_BAR": "1"},
])
def test_adapter_under_address_and_undefined_behaviour_sanitizers(options):
    """The whole host side -- adapter (buffer pool, held-back launches, the
    lazily synchronised host copies, spans into device memory), run-time
    binding, dispatcher, packed-state reader, and the test runtime -- built
    with -fsanitize=address,undefined, as the reference's `sanitize` preset
    builds its host code (cmake/RiftcoTransformerSanitizers.cmake)."""
    result = run_sanitized(os.path.join("asan", "test_hip_backend"),
                           os.path.join("asan", "librthip_fake.so"),
                           **options)
    assert result.returncode == 0, result.stdout + result.stderr[-4000:]
    assert "hip backend tests passed" in result.stdout
    assert "runtime error" not in result.stderr
    assert "AddressSanitizer" not in result.stderr


@pytest.mark.parametrize("options", [
    {},
    {"RIFTCO_TRANSFORMER_HIP_POOL": "0"},
    {"RIFTCO_TRANSFORMER_HIP_ASYNC": "1"},
    {"RIFTCO_TRANSFORMER_HIP_MERGE": "0"},
])
def test_adapter_from_four_threads_under_thread_sanitizer(options):
    """tests/cpp/test_threads.cpp: four threads share a weight, an input and
    the buffer pool; forward, input backward, host reads, storage release,
    and tensors whose first download or upload happens under contention.
    Every result equals the single-threaded one and ThreadSanitizer reports
    nothing (the counterpart of the reference's thread test of backend
    selection, tests/core/backend/test_backend.cpp:355-395)."""
    result = run_sanitized(os.path.join("tsan", "test_threads"),
                           os.path.join("tsan", "librthip_fake.so"),
                           **options)
    assert result.returncode == 0, result.stdout + result.stderr[-4000:]
    assert "hip backend thread tests passed" in result.stdout
    assert "ThreadSanitizer" not in result.stderr


def test_adapter_keeps_a_counted_mirror_without_host_visible_memory():
    expect_pass(run(RIFTCO_TRANSFORMER_HIP_LIBRARY=FAKE,
                    RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP="1",
                    FAKE_RTHIP_NO_BAR="1"))


def test_packed_state_reader_fails_as_the_reference_reader_does(tmp_path):
    """The adapter's reader of the packed model state on every malformed
    variant of the fixture: outcome and message must be the ones the
    reference's compiled reader gave (tests/golden/make_golden.py)."""
    import json
    import helpers
    golden = os.path.join(HERE, "golden")
    with open(os.path.join(golden, "packed_state.bin"), "rb") as handle:
        blob = handle.read()
    with open(os.path.join(golden, "packed_state_outcomes.json")) as handle:
        expected = json.load(handle)
    cases = helpers.packed_state_mutations(blob)
    paths = []
    for name, data in cases:
        path = tmp_path / name
        path.write_bytes(data)
        paths.append(str(path))
    result = run(["--parse-state", *paths])
    assert result.returncode == 0, result.stdout + result.stderr
    lines = result.stdout.splitlines()
    assert len(lines) == len(cases)
    for (name, _), line in zip(cases, lines):
        kind, _, rest = line.partition(" ")
        want = expected[name]
        assert [kind, rest] == [want[0], str(want[1])], name


def test_work_split_of_the_tiled_kernels():
    """Host arithmetic of tile_plan.hpp: runs cover every unit once, never
    exceed a tile, slots are unique (tests/cpp/test_tile_plan.cpp)."""
    binary = os.path.join(BUILD, "test_tile_plan")
    assert os.path.exists(binary), \
        "tests/cpp/build/test_tile_plan is not built (make -C tests/cpp)"
    result = subprocess.run([binary], capture_output=True, text=True,
                            timeout=120)
    assert result.returncode == 0, result.stdout + result.stderr
    assert "tile plan tests passed" in result.stdout


def test_work_split_of_the_small_batch_input_backward():
    """Host arithmetic of backward_split.hpp: chunks are whole walk steps and
    cover every weight row once, partial sums fit the workspace, no cheaper
    split exists (tests/cpp/test_backward_split.cpp)."""
    binary = os.path.join(BUILD, "test_backward_split")
    assert os.path.exists(binary), \
        "tests/cpp/build/test_backward_split is not built (make -C tests/cpp)"
    result = subprocess.run([binary], capture_output=True, text=True,
                            timeout=120)
    assert result.returncode == 0, result.stdout + result.stderr
    assert "backward split tests passed" in result.stdout


def test_shape_predicates_of_the_kernels():
    """What a launch may assume is decided on the host: the decode kernel's
    shapes, the tiled kernel's, and the bound that keeps the adapter term's
    partial sums inside the workspace (tests/cpp/test_kernel_predicates.hip,
    linked against librthip.so; nothing is launched)."""
    binary = os.path.join(BUILD, "test_kernel_predicates")
    assert os.path.exists(binary), \
        "tests/cpp/build/test_kernel_predicates is not built (make -C tests/cpp)"
    result = subprocess.run([binary], capture_output=True, text=True,
                            timeout=120)
    assert result.returncode == 0, result.stdout + result.stderr
    assert "kernel predicate tests passed" in result.stdout


def test_unavailable_when_the_runtime_sees_no_device():
    result = run(["--expect-unavailable"],
                 RIFTCO_TRANSFORMER_HIP_LIBRARY=FAKE, FAKE_RTHIP_NO_DEVICE="1")
    expect_pass(result, "no HIP device is visible")


def test_unavailable_when_the_library_is_missing():
    result = run(["--expect-unavailable"],
                 RIFTCO_TRANSFORMER_HIP_LIBRARY="/nonexistent/librthip.so")
    expect_pass(result, "cannot load the HIP runtime library")


def test_hardware_gate_refuses_the_test_plugin():
    result = run(["--expect-unavailable"],
                 RIFTCO_TRANSFORMER_HIP_LIBRARY=FAKE,
                 RIFTCO_TRANSFORMER_HIP_REJECT_TEST_PLUGIN="1")
    expect_pass(result, "test plugins are rejected")


def test_required_hardware_turns_unavailable_into_failure():
    result = run(RIFTCO_TRANSFORMER_HIP_LIBRARY=FAKE, FAKE_RTHIP_NO_DEVICE="1",
                 RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP="1")
    assert result.returncode == 1
    assert "require an available backend" in result.stderr


def test_in_tree_conformance_against_the_reference_headers():
    """hip_adapter.cpp compiled against the reference's own BackendAdapter and
    linked with the reference's own objects; built only where the reference
    tree exists."""
    if not os.path.exists(CONFORMANCE):
        pytest.skip("built only where /root/reference is present")
    env = dict(os.environ, RIFTCO_TRANSFORMER_HIP_LIBRARY=FAKE)
    result = subprocess.run([CONFORMANCE], env=env, capture_output=True,
                            text=True, timeout=300)
    assert result.returncode == 0, result.stdout + result.stderr
    assert "in-tree conformance tests passed" in result.stdout


@pytest.mark.gpu
def test_adapter_on_the_real_library():
    """The same binary against librthip.so on a real MI355X: kernels, device
    storage served through the PCIe BAR, resident == logical bytes."""
    result = run(RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP="1",
                 RIFTCO_TRANSFORMER_HIP_REJECT_TEST_PLUGIN="1")
    expect_pass(result)
    assert "unavailable" not in result.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("options", [
    {"RIFTCO_TRANSFORMER_HIP_POOL": "0"},
    {"RIFTCO_TRANSFORMER_HIP_ASYNC": "1"},
    {"RIFTCO_TRANSFORMER_HIP_MERGE": "0"},
])
def test_adapter_options_on_the_real_library(options):
    """The pool switched off, and operations queued without a synchronise per
    call: same results, because host reads go through a synchronising copy."""
    result = run(RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP="1",
                 RIFTCO_TRANSFORMER_HIP_REJECT_TEST_PLUGIN="1", **options)
    expect_pass(result)
