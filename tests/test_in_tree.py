"""The drop-in, proven at the reference's own registry with the reference's own
tests: tests/in_tree/apply_hip_backend.py edits a scratch copy of the
reference (Hip = 4, the registry case, the validated-once dispatcher), links
it with this repository's adapter and builds the reference's
tests/core/backend/test_quantized_linear_backend.cpp (ExecutionBackend::Hip in
its accelerator loop, :382-453,502-513) and test_backend.cpp (identity,
diagnostics, thread-local selection: :172-240,278-395).  The same script
sends `Linear::forward` of a packed layer with a low-rank adapter through one
fused graph node on hip, adds RT_BACKEND_HIP to the C ABI bridge, and builds
the reference's tests/nn/test_quantized_linear.cpp and
tests/core/test_quantization.cpp with hip in the place of their optional
accelerator (and the former's CPU-only tests repeated on hip), its
tests/model/test_qlora_model.cpp (the decoder-only model moved to hip and
back, and one QLoRA training step of the whole model on hip), plus two
programs of this repository: the fused layer against the reference's
composition on the CPU backend, and the bridge's identity checks.

Without a GPU they run against the host-only test runtime
(tests/fakes/fake_rthip.cpp), the role tests/fakes/fake_pjrt_tpu.cpp plays for
the reference's TPU backend; on the GPU box the prebuilt programs run against
the real librthip.so."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SCRIPT = os.path.join(ROOT, "tests", "in_tree", "apply_hip_backend.py")
BUILD = os.path.join(ROOT, "tests", "in_tree", "build")
FAKE = os.path.join(ROOT, "tests", "cpp", "build", "librthip_fake.so")
REAL = os.path.join(ROOT, "riftco-transformer_amd", "lib", "librthip.so")
REFERENCE = os.environ.get("REFERENCE", "/root/reference")


def run(program, library, **extra):
    environment = dict(os.environ, RIFTCO_TRANSFORMER_HIP_LIBRARY=library,
                       **extra)
    return subprocess.run([os.path.join(BUILD, program)], env=environment,
                          capture_output=True, text=True, timeout=300)


@pytest.fixture(scope="module")
def programs():
    if not os.path.isdir(os.path.join(REFERENCE, "src", "core")):
        pytest.skip("the reference tree is not present here")
    if not os.path.exists(FAKE):
        subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "cpp"),
                        "all"], check=True)
    subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "_ref"],
                   check=True, capture_output=True)
    subprocess.run([sys.executable, SCRIPT], check=True)
    return BUILD


def test_accelerator_loop_runs_hip_through_the_registry(programs):
    # required: "unavailable" would be a failure, so a pass means the aligned
    # and edge fixtures, both encodings, forward and input backward, byte
    # accounting included, ran on the hip adapter
    done = run("quantized_linear_backend_tests_hip_required", FAKE)
    assert done.returncode == 0, done.stderr
    assert "quantized-linear backend tests passed" in done.stdout
    # the test plugin can be refused, as the reference's hardware gates refuse
    # the fake PJRT plugin; the backend is then unavailable and the gate fails
    refused = run("quantized_linear_backend_tests_hip_required", FAKE,
                  RIFTCO_TRANSFORMER_HIP_REJECT_TEST_PLUGIN="1")
    assert refused.returncode == 1
    assert "hip quantized-linear tests require an available backend" in \
        refused.stderr


def test_unavailable_hip_rejects_weight_transfer(programs):
    # no library: the "unavailable" branch of the same test
    # (:481-499: weight.to(Hip) must throw "... unavailable")
    done = run("quantized_linear_backend_tests", "/nonexistent/librthip.so")
    assert done.returncode == 0, done.stderr
    gate = run("quantized_linear_backend_tests_hip_required",
               "/nonexistent/librthip.so")
    assert gate.returncode == 1


@pytest.mark.parametrize("library", [FAKE, "/nonexistent/librthip.so"])
def test_identity_diagnostics_and_thread_local_selection(programs, library):
    done = run("backend_tests", library)
    assert done.returncode == 0, done.stderr
    assert "backend tests passed" in done.stdout


def test_nn_tests_run_on_hip(programs):
    """tests/nn/test_quantized_linear.cpp: the graph of 2 nodes / 20 elements
    and the VJP (:140-183), the packed bytes across an Adam step and the
    merged export (:185-267) repeated on hip, and Module::to to hip and back
    (:269-318); the program prints a line when the hip copies ran."""
    done = run("quantized_linear_tests", FAKE)
    assert done.returncode == 0, done.stderr
    assert "quantized Linear tests ran on hip" in done.stdout
    assert "quantized Linear tests passed" in done.stdout
    without = run("quantized_linear_tests", "/nonexistent/librthip.so")
    assert without.returncode == 0, without.stderr
    assert "ran on hip" not in without.stdout


def test_quantization_transfer_keeps_bytes_on_hip(programs):
    # tests/core/test_quantization.cpp:400-435 with hip as the accelerator
    done = run("quantization_tests", FAKE)
    assert done.returncode == 0, done.stderr
    assert "NF4 quantization tests passed" in done.stdout


def test_qlora_model_trains_on_hip(programs):
    """tests/model/test_qlora_model.cpp: the decoder-only model is quantized,
    given adapters, and -- in the copy the script adds -- moved to hip before
    one step of cross entropy, backward and paged Adam (:136-274: packed byte
    counts unchanged by the step, merged export equal to the adapted output);
    Module::to to hip and back keeps the packed payload (:276-323)."""
    done = run("qlora_model_tests", FAKE)
    assert done.returncode == 0, done.stderr
    assert "QLoRA model trained on hip" in done.stdout
    assert "QLoRA model moved to hip and back" in done.stdout
    assert "QLoRA model tests passed" in done.stdout
    without = run("qlora_model_tests", "/nonexistent/librthip.so")
    assert without.returncode == 0, without.stderr
    assert "on hip" not in without.stdout and "to hip" not in without.stdout


def test_fused_linear_equals_the_reference_composition(programs):
    done = run("fused_linear_tests", FAKE,
               RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP="1")
    assert done.returncode == 0, done.stderr
    assert "fused Linear tests passed" in done.stdout
    skipped = run("fused_linear_tests", "/nonexistent/librthip.so")
    assert skipped.returncode == 0 and "skipped" in skipped.stdout
    gate = run("fused_linear_tests", "/nonexistent/librthip.so",
               RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP="1")
    assert gate.returncode == 1


def test_c_abi_backend_identity(programs):
    done = run("c_api_identity_tests", FAKE,
               RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP="1")
    assert done.returncode == 0, done.stderr
    assert "hip backend selected through the C ABI" in done.stdout
    refused = run("c_api_identity_tests", "/nonexistent/librthip.so")
    assert refused.returncode == 0, refused.stderr
    assert "hip backend refused through the C ABI" in refused.stdout
    gate = run("c_api_identity_tests", "/nonexistent/librthip.so",
               RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP="1")
    assert gate.returncode == 1


@pytest.mark.gpu
def test_reference_tests_on_the_device():
    """The programs built in the build container, against the real library
    on an MI355X: the reference's accelerator test with hip required (its
    resident == logical assertion holds because HBM is host-visible), its
    backend, nn and quantization tests, the fused layer and the C ABI
    bridge."""
    required = os.path.join(BUILD,
                            "quantized_linear_backend_tests_hip_required")
    if not os.path.exists(required):
        pytest.skip("tests/in_tree/build was not built (no reference tree)")
    for program in ("quantized_linear_backend_tests_hip_required",
                    "backend_tests", "quantized_linear_tests",
                    "quantization_tests", "qlora_model_tests",
                    "fused_linear_tests", "c_api_identity_tests"):
        done = run(program, REAL, RIFTCO_TRANSFORMER_HIP_REJECT_TEST_PLUGIN="1",
                   RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP="1")
        assert done.returncode == 0, program + done.stdout + done.stderr
        assert "tests passed" in done.stdout
        if program == "quantized_linear_tests":
            assert "quantized Linear tests ran on hip" in done.stdout
        if program == "qlora_model_tests":
            assert "QLoRA model trained on hip" in done.stdout
            assert "QLoRA model moved to hip and back" in done.stdout
