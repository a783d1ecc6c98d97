"""The C-ABI library without a GPU: it loads, exports every symbol that
include/rthip.h declares, validates arguments, and reports 'unavailable'
instead of computing anything when no device is present."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "rthip.h")


def declared_symbols():
    with open(HEADER) as handle:
        text = handle.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rthip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(package, library):
    raw = ctypes.CDLL(package.LIBRARY_PATH)
    declared = declared_symbols()
    assert len(declared) >= 16
    for name in declared:
        assert hasattr(raw, name), f"{name} is declared but not exported"
    # and the Python prototypes cover exactly the declared set
    assert sorted(package.EXPORTED_SYMBOLS) == declared


def test_abi_version(package, library):
    assert library.abi_version() == (1, 10)


def test_select_algorithm_is_pure_host_logic(package, library):
    select = library.select_algorithm
    fwd, bwd = package.FORWARD, package.INPUT_BACKWARD
    # decode shapes -> streaming GEMV
    assert select(fwd, 1, 4096, 4096, 64) == package.ALGORITHM_GEMV
    assert select(fwd, 1, 4096, 11008, 64) == package.ALGORITHM_GEMV
    assert select(fwd, 1, 11008, 4096, 64) == package.ALGORITHM_GEMV
    # three and four rows of a wide layer: one 512-thread team per weight row
    assert select(fwd, 2, 11008, 4096, 64) == package.ALGORITHM_GEMV
    assert select(fwd, 3, 11008, 4096, 64) == package.ALGORITHM_GEMV
    assert select(fwd, 4, 16384, 4096, 64) == package.ALGORITHM_GEMV
    assert select(fwd, 5, 16384 + 64, 4096, 64) == package.ALGORITHM_SKINNY
    # one row of up to 32768 weights, two of up to 24576: the same one-team
    # form; more rows as two launches where two launches cover them
    assert select(fwd, 1, 28672, 8192, 64) == package.ALGORITHM_GEMV
    assert select(fwd, 2, 24576, 1024, 64) == package.ALGORITHM_GEMV
    assert select(fwd, 2, 32768, 1024, 64) == package.ALGORITHM_GEMV
    assert select(fwd, 4, 24576, 1024, 64) == package.ALGORITHM_GEMV
    assert select(fwd, 3, 28672, 8192, 64) == package.ALGORITHM_SKINNY
    assert select(fwd, 5, 24576, 8192, 64) == package.ALGORITHM_SKINNY
    assert select(fwd, 1, 32768 + 64, 1024, 64) == package.ALGORITHM_SKINNY
    # prefill / training -> MFMA GEMM, both directions
    assert select(fwd, 2048, 4096, 11008, 64) == package.ALGORITHM_MFMA
    # small batches -> weights decoded straight into MFMA operands
    assert select(fwd, 16, 256, 768, 64) == package.ALGORITHM_SKINNY
    assert select(fwd, 64, 11008, 4096, 64) == package.ALGORITHM_SKINNY
    assert select(fwd, 16, 128, 768, 32) == package.ALGORITHM_SKINNY
    # up to 64 rows and a row width of 1024..4096 -> x resident in registers
    assert select(fwd, 16, 4096, 11008, 64) == package.ALGORITHM_RESIDENT
    assert select(fwd, 5, 4096, 4096, 64) == package.ALGORITHM_RESIDENT
    assert select(fwd, 8, 3072, 1000, 32) == package.ALGORITHM_RESIDENT
    assert select(fwd, 17, 4096, 4096, 64) == package.ALGORITHM_RESIDENT
    assert select(fwd, 64, 4096, 11008, 64) == package.ALGORITHM_RESIDENT
    # 65...112 rows: the first 64 and the rest as two small-batch launches
    # (the family of the first part is reported), the tiled GEMM after that;
    # the register-resident kernel takes up to 128 rows in one launch and
    # 129...224 as 128 and the rest
    assert select(fwd, 65, 4096, 11008, 64) == package.ALGORITHM_RESIDENT
    assert select(fwd, 112, 11008, 4096, 64) == package.ALGORITHM_SKINNY
    assert select(fwd, 113, 11008, 4096, 64) == package.ALGORITHM_MFMA
    assert select(fwd, 128, 4096, 11008, 64) == package.ALGORITHM_RESIDENT
    assert select(fwd, 224, 4096, 4096, 64) == package.ALGORITHM_RESIDENT
    assert select(fwd, 225, 4096, 11008, 64) == package.ALGORITHM_MFMA
    assert select(fwd, 16, 11008, 4096, 64) == package.ALGORITHM_SKINNY
    assert select(fwd, 16, 5120, 4096, 64) == package.ALGORITHM_SKINNY
    # (row width a multiple of 32 but not of 64 -> tiled GEMM)
    assert select(fwd, 16, 96, 768, 32) == package.ALGORITHM_MFMA
    assert select(fwd, 16, 40, 768, 32) == package.ALGORITHM_GENERIC
    assert select(bwd, 2048, 4096, 11008, 64) == package.ALGORITHM_MFMA
    assert select(bwd, 2048, 11008, 4096, 64) == package.ALGORITHM_MFMA
    # up to 64 rows and a row width that is a multiple of 8 -> the backward
    # kernel that walks the weight as it lies in memory
    # decode-sized input backward: the weight streamed as it lies in memory
    assert select(bwd, 1, 4096, 11008, 64) == package.ALGORITHM_GEMV
    assert select(bwd, 4, 11008, 4096, 64) == package.ALGORITHM_GEMV
    assert select(bwd, 2, 4096, 4096, 64) == package.ALGORITHM_GEMV
    # (three and four rows of a small weight: the small-batch kernel)
    assert select(bwd, 4, 4096, 4096, 64) == package.ALGORITHM_SKINNY
    assert select(bwd, 4, 4096, 4096, 32) == package.ALGORITHM_SKINNY
    assert select(bwd, 5, 4096, 11008, 64) == package.ALGORITHM_SKINNY
    assert select(bwd, 64, 11008, 4096, 64) == package.ALGORITHM_SKINNY
    assert select(bwd, 16, 40, 768, 32) == package.ALGORITHM_SKINNY
    # 65...96 rows: two launches of it, unless dx is much wider than dy;
    # up to 192 rows (three launches) where dy is at least twice as wide
    assert select(bwd, 65, 4096, 11008, 64) == package.ALGORITHM_SKINNY
    assert select(bwd, 96, 4096, 4096, 64) == package.ALGORITHM_SKINNY
    assert select(bwd, 97, 4096, 4096, 64) == package.ALGORITHM_MFMA
    assert select(bwd, 97, 4096, 11008, 64) == package.ALGORITHM_SKINNY
    assert select(bwd, 192, 4096, 11008, 64) == package.ALGORITHM_SKINNY
    assert select(bwd, 193, 4096, 11008, 64) == package.ALGORITHM_MFMA
    # (dx much wider than dy: only while the rest fits the streaming kernel)
    assert select(bwd, 68, 11008, 4096, 64) == package.ALGORITHM_SKINNY
    assert select(bwd, 69, 11008, 4096, 64) == package.ALGORITHM_MFMA
    assert select(bwd, 16, 36, 768, 32) == package.ALGORITHM_GENERIC
    # the reference's edge layout -> shape-agnostic kernels
    assert select(fwd, 2, 33, 33, 32) == package.ALGORITHM_GENERIC
    assert select(bwd, 2, 33, 33, 32) == package.ALGORITHM_GENERIC


def test_argument_validation_needs_no_device(package, library):
    with pytest.raises(package.InvalidArgument):
        library.select_algorithm(package.FORWARD, 0, 64, 64, 64)
    with pytest.raises(package.InvalidArgument):
        library.select_algorithm(package.FORWARD, 1, 64, 64, 48)
    with pytest.raises(package.InvalidArgument):
        library.select_algorithm(2, 1, 64, 64, 64)
    assert "block size" in library.last_error() or library.last_error()


def test_reports_unavailable_without_a_device(package, library):
    if library.is_available():
        pytest.skip("a device is present")
    with pytest.raises(package.Unavailable) as error:
        library.device_count()
    assert "device" in error.value.message
    with pytest.raises(package.Unavailable):
        library.malloc(64)
    # a compute call is refused before anything is launched
    weight = package.DeviceWeight(
        64, 64, 64, package.SCALE_FLOAT32, _Fake(0x1000), _Fake(0x2000), None)
    with pytest.raises(package.Unavailable):
        library.linear_forward(0x3000, weight, None, 0x4000, 1)


def test_lora_arguments_are_checked_before_any_device_work(package, library):
    weight = package.DeviceWeight(
        64, 64, 64, package.SCALE_FLOAT32, _Fake(0x1000), _Fake(0x2000), None)
    call = library.lora_linear_forward
    # (x, weight, bias, A, B, rank, scale, reduced, y, rows)
    with pytest.raises(package.InvalidArgument):  # B missing
        call(0x3000, weight, None, 0x5000, 0, 8, 1.0, 0x7000, 0x4000, 1)
    with pytest.raises(package.InvalidArgument):  # reduced missing
        call(0x3000, weight, None, 0x5000, 0x6000, 8, 1.0, 0, 0x4000, 1)
    with pytest.raises(package.InvalidArgument):
        call(0x3000, weight, None, 0x5000, 0x6000, 0, 1.0, 0x7000, 0x4000, 1)
    with pytest.raises(package.InvalidArgument):
        call(0x3000, weight, None, 0x5000, 0x6000, 8, float("inf"), 0x7000,
             0x4000, 1)
    with pytest.raises(package.InvalidArgument):  # reduced aliases x
        call(0x3000, weight, None, 0x5000, 0x6000, 8, 1.0, 0x3000, 0x4000, 1)
    assert "alias" in library.last_error()
    with pytest.raises(package.InvalidArgument):
        library.lora_reduce(0x3000, 0, 0x7000, 1, 64, 8)
    with pytest.raises(package.InvalidArgument):
        library.lora_reduce(0x3000, 0x5000, 0x7000, 1, 64, 0)


def test_adapter_backward_arguments_are_checked_first(package, library):
    weight = package.DeviceWeight(
        64, 64, 64, package.SCALE_FLOAT32, _Fake(0x1000), _Fake(0x2000), None)
    call = library.lora_backward
    # (dy, x, reduced, B, rank, scale, d_reduced, dA, dB, rows, I, O)
    with pytest.raises(package.InvalidArgument):  # no B
        call(0x3000, 0x4000, 0x5000, 0, 8, 1.0, 0x7000, 0x8000, 0x9000, 1,
             64, 64)
    with pytest.raises(package.InvalidArgument):  # dA wanted, no x
        call(0x3000, None, 0x5000, 0x6000, 8, 1.0, 0x7000, 0x8000, 0x9000,
             1, 64, 64)
    assert "input" in library.last_error()
    with pytest.raises(package.InvalidArgument):  # dB wanted, no reduced
        call(0x3000, 0x4000, None, 0x6000, 8, 1.0, 0x7000, 0x8000, 0x9000,
             1, 64, 64)
    with pytest.raises(package.InvalidArgument):  # rank zero
        call(0x3000, 0x4000, 0x5000, 0x6000, 0, 1.0, 0x7000, 0x8000, 0x9000,
             1, 64, 64)
    with pytest.raises(package.InvalidArgument):  # scale not finite
        call(0x3000, 0x4000, 0x5000, 0x6000, 8, float("nan"), 0x7000, 0x8000,
             0x9000, 1, 64, 64)
    with pytest.raises(package.InvalidArgument):  # dA written over x
        call(0x3000, 0x4000, 0x5000, 0x6000, 8, 1.0, 0x7000, 0x4000, 0x9000,
             1, 64, 64)
    assert "alias" in library.last_error()
    with pytest.raises(package.InvalidArgument):  # dA and dB in one buffer
        call(0x3000, 0x4000, 0x5000, 0x6000, 8, 1.0, 0x7000, 0x8000, 0x8000,
             1, 64, 64)
    fused = library.lora_linear_input_backward
    # (dy, weight, A, d_reduced, rank, dx, rows)
    with pytest.raises(package.InvalidArgument):  # no A
        fused(0x3000, weight, 0, 0x7000, 8, 0x4000, 1)
    with pytest.raises(package.InvalidArgument):  # rank zero
        fused(0x3000, weight, 0x5000, 0x7000, 0, 0x4000, 1)
    with pytest.raises(package.InvalidArgument):  # dx over d_reduced
        fused(0x3000, weight, 0x5000, 0x7000, 8, 0x7000, 1)
    with pytest.raises(package.InvalidArgument):  # dx over dy
        fused(0x3000, weight, 0x5000, 0x7000, 8, 0x3000, 1)


def test_group_arguments_are_checked_before_any_device_work(package, library):
    weight = package.DeviceWeight(
        64, 64, 64, package.SCALE_FLOAT32, _Fake(0x1000), _Fake(0x2000), None)
    call = library.linear_forward_group
    with pytest.raises(package.InvalidArgument):  # one output for two members
        call(0x3000, [(weight, None, 0x4000), (weight, None, 0x4000)], 1)
    assert "same output" in library.last_error()
    with pytest.raises(package.InvalidArgument):  # output aliases the input
        call(0x3000, [(weight, None, 0x3000)], 1)
    with pytest.raises(package.InvalidArgument):  # no output
        call(0x3000, [(weight, None, 0)], 1)
    with pytest.raises(package.InvalidArgument):  # no rows
        call(0x3000, [(weight, None, 0x4000)], 0)
    with pytest.raises(package.InvalidArgument):  # too many members
        call(0x3000, [(weight, None, 0x4000 + 256 * m) for m in range(65)], 1)
    other = package.DeviceWeight(
        64, 128, 64, package.SCALE_FLOAT32, _Fake(0x1000), _Fake(0x2000), None)
    with pytest.raises(ValueError):  # different input widths
        call(0x3000, [(weight, None, 0x4000), (other, None, 0x5000)], 1)
    if not library.is_available():
        with pytest.raises(package.Unavailable):
            call(0x3000, [(weight, None, 0x4000)], 1)


def test_matmul_arguments_are_checked_before_any_device_work(package,
                                                              library):
    with pytest.raises(package.InvalidArgument):
        library.matmul(0, 0x2000, 0x3000, 1, 2, 3, 4)
    with pytest.raises(package.InvalidArgument):
        library.matmul(0x1000, 0x2000, 0x3000, 1, 0, 3, 4)
    with pytest.raises(package.InvalidArgument):
        library.matmul(0x1000, 0x2000, 0x1000, 1, 2, 3, 4)
    with pytest.raises(package.InvalidArgument):
        library.matmul(0x1000, 0x2000, 0x3000, 1, 2 ** 40, 2 ** 40, 4)


def test_quantize_arguments_are_checked_before_any_device_work(package,
                                                                library):
    fp32, nested = package.SCALE_FLOAT32, package.SCALE_DOUBLE_QUANTIZED_UINT8
    with pytest.raises(package.InvalidArgument):
        library.quantize(0, 64, 64, fp32, 0, 0x2000, 0x3000)
    with pytest.raises(package.InvalidArgument):
        library.quantize(0x1000, 0, 64, fp32, 0, 0x2000, 0x3000)
    with pytest.raises(package.InvalidArgument):
        library.quantize(0x1000, 64, 48, fp32, 0, 0x2000, 0x3000)
    with pytest.raises(package.InvalidArgument):  # no second-level buffer
        library.quantize(0x1000, 64, 64, nested, 32, 0x2000, 0x3000)
    with pytest.raises(package.InvalidArgument):  # bad second-level block
        library.quantize(0x1000, 64, 64, nested, 40, 0x2000, 0x3000, 0x4000,
                         0x5000)
    with pytest.raises(package.InvalidArgument):
        library.quantize(0x1000, 64, 64, 7, 0, 0x2000, 0x3000)


class _Fake:
    """Stands in for a tensor: only its address is ever passed on."""

    def __init__(self, address):
        self._address = address

    def data_ptr(self):
        return self._address


def test_kernel_name_follows_the_launch(package, library):
    """rthip_nf4_forward_kernel_name: the instance per shape, as a profiler
    prints it (bench.py matches stored counter summaries against it)."""
    name = lambda *a, **k: library.forward_kernel_name(*a, **k)  # noqa: E731
    fp32 = package.SCALE_FLOAT32
    nested = package.SCALE_DOUBLE_QUANTIZED_UINT8
    assert name(1, 4096, [4096], 64, fp32) == \
        "gemv1_forward_kernel<1, 1, 8, 2, 4, false, false, 1>"
    assert name(1, 4096, [4096] * 3, 64, fp32) == \
        "gemv1_forward_kernel<1, 1, 8, 2, 4, false, false, 4>"
    assert name(1, 4096, [11008, 11008], 64, nested, 256) == \
        "gemv1_forward_kernel<1, 1, 8, 2, 4, true, true, 4>"
    assert name(1, 11008, [4096], 64, nested, 256) == \
        "gemv1_forward_kernel<1, 3, 4, 2, 2, true, false, 1>"
    assert name(4, 11008, [4096], 64, fp32) == \
        "gemv1_forward_kernel<4, 3, 2, 2, 2, false, false, 1>"
    assert name(3, 8192, [4096], 64, fp32) == \
        "gemv1_forward_kernel<4, 2, 4, 2, 2, false, false, 1>"
    assert name(5, 4096, [4096], 64, fp32) == ""
    assert name(1, 4096, [4100], 64, fp32) == ""
    with pytest.raises(package.InvalidArgument):
        name(1, 4096, [], 64, fp32)
