"""Pins the CPU restatement (oracle/) to the known-answer vectors the
reference's own unit tests hold.  Each test names the reference test it
restates (paths under /root/reference)."""
import numpy as np
import pytest

import helpers
from oracle.binding import (SCALE_DOUBLE_QUANTIZED_UINT8, SCALE_FLOAT32,
                            Nf4Weight)

CODEBOOK = np.array([
    -1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453,
    -0.28444138169288635, -0.18477343022823334, -0.09105003625154495, 0.0,
    0.07958029955625534, 0.16093020141124725, 0.24611230194568634,
    0.33791524171829224, 0.44070982933044434, 0.5626170039176941,
    0.7229568362236023, 1.0], dtype=np.float32)


def unpack(codes, index):
    byte = int(codes[index // 2])
    return byte & 0x0F if index % 2 == 0 else byte >> 4


def test_codebook_literals_and_canonical_packing(oracle):
    # tests/core/test_quantization.cpp:62-112
    codebook = oracle.codebook()
    assert np.array_equal(codebook.view(np.uint32), CODEBOOK.view(np.uint32))
    assert np.all(np.diff(codebook) > 0)
    assert codebook[7] == 0.0
    weight = oracle.quantize(CODEBOOK, 32)
    assert weight.codes.tolist() == [0x10, 0x32, 0x54, 0x76, 0x98, 0xBA,
                                     0xDC, 0xFE]
    assert weight.fp32_scales.tolist() == [1.0]
    restored = oracle.dequantize(weight).ravel()
    assert np.array_equal(restored.view(np.uint32), CODEBOOK.view(np.uint32))


def test_midpoint_tie_chooses_lower_code(oracle):
    # tests/core/test_quantization.cpp:114-125
    values = np.zeros(32, dtype=np.float32)
    values[0] = CODEBOOK[8] * np.float32(0.5)
    values[-1] = 1.0
    weight = oracle.quantize(values, 32)
    assert unpack(weight.codes, 0) == 7
    assert oracle.nearest_code(CODEBOOK[8] * np.float32(0.5)) == 7


def test_zero_blocks_use_code_seven_and_zero_scale(oracle):
    # tests/core/test_quantization.cpp:127-137
    weight = oracle.quantize(np.zeros(33, dtype=np.float32), 32)
    assert weight.fp32_scales.tolist() == [0.0, 0.0]
    assert all(unpack(weight.codes, i) == 7 for i in range(33))
    assert weight.codes[-1] == 0x07


def test_partial_block_has_its_own_scale(oracle):
    # tests/core/test_quantization.cpp:139-152
    values = np.full(33, 0.25, dtype=np.float32)
    values[0] = -2.0
    values[-1] = 10.0
    weight = oracle.quantize(values, 32)
    assert weight.fp32_scales.tolist() == [2.0, 10.0]
    assert unpack(weight.codes, 0) == 0 and unpack(weight.codes, 32) == 15
    restored = oracle.dequantize(weight).ravel()
    assert restored[0] == -2.0 and restored[32] == 10.0


def test_double_quantized_scale_packing_and_bytes(oracle):
    # tests/core/test_quantization.cpp:155-205
    values = np.repeat(np.arange(33, dtype=np.float32), 32)
    weight = oracle.quantize(values, 32, double_quantized=True,
                             second_level_block=32)
    assert weight.encoding == SCALE_DOUBLE_QUANTIZED_UINT8
    assert weight.fp32_scales is None
    assert weight.scale_codes.size == 33
    assert weight.second_level.tolist() == [16.0, 16.0]
    assert weight.offset == 16.0
    assert weight.scale_codes[0] == 1
    assert weight.scale_codes[16] == 128
    assert weight.scale_codes[32] == 255
    restored = oracle.dequantize(weight).ravel()
    assert restored[0] == 0.0
    assert restored[16 * 32] == 16.0
    assert restored[32 * 32] == 32.0
    # packed 528, scales 33 + 2*4 + 4 = 45, logical 573, fp32 4224
    assert weight.codes.size == 528
    assert oracle.scale_payload_bytes(weight) == 45
    assert weight.payload_bytes == 573
    assert weight.element_count * 4 == 4224


def test_sixty_four_zeros_use_36_bytes(oracle):
    # tests/core/test_quantization.cpp:368-376
    weight = oracle.quantize(np.zeros(64, dtype=np.float32), 64)
    assert weight.codes.size == 32
    assert oracle.scale_payload_bytes(weight) == 4
    assert weight.payload_bytes == 36


def scalar_zero():
    return Nf4Weight(1, 1, 32, np.array([0x07], dtype=np.uint8),
                     SCALE_FLOAT32, fp32_scales=np.zeros(1, np.float32))


def double_scalar_zero():
    return Nf4Weight(1, 1, 32, np.array([0x07], dtype=np.uint8),
                     SCALE_DOUBLE_QUANTIZED_UINT8,
                     scale_codes=np.array([128], dtype=np.uint8),
                     second_level=np.zeros(1, np.float32),
                     second_level_block=32, offset=0.0)


def test_payload_validation_accepts_canonical_scalars(oracle):
    # tests/core/test_quantization.cpp:207-223
    oracle.validate_payload(scalar_zero())
    oracle.validate_payload(double_scalar_zero())
    assert oracle.dequantize(scalar_zero()).ravel()[0] == 0.0


@pytest.mark.parametrize("mutate", [
    # tests/core/test_quantization.cpp:225-345, one entry per require_throws
    lambda w: setattr(w, "codes", np.zeros(0, np.uint8)),
    lambda w: setattr(w, "fp32_scales", np.zeros(0, np.float32)),
    lambda w: setattr(w, "codes", np.array([0xF7], np.uint8)),
    lambda w: setattr(w, "codes", np.array([0x08], np.uint8)),
    lambda w: setattr(w, "fp32_scales", np.array([-1.0], np.float32)),
    lambda w: setattr(w, "fp32_scales", np.array([np.inf], np.float32)),
])
def test_payload_validation_rejects_legacy(oracle, mutate):
    weight = scalar_zero()
    mutate(weight)
    with pytest.raises(ValueError):
        oracle.validate_payload(weight)


@pytest.mark.parametrize("mutate", [
    lambda w: setattr(w, "fp32_scales", np.zeros(1, np.float32)),
    lambda w: setattr(w, "scale_codes", np.zeros(0, np.uint8)),
    lambda w: setattr(w, "second_level_block", 16),
    lambda w: setattr(w, "second_level", np.zeros(0, np.float32)),
    lambda w: setattr(w, "second_level", np.array([-1.0], np.float32)),
    lambda w: setattr(w, "offset", float("inf")),
])
def test_payload_validation_rejects_double_quantized(oracle, mutate):
    weight = double_scalar_zero()
    mutate(weight)
    with pytest.raises(ValueError):
        oracle.validate_payload(weight)


def test_block_sizes_and_nonfinite_sources(oracle):
    # src/core/quantization/nf4.cpp:39-53; test_quantization.cpp:347-359
    supported = [32, 64, 128, 256, 512, 1024, 2048, 4096]
    for size in range(1, 8200):
        assert oracle.block_size_supported(size) == (size in supported)
    values = np.zeros(32, dtype=np.float32)
    values[0] = np.nan
    with pytest.raises(ValueError):
        oracle.quantize(values, 32)
    # "double quantization should reject an unsupported scale block size"
    # (test_quantization.cpp:349-355) and an unsupported first-level one
    zeros = np.zeros(32, dtype=np.float32)
    for block, second in ((32, 16), (48, 256), (32, 8192)):
        with pytest.raises(ValueError, match="NF4 block size must be one of"):
            oracle.quantize(zeros, block, True, second)
    with pytest.raises(ValueError, match="NF4 block size must be one of"):
        oracle.quantize(zeros, 16)
    oracle.quantize(zeros, 32, True, 32)


def test_lora_composes_its_scaled_low_rank_delta(oracle):
    """tests/nn/test_lora.cpp:208-243: A = [[1,0,0],[0,1,0]], B = [[1,2],[-1,3]],
    alpha 4 at rank 2 (scale 2), x = [1,2,3]; the dense base of that test
    contributes [14.5, 4.5] (W x + b), supplied here as the bias of an all-zero
    packed weight.  Expected output [24.5, 14.5]."""
    weight = oracle.quantize(np.zeros((2, 32), dtype=np.float32), 32)
    x = np.zeros((1, 32), dtype=np.float32)
    x[0, :3] = [1.0, 2.0, 3.0]
    lora_a = np.zeros((2, 32), dtype=np.float32)
    lora_a[0, 0] = 1.0
    lora_a[1, 1] = 1.0
    lora_b = np.array([[1.0, 2.0], [-1.0, 3.0]], dtype=np.float32)
    bias = np.array([14.5, 4.5], dtype=np.float32)
    y = oracle.lora_forward(x, weight, lora_a, lora_b, 4.0 / 2.0, bias)
    assert y.tolist() == [[24.5, 14.5]]


def test_lora_backward_of_that_fixture_by_hand(oracle):
    """The same adapter (tests/nn/test_lora.cpp:208-244) with the upstream
    gradient of that test, [1, -0.5]: scaled upstream [2, -1]; through B,
    d(reduced) = [2*1 + (-1)(-1), 2*2 + (-1)*3] = [3, 1]; reduced = x A^T =
    [1, 2]; so dB = outer([2, -1], [1, 2]), dA = outer([3, 1], x), and with an
    all-zero base weight dx = [3, 1] A = [3, 1, 0, ...]."""
    weight = oracle.quantize(np.zeros((2, 32), dtype=np.float32), 32)
    x = np.zeros((1, 32), dtype=np.float32)
    x[0, :3] = [1.0, 2.0, 3.0]
    lora_a = np.zeros((2, 32), dtype=np.float32)
    lora_a[0, 0] = 1.0
    lora_a[1, 1] = 1.0
    lora_b = np.array([[1.0, 2.0], [-1.0, 3.0]], dtype=np.float32)
    dy = np.array([[1.0, -0.5]], dtype=np.float32)
    dx, d_a, d_b = oracle.lora_backward(dy, x, weight, lora_a, lora_b, 2.0)
    assert d_b.tolist() == [[2.0, 4.0], [-1.0, -2.0]]
    want_a = np.zeros((2, 32), dtype=np.float32)
    want_a[0, :3] = [3.0, 6.0, 9.0]
    want_a[1, :3] = [1.0, 2.0, 3.0]
    assert np.array_equal(d_a, want_a)
    want_x = np.zeros((1, 32), dtype=np.float32)
    want_x[0, :2] = [3.0, 1.0]
    assert np.array_equal(dx, want_x)


@pytest.mark.parametrize("double_quantized", [False, True])
def test_lora_backward_against_float64(oracle, double_quantized):
    """dx, dA, dB as fp64 matrix products of the loss's differential:
    y = x deq(W)^T + s (x A^T) B^T, so dx = dy deq(W) + s (dy B) A,
    dA = s (dy B)^T x, dB = s dy^T (x A^T).  A swapped operand, a dropped
    scale or a missing base term moves the result by its full size."""
    rows, in_w, out_w, rank, scale = 6, 256, 40, 4, 2.5
    weight = oracle.quantize(helpers.normal(71, (out_w, in_w), 0.02), 64,
                             double_quantized, 32)
    x = helpers.normal(72, (rows, in_w), 1.0)
    dy = helpers.normal(73, (rows, out_w), 1.0)
    lora_a = helpers.normal(74, (rank, in_w), 0.05)
    lora_b = helpers.normal(75, (out_w, rank), 0.05)
    dx, d_a, d_b = oracle.lora_backward(dy, x, weight, lora_a, lora_b, scale)
    dense = oracle.dequantize(weight).astype(np.float64)
    x64, dy64 = x.astype(np.float64), dy.astype(np.float64)
    a64, b64 = lora_a.astype(np.float64), lora_b.astype(np.float64)
    through_b = scale * (dy64 @ b64)
    assert np.allclose(dx, dy64 @ dense + through_b @ a64,
                       rtol=1e-4, atol=1e-5)
    assert np.allclose(d_a, through_b.T @ x64, rtol=1e-4, atol=1e-5)
    assert np.allclose(d_b, scale * dy64.T @ (x64 @ a64.T),
                       rtol=1e-4, atol=1e-5)
    # and each term is there at its full size
    assert np.abs(through_b @ a64).max() > 1e-2
    assert np.abs(dy64 @ dense).max() > 1e-2


def test_matmul_small_integer_case(oracle):
    left = np.array([[1, 2, 3], [4, 5, 6]], dtype=np.float32)
    right = np.array([[1, 0], [0, 1], [2, -1]], dtype=np.float32)
    assert oracle.matmul(left, right).tolist() == [[7.0, -1.0], [16.0, -1.0]]
    assert oracle.matmul_nt(left, np.ascontiguousarray(right.T)).tolist() == \
        [[7.0, -1.0], [16.0, -1.0]]
