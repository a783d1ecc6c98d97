"""Pins of the CPU restatement that need neither the reference nor fixtures:
what the mathematics fixes.  Each is chosen so that a plausible slip (wrong
nibble, transposed operand, dropped scale, block index per row instead of
flat) fails it."""
import numpy as np
import pytest

import helpers
from oracle.binding import (SCALE_DOUBLE_QUANTIZED_UINT8, SCALE_FLOAT32,
                            Nf4Weight)


def dense_by_hand(weight, codebook, scales):
    """deq(W) from first principles in numpy: flat index j -> byte j//2,
    low nibble for even j; block j // B over the FLATTENED weight."""
    count = weight.element_count
    flat = np.arange(count)
    byte = weight.codes[flat // 2]
    code = np.where(flat % 2 == 0, byte & 0x0F, byte >> 4)
    return (codebook[code] * scales[flat // weight.block_size]).astype(
        np.float32).reshape(weight.output_width, weight.input_width)


@pytest.mark.parametrize("shape,block", [((7, 48), 32), ((33, 33), 32),
                                         ((5, 200), 64), ((3, 64), 128)])
def test_dequantize_matches_first_principles(oracle, shape, block):
    dense = helpers.normal(21, shape, 0.02)
    weight = oracle.quantize(dense, block)
    expected = dense_by_hand(weight, oracle.codebook(), weight.fp32_scales)
    helpers.assert_bit_equal(oracle.dequantize(weight), expected)
    # absmax scaling: the block's extreme element round-trips exactly
    flat = dense.ravel()
    restored = oracle.dequantize(weight).ravel()
    for start in range(0, flat.size, block):
        chunk = flat[start:start + block]
        peak = start + int(np.argmax(np.abs(chunk)))
        assert restored[peak] == flat[peak]


@pytest.mark.parametrize("rows,shape,block,dq", [
    (3, (7, 48), 32, False), (2, (33, 33), 32, True),
    (4, (16, 256), 64, True), (1, (9, 130), 64, False)])
def test_products_match_fp64_brute_force(oracle, rows, shape, block, dq):
    out_w, in_w = shape
    weight = oracle.quantize(helpers.normal(22, shape, 0.02), block, dq, 32)
    dense = oracle.dequantize(weight)
    x = helpers.normal(23, (rows, in_w), 1.0)
    dy = helpers.normal(24, (rows, out_w), 1.0e-2)
    for faithful in (True, False):
        y = oracle.forward(x, weight, faithful=faithful)
        dx = oracle.input_backward(dy, weight, faithful=faithful)
        assert y.shape == (rows, out_w) and dx.shape == (rows, in_w)
        assert np.allclose(y, helpers.exact_forward(x, dense), rtol=0,
                           atol=2e-6 * np.sqrt(in_w))
        assert np.allclose(dx, helpers.exact_input_backward(dy, dense),
                           rtol=0, atol=2e-8 * np.sqrt(out_w))


def test_sequential_accumulation_order(oracle):
    # fp32 sums in ascending index order: reproduce one output by hand.
    weight = oracle.quantize(helpers.normal(25, (4, 96), 0.02), 32)
    dense = oracle.dequantize(weight)
    x = helpers.normal(26, (2, 96), 1.0)
    total = np.float32(0.0)
    for i in range(96):
        total = np.float32(total + np.float32(x[1, i] * dense[2, i]))
    assert oracle.forward(x, weight, faithful=True)[1, 2] == total
    dy = helpers.normal(27, (2, 4), 1.0)
    total = np.float32(0.0)
    for o in range(4):
        total = np.float32(total + np.float32(dy[0, o] * dense[o, 5]))
    assert oracle.input_backward(dy, weight, faithful=True)[0, 5] == total


def test_special_cases(oracle):
    codebook = oracle.codebook()
    # all codes 7 -> every output is zero whatever the scales are
    zero = Nf4Weight(4, 64, 32, np.full(128, 0x77, np.uint8), SCALE_FLOAT32,
                     fp32_scales=np.full(8, 3.5, np.float32))
    x = helpers.normal(28, (2, 64), 1.0)
    assert not oracle.forward(x, zero).any()
    # unit scales and a one-hot x pick out a codebook column
    codes = (np.arange(128) % 256).astype(np.uint8)
    ramp = Nf4Weight(4, 64, 32, codes, SCALE_FLOAT32,
                     fp32_scales=np.ones(8, np.float32))
    for column in (0, 1, 17, 63):
        one_hot = np.zeros((1, 64), np.float32)
        one_hot[0, column] = 1.0
        y = oracle.forward(one_hot, ramp).ravel()
        for row in range(4):
            flat = row * 64 + column
            byte = int(codes[flat // 2])
            code = byte & 15 if flat % 2 == 0 else byte >> 4
            assert y[row] == codebook[code]
    # linearity in the scale: doubling every scale doubles y exactly
    doubled = Nf4Weight(4, 64, 32, codes, SCALE_FLOAT32,
                        fp32_scales=np.full(8, 2.0, np.float32))
    assert np.array_equal(oracle.forward(x, doubled),
                          2.0 * oracle.forward(x, ramp))


def test_double_quantized_scale_decode(oracle):
    # second-level scale 0 -> every block scale equals the offset
    flat = Nf4Weight(2, 64, 32, np.zeros(64, np.uint8),
                     SCALE_DOUBLE_QUANTIZED_UINT8,
                     scale_codes=np.array([1, 90, 128, 255], np.uint8),
                     second_level=np.zeros(1, np.float32),
                     second_level_block=32, offset=0.375)
    assert oracle.decode_scales(flat).tolist() == [0.375] * 4
    # general case against the formula evaluated in numpy float32
    weight = Nf4Weight(1, 32 * 70, 32, np.zeros(16 * 70, np.uint8),
                       SCALE_DOUBLE_QUANTIZED_UINT8,
                       scale_codes=(np.arange(70) * 37 % 256).astype(np.uint8),
                       second_level=np.array([0.5, 0.25, 3.0], np.float32),
                       second_level_block=32, offset=0.125)
    factor = ((weight.scale_codes.astype(np.int32) - 128).astype(np.float32)
              / np.float32(127.0))
    delta = weight.second_level[np.arange(70) // 32] * factor
    expected = np.maximum(np.float32(0.125) + delta, np.float32(0.0))
    helpers.assert_bit_equal(oracle.decode_scales(weight), expected)
    # clamp at zero and saturation at FLT_MAX
    low = Nf4Weight(1, 32, 32, np.zeros(16, np.uint8),
                    SCALE_DOUBLE_QUANTIZED_UINT8,
                    scale_codes=np.array([1], np.uint8),
                    second_level=np.array([2.0], np.float32),
                    second_level_block=32, offset=1.0)
    assert oracle.decode_scales(low)[0] == 0.0
    fmax = np.finfo(np.float32).max
    high = Nf4Weight(1, 32, 32, np.zeros(16, np.uint8),
                     SCALE_DOUBLE_QUANTIZED_UINT8,
                     scale_codes=np.array([255], np.uint8),
                     second_level=np.array([fmax], np.float32),
                     second_level_block=32, offset=float(fmax))
    assert oracle.decode_scales(high)[0] == fmax


def test_double_quantizer_round_trip_bound(oracle):
    # |decode(encode(s)) - s| <= t_g / 254 + rounding: the 8-bit grid step.
    scales = np.abs(helpers.normal(29, (1000,), 0.05)) + np.float32(0.01)
    codes, second, offset = oracle.double_quantize_scales(scales, 256)
    weight = Nf4Weight(1, 64 * 1000, 64, np.zeros(32 * 1000, np.uint8),
                       SCALE_DOUBLE_QUANTIZED_UINT8, scale_codes=codes,
                       second_level=second, second_level_block=256,
                       offset=offset)
    decoded = oracle.decode_scales(weight)
    step = second[np.arange(1000) // 256] / 127.0
    assert np.all(np.abs(decoded - scales) <= 0.5 * step * 1.0001 + 1e-9)
    assert abs(offset - scales.astype(np.float64).mean()) < 1e-8
    for group in range(4):
        chunk = scales[group * 256:(group + 1) * 256]
        assert second[group] == np.abs(chunk - np.float32(offset)).max()


def test_bias_is_a_separate_add(oracle):
    # src/nn/linear.cpp:165-168
    weight = oracle.quantize(helpers.normal(30, (8, 64), 0.02), 64)
    x = helpers.normal(31, (3, 64), 1.0)
    bias = helpers.normal(32, (8,), 0.01)
    helpers.assert_bit_equal(oracle.forward(x, weight, bias),
                             oracle.forward(x, weight) + bias[None, :])


def test_lora_with_zero_b_is_the_plain_layer(oracle):
    """A freshly attached adapter has B = 0 (tests/nn/test_lora.cpp:150-157):
    the layer's output is then exactly the base output."""
    dense = helpers.normal(30, (48, 128), 0.02)
    weight = oracle.quantize(dense, 64)
    x = helpers.normal(31, (4, 128), 1.0)
    bias = helpers.normal(32, (48,), 0.01)
    lora_a = helpers.normal(33, (8, 128), 0.05)
    lora_b = np.zeros((48, 8), dtype=np.float32)
    helpers.assert_bit_equal(
        oracle.lora_forward(x, weight, lora_a, lora_b, 2.0, bias),
        oracle.forward(x, weight, bias))


def test_lora_matches_float64_composition(oracle):
    dense = helpers.normal(34, (96, 256), 0.02)
    weight = oracle.quantize(dense, 64, True, 32)
    x = helpers.normal(35, (6, 256), 1.0)
    lora_a = helpers.normal(36, (16, 256), 0.05)
    lora_b = helpers.normal(37, (96, 16), 0.05)
    deq = oracle.dequantize(weight).astype(np.float64)
    exact = x.astype(np.float64) @ deq.T + 0.5 * (
        (x.astype(np.float64) @ lora_a.astype(np.float64).T)
        @ lora_b.astype(np.float64).T)
    got = oracle.lora_forward(x, weight, lora_a, lora_b, 0.5)
    assert np.max(np.abs(got - exact)) <= 1e-5 * np.max(np.abs(exact))
