"""Where oracle/_ref was built (the container that holds the reference), diff
the C restatement against the compiled reference on fresh seeded inputs,
including error behaviour.  Skipped where the reference build is absent."""
import numpy as np
import pytest

import helpers
from oracle.binding import (SCALE_DOUBLE_QUANTIZED_UINT8, SCALE_FLOAT32,
                            Nf4Weight)


def same_payload(a, b):
    assert np.array_equal(a.codes, b.codes)
    if a.encoding == SCALE_FLOAT32:
        helpers.assert_bit_equal(a.fp32_scales, b.fp32_scales)
    else:
        assert np.array_equal(a.scale_codes, b.scale_codes)
        helpers.assert_bit_equal(a.second_level, b.second_level)
        helpers.assert_bit_equal(np.float32(a.offset), np.float32(b.offset))


@pytest.mark.parametrize("shape,block,second", [
    ((768, 256), 64, 256), ((33, 33), 32, 32), ((17, 96), 32, 64),
    ((5, 4096), 4096, 32), ((64, 1000), 128, 32), ((1, 1), 32, 32)])
@pytest.mark.parametrize("double_quantized", [False, True])
@pytest.mark.parametrize("sigma", [0.02, 1.0])
def test_bitwise_agreement(oracle, reference, shape, block, second,
                           double_quantized, sigma):
    out_w, in_w = shape
    dense = helpers.normal(41, shape, sigma)
    dense.ravel()[::7] = 0.0  # exact zeros and ties at code 7
    mine = oracle.quantize(dense, block, double_quantized, second)
    theirs = reference.quantize(dense, block, double_quantized, second)
    same_payload(mine, theirs)
    helpers.assert_bit_equal(oracle.dequantize(mine),
                             reference.dequantize(mine))
    x = helpers.normal(42, (3, in_w), 1.0)
    dy = helpers.normal(43, (3, out_w), 1.0e-2)
    helpers.assert_bit_equal(oracle.forward(x, mine, faithful=True),
                             reference.forward(x, mine))
    helpers.assert_bit_equal(oracle.forward(x, mine),
                             reference.forward(x, mine))
    helpers.assert_bit_equal(oracle.input_backward(dy, mine, faithful=True),
                             reference.input_backward(dy, mine))
    helpers.assert_bit_equal(oracle.input_backward(dy, mine),
                             reference.input_backward(dy, mine))


def test_zero_block_and_constant_scales(oracle, reference):
    dense = np.zeros((4, 64), np.float32)
    dense[2] = 0.5
    for dq in (False, True):
        same_payload(oracle.quantize(dense, 32, dq, 32),
                     reference.quantize(dense, 32, dq, 32))


def test_validation_agrees(oracle, reference):
    def legacy(codes, scales):
        return Nf4Weight(1, 1, 32, np.array(codes, np.uint8), SCALE_FLOAT32,
                         fp32_scales=np.array(scales, np.float32))

    def nested(**changes):
        weight = Nf4Weight(1, 1, 32, np.array([0x07], np.uint8),
                           SCALE_DOUBLE_QUANTIZED_UINT8,
                           scale_codes=np.array([128], np.uint8),
                           second_level=np.zeros(1, np.float32),
                           second_level_block=32, offset=0.0)
        for key, value in changes.items():
            setattr(weight, key, value)
        return weight

    good = [legacy([0x07], [0.0]), nested()]
    bad = [
        legacy([], [0.0]), legacy([0x07], []), legacy([0xF7], [0.0]),
        legacy([0x08], [0.0]), legacy([0x07], [-1.0]),
        legacy([0x07], [np.inf]),
        nested(fp32_scales=np.zeros(1, np.float32)),
        nested(scale_codes=np.zeros(0, np.uint8)),
        nested(second_level_block=16),
        nested(second_level=np.zeros(0, np.float32)),
        nested(second_level=np.array([-1.0], np.float32)),
        nested(offset=float("inf")),
    ]
    for weight in good:
        oracle.validate_payload(weight)
        reference.validate_payload(weight)
    for weight in bad:
        with pytest.raises(ValueError) as mine:
            oracle.validate_payload(weight)
        with pytest.raises(ValueError) as theirs:
            reference.validate_payload(weight)
        assert str(mine.value) == str(theirs.value)


def test_scale_storage_verdicts_agree(oracle, reference):
    """nf4o_validate_scale_storage against the reference dispatcher's own
    check (dispatch.cpp:108-154), outcome, exception type and message."""
    for name, weight, expected in helpers.scale_storage_cases():
        mine = helpers.verdict(oracle.validate_scale_storage, weight,
                               expected)
        theirs = helpers.verdict(reference.validate_scale_storage, weight,
                                 expected)
        assert mine == theirs, name


def test_memory_usage_known_answers(oracle, reference):
    # tests/core/test_quantization.cpp:188-198 and :368-376
    values = np.repeat(np.arange(33, dtype=np.float32), 32)
    weight = oracle.quantize(values, 32, True, 32)
    usage = reference.memory_usage(weight)
    assert usage == {
        "packed_code_bytes": 528, "scale_bytes": 45,
        "logical_payload_bytes": 573, "resident_payload_bytes": 573,
        "fp32_equivalent_bytes": 4224, "fp32_scale_bytes": 0,
        "scale_code_bytes": 33, "second_level_scale_bytes": 8,
        "scale_offset_bytes": 4}
    assert oracle.scale_payload_bytes(weight) == usage["scale_bytes"]
    assert weight.payload_bytes == usage["logical_payload_bytes"]


@pytest.mark.parametrize("rows,shared,columns", [
    (1, 1, 1), (3, 33, 5), (16, 256, 8), (7, 1000, 64)])
def test_matmul_bitwise(oracle, reference, rows, shared, columns):
    left = helpers.normal(44, (rows, shared), 1.0)
    right = helpers.normal(45, (shared, columns), 0.05)
    theirs = reference.matmul(left, right)
    helpers.assert_bit_equal(oracle.matmul(left, right), theirs)
    # the transposed-operand form is the same sum
    helpers.assert_bit_equal(
        oracle.matmul_nt(left, np.ascontiguousarray(right.T)), theirs)


@pytest.mark.parametrize("shape,block,rank", [
    ((768, 256), 64, 8), ((33, 33), 32, 2), ((64, 1000), 128, 16),
    ((40, 96), 32, 64)])
@pytest.mark.parametrize("double_quantized", [False, True])
@pytest.mark.parametrize("with_bias", [False, True])
def test_lora_linear_forward_bitwise(oracle, reference, shape, block, rank,
                                     double_quantized, with_bias):
    out_w, in_w = shape
    dense = helpers.normal(46, shape, 0.02)
    weight = oracle.quantize(dense, block, double_quantized, 32)
    x = helpers.normal(47, (5, in_w), 1.0)
    lora_a = helpers.normal(48, (rank, in_w), 0.05)
    lora_b = helpers.normal(49, (out_w, rank), 0.05)
    bias = helpers.normal(50, (out_w,), 0.01) if with_bias else None
    helpers.assert_bit_equal(
        oracle.lora_forward(x, weight, lora_a, lora_b, 16.0 / rank, bias),
        reference.lora_forward(x, weight, lora_a, lora_b, 16.0 / rank, bias))


@pytest.mark.parametrize("name", sorted(helpers.LORA_STEP_CASES))
def test_lora_linear_step_bitwise(oracle, reference, name):
    """The restated adapter backward against the gradients the reference's
    autograd leaves on x, A and B of a real Linear that packed the weight
    itself (quantize_weight_nf4[_double_quantized], attach_lora, forward,
    backward)."""
    case = helpers.lora_step_inputs(name)
    y, dx, d_a, d_b = reference.lora_linear_step(
        case["dense"], case["block"], case["second"], case["x"], case["dy"],
        case["lora_a"], case["lora_b"], case["alpha"], bias=case["bias"])
    weight = oracle.quantize(case["dense"], case["block"],
                             case["second"] != 0, case["second"] or 256)
    helpers.assert_bit_equal(
        oracle.lora_forward(case["x"], weight, case["lora_a"],
                            case["lora_b"], case["scale"], case["bias"]), y)
    ours = oracle.lora_backward(case["dy"], case["x"], weight, case["lora_a"],
                                case["lora_b"], case["scale"])
    helpers.assert_bit_equal(ours[0], dx, "dx")
    helpers.assert_bit_equal(ours[1], d_a, "dA")
    helpers.assert_bit_equal(ours[2], d_b, "dB")
