"""The CPU restatement against the golden vectors written from the COMPILED
reference (tests/golden/make_golden.py): payload bytes, dequantised weights,
y and dx must agree bit for bit."""
import json
import os

import numpy as np
import pytest

import helpers

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def digests():
    with open(os.path.join(GOLDEN, "digests.json")) as handle:
        return json.load(handle)


def check_payload(weight, expected):
    assert helpers.sha256(weight.codes) == expected["codes_sha256"]
    if "fp32_scales_sha256" in expected:
        assert helpers.sha256(weight.fp32_scales) == \
            expected["fp32_scales_sha256"]
    else:
        assert helpers.sha256(weight.scale_codes) == \
            expected["scale_codes_sha256"]
        assert helpers.sha256(weight.second_level) == \
            expected["second_level_sha256"]
        assert int(np.float32(weight.offset).view(np.uint32)) == \
            expected["offset_bits"]


CLOSED_FORM = {
    "aligned": (helpers.aligned_weight, helpers.aligned_input,
                helpers.aligned_upstream),
    "edge": (helpers.edge_weight, helpers.edge_input, helpers.edge_upstream),
}


@pytest.mark.parametrize("name", ["aligned", "edge"])
@pytest.mark.parametrize("double_quantized", [False, True])
def test_closed_form_fixtures(oracle, name, double_quantized):
    golden = np.load(os.path.join(GOLDEN, "closed_form.npz"))
    make_weight, make_input, make_upstream = CLOSED_FORM[name]
    tag = f"{name}_{'dq' if double_quantized else 'fp32'}"
    weight = oracle.quantize(make_weight(), 32, double_quantized, 32)
    assert np.array_equal(weight.codes, golden[f"{tag}_codes"])
    if double_quantized:
        assert np.array_equal(weight.scale_codes,
                              golden[f"{tag}_scale_codes"])
        helpers.assert_bit_equal(weight.second_level,
                                 golden[f"{tag}_second_level"])
        helpers.assert_bit_equal(np.float32(weight.offset),
                                 golden[f"{tag}_offset"])
    else:
        helpers.assert_bit_equal(weight.fp32_scales,
                                 golden[f"{tag}_fp32_scales"])
    helpers.assert_bit_equal(oracle.dequantize(weight),
                             golden[f"{tag}_dequantized"], "dequantize")
    for faithful in (True, False):
        helpers.assert_bit_equal(
            oracle.forward(make_input(), weight, faithful=faithful),
            golden[f"{tag}_forward"], "forward")
        helpers.assert_bit_equal(
            oracle.input_backward(make_upstream(), weight, faithful=faithful),
            golden[f"{tag}_input_backward"], "input backward")
    if name == "edge":
        # tests/core/backend/test_quantized_linear_backend.cpp:272-302
        assert weight.element_count % 2 == 1
        assert weight.block_count == 35
        assert weight.element_count % 32 == 1
        assert weight.codes[-1] & 0xF0 == 0
        if double_quantized:
            assert weight.second_level.size == 2


@pytest.mark.parametrize("double_quantized", [False, True])
def test_config1(oracle, digests, double_quantized):
    golden = np.load(os.path.join(GOLDEN, "config1.npz"))
    meta = digests["config1"]
    x = helpers.normal(1, (16, 256), 1.0)
    dense = helpers.normal(2, (768, 256), 0.02)
    bias = helpers.normal(3, (768,), 0.01)
    dy = helpers.normal(4, (16, 768), 1.0e-2)
    assert helpers.sha256(x) == meta["inputs"]["x"], "random stream drifted"
    assert helpers.sha256(dense) == meta["inputs"]["w"]
    assert helpers.sha256(bias) == meta["inputs"]["bias"]
    assert helpers.sha256(dy) == meta["inputs"]["dy"]
    tag = "dq" if double_quantized else "fp32"
    weight = oracle.quantize(dense, 64, double_quantized, 256)
    check_payload(weight, meta[tag])
    assert helpers.sha256(oracle.dequantize(weight)) == \
        meta[tag]["dequantized_sha256"]
    helpers.assert_bit_equal(oracle.forward(x, weight, faithful=True),
                             golden[f"{tag}_forward"])
    helpers.assert_bit_equal(oracle.forward(x, weight, bias, faithful=True),
                             golden[f"{tag}_forward_bias"])
    helpers.assert_bit_equal(oracle.input_backward(dy, weight, faithful=True),
                             golden[f"{tag}_input_backward"])


@pytest.mark.parametrize("name,out_w,in_w,seed", [
    ("q_proj", 4096, 4096, 11),
    ("gate_proj", 11008, 4096, 12),
    ("down_proj", 4096, 11008, 13),
])
@pytest.mark.parametrize("double_quantized", [False, True])
def test_llama_rows(oracle, digests, name, out_w, in_w, seed,
                    double_quantized):
    golden = np.load(os.path.join(GOLDEN, "llama_rows.npz"))
    meta = digests["llama"][name]
    dense = helpers.normal(seed, (out_w, in_w), 0.02)
    x = helpers.normal(seed + 100, (1, in_w), 1.0)
    dy = helpers.normal(seed + 200, (1, out_w), 1.0e-2)
    assert helpers.sha256(dense) == meta["inputs"]["w"]
    tag = "dq" if double_quantized else "fp32"
    weight = oracle.quantize(dense, 64, double_quantized, 256)
    check_payload(weight, meta[tag])
    assert weight.payload_bytes == meta[tag]["payload_bytes"]
    assert helpers.sha256(oracle.dequantize(weight)) == \
        meta[tag]["dequantized_sha256"]
    helpers.assert_bit_equal(oracle.forward(x, weight),
                             golden[f"{name}_{tag}_forward"])
    helpers.assert_bit_equal(oracle.input_backward(dy, weight),
                             golden[f"{name}_{tag}_input_backward"])


def test_payload_bytes_match_the_published_figures(oracle, digests):
    # expected: 9 437 184 / 25 362 432 B (fp32 scales), 8 654 852 /
    # 23 259 908 B (double-quantised, C = 256).
    llama = digests["llama"]
    assert llama["q_proj"]["fp32"]["payload_bytes"] == 9437184
    assert llama["gate_proj"]["fp32"]["payload_bytes"] == 25362432
    assert llama["down_proj"]["fp32"]["payload_bytes"] == 25362432
    assert llama["q_proj"]["dq"]["payload_bytes"] == 8654852
    assert llama["gate_proj"]["dq"]["payload_bytes"] == 23259908


def test_scale_storage_verdicts(oracle):
    """The restated scale-storage check gives the verdicts the compiled
    reference's dispatcher gave (tests/golden/scale_storage_verdicts.json,
    written by make_golden.py)."""
    with open(os.path.join(GOLDEN, "scale_storage_verdicts.json")) as handle:
        expected = json.load(handle)
    cases = helpers.scale_storage_cases()
    assert sorted(expected) == sorted(name for name, _, _ in cases)
    outcomes = set()
    for name, weight, count in cases:
        got = helpers.verdict(oracle.validate_scale_storage, weight, count)
        assert got == expected[name], name
        outcomes.add(got[1])
    # "ok" and every message the check can give for finite arithmetic (a
    # non-finite reconstruction needs a non-finite second-level scale or
    # offset, and those are rejected first)
    assert len(outcomes) == 6


@pytest.mark.parametrize("name", sorted(helpers.LORA_STEP_CASES))
def test_lora_steps(oracle, name):
    """Forward value and gradients of a Linear with a packed weight and an
    adapter, as the compiled reference's autograd produced them."""
    golden = np.load(os.path.join(GOLDEN, "lora_steps.npz"))
    case = helpers.lora_step_inputs(name)
    digest = helpers.sha256(np.concatenate(
        [case[key].ravel() for key in
         ("dense", "x", "dy", "lora_a", "lora_b")]))
    assert digest == bytes(golden[f"{name}_inputs_sha256"]).decode()
    weight = oracle.quantize(case["dense"], case["block"],
                             case["second"] != 0, case["second"] or 256)
    helpers.assert_bit_equal(
        oracle.lora_forward(case["x"], weight, case["lora_a"],
                            case["lora_b"], case["scale"], case["bias"]),
        golden[f"{name}_y"])
    dx, d_a, d_b = oracle.lora_backward(
        case["dy"], case["x"], weight, case["lora_a"], case["lora_b"],
        case["scale"])
    helpers.assert_bit_equal(dx, golden[f"{name}_dx"], "dx")
    helpers.assert_bit_equal(d_a, golden[f"{name}_d_lora_a"], "dA")
    helpers.assert_bit_equal(d_b, golden[f"{name}_d_lora_b"], "dB")
