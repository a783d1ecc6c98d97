"""Writes the golden vectors under tests/golden/ from the COMPILED REFERENCE.

Run in the build container, where /root/reference exists:

    make -C oracle _ref && python tests/golden/make_golden.py

Every expected value stored here was produced by the reference's own C++ CPU
backend (oracle/_ref/libnf4ref.so, built from the reference sources by
oracle/Makefile); the C restatement in oracle/ is not involved.  The fixtures
hold inputs' digests, packed payload digests and expected outputs -- data, no
reference source.  Inputs are regenerated from seeds by tests/helpers.py; the
stored digests detect a drifting random generator.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(HERE))

import helpers  # noqa: E402
from oracle.binding import Reference  # noqa: E402


def payload_digest(weight) -> dict:
    digest = {"codes_sha256": helpers.sha256(weight.codes)}
    if weight.fp32_scales is not None:
        digest["fp32_scales_sha256"] = helpers.sha256(weight.fp32_scales)
    else:
        digest["scale_codes_sha256"] = helpers.sha256(weight.scale_codes)
        digest["second_level_sha256"] = helpers.sha256(weight.second_level)
        digest["offset_bits"] = int(
            np.float32(weight.offset).view(np.uint32))
    return digest


def closed_form(reference) -> dict:
    """Aligned [3 x 32] and edge [33 x 33] fixtures, block 32, both encodings
    (tests/core/backend/test_quantized_linear_backend.cpp:250-302)."""
    arrays = {}
    cases = {
        "aligned": (helpers.aligned_weight(), helpers.aligned_input(),
                    helpers.aligned_upstream()),
        "edge": (helpers.edge_weight(), helpers.edge_input(),
                 helpers.edge_upstream()),
    }
    for name, (dense, x, dy) in cases.items():
        for double_quantized in (False, True):
            tag = f"{name}_{'dq' if double_quantized else 'fp32'}"
            weight = reference.quantize(dense, 32, double_quantized, 32)
            arrays[f"{tag}_codes"] = weight.codes
            if double_quantized:
                arrays[f"{tag}_scale_codes"] = weight.scale_codes
                arrays[f"{tag}_second_level"] = weight.second_level
                arrays[f"{tag}_offset"] = np.float32(weight.offset)
            else:
                arrays[f"{tag}_fp32_scales"] = weight.fp32_scales
            arrays[f"{tag}_dequantized"] = reference.dequantize(weight)
            arrays[f"{tag}_forward"] = reference.forward(x, weight)
            arrays[f"{tag}_input_backward"] = reference.input_backward(
                dy, weight)
    return arrays


def config1(reference):
    """The tiny parity configuration: x [16,256] ~N(0,1), W [768,256] ~N(0,0.02), block 64,
    bias [768] ~N(0,0.01); plus an upstream [16,768] ~N(0,1e-2) for backward."""
    x = helpers.normal(1, (16, 256), 1.0)
    dense = helpers.normal(2, (768, 256), 0.02)
    bias = helpers.normal(3, (768,), 0.01)
    dy = helpers.normal(4, (16, 768), 1.0e-2)
    arrays = {}
    meta = {"inputs": {"x": helpers.sha256(x), "w": helpers.sha256(dense),
                       "bias": helpers.sha256(bias),
                       "dy": helpers.sha256(dy)}}
    for double_quantized in (False, True):
        tag = "dq" if double_quantized else "fp32"
        weight = reference.quantize(dense, 64, double_quantized, 256)
        meta[tag] = payload_digest(weight)
        meta[tag]["dequantized_sha256"] = helpers.sha256(
            reference.dequantize(weight))
        arrays[f"{tag}_forward_bias"] = reference.forward(x, weight, bias)
        arrays[f"{tag}_forward"] = reference.forward(x, weight)
        arrays[f"{tag}_input_backward"] = reference.input_backward(dy, weight)
        if double_quantized:
            arrays["dq_scale_codes"] = weight.scale_codes
            arrays["dq_second_level"] = weight.second_level
            arrays["dq_offset"] = np.float32(weight.offset)
        else:
            arrays["fp32_scales"] = weight.fp32_scales
    return arrays, meta


LLAMA_CASES = {
    # name: (output_width, input_width, weight seed)
    "q_proj": (4096, 4096, 11),
    "gate_proj": (11008, 4096, 12),
    "down_proj": (4096, 11008, 13),
}


def llama(reference):
    """One row through each distinct Llama-7B projection shape, both scale
    encodings: payload digests, digest of deq(W), full y and dx rows."""
    arrays = {}
    meta = {}
    for name, (out_w, in_w, seed) in LLAMA_CASES.items():
        dense = helpers.normal(seed, (out_w, in_w), 0.02)
        x = helpers.normal(seed + 100, (1, in_w), 1.0)
        dy = helpers.normal(seed + 200, (1, out_w), 1.0e-2)
        meta[name] = {"inputs": {"w": helpers.sha256(dense),
                                 "x": helpers.sha256(x),
                                 "dy": helpers.sha256(dy)}}
        for double_quantized in (False, True):
            tag = "dq" if double_quantized else "fp32"
            weight = reference.quantize(dense, 64, double_quantized, 256)
            entry = payload_digest(weight)
            entry["payload_bytes"] = weight.payload_bytes
            entry["dequantized_sha256"] = helpers.sha256(
                reference.dequantize(weight))
            meta[name][tag] = entry
            arrays[f"{name}_{tag}_forward"] = reference.forward(x, weight)
            arrays[f"{name}_{tag}_input_backward"] = \
                reference.input_backward(dy, weight)
            print(name, tag, "done", flush=True)
    return arrays, meta


def packed_state(reference):
    """A three-entry packed model state (edge fp32, edge nested, aligned
    nested) written by oracle/packed_state.py, kept only because the
    reference's own reader (oracle/_ref/libstateref.so) returns exactly the
    fields it was written from; and, for each malformed variant of it, what
    that reader throws."""
    from oracle import packed_state as restated
    reader = restated.ReferenceReader()
    weights = [
        reference.quantize(helpers.edge_weight(), 32, False, 32),
        reference.quantize(helpers.edge_weight(), 32, True, 32),
        reference.quantize(helpers.aligned_weight(), 32, True, 32),
    ]
    entries = [restated.from_nf4_weight(weight) for weight in weights]
    blob = restated.serialize(entries)
    parsed = reader.parse(blob)
    assert len(parsed) == len(entries)
    for got, want in zip(parsed, entries):
        assert got.shape == list(want.shape)
        assert got.block_size == want.block_size
        assert got.double_quantized == want.double_quantized
        assert np.array_equal(got.packed_codes, want.packed_codes)
        assert np.array_equal(bits_of(got.block_scales),
                              bits_of(want.block_scales))
        if want.double_quantized:
            assert np.array_equal(got.scale_codes, want.scale_codes)
            assert np.array_equal(bits_of(got.second_level_scales),
                                  bits_of(want.second_level_scales))
            assert got.scale_block_size == want.scale_block_size
            assert np.float32(got.offset).view(np.uint32) == \
                np.float32(want.offset).view(np.uint32)
    outcomes = {}
    for name, data in helpers.packed_state_mutations(blob):
        try:
            outcomes[name] = ["ok", len(reader.parse(data))]
        except (ValueError, OverflowError) as error:
            outcomes[name] = [type(error).__name__, str(error)]
    with open(os.path.join(HERE, "packed_state.bin"), "wb") as handle:
        handle.write(blob)
    with open(os.path.join(HERE, "packed_state_outcomes.json"), "w") as handle:
        json.dump(outcomes, handle, indent=1, sort_keys=True)


def scale_storage_verdicts(reference):
    """What the reference's dispatcher says about each scale storage of
    helpers.scale_storage_cases() (its require_scale_storage, reached through
    a forward request on the CPU backend)."""
    verdicts = {
        name: helpers.verdict(reference.validate_scale_storage, weight,
                              expected)
        for name, weight, expected in helpers.scale_storage_cases()}
    with open(os.path.join(HERE, "scale_storage_verdicts.json"), "w") as out:
        json.dump(verdicts, out, indent=1, sort_keys=True)


def lora_steps(reference) -> dict:
    """Forward value and the gradients on x, A and B that the reference's
    autograd leaves after one backward pass through a real Linear (packed
    weight, adapter attached) for each of helpers.LORA_STEP_CASES."""
    arrays = {}
    for name in helpers.LORA_STEP_CASES:
        case = helpers.lora_step_inputs(name)
        y, dx, d_a, d_b = reference.lora_linear_step(
            case["dense"], case["block"], case["second"], case["x"],
            case["dy"], case["lora_a"], case["lora_b"], case["alpha"],
            bias=case["bias"])
        arrays[f"{name}_y"] = y
        arrays[f"{name}_dx"] = dx
        arrays[f"{name}_d_lora_a"] = d_a
        arrays[f"{name}_d_lora_b"] = d_b
        arrays[f"{name}_inputs_sha256"] = np.frombuffer(
            helpers.sha256(np.concatenate(
                [case[key].ravel() for key in
                 ("dense", "x", "dy", "lora_a", "lora_b")])).encode(),
            dtype=np.uint8)
    return arrays


def bits_of(array):
    return np.ascontiguousarray(array, dtype=np.float32).view(np.uint32)


def main():
    reference = Reference()
    packed_state(reference)
    scale_storage_verdicts(reference)
    np.savez_compressed(os.path.join(HERE, "lora_steps.npz"),
                        **lora_steps(reference))
    np.savez_compressed(os.path.join(HERE, "closed_form.npz"),
                        **closed_form(reference))
    arrays, meta1 = config1(reference)
    np.savez_compressed(os.path.join(HERE, "config1.npz"), **arrays)
    arrays, meta2 = llama(reference)
    np.savez_compressed(os.path.join(HERE, "llama_rows.npz"), **arrays)
    with open(os.path.join(HERE, "digests.json"), "w") as handle:
        json.dump({"numpy": np.__version__, "config1": meta1,
                   "llama": meta2}, handle, indent=1, sort_keys=True)
    print("golden vectors written to", HERE)


if __name__ == "__main__":
    main()
