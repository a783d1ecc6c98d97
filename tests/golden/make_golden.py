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
    """BASELINE config 1: x [16,256] ~N(0,1), W [768,256] ~N(0,0.02), block 64,
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


def main():
    reference = Reference()
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
