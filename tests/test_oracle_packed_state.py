"""The oracle's restatement of the packed model state (oracle/packed_state.py)
against the reference's reader: through the committed fixture everywhere, and
directly against the compiled reader where oracle/_ref was built.

Reference: src/c_api/model_state.cpp:34-113 (writer), :166-300 (reader); the
reference's own test is a round trip plus a truncated load
(tests/abi/test_c_api.c:3267-3302).
"""
import json
import os
import struct

import numpy as np
import pytest

import helpers
from oracle import packed_state
from oracle.binding import SCALE_DOUBLE_QUANTIZED_UINT8

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def golden_blob() -> bytes:
    with open(os.path.join(GOLDEN, "packed_state.bin"), "rb") as handle:
        return handle.read()


def outcome_of(parse, data):
    try:
        return ["ok", len(parse(data))]
    except (ValueError, OverflowError) as error:
        return [type(error).__name__, str(error)]


def assert_same_entries(got, want):
    assert len(got) == len(want)
    for mine, theirs in zip(got, want):
        assert list(mine.shape) == list(theirs.shape)
        assert mine.block_size == theirs.block_size
        assert mine.double_quantized == theirs.double_quantized
        assert np.array_equal(mine.packed_codes, theirs.packed_codes)
        helpers.assert_bit_equal(mine.block_scales, theirs.block_scales)
        if mine.double_quantized:
            assert np.array_equal(mine.scale_codes, theirs.scale_codes)
            helpers.assert_bit_equal(mine.second_level_scales,
                                     theirs.second_level_scales)
            assert mine.scale_block_size == theirs.scale_block_size
            helpers.assert_bit_equal(np.float32(mine.offset),
                                     np.float32(theirs.offset))


def test_fixture_reads_back_as_the_weights_it_was_written_from(oracle):
    """The fixture was accepted by the reference's reader with these fields
    (tests/golden/make_golden.py); the payloads are the closed-form weights."""
    entries = packed_state.parse(golden_blob())
    assert [e.shape for e in entries] == [[33, 33], [33, 33], [3, 32]]
    assert [e.double_quantized for e in entries] == [False, True, True]
    assert [e.block_size for e in entries] == [32, 32, 32]
    stored = np.load(os.path.join(GOLDEN, "closed_form.npz"))
    assert np.array_equal(entries[0].packed_codes, stored["edge_fp32_codes"])
    helpers.assert_bit_equal(entries[0].block_scales,
                             stored["edge_fp32_fp32_scales"])
    for entry, tag in ((entries[1], "edge_dq"), (entries[2], "aligned_dq")):
        assert np.array_equal(entry.packed_codes, stored[f"{tag}_codes"])
        assert np.array_equal(entry.scale_codes, stored[f"{tag}_scale_codes"])
        helpers.assert_bit_equal(entry.second_level_scales,
                                 stored[f"{tag}_second_level"])
        helpers.assert_bit_equal(np.float32(entry.offset),
                                 stored[f"{tag}_offset"])
        assert entry.scale_block_size == 32
        assert entry.block_scales.size == 0
    assert packed_state.serialize(entries) == golden_blob()


def test_known_layout_of_the_smallest_state():
    """One scalar zero weight, by hand from the writer's field order
    (src/c_api/model_state.cpp:44-111): 8 + 8 + 7*8 + 4 + 4 + 2*8 + 1 + 4."""
    entry = packed_state.PackedWeightState(
        [1, 1], 32, np.array([0x07], np.uint8), np.zeros(1, np.float32))
    blob = packed_state.serialize([entry])
    assert len(blob) == 101
    assert blob[:8] == b"RTNF4S1\x00"
    assert struct.unpack_from("<8Q", blob, 8) == (1, 2, 32, 1, 1, 0, 0, 0)
    assert struct.unpack_from("<2I", blob, 72) == (0, 0)
    assert struct.unpack_from("<2Q", blob, 80) == (1, 1)
    assert blob[96:] == b"\x07\x00\x00\x00\x00"
    nested = packed_state.PackedWeightState(
        [1, 1], 64, np.array([0x07], np.uint8), np.zeros(0, np.float32),
        True, np.array([128], np.uint8), np.array([2.0], np.float32), 256, 0.5)
    blob = packed_state.serialize([nested])
    assert struct.unpack_from("<8Q", blob, 8) == (1, 2, 64, 1, 0, 1, 1, 256)
    assert struct.unpack_from("<fI", blob, 72) == (0.5, 1)
    assert blob[96:] == b"\x07\x80" + struct.pack("<f", 2.0)


def test_malformed_states_fail_as_the_reference_reader_does():
    with open(os.path.join(GOLDEN, "packed_state_outcomes.json")) as handle:
        expected = json.load(handle)
    cases = helpers.packed_state_mutations(golden_blob())
    assert sorted(name for name, _ in cases) == sorted(expected)
    for name, data in cases:
        assert outcome_of(packed_state.parse, data) == expected[name], name
    kinds = {outcome[0] for outcome in expected.values()}
    assert kinds == {"ok", "ValueError", "OverflowError"}


@pytest.fixture(scope="module")
def reference_reader():
    if not packed_state.ReferenceReader.available():
        pytest.skip("oracle/_ref/libstateref.so is not built here")
    return packed_state.ReferenceReader()


def random_state(oracle, seed):
    generator = np.random.default_rng(seed)
    entries = []
    for index in range(int(generator.integers(1, 5))):
        rows = int(generator.integers(1, 40))
        columns = int(generator.integers(1, 70))
        block = int(generator.choice([32, 64, 128]))
        nested = bool(generator.integers(0, 2))
        dense = helpers.normal(seed * 10 + index, (rows, columns), 0.02)
        weight = oracle.quantize(dense, block, nested, 32)
        assert (weight.encoding == SCALE_DOUBLE_QUANTIZED_UINT8) == nested
        entries.append(packed_state.from_nf4_weight(weight))
    return entries


def test_written_states_are_read_identically_by_the_reference(
        oracle, reference_reader):
    for seed in range(20):
        entries = random_state(oracle, 500 + seed)
        blob = packed_state.serialize(entries)
        assert_same_entries(reference_reader.parse(blob), entries)
        assert_same_entries(packed_state.parse(blob), entries)


def test_random_damage_is_judged_as_by_the_reference(oracle,
                                                     reference_reader):
    generator = np.random.default_rng(77)
    agreed = {"ok": 0, "ValueError": 0, "OverflowError": 0}
    for seed in range(12):
        blob = packed_state.serialize(random_state(oracle, 900 + seed))
        for _ in range(60):
            data = bytearray(blob)
            kind = int(generator.integers(0, 3))
            if kind == 0:
                data = data[:int(generator.integers(0, len(data)))]
            elif kind == 1:
                # overwrite an aligned 8-byte word in the first 200 bytes
                position = 8 * int(generator.integers(1, 25))
                if position + 8 <= len(data):
                    values = [0, 1, 2, 3, 31, 1 << 40, 1 << 62, (1 << 64) - 1]
                    value = values[int(generator.integers(0, len(values)))]
                    struct.pack_into("<Q", data, position, value)
            else:
                position = int(generator.integers(0, min(len(data), 200)))
                data[position] ^= 1 << int(generator.integers(0, 8))
            data = bytes(data)
            mine = outcome_of(packed_state.parse, data)
            theirs = outcome_of(reference_reader.parse, data)
            assert mine == theirs
            agreed[mine[0]] += 1
            if mine[0] == "ok":
                assert_same_entries(packed_state.parse(data),
                                    reference_reader.parse(data))
    assert all(count > 0 for count in agreed.values()), agreed
