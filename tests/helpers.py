"""Test helpers: deterministic inputs, the reference tests' closed-form
fixtures restated as numpy generators, and the error measures of the parity
bar."""
from __future__ import annotations

import hashlib

import numpy as np

# The seven Llama-7B projection shapes (output_width, input_width).
LLAMA_SHAPES = {
    "q_proj": (4096, 4096),
    "k_proj": (4096, 4096),
    "v_proj": (4096, 4096),
    "o_proj": (4096, 4096),
    "gate_proj": (11008, 4096),
    "up_proj": (11008, 4096),
    "down_proj": (4096, 11008),
}


def normal(seed: int, shape, sigma: float) -> np.ndarray:
    """N(0, sigma) fp32 values from numpy's PCG64 stream `seed`."""
    rng = np.random.default_rng(seed)
    return (rng.standard_normal(shape, dtype=np.float32) *
            np.float32(sigma)).astype(np.float32)


def bits(array: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(array, dtype=np.float32).view(np.uint32)


def sha256(array: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(array).tobytes()).hexdigest()


def assert_bit_equal(actual, expected, what: str = "") -> None:
    a, e = bits(actual), bits(expected)
    assert a.shape == e.shape, f"{what}: shape {a.shape} != {e.shape}"
    if not np.array_equal(a, e):
        bad = np.flatnonzero(a.ravel() != e.ravel())
        index = int(bad[0])
        raise AssertionError(
            f"{what}: {bad.size} of {a.size} values differ bitwise; first at "
            f"flat index {index}: {np.ravel(actual)[index]!r} != "
            f"{np.ravel(expected)[index]!r}")


# ---- closed-form fixtures ------------------------------------------------
# Integer-formula tensors of the reference's backend parity test
# (tests/core/backend/test_quantized_linear_backend.cpp:89-169).

def aligned_weight() -> np.ndarray:  # :89-100
    index = np.arange(3 * 32)
    values = ((index % 19) - 9).astype(np.float32) * np.float32(0.1375)
    values[0] = -2.0
    values[31] = 1.75
    values[32] = 3.0
    values[-1] = -4.0
    return values.reshape(3, 32)


def aligned_input() -> np.ndarray:  # :102-109
    index = np.arange(2 * 32)
    return (((index % 11) - 5).astype(np.float32) *
            np.float32(0.2)).reshape(2, 32)


def aligned_upstream() -> np.ndarray:  # :111-124
    return np.array([[0.25, -0.75, 1.5], [-1.0, 0.5, 0.125]],
                    dtype=np.float32)


EDGE = 33


def edge_weight() -> np.ndarray:  # :126-142
    index = np.arange(EDGE * EDGE)
    values = ((index % 37) - 18).astype(np.float32) * np.float32(0.0625)
    values[0] = -3.0
    values[31] = 2.5
    values[32] = -2.75
    values[1023] = 4.0
    values[1024] = -4.5
    values[-1] = 5.0
    return values.reshape(EDGE, EDGE)


def edge_input() -> np.ndarray:  # :144-155
    index = np.arange(2 * EDGE)
    return (((index % 17) - 8).astype(np.float32) *
            np.float32(0.125)).reshape(2, EDGE)


def edge_upstream() -> np.ndarray:  # :157-168
    index = np.arange(2 * EDGE)
    return (((index % 13) - 6).astype(np.float32) *
            np.float32(0.075)).reshape(2, EDGE)


# ---- error measures ------------------------------------------------------

def reference_close(actual, expected, tolerance: float = 3.0e-5) -> bool:
    """The reference's own check: |a-e| <= tol * max(1, |a|, |e|)
    (tests/core/backend/test_quantized_linear_backend.cpp:46-70)."""
    actual = np.asarray(actual, dtype=np.float32)
    expected = np.asarray(expected, dtype=np.float32)
    scale = np.maximum(1.0, np.maximum(np.abs(actual), np.abs(expected)))
    return bool(np.all(np.isfinite(actual)) and
                np.all(np.abs(actual - expected) <= tolerance * scale))


def rms(values) -> float:
    values = np.asarray(values, dtype=np.float64)
    return float(np.sqrt(np.mean(values * values)))


def normalized_error(actual, expected, contraction: int, activation_rms: float,
                     weight_rms: float) -> float:
    """max |a - e| / (sqrt(K) * rms(activations) * rms(deq W)): the error in
    units of one standard deviation of an output."""
    difference = np.abs(np.asarray(actual, dtype=np.float64) -
                        np.asarray(expected, dtype=np.float64)).max()
    return float(difference /
                 (np.sqrt(contraction) * activation_rms * weight_rms))


def exact_forward(x, dense) -> np.ndarray:
    """fp64-accumulated x . dense^T."""
    return np.asarray(x, np.float64) @ np.asarray(dense, np.float64).T


def exact_input_backward(dy, dense) -> np.ndarray:
    """fp64-accumulated dy . dense."""
    return np.asarray(dy, np.float64) @ np.asarray(dense, np.float64)


# ---- packed model state (src/c_api/model_state.cpp under /root/reference) --

def packed_state_mutations(blob: bytes):
    """(name, bytes) pairs: malformed variants of a valid packed model state
    whose first entry uses fp32 block scales and whose second is nested.
    Offsets follow the entry header: rank 0, block size 8, packed codes 16,
    block scales 24, scale codes 32, second-level scales 40, second-level
    block size 48, offset 56, flags 60, dimensions 64."""
    import struct

    def patched(position, fmt, value):
        data = bytearray(blob)
        struct.pack_into(fmt, data, position, value)
        return bytes(data)

    first = 16
    # the second entry starts after the first one's header, dimensions and
    # payload
    packed, scales = struct.unpack_from("<2Q", blob, first + 16)
    second = first + 64 + 16 + packed + 4 * scales
    big = (1 << 64) - 1
    cases = [("intact", blob)]
    for cut in (0, 4, 7, 8, 12, 15, 16, 20, 50, 79, 80, 95, 96, second - 1,
                second, second + 30, second + 80, len(blob) - 1):
        cases.append((f"cut_{cut}", blob[:cut]))
    cases += [
        ("magic", b"RTNF4S2\x00" + blob[8:]),
        ("count_zero", patched(8, "<Q", 0)),
        ("count_huge", patched(8, "<Q", big)),
        ("count_more", patched(8, "<Q", 4)),
        ("count_fewer", patched(8, "<Q", 1)),
        ("rank_three", patched(first, "<Q", 3)),
        ("rank_zero", patched(first, "<Q", 0)),
        ("flags_two", patched(first + 60, "<I", 2)),
        ("flags_flipped_first", patched(first + 60, "<I", 1)),
        ("flags_flipped_second", patched(second + 60, "<I", 0)),
        ("fp32_with_scale_codes", patched(first + 32, "<Q", 1)),
        ("fp32_with_second_level", patched(first + 40, "<Q", 1)),
        ("fp32_with_scale_block", patched(first + 48, "<Q", 32)),
        ("fp32_with_offset", patched(first + 56, "<I", 1)),
        ("nested_with_block_scales", patched(second + 24, "<Q", 1)),
        ("nested_without_scale_block", patched(second + 48, "<Q", 0)),
        ("packed_overflow", patched(first + 16, "<Q", big)),
        ("scales_overflow", patched(first + 24, "<Q", 1 << 62)),
        ("second_level_overflow", patched(second + 40, "<Q", 1 << 62)),
        ("packed_too_long", patched(first + 16, "<Q", 1 << 40)),
        ("packed_one_more", patched(first + 16, "<Q", packed + 1)),
        ("packed_one_fewer", patched(first + 16, "<Q", packed - 1)),
        ("trailing", blob + b"\x00"),
        ("block_size_unchecked", patched(first + 8, "<Q", 7)),
    ]
    return cases


def scale_storage_cases():
    """(name, scale storage, expected scale count) triples for the
    dispatcher's scale-storage check
    (src/core/backend/nn/quantized_linear/dispatch.cpp:108-154): sound
    storages of both encodings and, for every condition the check names, a
    storage that breaks it alone -- and a few that break two, which pins the
    order of the checks."""
    from oracle.binding import (SCALE_DOUBLE_QUANTIZED_UINT8, SCALE_FLOAT32,
                                Nf4Weight)
    f32 = np.float32
    big = float(np.finfo(np.float32).max)

    def storage(encoding, fp32=None, codes=None, second=None, block=0,
                offset=0.0):
        return Nf4Weight(
            1, 1, 32, np.array([0x07], np.uint8), encoding,
            fp32_scales=None if fp32 is None else np.array(fp32, f32),
            scale_codes=None if codes is None else np.array(codes, np.uint8),
            second_level=None if second is None else np.array(second, f32),
            second_level_block=block, offset=offset)

    def legacy(scales, **more):
        return storage(SCALE_FLOAT32, fp32=scales, **more)

    def nested(codes, second, block=32, offset=0.5, **more):
        return storage(SCALE_DOUBLE_QUANTIZED_UINT8, codes=codes,
                       second=second, block=block, offset=offset, **more)

    many = list(range(70))
    return [
        ("legacy ok", legacy([0.0, 1.5, big]), 3),
        ("legacy one", legacy([2.0]), 1),
        ("legacy too few", legacy([1.0, 2.0]), 3),
        ("legacy too many", legacy([1.0, 2.0, 3.0]), 2),
        ("legacy with scale codes", legacy([1.0], codes=[128]), 1),
        ("legacy with second level", legacy([1.0], second=[1.0]), 1),
        ("legacy with block size", legacy([1.0], block=32), 1),
        ("legacy with offset", legacy([1.0], offset=0.25), 1),
        ("legacy negative zero offset", legacy([1.0], offset=-0.0), 1),
        ("legacy negative", legacy([1.0, -1.0e-30]), 2),
        ("legacy negative zero", legacy([1.0, -0.0]), 2),
        ("legacy infinite", legacy([np.inf, 1.0]), 2),
        ("legacy nan", legacy([1.0, np.nan]), 2),
        ("legacy too few and negative", legacy([-1.0]), 2),
        ("nested ok", nested([0, 128, 255], [1.0]), 3),
        ("nested two groups", nested(many, [1.0, 2.0, 0.0]), 70),
        ("nested block 64", nested(many, [1.0, 0.5], block=64), 70),
        ("nested with fp32", nested([128], [1.0], fp32=[1.0]), 1),
        ("nested too few codes", nested([128, 128], [1.0]), 3),
        ("nested too many codes", nested([128, 128, 128], [1.0]), 2),
        ("nested zero block", nested([128], [1.0], block=0), 1),
        ("nested block 16", nested([128], [1.0], block=16), 1),
        ("nested block 48", nested([128], [1.0], block=48), 1),
        ("nested block 8192", nested([128], [1.0], block=8192), 1),
        ("nested infinite offset", nested([128], [1.0], offset=np.inf), 1),
        ("nested nan offset", nested([128], [1.0], offset=np.nan), 1),
        ("nested negative offset", nested([128], [1.0], offset=-0.5), 1),
        ("nested negative zero offset", nested([128], [1.0], offset=-0.0), 1),
        ("nested too few groups", nested(many, [1.0, 2.0]), 70),
        ("nested too many groups", nested(many, [1.0, 2.0, 3.0, 4.0]), 70),
        ("nested no groups", nested([128], []), 1),
        ("nested negative second level", nested([128], [-1.0]), 1),
        ("nested infinite second level", nested([128], [np.inf]), 1),
        ("nested nan second level", nested(many, [1.0, np.nan, 1.0]), 70),
        ("nested saturating sum", nested([255], [big], offset=big), 1),
        ("nested clamped below", nested([1], [big], offset=1.0), 1),
        ("nested overflowing product",
         nested([255, 1], [big], offset=0.0), 2),
        ("nested bad block and bad count",
         nested(many, [1.0], block=16), 70),
        ("nested bad count and negative second level",
         nested(many, [-1.0], block=32), 70),
        ("unknown encoding", storage(2, fp32=[1.0]), 1),
    ]


def verdict(function, *arguments):
    """("ok", "") or (exception type name, message) of one call."""
    try:
        function(*arguments)
    except (ValueError, OverflowError, RuntimeError, TypeError) as error:
        return [type(error).__name__, str(error)]
    return ["ok", ""]


# ---- one training step through a Linear with a packed weight and an adapter --

# name: (rows, input_width, output_width, rank, alpha, block size, second-level
#        block size or 0 for fp32 scales, with bias)
LORA_STEP_CASES = {
    "rank3_fp32": (5, 128, 24, 3, 8.0, 64, 0, False),
    "rank4_nested_bias": (3, 256, 40, 4, 16.0, 32, 32, True),
    "one_row_rank1": (1, 64, 8, 1, 2.0, 64, 0, True),
    "odd_widths_nested": (7, 192, 33, 5, 8.0, 64, 256, False),
    "rank16": (9, 512, 48, 16, 32.0, 64, 0, False),
}


def lora_step_inputs(name: str) -> dict:
    """Seeded inputs of LORA_STEP_CASES[name]."""
    rows, in_w, out_w, rank, alpha, block, second, with_bias = \
        LORA_STEP_CASES[name]
    seed = 500 + 10 * sorted(LORA_STEP_CASES).index(name)
    return {
        "dense": normal(seed, (out_w, in_w), 0.02),
        "x": normal(seed + 1, (rows, in_w), 1.0),
        "dy": normal(seed + 2, (rows, out_w), 1.0e-2),
        "lora_a": normal(seed + 3, (rank, in_w), 0.05),
        "lora_b": normal(seed + 4, (out_w, rank), 0.05),
        "bias": normal(seed + 5, (out_w,), 0.01) if with_bias else None,
        "alpha": alpha, "rank": rank, "block": block, "second": second,
        # LowRankAdapter's scale: alpha / float(rank), one rounded division
        "scale": float(np.float32(alpha) / np.float32(rank)),
    }
