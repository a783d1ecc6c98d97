"""TEST INFRASTRUCTURE ONLY: the reference's packed model state in numpy.

A restatement of the ``RTNF4S1`` byte format that carries every packed NF4
Linear weight of a model in a checkpoint:

  writer  packed_model_state_bytes   src/c_api/model_state.cpp:34-113
  reader  parse_packed_model_state   src/c_api/model_state.cpp:166-300

Layout (all integers and floats little-endian):

  8 bytes   magic  'R' 'T' 'N' 'F' '4' 'S' '1' NUL
  u64       weight count (>= 1)
  per weight
    u64  rank (must be 2)         u64  block size
    u64  packed code bytes        u64  fp32 block scale count
    u64  scale code count         u64  second-level scale count
    u64  second-level block size  f32  offset       u32  flags (1 = nested)
    u64  x rank   dimensions
    u8   x packed code bytes
    f32  x block scale count
    u8   x scale code count       (nested only)
    f32  x second-level count     (nested only)

``parse`` raises what the reader throws, with its messages: ``ValueError`` for
std::invalid_argument, ``OverflowError`` for std::overflow_error.  The reader
checks the container only; whether a payload is a valid NF4 weight is decided
later by QuantizedWeight::from_packed_nf4 (``Oracle.validate_payload``).

Pinned against the reference's own reader compiled from model_state.cpp
(``oracle/_ref/libstateref.so``, tests/test_oracle_vs_reference.py), whose
acceptance of ``serialize``'s output with identical fields also pins the writer,
and against the committed fixture tests/golden/packed_state.bin.
"""
from __future__ import annotations

import ctypes
import dataclasses
import os
import struct
from typing import List, Optional, Sequence

import numpy as np

MAGIC = b"RTNF4S1\x00"
_SIZE_MAX = (1 << 64) - 1
_MINIMUM_ENTRY_BYTES = 80


@dataclasses.dataclass
class PackedWeightState:
    """PackedLinearWeightState
    (include/riftco_transformer/model/decoder_only_transformer.hpp) with the
    payload arrays as numpy."""

    shape: List[int]
    block_size: int
    packed_codes: np.ndarray                    # uint8
    block_scales: np.ndarray                    # float32, empty when nested
    double_quantized: bool = False
    scale_codes: Optional[np.ndarray] = None    # uint8
    second_level_scales: Optional[np.ndarray] = None   # float32
    scale_block_size: int = 0
    offset: float = 0.0


def serialize(weights: Sequence[PackedWeightState]) -> bytes:
    """packed_model_state_bytes, src/c_api/model_state.cpp:34-113."""
    out = bytearray(MAGIC)
    out += struct.pack("<Q", len(weights))
    for weight in weights:
        nested = weight.double_quantized
        codes = np.ascontiguousarray(weight.packed_codes, dtype=np.uint8)
        block_scales = np.ascontiguousarray(weight.block_scales,
                                            dtype="<f4")
        scale_codes = (np.ascontiguousarray(weight.scale_codes, dtype=np.uint8)
                       if nested else np.zeros(0, np.uint8))
        second = (np.ascontiguousarray(weight.second_level_scales, dtype="<f4")
                  if nested else np.zeros(0, "<f4"))
        out += struct.pack(
            "<7Q", len(weight.shape), weight.block_size, codes.size,
            block_scales.size, scale_codes.size, second.size,
            weight.scale_block_size if nested else 0)
        out += np.float32(weight.offset if nested else 0.0).tobytes()
        out += struct.pack("<I", 1 if nested else 0)
        for dimension in weight.shape:
            out += struct.pack("<Q", dimension)
        out += codes.tobytes()
        out += block_scales.tobytes()
        if nested:
            out += scale_codes.tobytes()
            out += second.tobytes()
    return bytes(out)


class _Reader:
    """PackedModelStateReader, src/c_api/model_state.cpp:115-164."""

    def __init__(self, data: bytes):
        self._view = memoryview(data)
        self._position = 0

    def remaining(self) -> int:
        return len(self._view) - self._position

    def take(self, count: int, description: str) -> memoryview:
        if count > self.remaining():
            raise ValueError("truncated packed model state: " + description)
        result = self._view[self._position:self._position + count]
        self._position += count
        return result

    def u32(self, description: str) -> int:
        return struct.unpack("<I", self.take(4, description))[0]

    def u64(self, description: str) -> int:
        return struct.unpack("<Q", self.take(8, description))[0]


def parse(data: bytes) -> List[PackedWeightState]:
    """parse_packed_model_state, src/c_api/model_state.cpp:166-300."""
    reader = _Reader(data)
    if bytes(reader.take(len(MAGIC), "magic")) != MAGIC:
        raise ValueError("unknown packed model state format")
    count = reader.u64("weight count")
    if count == 0 or count > reader.remaining() // _MINIMUM_ENTRY_BYTES:
        raise ValueError(
            "packed model state weight count is inconsistent with its size")
    result = []
    for _ in range(count):
        rank = reader.u64("rank")
        if rank != 2:
            raise ValueError("packed decoder Linear weights must have rank two")
        block_size = reader.u64("block size")
        packed_count = reader.u64("packed code count")
        block_scale_count = reader.u64("block scale count")
        scale_code_count = reader.u64("scale code count")
        second_scale_count = reader.u64("second-level scale count")
        scale_block_size = reader.u64("scale block size")
        offset_bits = reader.u32("scale offset")
        flags = reader.u32("flags")
        if flags > 1:
            raise ValueError("packed model state has unknown flags")
        nested = flags == 1
        if ((not nested and (scale_code_count != 0 or second_scale_count != 0
                             or scale_block_size != 0 or offset_bits != 0))
                or (nested and (block_scale_count != 0
                                or scale_block_size == 0))):
            raise ValueError(
                "packed model state has inconsistent NF4 scale metadata")
        required = rank * 8
        for value, element_size in ((packed_count, 1), (block_scale_count, 4),
                                    (scale_code_count, 1),
                                    (second_scale_count, 4)):
            if value > (_SIZE_MAX - required) // element_size:
                raise OverflowError(
                    "packed model state entry size exceeds addressable memory")
            required += value * element_size
        if required > reader.remaining():
            raise ValueError("truncated packed model state: weight payload")
        shape = [reader.u64("dimension") for _ in range(rank)]
        codes = np.frombuffer(reader.take(packed_count, "packed codes"),
                              dtype=np.uint8).copy()
        block_scales = np.frombuffer(
            reader.take(4 * block_scale_count, "block scale"),
            dtype="<f4").astype(np.float32)
        weight = PackedWeightState(shape, block_size, codes, block_scales)
        if nested:
            weight.double_quantized = True
            weight.scale_codes = np.frombuffer(
                reader.take(scale_code_count, "scale codes"),
                dtype=np.uint8).copy()
            weight.second_level_scales = np.frombuffer(
                reader.take(4 * second_scale_count, "second-level scale"),
                dtype="<f4").astype(np.float32)
            weight.scale_block_size = scale_block_size
            weight.offset = float(
                np.frombuffer(struct.pack("<I", offset_bits), "<f4")[0])
        result.append(weight)
    if reader.remaining() != 0:
        raise ValueError("packed model state contains trailing bytes")
    return result


def from_nf4_weight(weight) -> PackedWeightState:
    """An ``oracle.binding.Nf4Weight`` as one entry of the packed state."""
    nested = weight.encoding == 1
    return PackedWeightState(
        shape=[weight.output_width, weight.input_width],
        block_size=weight.block_size,
        packed_codes=weight.codes,
        block_scales=(np.zeros(0, np.float32) if nested
                      else weight.fp32_scales),
        double_quantized=nested,
        scale_codes=weight.scale_codes if nested else None,
        second_level_scales=weight.second_level if nested else None,
        scale_block_size=weight.second_level_block if nested else 0,
        offset=float(weight.offset) if nested else 0.0,
    )


class ReferenceReader:
    """The reference's own parse_packed_model_state, compiled from its source
    into ``oracle/_ref/libstateref.so`` (present only where that build was
    made).  ``parse`` has the contract of the module-level ``parse``."""

    LIBRARY = os.path.join(os.path.dirname(os.path.abspath(__file__)),
                           "_ref", "libstateref.so")

    @classmethod
    def available(cls) -> bool:
        return os.path.exists(cls.LIBRARY)

    def __init__(self):
        lib = ctypes.CDLL(self.LIBRARY)
        lib.stateref_parse.restype = ctypes.c_int
        lib.stateref_parse.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
        lib.stateref_message.restype = ctypes.c_char_p
        lib.stateref_weight_count.restype = ctypes.c_size_t
        lib.stateref_weight_header.restype = ctypes.c_int
        lib.stateref_weight_header.argtypes = [
            ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p]
        lib.stateref_weight_payload.restype = ctypes.c_int
        lib.stateref_weight_payload.argtypes = [
            ctypes.c_size_t] + [ctypes.c_void_p] * 4
        self._lib = lib

    def parse(self, data: bytes) -> List[PackedWeightState]:
        buffer = np.frombuffer(data, dtype=np.uint8)
        pointer = buffer.ctypes.data if buffer.size else None
        status = self._lib.stateref_parse(pointer, buffer.size)
        if status != 0:
            message = self._lib.stateref_message().decode()
            raise {1: ValueError, 3: OverflowError}.get(
                status, RuntimeError)(message)
        result = []
        for index in range(self._lib.stateref_weight_count()):
            header = np.zeros(9, np.uint64)
            offset_bits = np.zeros(1, np.uint32)
            assert self._lib.stateref_weight_header(
                index, header.ctypes.data, offset_bits.ctypes.data) == 0
            (rows, columns, block_size, code_bytes, block_scales, scale_codes,
             second, scale_block_size, nested) = (int(v) for v in header)
            arrays = (np.zeros(code_bytes, np.uint8),
                      np.zeros(block_scales, np.float32),
                      np.zeros(scale_codes, np.uint8),
                      np.zeros(second, np.float32))
            assert self._lib.stateref_weight_payload(
                index, *(a.ctypes.data if a.size else None
                         for a in arrays)) == 0
            weight = PackedWeightState([rows, columns], block_size, arrays[0],
                                       arrays[1])
            if nested:
                weight.double_quantized = True
                weight.scale_codes = arrays[2]
                weight.second_level_scales = arrays[3]
                weight.scale_block_size = scale_block_size
                weight.offset = float(offset_bits.view(np.float32)[0])
            result.append(weight)
        return result
