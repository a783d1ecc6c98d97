"""ctypes binding of the kernel C ABI (include/rthip.h -> lib/librthip.so).

This is plumbing for tests and measurement: PyTorch supplies device memory and
the current HIP stream, every computation goes through the C ABI.  There is no
fallback of any kind -- a missing library, a missing symbol or a failing call
raises.
"""
from __future__ import annotations

import ctypes
import dataclasses
import os
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(_HERE, "lib", "librthip.so")

OK = 0
INVALID_ARGUMENT = 1
UNAVAILABLE = 2
OUT_OF_MEMORY = 3
RUNTIME_ERROR = 4
UNSUPPORTED = 5
OVERFLOW = 6

SCALE_FLOAT32 = 0
SCALE_DOUBLE_QUANTIZED_UINT8 = 1

ALGORITHM_AUTO = 0
ALGORITHM_GENERIC = 1
ALGORITHM_GEMV = 2
ALGORITHM_MFMA = 3
ALGORITHM_SKINNY = 4
ALGORITHM_RESIDENT = 5
ALGORITHM_NAMES = {0: "auto", 1: "generic", 2: "gemv", 3: "mfma",
                   4: "skinny", 5: "resident"}

FORWARD = 0
INPUT_BACKWARD = 1


class RthipError(RuntimeError):
    """A C-ABI call returned a non-zero status."""

    def __init__(self, status: int, message: str):
        super().__init__(f"rthip status {status}: {message}")
        self.status = status
        self.message = message


class InvalidArgument(RthipError, ValueError):
    pass


class Unavailable(RthipError):
    pass


class Unsupported(RthipError):
    pass


class Overflow(RthipError, OverflowError):
    pass


_ERRORS = {
    INVALID_ARGUMENT: InvalidArgument,
    UNAVAILABLE: Unavailable,
    OUT_OF_MEMORY: RthipError,
    RUNTIME_ERROR: RthipError,
    UNSUPPORTED: Unsupported,
    OVERFLOW: Overflow,
}

_u64 = ctypes.c_uint64
_i32 = ctypes.c_int32
_f32 = ctypes.c_float
_ptr = ctypes.c_void_p
_size = ctypes.c_size_t

# The six values that describe a packed weight, in ABI order.
_WEIGHT = [_ptr, _ptr, _ptr, _i32, _u64, _f32]



class Member(ctypes.Structure):
    """rthip_nf4_member: one weight of a group that shares its input."""

    _fields_ = [("codes", _ptr), ("primary_scales", _ptr),
                ("secondary_scales", _ptr), ("offset", _f32),
                ("bias_or_null", _ptr), ("y", _ptr), ("output_width", _u64)]


class LoraMember(ctypes.Structure):
    """rthip_nf4_lora_member: a member with an optional adapter term."""

    _fields_ = [("base", Member), ("lora_a", _ptr), ("lora_b", _ptr),
                ("reduced", _ptr), ("lora_rank", _u64), ("lora_scale", _f32)]


_PROTOTYPES = {
    "rthip_abi_version": (ctypes.c_uint32, []),
    "rthip_last_error": (ctypes.c_char_p, []),
    "rthip_device_count": (_i32, [ctypes.POINTER(_i32)]),
    "rthip_device_description": (_i32, [ctypes.c_char_p, _size]),
    "rthip_device_memory_host_visible": (_i32, [ctypes.POINTER(_i32)]),
    "rthip_malloc": (_i32, [ctypes.POINTER(_ptr), _size]),
    "rthip_free": (_i32, [_ptr]),
    "rthip_copy_to_device": (_i32, [_ptr, _ptr, _size]),
    "rthip_copy_to_host": (_i32, [_ptr, _ptr, _size]),
    "rthip_fill_f32": (_i32, [_ptr, _f32, _u64, _ptr]),
    "rthip_stream_synchronize": (_i32, [_ptr]),
    "rthip_nf4_linear_forward": (
        _i32, [_ptr] + _WEIGHT + [_ptr, _ptr, _u64, _u64, _u64, _u64, _ptr]),
    "rthip_nf4_linear_input_backward": (
        _i32, [_ptr] + _WEIGHT + [_ptr, _u64, _u64, _u64, _u64, _ptr]),
    "rthip_nf4_linear_input_backward_no_alloc": (
        _i32, [_ptr] + _WEIGHT + [_ptr, _u64, _u64, _u64, _u64, _ptr]),
    "rthip_release_workspaces": (_i32, [_ptr, _i32]),
    "rthip_nf4_linear_forward_with": (
        _i32,
        [_i32, _ptr] + _WEIGHT + [_ptr, _ptr, _u64, _u64, _u64, _u64, _ptr]),
    "rthip_nf4_linear_input_backward_with": (
        _i32, [_i32, _ptr] + _WEIGHT + [_ptr, _u64, _u64, _u64, _u64, _ptr]),
    "rthip_nf4_linear_forward_group": (
        _i32, [_ptr, ctypes.POINTER(Member), _u64, _i32, _u64, _u64, _u64,
               _u64, _ptr]),
    "rthip_nf4_lora_linear_forward_group": (
        _i32, [_ptr, ctypes.POINTER(LoraMember), _u64, _i32, _u64, _u64, _u64,
               _u64, _ptr]),
    "rthip_matmul": (
        _i32, [_ptr, _ptr, _ptr, _u64, _u64, _u64, _u64, _ptr]),
    "rthip_lora_reduce": (_i32, [_ptr, _ptr, _ptr, _u64, _u64, _u64, _ptr]),
    "rthip_nf4_lora_linear_forward": (
        _i32,
        [_ptr] + _WEIGHT + [_ptr, _ptr, _ptr, _u64, _f32, _ptr, _ptr, _u64,
                            _u64, _u64, _u64, _ptr]),
    "rthip_nf4_lora_linear_forward_with": (
        _i32,
        [_i32, _ptr] + _WEIGHT + [_ptr, _ptr, _ptr, _u64, _f32, _ptr, _ptr,
                                  _u64, _u64, _u64, _u64, _ptr]),
    "rthip_lora_backward": (
        _i32, [_ptr, _ptr, _ptr, _ptr, _u64, _f32, _ptr, _ptr, _ptr, _u64,
               _u64, _u64, _ptr]),
    "rthip_nf4_lora_linear_input_backward": (
        _i32, [_ptr] + _WEIGHT + [_ptr, _ptr, _u64, _ptr, _u64, _u64, _u64,
                                  _u64, _ptr]),
    "rthip_nf4_lora_linear_input_backward_with": (
        _i32, [_i32, _ptr] + _WEIGHT + [_ptr, _ptr, _u64, _ptr, _u64, _u64,
                                        _u64, _u64, _ptr]),
    "rthip_nf4_select_algorithm": (
        _i32, [_i32, _u64, _u64, _u64, _u64, ctypes.POINTER(_i32)]),
    "rthip_nf4_forward_kernel_name": (
        _i32, [_u64, _u64, ctypes.POINTER(_u64), _u64, _u64, _i32, _u64,
               ctypes.c_char_p, _u64]),
    "rthip_nf4_dequantize": (_i32, _WEIGHT + [_ptr, _u64, _u64, _ptr]),
    "rthip_nf4_quantize": (
        _i32, [_ptr, _u64, _u64, _i32, _u64, _ptr, _ptr, _ptr, _ptr,
               ctypes.POINTER(_f32), _ptr]),
    "rthip_nf4_check_payload": (_i32, _WEIGHT + [_u64, _u64, _ptr]),
}

EXPORTED_SYMBOLS = tuple(_PROTOTYPES)


@dataclasses.dataclass
class DeviceWeight:
    """A packed NF4 weight whose payload lives in device memory.

    The tensors are kept alive here; the ABI only ever sees their addresses.
    """

    output_width: int
    input_width: int
    block_size: int
    encoding: int
    codes: object                      # torch.uint8 [ceil(O*I/2)]
    primary_scales: object             # torch.float32 or torch.uint8 [blocks]
    secondary_scales: Optional[object]  # torch.float32 [groups] or None
    second_level_block: int = 0
    offset: float = 0.0

    def abi_arguments(self):
        secondary = (None if self.secondary_scales is None
                     else self.secondary_scales.data_ptr())
        return [self.codes.data_ptr(), self.primary_scales.data_ptr(),
                secondary, self.encoding, self.second_level_block,
                self.offset]

    @property
    def payload_bytes(self) -> int:
        total = self.codes.numel() + (
            self.primary_scales.numel() * self.primary_scales.element_size())
        if self.secondary_scales is not None:
            total += self.secondary_scales.numel() * 4 + 4
        return total


class Library:
    """librthip.so with typed entry points."""

    def __init__(self, path: str = LIBRARY_PATH):
        if not os.path.exists(path):
            raise FileNotFoundError(
                f"{path} is missing: build it with "
                "`make -C riftco-transformer_amd` (or __graft_entry__.build())")
        self.path = path
        # PyTorch wheels bundle their own HIP runtime under the same SONAME.
        # Loading torch first makes this library bind to that one runtime, so
        # that torch's device pointers and streams are valid here; without
        # torch the system runtime is used.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        self._lib = ctypes.CDLL(path)
        for name, (restype, argtypes) in _PROTOTYPES.items():
            function = getattr(self._lib, name)  # AttributeError if absent
            function.restype = restype
            function.argtypes = argtypes

    # -- helpers ---------------------------------------------------------
    def last_error(self) -> str:
        return (self._lib.rthip_last_error() or b"").decode()

    def _check(self, status: int) -> None:
        if status != OK:
            raise _ERRORS.get(status, RthipError)(status, self.last_error())

    # -- library / device -------------------------------------------------
    def abi_version(self):
        value = self._lib.rthip_abi_version()
        return value >> 16, value & 0xFFFF

    def device_count(self) -> int:
        count = _i32(0)
        self._check(self._lib.rthip_device_count(ctypes.byref(count)))
        return count.value

    def is_available(self) -> bool:
        count = _i32(0)
        return self._lib.rthip_device_count(ctypes.byref(count)) == OK

    def device_description(self) -> str:
        buffer = ctypes.create_string_buffer(256)
        self._check(self._lib.rthip_device_description(buffer, 256))
        return buffer.value.decode()

    def device_memory_host_visible(self) -> bool:
        visible = _i32(0)
        self._check(self._lib.rthip_device_memory_host_visible(
            ctypes.byref(visible)))
        return bool(visible.value)

    # -- memory ------------------------------------------------------------
    def malloc(self, size: int) -> int:
        pointer = _ptr()
        self._check(self._lib.rthip_malloc(ctypes.byref(pointer), size))
        return pointer.value or 0

    def free(self, pointer: int) -> None:
        self._check(self._lib.rthip_free(pointer))

    def copy_to_device(self, device: int, host: int, size: int) -> None:
        self._check(self._lib.rthip_copy_to_device(device, host, size))

    def copy_to_host(self, host: int, device: int, size: int) -> None:
        self._check(self._lib.rthip_copy_to_host(host, device, size))

    def fill_f32(self, device: int, value: float, count: int,
                 stream: int = 0) -> None:
        self._check(self._lib.rthip_fill_f32(device, value, count, stream))

    def synchronize(self, stream: int = 0) -> None:
        self._check(self._lib.rthip_stream_synchronize(stream))

    # -- the hot path --------------------------------------------------------
    def select_algorithm(self, direction: int, rows: int, input_width: int,
                         output_width: int, block_size: int) -> int:
        algorithm = _i32(0)
        self._check(self._lib.rthip_nf4_select_algorithm(
            direction, rows, input_width, output_width, block_size,
            ctypes.byref(algorithm)))
        return algorithm.value

    def forward_kernel_name(self, rows: int, input_width: int, output_widths,
                            block_size: int, encoding: int,
                            second_level_block: int = 0) -> str:
        """The one-row decode kernel instance a forward of these weights
        launches, as a profiler prints it ("" where another family serves
        the call)."""
        widths = (_u64 * len(output_widths))(*output_widths)
        name = ctypes.create_string_buffer(160)
        self._check(self._lib.rthip_nf4_forward_kernel_name(
            rows, input_width, widths, len(output_widths), block_size,
            encoding, second_level_block, name, len(name)))
        return name.value.decode()

    def linear_forward(self, x_ptr: int, weight: DeviceWeight,
                       bias_ptr: Optional[int], y_ptr: int, rows: int,
                       stream: int = 0,
                       algorithm: Optional[int] = None) -> None:
        tail = [bias_ptr, y_ptr, rows, weight.input_width,
                weight.output_width, weight.block_size, stream]
        if algorithm is None:
            status = self._lib.rthip_nf4_linear_forward(
                x_ptr, *weight.abi_arguments(), *tail)
        else:
            status = self._lib.rthip_nf4_linear_forward_with(
                algorithm, x_ptr, *weight.abi_arguments(), *tail)
        self._check(status)

    def linear_forward_group(self, x_ptr: int, members, rows: int,
                             stream: int = 0) -> None:
        """members: (weight, bias_ptr or None, y_ptr) triples whose weights
        share input width, block size and scale encoding."""
        first = members[0][0]
        array = (Member * len(members))()
        for slot, (weight, bias_ptr, y_ptr) in zip(array, members):
            if (weight.input_width, weight.block_size, weight.encoding,
                    weight.second_level_block) != (
                    first.input_width, first.block_size, first.encoding,
                    first.second_level_block):
                raise ValueError("the weights of a group must share input "
                                 "width, block size and scale encoding")
            slot.codes = weight.codes.data_ptr()
            slot.primary_scales = weight.primary_scales.data_ptr()
            slot.secondary_scales = (
                None if weight.secondary_scales is None
                else weight.secondary_scales.data_ptr())
            slot.offset = weight.offset
            slot.bias_or_null = bias_ptr
            slot.y = y_ptr
            slot.output_width = weight.output_width
        self._check(self._lib.rthip_nf4_linear_forward_group(
            x_ptr, array, len(members), first.encoding,
            first.second_level_block, rows, first.input_width,
            first.block_size, stream))

    def lora_linear_forward_group(self, x_ptr: int, members, rows: int,
                                  stream: int = 0) -> None:
        """members: (weight, bias_ptr or None, y_ptr, adapter) where adapter is
        None or (lora_a_ptr or None, lora_b_ptr, reduced_ptr, rank, scale);
        with lora_a None, `reduced` already holds x.A^T."""
        first = members[0][0]
        array = (LoraMember * len(members))()
        for slot, (weight, bias_ptr, y_ptr, adapter) in zip(array, members):
            if (weight.input_width, weight.block_size, weight.encoding,
                    weight.second_level_block) != (
                    first.input_width, first.block_size, first.encoding,
                    first.second_level_block):
                raise ValueError("the weights of a group must share input "
                                 "width, block size and scale encoding")
            slot.base.codes = weight.codes.data_ptr()
            slot.base.primary_scales = weight.primary_scales.data_ptr()
            slot.base.secondary_scales = (
                None if weight.secondary_scales is None
                else weight.secondary_scales.data_ptr())
            slot.base.offset = weight.offset
            slot.base.bias_or_null = bias_ptr
            slot.base.y = y_ptr
            slot.base.output_width = weight.output_width
            if adapter is not None:
                (slot.lora_a, slot.lora_b, slot.reduced, slot.lora_rank,
                 slot.lora_scale) = adapter
        self._check(self._lib.rthip_nf4_lora_linear_forward_group(
            x_ptr, array, len(members), first.encoding,
            first.second_level_block, rows, first.input_width,
            first.block_size, stream))

    def matmul(self, left_ptr: int, right_ptr: int, out_ptr: int,
               batch_count: int, rows: int, shared: int, columns: int,
               stream: int = 0) -> None:
        self._check(self._lib.rthip_matmul(
            left_ptr, right_ptr, out_ptr, batch_count, rows, shared, columns,
            stream))

    def quantize(self, values_ptr: int, element_count: int, block_size: int,
                 encoding: int, second_level_block: int, codes_ptr: int,
                 primary_ptr: int, secondary_ptr: Optional[int] = None,
                 scratch_ptr: Optional[int] = None, stream: int = 0) -> float:
        """rthip_nf4_quantize; returns the offset (0.0 for fp32 scales)."""
        offset = _f32(0.0)
        self._check(self._lib.rthip_nf4_quantize(
            values_ptr, element_count, block_size, encoding,
            second_level_block, codes_ptr, primary_ptr, secondary_ptr,
            scratch_ptr, ctypes.byref(offset), stream))
        return float(offset.value)

    def lora_reduce(self, x_ptr: int, lora_a_ptr: int, reduced_ptr: int,
                    rows: int, input_width: int, rank: int,
                    stream: int = 0) -> None:
        self._check(self._lib.rthip_lora_reduce(
            x_ptr, lora_a_ptr, reduced_ptr, rows, input_width, rank, stream))

    def lora_linear_forward(self, x_ptr: int, weight: DeviceWeight,
                            bias_ptr: Optional[int],
                            lora_a_ptr: Optional[int],
                            lora_b_ptr: int, rank: int, lora_scale: float,
                            reduced_ptr: int, y_ptr: int, rows: int,
                            stream: int = 0,
                            algorithm: Optional[int] = None) -> None:
        tail = [bias_ptr, lora_a_ptr, lora_b_ptr, rank, lora_scale,
                reduced_ptr, y_ptr, rows, weight.input_width,
                weight.output_width, weight.block_size, stream]
        if algorithm is None:
            status = self._lib.rthip_nf4_lora_linear_forward(
                x_ptr, *weight.abi_arguments(), *tail)
        else:
            status = self._lib.rthip_nf4_lora_linear_forward_with(
                algorithm, x_ptr, *weight.abi_arguments(), *tail)
        self._check(status)

    def lora_backward(self, dy_ptr: int, x_ptr: Optional[int],
                      reduced_ptr: Optional[int], lora_b_ptr: int, rank: int,
                      lora_scale: float, d_reduced_ptr: int,
                      d_lora_a_ptr: Optional[int],
                      d_lora_b_ptr: Optional[int], rows: int,
                      input_width: int, output_width: int,
                      stream: int = 0) -> None:
        """rthip_lora_backward: d_reduced, and dA / dB where a buffer is
        given."""
        self._check(self._lib.rthip_lora_backward(
            dy_ptr, x_ptr, reduced_ptr, lora_b_ptr, rank, lora_scale,
            d_reduced_ptr, d_lora_a_ptr, d_lora_b_ptr, rows, input_width,
            output_width, stream))

    def lora_linear_input_backward(self, dy_ptr: int, weight: DeviceWeight,
                                   lora_a_ptr: int, d_reduced_ptr: int,
                                   rank: int, dx_ptr: int, rows: int,
                                   stream: int = 0,
                                   algorithm: Optional[int] = None) -> None:
        """dx = dy . deq(W) + d_reduced . A."""
        tail = [lora_a_ptr, d_reduced_ptr, rank, dx_ptr, rows,
                weight.input_width, weight.output_width, weight.block_size,
                stream]
        if algorithm is None:
            status = self._lib.rthip_nf4_lora_linear_input_backward(
                dy_ptr, *weight.abi_arguments(), *tail)
        else:
            status = self._lib.rthip_nf4_lora_linear_input_backward_with(
                algorithm, dy_ptr, *weight.abi_arguments(), *tail)
        self._check(status)

    def linear_input_backward(self, dy_ptr: int, weight: DeviceWeight,
                              dx_ptr: int, rows: int, stream: int = 0,
                              algorithm: Optional[int] = None) -> None:
        tail = [dx_ptr, rows, weight.input_width, weight.output_width,
                weight.block_size, stream]
        if algorithm is None:
            status = self._lib.rthip_nf4_linear_input_backward(
                dy_ptr, *weight.abi_arguments(), *tail)
        else:
            status = self._lib.rthip_nf4_linear_input_backward_with(
                algorithm, dy_ptr, *weight.abi_arguments(), *tail)
        self._check(status)

    def linear_input_backward_no_alloc(self, dy_ptr: int,
                                       weight: DeviceWeight, dx_ptr: int,
                                       rows: int, stream: int = 0) -> None:
        """The small-batch input backward with its partial sums in the
        library's own device array: nothing is allocated."""
        self._check(self._lib.rthip_nf4_linear_input_backward_no_alloc(
            dy_ptr, *weight.abi_arguments(), dx_ptr, rows,
            weight.input_width, weight.output_width, weight.block_size,
            stream))

    def release_workspaces(self, stream: int = 0,
                           every_stream: bool = True) -> None:
        self._check(self._lib.rthip_release_workspaces(
            stream, 1 if every_stream else 0))

    def check_payload(self, weight: DeviceWeight,
                      element_count: Optional[int] = None,
                      stream: int = 0) -> None:
        """Raises InvalidArgument, with the reference's message, unless the
        payload satisfies the content rules of a canonical NF4 payload."""
        if element_count is None:
            element_count = weight.output_width * weight.input_width
        self._check(self._lib.rthip_nf4_check_payload(
            *weight.abi_arguments(), element_count, weight.block_size, stream))

    def dequantize(self, weight: DeviceWeight, out_ptr: int,
                   element_count: Optional[int] = None,
                   stream: int = 0) -> None:
        if element_count is None:
            element_count = weight.output_width * weight.input_width
        self._check(self._lib.rthip_nf4_dequantize(
            *weight.abi_arguments(), out_ptr, element_count,
            weight.block_size, stream))


_library: Optional[Library] = None


def load_library() -> Library:
    """The process-wide Library; raises if librthip.so is not built."""
    global _library
    if _library is None:
        _library = Library()
    return _library
