"""TEST INFRASTRUCTURE ONLY: ctypes access to the CPU checkers.

``Oracle``     wraps ``oracle/liboracle.so`` -- the plain-C restatement of the
               reference CPU backend (``nf4_oracle.c``).
``Reference``  wraps ``oracle/_ref/libnf4ref.so`` -- the reference's own C++
               CPU backend, compiled from its sources by ``oracle/Makefile``;
               present only where that build was made.

Only tests, the smoke check and the CPU-baseline leg of the benchmark may
import this module.  Both classes expose the same methods over numpy arrays so
that a test can diff one against the other.
"""
from __future__ import annotations

import ctypes
import dataclasses
import os
from typing import Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_LIBRARY = os.path.join(_HERE, "liboracle.so")
REFERENCE_LIBRARY = os.path.join(_HERE, "_ref", "libnf4ref.so")

SCALE_FLOAT32 = 0
SCALE_DOUBLE_QUANTIZED_UINT8 = 1

_STATUS_EXCEPTIONS = {
    1: ValueError,       # std::invalid_argument
    2: AssertionError,   # std::logic_error
    3: OverflowError,    # std::overflow_error
    4: RuntimeError,     # std::runtime_error
}


@dataclasses.dataclass
class Nf4Weight:
    """Canonical host payload of one packed NF4 weight, row-major [O, I].

    Mirrors Nf4Payload (include/riftco_transformer/core/quantized_weight.hpp:39-43).
    """

    output_width: int
    input_width: int
    block_size: int
    codes: np.ndarray                      # uint8 [ceil(O*I/2)]
    encoding: int = SCALE_FLOAT32
    fp32_scales: Optional[np.ndarray] = None     # float32 [blocks]
    scale_codes: Optional[np.ndarray] = None     # uint8   [blocks]
    second_level: Optional[np.ndarray] = None    # float32 [ceil(blocks/C)]
    second_level_block: int = 0
    offset: float = 0.0

    @property
    def element_count(self) -> int:
        return self.output_width * self.input_width

    @property
    def block_count(self) -> int:
        return -(-self.element_count // self.block_size)

    @property
    def scale_payload_bytes(self) -> int:
        if self.encoding == SCALE_FLOAT32:
            return 4 * self.fp32_scales.size
        return self.scale_codes.size + 4 * self.second_level.size + 4

    @property
    def payload_bytes(self) -> int:
        return self.codes.size + self.scale_payload_bytes


class _Scales(ctypes.Structure):
    _fields_ = [
        ("encoding", ctypes.c_int32),
        ("fp32_scales", ctypes.c_void_p),
        ("fp32_count", ctypes.c_size_t),
        ("quantized_scales", ctypes.c_void_p),
        ("quantized_count", ctypes.c_size_t),
        ("second_level", ctypes.c_void_p),
        ("second_level_count", ctypes.c_size_t),
        ("second_level_block", ctypes.c_size_t),
        ("offset", ctypes.c_float),
    ]


def _ptr(array: Optional[np.ndarray]) -> Optional[int]:
    if array is None or array.size == 0:
        return None
    return array.ctypes.data


def _f32(array) -> np.ndarray:
    return np.ascontiguousarray(array, dtype=np.float32)


def _scales_struct(weight: Nf4Weight) -> _Scales:
    fp32 = weight.fp32_scales
    codes = weight.scale_codes
    second = weight.second_level
    return _Scales(
        weight.encoding,
        _ptr(fp32), 0 if fp32 is None else fp32.size,
        _ptr(codes), 0 if codes is None else codes.size,
        _ptr(second), 0 if second is None else second.size,
        weight.second_level_block,
        weight.offset,
    )


class Oracle:
    """The C restatement (liboracle.so)."""

    kind = "port"

    def __init__(self, path: str = ORACLE_LIBRARY):
        if not os.path.exists(path):
            raise FileNotFoundError(
                f"{path} is not built; run `make -C oracle` (or "
                "__graft_entry__.build())"
            )
        lib = ctypes.CDLL(path)
        self._lib = lib
        sz, vp, i32 = ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int
        sp = ctypes.POINTER(_Scales)
        lib.nf4o_codebook.restype = ctypes.POINTER(ctypes.c_float)
        lib.nf4o_codebook.argtypes = []
        lib.nf4o_block_size_supported.restype = i32
        lib.nf4o_block_size_supported.argtypes = [sz]
        lib.nf4o_nearest_code.restype = ctypes.c_uint8
        lib.nf4o_nearest_code.argtypes = [ctypes.c_float]
        lib.nf4o_quantize.restype = i32
        lib.nf4o_quantize.argtypes = [vp, sz, sz, vp, vp]
        lib.nf4o_double_quantize_scales.restype = i32
        lib.nf4o_double_quantize_scales.argtypes = [
            vp, sz, sz, vp, vp, ctypes.POINTER(ctypes.c_float)]
        lib.nf4o_decode_scale.restype = ctypes.c_float
        lib.nf4o_decode_scale.argtypes = [sp, sz]
        lib.nf4o_dequantize.restype = None
        lib.nf4o_dequantize.argtypes = [vp, sp, sz, sz, vp]
        for name in ("nf4o_linear_forward", "nf4o_linear_input_backward",
                     "nf4o_linear_forward_rowcached",
                     "nf4o_linear_input_backward_rowcached"):
            fn = getattr(lib, name)
            fn.restype = None
            fn.argtypes = [vp, vp, sp, vp, sz, sz, sz, sz]
        lib.nf4o_add_bias.restype = None
        lib.nf4o_add_bias.argtypes = [vp, vp, sz, sz]
        for name in ("nf4o_matmul", "nf4o_matmul_nt"):
            fn = getattr(lib, name)
            fn.restype = None
            fn.argtypes = [vp, vp, vp, sz, sz, sz]
        lib.nf4o_lora_linear_forward.restype = None
        lib.nf4o_lora_linear_forward.argtypes = [
            vp, vp, sp, vp, vp, vp, sz, ctypes.c_float, vp, sz, sz, sz, sz]
        lib.nf4o_lora_linear_backward.restype = None
        lib.nf4o_lora_linear_backward.argtypes = [
            vp, vp, vp, sp, vp, vp, sz, ctypes.c_float, vp, vp, vp, sz, sz,
            sz, sz]
        lib.nf4o_validate_payload.restype = i32
        lib.nf4o_validate_payload.argtypes = [
            sz, sz, vp, sz, sp, ctypes.POINTER(ctypes.c_char_p)]
        lib.nf4o_validate_scale_storage.restype = i32
        lib.nf4o_validate_scale_storage.argtypes = [
            sp, sz, ctypes.POINTER(ctypes.c_char_p)]
        lib.nf4o_scale_payload_bytes.restype = sz
        lib.nf4o_scale_payload_bytes.argtypes = [sp]

    # -- codec -----------------------------------------------------------
    def codebook(self) -> np.ndarray:
        return np.ctypeslib.as_array(self._lib.nf4o_codebook(), (16,)).copy()

    def block_size_supported(self, block_size: int) -> bool:
        return bool(self._lib.nf4o_block_size_supported(block_size))

    def nearest_code(self, value: float) -> int:
        return int(self._lib.nf4o_nearest_code(np.float32(value)))

    def quantize(self, values, block_size: int = 64, double_quantized=False,
                 second_level_block: int = 256) -> Nf4Weight:
        values = _f32(values)
        if values.ndim == 1:
            values = values.reshape(1, -1)
        # QuantizedWeight::quantize_nf4[_double_quantized] check both block
        # sizes before anything is packed
        # (src/core/quantization/quantized_weight.cpp:48-53,308,320-321)
        for size in ((block_size, second_level_block) if double_quantized
                     else (block_size,)):
            if not self.block_size_supported(size):
                raise ValueError("NF4 block size must be one of "
                                 "32, 64, 128, 256, 512, 1024, 2048, or 4096")
        out_w, in_w = values.shape
        count = values.size
        blocks = -(-count // block_size)
        codes = np.zeros(-(-count // 2), dtype=np.uint8)
        scales = np.zeros(blocks, dtype=np.float32)
        status = self._lib.nf4o_quantize(
            values.ctypes.data, count, block_size, codes.ctypes.data,
            scales.ctypes.data)
        self._raise(status, "NF4 source values must be finite")
        if not double_quantized:
            return Nf4Weight(out_w, in_w, block_size, codes, SCALE_FLOAT32,
                             fp32_scales=scales)
        scale_codes, second, offset = self.double_quantize_scales(
            scales, second_level_block)
        return Nf4Weight(out_w, in_w, block_size, codes,
                         SCALE_DOUBLE_QUANTIZED_UINT8, scale_codes=scale_codes,
                         second_level=second,
                         second_level_block=second_level_block, offset=offset)

    def double_quantize_scales(self, scales, second_level_block: int):
        scales = _f32(scales)
        groups = -(-scales.size // second_level_block)
        scale_codes = np.zeros(scales.size, dtype=np.uint8)
        second = np.zeros(groups, dtype=np.float32)
        offset = ctypes.c_float(0.0)
        status = self._lib.nf4o_double_quantize_scales(
            scales.ctypes.data, scales.size, second_level_block,
            scale_codes.ctypes.data, second.ctypes.data, ctypes.byref(offset))
        self._raise(status, "NF4 scale mean exceeds the FP32 range")
        return scale_codes, second, float(offset.value)

    def decode_scales(self, weight: Nf4Weight) -> np.ndarray:
        view = _scales_struct(weight)
        return np.array(
            [self._lib.nf4o_decode_scale(ctypes.byref(view), index)
             for index in range(weight.block_count)], dtype=np.float32)

    # -- the path --------------------------------------------------------
    def dequantize(self, weight: Nf4Weight) -> np.ndarray:
        out = np.empty(weight.element_count, dtype=np.float32)
        view = _scales_struct(weight)
        self._lib.nf4o_dequantize(
            weight.codes.ctypes.data, ctypes.byref(view),
            weight.element_count, weight.block_size, out.ctypes.data)
        return out.reshape(weight.output_width, weight.input_width)

    def _linear(self, name, activations, weight, in_w, out_w):
        activations = _f32(activations).reshape(-1, in_w)
        rows = activations.shape[0]
        out = np.empty((rows, out_w), dtype=np.float32)
        view = _scales_struct(weight)
        getattr(self._lib, name)(
            activations.ctypes.data, weight.codes.ctypes.data,
            ctypes.byref(view), out.ctypes.data, rows, weight.input_width,
            weight.output_width, weight.block_size)
        return out

    def forward(self, x, weight: Nf4Weight, bias=None, faithful=False):
        name = "nf4o_linear_forward" if faithful else \
            "nf4o_linear_forward_rowcached"
        y = self._linear(name, x, weight, weight.input_width,
                         weight.output_width)
        if bias is not None:
            bias = _f32(bias)
            self._lib.nf4o_add_bias(y.ctypes.data, bias.ctypes.data,
                                    y.shape[0], y.shape[1])
        return y

    def input_backward(self, dy, weight: Nf4Weight, faithful=False):
        name = "nf4o_linear_input_backward" if faithful else \
            "nf4o_linear_input_backward_rowcached"
        return self._linear(name, dy, weight, weight.output_width,
                            weight.input_width)

    def matmul(self, left, right) -> np.ndarray:
        """left [rows, shared] x right [shared, columns]."""
        left, right = _f32(left), _f32(right)
        out = np.empty((left.shape[0], right.shape[1]), dtype=np.float32)
        self._lib.nf4o_matmul(left.ctypes.data, right.ctypes.data,
                              out.ctypes.data, left.shape[0], left.shape[1],
                              right.shape[1])
        return out

    def matmul_nt(self, left, right_t) -> np.ndarray:
        """left [rows, shared] x right_t[columns, shared]^T."""
        left, right_t = _f32(left), _f32(right_t)
        out = np.empty((left.shape[0], right_t.shape[0]), dtype=np.float32)
        self._lib.nf4o_matmul_nt(left.ctypes.data, right_t.ctypes.data,
                                 out.ctypes.data, left.shape[0],
                                 left.shape[1], right_t.shape[0])
        return out

    def lora_forward(self, x, weight: Nf4Weight, lora_a, lora_b,
                     lora_scale: float, bias=None) -> np.ndarray:
        x = _f32(x).reshape(-1, weight.input_width)
        lora_a, lora_b = _f32(lora_a), _f32(lora_b)
        bias = None if bias is None else _f32(bias)
        out = np.empty((x.shape[0], weight.output_width), dtype=np.float32)
        view = _scales_struct(weight)
        self._lib.nf4o_lora_linear_forward(
            x.ctypes.data, weight.codes.ctypes.data, ctypes.byref(view),
            _ptr(bias), lora_a.ctypes.data, lora_b.ctypes.data,
            lora_a.shape[0], lora_scale, out.ctypes.data, x.shape[0],
            weight.input_width, weight.output_width, weight.block_size)
        return out

    def lora_backward(self, dy, x, weight: Nf4Weight, lora_a, lora_b,
                      lora_scale: float):
        """(dx, dA, dB) of a Linear with a packed weight and an adapter."""
        x = _f32(x).reshape(-1, weight.input_width)
        dy = _f32(dy).reshape(-1, weight.output_width)
        lora_a, lora_b = _f32(lora_a), _f32(lora_b)
        dx = np.empty_like(x)
        d_a = np.empty_like(lora_a)
        d_b = np.empty_like(lora_b)
        view = _scales_struct(weight)
        self._lib.nf4o_lora_linear_backward(
            dy.ctypes.data, x.ctypes.data, weight.codes.ctypes.data,
            ctypes.byref(view), lora_a.ctypes.data, lora_b.ctypes.data,
            lora_a.shape[0], lora_scale, dx.ctypes.data, d_a.ctypes.data,
            d_b.ctypes.data, x.shape[0], weight.input_width,
            weight.output_width, weight.block_size)
        return dx, d_a, d_b

    # -- validation ------------------------------------------------------
    def validate_payload(self, weight: Nf4Weight) -> None:
        view = _scales_struct(weight)
        message = ctypes.c_char_p()
        status = self._lib.nf4o_validate_payload(
            weight.element_count, weight.block_size, _ptr(weight.codes),
            weight.codes.size, ctypes.byref(view), ctypes.byref(message))
        self._raise(status, (message.value or b"").decode())

    def validate_scale_storage(self, weight: Nf4Weight,
                               expected_scale_count: int) -> None:
        view = _scales_struct(weight)
        message = ctypes.c_char_p()
        status = self._lib.nf4o_validate_scale_storage(
            ctypes.byref(view), expected_scale_count, ctypes.byref(message))
        self._raise(status, (message.value or b"").decode())

    def scale_payload_bytes(self, weight: Nf4Weight) -> int:
        view = _scales_struct(weight)
        return int(self._lib.nf4o_scale_payload_bytes(ctypes.byref(view)))

    @staticmethod
    def _raise(status: int, message: str) -> None:
        if status != 0:
            raise _STATUS_EXCEPTIONS.get(status, RuntimeError)(message)


class Reference:
    """The compiled reference CPU backend (oracle/_ref/libnf4ref.so)."""

    kind = "reference"

    @staticmethod
    def available(path: str = REFERENCE_LIBRARY) -> bool:
        return os.path.exists(path)

    def __init__(self, path: str = REFERENCE_LIBRARY):
        if not os.path.exists(path):
            raise FileNotFoundError(
                f"{path} is not built; run `make -C oracle _ref` where "
                "/root/reference exists"
            )
        lib = ctypes.CDLL(path)
        self._lib = lib
        sz, vp, i32, f32 = (ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int,
                            ctypes.c_float)
        lib.nf4ref_last_error.restype = ctypes.c_char_p
        lib.nf4ref_quantize.restype = i32
        lib.nf4ref_quantize.argtypes = [
            vp, sz, sz, sz, i32, sz, vp, vp, vp, vp,
            ctypes.POINTER(ctypes.c_float)]
        payload = [vp, sz, i32, vp, sz, vp, sz, vp, sz, sz, f32]
        lib.nf4ref_run.restype = i32
        lib.nf4ref_run.argtypes = [i32, vp, vp, sz, sz, sz, sz] + payload
        lib.nf4ref_memory_usage.restype = i32
        lib.nf4ref_memory_usage.argtypes = [sz, sz, sz] + payload + [vp]
        lib.nf4ref_matmul.restype = i32
        lib.nf4ref_matmul.argtypes = [vp, vp, vp, sz, sz, sz]
        lib.nf4ref_validate_scale_storage.restype = i32
        lib.nf4ref_validate_scale_storage.argtypes = [
            i32, vp, sz, vp, sz, vp, sz, sz, f32, sz]
        lib.nf4ref_lora_linear_backward.restype = i32
        lib.nf4ref_lora_linear_backward.argtypes = [
            vp, sz, sz, vp, vp, vp, vp, vp, sz, f32, sz, sz, sz, vp, vp, vp,
            vp]
        lib.nf4ref_lora_linear_forward.restype = i32
        lib.nf4ref_lora_linear_forward.argtypes = [
            vp, vp, vp, vp, sz, f32, vp, sz, sz, sz, sz] + payload

    def _check(self, status: int) -> None:
        if status != 0:
            message = self._lib.nf4ref_last_error().decode()
            raise _STATUS_EXCEPTIONS.get(status, RuntimeError)(message)

    @staticmethod
    def _payload_args(weight: Nf4Weight):
        fp32, codes, second = (weight.fp32_scales, weight.scale_codes,
                               weight.second_level)
        return [
            _ptr(weight.codes), weight.codes.size, weight.encoding,
            _ptr(fp32), 0 if fp32 is None else fp32.size,
            _ptr(codes), 0 if codes is None else codes.size,
            _ptr(second), 0 if second is None else second.size,
            weight.second_level_block, weight.offset,
        ]

    def quantize(self, values, block_size: int = 64, double_quantized=False,
                 second_level_block: int = 256) -> Nf4Weight:
        values = _f32(values)
        if values.ndim == 1:
            values = values.reshape(1, -1)
        out_w, in_w = values.shape
        count = values.size
        blocks = -(-count // block_size)
        codes = np.zeros(-(-count // 2), dtype=np.uint8)
        if not double_quantized:
            scales = np.zeros(blocks, dtype=np.float32)
            self._check(self._lib.nf4ref_quantize(
                values.ctypes.data, out_w, in_w, block_size, 0, 0,
                codes.ctypes.data, scales.ctypes.data, None, None, None))
            return Nf4Weight(out_w, in_w, block_size, codes, SCALE_FLOAT32,
                             fp32_scales=scales)
        # An unsupported second-level block is rejected by the reference
        # before anything is written; size the buffer defensively.
        groups = -(-blocks // max(second_level_block, 1))
        scale_codes = np.zeros(blocks, dtype=np.uint8)
        second = np.zeros(groups, dtype=np.float32)
        offset = ctypes.c_float(0.0)
        self._check(self._lib.nf4ref_quantize(
            values.ctypes.data, out_w, in_w, block_size, 1,
            second_level_block, codes.ctypes.data, None,
            scale_codes.ctypes.data, second.ctypes.data,
            ctypes.byref(offset)))
        return Nf4Weight(out_w, in_w, block_size, codes,
                         SCALE_DOUBLE_QUANTIZED_UINT8, scale_codes=scale_codes,
                         second_level=second,
                         second_level_block=second_level_block,
                         offset=float(offset.value))

    def _run(self, mode, activations, weight, rows, out_shape):
        out = np.empty(out_shape, dtype=np.float32)
        self._check(self._lib.nf4ref_run(
            mode, _ptr(activations), out.ctypes.data, rows,
            weight.input_width, weight.output_width, weight.block_size,
            *self._payload_args(weight)))
        return out

    def validate_payload(self, weight: Nf4Weight) -> None:
        # from_packed_nf4 validates; dequantizing one weight is the cheapest
        # call that reaches it.
        self._run(0, None, weight, 0,
                  (weight.output_width, weight.input_width))

    def validate_scale_storage(self, weight: Nf4Weight,
                               expected_scale_count: int) -> None:
        # require_scale_storage as the dispatcher applies it to a stored
        # weight (dispatch.cpp:108-154, reached through :203-230)
        self._check(self._lib.nf4ref_validate_scale_storage(
            *self._payload_args(weight)[2:], expected_scale_count))

    def dequantize(self, weight: Nf4Weight) -> np.ndarray:
        return self._run(0, None, weight, 0,
                         (weight.output_width, weight.input_width))

    def forward(self, x, weight: Nf4Weight, bias=None, faithful=True):
        x = _f32(x).reshape(-1, weight.input_width)
        y = self._run(1, x, weight, x.shape[0],
                      (x.shape[0], weight.output_width))
        if bias is not None:
            # src/nn/linear.cpp:165-168: a separate broadcast add
            y = y + _f32(bias)[None, :]
        return y

    def input_backward(self, dy, weight: Nf4Weight, faithful=True):
        dy = _f32(dy).reshape(-1, weight.output_width)
        return self._run(2, dy, weight, dy.shape[0],
                         (dy.shape[0], weight.input_width))

    def matmul(self, left, right) -> np.ndarray:
        left, right = _f32(left), _f32(right)
        out = np.empty((left.shape[0], right.shape[1]), dtype=np.float32)
        self._check(self._lib.nf4ref_matmul(
            left.ctypes.data, right.ctypes.data, out.ctypes.data,
            left.shape[0], left.shape[1], right.shape[1]))
        return out

    def lora_forward(self, x, weight: Nf4Weight, lora_a, lora_b,
                     lora_scale: float, bias=None) -> np.ndarray:
        x = _f32(x).reshape(-1, weight.input_width)
        lora_a, lora_b = _f32(lora_a), _f32(lora_b)
        bias = None if bias is None else _f32(bias)
        out = np.empty((x.shape[0], weight.output_width), dtype=np.float32)
        self._check(self._lib.nf4ref_lora_linear_forward(
            x.ctypes.data, _ptr(bias), lora_a.ctypes.data,
            lora_b.ctypes.data, lora_a.shape[0], lora_scale,
            out.ctypes.data, x.shape[0], weight.input_width,
            weight.output_width, weight.block_size,
            *self._payload_args(weight)))
        return out

    def lora_linear_step(self, dense_weight, block_size: int,
                         scale_block_size: int, x, dy, lora_a, lora_b,
                         alpha: float, bias=None):
        """Forward and backward through a real Linear of the reference that
        packs `dense_weight` itself and carries an adapter with the given A
        and B: returns (y, dx, dA, dB).  scale_block_size 0: fp32 scales."""
        dense_weight = _f32(dense_weight)
        output_width, input_width = dense_weight.shape
        x = _f32(x).reshape(-1, input_width)
        dy = _f32(dy).reshape(-1, output_width)
        lora_a, lora_b = _f32(lora_a), _f32(lora_b)
        bias = None if bias is None else _f32(bias)
        y = np.empty((x.shape[0], output_width), dtype=np.float32)
        dx = np.empty_like(x)
        d_a = np.empty_like(lora_a)
        d_b = np.empty_like(lora_b)
        self._check(self._lib.nf4ref_lora_linear_backward(
            dense_weight.ctypes.data, block_size, scale_block_size,
            _ptr(bias), x.ctypes.data, dy.ctypes.data, lora_a.ctypes.data,
            lora_b.ctypes.data, lora_a.shape[0], alpha, x.shape[0],
            input_width, output_width, y.ctypes.data, dx.ctypes.data,
            d_a.ctypes.data, d_b.ctypes.data))
        return y, dx, d_a, d_b

    def memory_usage(self, weight: Nf4Weight) -> dict:
        out = np.zeros(9, dtype=np.uintp)
        self._check(self._lib.nf4ref_memory_usage(
            weight.input_width, weight.output_width, weight.block_size,
            *self._payload_args(weight), out.ctypes.data))
        names = ["packed_code_bytes", "scale_bytes", "logical_payload_bytes",
                 "resident_payload_bytes", "fp32_equivalent_bytes",
                 "fp32_scale_bytes", "scale_code_bytes",
                 "second_level_scale_bytes", "scale_offset_bytes"]
        return dict(zip(names, (int(v) for v in out)))
