"""PyTorch plumbing around the C ABI: torch allocates device memory and owns
the stream, librthip.so does all the arithmetic.  Importing this module needs
torch; nothing here computes on the host."""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from .binding import (
    SCALE_DOUBLE_QUANTIZED_UINT8,
    SCALE_FLOAT32,
    DeviceWeight,
    load_library,
)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def upload_weight(output_width: int, input_width: int, block_size: int,
                  codes: np.ndarray, *, fp32_scales=None, scale_codes=None,
                  second_level=None, second_level_block: int = 0,
                  offset: float = 0.0, device="cuda") -> DeviceWeight:
    """Copies a canonical host payload (the fields of the reference's
    Nf4Payload) into device memory, byte for byte."""
    codes_t = torch.from_numpy(np.ascontiguousarray(codes)).to(device)
    if fp32_scales is not None:
        primary = torch.from_numpy(
            np.ascontiguousarray(fp32_scales, dtype=np.float32)).to(device)
        return DeviceWeight(output_width, input_width, block_size,
                            SCALE_FLOAT32, codes_t, primary, None)
    primary = torch.from_numpy(
        np.ascontiguousarray(scale_codes, dtype=np.uint8)).to(device)
    secondary = torch.from_numpy(
        np.ascontiguousarray(second_level, dtype=np.float32)).to(device)
    return DeviceWeight(output_width, input_width, block_size,
                        SCALE_DOUBLE_QUANTIZED_UINT8, codes_t, primary,
                        secondary, second_level_block, float(offset))


def quantize_weight(dense: torch.Tensor, block_size: int = 64,
                    double_quantized: bool = False,
                    second_level_block: int = 256) -> DeviceWeight:
    """Quantizes a dense [output_width, input_width] fp32 device tensor with
    rthip_nf4_quantize; the payload never leaves the device."""
    assert dense.is_cuda and dense.dtype == torch.float32 and \
        dense.is_contiguous() and dense.dim() == 2
    output_width, input_width = dense.shape
    count = dense.numel()
    blocks = (count + block_size - 1) // block_size
    codes = torch.empty((count + 1) // 2, dtype=torch.uint8,
                        device=dense.device)
    library = load_library()
    if not double_quantized:
        scales = torch.empty(blocks, dtype=torch.float32, device=dense.device)
        library.quantize(dense.data_ptr(), count, block_size, SCALE_FLOAT32, 0,
                         codes.data_ptr(), scales.data_ptr(), None, None,
                         _stream())
        return DeviceWeight(output_width, input_width, block_size,
                            SCALE_FLOAT32, codes, scales, None)
    groups = (blocks + second_level_block - 1) // second_level_block
    scale_codes = torch.empty(blocks, dtype=torch.uint8, device=dense.device)
    second = torch.empty(groups, dtype=torch.float32, device=dense.device)
    scratch = torch.empty(blocks, dtype=torch.float32, device=dense.device)
    offset = library.quantize(
        dense.data_ptr(), count, block_size, SCALE_DOUBLE_QUANTIZED_UINT8,
        second_level_block, codes.data_ptr(), scale_codes.data_ptr(),
        second.data_ptr(), scratch.data_ptr(), _stream())
    return DeviceWeight(output_width, input_width, block_size,
                        SCALE_DOUBLE_QUANTIZED_UINT8, codes, scale_codes,
                        second, second_level_block, offset)


def linear_forward(x: torch.Tensor, weight: DeviceWeight,
                   bias: Optional[torch.Tensor] = None,
                   out: Optional[torch.Tensor] = None,
                   algorithm: Optional[int] = None) -> torch.Tensor:
    """y = x . deq(W)^T (+ bias) through rthip_nf4_linear_forward."""
    assert x.is_cuda and x.dtype == torch.float32 and x.is_contiguous()
    rows = x.numel() // weight.input_width
    if out is None:
        out = torch.empty((rows, weight.output_width), dtype=torch.float32,
                          device=x.device)
    load_library().linear_forward(
        x.data_ptr(), weight, None if bias is None else bias.data_ptr(),
        out.data_ptr(), rows, _stream(), algorithm)
    return out


def linear_forward_group(x: torch.Tensor, weights, biases=None):
    """[x . deq(W_m)^T (+ bias_m) for every m] for weights that share x,
    through rthip_nf4_linear_forward_group (one launch for decode-sized x)."""
    assert x.is_cuda and x.dtype == torch.float32 and x.is_contiguous()
    rows = x.numel() // weights[0].input_width
    if biases is None:
        biases = [None] * len(weights)
    outs = [torch.empty((rows, weight.output_width), dtype=torch.float32,
                        device=x.device) for weight in weights]
    load_library().linear_forward_group(
        x.data_ptr(),
        [(weight, None if bias is None else bias.data_ptr(), out.data_ptr())
         for weight, bias, out in zip(weights, biases, outs)],
        rows, _stream())
    return outs


def lora_linear_forward_group(x: torch.Tensor, weights, adapters,
                              biases=None, reduce_first=False):
    """Like linear_forward_group for layers with low-rank adapters:
    adapters[m] is None or (lora_a, lora_b, lora_scale); ONE call of
    rthip_nf4_lora_linear_forward_group, which takes x . A_m^T itself
    (reduce_first: rthip_lora_reduce per adapter beforehand, and members that
    say their product is already there).  Returns (outputs, reduced) where
    reduced[m] is x . A_m^T or None."""
    assert x.is_cuda and x.dtype == torch.float32 and x.is_contiguous()
    library = load_library()
    rows = x.numel() // weights[0].input_width
    if biases is None:
        biases = [None] * len(weights)
    outs = [torch.empty((rows, weight.output_width), dtype=torch.float32,
                        device=x.device) for weight in weights]
    reduced = []
    members = []
    for weight, bias, out, adapter in zip(weights, biases, outs, adapters):
        entry = None
        if adapter is None:
            reduced.append(None)
        else:
            lora_a, lora_b, lora_scale = adapter
            rank = lora_a.shape[0]
            assert tuple(lora_a.shape) == (rank, weight.input_width)
            assert tuple(lora_b.shape) == (weight.output_width, rank)
            product = torch.empty((rows, rank), dtype=torch.float32,
                                  device=x.device)
            if reduce_first:
                library.lora_reduce(x.data_ptr(), lora_a.data_ptr(),
                                    product.data_ptr(), rows,
                                    weight.input_width, rank, _stream())
            reduced.append(product)
            entry = (None if reduce_first else lora_a.data_ptr(),
                     lora_b.data_ptr(), product.data_ptr(), rank, lora_scale)
        members.append((weight, None if bias is None else bias.data_ptr(),
                        out.data_ptr(), entry))
    library.lora_linear_forward_group(x.data_ptr(), members, rows, _stream())
    return outs, reduced


def lora_linear_forward(x: torch.Tensor, weight: DeviceWeight,
                        lora_a: torch.Tensor, lora_b: torch.Tensor,
                        lora_scale: float,
                        bias: Optional[torch.Tensor] = None,
                        out: Optional[torch.Tensor] = None,
                        reduced: Optional[torch.Tensor] = None,
                        algorithm: Optional[int] = None):
    """y = x . deq(W)^T (+ bias) + lora_scale * (x . A^T) . B^T through
    rthip_nf4_lora_linear_forward.  Returns (y, reduced) where reduced is
    x . A^T, [rows, rank]."""
    for tensor in (x, lora_a, lora_b):
        assert tensor.is_cuda and tensor.dtype == torch.float32 and \
            tensor.is_contiguous()
    rows = x.numel() // weight.input_width
    rank = lora_a.shape[0]
    assert tuple(lora_a.shape) == (rank, weight.input_width)
    assert tuple(lora_b.shape) == (weight.output_width, rank)
    if out is None:
        out = torch.empty((rows, weight.output_width), dtype=torch.float32,
                          device=x.device)
    if reduced is None:
        reduced = torch.empty((rows, rank), dtype=torch.float32,
                              device=x.device)
    load_library().lora_linear_forward(
        x.data_ptr(), weight, None if bias is None else bias.data_ptr(),
        lora_a.data_ptr(), lora_b.data_ptr(), rank, float(lora_scale),
        reduced.data_ptr(), out.data_ptr(), rows, _stream(), algorithm)
    return out, reduced


def lora_linear_backward(dy: torch.Tensor, x: torch.Tensor,
                         weight: DeviceWeight, lora_a: torch.Tensor,
                         lora_b: torch.Tensor, lora_scale: float,
                         reduced: torch.Tensor,
                         algorithm: Optional[int] = None):
    """The backward pass of a Linear with a packed (frozen) weight and a
    trainable adapter, through rthip_lora_backward and
    rthip_nf4_lora_linear_input_backward: returns (dx, dA, dB).  `reduced` is
    x . A^T as lora_linear_forward returned it."""
    for tensor in (dy, x, lora_a, lora_b, reduced):
        assert tensor.is_cuda and tensor.dtype == torch.float32 and \
            tensor.is_contiguous()
    rows = x.numel() // weight.input_width
    rank = lora_a.shape[0]
    assert dy.numel() == rows * weight.output_width
    assert tuple(lora_a.shape) == (rank, weight.input_width)
    assert tuple(lora_b.shape) == (weight.output_width, rank)
    assert reduced.numel() == rows * rank
    d_reduced = torch.empty((rows, rank), dtype=torch.float32,
                            device=x.device)
    d_a = torch.empty_like(lora_a)
    d_b = torch.empty_like(lora_b)
    dx = torch.empty((rows, weight.input_width), dtype=torch.float32,
                     device=x.device)
    library = load_library()
    library.lora_backward(
        dy.data_ptr(), x.data_ptr(), reduced.data_ptr(), lora_b.data_ptr(),
        rank, float(lora_scale), d_reduced.data_ptr(), d_a.data_ptr(),
        d_b.data_ptr(), rows, weight.input_width, weight.output_width,
        _stream())
    library.lora_linear_input_backward(
        dy.data_ptr(), weight, lora_a.data_ptr(), d_reduced.data_ptr(), rank,
        dx.data_ptr(), rows, _stream(), algorithm)
    return dx, d_a, d_b


def matmul(left: torch.Tensor, right: torch.Tensor,
           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """left [..., rows, shared] x right [..., shared, columns] through
    rthip_matmul (identical leading batch dimensions, no broadcasting)."""
    for tensor in (left, right):
        assert tensor.is_cuda and tensor.dtype == torch.float32 and \
            tensor.is_contiguous()
    assert left.shape[:-2] == right.shape[:-2]
    assert left.shape[-1] == right.shape[-2]
    rows, shared, columns = left.shape[-2], left.shape[-1], right.shape[-1]
    batch = 1
    for extent in left.shape[:-2]:
        batch *= extent
    if out is None:
        out = torch.empty(tuple(left.shape[:-2]) + (rows, columns),
                          dtype=torch.float32, device=left.device)
    load_library().matmul(left.data_ptr(), right.data_ptr(), out.data_ptr(),
                          batch, rows, shared, columns, _stream())
    return out


def linear_input_backward(dy: torch.Tensor, weight: DeviceWeight,
                          out: Optional[torch.Tensor] = None,
                          algorithm: Optional[int] = None) -> torch.Tensor:
    """dx = dy . deq(W) through rthip_nf4_linear_input_backward."""
    assert dy.is_cuda and dy.dtype == torch.float32 and dy.is_contiguous()
    rows = dy.numel() // weight.output_width
    if out is None:
        out = torch.empty((rows, weight.input_width), dtype=torch.float32,
                          device=dy.device)
    load_library().linear_input_backward(
        dy.data_ptr(), weight, out.data_ptr(), rows, _stream(), algorithm)
    return out


def check_payload(weight: DeviceWeight) -> None:
    """The content rules of require_canonical_payload
    (src/core/quantization/quantized_weight.cpp:102-174 under /root/reference)
    on a payload in device memory; raises InvalidArgument with the reference's
    message for the first rule that is broken."""
    load_library().check_payload(weight, stream=_stream())


def dequantize(weight: DeviceWeight) -> torch.Tensor:
    """deq(W) as an fp32 tensor through rthip_nf4_dequantize (checking aid)."""
    out = torch.empty((weight.output_width, weight.input_width),
                      dtype=torch.float32, device=weight.codes.device)
    load_library().dequantize(weight, out.data_ptr(), stream=_stream())
    return out
