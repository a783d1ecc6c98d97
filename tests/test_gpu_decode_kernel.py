"""The decode kernel for one to four rows of x (csrc/nf4_gemv1.hip) against
the CPU oracle and an fp64 accumulation, through the C ABI, on the shapes
that steer its instances: one to three stripes per thread, eight, four or two
weight rows per batch, fewer batches than compute units and many per
workgroup, both scale encodings (nested scales with batches on and off
second-level group boundaries, and with small and large groups), bias, the
adapter epilogue, and groups whose members differ in size or fall to another
kernel.  The bar is the one of test_gpu_parity.py:
    max|gpu - exact| / (sqrt(K) * rms(x) * rms(deq W)) <= 1e-5
against fp64 over the bit-exact dequantised weight, and the same measure
against the oracle's sequential fp32 sums plus the oracle's own distance from
fp64; outputs of a grouped launch equal the separate launches bit for bit.
"""
import numpy as np
import pytest

import helpers

pytestmark = pytest.mark.gpu

TOLERANCE = 1.0e-5


def upload(gpu, weight):
    return gpu.upload_weight(
        weight.output_width, weight.input_width, weight.block_size,
        weight.codes, fp32_scales=weight.fp32_scales,
        scale_codes=weight.scale_codes, second_level=weight.second_level,
        second_level_block=weight.second_level_block, offset=weight.offset)


def to_device(array):
    import torch
    return torch.from_numpy(np.ascontiguousarray(array)).cuda()


def host(tensor):
    import torch
    torch.cuda.synchronize()
    return tensor.cpu().numpy()


def served_by_decode_kernel(package, library, weight, rows, members=1):
    encoding = (package.SCALE_FLOAT32 if weight.scale_codes is None
                else package.SCALE_DOUBLE_QUANTIZED_UINT8)
    return library.forward_kernel_name(
        rows, weight.input_width, [weight.output_width] * members,
        weight.block_size, encoding, weight.second_level_block or 0)


def check_forward(gpu, oracle, weight, x, bias=None, oracle_rows=None):
    device_weight = upload(gpu, weight)
    dense = oracle.dequantize(weight)
    exact = helpers.exact_forward(x, dense)
    if bias is not None:
        exact = exact + bias.astype(np.float64)[None, :]
    sample = slice(0, x.shape[0] if oracle_rows is None else oracle_rows)
    cpu = oracle.forward(x[sample], weight, bias)
    scale = (weight.input_width, helpers.rms(x), helpers.rms(dense))
    cpu_error = helpers.normalized_error(cpu, exact[sample], *scale)
    y = host(gpu.linear_forward(to_device(x), device_weight,
                                None if bias is None else to_device(bias)))
    error = helpers.normalized_error(y, exact, *scale)
    assert error <= TOLERANCE, f"vs fp64: {error:.3g}"
    drift = helpers.normalized_error(y[sample], cpu, *scale)
    assert drift <= TOLERANCE + cpu_error, \
        f"vs CPU oracle: {drift:.3g} (cpu {cpu_error:.3g})"
    return y


@pytest.mark.parametrize("out_w,in_w,double_quantized,second_level_block", [
    (64, 64, False, 256),        # 8 batches: most workgroups have none
    (64, 64, True, 256),
    (4096, 4096, False, 256),    # one stripe, 8 rows per batch, 2 per CU
    (4096, 4096, True, 256),     # batches start on group boundaries
    (4096, 4096, True, 32),      # sixteen second-level groups per batch
    (4096, 4096, True, 4096),    # a group spans eight batches
    (1024, 8192, False, 256),    # two stripes, 4 rows per batch
    (1024, 8192, True, 256),
    (1024, 4160, True, 256),     # two stripes, the second mostly empty
    (512, 11008, False, 256),    # three stripes, batches off group boundaries
    (512, 11008, True, 256),
    (20000, 512, False, 256),    # ten batches per workgroup, short rows
    (20000, 512, True, 256),
])
@pytest.mark.parametrize("rows", [1, 2, 3, 4])
def test_decode_kernel_against_oracle_and_fp64(gpu, package, library, oracle,
                                               out_w, in_w, double_quantized,
                                               second_level_block, rows):
    weight = oracle.quantize(helpers.normal(11, (out_w, in_w), 0.02), 64,
                             double_quantized, second_level_block)
    assert served_by_decode_kernel(package, library, weight, rows).startswith(
        "gemv1_forward_kernel<"), "this shape should exercise the kernel"
    x = helpers.normal(12 + rows, (rows, in_w), 1.0)
    bias = helpers.normal(13, (out_w,), 0.01) if rows % 2 == 0 else None
    check_forward(gpu, oracle, weight, x, bias,
                  oracle_rows=1 if out_w * in_w > 2 ** 23 else None)


def test_shapes_the_decode_kernel_leaves_to_other_kernels(gpu, package,
                                                          library, oracle):
    """An output width that is no multiple of eight, a block size other than
    64, a row wider than three stripes, five rows: served by other kernels,
    with the same result quality."""
    cases = [(100, 256, 64, 1), (96, 256, 32, 1), (96, 256, 128, 2),
             (64, 16384, 64, 1), (96, 256, 64, 5)]
    for out_w, in_w, block, rows in cases:
        weight = oracle.quantize(helpers.normal(21, (out_w, in_w), 0.02),
                                 block, False, 256)
        assert served_by_decode_kernel(package, library, weight, rows) == ""
        check_forward(gpu, oracle, weight,
                      helpers.normal(22, (rows, in_w), 1.0))


@pytest.mark.parametrize("double_quantized", [False, True])
@pytest.mark.parametrize("rows", [1, 2, 4])
def test_groups_equal_their_members_launched_alone(gpu, package, library,
                                                   oracle, double_quantized,
                                                   rows):
    """Two to four weights on one x in one launch: members of different
    heights (a workgroup's batch sequence crosses member boundaries at
    different steps), a member that another kernel serves, a member with a
    bias."""
    import torch
    in_w = 4096
    widths = [4096, 1024, 11008, 72]
    weights = [oracle.quantize(helpers.normal(31 + m, (width, in_w), 0.02), 64,
                               double_quantized, 256)
               for m, width in enumerate(widths)]
    odd = oracle.quantize(helpers.normal(39, (100, in_w), 0.02), 64,
                          double_quantized, 256)  # 100 % 8 != 0
    device_weights = [upload(gpu, weight) for weight in weights]
    device_odd = upload(gpu, odd)
    x = to_device(helpers.normal(40 + rows, (rows, in_w), 1.0))
    bias = to_device(helpers.normal(41, (widths[1],), 0.01))
    for members in ([0, 1], [0, 1, 2], [0, 1, 2, 3], [3, 2, 1, 0],
                    [0, "odd", 1]):
        chosen = [device_odd if m == "odd" else device_weights[m]
                  for m in members]
        biases = [bias if m == 1 else None for m in members]
        together = gpu.linear_forward_group(x, chosen, biases)
        alone = [gpu.linear_forward(x, weight, b)
                 for weight, b in zip(chosen, biases)]
        torch.cuda.synchronize()
        for m, got, want in zip(members, together, alone):
            helpers.assert_bit_equal(host(got), host(want),
                                     f"member {m} of group {members}")
    # and the members themselves against the oracle
    for weight, device_weight in zip(weights, device_weights):
        got = gpu.linear_forward(x, device_weight)
        dense = oracle.dequantize(weight)
        exact = helpers.exact_forward(host(x), dense)
        error = helpers.normalized_error(host(got), exact, in_w,
                                         helpers.rms(host(x)),
                                         helpers.rms(dense))
        assert error <= TOLERANCE


@pytest.mark.parametrize("rows", [1, 3, 4])
def test_adapter_epilogue_of_the_decode_kernel(gpu, package, library, oracle,
                                               rows):
    """Bias and the low-rank adapter term in the kernel's final sums."""
    out_w, in_w, rank = 2048, 4096, 16
    weight = oracle.quantize(helpers.normal(51, (out_w, in_w), 0.02), 64, True,
                             256)
    device_weight = upload(gpu, weight)
    x = helpers.normal(52, (rows, in_w), 1.0)
    lora_a = helpers.normal(53, (rank, in_w), 0.05)
    lora_b = helpers.normal(54, (out_w, rank), 0.05)
    bias = helpers.normal(55, (out_w,), 0.01)
    scale = 0.5
    y = host(gpu.lora_linear_forward(
        to_device(x), device_weight, to_device(lora_a), to_device(lora_b),
        scale, bias=to_device(bias))[0])
    dense = oracle.dequantize(weight).astype(np.float64)
    exact = (x.astype(np.float64) @ dense.T + bias.astype(np.float64) +
             scale * (x.astype(np.float64) @ lora_a.astype(np.float64).T) @
             lora_b.astype(np.float64).T)
    error = helpers.normalized_error(y, exact, in_w, helpers.rms(x),
                                     helpers.rms(dense))
    assert error <= 2 * TOLERANCE, f"{error:.3g}"


@pytest.mark.parametrize("double_quantized", [False, True])
@pytest.mark.parametrize("rows", [1, 2, 4, 5, 16, 64, 130])
def test_groups_with_adapters_equal_their_members_launched_alone(
        gpu, package, library, oracle, double_quantized, rows):
    """rthip_nf4_lora_linear_forward_group: members with and without a
    low-rank adapter term (ranks 16, 4 and 33; x.A^T taken by the call, several
    adapters in one launch, or beforehand), with and without bias, one
    that the one-row kernel does not take (output width 100), at row counts
    of the decode kernel (<= 4), of the kernel that keeps x in registers
    (<= 128) and beyond (one launch per member).  Every output equals the
    member's own call bit for bit, and the adapted ones are within the bar of
    fp64 over deq(W)."""
    import torch
    in_w = 4096
    widths = [4096, 1024, 4096, 100]
    weights = [oracle.quantize(helpers.normal(61 + m, (width, in_w), 0.02), 64,
                               double_quantized, 256)
               for m, width in enumerate(widths)]
    device_weights = [upload(gpu, weight) for weight in weights]
    x = to_device(helpers.normal(70 + rows, (rows, in_w), 1.0))
    ranks = [16, None, 4, 33]
    adapters = []
    for m, rank in enumerate(ranks):
        if rank is None:
            adapters.append(None)
            continue
        adapters.append((to_device(helpers.normal(80 + m, (rank, in_w), 0.05)),
                         to_device(helpers.normal(90 + m, (widths[m], rank),
                                                  0.05)),
                         0.25 * (m + 1)))
    biases = [None, to_device(helpers.normal(95, (widths[1],), 0.01)),
              to_device(helpers.normal(96, (widths[2],), 0.01)), None]
    for members, reduce_first in (([0, 1, 2], False), ([0, 2], True),
                                  ([1, 0, 3, 2], False), ([3, 0], True),
                                  ([0, 2, 3], False)):
        together, reduced = gpu.lora_linear_forward_group(
            x, [device_weights[m] for m in members],
            [adapters[m] for m in members], [biases[m] for m in members],
            reduce_first=reduce_first)
        torch.cuda.synchronize()
        for m, got, product in zip(members, together, reduced):
            if adapters[m] is None:
                want = gpu.linear_forward(x, device_weights[m], biases[m])
            else:
                lora_a, lora_b, scale = adapters[m]
                want, own = gpu.lora_linear_forward(
                    x, device_weights[m], lora_a, lora_b, scale,
                    bias=biases[m])
                helpers.assert_bit_equal(host(product), host(own),
                                         f"x.A^T of member {m}")
            helpers.assert_bit_equal(host(got), host(want),
                                     f"member {m} of group {members}")
    # the adapted members against fp64
    together, _ = gpu.lora_linear_forward_group(x, device_weights, adapters,
                                                biases)
    x64 = host(x).astype(np.float64)
    for m, got in enumerate(together):
        dense = oracle.dequantize(weights[m]).astype(np.float64)
        exact = x64 @ dense.T
        if biases[m] is not None:
            exact = exact + host(biases[m]).astype(np.float64)
        if adapters[m] is not None:
            lora_a, lora_b, scale = adapters[m]
            exact = exact + scale * (
                x64 @ host(lora_a).astype(np.float64).T) @ \
                host(lora_b).astype(np.float64).T
        error = helpers.normalized_error(host(got), exact, in_w,
                                         helpers.rms(host(x)),
                                         helpers.rms(dense))
        assert error <= 2 * TOLERANCE, f"member {m}: {error:.3g}"


def test_grouped_adapter_arguments_are_checked(gpu, package, library, oracle):
    """A member that names an adapter without its reduced buffer, a rank of
    zero, and two members writing one output are refused before anything is
    launched."""
    import torch
    weight = upload(gpu, oracle.quantize(helpers.normal(7, (64, 256), 0.02),
                                         64, False, 256))
    x = torch.zeros(1, 256, device="cuda")
    y = torch.zeros(1, 64, device="cuda")
    z = torch.zeros(1, 64, device="cuda")
    b = torch.zeros(64, 4, device="cuda")
    reduced = torch.zeros(1, 4, device="cuda")
    raw = library
    with pytest.raises(package.RthipError, match="reduced buffer"):
        raw.lora_linear_forward_group(
            x.data_ptr(), [(weight, None, y.data_ptr(),
                            (None, b.data_ptr(), None, 4, 1.0))], 1)
    with pytest.raises(package.RthipError, match="rank"):
        raw.lora_linear_forward_group(
            x.data_ptr(), [(weight, None, y.data_ptr(),
                            (None, b.data_ptr(), reduced.data_ptr(), 0,
                             1.0))], 1)
    with pytest.raises(package.RthipError, match="same output"):
        raw.lora_linear_forward_group(
            x.data_ptr(), [(weight, None, y.data_ptr(), None),
                           (weight, None, y.data_ptr(), None)], 1)
    a = torch.zeros(4, 256, device="cuda")
    with pytest.raises(package.RthipError, match="same reduced"):
        raw.lora_linear_forward_group(
            x.data_ptr(),
            [(weight, None, y.data_ptr(),
              (a.data_ptr(), b.data_ptr(), reduced.data_ptr(), 4, 1.0)),
             (weight, None, z.data_ptr(),
              (a.data_ptr(), b.data_ptr(), reduced.data_ptr(), 4, 1.0))], 1)
    # and a well-formed single member runs
    raw.lora_linear_forward_group(
        x.data_ptr(), [(weight, None, z.data_ptr(),
                        (None, b.data_ptr(), reduced.data_ptr(), 4, 1.0))], 1)
    torch.cuda.synchronize()
