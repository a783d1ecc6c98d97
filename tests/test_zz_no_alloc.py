"""The entry point that allocates nothing
(rthip_nf4_linear_input_backward_no_alloc), through the C ABI: its dx must
equal, bit for bit, what rthip_nf4_linear_input_backward writes (same
kernels, same chunk split; only the memory the partial sums pass through
differs), on two calls in a row of which the second is smaller, so that what
the first call left in the library's device array cannot leak into the
second result."""
import numpy as np
import pytest

import helpers

pytestmark = pytest.mark.gpu


def upload(gpu, weight):
    return gpu.upload_weight(
        weight.output_width, weight.input_width, weight.block_size,
        weight.codes, fp32_scales=weight.fp32_scales,
        scale_codes=weight.scale_codes, second_level=weight.second_level,
        second_level_block=weight.second_level_block, offset=weight.offset)


def test_no_alloc_input_backward_matches_the_allocating_entry_point(
        gpu, package, library, oracle):
    import torch
    limit = 24 << 20
    # (output_width, input_width, rows): weight rows cut into several chunks
    # (partial sums pass through the array), then a smaller problem that is
    # cut differently, then one that is not cut at all
    cases = [(4096, 1024, 64), (2048, 512, 5), (128, 4096, 16)]
    previous_bytes = None
    for double_quantized in (False, True):
        for index, (out_w, in_w, rows) in enumerate(cases):
            dense = helpers.normal(300 + index, (out_w, in_w), 0.02)
            weight = oracle.quantize(dense, 64, double_quantized, 256)
            device_weight = upload(gpu, weight)
            dy = helpers.normal(310 + index, (rows, out_w), 1.0e-2)
            dy_device = torch.from_numpy(dy).cuda()
            expected = gpu.linear_input_backward(
                dy_device, device_weight, algorithm=package.ALGORITHM_SKINNY)
            got = torch.full((rows, in_w), float("nan"), device="cuda")
            library.linear_input_backward_no_alloc(
                dy_device.data_ptr(), device_weight, got.data_ptr(), rows,
                torch.cuda.current_stream().cuda_stream)
            torch.cuda.synchronize()
            helpers.assert_bit_equal(got.cpu().numpy(),
                                     expected.cpu().numpy(),
                                     f"{out_w}x{in_w}, {rows} rows")
            # and the oracle, to the reference's own bar on a few rows
            picked = min(rows, 2)
            want = oracle.input_backward(dy[:picked], weight)
            assert helpers.reference_close(got.cpu().numpy()[:picked], want)
            if index == 1:
                assert dy.nbytes < previous_bytes  # the second call is smaller
            previous_bytes = dy.nbytes

    # a problem whose partial sums exceed the array is refused, by name
    # (eleven chunks of 64 x 11264 partial sums = 31.7 MB)
    out_w, in_w, rows = 11264, 11264, 64
    codes = torch.zeros(out_w * in_w // 2, dtype=torch.uint8, device="cuda")
    scales = torch.ones(out_w * in_w // 64, device="cuda")
    big = package.DeviceWeight(out_w, in_w, 64, package.SCALE_FLOAT32, codes,
                               scales, None)
    dy_device = torch.zeros(rows, out_w, device="cuda")
    got = torch.zeros(rows, in_w, device="cuda")
    with pytest.raises(package.Unsupported) as refused:
        library.linear_input_backward_no_alloc(
            dy_device.data_ptr(), big, got.data_ptr(), rows,
            torch.cuda.current_stream().cuda_stream)
    assert str(limit) in str(refused.value)
    # more than 64 rows: not this entry point's family
    with pytest.raises(package.Unsupported):
        library.linear_input_backward_no_alloc(
            dy_device.data_ptr(), big, got.data_ptr(), 65,
            torch.cuda.current_stream().cuda_stream)


def test_no_alloc_array_is_bound_to_one_stream(gpu, package, library, oracle):
    """Calls that overlap on the GPU would race on the one static array, so
    it is bound to the stream of the first call: another stream is refused
    until rthip_release_workspaces has unbound it."""
    import torch
    out_w, in_w, rows = 4096, 1024, 64
    weight = oracle.quantize(helpers.normal(320, (out_w, in_w), 0.02), 64,
                             False, 256)
    device_weight = upload(gpu, weight)
    dy_device = torch.from_numpy(
        helpers.normal(321, (rows, out_w), 1.0e-2)).cuda()
    first = torch.empty(rows, in_w, device="cuda")
    main = torch.cuda.current_stream().cuda_stream
    library.linear_input_backward_no_alloc(dy_device.data_ptr(),
                                           device_weight, first.data_ptr(),
                                           rows, main)
    other = torch.cuda.Stream()
    torch.cuda.synchronize()
    second = torch.empty(rows, in_w, device="cuda")
    with pytest.raises(package.Unsupported) as refused:
        library.linear_input_backward_no_alloc(
            dy_device.data_ptr(), device_weight, second.data_ptr(), rows,
            other.cuda_stream)
    assert "another stream" in str(refused.value)
    library.release_workspaces(0, True)  # unbinds (after the stream is done)
    library.linear_input_backward_no_alloc(dy_device.data_ptr(),
                                           device_weight, second.data_ptr(),
                                           rows, other.cuda_stream)
    torch.cuda.synchronize()
    helpers.assert_bit_equal(second.cpu().numpy(), first.cpu().numpy(),
                             "the same call on the newly bound stream")
    # back to the stream the other tests use
    library.release_workspaces(0, True)
