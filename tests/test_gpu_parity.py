"""Parity of the HIP kernels with the CPU oracle, through the C ABI, on a real
MI355X.

The bar:
  * nibble unpack, codebook lookup, scale decode, deq(W): bit-exact;
  * y and dx: the reference's own |a-e| <= 3e-5*max(1,|a|,|e|) on its small
    fixtures, and on transformer-sized layers
        max|gpu - exact| / (sqrt(K) * rms(act) * rms(deq W)) <= 1e-5
    against an fp64 accumulation over the bit-exact dequantised weights, plus
        max|gpu - cpu|   / (sqrt(K) * rms(act) * rms(deq W))
            <= 1e-5 + (the same measure of cpu against fp64)
    for the oracle's sequential fp32 sums, whose own rounding walk reaches
    ~1.2e-5 at K = 11008.
"""
import json
import os

import numpy as np
import pytest

import helpers

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
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


def families(package):
    """AUTO plus every pinned kernel family; a family that does not accept a
    shape answers RTHIP_UNSUPPORTED and is skipped by `run`."""
    return (None, package.ALGORITHM_GENERIC, package.ALGORITHM_GEMV,
            package.ALGORITHM_MFMA, package.ALGORITHM_SKINNY,
            package.ALGORITHM_RESIDENT)


def run(package, function, *args, algorithm):
    """One launch with the family pinned; None when it refuses the shape."""
    try:
        return host(function(*args, algorithm=algorithm))
    except package.Unsupported:
        assert algorithm is not None, "AUTO must accept every shape"
        return None


def check_layer(gpu, package, library, oracle, weight, x, dy, bias=None,
                oracle_rows=None):
    """Both products of one layer, every applicable kernel family."""
    device_weight = upload(gpu, weight)
    dense = oracle.dequantize(weight)
    helpers.assert_bit_equal(host(gpu.dequantize(device_weight)), dense,
                             "deq(W) on the GPU")
    weight_rms = helpers.rms(dense)
    rows = x.shape[0]
    sample = slice(0, rows if oracle_rows is None else oracle_rows)

    exact = helpers.exact_forward(x, dense)
    if bias is not None:
        exact = exact + bias.astype(np.float64)[None, :]
    cpu = oracle.forward(x[sample], weight, bias)
    cpu_error = helpers.normalized_error(
        cpu, exact[sample], weight.input_width, helpers.rms(x), weight_rms)
    x_device = to_device(x)
    bias_device = None if bias is None else to_device(bias)
    for family in families(package):
        y = run(package, gpu.linear_forward, x_device, device_weight,
                bias_device, algorithm=family)
        if y is None:
            continue
        name = package.ALGORITHM_NAMES[family or 0]
        error = helpers.normalized_error(
            y, exact, weight.input_width, helpers.rms(x), weight_rms)
        assert error <= TOLERANCE, f"forward/{name} vs fp64: {error:.3g}"
        drift = helpers.normalized_error(
            y[sample], cpu, weight.input_width, helpers.rms(x), weight_rms)
        assert drift <= TOLERANCE + cpu_error, \
            f"forward/{name} vs CPU oracle: {drift:.3g} (cpu {cpu_error:.3g})"

    exact = helpers.exact_input_backward(dy, dense)
    cpu = oracle.input_backward(dy[sample], weight)
    cpu_error = helpers.normalized_error(
        cpu, exact[sample], weight.output_width, helpers.rms(dy), weight_rms)
    dy_device = to_device(dy)
    for family in families(package):
        dx = run(package, gpu.linear_input_backward, dy_device,
                 device_weight, algorithm=family)
        if dx is None:
            continue
        name = package.ALGORITHM_NAMES[family or 0]
        error = helpers.normalized_error(
            dx, exact, weight.output_width, helpers.rms(dy), weight_rms)
        assert error <= TOLERANCE, f"backward/{name} vs fp64: {error:.3g}"
        drift = helpers.normalized_error(
            dx[sample], cpu, weight.output_width, helpers.rms(dy), weight_rms)
        assert drift <= TOLERANCE + cpu_error, \
            f"backward/{name} vs CPU oracle: {drift:.3g} (cpu {cpu_error:.3g})"


# ---- the reference's own fixtures ------------------------------------------

CLOSED_FORM = {
    "aligned": (helpers.aligned_weight, helpers.aligned_input,
                helpers.aligned_upstream),
    "edge": (helpers.edge_weight, helpers.edge_input, helpers.edge_upstream),
}


@pytest.mark.parametrize("name", ["aligned", "edge"])
@pytest.mark.parametrize("double_quantized", [False, True])
def test_reference_fixtures(gpu, package, library, oracle, name,
                            double_quantized):
    """Counterpart of run_accelerator_oracle
    (tests/core/backend/test_quantized_linear_backend.cpp:382-453): aligned
    [3 x 32] and edge [33 x 33] layouts, block 32, both scale encodings,
    against the golden outputs of the compiled reference at its tolerance."""
    golden = np.load(os.path.join(GOLDEN, "closed_form.npz"))
    make_weight, make_input, make_upstream = CLOSED_FORM[name]
    tag = f"{name}_{'dq' if double_quantized else 'fp32'}"
    weight = oracle.quantize(make_weight(), 32, double_quantized, 32)
    device_weight = upload(gpu, weight)
    helpers.assert_bit_equal(host(gpu.dequantize(device_weight)),
                             golden[f"{tag}_dequantized"], "deq(W)")
    x, dy = make_input(), make_upstream()
    for family in families(package):
        y = run(package, gpu.linear_forward, to_device(x), device_weight,
                algorithm=family)
        assert y is None or \
            helpers.reference_close(y, golden[f"{tag}_forward"])
        dx = run(package, gpu.linear_input_backward, to_device(dy),
                 device_weight, algorithm=family)
        assert dx is None or \
            helpers.reference_close(dx, golden[f"{tag}_input_backward"])


@pytest.mark.parametrize("double_quantized", [False, True])
def test_config1_tiny_layer_with_bias(gpu, package, library, oracle,
                                      double_quantized):
    """The tiny parity configuration (x [16, 256], W [768, 256], bias) against
    the compiled reference's stored outputs."""
    golden = np.load(os.path.join(GOLDEN, "config1.npz"))
    x = helpers.normal(1, (16, 256), 1.0)
    dense = helpers.normal(2, (768, 256), 0.02)
    bias = helpers.normal(3, (768,), 0.01)
    dy = helpers.normal(4, (16, 768), 1.0e-2)
    tag = "dq" if double_quantized else "fp32"
    weight = oracle.quantize(dense, 64, double_quantized, 256)
    device_weight = upload(gpu, weight)
    y = host(gpu.linear_forward(to_device(x), device_weight, to_device(bias)))
    assert helpers.reference_close(y, golden[f"{tag}_forward_bias"])
    dx = host(gpu.linear_input_backward(to_device(dy), device_weight))
    assert helpers.reference_close(dx, golden[f"{tag}_input_backward"])
    check_layer(gpu, package, library, oracle, weight, x, dy, bias)


# ---- transformer-sized layers --------------------------------------------

@pytest.mark.parametrize("name,out_w,in_w,seed", [
    ("q_proj", 4096, 4096, 11),
    ("gate_proj", 11008, 4096, 12),
    ("down_proj", 4096, 11008, 13),
])
@pytest.mark.parametrize("double_quantized", [False, True])
def test_llama_rows_against_golden(gpu, package, library, oracle, name,
                                   out_w, in_w, seed, double_quantized):
    """One row (the decode GEMV) through each distinct Llama-7B projection:
    deq(W) digest and outputs against the compiled reference's vectors."""
    golden = np.load(os.path.join(GOLDEN, "llama_rows.npz"))
    with open(os.path.join(GOLDEN, "digests.json")) as handle:
        meta = json.load(handle)["llama"][name]
    tag = "dq" if double_quantized else "fp32"
    dense = helpers.normal(seed, (out_w, in_w), 0.02)
    x = helpers.normal(seed + 100, (1, in_w), 1.0)
    dy = helpers.normal(seed + 200, (1, out_w), 1.0e-2)
    weight = oracle.quantize(dense, 64, double_quantized, 256)
    device_weight = upload(gpu, weight)
    assert device_weight.payload_bytes == meta[tag]["payload_bytes"]
    deq = host(gpu.dequantize(device_weight))
    assert helpers.sha256(deq) == meta[tag]["dequantized_sha256"]
    weight_rms = helpers.rms(deq)
    y = host(gpu.linear_forward(to_device(x), device_weight))
    expected = golden[f"{name}_{tag}_forward"]
    exact = helpers.exact_forward(x, deq)
    own = helpers.normalized_error(expected, exact, in_w, helpers.rms(x),
                                   weight_rms)
    assert helpers.normalized_error(y, exact, in_w, helpers.rms(x),
                                    weight_rms) <= TOLERANCE
    assert helpers.normalized_error(y, expected, in_w, helpers.rms(x),
                                    weight_rms) <= TOLERANCE + own
    dx = host(gpu.linear_input_backward(to_device(dy), device_weight))
    expected = golden[f"{name}_{tag}_input_backward"]
    exact = helpers.exact_input_backward(dy, deq)
    own = helpers.normalized_error(expected, exact, out_w, helpers.rms(dy),
                                   weight_rms)
    assert helpers.normalized_error(dx, exact, out_w, helpers.rms(dy),
                                    weight_rms) <= TOLERANCE
    assert helpers.normalized_error(dx, expected, out_w, helpers.rms(dy),
                                    weight_rms) <= TOLERANCE + own


@pytest.mark.parametrize("rows", [1, 2, 3, 4, 5, 16, 64, 65, 67, 80, 81, 96,
                                  112, 113, 128, 129, 131, 190, 193, 224,
                                  225, 257, 300, 320, 321])
@pytest.mark.parametrize("double_quantized", [False, True])
def test_row_counts_across_the_gemv_mfma_crossover(
        gpu, package, library, oracle, rows, double_quantized):
    dense = helpers.normal(50, (1024, 2048), 0.02)
    weight = oracle.quantize(dense, 64, double_quantized, 256)
    x = helpers.normal(51 + rows, (rows, 2048), 1.0)
    dy = helpers.normal(52 + rows, (rows, 1024), 1.0e-2)
    check_layer(gpu, package, library, oracle, weight, x, dy)


@pytest.mark.parametrize("rows", [97, 128, 129, 192, 193])
def test_row_counts_where_the_upstream_is_much_wider(gpu, package, library,
                                                      oracle, rows):
    """An input backward whose dy is at least twice as wide as dx runs up to
    192 rows as parts of 64 through the small-batch kernel."""
    assert library.select_algorithm(
        package.INPUT_BACKWARD, rows, 512, 1152, 64) == (
            package.ALGORITHM_SKINNY if rows <= 192 else package.ALGORITHM_MFMA)
    weight = oracle.quantize(helpers.normal(54, (1152, 512), 0.02), 64, True,
                             256)
    x = helpers.normal(55 + rows, (rows, 512), 1.0)
    dy = helpers.normal(56 + rows, (rows, 1152), 1.0e-2)
    check_layer(gpu, package, library, oracle, weight, x, dy, oracle_rows=4)


@pytest.mark.parametrize("out_w,in_w,block,second", [
    (96, 160, 32, 32),      # narrow rows, tiles mostly empty
    (200, 352, 32, 64),     # output width not a multiple of the tile
    (128, 4096, 4096, 32),  # one block per row
    (64, 96, 64, 32),       # blocks straddle rows (96 % 64 != 0)
    (32, 11008, 128, 256),
    (136, 48, 32, 32),      # row width a multiple of 16 only
    (40, 50, 32, 32),       # nothing aligned
])
@pytest.mark.parametrize("double_quantized", [False, True])
def test_ragged_shapes_and_block_sizes(gpu, package, library, oracle, out_w,
                                       in_w, block, second, double_quantized):
    dense = helpers.normal(60, (out_w, in_w), 0.05)
    dense[::3, ::5] = 0.0
    weight = oracle.quantize(dense, block, double_quantized, second)
    for rows in (1, 3, 37):
        x = helpers.normal(61 + rows, (rows, in_w), 1.0)
        dy = helpers.normal(62 + rows, (rows, out_w), 1.0e-2)
        check_layer(gpu, package, library, oracle, weight, x, dy)


@pytest.mark.parametrize("out_w,in_w,block,double_quantized", [
    (33000, 64, 32, False),    # >= 256 output tiles: one workgroup per tile
    (300, 1280, 64, True),     # fewer (tile, slab) units than compute units
    (2000, 1600, 64, False),   # last pass over the compute units and last tile partly empty
    (5000, 2048, 64, True),    # runs of one and two units, tiles shared
    (1000, 16384, 128, False),  # many workgroups per output tile
    (30000, 512, 32, True),    # runs that cross from one tile into the next
])
def test_small_batch_work_split(gpu, package, library, oracle, out_w, in_w,
                                block, double_quantized):
    """Shapes chosen for how the small-batch family deals (tile, slab) units
    to workgroups: whole tiles written directly, partial tiles added by the
    second kernel, with bias."""
    dense = helpers.normal(65, (out_w, in_w), 0.02)
    weight = oracle.quantize(dense, block, double_quantized, 64)
    bias = helpers.normal(66, (out_w,), 0.01)
    for rows in (5, 17, 64):
        x = helpers.normal(67 + rows, (rows, in_w), 1.0)
        dy = helpers.normal(68 + rows, (rows, out_w), 1.0e-2)
        check_layer(gpu, package, library, oracle, weight, x, dy, bias=bias,
                    oracle_rows=min(rows, 5))


@pytest.mark.parametrize("out_w,in_w,block,second,double_quantized", [
    (4096, 4096, 64, 256, False),   # one tile per workgroup
    (11008, 4096, 64, 256, True),   # two or three tiles per workgroup
    (1000, 3072, 32, 32, True),     # block size 32, last tile partly empty
    (33, 2048, 128, 64, False),     # fewer tiles than compute units
    (530, 1024, 4096, 32, False),   # a quantisation block spans four rows
    (40000, 1024, 64, 64, True),    # more than eight tiles per compute unit
])
def test_resident_small_batch_family(gpu, package, library, oracle, out_w,
                                     in_w, block, second, double_quantized):
    """Up to 128 rows, in row groups of 16, with x resident in registers: row
    counts from the GEMV's to the family's limit (one to eight row groups, full
    and partly empty), with bias, against the oracle, fp64 and the other
    families (check_layer runs each that accepts the shape)."""
    dense = helpers.normal(73, (out_w, in_w), 0.02)
    dense[1] = 0.0
    weight = oracle.quantize(dense, block, double_quantized, second)
    assert library.select_algorithm(package.FORWARD, 64, in_w, out_w,
                                    block) == package.ALGORITHM_RESIDENT
    bias = helpers.normal(74, (out_w,), 0.01)
    assert library.select_algorithm(package.FORWARD, 128, in_w, out_w,
                                    block) == package.ALGORITHM_RESIDENT
    for rows in (1, 5, 16, 17, 33, 48, 64, 65, 81, 100, 128):
        x = helpers.normal(75 + rows, (rows, in_w), 1.0)
        dy = helpers.normal(76 + rows, (rows, out_w), 1.0e-2)
        check_layer(gpu, package, library, oracle, weight, x, dy, bias=bias,
                    oracle_rows=min(rows, 3))


@pytest.mark.parametrize("out_w,in_w,block,double_quantized", [
    (4096, 11008, 64, False),   # down_proj
    (300, 16384, 128, True),    # the widest row the GEMV takes
    (77, 8192 + 256, 32, True),  # just past two segments per 256 threads
])
def test_wide_rows_at_three_and_four_rows(gpu, package, library, oracle, out_w,
                                          in_w, block, double_quantized):
    """Rows wider than 8192 with three or four x rows run the GEMV with one
    512-thread team per weight row."""
    weight = oracle.quantize(helpers.normal(77, (out_w, in_w), 0.02), block,
                             double_quantized, 256)
    bias = helpers.normal(78, (out_w,), 0.01)
    for rows in (3, 4):
        assert library.select_algorithm(package.FORWARD, rows, in_w, out_w,
                                        block) == package.ALGORITHM_GEMV
        x = helpers.normal(79 + rows, (rows, in_w), 1.0)
        dy = helpers.normal(80 + rows, (rows, out_w), 1.0e-2)
        check_layer(gpu, package, library, oracle, weight, x, dy, bias=bias,
                    oracle_rows=2)


@pytest.mark.parametrize("out_w,in_w,block,double_quantized,gemv_rows", [
    (8192 // 16, 28672, 64, False, (1, 2)),  # a 70B feed-forward width
    (130, 16384 + 64, 64, True, (1, 2, 3, 4)),  # just past 4 x 256 segments
    (200, 13824, 128, True, (1, 2, 3, 4)),   # a 13B feed-forward width
    (65, 32768, 64, True, (1, 2)),           # the widest row
])
def test_rows_wider_than_12288(gpu, package, library, oracle, out_w, in_w,
                               block, double_quantized, gemv_rows):
    """Rows too wide for two 256-thread teams to hold their share in registers
    run the GEMV with one 512-thread team per weight row: two x rows from
    12289 weights on, one from 16385 to 32768.  Row counts the GEMV cannot
    hold at such a width run as two launches of fewer rows where that covers
    them (the family reported is still the GEMV), else through the
    small-batch kernel."""
    weight = oracle.quantize(helpers.normal(87, (out_w, in_w), 0.02), block,
                             double_quantized, 256)
    bias = helpers.normal(88, (out_w,), 0.01)
    for rows in (1, 2, 3, 4):
        assert (library.select_algorithm(package.FORWARD, rows, in_w, out_w,
                                         block) == package.ALGORITHM_GEMV) == \
            (rows in gemv_rows)
        x = helpers.normal(89 + rows, (rows, in_w), 1.0)
        dy = helpers.normal(90 + rows, (rows, out_w), 1.0e-2)
        check_layer(gpu, package, library, oracle, weight, x, dy, bias=bias,
                    oracle_rows=2)


@pytest.mark.parametrize("widths,in_w,block,double_quantized", [
    ((4096, 4096, 4096), 4096, 64, False),     # q/k/v
    ((11008, 11008), 4096, 64, True),          # gate/up
    ((77, 5, 1026, 33), 1040, 32, True),       # widths that end inside a batch
    ((64, 300), 8192 + 256, 128, False),       # one 512-thread team per row
    ((48, 50, 52, 54, 56, 58), 256, 64, True),  # more members than one launch
    ((130,), 512, 64, False),                  # a group of one
    ((1000, 24, 2050), 2048, 64, True),        # tile counts padded to eight
    ((9, 17, 300, 8, 130), 1024, 32, False),   # five members, x in registers
    ((520, 40), 3072, 128, True),
])
def test_group_of_weights_that_share_an_input(gpu, package, library, oracle,
                                              widths, in_w, block,
                                              double_quantized):
    """rthip_nf4_linear_forward_group against one call per member (bit for
    bit) and against the CPU oracle: up to four rows through the streaming
    kernel, five to sixty-four through the kernel that keeps x in registers
    (row widths of 1024...4096), anything else one launch per member."""
    weights = [oracle.quantize(helpers.normal(300 + m, (out_w, in_w), 0.02),
                               block, double_quantized, 256)
               for m, out_w in enumerate(widths)]
    device_weights = [upload(gpu, weight) for weight in weights]
    biases = [None if m % 2 else helpers.normal(320 + m, (out_w,), 0.01)
              for m, out_w in enumerate(widths)]
    device_biases = [None if bias is None else to_device(bias)
                     for bias in biases]
    # (65 and 68 rows: a call of its own serves the rows past 64 with the
    # streaming kernel, which a grouped launch of all rows would not)
    for rows in (1, 2, 3, 4, 7, 16, 40, 64, 65, 68, 70, 81, 128):
        x = helpers.normal(340 + rows, (rows, in_w), 1.0)
        x_device = to_device(x)
        together = gpu.linear_forward_group(x_device, device_weights,
                                            device_biases)
        for m, weight in enumerate(weights):
            alone = host(gpu.linear_forward(x_device, device_weights[m],
                                            device_biases[m]))
            helpers.assert_bit_equal(host(together[m]), alone,
                                     f"member {m} at {rows} rows")
        if rows in (1, 4, 16):
            for m in (0, len(weights) - 1):
                dense = oracle.dequantize(weights[m])
                cpu = oracle.forward(x, weights[m], biases[m])
                drift = helpers.normalized_error(
                    host(together[m]), cpu, in_w, helpers.rms(x),
                    helpers.rms(dense))
                assert drift <= 2 * TOLERANCE, \
                    f"member {m} at {rows} rows vs CPU oracle: {drift:.3g}"


@pytest.mark.parametrize("double_quantized", [False, True])
def test_launches_that_read_more_than_sixty_megabytes(gpu, package, library,
                                                      oracle,
                                                      double_quantized):
    """From 60 MB of codes per launch on, the decode kernel runs sixteen
    wavefronts per workgroup: the vocabulary projection (32000 x 4096) against
    the CPU oracle, and four 11008 x 4096 weights in one launch against one
    launch each (eight wavefronts per workgroup), bit for bit."""
    in_w = 4096
    x = helpers.normal(401, (1, in_w), 1.0)
    x_device = to_device(x)
    head = oracle.quantize(helpers.normal(400, (32000, in_w), 0.02), 64,
                           double_quantized, 256)
    y = host(gpu.linear_forward(x_device, upload(gpu, head)))
    drift = helpers.normalized_error(
        y, oracle.forward(x, head, None), in_w, helpers.rms(x),
        helpers.rms(oracle.dequantize(head)))
    # the largest deviation of 32000 outputs, not of 4096: twice the margin
    assert drift <= 2 * TOLERANCE, f"32000 x 4096 vs CPU oracle: {drift:.3g}"
    del head
    weights = [upload(gpu, oracle.quantize(
        helpers.normal(402 + m, (11008, in_w), 0.02), 64, double_quantized,
        256)) for m in range(2)]
    members = [weights[0], weights[1], weights[1], weights[0]]
    together = gpu.linear_forward_group(x_device, members)
    for m, weight in enumerate(members):
        helpers.assert_bit_equal(host(together[m]),
                                 host(gpu.linear_forward(x_device, weight)),
                                 f"member {m} of a 90 MB launch")


def test_group_arguments_are_checked(gpu, package, library, oracle):
    weight = upload(gpu, oracle.quantize(helpers.normal(1, (64, 64), 0.02),
                                         64, False, 256))
    x = to_device(helpers.normal(2, (1, 64), 1.0))
    y = to_device(np.zeros((1, 64), np.float32))
    call = library.linear_forward_group
    with pytest.raises(package.InvalidArgument):  # two members, one output
        call(x.data_ptr(), [(weight, None, y.data_ptr())] * 2, 1)
    with pytest.raises(package.InvalidArgument):  # output aliases the input
        call(x.data_ptr(), [(weight, None, x.data_ptr())], 1)
    with pytest.raises(package.InvalidArgument):
        call(x.data_ptr(), [(weight, None, 0)], 1)
    with pytest.raises(package.InvalidArgument):
        call(0, [(weight, None, y.data_ptr())], 1)
    with pytest.raises(package.InvalidArgument):
        call(x.data_ptr(), [(weight, None, y.data_ptr())], 0)


@pytest.mark.parametrize("out_w,in_w,block,second,double_quantized", [
    (4096, 4096, 64, 256, False),    # 32 column tiles x 8 chunks of rows
    (4096, 11008, 64, 256, True),    # 86 column tiles, more units than CUs
    (11008, 4096, 64, 256, True),    # chunks that end inside a 128-row walk
    (132, 1040, 32, 32, True),       # one chunk; columns end inside a tile
    (1028, 40, 4096, 32, False),     # one narrow tile, blocks span rows
    (20, 8, 32, 32, False),          # a single lane's run of columns
])
def test_small_batch_input_backward(gpu, package, library, oracle, out_w, in_w,
                                    block, second, double_quantized):
    """Up to 64 rows of dy against the packed weight walked as it lies in
    memory: one to four row groups, full and partly empty, against the oracle,
    fp64 and the other families (check_layer runs each that accepts the
    shape); and the same launch repeated, bit for bit (partial sums of row
    chunks are added in a fixed order)."""
    dense = helpers.normal(83, (out_w, in_w), 0.02)
    dense[out_w // 2] = 0.0
    weight = oracle.quantize(dense, block, double_quantized, second)
    device_weight = upload(gpu, weight)
    for rows in (1, 7, 16, 17, 40, 64):
        # (up to four rows may belong to the streaming family instead; the
        # small-batch kernel still runs them, pinned, in check_layer)
        assert library.select_algorithm(
            package.INPUT_BACKWARD, rows, in_w, out_w, block) in (
                (package.ALGORITHM_SKINNY, package.ALGORITHM_GEMV)
                if rows <= 4 else (package.ALGORITHM_SKINNY,))
        x = helpers.normal(84 + rows, (rows, in_w), 1.0)
        dy = helpers.normal(85 + rows, (rows, out_w), 1.0e-2)
        check_layer(gpu, package, library, oracle, weight, x, dy,
                    oracle_rows=min(rows, 3))
        dy_device = to_device(dy)
        first = host(gpu.linear_input_backward(dy_device, device_weight))
        for launch in range(3):
            helpers.assert_bit_equal(
                host(gpu.linear_input_backward(dy_device, device_weight)),
                first, f"{rows} rows, launch {launch}")
    # 65...96 rows run as two launches of this kernel (unless dx is much
    # wider than dy; up to 192 rows where dy is at least twice as wide as
    # dx), more rows go to the tiled kernel
    assert library.select_algorithm(
        package.INPUT_BACKWARD, 97 if out_w < 2 * in_w else 193, in_w, out_w,
        block) != package.ALGORITHM_SKINNY
    for rows in (66, 80):
        x = helpers.normal(84 + rows, (rows, in_w), 1.0)
        dy = helpers.normal(85 + rows, (rows, out_w), 1.0e-2)
        check_layer(gpu, package, library, oracle, weight, x, dy,
                    oracle_rows=2)


@pytest.mark.parametrize("out_w,in_w,block,second,double_quantized", [
    (4096, 4096, 64, 256, False),    # 4 column groups x 64 ranges of rows
    (4096, 4096, 64, 256, True),
    (4096, 11008, 64, 256, True),    # 11 column groups, the last one part empty
    (11008, 4096, 64, 256, True),    # ranges that end inside a wavefront's turn
    (11008, 4096, 64, 256, False),
    (132, 1280, 128, 32, True),      # two groups, three ranges, 33 chunks
    (1028, 8192, 4096, 32, False),   # blocks of 4096: 64 lanes share a scale
    (8, 64, 64, 32, False),          # four lanes, two chunks
    (4, 2048, 2048, 32, True),       # a single chunk
])
def test_streaming_input_backward(gpu, package, library, oracle, out_w, in_w,
                                  block, second, double_quantized):
    """One to four rows of dy against the packed weight streamed row by row,
    products on the 4x4x1 matrix instruction: against the oracle, fp64 and the
    other families, and repeated launches bit for bit (the ranges of weight
    rows are added in ascending order)."""
    dense = helpers.normal(183, (out_w, in_w), 0.02)
    dense[out_w // 2] = 0.0
    weight = oracle.quantize(dense, block, double_quantized, second)
    device_weight = upload(gpu, weight)
    for rows in (1, 2, 3, 4):
        # (three and four rows of a small weight go to the small-batch kernel;
        # check_layer still runs this family on them, pinned)
        if rows <= 2 or out_w * in_w >= 1 << 25:
            assert library.select_algorithm(
                package.INPUT_BACKWARD, rows, in_w, out_w,
                block) == package.ALGORITHM_GEMV
        x = helpers.normal(184 + rows, (rows, in_w), 1.0)
        dy = helpers.normal(185 + rows, (rows, out_w), 1.0e-2)
        check_layer(gpu, package, library, oracle, weight, x, dy)
        dy_device = to_device(dy)
        first = host(gpu.linear_input_backward(
            dy_device, device_weight, algorithm=package.ALGORITHM_GEMV))
        for launch in range(3):
            helpers.assert_bit_equal(
                host(gpu.linear_input_backward(
                    dy_device, device_weight,
                    algorithm=package.ALGORITHM_GEMV)),
                first, f"{rows} rows, launch {launch}")
    # five rows, a block size of 32, a width that is no multiple of 16: not
    # this family's
    assert library.select_algorithm(
        package.INPUT_BACKWARD, 5, in_w, out_w, block) != package.ALGORITHM_GEMV
    assert library.select_algorithm(
        package.INPUT_BACKWARD, 1, 4096, 4096, 32) != package.ALGORITHM_GEMV
    assert library.select_algorithm(
        package.INPUT_BACKWARD, 1, 4104, 4096, 64) != package.ALGORITHM_GEMV


def test_shared_output_tiles_are_added_in_a_fixed_order(gpu, package, library,
                                                        oracle):
    """When several workgroups hold parts of an output tile, the parts are
    added in ascending workgroup order whatever the timing of the launch.
    Twenty launches each at two shapes, interleaved with other work on the
    device, all bit-identical."""
    import torch
    for out_w, in_w, rows in ((1000, 4096 + 256, 40), (4096, 11008, 16)):
        weight = oracle.quantize(helpers.normal(90, (out_w, in_w), 0.02), 64,
                                 False, 256)
        device_weight = upload(gpu, weight)
        assert library.select_algorithm(
            package.FORWARD, rows, in_w, out_w, 64) == package.ALGORITHM_SKINNY
        x = to_device(helpers.normal(91, (rows, in_w), 1.0))
        first = host(gpu.linear_forward(x, device_weight))
        filler = torch.zeros(1 << 22, device="cuda")
        for launch in range(20):
            if launch % 3 == 0:
                filler.add_(1.0)      # something else in flight before it
            helpers.assert_bit_equal(
                host(gpu.linear_forward(x, device_weight)), first,
                f"launch {launch}")


def test_two_host_threads_launch_on_one_stream(gpu, package, library, oracle):
    """Kernels that hand partial results to a second kernel through the
    stream's scratch buffer (the small-batch forward and input backward, the
    tiled kernel's leftover tiles, the streaming and the shape-agnostic input
    backward, the adapter's d_reduced, the input backward that keeps its partial
    sums in the library's static array) are launched from two host threads at once
    on the same stream, each thread with its own input: a thread's sum kernel
    must never read the other thread's partial results.  Every output equals,
    bit for bit, the one the same call gives alone."""
    import threading
    import torch
    stream = torch.cuda.current_stream().cuda_stream
    cases = [  # (out_w, in_w, rows, direction)
        (4096, 11008, 16, "forward"),     # small batch, partial tiles
        (11008, 4096, 16, "backward"),    # row chunks
        (1000, 4096 + 256, 40, "forward"),
        (11008, 4096, 300, "forward"),    # tiled kernel, leftover tiles
        (11008, 4096, 1, "backward"),     # streamed weight, row ranges
        (1001, 4095, 3, "backward"),      # shape-agnostic kernel, row chunks
        (4096, 1024, 12, "adapter"),      # d_reduced in column slices
        (4096, 1024, 64, "no_alloc"),     # row chunks in the static array
    ]
    for out_w, in_w, rows, direction in cases:
        weight = oracle.quantize(helpers.normal(95, (out_w, in_w), 0.02), 64,
                                 False, 256)
        device_weight = upload(gpu, weight)
        width = in_w if direction == "forward" else out_w
        other = {"forward": out_w, "backward": in_w, "adapter": 8,
                 "no_alloc": in_w}[direction]
        inputs = [to_device(helpers.normal(96 + t, (rows, width), 1.0))
                  for t in range(2)]

        if direction == "adapter":
            rank = 8
            lora_b = to_device(helpers.normal(98, (out_w, rank), 0.05))

        def call(source, target):
            if direction == "adapter":
                # target: d_reduced [rows, rank] (source: dy [rows, out_w])
                library.lora_backward(source.data_ptr(), None, None,
                                      lora_b.data_ptr(), rank, 2.0,
                                      target.data_ptr(), None, None, rows,
                                      in_w, out_w, stream)
            elif direction == "forward":
                library.linear_forward(source.data_ptr(), device_weight, None,
                                       target.data_ptr(), rows, stream)
            elif direction == "no_alloc":
                library.linear_input_backward_no_alloc(
                    source.data_ptr(), device_weight, target.data_ptr(), rows,
                    stream)
            else:
                library.linear_input_backward(source.data_ptr(),
                                              device_weight,
                                              target.data_ptr(), rows, stream)

        expected = []
        for source in inputs:
            target = torch.empty(rows, other, device="cuda")
            call(source, target)
            expected.append(host(target))
        outputs = [[torch.empty(rows, other, device="cuda")
                    for _ in range(40)] for _ in range(2)]
        start = threading.Barrier(2)
        failures = []

        def worker(index):
            try:
                start.wait()
                for target in outputs[index]:
                    call(inputs[index], target)
            except Exception as error:  # noqa: BLE001
                failures.append(error)

        threads = [threading.Thread(target=worker, args=(t,))
                   for t in range(2)]
        for thread in threads:
            thread.start()
        for thread in threads:
            thread.join()
        assert not failures, failures
        torch.cuda.synchronize()
        for index in range(2):
            for launch, target in enumerate(outputs[index]):
                helpers.assert_bit_equal(
                    host(target), expected[index],
                    f"{direction} {out_w}x{in_w}, thread {index}, "
                    f"launch {launch}")


@pytest.mark.parametrize("rows,out_w,in_w,double_quantized", [
    (300, 1000, 1024, False),   # 24 tiles, each cut into four runs
    (130, 260, 1056, True),     # 6 tiles, runs of 8 and 9 steps
    (1280, 2560, 4096, True),   # 200 tiles dealt to 512 workgroups
    (2200, 3700, 512, False),   # 522 tiles: 512 whole, 10 cut into runs
    (200, 384, 256, False),     # too few steps: whole tiles only
    # forward in 256-row tiles (their count fills the device in whole rounds)
    (448, 16384, 96, True),     # the second tile row three quarters full
    (256, 32768, 64, False),    # one tile row, two steps
])
def test_gemm_leftover_tiles_are_dealt_in_units(gpu, package, library, oracle,
                                                rows, out_w, in_w,
                                                double_quantized):
    """Tile counts that do not fill the device evenly: the leftover tiles are
    cut along the contraction, partial tiles are added by a second kernel.
    Both directions, with bias, ragged edges in every dimension."""
    weight = oracle.quantize(helpers.normal(95, (out_w, in_w), 0.02), 64,
                             double_quantized, 256)
    assert library.select_algorithm(package.FORWARD, rows, in_w, out_w,
                                    64) == package.ALGORITHM_MFMA
    x = helpers.normal(96, (rows, in_w), 1.0)
    dy = helpers.normal(97, (rows, out_w), 1.0e-2)
    bias = helpers.normal(98, (out_w,), 0.01)
    check_layer(gpu, package, library, oracle, weight, x, dy, bias=bias,
                oracle_rows=2)
    # the same launch again gives the same bits
    device_weight = upload(gpu, weight)
    first = host(gpu.linear_forward(to_device(x), device_weight))
    for _ in range(3):
        helpers.assert_bit_equal(
            host(gpu.linear_forward(to_device(x), device_weight)), first)


@pytest.mark.parametrize("out_w,in_w", [(4096, 4096), (11008, 4096),
                                        (4096, 11008)])
@pytest.mark.parametrize("double_quantized", [False, True])
def test_small_batches_at_the_llama_shapes(gpu, package, library, oracle,
                                           out_w, in_w, double_quantized):
    """The small-batch decode configuration at full size: M in {4, 16, 64} on
    the three distinct Llama-7B projection shapes, both scale encodings; every
    family that takes the shape, every output against fp64, two rows against
    the CPU oracle."""
    weight = oracle.quantize(helpers.normal(99, (out_w, in_w), 0.02), 64,
                             double_quantized, 256)
    for rows in (4, 16, 64):
        x = helpers.normal(100 + rows, (rows, in_w), 1.0)
        dy = helpers.normal(101 + rows, (rows, out_w), 1.0e-2)
        check_layer(gpu, package, library, oracle, weight, x, dy,
                    oracle_rows=2)


def test_long_runs_of_the_small_batch_forward_are_summed_in_two_levels(
        gpu, package, library, oracle):
    """A 70B feed-forward weight (8192 x 28672) at 33 and 64 rows: 64 output
    tiles x 112 slabs over 256 workgroups are runs of 28 slabs, 7168
    contraction values per accumulator.  One fp32 chain of that length drifts
    1.0-1.6e-5 of an output's K-normalised scale, beyond the bar; the kernel
    folds its matrix sums into a second accumulator after every slab."""
    import torch
    out_w, in_w = 8192, 28672
    weight = oracle.quantize(helpers.normal(120, (out_w, in_w), 0.02), 64,
                             True, 256)
    device_weight = upload(gpu, weight)
    deq = gpu.dequantize(device_weight)
    weight_rms = float(deq.double().pow(2).mean().sqrt())
    for rows in (33, 64):
        assert library.select_algorithm(package.FORWARD, rows, in_w, out_w,
                                        64) == package.ALGORITHM_SKINNY
        x = helpers.normal(121 + rows, (rows, in_w), 1.0)
        x_device = to_device(x)
        y = gpu.linear_forward(x_device, device_weight)
        exact = x_device.double() @ deq.double().T
        scale = np.sqrt(in_w) * helpers.rms(x) * weight_rms
        error = float((y.double() - exact).abs().max()) / scale
        assert error <= TOLERANCE, f"{rows} rows vs fp64: {error:.3g}"
        cpu = oracle.forward(x[:2], weight)
        cpu_error = helpers.normalized_error(
            cpu, host(exact)[:2], in_w, helpers.rms(x), weight_rms)
        drift = helpers.normalized_error(host(y)[:2], cpu, in_w,
                                         helpers.rms(x), weight_rms)
        assert drift <= TOLERANCE + cpu_error
        del exact, y
    torch.cuda.empty_cache()


def test_zero_scale_blocks_and_saturated_scales(gpu, package, library,
                                                oracle):
    dense = helpers.normal(70, (64, 128), 0.02)
    dense[5] = 0.0          # zero blocks: scale 0, code 7
    dense[9, :64] = 0.0
    for dq in (False, True):
        weight = oracle.quantize(dense, 64, dq, 32)
        x = helpers.normal(71, (4, 128), 1.0)
        dy = helpers.normal(72, (4, 64), 1.0e-2)
        check_layer(gpu, package, library, oracle, weight, x, dy)


# ---- full-size properties -----------------------------------------------

@pytest.mark.parametrize("out_w,in_w,double_quantized", [
    (11008, 4096, False), (11008, 4096, True), (4096, 4096, False),
    (4096, 4096, True), (4096, 11008, True)])
def test_prefill_shapes_at_full_size(gpu, package, library, oracle, out_w,
                                     in_w, double_quantized):
    """M = 2048 at the Llama-7B layer shapes.  Size-independent checks: every output
    against an fp64 product over the bit-exact deq(W) (computed on the device
    by the vendor BLAS, an independent path), 32 seeded rows against the CPU
    oracle, and linearity y(a*x1 + x2) = a*y(x1) + y(x2) for a power of two."""
    import torch
    rows = 2048
    dense = helpers.normal(80, (out_w, in_w), 0.02)
    weight = oracle.quantize(dense, 64, double_quantized, 256)
    device_weight = upload(gpu, weight)
    deq = gpu.dequantize(device_weight)
    helpers.assert_bit_equal(host(deq), oracle.dequantize(weight), "deq(W)")
    weight_rms = helpers.rms(host(deq))
    picked = np.sort(np.random.default_rng(81).choice(rows, 32, replace=False))

    x = helpers.normal(82, (rows, in_w), 1.0)
    x_device = to_device(x)
    y = gpu.linear_forward(x_device, device_weight)
    exact = (x_device.double() @ deq.double().T)
    scale = np.sqrt(in_w) * helpers.rms(x) * weight_rms
    error = float((y.double() - exact).abs().max()) / scale
    assert error <= TOLERANCE, f"forward vs fp64: {error:.3g}"
    cpu = oracle.forward(x[picked], weight)
    cpu_error = helpers.normalized_error(
        cpu, host(exact)[picked], in_w, helpers.rms(x), weight_rms)
    drift = helpers.normalized_error(host(y)[picked], cpu, in_w,
                                     helpers.rms(x), weight_rms)
    assert drift <= TOLERANCE + cpu_error
    y2 = gpu.linear_forward(x_device * 4.0, device_weight)
    assert torch.equal(y2, y * 4.0), "scaling x by 4 must scale y exactly"
    del exact, y2

    dy = helpers.normal(83, (rows, out_w), 1.0e-2)
    dy_device = to_device(dy)
    dx = gpu.linear_input_backward(dy_device, device_weight)
    exact = (dy_device.double() @ deq.double())
    scale = np.sqrt(out_w) * helpers.rms(dy) * weight_rms
    error = float((dx.double() - exact).abs().max()) / scale
    assert error <= TOLERANCE, f"backward vs fp64: {error:.3g}"
    cpu = oracle.input_backward(dy[picked], weight)
    cpu_error = helpers.normalized_error(
        cpu, host(exact)[picked], out_w, helpers.rms(dy), weight_rms)
    drift = helpers.normalized_error(host(dx)[picked], cpu, out_w,
                                     helpers.rms(dy), weight_rms)
    assert drift <= TOLERANCE + cpu_error
    # <dy, y(x)> == <dx(dy), x>: the two kernels are adjoint to each other.
    # Both sides are sums of rows*width rounded products whose signs are
    # random, so the sums themselves are far smaller than the terms' total
    # magnitude and "relative to the sum" is no measure of the kernels.  The
    # rounding of y (at most TOLERANCE x its K-normalised scale per output,
    # checked above) moves <dy, y> by about TOLERANCE * scale_y * |dy|_2 when
    # the roundings are independent; likewise dx.  A transposed operand or a
    # dropped block changes a side by the size of a typical sum,
    # |dy|_2 * scale_y: 1 / (2 * TOLERANCE) times this bound.
    lhs = float((dy_device.double() * y.double()).sum())
    rhs = float((dx.double() * x_device.double()).sum())
    scale_y = np.sqrt(in_w) * helpers.rms(x) * weight_rms
    scale_dx = np.sqrt(out_w) * helpers.rms(dy) * weight_rms
    bound = TOLERANCE * (scale_y * float(np.linalg.norm(dy.ravel().astype(np.float64)))
                         + scale_dx * float(np.linalg.norm(x.ravel().astype(np.float64))))
    assert abs(lhs - rhs) <= bound


@pytest.mark.parametrize("out_w,in_w,double_quantized", [
    (11008, 4096, True), (4096, 11008, False)])
def test_adapter_step_at_full_size(gpu, package, library, oracle, out_w, in_w,
                                   double_quantized):
    """One training step of a layer with a rank-16 adapter at M = 2048: the
    fused forward and the backward (dx, dA, dB) against fp64 products over the
    bit-exact deq(W) computed on the device by the vendor BLAS, and a property
    that needs no reference: for a direction (U, V) in the space of (A, B),
    <dy, y(A + hU, B + hV) - y(A - hU, B - hV)> / 2h = <dA, U> + <dB, V>
    exactly (y is bilinear in (A, B), so the central difference has no
    truncation error; what is left is the rounding of the two forward
    passes)."""
    import torch
    rows, rank, scale = 2048, 16, 2.0
    dense = helpers.normal(190, (out_w, in_w), 0.02)
    weight = oracle.quantize(dense, 64, double_quantized, 256)
    device_weight = upload(gpu, weight)
    deq = gpu.dequantize(device_weight).double()
    x = to_device(helpers.normal(191, (rows, in_w), 1.0))
    dy = to_device(helpers.normal(192, (rows, out_w), 1.0e-2))
    lora_a = to_device(helpers.normal(193, (rank, in_w), 0.05))
    lora_b = to_device(helpers.normal(194, (out_w, rank), 0.05))
    y, reduced = gpu.lora_linear_forward(x, device_weight, lora_a, lora_b,
                                         scale)
    dx, d_a, d_b = gpu.lora_linear_backward(dy, x, device_weight, lora_a,
                                            lora_b, scale, reduced)
    x64, dy64 = x.double(), dy.double()
    a64, b64 = lora_a.double(), lora_b.double()
    reduced64 = x64 @ a64.T
    through_b = scale * (dy64 @ b64)
    for what, got, exact in (
            ("y", y, x64 @ deq.T + scale * (reduced64 @ b64.T)),
            ("dx", dx, dy64 @ deq + through_b @ a64),
            ("dA", d_a, through_b.T @ x64),
            ("dB", d_b, scale * (dy64.T @ reduced64))):
        unit = float(exact.pow(2).mean().sqrt())
        error = float((got.double() - exact).abs().max()) / unit
        assert error <= TOLERANCE, f"{what} vs fp64: {error:.3g}"
        del exact
    # directional derivative of <dy, y> in (A, B), central difference in fp64
    # arithmetic on the fp32 outputs of the forward kernel
    u = to_device(helpers.normal(195, (rank, in_w), 0.05))
    v = to_device(helpers.normal(196, (out_w, rank), 0.05))
    step = 2.0 ** -6

    def objective(sign):
        shifted, _ = gpu.lora_linear_forward(
            x, device_weight, lora_a + sign * step * u,
            lora_b + sign * step * v, scale)
        return float((dy64 * shifted.double()).sum())

    slope = (objective(1.0) - objective(-1.0)) / (2.0 * step)
    predicted = float((d_a.double() * u.double()).sum() +
                      (d_b.double() * v.double()).sum())
    # the rounding of y in the two forward passes: at most TOLERANCE of an
    # output's size per output, signs independent, over 2h
    y_unit = float(y.double().pow(2).mean().sqrt())
    noise = TOLERANCE * y_unit * float(dy64.norm()) / step
    assert abs(predicted) > 100 * noise      # the check has teeth
    assert abs(slope - predicted) <= noise, \
        f"slope {slope:.6g} vs <dA,U>+<dB,V> {predicted:.6g}, " \
        f"allowed {noise:.3g}"


def test_decode_shapes_small_batches(gpu, package, library, oracle):
    """M in {1, 4, 16, 64} on the three distinct Llama-7B shapes."""
    for name, (out_w, in_w) in (("q_proj", (4096, 4096)),
                                ("gate_proj", (11008, 4096)),
                                ("down_proj", (4096, 11008))):
        dense = helpers.normal(90, (out_w, in_w), 0.02)
        weight = oracle.quantize(dense, 64)
        for rows in (1, 4, 16, 64):
            x = helpers.normal(91 + rows, (rows, in_w), 1.0)
            dy = helpers.normal(92 + rows, (rows, out_w), 1.0e-2)
            check_layer(gpu, package, library, oracle, weight, x, dy,
                        oracle_rows=min(rows, 4))


# ---- the fused bias + low-rank adapter epilogue ---------------------------

@pytest.mark.parametrize("out_w,in_w,block,rank,row_counts", [
    (768, 256, 64, 8, (1, 16)),         # the tiny parity layer
    (33, 33, 32, 1, (2,)),              # shape-agnostic kernels, rank one
    (1000, 1600, 64, 2, (1, 5, 70)),    # rank that is not a multiple of 4
    (4096, 4096, 64, 16, (1, 4, 64, 70, 100, 150, 300)),  # 70, 150: two launches
    (512, 2048, 128, 100, (3, 40)),     # more than one 64-row adapter chunk
])
@pytest.mark.parametrize("double_quantized", [False, True])
def test_lora_linear_forward(gpu, package, library, oracle, out_w, in_w,
                             block, rank, row_counts, double_quantized):
    """y = x.deq(W)^T + b + s.(x.A^T).B^T against the oracle's restatement of
    the reference's composition and against fp64; every kernel family.
    Tolerance: 1e-5 of an output's standard deviation (and the oracle's own
    distance from fp64 on top, for the comparison with the oracle)."""
    dense = helpers.normal(100, (out_w, in_w), 0.02)
    weight = oracle.quantize(dense, block, double_quantized, 64)
    device_weight = upload(gpu, weight)
    deq = oracle.dequantize(weight).astype(np.float64)
    lora_a = helpers.normal(101, (rank, in_w), 0.05)
    lora_b = helpers.normal(102, (out_w, rank), 0.05)
    bias = helpers.normal(103, (out_w,), 0.01)
    lora_scale = 16.0 / rank
    for rows in row_counts:
        x = helpers.normal(104 + rows, (rows, in_w), 1.0)
        x64 = x.astype(np.float64)
        exact_reduced = x64 @ lora_a.astype(np.float64).T
        exact = (x64 @ deq.T + bias.astype(np.float64)[None, :] +
                 lora_scale * (exact_reduced @ lora_b.astype(np.float64).T))
        unit = helpers.rms(exact)
        sample = slice(0, min(rows, 5))
        cpu = oracle.lora_forward(x[sample], weight, lora_a, lora_b,
                                  lora_scale, bias)
        cpu_error = np.abs(cpu - exact[sample]).max() / unit
        for family in families(package):
            try:
                y, reduced = gpu.lora_linear_forward(
                    to_device(x), device_weight, to_device(lora_a),
                    to_device(lora_b), lora_scale, bias=to_device(bias),
                    algorithm=family)
            except package.Unsupported:
                assert family is not None
                continue
            y, reduced = host(y), host(reduced)
            name = package.ALGORITHM_NAMES[family or 0]
            reduced_error = np.abs(reduced - exact_reduced).max() / \
                helpers.rms(exact_reduced)
            assert reduced_error <= TOLERANCE, \
                f"x.A^T/{name} rows={rows}: {reduced_error:.3g}"
            error = np.abs(y - exact).max() / unit
            assert error <= TOLERANCE, \
                f"lora forward/{name} rows={rows} vs fp64: {error:.3g}"
            drift = np.abs(y[sample] - cpu).max() / unit
            assert drift <= TOLERANCE + cpu_error, \
                f"lora forward/{name} rows={rows} vs oracle: {drift:.3g}"


def adapter_backward_exact(dy, x, deq, lora_a, lora_b, lora_scale):
    """fp64: (dx, dA, dB, d_reduced) of y = x deq^T + s (x A^T) B^T."""
    dy64, x64 = dy.astype(np.float64), x.astype(np.float64)
    a64, b64 = lora_a.astype(np.float64), lora_b.astype(np.float64)
    through_b = lora_scale * (dy64 @ b64)
    return (dy64 @ deq + through_b @ a64, through_b.T @ x64,
            lora_scale * dy64.T @ (x64 @ a64.T), through_b)


@pytest.mark.parametrize("out_w,in_w,block,rank,row_counts", [
    (768, 256, 64, 8, (1, 16)),         # the tiny parity layer
    (33, 33, 32, 1, (2,)),              # shape-agnostic kernels, rank one
    (1000, 1600, 64, 2, (1, 5, 70)),    # rank that is not a multiple of 4
    (4096, 4096, 64, 16, (1, 3, 64, 80, 300)),  # 80: two launches
    (512, 2048, 128, 100, (3, 40)),     # more than one chunk of the rank
    (4096, 11008, 64, 24, (2, 17)),     # dx wider than dy, rank 24
    (2304, 1024, 64, 8, (100, 150)),    # dy much wider: three launches at 150
])
@pytest.mark.parametrize("double_quantized", [False, True])
def test_lora_linear_backward(gpu, package, library, oracle, out_w, in_w,
                              block, rank, row_counts, double_quantized):
    """dx = dy.deq(W) + ((dy s).B).A, dA and dB through rthip_lora_backward
    and rthip_nf4_lora_linear_input_backward, every input-backward family,
    against fp64 and (where the CPU finishes in seconds) against the oracle's
    restatement of the reference's autograd.  Tolerance: 1e-5 of the standard
    deviation of each gradient (plus the oracle's own distance from fp64 for
    the comparison with the oracle)."""
    import torch
    dense = helpers.normal(170, (out_w, in_w), 0.02)
    weight = oracle.quantize(dense, block, double_quantized, 64)
    device_weight = upload(gpu, weight)
    deq = oracle.dequantize(weight).astype(np.float64)
    lora_a = helpers.normal(171, (rank, in_w), 0.05)
    lora_b = helpers.normal(172, (out_w, rank), 0.05)
    lora_scale = 16.0 / rank
    a_device, b_device = to_device(lora_a), to_device(lora_b)
    for rows in row_counts:
        x = helpers.normal(173 + rows, (rows, in_w), 1.0)
        dy = helpers.normal(174 + rows, (rows, out_w), 1.0e-2)
        exact = adapter_backward_exact(dy, x, deq, lora_a, lora_b, lora_scale)
        units = [helpers.rms(value) for value in exact]
        cpu = None
        if rows * out_w * in_w <= 3.0e8:
            cpu = oracle.lora_backward(dy, x, weight, lora_a, lora_b,
                                       lora_scale)
        x_device, dy_device = to_device(x), to_device(dy)
        reduced = torch.empty((rows, rank), device="cuda")
        library.lora_reduce(x_device.data_ptr(), a_device.data_ptr(),
                            reduced.data_ptr(), rows, in_w, rank)
        ran = 0
        for family in families(package):
            try:
                got = gpu.lora_linear_backward(
                    dy_device, x_device, device_weight, a_device, b_device,
                    lora_scale, reduced, algorithm=family)
            except package.Unsupported:
                assert family is not None
                continue
            ran += 1
            got = [host(value) for value in got]
            name = package.ALGORITHM_NAMES[family or 0]
            for index, what in enumerate(("dx", "dA", "dB")):
                error = np.abs(got[index] - exact[index]).max() / units[index]
                assert error <= TOLERANCE, \
                    f"{what}/{name} rows={rows} vs fp64: {error:.3g}"
                if cpu is not None:
                    cpu_error = np.abs(cpu[index] - exact[index]).max() / \
                        units[index]
                    drift = np.abs(got[index] - cpu[index]).max() / \
                        units[index]
                    assert drift <= TOLERANCE + cpu_error, \
                        f"{what}/{name} rows={rows} vs oracle: {drift:.3g}"
        assert ran >= 2   # AUTO and at least the shape-agnostic family


def test_lora_backward_pieces_and_repeat_launches(gpu, package, library,
                                                  oracle):
    """d_reduced alone (no buffers for dA and dB), the gradients of a second
    call bit-equal to the first, and an adapter with B = 0 (a fresh adapter):
    dA and the adapter's share of dx vanish, dx equals the plain backward."""
    import torch
    rows, out_w, in_w, rank, scale = 12, 1536, 1024, 16, 2.0
    weight = oracle.quantize(helpers.normal(180, (out_w, in_w), 0.02), 64)
    device_weight = upload(gpu, weight)
    x = to_device(helpers.normal(181, (rows, in_w), 1.0))
    dy_host = helpers.normal(182, (rows, out_w), 1.0e-2)
    dy = to_device(dy_host)
    lora_a = to_device(helpers.normal(183, (rank, in_w), 0.05))
    lora_b_host = helpers.normal(184, (out_w, rank), 0.05)
    lora_b = to_device(lora_b_host)
    reduced = torch.empty((rows, rank), device="cuda")
    library.lora_reduce(x.data_ptr(), lora_a.data_ptr(), reduced.data_ptr(),
                        rows, in_w, rank)
    d_reduced = torch.full((rows, rank), 7.0, device="cuda")
    library.lora_backward(dy.data_ptr(), None, None, lora_b.data_ptr(), rank,
                          scale, d_reduced.data_ptr(), None, None, rows,
                          in_w, out_w)
    exact = scale * (dy_host.astype(np.float64) @
                     lora_b_host.astype(np.float64))
    assert np.abs(host(d_reduced) - exact).max() / helpers.rms(exact) \
        <= TOLERANCE
    first = [host(value) for value in gpu.lora_linear_backward(
        dy, x, device_weight, lora_a, lora_b, scale, reduced)]
    second = [host(value) for value in gpu.lora_linear_backward(
        dy, x, device_weight, lora_a, lora_b, scale, reduced)]
    for one, two in zip(first, second):
        helpers.assert_bit_equal(one, two)
    zero_b = torch.zeros_like(lora_b)
    dx, d_a, d_b = gpu.lora_linear_backward(dy, x, device_weight, lora_a,
                                            zero_b, scale, reduced)
    assert not host(d_a).any()
    assert host(d_b).any()
    helpers.assert_bit_equal(host(dx),
                             host(gpu.linear_input_backward(dy,
                                                            device_weight)))


def test_lora_forward_with_a_precomputed_first_product(gpu, package, library,
                                                       oracle):
    """One rthip_lora_reduce over the stacked A matrices of two projections
    that share x, then two forwards that take their slice of the result."""
    import torch
    rows, in_w, rank = 3, 1024, 8
    x = to_device(helpers.normal(120, (rows, in_w), 1.0))
    stacked_a = to_device(helpers.normal(121, (2 * rank, in_w), 0.05))
    reduced = torch.empty((rows, 2 * rank), dtype=torch.float32,
                          device="cuda")
    library.lora_reduce(x.data_ptr(), stacked_a.data_ptr(),
                        reduced.data_ptr(), rows, in_w, 2 * rank,
                        torch.cuda.current_stream().cuda_stream)
    for index, out_w in enumerate((256, 640)):
        dense = helpers.normal(122 + index, (out_w, in_w), 0.02)
        weight = oracle.quantize(dense, 64)
        device_weight = upload(gpu, weight)
        lora_a = stacked_a[index * rank:(index + 1) * rank].contiguous()
        lora_b = to_device(helpers.normal(124 + index, (out_w, rank), 0.05))
        mine = reduced[:, index * rank:(index + 1) * rank].contiguous()
        want, want_reduced = gpu.lora_linear_forward(
            x, device_weight, lora_a, lora_b, 2.0)
        helpers.assert_bit_equal(host(mine), host(want_reduced))
        got = torch.empty_like(want)
        library.lora_linear_forward(
            x.data_ptr(), device_weight, None, None, lora_b.data_ptr(), rank,
            2.0, mine.data_ptr(), got.data_ptr(), rows,
            torch.cuda.current_stream().cuda_stream)
        helpers.assert_bit_equal(host(got), host(want))


def test_lora_with_zero_b_equals_the_plain_forward(gpu, package, library,
                                                   oracle):
    """A freshly attached adapter (B = 0) leaves the output bit-identical to
    the plain kernel's."""
    dense = helpers.normal(110, (4096, 4096), 0.02)
    weight = oracle.quantize(dense, 64)
    device_weight = upload(gpu, weight)
    lora_a = to_device(helpers.normal(111, (16, 4096), 0.05))
    lora_b = to_device(np.zeros((4096, 16), dtype=np.float32))
    for rows in (1, 16, 200):
        x = to_device(helpers.normal(112 + rows, (rows, 4096), 1.0))
        plain = host(gpu.linear_forward(x, device_weight))
        fused, _ = gpu.lora_linear_forward(x, device_weight, lora_a, lora_b,
                                           1.0)
        helpers.assert_bit_equal(host(fused), plain)


# ---- dense fp32 matmul ----------------------------------------------------

@pytest.mark.parametrize("batch,rows,shared,columns", [
    (1, 2, 3, 2),           # tests/core: tiny, plain kernel
    (1, 5, 33, 7),          # nothing aligned: plain kernel
    (3, 40, 64, 48),        # batched
    (1, 300, 16, 4096),     # adapter second product: K = rank
    (1, 70, 4096, 16),      # adapter first product: N = rank
    (1, 16, 300, 1000),     # gradient shape: rows = rank
    (2, 129, 100, 132),     # every edge of the tile
    (1, 512, 2048, 1024),
    (1, 200, 1000, 260),    # sliced contraction, last slice ends mid-step
    (1, 2048, 4096, 16),    # sliced contraction, many row tiles
    (1, 1280, 1024, 2560),  # 200 tiles dealt in runs to 512 workgroups
    (1, 2200, 520, 3700),   # 522 tiles: 512 whole, 10 dealt; ragged edges
    (2, 1280, 256, 1300),   # batched: whole tiles only
])
def test_dense_matmul(gpu, package, library, oracle, batch, rows, shared,
                      columns):
    """rthip_matmul against the oracle's restatement of the reference loop and
    against fp64; tolerance 1e-5 of an output's standard deviation (plus the
    oracle's own distance from fp64 for the comparison with the oracle)."""
    left = helpers.normal(130, (batch, rows, shared), 1.0)
    right = helpers.normal(131, (batch, shared, columns), 0.05)
    got = host(gpu.matmul(to_device(left), to_device(right)))
    assert got.shape == (batch, rows, columns)
    for index in range(batch):
        exact = left[index].astype(np.float64) @ \
            right[index].astype(np.float64)
        unit = helpers.rms(exact)
        error = np.abs(got[index] - exact).max() / unit
        assert error <= TOLERANCE, f"matmul vs fp64: {error:.3g}"
        sample = slice(0, min(rows, 8))
        cpu = oracle.matmul(left[index][sample], right[index])
        cpu_error = np.abs(cpu - exact[sample]).max() / unit
        drift = np.abs(got[index][sample] - cpu).max() / unit
        assert drift <= TOLERANCE + cpu_error, f"matmul vs oracle: {drift:.3g}"


def test_sliced_matmul_is_deterministic(gpu, package, library):
    """A sliced contraction adds its partial results in a fixed order."""
    left = to_device(helpers.normal(132, (1, 70, 4096), 1.0))
    right = to_device(helpers.normal(133, (1, 4096, 16), 0.05))
    first = host(gpu.matmul(left, right))
    for _ in range(3):
        helpers.assert_bit_equal(host(gpu.matmul(left, right)), first)


def test_dense_matmul_small_integers_are_exact(gpu, package, library):
    left = np.arange(12, dtype=np.float32).reshape(1, 3, 4) - 5.0
    right = np.arange(20, dtype=np.float32).reshape(1, 4, 5) - 9.0
    got = host(gpu.matmul(to_device(left), to_device(right)))
    assert np.array_equal(got[0], left[0] @ right[0])


# ---- the quantizer on the device ------------------------------------------

def payload_of(device_weight):
    import torch
    torch.cuda.synchronize()
    return (device_weight.codes.cpu().numpy(),
            device_weight.primary_scales.cpu().numpy(),
            None if device_weight.secondary_scales is None
            else device_weight.secondary_scales.cpu().numpy(),
            np.float32(device_weight.offset))


@pytest.mark.parametrize("shape,block,second", [
    ((768, 256), 64, 256), ((33, 33), 32, 32), ((17, 96), 32, 64),
    ((5, 4096), 4096, 32), ((64, 1000), 128, 32), ((1, 1), 32, 32),
    ((4096, 4096), 64, 256), ((1000, 11008), 64, 256)])
@pytest.mark.parametrize("double_quantized", [False, True])
@pytest.mark.parametrize("sigma", [0.02, 1.0])
def test_device_quantizer_is_bit_exact(gpu, package, library, oracle, shape,
                                       block, second, double_quantized,
                                       sigma):
    """Codes, block scales, scale codes, second-level scales and the offset
    must equal the oracle's (which is pinned to the compiled reference)."""
    dense = helpers.normal(140, shape, sigma)
    dense.ravel()[::7] = 0.0   # exact zeros: ties at code 7
    if dense.shape[0] > 8:
        dense[3] = 0.0         # a whole zero block or more
    want = oracle.quantize(dense, block, double_quantized, second)
    got = gpu.quantize_weight(to_device(dense), block, double_quantized,
                              second)
    codes, primary, secondary, offset = payload_of(got)
    assert np.array_equal(codes, want.codes)
    if not double_quantized:
        helpers.assert_bit_equal(primary, want.fp32_scales)
    else:
        assert np.array_equal(primary, want.scale_codes)
        helpers.assert_bit_equal(secondary, want.second_level)
        helpers.assert_bit_equal(offset, np.float32(want.offset))


def test_device_quantizer_scale_mean_with_a_wide_exponent_range(
        gpu, package, library, oracle):
    """Scales that span 2^40: the double sum is then order-dependent and the
    device must add in index order like the reference."""
    rng = np.random.default_rng(141)
    blocks = 5000
    magnitudes = (2.0 ** rng.integers(-30, 10, blocks)) * \
        (1.0 + rng.random(blocks))
    dense = np.zeros((blocks, 32), dtype=np.float32)
    dense[:, 0] = magnitudes.astype(np.float32)
    dense[:, 1:] = (dense[:, :1] *
                    rng.uniform(-1, 1, (blocks, 31))).astype(np.float32)
    want = oracle.quantize(dense, 32, True, 64)
    got = gpu.quantize_weight(to_device(dense), 32, True, 64)
    codes, primary, secondary, offset = payload_of(got)
    assert np.array_equal(codes, want.codes)
    assert np.array_equal(primary, want.scale_codes)
    helpers.assert_bit_equal(secondary, want.second_level)
    helpers.assert_bit_equal(offset, np.float32(want.offset))


def test_device_quantizer_rejects_non_finite_values(gpu, package, library):
    dense = helpers.normal(142, (64, 64), 0.02)
    dense[10, 3] = np.inf
    with pytest.raises(package.InvalidArgument) as error:
        gpu.quantize_weight(to_device(dense), 64)
    assert "finite" in error.value.message
    dense[10, 3] = np.nan
    with pytest.raises(package.InvalidArgument):
        gpu.quantize_weight(to_device(dense), 64, True, 32)


def test_quantize_then_multiply_on_the_device(gpu, package, library, oracle):
    """The device quantizer feeds the kernels directly."""
    dense = helpers.normal(143, (512, 1024), 0.02)
    weight = gpu.quantize_weight(to_device(dense), 64, True, 256)
    host_weight = oracle.quantize(dense, 64, True, 256)
    helpers.assert_bit_equal(host(gpu.dequantize(weight)),
                             oracle.dequantize(host_weight))
    x = helpers.normal(144, (3, 1024), 1.0)
    y = host(gpu.linear_forward(to_device(x), weight))
    exact = helpers.exact_forward(x, oracle.dequantize(host_weight))
    error = helpers.normalized_error(
        y, exact, 1024, helpers.rms(x),
        helpers.rms(oracle.dequantize(host_weight)))
    assert error <= TOLERANCE


# ---- the ABI's error behaviour on a live device --------------------------

def test_abi_rejects_bad_arguments(gpu, package, library, oracle):
    import torch
    weight = oracle.quantize(helpers.normal(95, (64, 64), 0.02), 64)
    device_weight = upload(gpu, weight)
    x = torch.zeros(64, device="cuda")
    y = torch.zeros(64, device="cuda")
    with pytest.raises(package.InvalidArgument):
        library.linear_forward(x.data_ptr(), device_weight, None,
                               x.data_ptr(), 1)           # aliasing
    with pytest.raises(package.InvalidArgument):
        library.linear_forward(0, device_weight, None, y.data_ptr(), 1)
    with pytest.raises(package.InvalidArgument):
        library.linear_forward(x.data_ptr(), device_weight, None,
                               y.data_ptr(), 0)           # zero rows
    bad = package.DeviceWeight(64, 64, 48, 0, device_weight.codes,
                               device_weight.primary_scales, None)
    with pytest.raises(package.InvalidArgument):
        library.linear_forward(x.data_ptr(), bad, None, y.data_ptr(), 1)
    odd = oracle.quantize(helpers.normal(96, (3, 33), 0.02), 32)
    with pytest.raises(package.Unsupported):       # blocks of 32, 33 columns
        library.linear_input_backward(x.data_ptr(), upload(gpu, odd),
                                      y.data_ptr(), 1,
                                      algorithm=package.ALGORITHM_GEMV)
    with pytest.raises(package.Unsupported):       # five rows of dy
        library.linear_input_backward(x.data_ptr(), device_weight,
                                      y.data_ptr(), 5,
                                      algorithm=package.ALGORITHM_GEMV)
    with pytest.raises(package.Unsupported):
        library.linear_forward(x.data_ptr(), upload(gpu, odd), None,
                               y.data_ptr(), 1,
                               algorithm=package.ALGORITHM_MFMA)


def test_memory_entry_points(gpu, package, library):
    import torch
    pointer = library.malloc(4096)
    assert pointer % 256 == 0
    source = np.arange(1024, dtype=np.float32)
    library.copy_to_device(pointer, source.ctypes.data, 4096)
    back = np.zeros(1024, dtype=np.float32)
    library.copy_to_host(back.ctypes.data, pointer, 4096)
    assert np.array_equal(source, back)
    library.fill_f32(pointer, 2.5, 1024)
    library.synchronize()
    library.copy_to_host(back.ctypes.data, pointer, 4096)
    assert np.all(back == 2.5)
    library.free(pointer)
    assert "MI355X" in library.device_description() or \
        "gfx950" in library.device_description()


# ---- content rules of a canonical payload, checked on the device -----------

def verdict(function, *arguments):
    try:
        function(*arguments)
        return ""
    except ValueError as error:
        # the library's message without the binding's "rthip status N: "
        return getattr(error, "message", str(error))


def damaged_payloads(oracle):
    """(name, weight) pairs: valid payloads and payloads that break one or
    several rules of require_canonical_payload, in places chosen so that the
    rule the reference reports first differs from case to case."""
    import copy
    dense = helpers.normal(150, (300, 1000), 0.02)
    dense[3:5] = 0.0                      # whole zero blocks
    dense.ravel()[-1] = 0.01
    plain = oracle.quantize(dense, 64, False, 256)
    nested = oracle.quantize(dense, 64, True, 256)
    odd = oracle.quantize(helpers.normal(151, (33, 33), 0.02), 32, False, 32)
    odd_nested = oracle.quantize(helpers.normal(151, (33, 33), 0.02), 32,
                                 True, 32)
    zero_block = 3 * 1000 // 64 + 1       # a block inside the zero rows
    cases = [("plain", plain), ("nested", nested), ("odd", odd),
             ("odd nested", odd_nested)]

    def changed(name, base, **edits):
        weight = copy.deepcopy(base)
        for field, (index, value) in edits.items():
            if field == "offset":
                weight.offset = value
            else:
                getattr(weight, field)[index] = value
        cases.append((name, weight))

    changed("unused nibble", odd, codes=(-1, 0xF7))
    changed("unused nibble nested", odd_nested, codes=(-1, 0x17))
    changed("negative scale", plain, fp32_scales=(17, -1.0))
    changed("infinite scale", plain, fp32_scales=(4000, np.inf))
    changed("nan scale at the end", plain, fp32_scales=(-1, np.nan))
    changed("negative zero scale is a zero scale", plain,
            fp32_scales=(zero_block, -0.0))
    changed("code in a zero block", plain, codes=(zero_block * 32 + 5, 0x70))
    changed("code in a zero block, first byte", plain,
            codes=(zero_block * 32, 0x87))
    changed("zeroed scale of a used block", plain, fp32_scales=(2000, 0.0))
    changed("zero block below a bad scale", plain,
            codes=(zero_block * 32 + 5, 0x70), fp32_scales=(3000, -1.0))
    changed("bad scale below a zero block", plain,
            codes=(zero_block * 32 + 5, 0x70), fp32_scales=(2, np.nan))
    changed("nibble before everything", odd, codes=(-1, 0xF7),
            fp32_scales=(0, np.nan))
    changed("nested tolerates codes under a zero scale", nested,
            codes=(zero_block * 32 + 5, 0x70))
    changed("second-level nan", nested, second_level=(3, np.nan))
    changed("second-level negative", nested, second_level=(-1, -1.0e-3))
    changed("second-level infinite", nested, second_level=(0, np.inf))
    changed("offset nan", nested, offset=(None, float("nan")))
    changed("offset negative", nested, offset=(None, -1.0))
    changed("offset before second-level", nested, offset=(None, float("inf")),
            second_level=(0, np.nan))
    # a huge second-level scale saturates the decoded scale instead of
    # overflowing it, which the rules accept
    changed("saturating second-level scale", nested,
            second_level=(1, np.float32(3.0e38)))
    return cases


def test_device_payload_check_follows_the_reference_rules(gpu, package,
                                                          library, oracle):
    """rthip_nf4_check_payload accepts and refuses exactly what the oracle's
    require_canonical_payload does, with the same message."""
    seen = set()
    for name, weight in damaged_payloads(oracle):
        expected = verdict(oracle.validate_payload, weight)
        got = verdict(gpu.check_payload, upload(gpu, weight))
        assert got == expected, f"{name}: {got!r} instead of {expected!r}"
        seen.add(expected)
    assert len(seen) == 6, seen   # valid + the five content rules


def test_device_payload_check_on_a_transformer_layer(gpu, package, library,
                                                     oracle):
    """A full 11008 x 4096 layer: valid as quantised on the device, refused
    after one byte of a zero block or one scale is damaged."""
    import torch
    dense = helpers.normal(152, (11008, 4096), 0.02)
    dense[100] = 0.0
    for nested in (False, True):
        weight = gpu.quantize_weight(to_device(dense), 64, nested, 256)
        gpu.check_payload(weight)
        if nested:
            weight.secondary_scales[-1] = float("nan")
            torch.cuda.synchronize()
            assert verdict(gpu.check_payload, weight) == \
                "NF4 second-level scales must be finite and nonnegative"
        else:
            weight.codes[100 * 2048 + 77] = 0x72
            torch.cuda.synchronize()
            assert verdict(gpu.check_payload, weight) == \
                "zero-scale NF4 blocks must use canonical zero code 7"
            weight.primary_scales[-1] = -1.0
            assert verdict(gpu.check_payload, weight) == \
                "zero-scale NF4 blocks must use canonical zero code 7"
            weight.codes[100 * 2048 + 77] = 0x77
            assert verdict(gpu.check_payload, weight) == \
                "NF4 block scales must be finite and nonnegative"


# ---- replay from a HIP graph ----------------------------------------------

def test_every_family_replays_from_a_graph(gpu, package, library, oracle):
    """A decode loop is launch-bound and runs from a HIP graph (the benchmark
    does).  One graph holds a launch of every forward family, the partial-tile
    path of the small-batch family with its second kernel and workspace, the
    adapter epilogue, the input backward and the adapter's backward; each of
    several replays, with
    eager launches and synchronisations in between and fresh inputs written
    into the captured buffers, must equal the eager result bit for bit."""
    import torch
    weight = oracle.quantize(helpers.normal(160, (1000, 2048), 0.02), 64,
                             True, 256)
    device_weight = upload(gpu, weight)
    bias = to_device(helpers.normal(161, (1000,), 0.01))
    lora_a = to_device(helpers.normal(162, (8, 2048), 0.05))
    lora_b = to_device(helpers.normal(163, (1000, 8), 0.05))
    # name -> (rows, pinned family or None for the automatic choice)
    launches = {"gemv": (2, None), "resident": (9, None),
                "resident, three row groups": (40, None),
                "skinny": (40, package.ALGORITHM_SKINNY),
                "resident, two launches": (130, None), "mfma": (300, None)}
    inputs = {name: torch.zeros((rows, 2048), device="cuda")
              for name, (rows, _) in launches.items()}
    upstream = torch.zeros((300, 1000), device="cuda")
    for name, (rows, family) in launches.items():
        if family is None:
            assert package.ALGORITHM_NAMES[library.select_algorithm(
                package.FORWARD, rows, 2048, 1000, 64)] == name.split(",")[0]
    assert library.select_algorithm(package.INPUT_BACKWARD, 40, 2048, 1000,
                                    64) == package.ALGORITHM_SKINNY

    def launch_all():
        outputs = {name: gpu.linear_forward(x, device_weight, bias,
                                            algorithm=launches[name][1])
                   for name, x in inputs.items()}
        outputs["adapter"], _ = gpu.lora_linear_forward(
            inputs["resident"], device_weight, lora_a, lora_b, 0.5, bias)
        outputs["backward"] = gpu.linear_input_backward(upstream,
                                                        device_weight)
        # up to 64 rows: the kernel that walks the weight row by row, here
        # with its row chunks summed through the workspace
        outputs["small backward"] = gpu.linear_input_backward(
            upstream[:40].contiguous(), device_weight)
        # up to four rows: the weight streamed row by row, the row ranges
        # summed through the workspace, on the vector ALU (one row) and on the
        # 4x4x1 matrix instruction (three)
        for rows in (1, 3):
            outputs[f"streaming backward, {rows}"] = \
                gpu.linear_input_backward(
                    upstream[:rows].contiguous(), device_weight,
                    algorithm=package.ALGORITHM_GEMV)
        # the adapter's gradients (column slices summed through the
        # workspace) and the input backward with the adapter's share of dx in
        # its epilogue, tiled (300 rows) and small-batch (9 rows)
        for name, rows in (("mfma", 300), ("resident", 9)):
            x = inputs[name]
            reduced = torch.empty((rows, 8), device="cuda")
            library.lora_reduce(x.data_ptr(), lora_a.data_ptr(),
                                reduced.data_ptr(), rows, 2048, 8,
                                torch.cuda.current_stream().cuda_stream)
            (outputs[f"adapter backward {rows}, dx"],
             outputs[f"adapter backward {rows}, dA"],
             outputs[f"adapter backward {rows}, dB"]) = \
                gpu.lora_linear_backward(
                    upstream[:rows].contiguous(), x, device_weight, lora_a,
                    lora_b, 0.5, reduced)
        return outputs

    def refill(seed):
        for index, x in enumerate(inputs.values()):
            x.copy_(to_device(helpers.normal(seed + index, tuple(x.shape),
                                             1.0)))
        upstream.copy_(to_device(helpers.normal(seed + 9, (300, 1000),
                                                1.0e-2)))

    refill(170)
    launch_all()                      # first use allocates the workspace
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            captured = launch_all()
    for replay in range(4):
        refill(180 + 10 * replay)
        eager = {name: host(value) for name, value in launch_all().items()}
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, value in captured.items():
            helpers.assert_bit_equal(host(value), eager[name],
                                     f"replay {replay}, {name}")


# ---- a seeded sweep over small random problems -------------------------------

def test_random_small_problems(gpu, package, library, oracle):
    """Forty seeded problems with every quantity drawn at random -- widths that
    are and are not multiples of the kernels' tile sizes, every block size up
    to 512, both encodings, with and without bias -- through every family that
    accepts them, against the oracle and fp64."""
    generator = np.random.default_rng(2024)
    widths = [16, 32, 33, 48, 64, 80, 96, 128, 160, 192, 256, 320, 512, 1024,
              2048]
    for case in range(40):
        in_w = int(generator.choice(widths))
        out_w = int(generator.integers(1, 400))
        rows = int(generator.choice([1, 2, 3, 4, 5, 8, 15, 16, 17, 31, 64, 65,
                                     100]))
        block = int(generator.choice([32, 64, 128, 256, 512]))
        second = int(generator.choice([32, 64, 256]))
        nested = bool(generator.integers(0, 2))
        with_bias = bool(generator.integers(0, 2))
        dense = helpers.normal(3000 + case, (out_w, in_w), 0.02)
        if case % 4 == 0:
            dense[generator.integers(0, out_w)] = 0.0
        weight = oracle.quantize(dense, block, nested, second)
        x = helpers.normal(3100 + case, (rows, in_w), 1.0)
        dy = helpers.normal(3200 + case, (rows, out_w), 1.0e-2)
        bias = helpers.normal(3300 + case, (out_w,), 0.01) \
            if with_bias else None
        try:
            check_layer(gpu, package, library, oracle, weight, x, dy,
                        bias=bias, oracle_rows=min(rows, 4))
        except AssertionError as error:
            raise AssertionError(
                f"case {case}: rows={rows} out={out_w} in={in_w} "
                f"block={block} second={second} nested={nested} "
                f"bias={with_bias}: {error}") from error
