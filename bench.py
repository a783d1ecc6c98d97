"""Benchmark of the packed NF4 linear path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--full]

Headline workload (the configuration the metric is quoted on): decode GEMV,
M = 1, the seven Llama-7B projection shapes per layer (q/k/v/o 4096x4096,
gate/up 11008x4096, down 4096x11008), NF4 block 64 with fp32 absmax scales, no
bias.  One step = one token through all 7 projections of L layers, every layer
holding its own packed weights, so the working set (L x 113.8 MB) is far
larger than the 256 MB last-level cache and every step streams it from HBM.
Projections that read the same activations (q/k/v; gate/up) go out in ONE
launch through rthip_nf4_linear_forward_group -- four launches per layer, as
the backend adapter issues them for unchanged callers -- and
--one-launch-per-projection times the seven-launch form instead (both are in
the line either way, see roofline.decode_steps).  `value` = algorithmic bytes
(packed codes + scale payload) per second with everything resident in HBM
before the timed region.

Everything that the metric names is inside `roofline`, so that a reader of
that object alone can recompute it:
  roofline      HBM roofline of the dominant decode kernel (bytes per launch /
                average launch duration from HIP events on the launch stream;
                traffic from the tracked rocprofv3 counter summary, refused
                when that summary was taken with other kernel instances than
                this build launches)
    .decode_steps   the decode step four ways: launches per shared input or per
                    projection, fp32 or nested (double-quantised) scales
    .gemm           M = 2048 forward and input-backward GEMMs (prefill /
                    training shapes, both scale encodings) against the fp32
                    MFMA peak
    .small_batch    M in {1, 4, 16, 64} on the three distinct shapes
    .large_launches M = 1 launches of 74 to 117 MB (lm_head; four gate/up
                    weights in one launch; a 70B model's feed-forward shapes)
    .practical_roof a plain streaming read of the same sizes, one launch per
                    buffer, and an empty launch: what the device gives a kernel
                    that only reads, beside the 8 TB/s of the data sheet
  cpu_baseline  the reference CPU backend (kind "reference": oracle/_ref, built
                in the build container from the reference's own sources and
                shipped prebuilt; kind "port": the C restatement, where that
                library is absent) timed on this host, single thread, on one
                layer; host_cpu names the processor
With --full the line also carries
  small_batch_groups, mid_batch (M in {128 ... 1024}), ragged_shapes (4097 x
  4095), small_batch_input_backward, lora (fused adapter forward and
  backward), matmul (dense fp32) and quantizer.

Packed payloads are synthetic: uniformly random nibbles (NF4 codes of normal
weights are close to uniform by construction) and block scales drawn around
the absmax of 64 samples of N(0, 0.02), generated on the device.
"""
import argparse
import ctypes
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_FP32_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix, published

LAYER_SHAPES = [  # (name, output_width, input_width)
    ("q_proj", 4096, 4096), ("k_proj", 4096, 4096), ("v_proj", 4096, 4096),
    ("o_proj", 4096, 4096), ("gate_proj", 11008, 4096),
    ("up_proj", 11008, 4096), ("down_proj", 4096, 11008),
]
BLOCK = 64
SECOND_LEVEL_BLOCK = 256


def synthetic_weight(package, torch, out_w, in_w, double_quantized, seed):
    """A packed weight generated directly in HBM."""
    generator = torch.Generator(device="cuda")
    generator.manual_seed(seed)
    count = out_w * in_w
    blocks = count // BLOCK
    codes = torch.randint(0, 256, (count // 2,), dtype=torch.uint8,
                          device="cuda", generator=generator)
    if not double_quantized:
        scales = (torch.rand(blocks, device="cuda", generator=generator) *
                  0.03 + 0.035)
        return package.DeviceWeight(out_w, in_w, BLOCK, package.SCALE_FLOAT32,
                                    codes, scales, None)
    scale_codes = torch.randint(1, 256, (blocks,), dtype=torch.uint8,
                                device="cuda", generator=generator)
    groups = -(-blocks // SECOND_LEVEL_BLOCK)
    second = (torch.rand(groups, device="cuda", generator=generator) *
              0.01 + 0.02)
    return package.DeviceWeight(
        out_w, in_w, BLOCK, package.SCALE_DOUBLE_QUANTIZED_UINT8, codes,
        scale_codes, second, SECOND_LEVEL_BLOCK, 0.05)


def capture(torch, body):
    """Records body()'s launches into a HIP graph and returns its replay.  The
    decode kernels last microseconds, far less than a Python-level launch, so
    the launch-bound loops are replayed as graphs (kernel nodes only)."""
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        body()
    return graph.replay


def time_region(torch, body, repeats):
    """Milliseconds for `repeats` calls of body(), bracketed by HIP events on
    the stream the kernels are launched on."""
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(repeats):
        body()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop)


def warm(torch, body, seconds=0.03):
    """Runs body() for a while: the first milliseconds out of idle run at a
    lower clock, which a sub-millisecond warm-up does not get past."""
    torch.cuda.synchronize()
    start = time.perf_counter()
    while time.perf_counter() - start < seconds:
        body()
        torch.cuda.synchronize()


# Projections of a layer that read the same activations (one launch each when
# the step is run through rthip_nf4_linear_forward_group).
SHARED_INPUT_GROUPS = [("q_proj", "k_proj", "v_proj"), ("o_proj",),
                       ("gate_proj", "up_proj"), ("down_proj",)]


def bench_decode(package, device, torch, layers, steps, warmup, use_graph,
                 double_quantized=False, grouped=False):
    """One token through all 7 projections of `layers` layers.  grouped:
    projections that share their input go through ONE call of the group entry
    point (4 launches per layer instead of 7); otherwise one call each."""
    library = package.load_library()
    names = [name for name, _, _ in LAYER_SHAPES]
    x = {width: torch.randn(1, width, device="cuda")
         for width in (4096, 11008)}
    weights = []
    launches = []  # (x pointer, [(weight, bias pointer, y pointer), ...])
    outputs = []
    for layer in range(layers):
        of_layer = {}
        for index, (name, out_w, in_w) in enumerate(LAYER_SHAPES):
            of_layer[name] = synthetic_weight(package, torch, out_w, in_w,
                                              double_quantized,
                                              1000 * layer + index)
            weights.append(of_layer[name])
        groups = SHARED_INPUT_GROUPS if grouped else [(n,) for n in names]
        for group in groups:
            members = []
            for slot, name in enumerate(group):
                weight = of_layer[name]
                if layer == 0:
                    outputs.append(torch.empty(1, weight.output_width,
                                               device="cuda"))
                y = [t for t in outputs
                     if t.shape[1] == weight.output_width][slot]
                members.append((weight, None, y.data_ptr()))
            launches.append((x[members[0][0].input_width].data_ptr(), members))

    def launch_all(items):
        stream = torch.cuda.current_stream().cuda_stream
        for x_ptr, members in items:
            if len(members) == 1:
                weight, _, y_ptr = members[0]
                library.linear_forward(x_ptr, weight, None, y_ptr, 1, stream)
            else:
                library.linear_forward_group(x_ptr, members, 1, stream)

    launch_all(launches)  # first use outside any capture
    torch.cuda.synchronize()
    step = lambda: launch_all(launches)
    if use_graph:
        step = capture(torch, step)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter()
    milliseconds = time_region(torch, step, steps)
    wall = time.perf_counter() - wall
    bytes_per_step = sum(w.payload_bytes for w in weights)
    launches_per_step = len(launches)
    seconds = milliseconds / 1e3
    gbs = bytes_per_step * steps / seconds / 1e9

    # The dominant kernel: the K = 4096 instantiation (6 of 7 projections);
    # in a grouped step, its launches that cover more than one weight.
    dominant = [item for item in launches
                if item[1][0][0].input_width == 4096 and
                (not grouped or len(item[1]) > 1)]

    dominant_pass = lambda: launch_all(dominant)
    if use_graph:
        dominant_pass = capture(torch, dominant_pass)
    dominant_pass()
    dominant_ms = time_region(torch, dominant_pass, steps)
    dominant_bytes = sum(member[0].payload_bytes
                         for item in dominant for member in item[1])
    average_us = dominant_ms * 1e3 / (steps * len(dominant))
    achieved = dominant_bytes * steps / (dominant_ms / 1e3) / 1e9
    # the kernel instances of those launches, as a profiler prints them
    encoding = weights[0].encoding
    instances = sorted({
        library.forward_kernel_name(
            1, 4096, [member[0].output_width for member in item[1]], BLOCK,
            encoding, SECOND_LEVEL_BLOCK if double_quantized else 0)
        for item in dominant})
    traffic, traffic_source = profiled_traffic(grouped, instances)
    return {
        "value": gbs,
        "ms_per_step": milliseconds / steps,
        "wall_seconds": wall,
        "bytes_per_step": bytes_per_step,
        "launches_per_step": launches_per_step,
        "roofline": {
            "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic, "traffic_source": traffic_source,
            "kernel": ", ".join(instances),
            "bytes_per_launch": dominant_bytes / len(dominant),
            "avg_launch_us": average_us,
        },
    }


TRAFFIC_PROFILE = os.path.join(ROOT, "profiles",
                               "decode_gemv_hbm_traffic_pmc.txt")


def profiled_traffic(grouped, instances):
    """HBM bytes per launch of the dominant kernel as the tracked rocprofv3
    counter summary has them (a counter run cannot be nested inside this
    timing run): FETCH_SIZE and WRITE_SIZE averages of the kernel instances
    in `instances` (the names this build reports for the launches that were
    timed), each scaled by what the same counter read for torch's
    2^28-element copy (2^20 KiB read, 2^20 KiB written).  Returns (bytes,
    where it came from), or (None, why not): a summary that was taken with
    other instances than this build launches has no row for them and is
    refused, not quoted."""
    section = ("projections that share x in one launch" if grouped
               else "one launch per projection")
    try:
        with open(TRAFFIC_PROFILE) as handle:
            text = handle.read()
    except OSError as error:
        return None, "no profile: %s" % error
    if section not in text:
        return None, "the profile has no section '%s'" % section
    body = text[text.index(section) + len(section):]
    for other in ("projections that share x in one launch",
                  "one launch per projection"):
        if other != section and other in body:
            body = body[:body.index(other)]
    if not instances or "" in instances:
        return None, "the timed launches are not served by the decode kernel"
    readings = {}
    for line in body.splitlines():
        fields = line.split()
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            if counter not in fields:
                continue
            average = float(fields[fields.index(counter) + 2])
            calls = float(fields[fields.index(counter) + 1])
            if line.startswith("at::native::vectorized_elementwise_kernel"):
                # the 2^28-element copy is the largest of torch's launches
                if average >= readings.get((counter, "copy"), (0.0, 0))[0]:
                    readings[counter, "copy"] = (average, calls)
            for name in instances:
                if ("rthip::" + name) in line.replace(
                        "(anonymous namespace)::", ""):
                    total, count = readings.get((counter, "kernel"), (0, 0))
                    readings[counter, "kernel"] = (total + average * calls,
                                                   count + calls)
                    readings[counter, name] = True
    missing = [name for name in instances
               if (("FETCH_SIZE", name) not in readings or
                   ("WRITE_SIZE", name) not in readings)]
    if missing:
        return None, ("the profile was taken with other kernel instances: "
                      "no row for %s" % ", ".join(missing))
    try:
        kib = sum(readings[counter, "kernel"][0] /
                  readings[counter, "kernel"][1] * 2.0 ** 20 /
                  readings[counter, "copy"][0]
                  for counter in ("FETCH_SIZE", "WRITE_SIZE"))
    except KeyError as missing_row:
        return None, "the profile has no row for %s" % (missing_row.args[0],)
    return int(kib * 1024), (
        "profiles/decode_gemv_hbm_traffic_pmc.txt: rocprofv3 --pmc "
        "FETCH_SIZE / WRITE_SIZE per dispatch, each scaled by its reading "
        "for a copy of 2^30 B")


def bench_gemm(package, device, torch, steps):
    """Prefill / training forward and the input backward: M = 2048."""
    rows = 2048
    results = []
    cases = [
        ("forward", 11008, 4096, False), ("forward", 11008, 4096, True),
        ("forward", 4096, 4096, False), ("forward", 4096, 4096, True),
        ("input_backward", 4096, 11008, True),
        ("input_backward", 11008, 4096, True),
    ]
    for direction, out_w, in_w, double_quantized in cases:
        weight = synthetic_weight(package, torch, out_w, in_w,
                                  double_quantized, 77)
        if direction == "forward":
            source = torch.randn(rows, in_w, device="cuda")
            target = torch.empty(rows, out_w, device="cuda")
            body = lambda: device.linear_forward(source, weight, out=target)
        else:
            source = torch.randn(rows, out_w, device="cuda") * 1e-2
            target = torch.empty(rows, in_w, device="cuda")
            body = lambda: device.linear_input_backward(source, weight,
                                                        out=target)
        for _ in range(20):  # the first launches after idle run at low clocks
            body()
        milliseconds = time_region(torch, body, steps) / steps
        flops = 2.0 * rows * out_w * in_w
        tflops = flops / (milliseconds / 1e3) / 1e12
        results.append({
            "direction": direction, "rows": rows, "output_width": out_w,
            "input_width": in_w,
            "scales": "double_quantized" if double_quantized else "fp32",
            "ms": milliseconds,
            "roofline": {"bound": "mfma", "achieved": tflops,
                         "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": tflops / MFMA_FP32_PEAK_TFLOPS,
                         "traffic": None},
        })
        del source, target, weight
    return results


def bench_small_batch(package, device, torch, steps):
    """Small-batch decode: M in {1, 4, 16, 64}, fp32 scales; rotating weights."""
    results = []
    copies = 12  # 12 x >= 9.4 MB per shape: beyond the last-level cache
    for name, out_w, in_w in (LAYER_SHAPES[0], LAYER_SHAPES[4],
                              LAYER_SHAPES[6]):
        weights = [synthetic_weight(package, torch, out_w, in_w, False, 500 + i)
                   for i in range(copies * (3 if out_w * in_w < 2 ** 25 else 1))]
        for rows in (1, 4, 16, 64):
            source = torch.randn(rows, in_w, device="cuda")
            target = torch.empty(rows, out_w, device="cuda")

            def body():
                for weight in weights:
                    device.linear_forward(source, weight, out=target)

            body()
            torch.cuda.synchronize()
            body = capture(torch, body)
            body()
            milliseconds = time_region(torch, body, steps) / (
                steps * len(weights))
            results.append({
                "shape": name, "rows": rows, "us": milliseconds * 1e3,
                "gb_per_s": weights[0].payload_bytes / milliseconds / 1e6,
                "tflop_per_s": 2.0 * rows * out_w * in_w / milliseconds / 1e9,
            })
        del weights
    return results


def bench_mid_batch(package, device, torch, steps):
    """Forward at row counts between the small-batch kernels and prefill."""
    results = []
    for name, out_w, in_w in (LAYER_SHAPES[0], LAYER_SHAPES[4],
                              LAYER_SHAPES[6]):
        weights = [synthetic_weight(package, torch, out_w, in_w, False, 700 + i)
                   for i in range(4)]
        for rows in (128, 192, 256, 272, 512, 1024):
            source = torch.randn(rows, in_w, device="cuda")
            target = torch.empty(rows, out_w, device="cuda")

            def body():
                for weight in weights:
                    device.linear_forward(source, weight, out=target)

            body()
            torch.cuda.synchronize()
            body = capture(torch, body)
            warm(torch, body)
            milliseconds = time_region(torch, body, steps) / (
                steps * len(weights))
            tflops = 2.0 * rows * out_w * in_w / milliseconds / 1e9
            results.append({
                "shape": name, "rows": rows, "us": milliseconds * 1e3,
                "tflop_per_s": tflops,
                "frac_of_fp32_mfma_peak": tflops / MFMA_FP32_PEAK_TFLOPS,
            })
        del weights
    return results


def bench_small_batch_groups(package, device, torch, steps):
    """Projections that read the same x (q/k/v; gate/up) at M in {4, 16, 64}:
    one launch per projection against one launch per group
    (rthip_nf4_linear_forward_group).  us and rates are per GROUP."""
    library = package.load_library()
    results = []
    for name, shapes in (("q/k/v", [(4096, 4096)] * 3),
                         ("gate/up", [(11008, 4096)] * 2)):
        copies = 12 if name == "q/k/v" else 6
        groups = [[synthetic_weight(package, torch, out_w, in_w, False,
                                    1200 + 10 * copy + index)
                   for index, (out_w, in_w) in enumerate(shapes)]
                  for copy in range(copies)]
        payload = sum(weight.payload_bytes for weight in groups[0])
        flops_per_row = sum(2.0 * out_w * in_w for out_w, in_w in shapes)
        for rows in (4, 16, 64):
            source = torch.randn(rows, 4096, device="cuda")
            outputs = [torch.empty(rows, out_w, device="cuda")
                       for out_w, _ in shapes]

            def one_by_one():
                for group in groups:
                    for weight, out in zip(group, outputs):
                        device.linear_forward(source, weight, out=out)

            def together():
                stream = torch.cuda.current_stream().cuda_stream
                for group in groups:
                    library.linear_forward_group(
                        source.data_ptr(),
                        [(weight, None, out.data_ptr())
                         for weight, out in zip(group, outputs)], rows, stream)

            timings = {}
            for label, body in (("one_by_one", one_by_one),
                                ("together", together)):
                body()
                torch.cuda.synchronize()
                body = capture(torch, body)
                body()
                timings[label] = time_region(torch, body, steps) / (
                    steps * len(groups)) * 1e3
            results.append({
                "group": name, "rows": rows,
                "one_launch_per_projection_us": timings["one_by_one"],
                "one_launch_per_group_us": timings["together"],
                "gb_per_s": payload / timings["together"] / 1e3,
                "tflop_per_s": rows * flops_per_row / timings["together"] / 1e6,
            })
        del groups
    return results


def bench_ragged(package, device, torch, steps):
    """A shape none of the tuned families takes (row width 4095: not a
    multiple of 16, blocks straddle rows): the shape-agnostic kernels, forward
    and input backward, at M in {1, 16}."""
    out_w, in_w = 4097, 4095
    count = out_w * in_w
    generator = torch.Generator(device="cuda")
    generator.manual_seed(77)
    codes = torch.randint(0, 256, ((count + 1) // 2,), dtype=torch.uint8,
                          device="cuda", generator=generator)
    if count % 2:
        codes[-1] &= 0x0F        # the unused high nibble stays zero
    scales = torch.rand(-(-count // BLOCK), device="cuda",
                        generator=generator) * 0.03 + 0.035
    weight = package.DeviceWeight(out_w, in_w, BLOCK, package.SCALE_FLOAT32,
                                  codes, scales, None)
    results = []
    for rows in (1, 16):
        source = torch.randn(rows, in_w, device="cuda")
        upstream = torch.randn(rows, out_w, device="cuda") * 1.0e-2
        target = torch.empty(rows, out_w, device="cuda")
        gradient = torch.empty(rows, in_w, device="cuda")
        timings = {}
        for label, body in (
                ("forward", lambda: device.linear_forward(source, weight,
                                                          out=target)),
                ("input_backward", lambda: device.linear_input_backward(
                    upstream, weight, out=gradient))):
            body()
            torch.cuda.synchronize()
            timings[label] = time_region(torch, body, steps) / steps * 1e3
        results.append({
            "shape": f"{out_w}x{in_w}", "rows": rows,
            "forward_us": timings["forward"],
            "input_backward_us": timings["input_backward"],
            "forward_gb_per_s": weight.payload_bytes / timings["forward"] / 1e3,
            "input_backward_gb_per_s":
                weight.payload_bytes / timings["input_backward"] / 1e3,
        })
    return results


def bench_large_launches(package, device, torch, steps):
    """M = 1 launches that move more bytes than one projection: the lm_head of
    the same model (32000 x 4096), gate/up of two layers in one grouped
    launch, and the feed-forward projections of a 70B model (117 MB each; the
    second has rows of 28672 weights).  They show the rate the GEMV streams at once a launch's fixed cost
    (about 3 us) is spread over enough bytes."""
    library = package.load_library()
    results = []
    cases = [("lm_head 32000x4096", [(32000, 4096)]),
             ("4 x 11008x4096 in one launch", [(11008, 4096)] * 4),
             ("70B feed-forward 28672x8192", [(28672, 8192)]),
             ("70B feed-forward 8192x28672", [(8192, 28672)])]
    for name, shapes in cases:
        x = torch.randn(1, shapes[0][1], device="cuda")
        copies = 6  # 6 x >= 74 MB: beyond the last-level cache
        groups = [[synthetic_weight(package, torch, out_w, in_w, False,
                                    900 + 10 * copy + index)
                   for index, (out_w, in_w) in enumerate(shapes)]
                  for copy in range(copies)]
        outputs = [torch.empty(1, out_w, device="cuda")
                   for out_w, _ in shapes]

        def body():
            stream = torch.cuda.current_stream().cuda_stream
            for group in groups:
                library.linear_forward_group(
                    x.data_ptr(),
                    [(weight, None, y.data_ptr())
                     for weight, y in zip(group, outputs)], 1, stream)

        body()
        torch.cuda.synchronize()
        body = capture(torch, body)
        body()
        milliseconds = time_region(torch, body, steps) / (steps * copies)
        payload = sum(weight.payload_bytes for weight in groups[0])
        gbs = payload / milliseconds / 1e6
        results.append({
            "launch": name, "bytes": payload, "us": milliseconds * 1e3,
            "roofline": {"bound": "hbm", "achieved": gbs,
                         "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": gbs / HBM_PEAK_GBS, "traffic": None},
        })
        del groups
    return results


class Probes:
    """librthip_probe.so: a plain streaming read and an empty launch."""

    def __init__(self, path):
        self._lib = ctypes.CDLL(path)
        self._lib.rthip_probe_streaming_read.restype = ctypes.c_int
        self._lib.rthip_probe_streaming_read.argtypes = [
            ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]
        self._lib.rthip_probe_empty_launch.restype = ctypes.c_int
        self._lib.rthip_probe_empty_launch.argtypes = [ctypes.c_void_p]

    def probe_streaming_read(self, data_ptr, size, stream):
        status = self._lib.rthip_probe_streaming_read(data_ptr, size, stream)
        if status != 0:
            raise RuntimeError("streaming-read probe: status %d" % status)

    def probe_empty_launch(self, stream):
        status = self._lib.rthip_probe_empty_launch(stream)
        if status != 0:
            raise RuntimeError("empty-launch probe: status %d" % status)


def load_probes(package):
    path = os.path.join(os.path.dirname(os.path.abspath(package.__file__)),
                        "lib", "librthip_probe.so")
    if not os.path.exists(path):
        raise RuntimeError(
            "%s is missing: run `make -C riftco-transformer_amd`" % path)
    return Probes(path)


def bench_practical_roof(package, torch, steps):
    """What the device gives a kernel that only reads: one launch of a plain
    streaming read (rthip_probe_streaming_read of librthip_probe.so, a
    library of two measurement launches beside the product's) per buffer,
    buffers rotating through more than the last-level cache, replayed as a
    graph exactly like the decode step; and an empty launch of the same grid.
    The sizes are the packed payloads of the decode shapes and of the large
    launches."""
    library = load_probes(package)
    stream = lambda: torch.cuda.current_stream().cuda_stream
    results = {"streaming_read": []}

    def timed(body, launches):
        body()
        torch.cuda.synchronize()
        replay = capture(torch, body)
        replay()
        return time_region(torch, replay, steps) / (steps * launches) * 1e3

    copies = 24
    results["empty_launch_us"] = timed(
        lambda: [library.probe_empty_launch(stream()) for _ in range(copies)],
        copies)
    for label, size in (("4096x4096 payload", 9437184),
                        ("11008x4096 payload", 25362432),
                        ("32000x4096 payload", 73728000),
                        ("256 MiB", 256 << 20)):
        count = max(3, -(-(640 << 20) // size))  # >= 640 MB in rotation
        buffers = [torch.empty(size, dtype=torch.uint8, device="cuda")
                   for _ in range(count)]
        for buffer in buffers:
            buffer.random_(0, 256)
        microseconds = timed(
            lambda: [library.probe_streaming_read(b.data_ptr(), size,
                                                  stream())
                     for b in buffers], count)
        results["streaming_read"].append({
            "what": label, "bytes": size, "us": microseconds,
            "gb_per_s": size / microseconds / 1e3,
            "frac_of_peak": size / microseconds / 1e3 / HBM_PEAK_GBS})
        del buffers
    return results


def bench_small_batch_backward(package, device, torch, steps):
    """Input backward at M in {1, 16, 64}, nested scales; rotating weights."""
    results = []
    for name, out_w, in_w in (LAYER_SHAPES[4], LAYER_SHAPES[6]):
        weights = [synthetic_weight(package, torch, out_w, in_w, True, 700 + i)
                   for i in range(12)]
        for rows in (1, 16, 64):
            upstream = torch.randn(rows, out_w, device="cuda") * 1.0e-2
            target = torch.empty(rows, in_w, device="cuda")

            def body():
                for weight in weights:
                    device.linear_input_backward(upstream, weight, out=target)

            body()
            torch.cuda.synchronize()
            body = capture(torch, body)
            body()
            milliseconds = time_region(torch, body, steps) / (
                steps * len(weights))
            results.append({
                "shape": name, "rows": rows, "us": milliseconds * 1e3,
                "gb_per_s": weights[0].payload_bytes / milliseconds / 1e6,
                "tflop_per_s": 2.0 * rows * out_w * in_w / milliseconds / 1e9,
            })
        del weights
    return results


def bench_lora(package, device, torch, steps):
    """The fused bias + low-rank adapter forward (rank 16) beside the plain
    forward on the same weights, and the same for the backward pass (dx with
    the adapter's share in its epilogue, plus d_reduced, dA and dB): what the
    adapter costs per call."""
    results = []
    rank = 16
    for name, out_w, in_w in (LAYER_SHAPES[0], LAYER_SHAPES[4]):
        copies = 36 if out_w * in_w < 2 ** 25 else 12
        weights = [synthetic_weight(package, torch, out_w, in_w, False, 700 + i)
                   for i in range(copies)]
        lora_a = torch.randn(rank, in_w, device="cuda") * 0.05
        lora_b = torch.randn(out_w, rank, device="cuda") * 0.05
        bias = torch.randn(out_w, device="cuda") * 0.01
        for rows in (1, 16, 2048):
            used = weights if rows < 2048 else weights[:2]
            source = torch.randn(rows, in_w, device="cuda")
            target = torch.empty(rows, out_w, device="cuda")
            reduced = torch.empty(rows, rank, device="cuda")

            def plain():
                for weight in used:
                    device.linear_forward(source, weight, bias, out=target)

            def fused():
                for weight in used:
                    device.lora_linear_forward(
                        source, weight, lora_a, lora_b, 1.0, bias=bias,
                        out=target, reduced=reduced)

            # the backward pass of the same layer: the packed product alone,
            # the adapter's own gradients (d_reduced, dA, dB), and both with
            # the adapter's share of dx in the epilogue
            upstream = torch.randn(rows, out_w, device="cuda") * 1.0e-2
            gradient = torch.empty(rows, in_w, device="cuda")
            d_reduced = torch.empty(rows, rank, device="cuda")
            d_a = torch.empty_like(lora_a)
            d_b = torch.empty_like(lora_b)
            library = package.load_library()
            stream = lambda: torch.cuda.current_stream().cuda_stream

            def adapter_gradients():
                library.lora_backward(
                    upstream.data_ptr(), source.data_ptr(),
                    reduced.data_ptr(), lora_b.data_ptr(), rank, 1.0,
                    d_reduced.data_ptr(), d_a.data_ptr(), d_b.data_ptr(),
                    rows, in_w, out_w, stream())

            def plain_backward():
                for weight in used:
                    device.linear_input_backward(upstream, weight,
                                                 out=gradient)

            def gradients_only():
                for weight in used:
                    adapter_gradients()

            def fused_backward():
                for weight in used:
                    adapter_gradients()
                    library.lora_linear_input_backward(
                        upstream.data_ptr(), weight, lora_a.data_ptr(),
                        d_reduced.data_ptr(), rank, gradient.data_ptr(), rows,
                        stream())

            timings = {}
            for label, body in (("plain", plain), ("fused", fused),
                                ("plain_backward", plain_backward),
                                ("gradients_only", gradients_only),
                                ("fused_backward", fused_backward)):
                body()
                torch.cuda.synchronize()
                body = capture(torch, body)
                warm(torch, body)
                timings[label] = time_region(torch, body, steps) / (
                    steps * len(used)) * 1e3
            results.append({
                "shape": name, "rows": rows, "rank": rank,
                "plain_us": timings["plain"], "with_adapter_us": timings["fused"],
                "input_backward_us": timings["plain_backward"],
                "adapter_gradients_us": timings["gradients_only"],
                "backward_with_adapter_us": timings["fused_backward"],
            })
        del weights
    return results


def bench_decode_with_adapters(package, device, torch, layers, steps,
                               rank=16):
    """The decode step of a model whose query and value projections carry
    unmerged low-rank adapters (QLoRA serving), M = 1, fp32 scales, three
    ways: one call per projection (q and v through
    rthip_nf4_lora_linear_forward: x.A^T and the packed product, two launches
    each), the shared-input groups with q/k/v through
    rthip_nf4_lora_linear_forward_group (which takes both x.A^T in one launch
    of its own), and the same with the products taken beforehand by ONE
    rthip_lora_reduce over the stacked A of q and v (rows = 1: the members'
    reduced vectors lie side by side)."""
    library = package.load_library()
    x = {width: torch.randn(1, width, device="cuda")
         for width in (4096, 11008)}
    outputs = {}
    per_layer = []
    payload = 0
    for layer in range(layers):
        weights = {}
        for index, (name, out_w, in_w) in enumerate(LAYER_SHAPES):
            weights[name] = synthetic_weight(package, torch, out_w, in_w,
                                             False, 3000 * (layer + 1) + index)
            payload += weights[name].payload_bytes
            outputs.setdefault(name, torch.empty(1, out_w, device="cuda"))
        stacked_a = torch.randn(2 * rank, 4096, device="cuda") * 0.05
        factors = {name: torch.randn(4096, rank, device="cuda") * 0.05
                   for name in ("q_proj", "v_proj")}
        reduced = torch.zeros(1, 2 * rank, device="cuda")
        per_layer.append((weights, stacked_a, factors, reduced))
    scale = 2.0

    def adapter(entry, name):
        _, stacked_a, factors, reduced = entry
        slot = 0 if name == "q_proj" else 1
        return (stacked_a[slot * rank:(slot + 1) * rank],
                factors[name], reduced[:, slot * rank:(slot + 1) * rank])

    def per_projection():
        stream = torch.cuda.current_stream().cuda_stream
        for entry in per_layer:
            for name, _, in_w in LAYER_SHAPES:
                weight = entry[0][name]
                if name in entry[2]:
                    lora_a, lora_b, product = adapter(entry, name)
                    library.lora_linear_forward(
                        x[in_w].data_ptr(), weight, None, lora_a.data_ptr(),
                        lora_b.data_ptr(), rank, scale, product.data_ptr(),
                        outputs[name].data_ptr(), 1, stream)
                else:
                    library.linear_forward(x[in_w].data_ptr(), weight, None,
                                           outputs[name].data_ptr(), 1,
                                           stream)

    def grouped(stacked):
        stream = torch.cuda.current_stream().cuda_stream
        for entry in per_layer:
            weights, stacked_a, _, reduced = entry
            if stacked:
                library.lora_reduce(x[4096].data_ptr(), stacked_a.data_ptr(),
                                    reduced.data_ptr(), 1, 4096, 2 * rank,
                                    stream)
            for group in SHARED_INPUT_GROUPS:
                members = []
                for name in group:
                    entry_adapter = None
                    if name in entry[2]:
                        lora_a, lora_b, product = adapter(entry, name)
                        entry_adapter = (
                            None if stacked else lora_a.data_ptr(),
                            lora_b.data_ptr(), product.data_ptr(), rank,
                            scale)
                    members.append((weights[name], None,
                                    outputs[name].data_ptr(), entry_adapter))
                in_w = members[0][0].input_width
                if len(members) == 1:
                    library.linear_forward(x[in_w].data_ptr(), members[0][0],
                                           None, members[0][2], 1, stream)
                else:
                    library.lora_linear_forward_group(x[in_w].data_ptr(),
                                                      members, 1, stream)

    results = {"rank": rank, "layers": layers, "bytes_per_step": payload,
               "adapters_on": ["q_proj", "v_proj"]}
    for label, body in (
            ("one_call_per_projection", per_projection),
            ("shared_input_groups", lambda: grouped(False)),
            ("shared_input_groups_stacked_reduce", lambda: grouped(True))):
        body()
        torch.cuda.synchronize()
        replay = capture(torch, body)
        warm(torch, replay, 0.02)
        milliseconds = time_region(torch, replay, steps) / steps
        results[label] = {"ms_per_step": milliseconds,
                          "gb_per_s": payload / milliseconds / 1e6}
    return results


def bench_matmul(package, device, torch, steps):
    """Dense fp32 matmul at the layer's shapes and at adapter shapes."""
    results = []
    for rows, shared, columns in ((2048, 4096, 4096), (2048, 4096, 11008),
                                  (2048, 16, 4096), (2048, 4096, 16)):
        left = torch.randn(rows, shared, device="cuda")
        right = torch.randn(shared, columns, device="cuda") * 0.02
        out = torch.empty(rows, columns, device="cuda")
        body = lambda: device.matmul(left, right, out=out)
        warm(torch, body)
        milliseconds = time_region(torch, body, steps) / steps
        tflops = 2.0 * rows * shared * columns / (milliseconds / 1e3) / 1e12
        results.append({
            "rows": rows, "shared": shared, "columns": columns,
            "ms": milliseconds,
            "roofline": {"bound": "mfma", "achieved": tflops,
                         "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": tflops / MFMA_FP32_PEAK_TFLOPS,
                         "traffic": None},
        })
        del left, right, out
    return results


def bench_quantizer(package, device, torch):
    """The device quantizer on one 11008 x 4096 weight (45 M values)."""
    results = []
    dense = torch.randn(11008, 4096, device="cuda") * 0.02
    for double_quantized in (False, True):
        device.quantize_weight(dense, BLOCK, double_quantized, 256)
        torch.cuda.synchronize()
        begin = time.perf_counter()
        repeats = 5
        for _ in range(repeats):
            device.quantize_weight(dense, BLOCK, double_quantized, 256)
        torch.cuda.synchronize()
        seconds = (time.perf_counter() - begin) / repeats
        results.append({
            "shape": "11008x4096",
            "scales": "double_quantized" if double_quantized else "fp32",
            "ms": seconds * 1e3,
            "gvalues_per_s": dense.numel() / seconds / 1e9,
        })
    return results


def host_cpu_model():
    try:
        with open("/proc/cpuinfo") as handle:
            for line in handle:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(budget_seconds=12.0):
    """The reference CPU backend (oracle/_ref when built, else the C
    restatement) on this host, single thread: whole Llama-7B layers (7
    projections, M = 1, fp32 scales), repeated until the time budget is spent."""
    import numpy as np
    from oracle.binding import Nf4Weight, Oracle, Reference
    backend = Reference() if Reference.available() else Oracle()
    rng = np.random.default_rng(3)
    layer = []
    for _, out_w, in_w in LAYER_SHAPES:
        count = out_w * in_w
        codes = rng.integers(0, 256, count // 2, dtype=np.uint8)
        scales = (rng.random(count // BLOCK, dtype=np.float32) *
                  np.float32(0.03) + np.float32(0.035))
        weight = Nf4Weight(out_w, in_w, BLOCK, codes, 0, fp32_scales=scales)
        layer.append((weight, rng.standard_normal((1, in_w), dtype=np.float32)))
    total_bytes = 0
    passes = 0
    begin = time.perf_counter()
    while True:
        for weight, x in layer:
            backend.forward(x, weight, faithful=True)
            total_bytes += weight.payload_bytes
        passes += 1
        seconds = time.perf_counter() - begin
        if seconds >= budget_seconds:
            break
    # The M = 2048 products would take minutes per call on one core: time a
    # few rows of the same shapes and scale linearly (the reference loops are
    # linear in the row count).
    gate, _ = layer[4]
    prefill = {}
    for name, rows, run in (
            ("forward_11008x4096", 4,
             lambda x: backend.forward(x, gate, faithful=True)),
            ("input_backward_11008x4096", 2,
             lambda dy: backend.input_backward(dy, gate, faithful=True))):
        width = gate.input_width if name.startswith("forward") \
            else gate.output_width
        sample = rng.standard_normal((rows, width), dtype=np.float32)
        start = time.perf_counter()
        run(sample)
        elapsed = time.perf_counter() - start
        macs = rows * gate.output_width * gate.input_width
        prefill[name] = {
            "rows_timed": rows, "gmac_per_s": macs / elapsed / 1e9,
            "seconds_for_2048_rows_extrapolated": elapsed * 2048 / rows,
        }
    return {
        "value": total_bytes / seconds / 1e9, "unit": "GB/s", "cores": 1,
        "kind": backend.kind, "host_cpu": host_cpu_model(),
        "seconds": seconds,
        "sample": "%d passes over one Llama-7B layer (7 projections at M=1, "
                  "fp32 scales, %.1f MB packed per pass)"
                  % (passes, total_bytes / passes / 1e6),
        "prefill": prefill,
    }


def rounded(value, digits=4):
    """Floats to `digits` significant digits, recursively: keeps the line
    short enough to be read where only its tail is kept."""
    if isinstance(value, float):
        return float("%.*g" % (digits, value))
    if isinstance(value, dict):
        return {key: rounded(item, digits) for key, item in value.items()}
    if isinstance(value, list):
        return [rounded(item, digits) for item in value]
    return value


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=20)
    parser.add_argument("--warmup", type=int, default=3)
    parser.add_argument("--layers", type=int, default=32)
    parser.add_argument("--skip-extras", action="store_true",
                        help="only the headline decode workload")
    parser.add_argument("--skip-cpu", action="store_true")
    parser.add_argument("--full", action="store_true",
                        help="also the sections off the metric: mid-size "
                             "batches, ragged shapes, the adapter, dense "
                             "matmul, the quantizer, small-batch groups and "
                             "input backward")
    parser.add_argument("--gemm-only", action="store_true",
                        help="run only the M = 2048 GEMM section (for "
                             "rocprofv3 counter runs)")
    parser.add_argument("--small-batch-only", action="store_true",
                        help="run only the launches of up to 64 rows, "
                             "forward and input backward (for counter runs)")
    parser.add_argument("--adapter-only", action="store_true",
                        help="run only the low-rank adapter section, forward "
                             "and backward (for rocprofv3 kernel traces)")
    parser.add_argument("--practical-roof-only", action="store_true",
                        help="run only the streaming-read and empty-launch "
                             "probes and a 1 GiB elementwise copy beside "
                             "them (for rocprofv3 kernel traces)")
    parser.add_argument("--traffic-calibration", action="store_true",
                        help="for rocprofv3 --pmc runs: a 1 GiB elementwise "
                             "copy of known traffic, then one decode step "
                             "launched kernel by kernel, nothing else")
    parser.add_argument("--one-launch-per-projection", action="store_true",
                        help="headline decode step (and the traffic "
                             "calibration) with one launch per projection, "
                             "7 per layer, instead of one per shared input")
    parser.add_argument("--no-graph", action="store_true",
                        help="launch the decode kernels one by one from "
                             "Python instead of replaying a HIP graph")
    arguments = parser.parse_args()
    if arguments.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; the path has no "
                 "collectives or sharding (--gpus %d refused)" % arguments.gpus)

    import torch
    package = importlib.import_module("riftco-transformer_amd")
    device = importlib.import_module("riftco-transformer_amd.device")
    library = package.load_library()
    if not torch.cuda.is_available() or not library.is_available():
        sys.exit("bench.py: no usable MI355X: " + library.last_error())
    grouped = not arguments.one_launch_per_projection

    if arguments.practical_roof_only:
        # torch's elementwise kernel beside the probes, in the same trace: it
        # reads 2^30 B and writes 2^30 B per call
        source = torch.zeros(2 ** 28, device="cuda")
        target = torch.empty_like(source)
        for _ in range(5):
            torch.add(source, 1.0, out=target)
        torch.cuda.synchronize()
        begin = time.perf_counter()
        for _ in range(10):
            torch.add(source, 1.0, out=target)
        torch.cuda.synchronize()
        copy_ms = (time.perf_counter() - begin) * 100.0
        del source, target
        print(json.dumps({
            "elementwise_copy_1gib": {
                "ms": copy_ms, "read_plus_write_gb_per_s": 2 ** 31 / copy_ms / 1e6},
            "practical_roof": bench_practical_roof(package, torch,
                                                   arguments.steps)}))
        return

    if arguments.traffic_calibration:
        # torch's elementwise kernel reads 2^30 B and writes 2^30 B per call:
        # the yardstick for FETCH_SIZE / WRITE_SIZE readings.
        source = torch.zeros(2 ** 28, device="cuda")
        target = torch.empty_like(source)
        for _ in range(3):
            torch.add(source, 1.0, out=target)
        torch.cuda.synchronize()
        bench_decode(package, device, torch, arguments.layers, 1, 0, False,
                     grouped=grouped)
        print(json.dumps({"traffic_calibration": "done",
                          "copy_bytes_read": 2 ** 30,
                          "copy_bytes_written": 2 ** 30}))
        return

    if arguments.adapter_only:
        print(json.dumps({"lora": bench_lora(package, device, torch,
                                             arguments.steps)}))
        return

    if arguments.gemm_only:
        # For counter runs: nothing but the M = 2048 launches.
        print(json.dumps({"gemm": bench_gemm(package, device, torch,
                                             arguments.steps)}))
        return

    if arguments.small_batch_only:
        print(json.dumps({
            "ragged_shapes": bench_ragged(package, device, torch,
                                          arguments.steps),
            "small_batch": bench_small_batch(package, device, torch,
                                             arguments.steps),
            "small_batch_groups": bench_small_batch_groups(
                package, device, torch, arguments.steps),
            "small_batch_input_backward": bench_small_batch_backward(
                package, device, torch, arguments.steps)}))
        return

    def decode_step(grouped_launches, double_quantized, steps):
        result = bench_decode(package, device, torch, arguments.layers, steps,
                              arguments.warmup, not arguments.no_graph,
                              double_quantized=double_quantized,
                              grouped=grouped_launches)
        summary = {
            "launches": ("per_shared_input" if grouped_launches
                         else "per_projection"),
            "scales": "double_quantized" if double_quantized else "fp32",
            "launches_per_step": result["launches_per_step"],
            "bytes_per_step": result["bytes_per_step"],
            "ms_per_step": result["ms_per_step"],
            "gb_per_s": result["value"],
            "frac_of_hbm_peak": result["value"] / HBM_PEAK_GBS,
            "dominant_kernel": result["roofline"]["kernel"],
            "dominant_kernel_frac": result["roofline"]["frac"],
            "dominant_kernel_us": result["roofline"]["avg_launch_us"],
        }
        return result, summary

    decode, headline_summary = decode_step(grouped, False, arguments.steps)
    roofline = decode["roofline"]
    line = {
        "metric": "NF4 linear: HBM GB/s at M=1, TFLOP/s at M=2048, % of "
                  "MI355X roofline",
        "value": decode["value"], "unit": "GB/s", "n_gpus": 1,
        "steps": arguments.steps, "warmup": arguments.warmup,
        "ms_per_step": decode["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "decode GEMV M=1, Llama-7B layer shapes "
                        "(q/k/v/o 4096x4096, gate/up 11008x4096, down "
                        "4096x11008), NF4 block 64, fp32 absmax scales, "
                        "%d layers x 7 projections per step%s" % (
                            arguments.layers,
                            ", projections that share their input launched "
                            "together (4 launches per layer)" if grouped
                            else ", one launch per projection"),
            "layers": arguments.layers,
            "bytes_per_step": decode["bytes_per_step"],
            "launches_per_step": decode["launches_per_step"],
            "launch": "per-kernel" if arguments.no_graph else "hip-graph",
            "device": library.device_description(),
        },
        "roofline": roofline,
    }
    del decode
    roofline["decode_steps"] = [headline_summary]
    if not arguments.skip_extras:
        fewer = max(3, arguments.steps // 2)
        few = max(3, arguments.steps // 4)
        # The decode step the other three ways: the other launch grouping,
        # and both with the reference's double-quantised scale encoding
        # (3.34 GB of packed payload per step instead of 3.64).
        for grouped_launches, double_quantized in (
                (not grouped, False), (grouped, True), (not grouped, True)):
            result, summary = decode_step(grouped_launches, double_quantized,
                                          fewer)
            del result
            roofline["decode_steps"].append(summary)
        roofline["gemm"] = [
            {"direction": case["direction"],
             "weight": "%dx%d" % (case["output_width"], case["input_width"]),
             "rows": case["rows"], "scales": case["scales"], "ms": case["ms"],
             "tflop_per_s": case["roofline"]["achieved"],
             "frac_of_fp32_mfma_peak": case["roofline"]["frac"]}
            for case in bench_gemm(package, device, torch, few)]
        roofline["small_batch"] = bench_small_batch(package, device, torch,
                                                    few)
        roofline["large_launches"] = [
            {"launch": case["launch"], "bytes": case["bytes"],
             "us": case["us"], "gb_per_s": case["roofline"]["achieved"],
             "frac_of_hbm_peak": case["roofline"]["frac"]}
            for case in bench_large_launches(package, device, torch, fewer)]
        roofline["practical_roof"] = bench_practical_roof(package, torch,
                                                          fewer)
        if arguments.full:
            line["small_batch_groups"] = bench_small_batch_groups(
                package, device, torch, few)
            line["mid_batch"] = bench_mid_batch(package, device, torch, few)
            line["ragged_shapes"] = bench_ragged(package, device, torch, few)
            line["small_batch_input_backward"] = bench_small_batch_backward(
                package, device, torch, few)
            line["lora"] = bench_lora(package, device, torch, few)
            line["decode_with_adapters"] = bench_decode_with_adapters(
                package, device, torch, arguments.layers, fewer)
            line["matmul"] = bench_matmul(package, device, torch, few)
            line["quantizer"] = bench_quantizer(package, device, torch)
    if not arguments.skip_cpu:
        line["cpu_baseline"] = cpu_baseline()
    print(json.dumps(rounded(line, 5)))


if __name__ == "__main__":
    main()
