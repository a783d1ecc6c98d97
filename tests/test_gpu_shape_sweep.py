"""Seeded random shapes through the automatic kernel selection, both
directions, against an fp64 product over the device's own dequantised weight
(which test_gpu_parity.py pins bit for bit to the oracle).  The shapes the
other GPU tests name were chosen with the kernels in mind; these are not:
block sizes 32...256, row widths from 8 to 28672 weights, output widths that
are multiples of nothing, row counts on both sides of every kernel family's
limits, both scale encodings with small and large second-level groups, with
and without bias, and the forward with a low-rank adapter.  The bar is the
suite's:
    max|gpu - exact| / (sqrt(K) * rms(activations) * rms(deq W)) <= 1e-5
(K at least 64, so that tiny contractions are not held to fewer roundings than
they perform).  A sweep like this one found the single accumulator chain of
the small-batch forward on 28672 x 8192 (1.5e-5)."""
import random

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TOLERANCE = 1.0e-5


def synthetic_weight(package, torch, out_w, in_w, block, double_quantized,
                     second_level_block, seed, code_offset=0):
    """A packed weight made on the device: random codes, block scales in
    [0.035, 0.065] (fp32) or random scale codes over second-level scales in
    [0.02, 0.03] with offset 0.05 (nested).  code_offset: bytes by which the
    code array is moved off its 256-byte aligned allocation."""
    generator = torch.Generator(device="cuda")
    generator.manual_seed(seed)
    count = out_w * in_w
    blocks = count // block
    codes = torch.randint(0, 256, (count // 2 + code_offset,),
                          dtype=torch.uint8, device="cuda",
                          generator=generator)[code_offset:]
    if not double_quantized:
        scales = torch.rand(blocks, device="cuda",
                            generator=generator) * 0.03 + 0.035
        return package.DeviceWeight(out_w, in_w, block, package.SCALE_FLOAT32,
                                    codes, scales, None)
    scale_codes = torch.randint(1, 256, (blocks,), dtype=torch.uint8,
                                device="cuda", generator=generator)
    groups = -(-blocks // second_level_block)
    second = torch.rand(groups, device="cuda",
                        generator=generator) * 0.01 + 0.02
    return package.DeviceWeight(
        out_w, in_w, block, package.SCALE_DOUBLE_QUANTIZED_UINT8, codes,
        scale_codes, second, second_level_block, 0.05)


def draw_case(rng, wide):
    if wide:
        block = 64
        in_w = rng.choice([256, 1024, 3072, 4096, 5120, 8192, 11008, 12352,
                           13824, 16448, 20480, 28672])
        out_w = rng.choice([64, 200, 512, 1000, 2048, 4096, 5000, 8192,
                            16384])
        rows = rng.choice([1, 2, 3, 4, 5, 16, 17, 48, 64, 65, 69, 80, 96, 97,
                           112, 113, 128, 129, 150, 192, 193, 224, 225, 256,
                           257, 300, 320, 448, 512, 1024, 2048])
    else:
        block = rng.choice([32, 64, 64, 128, 256])
        in_w = rng.choice([1, 2, 3, 5, 8, 16, 17, 33, 43, 64, 86, 100,
                           160]) * rng.choice([block, block, 64, 16, 8])
        out_w = rng.choice([8, 24, 64, 72, 100, 130, 257, 1000, 1024, 2047,
                            4096, 4100, 6000])
        rows = rng.choice([1, 2, 3, 4, 5, 7, 16, 17, 33, 63, 64, 65, 100, 128,
                           129, 200, 257, 300])
    return block, in_w, out_w, rows


@pytest.mark.parametrize("seed,wide", [(7, True), (11, True), (3, False),
                                       (4, False)])
def test_random_shapes_through_the_automatic_selection(gpu, package, library,
                                                       seed, wide):
    import torch
    rng = random.Random(seed)
    families = set()
    done = 0
    while done < 60:
        block, in_w, out_w, rows = draw_case(rng, wide)
        count = out_w * in_w
        if count % block or count % 2 or in_w > 32768 or count > 2 ** 28:
            continue
        double_quantized = rng.random() < 0.5
        second_level_block = rng.choice([32, 256])
        with_bias = rng.random() < 0.5
        rank = rng.choice([1, 4, 16, 33])
        # one case in six hands over arrays that are off the alignment the
        # fast kernels need (codes by 1-7 bytes, activations by 4-12): the
        # selection has to notice and fall back
        code_offset = rng.choice([1, 2, 4, 7]) if rng.random() < 0.17 else 0
        shift = rng.choice([1, 2, 3]) if rng.random() < 0.17 else 0
        label = (f"seed {seed} case {done}: block {block}, W {out_w}x{in_w}, "
                 f"{rows} rows, nested {double_quantized}/"
                 f"{second_level_block}, bias {with_bias}, rank {rank}, "
                 f"codes +{code_offset} B, activations +{4 * shift} B")
        weight = synthetic_weight(package, torch, out_w, in_w, block,
                                  double_quantized, second_level_block,
                                  1000 * seed + done, code_offset)
        deq = gpu.dequantize(weight).double()
        weight_rms = float(deq.pow(2).mean().sqrt())
        x = torch.randn(rows * in_w + shift,
                        device="cuda")[shift:].view(rows, in_w)
        dy = (torch.randn(rows * out_w + shift, device="cuda") *
              0.01)[shift:].view(rows, out_w)
        assert x.data_ptr() % 16 == 4 * shift
        bias = torch.randn(out_w, device="cuda") * 0.01 if with_bias else None
        forward_scale = (np.sqrt(max(in_w, 64)) *
                         float(x.pow(2).mean().sqrt()) * weight_rms)
        backward_scale = (np.sqrt(max(out_w, 64)) *
                          float(dy.pow(2).mean().sqrt()) * weight_rms)

        exact = x.double() @ deq.T
        if bias is not None:
            exact = exact + bias.double()[None, :]
        y = gpu.linear_forward(x, weight, bias)
        error = float((y.double() - exact).abs().max()) / forward_scale
        assert error <= TOLERANCE, f"{label}: forward {error:.3g}"

        dx = gpu.linear_input_backward(dy, weight)
        error = float((dx.double() - dy.double() @ deq).abs().max()) / \
            backward_scale
        assert error <= TOLERANCE, f"{label}: input backward {error:.3g}"

        a = torch.randn(rank, in_w, device="cuda") * 0.05
        b = torch.randn(out_w, rank, device="cuda") * 0.05
        with_adapter = gpu.lora_linear_forward(x, weight, a, b, 0.5,
                                               bias=bias)[0]
        term = 0.5 * (x.double() @ a.double().T) @ b.double().T
        # the adapter's own sums (rank and row width long) round like fp32
        # sums of their size: allow them their share
        slack = 4.0e-7 * float(term.abs().max())
        error = float((with_adapter.double() - (exact + term)).abs().max())
        assert error <= TOLERANCE * forward_scale + slack, \
            f"{label}: forward with adapter {error / forward_scale:.3g}"

        families.add(package.ALGORITHM_NAMES[library.select_algorithm(
            package.FORWARD, rows, in_w, out_w, block)])
        done += 1
        del deq, exact, y, dx, with_adapter, term, weight
    # a sweep that no longer reaches the kernel families tests nothing
    assert {"gemv", "mfma", "skinny"} <= families, families


@pytest.mark.parametrize("seed", [5, 6])
def test_random_groups_with_adapters_equal_single_calls(gpu, package, library,
                                                        seed):
    """rthip_nf4_lora_linear_forward_group on random groups: two to five
    members of one x, each with or without bias and with or without an
    adapter of rank 1...33 (its x.A^T taken by the call or beforehand), row
    widths and row counts on both sides of what the decode kernel and the
    kernel that keeps x in registers take.  Every output, and every x.A^T,
    equals the member's own call bit for bit."""
    import torch
    rng = random.Random(seed)
    generator = torch.Generator(device="cuda")
    generator.manual_seed(seed)
    normal = lambda *shape: torch.randn(*shape, device="cuda",  # noqa: E731
                                        generator=generator)
    for case in range(40):
        in_w = rng.choice([256, 1024, 2048, 4096, 5120, 11008, 12352])
        rows = rng.choice([1, 2, 3, 4, 5, 16, 33, 64, 128, 129])
        double_quantized = rng.random() < 0.5
        widths = [rng.choice([64, 72, 100, 512, 1000, 1024, 4096])
                  for _ in range(rng.choice([2, 3, 4, 5]))]
        weights = [synthetic_weight(package, torch, width, in_w, 64,
                                    double_quantized, 256,
                                    1000 * seed + 10 * case + m)
                   for m, width in enumerate(widths)]
        x = normal(rows, in_w)
        adapters, biases = [], []
        for width in widths:
            adapters.append(None)
            if rng.random() < 0.6:
                rank = rng.choice([1, 4, 8, 16, 33])
                adapters[-1] = (normal(rank, in_w) * 0.05,
                                normal(width, rank) * 0.05,
                                rng.choice([0.5, 2.0]))
            biases.append(normal(width) * 0.01 if rng.random() < 0.5
                          else None)
        outputs, products = gpu.lora_linear_forward_group(
            x, weights, adapters, biases, reduce_first=rng.random() < 0.3)
        torch.cuda.synchronize()
        label = (f"seed {seed} case {case}: I={in_w} rows={rows} "
                 f"widths={widths}")
        for m, weight in enumerate(weights):
            if adapters[m] is None:
                want = gpu.linear_forward(x, weight, biases[m])
            else:
                lora_a, lora_b, scale = adapters[m]
                want, own = gpu.lora_linear_forward(x, weight, lora_a, lora_b,
                                                    scale, bias=biases[m])
                assert torch.equal(own, products[m]), \
                    f"{label}: x.A^T of member {m}"
            assert torch.equal(want, outputs[m]), f"{label}: member {m}"
