"""Headline benchmark: INT4-g128 packed matvec, weight 4096x14336 (N x K), on one MI355X.

One step = one launch of the packed matvec at M=1 on the next of several distinct weight
copies (more than 512 MB in total, so the 256 MB Infinity Cache cannot serve the stream).
Prints ONE JSON line; `value` is the effective weight bandwidth (codes + scales bytes per
second) with every input resident in HBM.  `roofline` prices the same launches by their
algorithmic bytes; `cpu_baseline` times the oracle's reconstruct-then-matmul on host cores.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
"""

import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROWS, WIDTH, GROUP, BITS = 4096, 14336, 128, 4
CODE_BYTES = ROWS * WIDTH * BITS // 8
SCALE_BYTES = ROWS * (WIDTH // GROUP) * 2
WEIGHT_BYTES = CODE_BYTES + SCALE_BYTES
HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (see
# profiles/packed_matvec_stream4_int4_g128_4096x14336_m1.md), M=1.
MEASURED_TRAFFIC_BYTES = 30_641_000


def algorithmic_bytes(samples: int) -> int:
    return WEIGHT_BYTES + samples * WIDTH * 2 + samples * ROWS * 2


def make_copies(count: int, device: torch.device):
    """Distinct synthetic layers: seeded uniform codes and fp16 scales of the magnitude an
    N(0, 0.02^2) weight gives (absmax/8 of 128 normals ~ 0.0065)."""
    generator = torch.Generator(device=device).manual_seed(20240601)
    copies = []
    for _ in range(count):
        packed = torch.randint(0, 256, (CODE_BYTES,), dtype=torch.uint8, device=device, generator=generator)
        scales = (torch.rand((ROWS, WIDTH // GROUP), device=device, generator=generator) * 0.004 + 0.005).half()
        copies.append((packed, scales))
    return copies


class Launcher:
    """Pre-bound arguments of mk_packed_matvec for one (weight copy, M)."""

    def __init__(self, x, packed, scales, values, y, *, zeros=None, rows=ROWS, width=WIDTH, group=GROUP,
                 bits=BITS, uniform=True, grid_min=-8.0, grid_step=1.0):
        from mlkit_amd import native

        self.function = native.library().mk_packed_matvec
        self.keep = (x, packed, scales, values, y, zeros)
        self.arguments = (
            x.data_ptr(), native.dtype_code(x), packed.data_ptr(), scales.data_ptr(), native.dtype_code(scales),
            values.data_ptr(), values.numel(), None if zeros is None else zeros.data_ptr(), None, 0,
            y.data_ptr(), x.shape[0], rows, width, group, bits, int(uniform), grid_min, grid_step,
        )

    def __call__(self, stream: int) -> None:
        status = self.function(*self.arguments, stream)
        if status:
            from mlkit_amd import native

            native.check(status)


def timed_region(launchers, steps, warmup, use_graph=True):
    """Returns (seconds by wall clock, seconds by HIP events) for exactly `steps` launches."""
    stream = torch.cuda.current_stream()
    count = len(launchers)
    for step in range(warmup):
        launchers[step % count](stream.cuda_stream)
    torch.cuda.synchronize()
    graph = None
    if use_graph:
        try:
            side = torch.cuda.Stream()
            side.wait_stream(stream)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                capture = torch.cuda.current_stream().cuda_stream
                for step in range(steps):
                    launchers[(warmup + step) % count](capture)
            graph.replay()  # untimed: uploads the graph
            torch.cuda.synchronize()
        except Exception as error:  # capture unsupported: time eager launches instead
            print(f"[bench] graph capture unavailable ({error}); timing eager launches", file=sys.stderr)
            graph = None
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    started = time.perf_counter()
    begin.record()
    if graph is not None:
        graph.replay()
    else:
        raw = stream.cuda_stream
        for step in range(steps):
            launchers[(warmup + step) % count](raw)
    end.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - started
    return wall, begin.elapsed_time(end) / 1e3, graph is not None


def cpu_baseline():
    """Oracle reconstruct-then-matmul (unpack -> values[codes]*scale -> fp32 matmul) on the
    host cores, on the full 4096x14336 layer at M=1: a bounded number of repetitions."""
    from oracle import bitstream, matvec as oracle_matvec, scaling

    rng = np.random.default_rng(7)
    packed = rng.integers(0, 256, CODE_BYTES, dtype=np.uint8)
    scales = (rng.random((ROWS, WIDTH // GROUP), dtype=np.float32) * 0.004 + 0.005).astype(np.float16).astype(np.float32)
    values = scaling.int_values(4)
    x = rng.standard_normal((1, WIDTH), dtype=np.float32).astype(np.float16).astype(np.float32)
    threads = torch.get_num_threads()
    full = []
    budget = time.perf_counter() + 20.0
    dense = None
    while len(full) < 3 and (not full or time.perf_counter() < budget):
        started = time.perf_counter()
        dense = oracle_matvec.dequantise(packed, BITS, (ROWS, WIDTH), scales, values, GROUP)
        oracle_matvec.reconstruct_then_matmul(x, None, BITS, (ROWS, WIDTH), scales, values, GROUP, dense=dense)
        full.append(time.perf_counter() - started)
    matmul_only = []
    for _ in range(10):
        started = time.perf_counter()
        oracle_matvec.reconstruct_then_matmul(x, None, BITS, (ROWS, WIDTH), scales, values, GROUP, dense=dense)
        matmul_only.append(time.perf_counter() - started)
    seconds = float(np.median(full))
    return {
        "value": WEIGHT_BYTES / seconds / 1e9,
        "unit": "GB/s effective weight bandwidth",
        "cores": threads,
        "kind": "port",
        "sample": f"{len(full)} x full 4096x14336 INT4-g128 layer at M=1, oracle unpack+dequantise+fp32 matmul "
                  f"(numpy); median {seconds * 1e3:.0f} ms; matmul alone with the dense weight cached "
                  f"{float(np.median(matmul_only)) * 1e3:.2f} ms; os.cpu_count()={os.cpu_count()}",
    }


def _time(function, repeats=20, warmup=3):
    """Milliseconds per call by HIP events on the current stream (where the kernels launch)."""
    for _ in range(warmup):
        function()
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    begin.record()
    for _ in range(repeats):
        function()
    end.record()
    torch.cuda.synchronize()
    return begin.elapsed_time(end) / repeats


def gptq_layer(device: torch.device, generator: torch.Generator) -> dict:
    """GPTQ, INT4 g128, 4096 x 11008, refit = block = 128; the Hessian product and the Cholesky
    factorisation (outside the kernels of this repository) are timed apart."""
    import mlkit_amd as mk
    from mlkit_amd.quantization.core import Ctx

    rows, width = 4096, 11008
    target = (torch.randn((rows, width), device=device, generator=generator) * 0.02).half().float()
    inputs = torch.randn((16384, width), device=device, generator=generator).half()
    hot = torch.randperm(width, device=device, generator=generator)[: width // 100]
    inputs[:, hot] *= 30
    hessian = (inputs.float().T @ inputs.float()) / inputs.shape[0]
    del inputs
    from mlkit_amd.quantization import feedback

    def wall_ms(function, repeats=3):
        """Median wall-clock time of `function`, synchronised on both sides."""
        times = []
        for _ in range(repeats):
            torch.cuda.synchronize()
            started = time.perf_counter()
            function()
            torch.cuda.synchronize()
            times.append((time.perf_counter() - started) * 1e3)
        return sorted(times)[len(times) // 2]

    quantizer = mk.gptq(mk.int(4, group=128))
    result = quantizer(target, Ctx("warmup", H=hessian))
    factor_ms = wall_ms(lambda: mk.feedback_coefficients(hessian.clone(), 1))
    total_ms = wall_ms(lambda: quantizer(target, Ctx("down_proj", H=hessian)))
    # the sweep alone: the same call with the coefficients handed over ready-made
    ready = mk.feedback_coefficients(hessian.clone(), 1)
    original = feedback.feedback_coefficients
    feedback.feedback_coefficients = lambda *args, **kwargs: ready
    try:
        sweep_ms = wall_ms(lambda: quantizer(target, Ctx("down_proj", H=hessian)))
    finally:
        feedback.feedback_coefficients = original
    update_flops = sum(2 * rows * 128 * (width - stop) for stop in range(128, width, 128))
    rtn = mk.int(4, group=128)(target)
    return {
        "total_ms": total_ms, "coefficients_ms": factor_ms, "sweep_and_update_ms": sweep_ms,
        "columns_per_s": width / (sweep_ms / 1e3), "trailing_update_flops": update_flops,
        "proxy_loss": float(mk.proxy_loss(target, result.w, hessian)),
        "rtn_proxy_loss": float(mk.proxy_loss(target, rtn.w, hessian)),
    }


def other_kernels(device: torch.device) -> dict:
    """Timings of the other kernels of the path at the shapes of the benchmark configurations
    (`--kernels`); each entry carries its algorithmic bytes or flops and the rate they give."""
    import mlkit_amd as mk
    from mlkit_amd.kernels import hadamard, packed_linear, scalar_decode, scalar_encode
    from mlkit_amd.quantization.transforms import OnlineRotation
    from mlkit_amd.quantization.core import Ctx

    out = {}
    generator = torch.Generator(device=device).manual_seed(1)
    weight = (torch.randn((ROWS, WIDTH), device=device, generator=generator) * 0.02).half().float()
    elements = ROWS * WIDTH
    values = torch.arange(-8, 8, dtype=torch.float32, device=device)

    def entry(ms, nbytes=None, flops=None, **extra):
        record = {"ms": ms, **extra}
        if nbytes is not None:
            record.update(bytes=nbytes, GBps=nbytes / ms / 1e6, hbm_frac=nbytes / ms / 1e6 / HBM_PEAK_GBPS)
        if flops is not None:
            record.update(flops=flops, TFLOPs=flops / ms / 1e9)
        return record

    fit = lambda: scalar_encode.fit_scales(weight, GROUP, asym=False, reciprocal=0.125, value_minimum=-8.0,  # noqa: E731
                                           scale_format="fp16", store_zero=False)
    scales, _ = fit()
    out["fit_scales 4096x14336 g128"] = entry(_time(fit), elements * 4 + scales.numel() * 4)
    encode = lambda: scalar_encode.encode(weight, scales, None, values, GROUP, None, integer=True,  # noqa: E731
                                          minimum=-8.0, maximum=7.0)
    codes = encode()
    out["encode int4 4096x14336 g128"] = entry(_time(encode), elements * 5 + scales.numel() * 4)
    out["decode codes 4096x14336 g128"] = entry(
        _time(lambda: scalar_decode.decode(codes, scales, values, None, GROUP)), elements * 5 + scales.numel() * 4)
    seven = torch.tensor([-1, -0.5, -0.25, 0, 0.25, 0.5, 1], device=device)
    fractions = torch.linspace(0.5, 1.0, 20, device=device)
    square = weight[:, :4096].contiguous()
    base, _ = scalar_encode.fit_scales(square, 64, asym=False, reciprocal=1.0, value_minimum=-1.0,
                                       scale_format="fp16", store_zero=False)
    out["search_scales codebook7 4096x4096 g64, 21 candidates"] = entry(
        _time(lambda: scalar_encode.search_scales(square, base, None, seven, fractions, 64, None, "fp16",
                                                  integer=False, minimum=-1.0, maximum=1.0), repeats=5),
        4096 * 4096 * 4 + 2 * base.numel() * 4)
    packed = mk.pack(codes[:8], 4)  # layout only; the timed stream is synthetic
    packed = torch.randint(0, 256, (CODE_BYTES,), dtype=torch.uint8, device=device, generator=generator)
    dense = torch.empty((ROWS, WIDTH), device=device, dtype=torch.float16)
    layout = packed_linear.layout_for(BITS, WIDTH, GROUP)
    half_scales = scales.half()
    out["packed decode int4 4096x14336 -> fp16"] = entry(
        _time(lambda: packed_linear.decode(packed, half_scales, values, None, dense, GROUP, layout, True, -8.0, 1.0)),
        CODE_BYTES + SCALE_BYTES + elements * 2)

    rotated = torch.empty_like(weight)
    out["fwht 4096x14336 fp32 as 7x2048 blocks"] = entry(
        _time(lambda: hadamard.transform(weight.view(ROWS, 7, 2048), out=rotated.view(ROWS, 7, 2048))), elements * 8)
    tall = weight.view(WIDTH, ROWS)
    out["fwht 14336x4096 fp32"] = entry(_time(lambda: hadamard.transform(tall, out=rotated.view(WIDTH, ROWS))), elements * 8)
    out["rht 4096x14336 fp32 (28x512 Paley: fwht + basis mix)"] = entry(
        _time(lambda: mk.rht(weight, seed=3), repeats=5), elements * 8, launches=2)
    for samples in (1, 8):
        for width in (4096, 14336):
            x = torch.randn((samples, width), device=device, generator=generator).half()
            out[f"rht activations M={samples} K={width} fp16"] = {"us": _time(lambda: mk.rht(x, seed=3), 50) * 1e3}
            hook = OnlineRotation(3)
            out[f"online rotation hook M={samples} K={width} fp16"] = {"us": _time(lambda: hook(x), 50) * 1e3}

    # other matvec shapes and codecs, M = 1 and 8: HIP-graph launches through the C ABI over
    # enough distinct weight copies (> 512 MB) that the Infinity Cache cannot serve them
    def matvec(rows, width, group, bits, table, uniform, asym, label, dtype=torch.float16):
        code_bytes = rows * width * bits // 8
        count = max(2, min(40, -(-(512 * 2**20) // code_bytes)))
        streams = [torch.randint(0, 256, (code_bytes,), dtype=torch.uint8, device=device, generator=generator)
                   for _ in range(count)]
        side = (torch.rand((rows, width // group), device=device, generator=generator) * 0.004 + 0.005).half()
        zeros = side.clone() if asym else None
        for samples in (1, 8):
            x = torch.randn((samples, width), device=device, generator=generator).to(dtype)
            y = torch.empty((samples, rows), device=device, dtype=dtype)
            launchers = [Launcher(x, stream, side, table, y, zeros=zeros, rows=rows, width=width, group=group,
                                  bits=bits, uniform=uniform, grid_min=float(table[0]),
                                  grid_step=float(table[1] - table[0])) for stream in streams]
            _, seconds, _ = timed_region(launchers, 400, 40)
            nbytes = code_bytes + side.numel() * 2 * (2 if asym else 1) + samples * (width + rows) * 2
            out[f"matvec {label} {rows}x{width} M={samples}"] = entry(seconds / 400 * 1e3, nbytes, copies=count)

    nf4 = mk.NF4_VALUES.to(device)
    matvec(4096, 4096, 128, 4, values, True, True, "int4 asym g128")
    matvec(ROWS, WIDTH, 128, 4, values, True, False, "int4 g128, bf16 activations", dtype=torch.bfloat16)
    matvec(ROWS, WIDTH, 64, 2, torch.arange(-2, 2, dtype=torch.float32, device=device), True, False, "int2 g64")
    matvec(ROWS, WIDTH, 64, 3, torch.arange(-4, 4, dtype=torch.float32, device=device), True, False, "int3 g64")
    matvec(ROWS, WIDTH, 64, 4, nf4, False, False, "nf4 g64")
    matvec(ROWS, WIDTH, 64, 3, seven, False, False, "codebook7 g64")
    matvec(151936, 896, 128, 4, values, True, False, "int4 g128 (tied head)")
    matvec(ROWS, WIDTH, 128, 8, torch.arange(-128, 128, dtype=torch.float32, device=device), True, False, "int8 g128")
    for rows, width in ((896, 896), (128, 896), (4864, 896), (896, 4864)):
        matvec(rows, width, 128, 4, values, True, False, "int4 g128 (decoder layer)")
    del weight, rotated, dense, codes

    out["gptq int4 g128 4096x11008"] = gptq_layer(device, generator)
    return out


def main() -> None:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=2000)
    parser.add_argument("--warmup", type=int, default=200)
    parser.add_argument("--copies", type=int, default=18)
    parser.add_argument("--no-graph", action="store_true")
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--kernels", action="store_true",
                        help="also time the other kernels of the path (adds a `kernels` object to the line)")
    parser.add_argument("--profile-gptq", action="store_true",
                        help="for rocprofv3: only run the GPTQ layer (4096 x 11008) and print its timings")
    parser.add_argument("--profile-launches", type=int, default=0,
                        help="for rocprofv3: only launch the M=1 matvec this many times, plus three "
                             "256 MiB device copies whose counters calibrate FETCH_SIZE / WRITE_SIZE")
    parser.add_argument("--profile-rows", type=int, default=1,
                        help="activation rows M of the --profile-launches launches")
    options = parser.parse_args()
    if options.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a HIP device")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    values = torch.arange(-8, 8, dtype=torch.float32, device=device)
    copies = make_copies(options.copies, device)
    generator = torch.Generator(device=device).manual_seed(5)

    if options.profile_gptq:
        print(json.dumps(gptq_layer(device, generator)))
        return
    if options.profile_launches:
        x = torch.randn((options.profile_rows, WIDTH), device=device, generator=generator).half()
        y = torch.empty((options.profile_rows, ROWS), device=device, dtype=torch.float16)
        launchers = [Launcher(x, packed, scales, values, y) for packed, scales in copies]
        raw = torch.cuda.current_stream().cuda_stream
        for step in range(options.profile_launches):
            launchers[step % len(launchers)](raw)
        source = torch.empty(256 * 2**20, dtype=torch.uint8, device=device)
        target = torch.empty_like(source)
        for _ in range(3):
            target.copy_(source)
        torch.cuda.synchronize()
        return

    results = {}
    for samples in (1, 2, 4, 8):
        x = torch.randn((samples, WIDTH), device=device, generator=generator).half()
        y = torch.empty((samples, ROWS), device=device, dtype=torch.float16)
        launchers = [Launcher(x, packed, scales, values, y) for packed, scales in copies]
        wall, event_seconds, graphed = timed_region(launchers, options.steps, options.warmup,
                                                    use_graph=not options.no_graph)
        per_launch = event_seconds / options.steps
        resident = [launchers[0]]
        _, resident_seconds, _ = timed_region(resident, options.steps, options.warmup,
                                              use_graph=not options.no_graph)
        results[samples] = {
            "us_per_call": per_launch * 1e6,
            "wall_us_per_call": wall / options.steps * 1e6,
            "effective_weight_GBps": WEIGHT_BYTES / per_launch / 1e9,
            "algorithmic_GBps": algorithmic_bytes(samples) / per_launch / 1e9,
            "cache_resident_us_per_call": resident_seconds / options.steps * 1e6,
            "graph": graphed,
        }
    head = results[1]
    per_launch = head["us_per_call"] / 1e6
    achieved = algorithmic_bytes(1) / per_launch / 1e9
    line = {
        "metric": "effective weight GB/s, INT4-g128 packed matvec 4096x14336, M=1",
        "value": head["effective_weight_GBps"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": options.steps,
        "warmup": options.warmup,
        "ms_per_step": per_launch * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 activations, u4 codes, f32 accumulate",
        "data": "synthetic seeded codes and fp16 scales",
        "config": {
            "workload": "INT4 symmetric g128 packed matvec, weight 4096x14336 (N x K), M=1; "
                        f"{options.copies} distinct weight copies ({options.copies * WEIGHT_BYTES / 2**20:.0f} MiB) in rotation",
            "launch": "HIP graph of back-to-back launches" if head["graph"] else "eager launches",
            "by_rows": {str(k): v for k, v in results.items()},
        },
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "traffic": MEASURED_TRAFFIC_BYTES,
        },
        "cpu_baseline": None if options.no_cpu_baseline else cpu_baseline(),
    }
    if options.kernels:
        del copies, launchers
        torch.cuda.empty_cache()
        line["kernels"] = other_kernels(device)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
