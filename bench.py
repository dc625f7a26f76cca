"""Headline benchmark: INT4-g128 packed matvec, weight 4096x14336 (N x K), M=1, on one MI355X.

One step = one ``mk_packed_matvec`` call on one 4096x14336 weight matrix and one activation
row: the launch ``PackedLinear.forward`` issues per layer.  ``config`` also carries the same
call at M = 2, 4, 8 (``us_M*``, ``frac_M*``) and the grouped launch (``mk_packed_matvec_group``
over eight such matrices that read one activation row each, as the experts of a
mixture-of-experts layer or sibling projections do; ``--members 8`` makes that the step).
Weight copies rotate so that more than 512 MB of distinct weights pass between two uses of a
copy and the 256 MB Infinity Cache cannot serve the stream.

The timed region is a HIP graph of ``--steps`` calls; ``ms_per_step`` is the median over
``--replays`` timed replays (HIP events on the stream the graph runs on).  Prints ONE JSON line:
``value`` is the effective weight bandwidth (codes + scales bytes per second) with every input
resident in HBM; ``roofline`` prices the same launches by their algorithmic bytes;
``cpu_baseline`` times the CPU restatement (reconstruct-then-matmul, GPTQ sweep, Walsh-Hadamard
transform) on the host's cores; ``kernels`` holds the other kernels of the path with their own
roofline fractions (fp32 MFMA for the GPTQ trailing update, HBM for the rest).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--members G] [--replays R]
"""

import argparse
import json
import os
import statistics
import sys
import time

import numpy as np
import torch

ROWS, WIDTH, GROUP, BITS = 4096, 14336, 128, 4
CODE_BYTES = ROWS * WIDTH * BITS // 8
SCALE_BYTES = ROWS * (WIDTH // GROUP) * 2
WEIGHT_BYTES = CODE_BYTES + SCALE_BYTES
HBM_PEAK_GBPS = 8000.0
MFMA_FP32_PEAK_TFLOPS = 157.3
MINIMUM_ROTATING_BYTES = 512 * 2**20
# HBM bytes per matrix of a launch, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE; recorded, not
# measured by this script.
RECORDED_TRAFFIC = {
    "single": {"bytes_per_launch": 30_725_530,
               "source": "profiles/packed_matvec_long_rows_int4_g128_4096x14336_m1.md (rocprofv3 --pmc FETCH_SIZE, then "
                         "WRITE_SIZE); recorded there, not measured in this run"},
    "group_of_8": {"bytes_per_launch": 243_562_906,
                   "source": "profiles/packed_matvec_long_rows_int4_g128_4096x14336_m1_group8.md (rocprofv3 --pmc FETCH_SIZE, "
                             "then WRITE_SIZE of the 8-matrix launch); recorded there, not measured in this run"},
}


def algorithmic_bytes(samples: int) -> int:
    """Per matrix: codes + scales + the activation rows read + the outputs written."""
    return WEIGHT_BYTES + samples * WIDTH * 2 + samples * ROWS * 2


def make_copies(count: int, device: torch.device, rows=ROWS, width=WIDTH, group=GROUP, bits=BITS):
    """Distinct synthetic layers: seeded uniform codes and fp16 scales of the magnitude an
    N(0, 0.02^2) weight gives (absmax/8 of 128 normals ~ 0.0065)."""
    generator = torch.Generator(device=device).manual_seed(20240601)
    copies = []
    for _ in range(count):
        packed = torch.randint(0, 256, (rows * width * bits // 8,), dtype=torch.uint8, device=device, generator=generator)
        scales = (torch.rand((rows, width // group), device=device, generator=generator) * 0.004 + 0.005).half()
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


class GroupLauncher:
    """One mk_packed_matvec_group call over `members` weight copies that read `x`."""

    def __init__(self, x, members, values, *, rows=ROWS, width=WIDTH, group=GROUP):
        from mlkit_amd.kernels import packed_linear

        count = len(members)
        layout = packed_linear.layout_for(BITS, width, group)
        self.launch = packed_linear.GroupLaunch(
            [packed for packed, _ in members], [scales for _, scales in members], values, [None] * count, [None] * count,
            [rows] * count, width, group, layout, uniform_grid=True, grid_minimum=-8.0, grid_step=1.0)
        self.x = x
        self.outputs = [torch.empty((x.shape[0], rows), device=x.device, dtype=x.dtype) for _ in range(count)]

    def __call__(self, stream: int) -> None:
        self.launch(self.x, self.outputs, stream)


def timed_graph(launchers, steps, warmup, replays, minimum_span_ms=1.0):
    """Per-step seconds of a HIP graph of `steps` launches: the graph is replayed `replays`
    times, each timed by a pair of HIP events on the replay stream around enough back-to-back
    launches of the graph to span about a millisecond.  Returns (median, minimum, maximum,
    graph launches per timed replay)."""
    stream = torch.cuda.current_stream()
    count = len(launchers)
    for step in range(max(warmup, count)):
        launchers[step % count](stream.cuda_stream)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(stream)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        capture = torch.cuda.current_stream().cuda_stream
        for step in range(steps):
            launchers[(warmup + step) % count](capture)
    for _ in range(3):  # untimed: uploads the graph, warms the clocks
        graph.replay()
    torch.cuda.synchronize()
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    begin.record()
    graph.replay()
    end.record()
    torch.cuda.synchronize()
    batch = max(1, int(np.ceil(minimum_span_ms / max(begin.elapsed_time(end), 1e-3))))
    samples = []
    for _ in range(replays):
        begin.record()
        for _ in range(batch):
            graph.replay()
        end.record()
        torch.cuda.synchronize()
        samples.append(begin.elapsed_time(end) / 1e3 / (batch * steps))
    return statistics.median(samples), min(samples), max(samples), batch


def launch_floor(device: torch.device, values: torch.Tensor) -> float:
    """Seconds per call of the same entry point on a 16 x 32 layer (512 codes: no work to speak of), in the same
    kind of graph of back-to-back calls: what a dependent launch costs before any weight streams."""
    packed = torch.zeros(16 * 32 // 2, dtype=torch.uint8, device=device)
    scales = torch.ones((16, 1), dtype=torch.float16, device=device)
    x = torch.ones((1, 32), dtype=torch.float16, device=device)
    y = torch.empty((1, 16), dtype=torch.float16, device=device)
    tiny = Launcher(x, packed, scales, values, y, rows=16, width=32, group=32)
    return timed_graph([tiny], 200, 20, 20)[0]


def _blas_threads(limit: int | None):
    try:
        import threadpoolctl

        return threadpoolctl.threadpool_limits(limits=limit) if limit else threadpoolctl.threadpool_info()
    except Exception:  # threadpoolctl is optional
        return None


def cpu_matvec_baseline() -> dict:
    """The CPU restatement of the reference's CPU path, reconstruct-then-matmul (unpack ->
    values[codes] * scale -> fp32 matmul), on the whole 4096x14336 layer at M=1: as tensor
    operations on all of the host's cores (the reported value), and as numpy on one thread beside
    it.  Whole passes (reconstruction included) for about 10 s and 6 s, the first of each untimed;
    then the product alone on the reconstructed weight."""
    from oracle import matvec as oracle_matvec, scaling

    rng = np.random.default_rng(7)
    packed = rng.integers(0, 256, CODE_BYTES, dtype=np.uint8)
    scales = (rng.random((ROWS, WIDTH // GROUP), dtype=np.float32) * 0.004 + 0.005).astype(np.float16).astype(np.float32)
    values = scaling.int_values(4)
    x = rng.standard_normal((1, WIDTH), dtype=np.float32).astype(np.float16).astype(np.float32)

    def passes(function, seconds, most):
        times = []
        budget = time.perf_counter() + seconds
        while len(times) < most and (len(times) < 2 or time.perf_counter() < budget):
            started = time.perf_counter()
            function()
            times.append(time.perf_counter() - started)
        return float(np.median(times[1:]))      # the first pass warms the caches

    tensors = [torch.from_numpy(array) for array in (x, packed, scales, values)]
    threads = torch.get_num_threads()
    whole_torch = passes(lambda: oracle_matvec.reconstruct_then_matmul_torch(
        tensors[0], tensors[1], BITS, (ROWS, WIDTH), tensors[2], tensors[3], GROUP), 10.0, 12)
    _, dense = oracle_matvec.reconstruct_then_matmul_torch(tensors[0], tensors[1], BITS, (ROWS, WIDTH), tensors[2],
                                                           tensors[3], GROUP)
    product_torch = passes(lambda: oracle_matvec.reconstruct_then_matmul_torch(
        tensors[0], None, BITS, (ROWS, WIDTH), None, None, GROUP, dense=dense), 2.0, 12)
    del dense
    limiter = _blas_threads(1)
    try:
        whole_numpy = passes(lambda: oracle_matvec.reconstruct_then_matmul(
            x, packed, BITS, (ROWS, WIDTH), scales, values, GROUP), 6.0, 5)
    finally:
        if limiter is not None and hasattr(limiter, "restore_original_limits"):
            limiter.restore_original_limits()
    return {
        "value": WEIGHT_BYTES / whole_torch / 1e9,
        "unit": "GB/s effective weight bandwidth",
        "cores": threads,
        "kind": "port",
        "us_per_call": whole_torch * 1e6,
        "matmul_only_us_per_call": product_torch * 1e6,
        "one_thread_numpy_GBps": WEIGHT_BYTES / whole_numpy / 1e9,
        "os_cpu_count": os.cpu_count(),
        "sample": f"whole 4096x14336 INT4-g128 layer, M=1, reconstruct-then-matmul as torch tensor operations on "
                  f"{threads} threads (torch.get_num_threads()), median of the passes that fit 10 s: {whole_torch * 1e3:.0f} ms "
                  f"per call; the fp32 product alone on the reconstructed weight {product_torch * 1e3:.2f} ms; the numpy "
                  f"restatement on one thread {whole_numpy * 1e3:.0f} ms per call; os.cpu_count()={os.cpu_count()}",
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


def _entry(ms, nbytes=None, flops=None, **extra):
    record = {"ms": ms, **extra}
    if nbytes is not None:
        record.update(bytes=nbytes, GBps=nbytes / ms / 1e6, hbm_frac=nbytes / ms / 1e6 / HBM_PEAK_GBPS)
    if flops is not None:
        record.update(flops=flops, TFLOPs=flops / ms / 1e9)
    return record


def gptq_layer(device: torch.device, generator: torch.Generator, cpu_rows: int = 0) -> dict:
    """GPTQ, INT4 g128, 4096 x 11008, refit = block = 128.  The Hessian product and the Cholesky
    factorisation (outside the parity boundary) are timed apart; the wide trailing updates
    (`block_update_from_deviations_kernel`, fp32 matrix cores) are replayed on their own through
    mk_feedback_block_update_staged and priced against the fp32 MFMA peak; with `cpu_rows` the
    CPU restatement sweeps that many rows with the same coefficient matrix, is timed, and its
    codes are compared with the device's."""
    import mlkit_amd as mk
    from mlkit_amd import native
    from mlkit_amd.quantization import feedback
    from mlkit_amd.quantization.core import Ctx

    rows, width, block, deferred = 4096, 11008, 128, feedback.DEFERRED_TILES
    target = (torch.randn((rows, width), device=device, generator=generator) * 0.02).half().float()
    inputs = torch.randn((16384, width), device=device, generator=generator).half()
    hot = torch.randperm(width, device=device, generator=generator)[: width // 100]
    inputs[:, hot] *= 30
    hessian = torch.zeros((width, width), device=device)
    for band in inputs.split(2048):
        hessian.addmm_(band.float().T, band.float())
    hessian /= inputs.shape[0]
    del inputs

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
        # the same sweep on a table of sixteen values (NF4, one scale per 64 columns)
        table_quantizer = mk.gptq(mk.nf4(group=64))
        table_quantizer(target, Ctx("warmup", H=hessian))
        table_sweep_ms = wall_ms(lambda: table_quantizer(target, Ctx("down_proj", H=hessian)))
        # and on a table of 253 values (the e4m3 minifloat grid, one scale per 64 columns)
        wide_quantizer = mk.gptq(mk.scaled(mk.grid.fp("e4m3"), group=64))
        wide_quantizer(target, Ctx("warmup", H=hessian))
        wide_sweep_ms = wall_ms(lambda: wide_quantizer(target, Ctx("down_proj", H=hessian)))
    finally:
        feedback.feedback_coefficients = original
    update_flops = sum(2 * rows * block * (width - stop) for stop in range(block, width, block))
    rtn = mk.int(4, group=128)(target)
    out = {
        "total_ms": total_ms, "coefficients_ms": factor_ms, "sweep_and_update_ms": sweep_ms,
        "columns_per_s": width / (sweep_ms / 1e3), "weights_per_s": rows * width / (sweep_ms / 1e3),
        "nf4_g64_sweep_and_update_ms": table_sweep_ms,
        "e4m3_g64_sweep_and_update_ms": wide_sweep_ms,
        "trailing_update_flops": update_flops,
        "proxy_loss": float(mk.proxy_loss(target, result.w, hessian)),
        "rtn_proxy_loss": float(mk.proxy_loss(target, rtn.w, hessian)),
    }
    # The wide (deferred, chained) trailing updates of the sweep, replayed alone: every group of
    # `deferred` tiles updates all columns to its right in one launch.
    coefficients = ready[0]
    deviations = (target - result.w).T.contiguous()          # [width, rows], as the sweep stores them
    scratch = torch.zeros_like(target)
    library, stream = native.library(), native.current_stream(device)
    wide = [(start, start + deferred * block) for start in range(0, width, deferred * block)
            if start + deferred * block < width and (width - start - deferred * block) % 128 == 0]
    wide_flops = sum(2 * rows * deferred * block * (width - begin) for _, begin in wide)

    def replay_updates():
        for start, begin in wide:
            native.check(library.mk_feedback_block_update_staged(
                scratch.data_ptr(), deviations.data_ptr(), coefficients.data_ptr(), rows, width, start, block, deferred,
                begin, width, stream))

    update_ms = _time(replay_updates, repeats=5, warmup=2)
    tflops = wide_flops / update_ms / 1e9
    out["trailing_update_roofline"] = {
        "kernel": "block_update_from_deviations_kernel", "bound": "mfma", "achieved": tflops, "peak": MFMA_FP32_PEAK_TFLOPS,
        "unit": "TFLOP/s", "frac": tflops / MFMA_FP32_PEAK_TFLOPS, "launches": len(wide), "ms_all_launches": update_ms,
        "flops_all_launches": wide_flops,
        "note": f"the {len(wide)} chained launches ({deferred} tiles of {block} columns each, all columns to their right) that "
                f"carry {wide_flops / update_flops:.0%} of the layer's trailing-update flops",
    }
    del deviations, scratch
    if cpu_rows:
        from oracle import feedback as oracle_feedback, scaling

        picked = torch.linspace(0, rows - 1, cpu_rows, device=device).long()
        host_coefficients = coefficients.cpu().numpy()
        host_weight = target[picked].cpu().numpy()
        started = time.perf_counter()
        expected = oracle_feedback.sweep(host_weight, host_coefficients, scaling.int_values(4), group=128, integer=True,
                                         refit=128, block=128)
        seconds = time.perf_counter() - started
        mismatches = int((result.codes[picked].cpu().numpy() != expected["codes"]).sum())
        out["cpu_baseline"] = {
            "value": cpu_rows * width / seconds, "unit": "weights/s", "cores": int(os.environ.get("OMP_NUM_THREADS", 0)) or os.cpu_count(),
            "kind": "port",
            "sample": f"{cpu_rows} rows spread over the 4096 x 11008 layer, all 11008 columns, the C restatement of the sweep "
                      f"(OpenMP over rows) with the device's coefficient matrix: {seconds:.1f} s; device: "
                      f"{rows * width / (sweep_ms / 1e3):.3e} weights/s",
            "code_mismatches_vs_device": mismatches, "codes_compared": cpu_rows * width,
        }
    return out


def vector_ldlq_layer(device: torch.device, generator: torch.Generator, cpu_rows: int = 0) -> dict:
    """LDLQ with vector grids at the shapes of the reference's own benchmark cases
    (benchmarks/results: "algorithms/ldlq-e8p-step8/llama-attention-2048x2048",
    "ldlq-vector8-256-step8", "kernels/lattice_search/e8p-2m-vectors", "operations/nearest/..."):
    the E8P lattice and a 256-codeword 8-dimensional codebook, step 8, one region, one scale per
    row.  With `cpu_rows` the CPU restatement sweeps that many rows with the device's
    coefficient matrix and its codes are compared with the device's."""
    import mlkit_amd as mk
    from mlkit_amd.kernels import lattice_search
    from mlkit_amd.quantization import feedback
    from mlkit_amd.quantization.core import Ctx
    from mlkit_amd.quantization.lattice import device_table

    rows = width = 2048
    target = (torch.randn((rows, width), device=device, generator=generator) * 0.02).half().float()
    inputs = torch.randn((8192, width), device=device, generator=generator)
    hessian = inputs.T @ inputs / inputs.shape[0]
    del inputs
    codebook = torch.randn((256, 8), device=device, generator=generator)

    def wall_ms(function, repeats=5):
        times = []
        for _ in range(repeats):
            torch.cuda.synchronize()
            started = time.perf_counter()
            function()
            torch.cuda.synchronize()
            times.append((time.perf_counter() - started) * 1e3)
        return sorted(times)[len(times) // 2]

    out = {}
    vectors = torch.randn((2_000_000, 8), device=device, generator=generator)
    table = device_table(device)
    ms = _time(lambda: lattice_search.search(vectors, table), repeats=10)
    out["e8p search 2M vectors"] = {"ms": ms, "vectors_per_s": vectors.shape[0] / ms * 1e3}
    ms = _time(lambda: lattice_search.nearest(vectors[:1_000_000], codebook), repeats=10)
    out["nearest 1M vectors x 256 codewords"] = {"ms": ms, "vectors_per_s": 1e6 / ms * 1e3}
    large = torch.randn((65536, 8), device=device, generator=generator)
    ms = _time(lambda: lattice_search.nearest(vectors[:65536], large), repeats=5)
    out["nearest 65k vectors x 65k codewords"] = {"ms": ms, "vectors_per_s": 65536 / ms * 1e3}
    del vectors
    ready = mk.feedback_coefficients(hessian.clone(), 8)
    out["coefficients_ms"] = wall_ms(lambda: mk.feedback_coefficients(hessian.clone(), 8))
    for label, inner, lattice in (("e8p", mk.scaled(mk.grid.e8p(), group=None), True),
                                  ("vector8-256", mk.scaled(mk.grid.vector(codebook.cpu()), group=None), False)):
        quantizer = mk.ldlq(inner, step=8, backend="hip")
        result = quantizer(target, Ctx("warmup", H=hessian))
        total_ms = wall_ms(lambda: quantizer(target, Ctx("attention", H=hessian)))
        original = feedback.feedback_coefficients
        feedback.feedback_coefficients = lambda *args, **kwargs: ready
        try:
            sweep_ms = wall_ms(lambda: quantizer(target, Ctx("attention", H=hessian)))
        finally:
            feedback.feedback_coefficients = original
        direct = inner(target, Ctx("attention", H=hessian))
        entry = {"total_ms": total_ms, "sweep_and_update_ms": sweep_ms, "weights_per_s": rows * width / (sweep_ms / 1e3),
                 "proxy_loss": float(mk.proxy_loss(target, result.w, hessian)),
                 "direct_rounding_proxy_loss": float(mk.proxy_loss(target, direct.w, hessian))}
        if cpu_rows:
            from oracle import lattice as oracle_lattice

            picked = torch.linspace(0, rows - 1, cpu_rows, device=device).long()
            points = oracle_lattice.e8p_points() if lattice else codebook.cpu().numpy()
            host_coefficients, host_weight = ready[0].cpu().numpy(), target[picked].cpu().numpy()
            started = time.perf_counter()
            expected = oracle_lattice.vector_sweep(host_weight, host_coefficients, points, group=width, dimension=8,
                                                   lattice=lattice, refit=None, block=128)
            seconds = time.perf_counter() - started
            entry["cpu_baseline"] = {
                "value": cpu_rows * width / seconds, "unit": "weights/s", "cores": 1, "kind": "port",
                "sample": f"{cpu_rows} rows spread over the layer, all {width} columns, the numpy restatement of the "
                          f"sweep with the device's coefficient matrix: {seconds:.1f} s",
                "code_mismatches_vs_device": int((result.codes[picked].cpu().numpy() != expected["codes"]).sum()),
                "codes_compared": cpu_rows * width // 8,
            }
        out[f"ldlq {label} step 8, {rows}x{width}"] = entry
    return out


def rotated_layer(device: torch.device, generator: torch.Generator, values: torch.Tensor) -> dict:
    """Config 5: the rotated INT4-g128 layers at M = 1 and 8.  One step = the online rotation of
    the activations plus the packed matvec, enqueued by one mk_rotated_packed_matvec call; the
    unrotated matvec of the same layer is timed beside it.  The 14336-wide layer is rotated as
    the reference does it (a 28 x 28 Paley basis over blocks of 512) and as seven separate
    blocks of 2048."""
    from mlkit_amd import native
    from mlkit_amd.quantization.transforms import OnlineRotation

    library = native.library()
    out = {}
    for rows, width, block in ((ROWS, WIDTH, None), (WIDTH, 4096, None), (ROWS, WIDTH, 2048)):
        copies = make_copies(max(2, -(-MINIMUM_ROTATING_BYTES // (rows * width // 2))), device, rows=rows, width=width)
        order, power, basis, signs, scale, keep = OnlineRotation(17, block).launch_arguments(width, device)
        for samples in (1, 8):
            x = torch.randn((samples, width), device=device, generator=generator).half()
            y = torch.empty((samples, rows), device=device, dtype=torch.float16)
            rotated = torch.empty_like(x)

            def rotated_call(packed, scales):
                arguments = (x.data_ptr(), native.MK_F16, rotated.data_ptr(), order, power, basis, signs, scale,
                             packed.data_ptr(), scales.data_ptr(), native.MK_F16, values.data_ptr(), 16, None, None, 0,
                             y.data_ptr(), samples, rows, width, GROUP, BITS, 1, -8.0, 1.0)
                return lambda stream: native.check(library.mk_rotated_packed_matvec(*arguments, stream))

            with_rotation = [rotated_call(packed, scales) for packed, scales in copies]
            plain = [Launcher(x, packed, scales, values, y, rows=rows, width=width) for packed, scales in copies]
            rotated_s = timed_graph(with_rotation, 200, 20, 20)[0]
            plain_s = timed_graph(plain, 200, 20, 20)[0]
            label = f"{rows}x{width} M={samples}" + (f", separate blocks of {block}" if block else "")
            out[label] = {
                "rotation": (f"{order} separate fwht {power}" if block else f"{order} x {power}") if order > 1 else f"fwht {power}",
                "rotated_us": rotated_s * 1e6, "unrotated_us": plain_s * 1e6, "rotation_costs_us": (rotated_s - plain_s) * 1e6,
            }
        del copies
    return out


def other_kernels(device: torch.device, full: bool) -> dict:
    """The other kernels of the path at the shapes of the benchmark configurations; each entry
    carries its algorithmic bytes or flops and the rate they give.  `full` adds the decoder-layer
    shapes, the tied head and the wider codecs."""
    import mlkit_amd as mk
    from mlkit_amd.kernels import hadamard, packed_linear, scalar_decode, scalar_encode
    from mlkit_amd.quantization import bitstream

    out = {}
    generator = torch.Generator(device=device).manual_seed(1)
    weight = (torch.randn((ROWS, WIDTH), device=device, generator=generator) * 0.02).half().float()
    elements = ROWS * WIDTH
    values = torch.arange(-8, 8, dtype=torch.float32, device=device)

    fit = lambda: scalar_encode.fit_scales(weight, GROUP, asym=False, reciprocal=0.125, value_minimum=-8.0,  # noqa: E731
                                           scale_format="fp16", store_zero=False)
    scales, _ = fit()
    out["fit_scales 4096x14336 g128"] = _entry(_time(fit), elements * 4 + scales.numel() * 4)
    encode = lambda: scalar_encode.encode(weight, scales, None, values, GROUP, None, integer=True,  # noqa: E731
                                          minimum=-8.0, maximum=7.0)
    codes = encode()
    out["encode int4 4096x14336 g128"] = _entry(_time(encode), elements * 5 + scales.numel() * 4)
    out["decode codes 4096x14336 g128"] = _entry(
        _time(lambda: scalar_decode.decode(codes, scales, values, None, GROUP)), elements * 5 + scales.numel() * 4)
    # (the range check of the codes is collected in a device flag and read once afterwards, as mk.optimize does)
    overflow = torch.zeros(1, dtype=torch.int32, device=device)
    out["pack int4 4096x14336"] = _entry(_time(lambda: mk.pack(codes, 4, overflow=overflow), repeats=10), elements + elements // 2)
    bitstream.check_overflow(overflow, 4)
    stream = mk.pack(codes, 4)
    out["unpack int4 4096x14336"] = _entry(_time(lambda: mk.unpack(stream, 4, (ROWS, WIDTH)), repeats=10),
                                           elements + elements // 2)
    seven = torch.tensor([-1, -0.5, -0.25, 0, 0.25, 0.5, 1], device=device)
    fractions = torch.linspace(0.5, 1.0, 20, device=device)
    square = weight[:, :4096].contiguous()
    base, _ = scalar_encode.fit_scales(square, 64, asym=False, reciprocal=1.0, value_minimum=-1.0,
                                       scale_format="fp16", store_zero=False)
    search_ms = _time(lambda: scalar_encode.search_scales(square, base, None, seven, fractions, 64, None, "fp16",
                                                          integer=False, minimum=-1.0, maximum=1.0), repeats=5)
    # bound by vector-ALU work (an IEEE division and a table search per element and candidate), not by HBM
    out["search_scales codebook7 4096x4096 g64, 21 candidates"] = {
        "ms": search_ms, "bound": "valu", "bytes": 4096 * 4096 * 4 + 2 * base.numel() * 4,
        "candidate_elements_per_s": 21 * 4096 * 4096 / (search_ms / 1e3)}
    dense = torch.empty((ROWS, WIDTH), device=device, dtype=torch.float16)
    layout = packed_linear.layout_for(BITS, WIDTH, GROUP)
    half_scales = scales.half()
    out["packed decode int4 4096x14336 -> fp16"] = _entry(
        _time(lambda: packed_linear.decode(stream, half_scales, values, None, dense, GROUP, layout, True, -8.0, 1.0)),
        CODE_BYTES + SCALE_BYTES + elements * 2)

    rotated = torch.empty_like(weight)
    fwht_ms = _time(lambda: hadamard.transform(weight.view(ROWS, 7, 2048), out=rotated.view(ROWS, 7, 2048)))
    out["fwht 4096x14336 fp32 as 7x2048 blocks"] = _entry(fwht_ms, elements * 8)
    out["fwht_roofline"] = {"kernel": "fwht_rows_kernel<32> (a row in the registers of one wavefront)", "bound": "hbm", "achieved": elements * 8 / fwht_ms / 1e6,
                            "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": elements * 8 / fwht_ms / 1e6 / HBM_PEAK_GBPS,
                            "workload": "4096 x 14336 fp32 as 7 x 2048 blocks, read and written once"}
    tall = weight.view(WIDTH, ROWS)
    out["fwht 14336x4096 fp32"] = _entry(_time(lambda: hadamard.transform(tall, out=rotated.view(WIDTH, ROWS))), elements * 8)
    out["rht 4096x14336 fp32 (28x512 Paley)"] = _entry(_time(lambda: mk.rht(weight, seed=3), repeats=5), elements * 8)

    # other matvec shapes and codecs, M = 1 and 8: HIP-graph launches through the C ABI over
    # enough distinct weight copies (> 512 MB) that the Infinity Cache cannot serve them
    def matvec(rows, width, group, bits, table, uniform, asym, label, dtype=torch.float16, grouped=False,
               side_dtype=torch.float16):
        code_bytes = rows * width * bits // 8
        count = max(2, min(40, -(-MINIMUM_ROTATING_BYTES // code_bytes)))
        streams = [torch.randint(0, 256, (code_bytes,), dtype=torch.uint8, device=device, generator=generator)
                   for _ in range(count)]
        side = (torch.rand((rows, width // group), device=device, generator=generator) * 0.004 + 0.005).to(side_dtype)
        zeros = side.clone() if asym else None
        for samples in (1, 8):
            x = torch.randn((samples, width), device=device, generator=generator).to(dtype)
            y = torch.empty((samples, rows), device=device, dtype=dtype)
            launchers = [Launcher(x, stream, side, table, y, zeros=zeros, rows=rows, width=width, group=group,
                                  bits=bits, uniform=uniform, grid_min=float(table[0]),
                                  grid_step=float(table[1] - table[0])) for stream in streams]
            seconds = timed_graph(launchers, 200, 20, 20)[0]
            nbytes = (code_bytes + side.numel() * side.element_size() * (2 if asym else 1)
                      + samples * (width + rows) * x.element_size())
            out[f"matvec {label} {rows}x{width} M={samples}"] = _entry(seconds * 1e3, nbytes, copies=count)
            if grouped and count >= 16:   # eight matrices per launch (mk_packed_matvec_group)
                layout = packed_linear.layout_for(bits, width, group)
                calls = []
                for first in range(0, count - 7, 8):
                    launch = packed_linear.GroupLaunch(streams[first:first + 8], [side] * 8, table, [zeros] * 8, [None] * 8,
                                                       [rows] * 8, width, group, layout, uniform_grid=uniform,
                                                       grid_minimum=float(table[0]), grid_step=float(table[1] - table[0]))
                    outputs = [torch.empty((samples, rows), device=device, dtype=dtype) for _ in range(8)]
                    calls.append(lambda stream, launch=launch, outputs=outputs: launch(x, outputs, stream))
                seconds = timed_graph(calls, 50, 8, 20)[0]
                out[f"matvec {label} {rows}x{width} M={samples}, 8 matrices per launch"] = _entry(
                    seconds * 1e3, 8 * nbytes, us_per_matrix=seconds * 1e6 / 8, copies=count)

    nf4 = mk.NF4_VALUES.to(device)
    matvec(4096, 4096, 128, 4, values, True, True, "int4 asym g128")
    matvec(ROWS, WIDTH, 64, 2, torch.arange(-2, 2, dtype=torch.float32, device=device), True, False, "int2 g64", grouped=True)
    matvec(ROWS, WIDTH, 64, 3, torch.arange(-4, 4, dtype=torch.float32, device=device), True, False, "int3 g64", grouped=True)
    matvec(ROWS, WIDTH, 64, 4, nf4, False, False, "nf4 g64", grouped=True)
    matvec(ROWS, WIDTH, 64, 3, seven, False, False, "codebook7 g64", grouped=True)
    # fp32 activations and fp32 scales (what the reference's own fp32 tests use): digit planes against v_dot8_i32_i4
    matvec(ROWS, WIDTH, 128, 4, values, True, False, "int4 g128, fp32 activations and scales", dtype=torch.float32,
           side_dtype=torch.float32)
    if full:
        matvec(ROWS, WIDTH, 128, 4, values, True, False, "int4 g128, bf16 activations", dtype=torch.bfloat16)
        matvec(151936, 896, 128, 4, values, True, False, "int4 g128 (tied head)")
        # down projections of larger decoders: rows of more than 16384 codes (two spans of 2048 codes per wavefront)
        matvec(3584, 18944, 128, 4, values, True, False, "int4 g128 (K = 18944)")
        matvec(8192, 28672, 128, 4, values, True, False, "int4 g128 (K = 28672)")
        matvec(ROWS, WIDTH, 128, 8, torch.arange(-128, 128, dtype=torch.float32, device=device), True, False, "int8 g128")
        for rows, width in ((896, 896), (128, 896), (4864, 896), (896, 4864)):
            matvec(rows, width, 128, 4, values, True, False, "int4 g128 (decoder layer)")
    del weight, rotated, dense, codes
    out["rotated layers (config 5)"] = rotated_layer(device, generator, values)
    return out


# name -> (group, bits, table, uniform grid, activation and scale dtype)
PROFILE_CODECS = {
    "int4": None,
    "int2": (64, 2, [-2, -1, 0, 1], True, torch.float16),
    "int3": (64, 3, [-4, -3, -2, -1, 0, 1, 2, 3], True, torch.float16),
    "nf4": (64, 4, None, False, torch.float16),
    "codebook7": (64, 3, [-1, -0.5, -0.25, 0, 0.25, 0.5, 1], False, torch.float16),
    "int4-fp32": (128, 4, list(range(-8, 8)), True, torch.float32),
}


def codec_launchers(name: str, samples: int, device: torch.device, generator: torch.Generator) -> list:
    """Eager-call launchers of one of the other codecs at 4096 x 14336 over rotating weight copies (what
    other_kernels() times), for counter runs."""
    import mlkit_amd as mk

    group, bits, table, uniform, dtype = PROFILE_CODECS[name]
    table = mk.NF4_VALUES.to(device) if table is None else torch.tensor(table, dtype=torch.float32, device=device)
    code_bytes = ROWS * WIDTH * bits // 8
    count = max(2, min(40, -(-MINIMUM_ROTATING_BYTES // code_bytes)))
    streams = [torch.randint(0, 256, (code_bytes,), dtype=torch.uint8, device=device, generator=generator) for _ in range(count)]
    side = (torch.rand((ROWS, WIDTH // group), device=device, generator=generator) * 0.004 + 0.005).to(dtype)
    x = torch.randn((samples, WIDTH), device=device, generator=generator).to(dtype)
    y = torch.empty((samples, ROWS), device=device, dtype=dtype)
    return [Launcher(x, stream, side, table, y, rows=ROWS, width=WIDTH, group=group, bits=bits, uniform=uniform,
                     grid_min=float(table[0]), grid_step=float(table[1] - table[0])) for stream in streams]


def cpu_fwht_baseline() -> dict:
    """The stagewise CPU transform on 256 rows of 7 x 2048 blocks (numpy, one thread)."""
    from oracle import transforms

    rng = np.random.default_rng(3)
    rows = 256
    value = rng.standard_normal((rows * 7, 2048), dtype=np.float32)
    for _ in range(2):
        transforms.fwht(value)
    times = []
    for _ in range(10):
        started = time.perf_counter()
        transforms.fwht(value)
        times.append(time.perf_counter() - started)
    seconds = float(np.median(times))
    return {"value": value.size * 8 / seconds / 1e9, "unit": "GB/s (read + write once)", "cores": 1, "kind": "port",
            "sample": f"{rows} rows of the 4096 x 14336 fp32 matrix as 7 x 2048 blocks, stagewise numpy transform, 10 repetitions "
                      f"after 2 warm-ups, median {seconds * 1e3:.1f} ms"}


def main() -> None:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=100)
    parser.add_argument("--warmup", type=int, default=20)
    parser.add_argument("--members", type=int, default=1,
                        help="weight matrices per step: 1 = one mk_packed_matvec call (the metric's configuration), 2..8 = one "
                             "mk_packed_matvec_group call over that many matrices")
    parser.add_argument("--gptq-cpu-rows", type=int, default=4096,
                        help="rows of the 4096 x 11008 layer that the CPU restatement of the GPTQ sweep covers (all by default)")
    parser.add_argument("--replays", type=int, default=60, help="timed replays of the graph; the median is reported")
    parser.add_argument("--copies", type=int, default=0, help="distinct weight copies in rotation (default: enough for 512 MB "
                                                               "between two uses of a copy)")
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--skip-kernels", action="store_true", help="only the headline matvec (no GPTQ / FWHT / codec legs)")
    parser.add_argument("--headline-only", action="store_true",
                        help="for rocprofv3 --kernel-trace --stats: only the headline leg (M=1, one call per step, rotating copies), "
                             "so that every launch of the kernel in the trace is one of the timed workload")
    parser.add_argument("--kernels", action="store_true", help="add the decoder-layer shapes, the tied head and wider codecs")
    parser.add_argument("--profile-gptq", action="store_true",
                        help="for rocprofv3: only run the GPTQ layer (4096 x 11008) and print its timings")
    parser.add_argument("--profile-vector", action="store_true",
                        help="for rocprofv3: only run the vector-grid searches and LDLQ layers (2048 x 2048) and print their record")
    parser.add_argument("--profile-launches", type=int, default=0,
                        help="for rocprofv3: only issue this many eager calls (grouped with --members > 1), plus three "
                             "256 MiB device copies whose counters calibrate FETCH_SIZE / WRITE_SIZE")
    parser.add_argument("--profile-rows", type=int, default=1, help="activation rows M of the --profile-launches calls")
    parser.add_argument("--profile-codec", default="int4", choices=sorted(PROFILE_CODECS),
                        help="codec of the --profile-launches calls (4096 x 14336; int4 = the metric's INT4-g128)")
    options = parser.parse_args()
    if options.headline_only:
        options.skip_kernels = options.no_cpu_baseline = True
        options.members = 1
    if options.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a HIP device")
    if not 1 <= options.members <= 8:
        sys.exit("--members must be 1..8")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    values = torch.arange(-8, 8, dtype=torch.float32, device=device)
    members = options.members
    # Between two uses of a weight set at least 512 MB of other weights are streamed.
    sets = -(-MINIMUM_ROTATING_BYTES // (members * WEIGHT_BYTES)) + 1
    copy_count = max(options.copies, sets * members, 18)
    copy_count = -(-copy_count // 8) * 8 if 8 % members == 0 else -(-copy_count // (8 * members)) * 8 * members
    copies = make_copies(copy_count, device)
    generator = torch.Generator(device=device).manual_seed(5)

    if options.profile_gptq:
        print(json.dumps(gptq_layer(device, generator)))
        return
    if options.profile_vector:
        print(json.dumps(vector_ldlq_layer(device, generator)))
        return
    if options.profile_launches:
        x = torch.randn((options.profile_rows, WIDTH), device=device, generator=generator).half()
        if options.profile_codec != "int4":
            launchers = codec_launchers(options.profile_codec, options.profile_rows, device, generator)
        elif members > 1:
            launchers = [GroupLauncher(x, copies[index:index + members], values) for index in range(0, copy_count, members)]
        else:
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
    flat = {}
    head_step = None
    for samples in ((1,) if options.headline_only else (1, 2, 4, 8)):
        x = torch.randn((samples, WIDTH), device=device, generator=generator).half()
        y = torch.empty((samples, ROWS), device=device, dtype=torch.float16)
        single = [Launcher(x, packed, scales, values, y) for packed, scales in copies]
        row = {}
        head = samples == 1 and members == 1
        steps = options.steps if head else max(options.steps, 50)
        replays = options.replays if head else max(20, options.replays // 2)
        median, low, high, batch = timed_graph(single, steps, options.warmup, replays)
        if head:
            head_step = (median, low, high, batch, steps, replays)
        row["single_call"] = {"us_per_matrix": median * 1e6, "min_us": low * 1e6, "max_us": high * 1e6,
                              "hbm_frac": algorithmic_bytes(samples) / median / 1e9 / HBM_PEAK_GBPS}
        if options.headline_only:
            results[samples] = row
            flat[f"us_M{samples}"] = median * 1e6
            flat[f"frac_M{samples}"] = row["single_call"]["hbm_frac"]
            break
        resident = timed_graph([single[0]], max(options.steps, 50), options.warmup, 10)[0]
        row["single_call"]["cache_resident_us"] = resident * 1e6
        flat[f"us_M{samples}"] = median * 1e6
        flat[f"frac_M{samples}"] = row["single_call"]["hbm_frac"]
        flat[f"cache_resident_us_M{samples}"] = resident * 1e6
        for count in sorted({2, 4, 8, members} - {1}):
            grouped = [GroupLauncher(x, copies[index:index + count], values) for index in range(0, copy_count - count + 1, count)]
            head = samples == 1 and count == members
            steps = options.steps if head else max(options.steps // 2, 25)
            replays = options.replays if head else max(20, options.replays // 3)
            median, low, high, batch = timed_graph(grouped, steps, options.warmup, replays)
            row[f"group_of_{count}"] = {"us_per_call": median * 1e6, "us_per_matrix": median * 1e6 / count,
                                        "min_us_per_matrix": low * 1e6 / count, "max_us_per_matrix": high * 1e6 / count,
                                        "hbm_frac": algorithmic_bytes(samples) * count / median / 1e9 / HBM_PEAK_GBPS}
            if count == 8:
                flat[f"group_of_8_us_per_matrix_M{samples}"] = median * 1e6 / count
                flat[f"group_of_8_frac_M{samples}"] = row["group_of_8"]["hbm_frac"]
            if head:
                head_step = (median, low, high, batch, steps, replays)
            del grouped
        results[samples] = row
    floor = launch_floor(device, values)
    flat["launch_floor_us"] = floor * 1e6
    flat["us_M1_above_launch_floor"] = flat["us_M1"] - floor * 1e6
    per_step, low, high, batch, steps, replays = head_step
    achieved = algorithmic_bytes(1) * members / per_step / 1e9
    traffic = RECORDED_TRAFFIC["group_of_8" if members == 8 else "single"] if members in (1, 8) else None
    one_step = ("one mk_packed_matvec call (one launch of one matrix, what PackedLinear.forward issues per layer)" if members == 1
                else f"one mk_packed_matvec_group call over {members} such matrices (one launch)")
    line = {
        "metric": "effective weight GB/s, INT4-g128 packed matvec 4096x14336, M=1",
        "value": WEIGHT_BYTES * members / per_step / 1e9,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": options.warmup,
        "ms_per_step": per_step * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 activations, u4 codes, f32 accumulate",
        "data": "synthetic seeded codes and fp16 scales",
        "config": {
            "workload": f"INT4 symmetric g128 packed matvec, weight 4096x14336 (N x K), M=1; one step = {one_step}; "
                        f"{copy_count} distinct weight copies ({copy_count * WEIGHT_BYTES / 2**20:.0f} MiB) in rotation",
            "matrices_per_step": members,
            "us_per_call": per_step * 1e6,
            "launch": "HIP graph of `steps` back-to-back calls on one stream",
            "replays": replays, "graph_launches_per_timed_replay": batch, "statistic": "median",
            "min_ms_per_step": low * 1e3, "max_ms_per_step": high * 1e3,
            **flat,
        },
        "roofline": {
            "kernel": ("long_rows_kernel<1,false,16,f16> (one launch per step)" if members == 1 else
                       f"long_rows_kernel<1,false,16,f16> (one grouped launch of {members} matrices per step)"),
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "algorithmic_bytes_per_launch": algorithmic_bytes(1) * members,
            "traffic": None if traffic is None else traffic["bytes_per_launch"],
            "traffic_source": None if traffic is None else traffic["source"],
        },
        "cpu_baseline": None if options.no_cpu_baseline else cpu_matvec_baseline(),
        "by_rows": {str(k): v for k, v in results.items()},
    }
    if not options.skip_kernels:
        del copies, single
        torch.cuda.empty_cache()
        kernels = other_kernels(device, options.kernels)
        kernels["gptq int4 g128 4096x11008"] = gptq_layer(device, generator, cpu_rows=0 if options.no_cpu_baseline else options.gptq_cpu_rows)
        kernels["vector grids"] = vector_ldlq_layer(device, generator, cpu_rows=0 if options.no_cpu_baseline else 16)
        if not options.no_cpu_baseline:
            kernels["fwht_cpu_baseline"] = cpu_fwht_baseline()
        line["kernels"] = kernels
        line["config"].update(kernel_summary(kernels))
    # the record's first fields are the contract's; nested detail follows, floats cut to five digits
    print(json.dumps(compact(line)))


def kernel_summary(kernels: dict) -> dict:
    """Flat scalars of the other kernels' figures, for records that keep scalars only."""
    flat = {}
    for label, entry in kernels.items():
        if label.startswith("matvec ") and isinstance(entry, dict) and "ms" in entry:
            key = label[len("matvec "):].replace(" ", "_").replace(",", "")
            flat[f"us:{key}"] = entry.get("us_per_matrix", entry["ms"] * 1e3)
            flat[f"frac:{key}"] = entry["hbm_frac"]
        elif isinstance(entry, dict) and "hbm_frac" in entry:
            flat[f"frac:{label.replace(' ', '_')}"] = entry["hbm_frac"]
    search = kernels.get("search_scales codebook7 4096x4096 g64, 21 candidates")
    if search:
        flat["search_scales_ms"] = search["ms"]
    gptq = kernels.get("gptq int4 g128 4096x11008", {})
    if gptq:
        flat["gptq_sweep_and_update_ms"] = gptq["sweep_and_update_ms"]
        flat["gptq_coefficients_ms"] = gptq["coefficients_ms"]
        flat["gptq_trailing_update_mfma_frac"] = gptq["trailing_update_roofline"]["frac"]
        flat["gptq_proxy_loss"] = gptq["proxy_loss"]
        if "cpu_baseline" in gptq:
            flat["gptq_cpu_weights_per_s"] = gptq["cpu_baseline"]["value"]
            flat["gptq_cpu_cores"] = gptq["cpu_baseline"]["cores"]
            flat["gptq_codes_compared"] = gptq["cpu_baseline"]["codes_compared"]
            flat["gptq_code_mismatches"] = gptq["cpu_baseline"]["code_mismatches_vs_device"]
    for label, entry in kernels.get("rotated layers (config 5)", {}).items():
        key = label.replace(" ", "_").replace(",", "")
        flat[f"rotated_us:{key}"] = entry["rotated_us"]
        flat[f"unrotated_us:{key}"] = entry["unrotated_us"]
    return flat


def compact(value):
    if isinstance(value, float):
        return float(f"{value:.5g}")
    if isinstance(value, dict):
        return {key: compact(item) for key, item in value.items()}
    if isinstance(value, (list, tuple)):
        return [compact(item) for item in value]
    return value


if __name__ == "__main__":
    main()
