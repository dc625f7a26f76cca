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
MEASURED_TRAFFIC_BYTES = 30_635_000


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

    def __init__(self, x, packed, scales, values, y):
        from mlkit_amd import native

        self.function = native.library().mk_packed_matvec
        self.keep = (x, packed, scales, values, y)
        self.arguments = (
            x.data_ptr(), native.MK_F16, packed.data_ptr(), scales.data_ptr(), native.MK_F16,
            values.data_ptr(), 16, None, None, 0, y.data_ptr(), x.shape[0], ROWS, WIDTH, GROUP,
            BITS, 1, -8.0, 1.0,
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


def main() -> None:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=2000)
    parser.add_argument("--warmup", type=int, default=200)
    parser.add_argument("--copies", type=int, default=18)
    parser.add_argument("--no-graph", action="store_true")
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--profile-launches", type=int, default=0,
                        help="for rocprofv3: only launch the M=1 matvec this many times, plus three "
                             "256 MiB device copies whose counters calibrate FETCH_SIZE / WRITE_SIZE")
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

    if options.profile_launches:
        x = torch.randn((1, WIDTH), device=device, generator=generator).half()
        y = torch.empty((1, ROWS), device=device, dtype=torch.float16)
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
    print(json.dumps(line))


if __name__ == "__main__":
    main()
