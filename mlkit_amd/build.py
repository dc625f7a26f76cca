"""Builds ``libmlkit_amd.so`` for gfx950 with hipcc (cross-compiles without a GPU).

``python -m mlkit_amd.build`` compiles every translation unit under ``csrc/`` in
parallel and links the shared library beside this file.  Nothing here runs at import
time: loading a prebuilt library is ``mlkit_amd.native``'s job.
"""

import concurrent.futures
import os
import pathlib
import subprocess
import sys
import time

ROOT = pathlib.Path(__file__).resolve().parent
CSRC = ROOT / "csrc"
OBJECTS = CSRC / "_build"
LIBRARY = ROOT / "libmlkit_amd.so"
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

COMMON_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # hipcc may not form packed fp32 arithmetic on its own (flag for the device pass;
    # the host pass prints a harmless "not a recognized feature" warning).
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
# Kernels whose results are compared bit for bit keep multiply and add separate.
EXACT_FLAGS = ["-ffp-contract=off"]

MATVEC_WIDTHS = range(2, 9)


def translation_units() -> list[tuple[str, pathlib.Path, list[str]]]:
    units: list[tuple[str, pathlib.Path, list[str]]] = []
    for width in MATVEC_WIDTHS:
        units.append((f"packed_matvec_b{width}", CSRC / "packed_matvec_bits.hip",
                      [f"-DMK_MATVEC_BITS={width}"]))
    exact = {"packed_decode", "scalar_codec", "error_feedback", "hadamard", "vector_feedback"}
    for source in sorted(CSRC.glob("*.hip")):
        if source.name == "packed_matvec_bits.hip":
            continue
        units.append((source.stem, source, EXACT_FLAGS if source.stem in exact else []))
    return units


def _compile(unit: tuple[str, pathlib.Path, list[str]]) -> tuple[str, float, str]:
    name, source, extra = unit
    target = OBJECTS / f"{name}.o"
    started = time.time()
    command = [HIPCC, *COMMON_FLAGS, *extra, "-c", str(source), "-o", str(target)]
    result = subprocess.run(command, capture_output=True, text=True)
    log = "\n".join(line for line in (result.stdout + result.stderr).splitlines()
                    if "packed-fp32-ops' is not a recognized feature" not in line)
    if result.returncode != 0:
        raise RuntimeError(f"hipcc failed for {source.name}:\n{log}")
    return name, time.time() - started, log


def build(verbose: bool = True, jobs: int | None = None, only: list[str] | None = None) -> pathlib.Path:
    """Compile all units (or, while developing, just the units named in ``only``, reusing the
    other objects of an earlier full build) and link the library; returns its path."""
    OBJECTS.mkdir(exist_ok=True)
    units = translation_units()
    chosen = [unit for unit in units if not only or unit[0] in only]
    jobs = jobs or min(len(units), os.cpu_count() or 4, 16)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        for name, seconds, log in pool.map(_compile, chosen):
            if verbose:
                print(f"[mlkit_amd.build] {name}.o  {seconds:6.1f}s", flush=True)
                if log.strip():
                    print(log)
    objects = [str(OBJECTS / f"{name}.o") for name, _, _ in units]
    link = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", str(LIBRARY), *objects]
    result = subprocess.run(link, capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError(f"link failed:\n{result.stdout}{result.stderr}")
    if verbose:
        print(f"[mlkit_amd.build] linked {LIBRARY}", flush=True)
    return LIBRARY


if __name__ == "__main__":
    build(verbose=True, only=sys.argv[1:] or None)   # e.g. `python -m mlkit_amd.build hadamard`
    sys.exit(0)
