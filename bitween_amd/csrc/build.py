"""Builds libbitween_hip.so (gfx950) next to its sources.

    python -m bitween_amd.csrc.build            the library
    python -m bitween_amd.csrc.build --tune     also libbitween_hip_tune.so, the measurement build (see build)

hipcc cross-compiles without a GPU.  The library is loaded by
bitween_amd.kernels.hip_loader; nothing is built at import time.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ["bw_quantize.hip", "bw_qgemv.hip", "bw_qgemm.hip", "bw_qgemm_rows.hip", "bw_qdgrad.hip"]
TUNE_SOURCES = ["bw_qgemm.hip", "bw_qgemm_rows.hip"]      # compiled a second time with -DBW_TUNE for the measurement build
LIB = os.path.join(HERE, "libbitween_hip.so")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off",                      # the quantiser's roundings must stay separate operations
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-function",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


TUNE_LIB = os.path.join(HERE, "libbitween_hip_tune.so")


def build(verbose=False, tune=False):
    """Compile every source to an object file (in parallel, one hipcc per file), then link the shared library.

    tune=True also makes libbitween_hip_tune.so, the measurement build: the same library with the prefill kernel
    compiled with -DBW_TUNE, which adds (1) kernel choices from the environment (BW_GEMM_NAT, BW_GEMM_BM,
    BW_GEMM_PANEL) for same-process A/B runs and (2) bw_tune_clock_buffer(): workgroups 0..255 of a prefill launch leave
    the core-clock and real-time ticks of their K loop there, from which the shader clock under that kernel follows
    (bench.py --only prefill_clock).  The package never loads it."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    compile_flags = [f for f in FLAGS if f != "-shared"] + ["-c"]
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in SOURCES]
    jobs = [[hipcc] + compile_flags + ["-o", o, os.path.join(HERE, s)] for s, o in zip(SOURCES, objs)]
    tune_objs = [os.path.join(objdir, s.replace(".hip", "_tune.o")) for s in TUNE_SOURCES]
    if tune:
        jobs += [[hipcc] + compile_flags + ["-DBW_TUNE", "-o", o, os.path.join(HERE, s)] for s, o in zip(TUNE_SOURCES, tune_objs)]
    with ThreadPoolExecutor(max_workers=min(len(jobs), os.cpu_count() or 1)) as pool:
        list(pool.map(lambda cmd: _run(cmd, verbose), jobs))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs, verbose)
    if tune:
        others = [o for s, o in zip(SOURCES, objs) if s not in TUNE_SOURCES]
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", TUNE_LIB] + tune_objs + others, verbose)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, tune="--tune" in sys.argv[1:]))
