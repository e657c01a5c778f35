"""Builds libilgpu_hip_algorithms.so for gfx950 with hipcc.

``python -m ilgpu_amd.build`` compiles every ``csrc/*.hip`` to an object file
(in parallel) and links them into ``ilgpu_amd/lib/libilgpu_hip_algorithms.so``.
hipcc cross-compiles, so no GPU is needed.  The shared library is kept in the
tree (git-ignored) so that it travels with the source to the machine that runs
it.  The same call builds the C++ host-layer test program and the
micro-benchmarks of ``bench_bounds.hip``.

``python -m ilgpu_amd.build --variant NAME -D MACRO=VALUE [-D ...] [--units a,b]``
builds ``ilgpu_amd/lib/variants/libNAME.so``: the named units (default: all)
recompiled with the given tuning macros, the rest taken from the last full
build.  ``ILGPU_HIP_ALGORITHMS_LIB=<that file>`` makes ``ilgpu_amd.capi``, and
with it ``bench.py`` and the tests, load the variant: this is how the measured
alternatives quoted in the kernels' comments were timed.
"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(LIB_DIR, "obj")
LIB_NAME = "libilgpu_hip_algorithms.so"
LIB_PATH = os.path.join(LIB_DIR, LIB_NAME)

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# -packed-fp32-ops is switched off: hipcc otherwise forms v_pk_*_f32 from
# plain float code.  The host pass does not know the feature and says so.
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def sources() -> list[str]:
    return sorted(
        os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src: str, obj_dir: str = OBJ_DIR, defines: tuple[str, ...] = ()) -> str:
    obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC, *FLAGS, *(f"-D{d}" for d in defines), "-c", src, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(jobs: int | None = None) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, sources()))
    link = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB_PATH,
            *objs]
    proc = subprocess.run(link, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    return LIB_PATH


def build_variant(name: str, defines: list[str], units: list[str] | None = None) -> str:
    """Links a library whose `units` (file names in csrc/ without .hip; all of
    them when None) are compiled with -D<define> for every entry of `defines`;
    the other units come from the objects of the last full build.  The units
    that include radix_sort_impl.hpp go together: its macros size tiles, and the
    temp size one unit reports has to be the layout another one writes."""
    all_sources = sources()
    if units is not None and any(u.startswith("radix_sort") for u in units):
        units = sorted(set(units) | {os.path.basename(s)[:-4] for s in all_sources
                                     if os.path.basename(s).startswith("radix_sort")})
    chosen = [s for s in all_sources
              if units is None or os.path.basename(s)[:-4] in units]
    if units is not None and len(chosen) != len(units):
        raise ValueError(f"unknown unit in {units}")
    var_dir = os.path.join(LIB_DIR, "variants")
    obj_dir = os.path.join(var_dir, "obj_" + name)
    os.makedirs(obj_dir, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        new = list(pool.map(lambda s: _compile(s, obj_dir, tuple(defines)), chosen))
    kept = [os.path.join(OBJ_DIR, os.path.basename(s)[:-4] + ".o")
            for s in all_sources if s not in chosen]
    missing = [o for o in kept if not os.path.exists(o)]
    if missing:
        raise RuntimeError(f"run a full build first: {missing[0]} is missing")
    out = os.path.join(var_dir, f"lib{name}.so")
    proc = subprocess.run([HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", out,
                           *new, *kept], capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    return out


BOUNDS_SRC = os.path.join(os.path.dirname(HERE), "bench_bounds.hip")
BOUNDS_BIN = os.path.join(LIB_DIR, "bench_bounds")


def build_bounds() -> str:
    """Compiles the micro-benchmarks that bound the kernels (a program of its
    own: it does not link the library)."""
    os.makedirs(LIB_DIR, exist_ok=True)
    cmd = [HIPCC, *FLAGS, BOUNDS_SRC, "-o", BOUNDS_BIN]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"bench_bounds build failed:\n{proc.stderr}")
    return BOUNDS_BIN


HOST_TEST_SRC = os.path.join(os.path.dirname(HERE), "tests", "cpp",
                             "host_api_tests.cpp")
HOST_TEST_BIN = os.path.join(os.path.dirname(HERE), "tests", "cpp",
                             "host_api_tests")


def build_host_example() -> str:
    """Compiles the C++ host-layer test program against the built library."""
    cmd = [HIPCC, "-x", "c++", "-std=c++17", "-O2", "-D__HIP_PLATFORM_AMD__",
           "-I/opt/rocm/include", HOST_TEST_SRC, "-o", HOST_TEST_BIN,
           "-L" + LIB_DIR, "-lilgpu_hip_algorithms",
           "-L/opt/rocm/lib", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN/../../ilgpu_amd/lib", "-Wl,-rpath,/opt/rocm/lib"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"host test build failed:\n{proc.stderr}")
    return HOST_TEST_BIN


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--variant", help="name of a tuning variant to build instead of the library")
    ap.add_argument("-D", dest="defines", action="append", default=[], metavar="MACRO=VALUE")
    ap.add_argument("--units", help="comma-separated csrc units the macros apply to (default: all)")
    cli = ap.parse_args()
    if cli.variant:
        print(build_variant(cli.variant, cli.defines,
                            cli.units.split(",") if cli.units else None))
    else:
        print(build())
        print(build_host_example())
        print(build_bounds())
