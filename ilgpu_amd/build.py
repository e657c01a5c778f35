"""Builds libilgpu_hip_algorithms.so for gfx950 with hipcc.

``python -m ilgpu_amd.build`` compiles every ``csrc/*.hip`` to an object file
(in parallel) and links them into ``ilgpu_amd/lib/libilgpu_hip_algorithms.so``.
hipcc cross-compiles, so no GPU is needed.  The shared library is kept in the
tree (git-ignored) so that it travels with the source to the machine that runs
it.
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


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
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
    print(build())
    print(build_host_example())
