"""Builds libdcp_hip.so (the C-ABI kernel library) in-tree with hipcc.

``python -m dcp_amd.build`` compiles every source under ``dcp_amd/csrc`` for
gfx950 and links ``dcp_amd/libdcp_hip.so``.  hipcc cross-compiles, so no GPU is
needed to build.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
INCLUDE = PKG_DIR.parent / "include"
LIB_PATH = Path(os.environ.get("DCP_LIB_PATH", PKG_DIR / "libdcp_hip.so"))
BUILD_DIR = PKG_DIR / "csrc" / "build"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wno-unused-value",
    f"-I{INCLUDE}",
    f"-I{CSRC}",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    # the attention kernels unroll whole tile streams (48 matrix instructions with their operand
    # reads and vector work); the default budget for "#pragma unroll" stops short of that
    "-mllvm",
    "-pragma-unroll-threshold=262144",
]


# extra compiler flags for experiments, e.g. DCP_EXTRA_HIPCC_FLAGS="-DFOO=1"
FLAGS += os.environ.get("DCP_EXTRA_HIPCC_FLAGS", "").split()


def sources():
    return sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.cpp")))


def _compile(src: Path) -> Path:
    obj = BUILD_DIR / (src.name + ".o")
    lang = ["-x", "hip"] if src.suffix == ".cpp" else []
    cmd = [HIPCC, *FLAGS, *lang, "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{proc.stderr}")
    return obj


def build(verbose: bool = True) -> Path:
    BUILD_DIR.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        objs = list(pool.map(_compile, srcs))
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(LIB_PATH)]
    cmd += [str(o) for o in objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources", file=sys.stderr)
    return LIB_PATH


HOST_CHECK_SRC = PKG_DIR.parent / "tests" / "abi_host" / "abi_host_check.cpp"
HOST_CHECK_BIN = HOST_CHECK_SRC.with_suffix("")


def build_abi_host_check(verbose: bool = True) -> Path:
    """Compiles the plain C++ host program of tests/abi_host against the built library (it
    includes only include/dcp_hip.h and the HIP runtime).  The GPU test runs the binary."""
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-O2", "-std=c++17", f"-I{INCLUDE}", str(HOST_CHECK_SRC),
           "-o", str(HOST_CHECK_BIN), f"-L{LIB_PATH.parent}", "-ldcp_hip", "-Wl,-rpath,$ORIGIN/../../dcp_amd", f"-Wl,-rpath,{LIB_PATH.parent}"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"host check failed to build:\n{proc.stderr}")
    if verbose:
        print(f"built {HOST_CHECK_BIN}", file=sys.stderr)
    return HOST_CHECK_BIN


PROBES_SRC = PKG_DIR.parent / "bench_probes.hip"
PROBES_LIB = PKG_DIR.parent / "libbench_probes.so"


def build_bench_probes(verbose: bool = True) -> Path:
    """Compiles bench_probes.hip (two measurement-only kernels that bench.py runs beside the
    product library) into libbench_probes.so next to bench.py.  Not part of libdcp_hip.so."""
    cmd = [HIPCC, *FLAGS, "-shared", str(PROBES_SRC), "-o", str(PROBES_LIB)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"bench probes failed to build:\n{proc.stderr}")
    if verbose:
        print(f"built {PROBES_LIB}", file=sys.stderr)
    return PROBES_LIB


if __name__ == "__main__":
    build()
    if LIB_PATH.name == "libdcp_hip.so":  # the host check links the library by its name
        build_abi_host_check()
        build_bench_probes()
