"""Builds the reference's own C++ stage packer into ``oracle/_ref/`` (test infrastructure).

The reference ships one natively compiled routine, ``dcp_cpp.greedy_selection_per_device``
(csrc/interface.cpp, csrc/pipeline_generator/pipeline_generator.{cpp,hpp}: a pybind11 module
with no other dependency).  Where the reference tree is present this script compiles those
sources where they lie -- nothing is copied -- into ``oracle/_ref/dcp_cpp<ext>.so``, which the
stage-packer tests load as the checker.  Without the reference tree it does nothing.

    python oracle/build_ref.py [reference root, default /root/reference]
"""

from __future__ import annotations

import subprocess
import sys
import sysconfig
from pathlib import Path

HERE = Path(__file__).resolve().parent
OUT_DIR = HERE / "_ref"


def module_path() -> Path:
    return OUT_DIR / ("dcp_cpp" + sysconfig.get_config_var("EXT_SUFFIX"))


def build(reference_root: str = "/root/reference", verbose: bool = True):
    """Returns the path of the built module, or None if the reference sources are absent."""
    root = Path(reference_root)
    sources = [root / "csrc" / "interface.cpp", root / "csrc" / "pipeline_generator" / "pipeline_generator.cpp"]
    if not all(s.exists() for s in sources):
        return None
    import pybind11

    OUT_DIR.mkdir(exist_ok=True)
    cmd = ["g++", "-O2", "-std=c++17", "-shared", "-fPIC", f"-I{sysconfig.get_paths()['include']}",
           f"-I{pybind11.get_include()}", *map(str, sources), "-o", str(module_path())]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("reference stage packer failed to compile:\n" + proc.stderr)
    if verbose:
        print(f"built {module_path()}", file=sys.stderr)
    return module_path()


if __name__ == "__main__":
    build(*sys.argv[1:2])
