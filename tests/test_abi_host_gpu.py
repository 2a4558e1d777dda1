"""The C ABI from a host that is neither Python nor torch: tests/abi_host/abi_host_check.cpp
(plain C++ + HIP runtime + include/dcp_hip.h) gathers blocks, runs the attention forward and a
block sum through libdcp_hip.so and checks them against CPU loops.  The binary is built by
``dcp_amd.build.build_abi_host_check`` (part of ``__graft_entry__.build``)."""

import subprocess

import pytest

pytestmark = pytest.mark.gpu


def test_plain_cpp_host_drives_the_library(gpu):
    from dcp_amd import build

    if not build.HOST_CHECK_BIN.exists():  # normally built with the library; a few seconds if not
        try:
            build.build_abi_host_check(verbose=False)
        except Exception as e:  # no compiler on this machine
            pytest.skip(f"tests/abi_host/abi_host_check is not built and cannot be built here: {e}")
    proc = subprocess.run([str(build.HOST_CHECK_BIN)], capture_output=True, text=True, timeout=100)
    print(proc.stdout, proc.stderr, flush=True)
    assert proc.returncode == 0, proc.stderr
    assert "ok" in proc.stdout
