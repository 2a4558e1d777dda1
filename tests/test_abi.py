"""The C-ABI library: it loads, exports every symbol include/dcp_hip.h declares,
and rejects bad arguments before launching anything (no GPU needed: only the
argument checks run here)."""

import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]


@pytest.fixture(scope="module")
def lib():
    from dcp_amd import _lib

    if not _lib.LIB_PATH.exists():
        from dcp_amd import build

        build.build(verbose=False)
    return _lib.load()


def _declared_symbols():
    text = (ROOT / "include" / "dcp_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dcp_[a-z_0-9]+)\s*\(", text)))


def test_header_and_library_agree(lib):
    from dcp_amd import _lib

    declared = _declared_symbols()
    assert len(declared) >= 12
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in dcp_hip.h but not exported"
    assert sorted(_lib.SIGNATURES) == declared, "ctypes signatures and header differ"


def test_version_and_error_string(lib):
    assert lib.dcp_version() >= 100
    assert isinstance(lib.dcp_last_error(), bytes)


def test_argument_errors_are_reported_without_a_launch(lib):
    from dcp_amd import _lib

    with pytest.raises(AssertionError, match="unsupported element size"):
        _lib.call("dcp_fused_copy_varlen", 0, 0, 0, 0, 0, 0, 0, 1, 16, 3, 0)
    with pytest.raises(AssertionError, match="Too many blocks"):
        _lib.call("dcp_update_out_lse", 0, 0, 0, 0, 1, 0, 0, 0, 0, 1, 64, 1, 1, 1, 1, 1, 1, 64, 128, 0, 0)
    with pytest.raises(ValueError, match="Unsupported dtype"):
        _lib.call("dcp_blockwise_sum", 0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 128, 7, 0)
    with pytest.raises(ValueError, match="head_dim"):
        _lib.call("dcp_attn_fwd", *([0] * 8), 1, 0, 0, 0, 0, 1, 1, 64, 64, 1, 1, 96, 0, 0, 1, 1.0, 0, 0, 0, 0)
    with pytest.raises(ValueError, match="bf16 and fp16"):
        _lib.call("dcp_attn_fwd", *([0] * 8), 1, 0, 0, 0, 0, 1, 1, 64, 64, 1, 1, 128, 0, 0, 1, 1.0, 2, 0, 0, 0)
    # empty problems are accepted and launch nothing
    _lib.call("dcp_fused_copy_varlen", 0, 0, 0, 0, 0, 0, 0, 0, 16, 2, 0)
    _lib.call("dcp_attn_fwd", *([0] * 8), 1, 0, 0, 0, 0, 0, 1, 0, 64, 1, 1, 128, 0, 0, 1, 1.0, 0, 0, 0, 0)
    assert lib.dcp_attn_fwd_workspace_bytes() >= 9 * 4
    assert lib.dcp_attn_bwd_workspace_bytes(2, 128, 64, 4, 128) >= 128 * 4 * 4 + 2 * 8 * 4


def test_backward_selection_and_its_workspace_size(lib):
    """dcp_attn_bwd_select returns the previous setting and only sets a known mode; the workspace the
    selected backward needs: the recomputing one the small scratch whatever the key count, the one
    that keeps dS in memory 4 KiB per (64-key tile, head, 32-query chunk) on top of it, with one tile
    more per row than total_kv / 64 and two spare pieces."""
    before = lib.dcp_attn_bwd_select(0)
    try:
        assert lib.dcp_attn_bwd_select(-1) == 0 and lib.dcp_attn_bwd_select(77) == 0 and lib.dcp_attn_bwd_select(-1) == 0
        batch, total_q, total_kv, bs, heads, d = 6, 6 * 256, 6 * 1024 + 5 * 256, 256, 4, 128
        base = lib.dcp_attn_bwd_workspace_bytes(batch, total_q, bs, heads, d)
        assert lib.dcp_attn_bwd_workspace_bytes_kv(batch, total_q, total_kv, bs, heads, d) == base
        assert lib.dcp_attn_bwd_select(2) == 0
        pieces = (total_kv // 64 + batch + 1) * heads * (bs // 32) + 2
        assert lib.dcp_attn_bwd_workspace_bytes_kv(batch, total_q, total_kv, bs, heads, d) == base + pieces * 4096
        assert lib.dcp_attn_bwd_workspace_bytes_kv(batch, total_q, 0, bs, heads, d) == base, "no key count: nothing to keep"
        assert lib.dcp_attn_bwd_workspace_bytes(batch, total_q, bs, heads, d) == base
    finally:
        lib.dcp_attn_bwd_select(before)


def test_profile_report_is_empty_when_disabled(lib):
    from dcp_amd import _lib

    assert _lib.profile_report() == {}
