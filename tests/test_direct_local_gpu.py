"""Plans run with the copies the executor can leave out (the kernels address the unpadded LOCAL_*
tensors by token offset: ``dcp_amd/runtime/flash_attention/direct.py``) against the same plans run
as written, every MemcpyInstr, scatter and sum executed: the same bits in out, lse, dQ and dKV."""

import numpy as np
import pytest
import torch

from tests.plan_cases import check_against_truth, dense_truth, make_case, run_executor

pytestmark = pytest.mark.gpu

CASES = {
    "ragged_gqa_d128": dict(seqlens=[1000, 333, 1, 257], block_size=256, n_heads=8, n_groups=2, head_dim=128,
                            head_block=4, qkv_scale=0.5),
    "one_head_blocks_d64": dict(seqlens=[300, 520, 77], block_size=128, n_heads=4, n_groups=2, head_dim=64, head_block=1),
    "lambda_two_ranges": dict(seqlens=[900, 130], block_size=128, n_heads=4, n_groups=1, head_dim=128, head_block=2,
                              mask="lambda", mask_kwargs=dict(n_starting=16, l_pretrain=300), qkv_scale=0.5),
    # several partials per row: inputs are read in place, partial outputs still go through slots and merges
    "split3": dict(seqlens=[700, 130], block_size=128, n_heads=4, n_groups=2, head_dim=128, head_block=1, n_kv_groups=3,
                   qkv_scale=0.5),
    "folded_stages": dict(seqlens=[900, 260], block_size=128, n_heads=4, n_groups=2, head_dim=64, head_block=2,
                          n_kv_groups=4, fold=True, qkv_scale=0.5),
    # queries that see no key at all (their merged LSE reads -1): empty first ranges of the shared-question mask
    "shared_question_fp16": dict(seqlens=[700, 65], block_size=64, n_heads=2, n_groups=1, head_dim=128, head_block=2,
                                 mask="shared_question", mask_kwargs=dict(question_proportion=0.3, n_answers=3),
                                 dtype="fp16", qkv_scale=0.5),
}


def _bits(t):
    return t.view(torch.int16).numpy() if t.dtype != torch.float32 else t.view(torch.int32).numpy()


def _kernels_of(case, monkeypatch, direct: bool, backward=True):
    from dcp_amd import _lib

    monkeypatch.setenv("DCP_DIRECT_LOCAL", "1" if direct else "0")
    _lib.profile_enable(True)
    try:
        res, ex = run_executor(case, backward=backward)
        ran = _lib.profile_report()
    finally:
        _lib.profile_enable(False)
    assert ex.direct_local == direct
    return res, ran


@pytest.mark.parametrize("name", list(CASES))
def test_results_are_bit_identical_with_and_without_the_copies(gpu, monkeypatch, name):
    case = make_case(**CASES[name])
    as_written, ran_all = _kernels_of(case, monkeypatch, direct=False)
    direct, ran_direct = _kernels_of(case, monkeypatch, direct=True)
    for what, a, b in zip(("out", "lse", "dq", "dkv"), as_written, direct):
        assert np.array_equal(_bits(a), _bits(b)), what
    check_against_truth(direct, dense_truth(case, backward=True))
    # and copies were in fact left out: fewer (or no) gather launches
    copies = lambda ran: sum(n for k, (n, _) in ran.items() if k.startswith("copy_"))
    assert copies(ran_direct) < copies(ran_all), (ran_direct, ran_all)


def test_single_stage_plan_runs_without_gather_and_scatter(gpu, monkeypatch):
    """One stage, one partial per row: nothing is left of the plan's block movement but the sums
    of dK/dV replicas (which go straight into LOCAL_dKV) and the copies of single-replica blocks."""
    case = make_case(**CASES["ragged_gqa_d128"])
    _, ran = _kernels_of(case, monkeypatch, direct=True)
    assert not any(k.startswith(("copy_", "merge_")) for k in ran), ran
    assert "attn_fwd_kernel" in ran and "blockwise_sum_kernel" in ran


def test_graph_replays_of_a_direct_plan(gpu, monkeypatch):
    monkeypatch.setenv("DCP_DIRECT_LOCAL", "1")
    case = make_case(**CASES["ragged_gqa_d128"])
    eager, _ = run_executor(case, backward=True)
    graphed, _ = run_executor(case, backward=True, use_graph=True)
    for a, b in zip(eager, graphed):
        assert np.array_equal(_bits(a), _bits(b))
