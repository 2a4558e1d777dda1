"""The backward that keeps dS in memory (dcp_attn_bwd_select(2), the default: the dK/dV kernel stores
the dS tiles it forms, a dQ kernel of one matrix product reads them back) against dense attention and
against the two-kernel backward that recomputes: both within the dense-attention bounds, and within
those bounds of each other (dQ adds the same rounded dS in another order; delta comes from different
kernels).  Results are bit-reproducible from run to run.  Past the executor's workspace limit the plan
falls back to recomputing."""

import numpy as np
import pytest
import torch

from tests.plan_cases import GRAD_TOL, check_against_truth, dense_truth, make_case, run_executor, scaled_err

pytestmark = pytest.mark.gpu

CASES = {
    "causal_gqa": dict(seqlens=[1536, 300], block_size=256, n_heads=8, n_groups=2, head_dim=128, head_block=4,
                       qkv_scale=0.5),
    "lambda_d64": dict(seqlens=[900, 130], block_size=128, n_heads=4, n_groups=1, head_dim=64, head_block=2,
                       mask="lambda", mask_kwargs=dict(n_starting=16, l_pretrain=300), qkv_scale=0.5),
    # 64-token blocks: a 128-key tile spans two slots, waves of a workgroup without keys of their own
    "ragged_split": dict(seqlens=[333, 1, 257, 64], block_size=64, n_heads=4, n_groups=2, head_dim=128, head_block=2,
                         n_kv_groups=2, qkv_scale=0.5),
    "shared_question_fp16": dict(seqlens=[700], block_size=128, n_heads=2, n_groups=1, head_dim=128, head_block=2,
                                 mask="shared_question", mask_kwargs=dict(question_proportion=0.3, n_answers=3),
                                 dtype="fp16", qkv_scale=0.5),
    # three q heads per kv head (the dQ kernel takes two heads per work item only where their number is even),
    # 320-token blocks (a 256-query work item and a ragged second one)
    "three_heads_per_kv_head": dict(seqlens=[700, 100], block_size=320, n_heads=6, n_groups=2, head_dim=128, head_block=3,
                                    qkv_scale=0.5),
    # 64-token blocks, key counts below and just above one 64-key piece
    "tiny_blocks": dict(seqlens=[70, 33, 5], block_size=64, n_heads=2, n_groups=1, head_dim=128, head_block=2,
                        qkv_scale=0.5),
}


def _bits(t):
    return t.view(torch.int16).numpy() if t.dtype != torch.float32 else t.view(torch.int32).numpy()


def _run(case, mode, lib, _lib):
    before = lib.dcp_attn_bwd_select(mode)
    try:
        _lib.profile_enable(True)
        result, _ = run_executor(case, backward=True)
        ran = _lib.profile_report()
    finally:
        _lib.profile_enable(False)
        lib.dcp_attn_bwd_select(before)
    return result, ran


@pytest.mark.parametrize("name", list(CASES))
def test_backward_through_ds_matches_dense_attention_and_the_recomputing_backward(gpu, name):
    from dcp_amd import _lib

    lib = _lib.load()
    case = make_case(**CASES[name])
    two, ran_two = _run(case, 0, lib, _lib)
    ds, ran_ds = _run(case, 2, lib, _lib)
    again, _ = _run(case, 2, lib, _lib)
    assert "attn_bwd_dq_kernel" in ran_two and "attn_bwd_dq_ds_kernel" not in ran_two, ran_two
    assert "attn_bwd_dq_ds_kernel" in ran_ds and "attn_bwd_dq_kernel" not in ran_ds, ran_ds
    check_against_truth(ds, dense_truth(case, backward=True))
    assert scaled_err(ds[3].float().numpy(), two[3].float().numpy()) <= GRAD_TOL
    assert np.abs(ds[2].float().numpy() - two[2].float().numpy()).max() <= GRAD_TOL
    assert np.array_equal(_bits(ds[2]), _bits(again[2])) and np.array_equal(_bits(ds[3]), _bits(again[3])), \
        "no atomics: the results do not depend on timing"


def test_executor_recomputes_when_ds_would_not_fit_the_workspace_limit(gpu, monkeypatch):
    from dcp_amd import _lib

    lib = _lib.load()
    case = make_case(**CASES["causal_gqa"])
    ds, ran = _run(case, 2, lib, _lib)
    assert "attn_bwd_dq_ds_kernel" in ran
    monkeypatch.setenv("DCP_BWD_DS_MAX_BYTES", "65536")
    small, ran_small = _run(case, 2, lib, _lib)
    assert "attn_bwd_dq_kernel" in ran_small and "attn_bwd_dq_ds_kernel" not in ran_small, ran_small
    assert scaled_err(ds[3].float().numpy(), small[3].float().numpy()) <= GRAD_TOL
    assert np.abs(ds[2].float().numpy() - small[2].float().numpy()).max() <= GRAD_TOL
