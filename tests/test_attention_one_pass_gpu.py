"""The one-pass backward (dcp_attn_bwd_select(1): dQ formed in the key-outer kernel, the key tiles of
a row adding their shares through a chain of fp32 partial sums) against dense attention and against
the default two-kernel backward: the same bounds against dense attention, the two backwards within
those bounds of each other (they add the same products in different orders), and the one-pass
results bit-reproducible from run to run."""

import numpy as np
import pytest
import torch

from tests.plan_cases import GRAD_TOL, check_against_truth, dense_truth, make_case, run_executor, scaled_err

pytestmark = pytest.mark.gpu

CASES = {
    # long chains: 12 key tiles per row at the end of the first sequence, causal diagonal tiles
    "causal_gqa": dict(seqlens=[1536, 300], block_size=256, n_heads=8, n_groups=2, head_dim=128, head_block=4,
                       qkv_scale=0.5),
    # two ranges per query (sink + window): tiles that see a query tile form two runs
    "lambda": dict(seqlens=[900, 130], block_size=128, n_heads=4, n_groups=1, head_dim=128, head_block=2,
                   mask="lambda", mask_kwargs=dict(n_starting=16, l_pretrain=300), qkv_scale=0.5),
    # ragged rows, one-token sequence, several partials per row, 64-token blocks (a key tile spans two slots)
    "ragged_split": dict(seqlens=[333, 1, 257, 64], block_size=64, n_heads=4, n_groups=2, head_dim=128, head_block=2,
                         n_kv_groups=2, qkv_scale=0.5),
    "shared_question_fp16": dict(seqlens=[700], block_size=128, n_heads=2, n_groups=1, head_dim=128, head_block=2,
                                 mask="shared_question", mask_kwargs=dict(question_proportion=0.3, n_answers=3),
                                 dtype="fp16", qkv_scale=0.5),
}


@pytest.fixture
def one_pass():
    from dcp_amd import _lib

    lib = _lib.load()
    before = lib.dcp_attn_bwd_select(1)
    yield lib
    lib.dcp_attn_bwd_select(before)


def _bits(t):
    return t.view(torch.int16).numpy() if t.dtype != torch.float32 else t.view(torch.int32).numpy()


@pytest.mark.parametrize("name", list(CASES))
def test_one_pass_backward_matches_dense_attention_and_the_two_kernel_backward(gpu, name):
    from dcp_amd import _lib

    lib = _lib.load()
    case = make_case(**CASES[name])
    before = lib.dcp_attn_bwd_select(0)
    try:
        two, _ = run_executor(case, backward=True)
        assert lib.dcp_attn_bwd_select(1) == 0
        # (the workspace size tells whether the one-pass kernels will run: it holds their partial sums)
        assert lib.dcp_attn_bwd_workspace_bytes(2, 256, 128, 2, 128) >= 2 * 128 * 2 * 128 * 4, \
            "the one-pass backward is not available on this device"
        _lib.profile_enable(True)
        one, _ = run_executor(case, backward=True)
        ran = _lib.profile_report()
        _lib.profile_enable(False)
        assert "attn_bwd_fused_kernel" in ran and "attn_bwd_dq_kernel" not in ran, ran
        again, _ = run_executor(case, backward=True)
    finally:
        _lib.profile_enable(False)
        lib.dcp_attn_bwd_select(before)
    check_against_truth(one, dense_truth(case, backward=True))
    assert scaled_err(one[3].float().numpy(), two[3].float().numpy()) <= GRAD_TOL
    assert np.abs(one[2].float().numpy() - two[2].float().numpy()).max() <= GRAD_TOL
    assert np.array_equal(_bits(one[2]), _bits(again[2])) and np.array_equal(_bits(one[3]), _bits(again[3])), \
        "the chain adds in key order: dQ does not depend on timing"


def test_one_pass_is_only_taken_when_selected(gpu, one_pass):
    """The workspace size says which backward a plan prepared now will run."""
    lib = one_pass
    with_chain = lib.dcp_attn_bwd_workspace_bytes(4, 1024, 256, 4, 128)
    lib.dcp_attn_bwd_select(0)
    without = lib.dcp_attn_bwd_workspace_bytes(4, 1024, 256, 4, 128)
    lib.dcp_attn_bwd_select(1)
    assert with_chain >= without + 4 * 256 * 4 * 128 * 4
    assert lib.dcp_attn_bwd_workspace_bytes(4, 1024, 256, 4, 64) == without  # head size 64: two kernels either way
