"""GPU parity of the blockwise attention path (gather -> range-masked paged
attention -> merge/scatter, and its backward) against the CPU oracle.

Tolerances (bf16 inputs, fp32 accumulation, oracle in fp64 on the same rounded
inputs): max-abs 2e-2 on out and dQ, max-abs 1e-3 on the fp32 LSE; dK/dV, which
reach magnitudes where one bf16 ulp exceeds 2e-2, elementwise 2e-2 * max(1, |ref|)
(tests/plan_cases.py)."""

import numpy as np
import pytest
import torch

from tests.plan_cases import (LSE_TOL, OUT_TOL, check_against_truth, dense_truth, make_case, run_executor,
                              run_plan_oracle)

pytestmark = pytest.mark.gpu


def _check_forward(case, res, out_tol=OUT_TOL):
    check_against_truth(res[:2], dense_truth(case), out_tol)


FWD_CASES = {
    # BASELINE config 1 shapes (blockwise causal, 8 heads, D=64, bs=256), run in bf16 on the GPU
    "c1_causal_d64": dict(seqlens=[512, 1024, 1536, 2048], block_size=256, n_heads=8, n_groups=8,
                          head_dim=64, head_block=1),
    "c1_every_block_its_own_partial": dict(seqlens=[512, 1024], block_size=256, n_heads=8, n_groups=8,
                                           head_dim=64, head_block=8, n_kv_groups=4),
    "gqa_ragged_d128": dict(seqlens=[1000, 333, 1, 257], block_size=256, n_heads=8, n_groups=2,
                            head_dim=128, head_block=4, qkv_scale=0.5),
    "gqa_hb1_split_fold": dict(seqlens=[700, 130], block_size=128, n_heads=4, n_groups=2, head_dim=128,
                               head_block=1, n_kv_groups=3, fold=True),
    "lambda_small_window": dict(seqlens=[1500, 640], block_size=128, n_heads=4, n_groups=1, head_dim=128,
                                head_block=4, mask="lambda",
                                mask_kwargs=dict(n_starting=16, l_pretrain=200)),
    "shared_prefix_hb5": dict(seqlens=[512 + 100 + 300 + 64], block_size=128, n_heads=10, n_groups=2,
                              head_dim=128, head_block=5, mask="shared_prefix",
                              mask_info=[dict(prefix=512, continuations=[100, 300, 64])],
                              n_kv_groups=2, kv_split="contiguous"),
    "causal_blockwise": dict(seqlens=[1100], block_size=128, n_heads=2, n_groups=2, head_dim=64,
                             head_block=2, mask="causal_blockwise",
                             mask_kwargs=dict(block_size=256, k_local=1)),
    "fp16": dict(seqlens=[400, 90], block_size=128, n_heads=4, n_groups=4, head_dim=128, head_block=2,
                 dtype="fp16"),
    # the masks of the reference's own end-to-end test (tests/runtime/test_flash_attention.py:40-45):
    # image tokens look forward inside their image (keys AFTER the query position)
    "multimodal": dict(seqlens=[100 + 200 + 150 + 200 + 90, 64 + 96 + 40], block_size=128, n_heads=4, n_groups=2,
                       head_dim=128, head_block=2, mask="modality_specific", qkv_scale=0.5,
                       mask_info=[dict(image_size=200, text_lengths=[100, 150, 90]),
                                  dict(image_size=96, text_lengths=[64, 40])]),
    "multimodal_image_to_self": dict(seqlens=[100 + 200 + 150 + 200 + 90], block_size=128, n_heads=4, n_groups=4,
                                     head_dim=64, head_block=4, mask="modality_specific", qkv_scale=0.5,
                                     mask_info=[dict(image_size=200, text_lengths=[100, 150, 90])],
                                     mask_kwargs=dict(limit_image_attn_to_self=True)),
    "shared_question": dict(seqlens=[1000, 517], block_size=128, n_heads=4, n_groups=2, head_dim=128, head_block=2,
                            mask="shared_question", qkv_scale=0.5,
                            mask_kwargs=dict(question_proportion=0.3, n_answers=3)),
    # the smallest block the kernels take (one query tile per row, one key tile per block) and rows of 1-2 tokens
    "tiny_blocks": dict(seqlens=[130, 1, 64, 2], block_size=64, n_heads=2, n_groups=1, head_dim=64, head_block=2,
                        qkv_scale=0.5),
    # scores spread over +-60 in the base-2 domain: later tiles keep exceeding the running reference
    # maximum by far more than the kernel's fast path tolerates, so its redo branch is exercised
    "large_scores": dict(seqlens=[2048, 700], block_size=256, n_heads=4, n_groups=2, head_dim=128, head_block=2,
                         qkv_scale=3.0),
    "large_scores_fp16": dict(seqlens=[1536], block_size=256, n_heads=2, n_groups=2, head_dim=64, head_block=2,
                              qkv_scale=3.0, dtype="fp16"),
}


# With inputs three times the usual size an output element reaches 13 in magnitude, where the
# output type's own spacing is 2^-4 (bf16, from 8 on): a result rounded correctly can be 3.1e-2
# away from the truth, so that case (bf16) allows one such step, 6.25e-2.  Every other case holds
# the plain 2e-2.
WIDE_OUT = {"large_scores": 6.25e-2}


@pytest.mark.parametrize("name", list(FWD_CASES))
def test_forward_matches_dense_truth(gpu, name):
    case = make_case(**FWD_CASES[name])
    res, _ = run_executor(case)
    _check_forward(case, res, WIDE_OUT.get(name, OUT_TOL))


def test_forward_matches_plan_oracle_buffers(gpu):
    """Same plan on the oracle's interpreter: the LOCAL outputs agree and the
    padded rows of every partial are (0, +inf) on both sides."""
    case = make_case([300, 520], 128, 4, 2, 64, 2, n_kv_groups=2)
    res, ex = run_executor(case)
    ref = run_plan_oracle(case)
    assert np.abs(res[0].float().numpy() - ref[0].float().numpy()).max() <= OUT_TOL
    assert np.abs(res[1].numpy() - ref[1].numpy()).max() <= LSE_TOL


# Same plan, same storage roundings: the oracle's interpreter keeps every buffer in the plan's own
# types (partial outputs, dQ versions and dK/dV replicas rounded to 16 bits where the plan stores
# them), so what is left between the two is the kernels' arithmetic (fp32 accumulation, P and dS
# rounded to 16 bits before the second products) and, wherever a value is stored, one step of the
# type at that value when the two sides land on different sides of a tie.  The interpreter adds
# those steps up per element along the plan (tests/plan_cases.py: SlackPlanOracle).  The bound is
# one and a half times that sum (a stored value may land one step away, and the arithmetic error
# that pushed it over the tie, below half a step of that value, travels on with it) plus, for the
# arithmetic itself, 5e-3 on out and dQ and 1e-2 * max(1, |ref|) on dK/dV (sums over every query of
# the row and every head of the group, where P and dS rounded to 16 bits add up): a quarter and a
# half of the bounds against dense attention.  The bound against dense attention (2e-2) has no room for
# the plan's own rounding in replica-heavy plans; this one does not need it.
TIGHT_CASES = {
    # one 65-token sequence, four one-head q head blocks per kv head, two partials per row: dK is the
    # sum of four bf16 replicas of magnitude 2-4 that cancel to ~0.1 (0.025 off dense attention)
    "replicas_cancel": dict(seqlens=[65], block_size=128, n_heads=16, n_groups=4, head_dim=128, head_block=1,
                            n_kv_groups=2, qkv_scale=0.5, seed=2027),
    "gqa_split3": dict(seqlens=[700, 130], block_size=128, n_heads=4, n_groups=2, head_dim=128, head_block=1,
                       n_kv_groups=3, qkv_scale=0.5),
    "folded_stages": dict(seqlens=[900, 260], block_size=128, n_heads=4, n_groups=2, head_dim=64, head_block=2,
                          n_kv_groups=4, fold=True, qkv_scale=0.5),
    "lambda_two_ranges": dict(seqlens=[600, 150], block_size=128, n_heads=4, n_groups=1, head_dim=128, head_block=4,
                              mask="lambda", mask_kwargs=dict(n_starting=16, l_pretrain=200), n_kv_groups=2,
                              qkv_scale=0.5),
}


@pytest.mark.parametrize("name", list(TIGHT_CASES))
def test_backward_matches_plan_oracle_with_the_same_roundings(gpu, name):
    case = make_case(**TIGHT_CASES[name])
    res, _ = run_executor(case, backward=True)
    ref, slack = run_plan_oracle(case, backward=True, with_slack=True)
    for what, got, want, room in zip(("out", "lse", "dq", "dkv"), res, ref, slack):
        got, want = got.float().numpy().astype(np.float64), want.float().numpy().astype(np.float64)
        if what == "lse":
            assert np.abs(got - want).max() <= LSE_TOL, what
            continue
        arithmetic = 1e-2 * np.maximum(1.0, np.abs(want)) if what == "dkv" else 5e-3
        excess = np.abs(got - want) - (1.5 * room.numpy().astype(np.float64) + arithmetic)
        assert excess.max() <= 0.0, (what, float(excess.max()), float(np.abs(got - want).max()))


# Head sizes the kernels are not built for run zero-padded at the next one that is (64, 128), as
# the reference pads head sizes to what its kernels take: multiples of 8 and one that is not.
FWD_CASES.update({
    "head_dim_96": dict(seqlens=[300, 77], block_size=128, n_heads=4, n_groups=2, head_dim=96, head_block=2,
                        n_kv_groups=2),
    "head_dim_40": dict(seqlens=[200], block_size=64, n_heads=2, n_groups=2, head_dim=40, head_block=2,
                        mask="lambda", mask_kwargs=dict(n_starting=8, l_pretrain=50)),
    "head_dim_100_fp16": dict(seqlens=[150, 40], block_size=64, n_heads=2, n_groups=1, head_dim=100, head_block=2,
                              dtype="fp16"),
})

BWD_CASES = {
    "causal_d64": dict(seqlens=[512, 300], block_size=256, n_heads=4, n_groups=4, head_dim=64, head_block=2),
    "gqa_ragged_d128": dict(seqlens=[1000, 333, 1, 257], block_size=256, n_heads=8, n_groups=2,
                            head_dim=128, head_block=4, qkv_scale=0.5),
    "gqa_hb1_split": dict(seqlens=[700, 130], block_size=128, n_heads=4, n_groups=2, head_dim=128,
                          head_block=1, n_kv_groups=3, qkv_scale=0.5),
    "lambda_small_window": dict(seqlens=[1500, 640], block_size=128, n_heads=4, n_groups=1, head_dim=128,
                                head_block=4, mask="lambda", qkv_scale=0.5,
                                mask_kwargs=dict(n_starting=16, l_pretrain=200)),
    "shared_prefix_hb5": dict(seqlens=[512 + 100 + 300 + 64], block_size=128, n_heads=10, n_groups=2,
                              head_dim=128, head_block=5, mask="shared_prefix", qkv_scale=0.5,
                              mask_info=[dict(prefix=512, continuations=[100, 300, 64])],
                              n_kv_groups=2, kv_split="contiguous"),
    "fp16": dict(seqlens=[400, 90], block_size=128, n_heads=4, n_groups=4, head_dim=128, head_block=2,
                 dtype="fp16", qkv_scale=0.5),
    "multimodal": FWD_CASES["multimodal"],
    "multimodal_image_to_self": FWD_CASES["multimodal_image_to_self"],
    "shared_question": FWD_CASES["shared_question"],
    "tiny_blocks": FWD_CASES["tiny_blocks"],
    "head_dim_96": dict(FWD_CASES["head_dim_96"], qkv_scale=0.5),
    "head_dim_40": dict(FWD_CASES["head_dim_40"], qkv_scale=0.5),
    "head_dim_100_fp16": dict(FWD_CASES["head_dim_100_fp16"], qkv_scale=0.5),
}


@pytest.mark.parametrize("name", list(BWD_CASES))
def test_backward_matches_dense_truth(gpu, name):
    case = make_case(**BWD_CASES[name])
    res, _ = run_executor(case, backward=True)
    check_against_truth(res, dense_truth(case, backward=True))


def test_other_head_sizes_allocate_nothing_per_call(gpu):
    """The executor stores a head size the kernels do not have at the next one they have, in every
    buffer it owns: nothing is padded or copied per call, so such a plan runs in captured graphs like
    any other, with the results of the eager run bit for bit, and no call allocates device memory."""
    case = make_case(**BWD_CASES["head_dim_96"])
    eager, ex = run_executor(case, backward=True)
    check_against_truth(eager, dense_truth(case, backward=True))
    graphed, _ = run_executor(case, backward=True, use_graph=True)
    for a, b in zip(eager, graphed):
        assert torch.equal(a.view(torch.int16) if a.dtype != torch.float32 else a.view(torch.int32),
                           b.view(torch.int16) if b.dtype != torch.float32 else b.view(torch.int32))
    # the prepared backward executes without allocating (the clones its API returns aside)
    layout = case["layout"]
    ex.execute(case["bw"], False)
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    ex.execute(case["bw"], False)
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before


def test_forward_workspace_is_reusable_and_may_hold_anything(gpu):
    """The forward kernel hands out work items through counters in a caller workspace that each
    launch resets itself: a workspace full of garbage, reused by every attention launch of a
    multi-partial plan and over repeated runs, changes nothing."""
    case = make_case(**FWD_CASES["c1_every_block_its_own_partial"])
    res, ex = run_executor(case)
    _check_forward(case, res)
    spaces = [a[-1] for a in ex._args_cache.values() if isinstance(a, tuple) and isinstance(a[-1], torch.Tensor)
              and a[-1].dtype == torch.int32 and a[-1].numel() <= 64]
    assert spaces, "the prepared attention instructions carry their workspaces"
    layout = case["layout"]
    lq = layout.to_local_q(case["q"]).cuda()
    lkv = layout.to_local_kv(case["kv"]).cuda()
    for fill in (0x7fffffff, -5):
        for w in spaces:
            w.fill_(fill)
        out, lse = ex.forward(lq, lkv)
        torch.cuda.synchronize()
        again = [layout.from_local_q(out.cpu()), layout.from_local_lse(lse.cpu())]
        assert torch.equal(again[0], res[0]) and torch.equal(again[1], res[1])
    # a missing workspace is an argument error, reported before anything is launched
    from dcp_amd import _lib

    with pytest.raises(AssertionError, match="workspace"):
        _lib.call("dcp_attn_fwd", *([16] * 8), 1, 16, 16, 16, 0, 1, 1, 64, 64, 1, 1, 128, 8, 8, 1, 1.0, 0, 0, 0, 0)
