"""Work units and their block-local masks (the dataloader side of the plan builder) against
what fixes them: a dense boolean expansion of the sequence mask, block by block; the reference's
rules for which pairs are work units; and the plan builder's own one-step route from the
sequence mask to row ranges (dcp/data/dataloader.py:1384-1546, dcp/core/scheduler.py:1143-1185)."""

import numpy as np
import pytest
import torch

from tests.plan_cases import check_against_truth, dense_truth, make_case, run_executor, run_plan_oracle

from dcp_amd.core.instructions import AttnInstr
from dcp_amd.runtime.flash_attention.single_device import _block_overlaps, _row_ranges
from dcp_amd.runtime.flash_attention.utils import (
    causal_blockwise_mask_fn,
    causal_range_mask_fn,
    lambda_mask_fn,
    modality_specific_mask_fn,
    shared_prefix_mask_fn,
    shared_question_mask_fn,
)
from dcp_amd.runtime.flash_attention.workload import (
    concat_local_attn_masks,
    generate_work_units,
    local_attn_mask,
    rows_of_work_units,
)


def _dense(seq_mask, L):
    a = np.zeros((L, L), dtype=bool)
    for i in range(L):
        for s, e in np.asarray(seq_mask[i]).reshape(-1, 2):
            a[i, s:min(e, L)] = True
    return a


def _dense_local(m, n_q, n_k):
    """Boolean [n_q, n_k] of a work unit's local mask."""
    planes = m[None] if m.ndim == 2 else m
    a = np.zeros((n_q, n_k), dtype=bool)
    for r in range(planes.shape[0]):
        for q in range(n_q):
            a[q, planes[r, 0, q]:planes[r, 1, q]] = True
    return a


CASES = {
    "causal": lambda L: causal_range_mask_fn([L], [L], torch.int32),
    "lambda": lambda L: lambda_mask_fn([L], [L], torch.int32, n_starting=5, l_pretrain=37),
    "shared_question": lambda L: shared_question_mask_fn([L], [L], torch.int32, question_proportion=0.3, n_answers=3),
    "causal_blockwise": lambda L: causal_blockwise_mask_fn([L], [L], torch.int32, block_size=48, k_local=1),
    "shared_prefix": lambda L: shared_prefix_mask_fn(
        [L], [L], torch.int32, [dict(prefix=L // 3, continuations=[L // 4, L - L // 3 - L // 4])]),
    "multimodal": lambda L: modality_specific_mask_fn(
        [L], [L], torch.int32, [dict(image_size=L // 5, text_lengths=[L // 4, L - L // 4 - 2 * (L // 5)])]),
}


@pytest.mark.parametrize("name", list(CASES))
@pytest.mark.parametrize("L,bs", [(200, 32), (97, 16), (64, 64), (130, 128)])
def test_local_masks_are_the_dense_mask_block_by_block(name, L, bs):
    seq_mask = CASES[name](L).numpy()
    dense = _dense(seq_mask, L)
    units = generate_work_units(seq_mask, L, bs)
    n_blocks = (L + bs - 1) // bs
    for i in range(n_blocks):
        n_q = min(bs, L - i * bs)
        for j in range(n_blocks):
            n_k = min(bs, L - j * bs)
            want = dense[i * bs:i * bs + n_q, j * bs:j * bs + n_k]
            m = units.get((i, j))
            if m is None:
                assert not want.any(), (i, j)  # a skipped pair holds no attended (query, key)
                continue
            assert m.dtype == np.int32 and m.shape[-1] == bs
            assert (m[..., n_q:] == -1).all()  # entries past the block's tokens stay -1
            assert (m[..., :n_q] >= 0).all() and (m[..., 1, :n_q] <= n_k).all()
            assert np.array_equal(_dense_local(m, n_q, n_k), want), (i, j)
    # every pair with an attended (query, key) is a work unit, and in block order per row
    for i, js in rows_of_work_units(units).items():
        assert js == sorted(js)
        assert set(js) >= set(_block_overlaps(seq_mask, i * bs, min(bs, L - i * bs), bs, n_blocks, L))


@pytest.mark.parametrize("name", list(CASES))
def test_concatenated_local_masks_equal_the_builders_row_ranges(name):
    L, bs = 230, 32
    seq_mask = CASES[name](L).numpy()
    units = generate_work_units(seq_mask, L, bs)
    n_blocks = (L + bs - 1) // bs
    for i, js in rows_of_work_units(units).items():
        n_q = min(bs, L - i * bs)
        n_keys = [min(bs, L - j * bs) for j in js]
        got = concat_local_attn_masks([units[(i, j)] for j in js], n_keys, n_q)
        # the builder's route, over the same kv blocks
        want = _row_ranges(seq_mask, i * bs, n_q, bs, js, n_keys)[..., :n_q]
        # (the reference shifts a piece by the real key counts of the blocks before it, the builder by
        # whole slots: the same, since only a sequence's last block is partial and it comes last)
        assert np.array_equal(got, want), (i, js)
        # over the builder's own choice of kv blocks (exact overlap, never more than the units'):
        # the same attended keys
        exact = _block_overlaps(seq_mask, i * bs, n_q, bs, n_blocks, L)
        assert set(exact) <= set(js)
        joined = concat_local_attn_masks([units[(i, j)] for j in exact], [min(bs, L - j * bs) for j in exact], n_q)
        assert _dense_local(joined, n_q, bs * len(exact)).sum() == _dense(seq_mask, L)[i * bs:i * bs + n_q].sum()


def test_work_unit_rule_is_the_hull_of_the_blocks_ranges():
    """Ranges of different queries on either side of a kv block: no query attends it, but the
    smallest start and the largest end straddle it, so the reference makes it a work unit with
    empty ranges only; with every range on one side it is skipped."""
    bs, L = 4, 16
    seq_mask = np.zeros((L, 2), dtype=np.int32)
    seq_mask[0:2] = [0, 4]     # queries 0-1 look at block 0
    seq_mask[2:4] = [8, 12]    # queries 2-3 look at block 2
    m = local_attn_mask(seq_mask, 0, 1, bs, L)
    assert m is not None and ((m[1] - m[0])[:4] <= 0).all()  # kept, and empty for every query
    assert local_attn_mask(seq_mask, 0, 3, bs, L) is None  # wholly to the right of every range
    assert _block_overlaps(seq_mask, 0, 4, bs, 4, L) == [0, 2]  # the builder keeps only real overlap
    # joining the three units of the row: queries 0-1 get block 0, queries 2-3 block 2 (shifted by 8)
    units = [local_attn_mask(seq_mask, 0, j, bs, L) for j in (0, 1, 2)]
    got = concat_local_attn_masks(units, [4, 4, 4], 4)
    assert got.tolist() == [[[0, 0, 8, 8], [4, 4, 12, 12]]]
    # two-range masks: a block no valid range's hull touches is skipped, planes are clamped into the block
    two = np.zeros((L, 2, 2), dtype=np.int32)
    two[:, 0] = [0, 2]
    two[:, 1] = [9, 14]
    assert local_attn_mask(two, 1, 1, bs, L) is None
    m = local_attn_mask(two, 1, 2, bs, L)
    assert m[0, :, :4].tolist() == [[0] * 4, [0] * 4] and m[1, :, :4].tolist() == [[1] * 4, [4] * 4]
    m = local_attn_mask(two, 1, 3, bs, L)
    assert m[1, :, :4].tolist() == [[0] * 4, [2] * 4]
    # causal generation looks at j <= i only
    c = causal_range_mask_fn([L], [L], torch.int32).numpy()
    assert set(generate_work_units(c, L, bs, causal=True)) == {(i, j) for i in range(4) for j in range(i + 1)}


def test_discontinuous_pieces_are_refused():
    a = np.full((2, 4), -1, dtype=np.int32)
    a[:, :2] = [[0, 0], [2, 2]]
    b = np.full((2, 4), -1, dtype=np.int32)
    b[:, :2] = [[1, 1], [3, 3]]  # starts one key into the second block: a hole after the first piece
    with pytest.raises(AssertionError, match="Discontinuous"):
        concat_local_attn_masks([a, b], [4, 4], 2)


PLAN_CASES = {
    "lambda": dict(seqlens=[700, 130], block_size=64, n_heads=4, n_groups=2, head_dim=64, head_block=2, mask="lambda",
                   mask_kwargs=dict(n_starting=16, l_pretrain=100), qkv_scale=0.5),
    "shared_prefix_two_stages": dict(seqlens=[512 + 100 + 300 + 64], block_size=128, n_heads=4, n_groups=2,
                                     head_dim=128, head_block=2, mask="shared_prefix", qkv_scale=0.5,
                                     mask_info=[dict(prefix=512, continuations=[100, 300, 64])], n_kv_groups=2,
                                     kv_split="contiguous"),
    "multimodal": dict(seqlens=[100 + 200 + 150 + 200 + 90], block_size=128, n_heads=4, n_groups=2, head_dim=128,
                       head_block=2, mask="modality_specific", qkv_scale=0.5,
                       mask_info=[dict(image_size=200, text_lengths=[100, 150, 90])]),
}


def _rows(plan):
    return [(len(t), [b.index for b in t]) for i in plan.instructions if isinstance(i, AttnInstr) for t in i.kv_block_table]


@pytest.mark.parametrize("name", list(PLAN_CASES))
def test_plans_through_block_local_masks_on_the_oracle(name):
    """The builder fed through the reference's work units: its plans reproduce whole-sequence
    attention on the oracle's interpreter, with rows at least as long as the exact-overlap ones."""
    case = make_case(**PLAN_CASES[name], work_units="reference")
    base = make_case(**PLAN_CASES[name])
    out, lse = run_plan_oracle(case)[:2]
    want = dense_truth(case)
    assert np.abs(out.float().numpy() - want[0]).max() <= 2e-2
    assert np.abs(lse.numpy() - want[1]).max() <= 1e-3
    n_ref = sum(n for n, _ in _rows(case["fw"]))
    n_base = sum(n for n, _ in _rows(base["fw"]))
    assert n_ref >= n_base


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(PLAN_CASES))
def test_plans_through_block_local_masks_on_the_gpu(gpu, name):
    case = make_case(**PLAN_CASES[name], work_units="reference")
    res, _ = run_executor(case, backward=True)
    check_against_truth(res, dense_truth(case, backward=True))
