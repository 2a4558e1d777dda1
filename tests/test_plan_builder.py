"""Host logic without a GPU: mask generators against brute force and closed
forms, the single-device plan builder (layout round trips, block tables,
concatenated ranges) and the whole plan run on the oracle's interpreter
against whole-sequence attention."""

import numpy as np
import pytest
import torch

from dcp_amd.core.instructions import AttnBackwardInstr, AttnInstr, AttnReductionInstr, BufferType, SumInstr
from dcp_amd.runtime.flash_attention.single_device import build_single_device_plans
from dcp_amd.runtime.flash_attention.utils import (
    MASK_FNS,
    causal_blockwise_mask_fn,
    causal_range_mask_fn,
    count_attended_pairs,
    lambda_mask_fn,
    modality_specific_mask_fn,
    shared_prefix_mask_fn,
    shared_question_mask_fn,
)
from oracle import dcp_oracle as oracle
from tests.plan_cases import dense_truth, make_case, run_plan_oracle


def _allowed(mask, seqlens, padded):
    """Boolean [L, L] per sequence from a range mask (brute force expansion)."""
    out, off = [], 0
    m = mask.numpy()
    for L, P in zip(seqlens, padded):
        a = np.zeros((L, L), dtype=bool)
        for i in range(L):
            row = m[off + i].reshape(-1, 2)
            for s, e in row:
                a[i, s:e] = True
        out.append(a)
        off += P
    return out


def test_causal_and_lambda_masks_against_definition():
    seq, pad = [5, 9], [8, 12]
    c = causal_range_mask_fn(seq, pad, torch.int32)
    assert c.shape == (20, 2) and c.dtype == torch.int32
    for a in _allowed(c, seq, pad):
        assert np.array_equal(a, np.tril(np.ones_like(a)))
    assert torch.all(c[5:8] == 0) and torch.all(c[17:] == 0)  # padding rows stay [0, 0)
    lam = lambda_mask_fn([40], [40], torch.int32, n_starting=4, l_pretrain=10)
    a = _allowed(lam, [40], [40])[0]
    for i in range(40):
        for j in range(40):
            assert a[i, j] == (j <= i and (j < 4 or j > i - 10))
    # pair counts: closed forms of the metric's FLOP accounting
    assert count_attended_pairs(c) == sum(L * (L + 1) // 2 for L in seq)
    assert count_attended_pairs(lam) == sum(min(i + 1, 14) for i in range(40)) == int(a.sum())


def test_shared_question_and_prefix_masks():
    sq = shared_question_mask_fn([50], [50], torch.int32, question_proportion=0.2, n_answers=4)
    a = _allowed(sq, [50], [50])[0]
    n_q, per = 10, 10
    for i in range(50):
        for j in range(50):
            if i < n_q:
                want = j <= i
            else:
                start = n_q + min((i - n_q) // per, 3) * per
                want = j < n_q or start <= j <= i
            assert a[i, j] == want, (i, j)
    sp = shared_prefix_mask_fn([30], [30], torch.int32, [dict(prefix=12, continuations=[5, 13])])
    b = _allowed(sp, [30], [30])[0]
    for i in range(30):
        for j in range(30):
            if i < 12:
                want = j <= i
            elif i < 17:
                want = j < 12 or 12 <= j <= i
            else:
                want = j < 12 or 17 <= j <= i
            assert b[i, j] == want, (i, j)
    p, cs = 12, [5, 13]
    assert count_attended_pairs(sp) == p * (p + 1) // 2 + sum(c * p + c * (c + 1) // 2 for c in cs)
    # equal answers: the shared-prefix generator reproduces the shared-question one
    same = shared_prefix_mask_fn([50], [50], torch.int32, [dict(prefix=10, continuations=[10, 10, 10, 10])])
    assert np.array_equal(_allowed(same, [50], [50])[0], a)


def test_causal_blockwise_and_modality_masks():
    cb = causal_blockwise_mask_fn([40], [40], torch.int32, block_size=8, k_local=1)
    a = _allowed(cb, [40], [40])[0]
    for i in range(40):
        blk, n_blocks = i // 8, 5
        for j in range(40):
            if blk == 0:
                want = j <= i
            elif blk == n_blocks - 1:
                want = j <= i  # everything before the previous block end, then from there causally
            else:
                want = j < 8 or max(8, i - 8) <= j <= i
            assert a[i, j] == want, (i, j)
    mm = modality_specific_mask_fn([20], [20], torch.int32, [dict(image_size=6, text_lengths=[5, 9])])
    b = _allowed(mm, [20], [20])[0]
    for i in range(20):
        for j in range(20):
            want = (j < 11) if 5 <= i < 11 else (j <= i)
            assert b[i, j] == want, (i, j)
    assert set(MASK_FNS) >= {"causal", "lambda", "shared_question", "causal_blockwise", "shared_prefix"}


def test_layout_roundtrips_and_local_order():
    seqs = [300, 520, 17]
    mask = causal_range_mask_fn(seqs, seqs, torch.int32)
    fw, bw, lay = build_single_device_plans(seqs, 128, 8, 2, 16, 2, mask)
    T = sum(seqs)
    g = torch.Generator().manual_seed(0)
    q = torch.randn(T, 8, 16, generator=g)
    kv = torch.randn(T, 2, 2, 16, generator=g)
    lse = torch.randn(8, T, generator=g)
    assert torch.equal(lay.from_local_q(lay.to_local_q(q)), q)
    assert torch.equal(lay.from_local_kv(lay.to_local_kv(kv)), kv)
    assert torch.equal(lay.from_local_lse(lay.to_local_lse(lse)), lse)
    # LOCAL order is (head block, sequence, block); cu_seqlens are its prefix sums
    assert [b[:3] for b in lay.q_blocks[:4]] == [(0, 0, 0), (0, 0, 1), (0, 0, 2), (0, 1, 0)]
    assert lay.local_cu_seqlens[-1] == 4 * T and fw.local_cu_seqlens == lay.local_cu_seqlens
    assert fw.buffer_info[BufferType.LOCAL_Q].buffer_shape == (4 * T, 2, 16)
    assert fw.buffer_info[BufferType.LOCAL_KV].buffer_shape == (2 * T, 2, 1, 16)  # GQA: one kv head per block
    assert fw.buffer_info[BufferType.LOCAL_LSE].buffer_shape == (2, 4 * T)
    # the gather is a genuine permutation of blocks
    memcpy = fw.instructions[0]
    assert any(s.index != d.index for s, d in memcpy.src_dst_pairs)


def test_rows_tables_and_concatenated_ranges():
    seqs = [700]
    mask = lambda_mask_fn(seqs, seqs, torch.int32, n_starting=16, l_pretrain=200)
    fw, bw, _ = build_single_device_plans(seqs, 128, 2, 2, 16, 1, mask)
    attn = next(i for i in fw.instructions if isinstance(i, AttnInstr))
    full = _allowed(mask, seqs, seqs)[0]
    m = attn.attn_mask.numpy()
    assert m.shape == (2, 2, sum(attn.seqlens_q))
    q0 = 0
    n_rows_head0 = len(attn.seqlens_q) // 2
    for b in range(n_rows_head0):  # rows of head block 0, in block order
        kv_ids = []  # recover kv block ids from the local->buffer gather
        slots = [x.index for x in attn.kv_block_table[b]]
        gather = {d.index: s.index for s, d in fw.instructions[0].src_dst_pairs if d.buffer_type == BufferType.BUFFER_KV}
        kv_ids = [gather[s] for s in slots]  # local kv index == block id for head block 0
        assert kv_ids == sorted(kv_ids)
        assert attn.seqlens_kv[b] == 128 * len(kv_ids)
        allowed = oracle.ranges_to_bool(m[:, :, q0 : q0 + 128], attn.seqlens_kv[b])
        n_q = attn.q_block_table[b][0].n_tokens
        cols = np.concatenate([np.arange(j * 128, (j + 1) * 128) for j in kv_ids])
        want = np.zeros((128, len(cols)), dtype=bool)
        valid = cols < 700
        want[:n_q, valid] = full[b * 128 : b * 128 + n_q][:, cols[valid]]
        assert np.array_equal(allowed, want), b
        # blocks nobody in the row attends are not in the row's table
        assert set(kv_ids) == {j for j in range(6) if full[b * 128 : b * 128 + n_q, j * 128 : min(700, (j + 1) * 128)].any()}
        q0 += 128
    # backward: one private dKV slot per (row, kv block), all distinct
    bwd = next(i for i in bw.instructions if isinstance(i, AttnBackwardInstr))
    slots = [x.index for row in bwd.dkv_block_table for x in row]
    assert len(slots) == len(set(slots)) == sum(len(r) for r in bwd.kv_block_table)
    sums = [i for i in bw.instructions if isinstance(i, SumInstr)]
    assert [s.output_is_unpadded for s in sums] == [0, 1, 1]


PLAN_CASES = {
    "c1_blockwise_causal_fp32_shapes": dict(seqlens=[512, 1024], block_size=256, n_heads=2, n_groups=2, head_dim=64,
                                           head_block=1, n_kv_groups=4),
    "gqa_ragged_fold": dict(seqlens=[300, 17, 129], block_size=64, n_heads=4, n_groups=2, head_dim=16, head_block=2,
                            n_kv_groups=3, fold=True),
    "lambda": dict(seqlens=[400], block_size=64, n_heads=2, n_groups=1, head_dim=16, head_block=2, mask="lambda",
                   mask_kwargs=dict(n_starting=8, l_pretrain=100), n_kv_groups=2),
    "shared_prefix_contiguous_split": dict(seqlens=[256 + 40 + 100], block_size=64, n_heads=5, n_groups=1,
                                           head_dim=16, head_block=5, mask="shared_prefix",
                                           mask_info=[dict(prefix=256, continuations=[40, 100])], n_kv_groups=2,
                                           kv_split="contiguous"),
}


@pytest.mark.parametrize("name", list(PLAN_CASES))
def test_plan_on_oracle_matches_whole_sequence_attention(name):
    """Any correct schedule must reproduce dense attention: gather, per-stage
    partials, merges, private dKV replicas and their sums all cancel out."""
    case = make_case(**PLAN_CASES[name])
    got = run_plan_oracle(case, backward=True)
    want = dense_truth(case, backward=True)
    tol = [1.6e-2, 1e-5, None, None]  # out: one bf16 rounding of O(1) values; lse: fp32
    for g, w, t in zip(got[:2], want[:2], tol[:2]):
        assert np.abs(g.float().numpy() - w).max() <= t
    for g, w in zip(got[2:], want[2:]):
        err = np.abs(g.float().numpy() - w) / np.maximum(1.0, np.abs(w))
        assert err.max() <= 2e-2
    if PLAN_CASES[name].get("fold"):
        kinds = [i.output_is_unpadded for i in case["fw"].instructions if isinstance(i, AttnReductionInstr)]
        assert 0 in kinds and kinds[-1] == 1
