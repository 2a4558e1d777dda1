"""Degenerate inputs on the GPU, through the operator layer and the C ABI: calls with no blocks,
no ops or no rows launch nothing and touch nothing; rows without queries, without keys, or whose
every query has an empty range give the documented outputs (out 0, LSE +inf, zero gradients) and
leave everything else as it was."""

import numpy as np
import pytest
import torch

from dcp_amd.ops import fused_ops
from tests.test_attention_direct_gpu import _check_direct, _paged_rows, _run_direct
from tests.plan_cases import GRAD_TOL, LSE_TOL, OUT_TOL

pytestmark = pytest.mark.gpu


def test_calls_with_nothing_to_do_touch_nothing(gpu):
    e64 = torch.zeros(0, dtype=torch.int64, device=gpu)
    e32 = torch.zeros(0, dtype=torch.int32, device=gpu)
    dst = torch.full((4, 64), 3.0, dtype=torch.bfloat16, device=gpu)
    fused_ops.fused_copy_bf16_varlen(e64, e32, e32, e64, e32, e32, e32, 64, 64)
    fused_ops.fused_copy_fp32_varlen_lse(e64, e32, e32, e64, e32, e32, e32, 2, 64, 64)
    fused_ops.fused_copy_bf16_varlen_dkv(e64, e64, e32, 64, 128, 16)
    fused_ops.fused_blockwise_sum(e64, torch.zeros((0, 2), dtype=torch.int32, device=gpu), e32, e32, e64, e32, e32, e32,
                                  torch.bfloat16, 2, 64, 64)
    src = torch.zeros((1, 8, 2, 64), dtype=torch.bfloat16, device=gpu)
    lse_s = torch.zeros((2, 1, 8), device=gpu)
    lse_d = torch.full((2, 8), 3.0, device=gpu)
    fused_ops.flash_attn_update_out_lse(src, dst.view(-1)[: 2 * 64].view(1, 2, 64), lse_s, lse_d, 2,
                                        torch.zeros((0, 1), dtype=torch.int32, device=gpu), e32, e32, e32, 8, 8 * 128, 128,
                                        8, 1, 8, 8, 64, 1, 8)
    # ops that exist but move nothing: zero elements / zero tokens
    srcb = torch.ones(64, dtype=torch.bfloat16, device=gpu)
    one64 = lambda t: torch.tensor([t.data_ptr()], dtype=torch.int64, device=gpu)
    z = torch.zeros(1, dtype=torch.int32, device=gpu)
    fused_ops.fused_copy_bf16_varlen(one64(srcb), z, z + 64, one64(dst), z, z + 64, z, 64, 64)
    torch.cuda.synchronize()
    assert (dst == 3.0).all() and (lse_d == 3.0).all()


def test_attention_with_no_rows(gpu):
    from dcp_amd.flash_attn_interface import _flash_attn_varlen_backward, _flash_attn_varlen_forward

    bs, h, d = 64, 2, 64
    q = torch.zeros((1, bs, h, d), dtype=torch.bfloat16, device=gpu)
    kv = torch.zeros((1, bs, 2, h, d), dtype=torch.bfloat16, device=gpu)
    out, lse = torch.full_like(q, 3.0), torch.full((h, 1, bs), 3.0, device=gpu)
    cu = torch.zeros(1, dtype=torch.int32, device=gpu)
    rng = torch.zeros((2, 0), dtype=torch.int32, device=gpu)
    t1 = torch.zeros((0, 1), dtype=torch.int32, device=gpu)
    _flash_attn_varlen_forward(q, kv[:, :, 0], kv[:, :, 1], cu, cu, 0, bs, bs, 0.0, None, attn_range=rng, q_block_table=t1,
                               kv_block_table=t1, out_block_table=t1, out_=out, lse_=lse)
    dq, dkv = torch.full_like(q, 3.0), torch.full_like(kv, 3.0)
    _flash_attn_varlen_backward(q, q, kv[:, :, 0], kv[:, :, 1], out, lse, dq, dkv[:, :, 0], dkv[:, :, 1], cu, cu, 0, 0, bs,
                                bs, 0.0, None, False, -1, -1, 0.0, None, False, attn_range=rng, q_block_table=t1,
                                kv_block_table=t1, out_block_table=t1, dq_block_table=t1, dkv_block_table=t1)
    torch.cuda.synchronize()
    for t in (out, lse, dq, dkv):
        assert (t == 3.0).all()


def test_rows_without_queries_keys_or_ranges(gpu):
    """Five rows: ordinary; no queries (two kv blocks); every range empty; no kv blocks at all;
    ordinary again.  Query positions past a row's queries keep the buffers' fill value."""
    bs = 64
    t = np.arange(bs)
    causal = np.stack([t * 0, t + 1 + bs])[None]
    none = np.zeros((1, 2, 30), dtype=np.int64)
    rows = [(bs, 2, causal), (0, 2, np.zeros((1, 2, 0), dtype=np.int64)), (30, 1, none),
            (20, 0, np.zeros((1, 2, 20), dtype=np.int64)), (50, 2, causal[:, :, :50])]
    pr = _paged_rows(gpu, rows, bs, hq=4, hkv=2, d=128, seed=11)
    res = _run_direct(pr)
    out, lse, dq, dkv = res
    with np.errstate(invalid="ignore"):  # +inf against +inf in the LSE of the row that attends nothing
        worst = _check_direct(pr, res)
    assert worst["out"] <= OUT_TOL and worst["dq"] <= GRAD_TOL and worst["dkv"] <= GRAD_TOL, worst
    # (the LSE of a query that attends nothing is +inf on the GPU; the oracle agrees, and inf - inf
    # is not a number, so it is checked here instead of through the error norm)
    for b, nq in ((2, 30), (3, 20)):
        assert np.isposinf(lse[:, b, :nq]).all() and not out[b, :nq].any() and not dq[b, :nq].any()
    assert np.isfinite(lse[:, 0, :bs]).all() and np.isfinite(lse[:, 4, :50]).all()
    # untouched: the row without queries, and the positions past each row's queries
    assert (out[1] == 3.0).all() and (dq[1] == 3.0).all() and (lse[:, 1] == 3.0).all()
    assert (out[2, 30:] == 3.0).all() and (out[4, 50:] == 3.0).all() and (dq[3, 20:] == 3.0).all()
    # keys nobody attends receive exact zeros: the kv blocks of the query-less row and of the row
    # whose ranges are all empty
    table = pr["host"]["dkv_table"]
    for b, nblk in ((1, 2), (2, 1)):
        for j in range(nblk):
            assert not dkv[int(table[b, j])].any()
