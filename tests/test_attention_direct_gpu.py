"""The attention entry points called directly (dcp_amd.flash_attn_interface, the reference's
_flash_attn_varlen_forward / _backward signatures, through the C ABI) on hand-built paged
problems that plans of ordinary size do not reach, against the numpy oracle in fp64 on the same
rounded inputs; plus plan-level cases with garbage in the slot padding and with every
(q block, kv block) pair as its own partial.

Bounds as in tests/plan_cases.py: max-abs 2e-2 on out and dQ, 1e-3 on the LSE, 2e-2 * max(1, |ref|)
on dK/dV."""

import numpy as np
import pytest
import torch

from oracle import dcp_oracle as oracle
from tests.plan_cases import (GRAD_TOL, LSE_TOL, OUT_TOL, check_against_truth, dense_truth, make_case, max_abs_err,
                              run_executor, scaled_err)

pytestmark = pytest.mark.gpu


def _paged_rows(gpu, rows, bs, hq, hkv, d, seed):
    """``rows`` = [(n_queries, n_kv_blocks, ranges[n_ranges, 2, n_queries])]: q/out/dout slots in
    row order, kv slots dealt from a seeded permutation, one private dK/dV slot per (row, kv block)."""
    g = torch.Generator().manual_seed(seed)
    n_rows = len(rows)
    n_kv = sum(r[1] for r in rows)
    dt = torch.bfloat16
    rnd = lambda *shape: (torch.randn(*shape, generator=g) * 0.5).to(dt)
    q, dout = rnd(n_rows, bs, hq, d), rnd(n_rows, bs, hq, d) * 2
    kv = rnd(n_kv, bs, 2, hkv, d)
    perm = torch.randperm(n_kv, generator=g).tolist()
    max_kv = max(r[1] for r in rows)
    kv_table = torch.full((n_rows, max_kv), -1, dtype=torch.int32)
    dkv_table = torch.full((n_rows, max_kv), -1, dtype=torch.int32)
    cu_q, cu_kv, nxt = [0], [0], 0
    n_ranges = max(np.asarray(r[2]).shape[0] for r in rows)
    total_q = sum(r[0] for r in rows)
    rng = torch.zeros(n_ranges, 2, total_q, dtype=torch.int32)
    for b, (nq, nblk, ranges) in enumerate(rows):
        ranges = torch.as_tensor(np.asarray(ranges), dtype=torch.int32)
        rng[: ranges.shape[0], :, cu_q[-1] : cu_q[-1] + nq] = ranges
        for j in range(nblk):
            kv_table[b, j] = perm[nxt]
            dkv_table[b, j] = nxt
            nxt += 1
        cu_q.append(cu_q[-1] + nq)
        cu_kv.append(cu_kv[-1] + nblk * bs)
    dev = lambda t: t.to(gpu).contiguous()
    i32 = lambda x: torch.tensor(x, dtype=torch.int32)
    slots = torch.arange(n_rows, dtype=torch.int32).reshape(n_rows, 1)
    return dict(q=dev(q), kv=dev(kv), dout=dev(dout), cu_q=dev(i32(cu_q)), cu_kv=dev(i32(cu_kv)),
                rng=dev(rng if n_ranges > 1 else rng[0]), slots=dev(slots), kv_table=dev(kv_table),
                dkv_table=dev(dkv_table), rows=rows, bs=bs, total_q=total_q, n_dkv=nxt, max_kv=max_kv,
                host=dict(q=q, kv=kv, dout=dout, kv_table=kv_table, dkv_table=dkv_table))


def _run_direct(pr, backward=True):
    from dcp_amd.flash_attn_interface import _flash_attn_varlen_backward, _flash_attn_varlen_forward

    gpu = pr["q"].device
    bs, (n_rows, _, hq, d) = pr["bs"], pr["q"].shape
    k, v = pr["kv"][:, :, 0], pr["kv"][:, :, 1]
    out = torch.full_like(pr["q"], 3.0)
    lse = torch.full((hq, n_rows, bs), 3.0, device=gpu)
    total_k = int(pr["cu_kv"][-1])
    _flash_attn_varlen_forward(pr["q"], k, v, pr["cu_q"], pr["cu_kv"], pr["total_q"], bs, pr["max_kv"] * bs, 0.0, d ** -0.5,
                               causal=False, window_size_left=-1, window_size_right=-1, softcap=0.0, alibi_slopes=None,
                               return_softmax=False, attn_range=pr["rng"], q_block_table=pr["slots"],
                               kv_block_table=pr["kv_table"], out_block_table=pr["slots"], out_=out, lse_=lse)
    res = [out, lse]
    if backward:
        dq = torch.full_like(pr["q"], 3.0)
        dkv = torch.full((pr["n_dkv"], bs, 2, k.shape[2], d), 3.0, dtype=pr["q"].dtype, device=gpu)
        _flash_attn_varlen_backward(pr["dout"], pr["q"], k, v, out, lse, dq, dkv[:, :, 0], dkv[:, :, 1], pr["cu_q"],
                                    pr["cu_kv"], pr["total_q"], total_k, bs, pr["max_kv"] * bs, 0.0, d ** -0.5, False, -1, -1,
                                    0.0, None, False, attn_range=pr["rng"], q_block_table=pr["slots"],
                                    kv_block_table=pr["kv_table"], out_block_table=pr["slots"], dq_block_table=pr["slots"],
                                    dkv_block_table=pr["dkv_table"])
        res += [dq, dkv]
    torch.cuda.synchronize()
    return [r.float().cpu().numpy() for r in res]


def _check_direct(pr, res):
    """Row by row against the oracle; returns the worst errors."""
    h = pr["host"]
    bs = pr["bs"]
    worst = dict(out=0.0, lse=0.0, dq=0.0, dkv=0.0)
    for b, (nq, nblk, ranges) in enumerate(pr["rows"]):
        if nq == 0 or nblk == 0:
            continue  # nothing to compare with: the caller states what such a row must leave behind
        slots = h["kv_table"][b, :nblk].long()
        kv = h["kv"][slots].float().numpy().reshape(nblk * bs, 2, -1, h["kv"].shape[-1])
        q, dout = h["q"][b, :nq].float().numpy(), h["dout"][b, :nq].float().numpy()
        allowed = oracle.ranges_to_bool(np.asarray(ranges), nblk * bs)
        t_out, t_lse = oracle.range_attention_fwd(q, kv[:, 0], kv[:, 1], allowed)
        worst["out"] = max(worst["out"], max_abs_err(res[0][b, :nq], t_out))
        # a query that attends nothing has lse = +inf in the oracle: the kernel must say +inf exactly
        # there and be finite everywhere else; finite entries are compared by value
        got_lse = np.asarray(res[1][:, b, :nq], dtype=np.float64)
        empty = np.isposinf(t_lse)
        assert np.array_equal(np.isposinf(got_lse), empty), f"row {b}: +inf LSE not exactly where no key is attended"
        assert np.isfinite(got_lse[~empty]).all() and np.isfinite(t_lse[~empty]).all(), f"row {b}: non-finite LSE"
        if (~empty).any():
            worst["lse"] = max(worst["lse"], float(np.abs(got_lse[~empty] - t_lse[~empty]).max()))
        if len(res) > 2:
            # the backward starts from the kernel's own (rounded) out and lse, as the executor's does
            t_dq, t_dk, t_dv = oracle.range_attention_bwd(q, kv[:, 0], kv[:, 1], res[0][b, :nq], res[1][:, b, :nq], dout, allowed)
            got = res[3][h["dkv_table"][b, :nblk].long().numpy()].reshape(nblk * bs, 2, -1, kv.shape[-1])
            worst["dq"] = max(worst["dq"], max_abs_err(res[2][b, :nq], t_dq))
            worst["dkv"] = max(worst["dkv"], scaled_err(got[:, 0], t_dk), scaled_err(got[:, 1], t_dv))
    return worst


def test_row_with_more_kv_blocks_than_the_kernels_keep_in_lds(gpu):
    """The forward and dQ kernels keep the first 1024 entries of a row's kv block table in LDS and
    read later entries from global memory: a row of 1100 blocks (64-token blocks), one with two
    ranges whose second lies wholly past block 1024, and an ordinary short row beside them."""
    bs, nblk = 64, 1100
    t = np.arange(bs)
    wide = np.stack([t * 7, (nblk - 1) * bs + t + 1])[None]                       # [t*7, last block's diagonal)
    two = np.stack([np.stack([t * 0, t * 0 + 100]), np.stack([1030 * bs + t, 1090 * bs + 5 * t + 1])])
    short = np.stack([t[:40] * 0, t[:40] + 1 + bs])[None]
    pr = _paged_rows(gpu, [(bs, nblk, wide), (bs, nblk, two), (40, 2, short)], bs, hq=2, hkv=1, d=64, seed=5)
    worst = _check_direct(pr, _run_direct(pr))
    assert worst["out"] <= OUT_TOL and worst["lse"] <= LSE_TOL and worst["dq"] <= GRAD_TOL and worst["dkv"] <= GRAD_TOL, worst


def test_dkv_of_a_row_whose_keys_do_not_fill_a_128_key_tile(gpu):
    """The dK/dV kernel works on 128 keys at a time; rows of 1 and 3 blocks of 64 keys end inside
    such a tile, and the slots of keys nobody attends receive zeros."""
    bs = 64
    t = np.arange(bs)
    one = np.stack([t * 0, np.minimum(t + 1, 20)])[None]       # only keys 0..19 are attended
    three = np.stack([t * 0 + 10, t + 1 + 2 * bs])[None]
    pr = _paged_rows(gpu, [(bs, 1, one), (50, 3, three[:, :, :50])], bs, hq=4, hkv=2, d=128, seed=6)
    res = _run_direct(pr)
    worst = _check_direct(pr, res)
    assert worst["out"] <= OUT_TOL and worst["lse"] <= LSE_TOL and worst["dq"] <= GRAD_TOL and worst["dkv"] <= GRAD_TOL, worst
    dkv = res[3]
    assert not (dkv[0, 20:] != 0).any(), "keys no query attends get exact zeros, not the buffer's fill value"


@pytest.mark.parametrize("name", ["ragged_gqa", "lambda"])
def test_slot_padding_may_hold_finite_garbage(gpu, name):
    """The gather overwrites only a block's tokens; the rest of its slot keeps what the memory
    held.  The kernels load whole tiles, so that padding reaches the matrix instructions: it
    must be masked out, not multiplied by zero weights that a non-finite product would spoil.
    Slots filled with +-200 (finite, as the C ABI requires) give the same results as zeroed ones."""
    cfg = dict(ragged_gqa=dict(seqlens=[1000, 333, 1, 257], block_size=256, n_heads=8, n_groups=2, head_dim=128,
                               head_block=4, qkv_scale=0.5, n_kv_groups=2),
               lambda_=dict(seqlens=[700, 90], block_size=128, n_heads=4, n_groups=1, head_dim=64, head_block=2,
                            mask="lambda", qkv_scale=0.5, mask_kwargs=dict(n_starting=16, l_pretrain=200)))
    case = make_case(**cfg[name if name != "lambda" else "lambda_"])
    clean, _ = run_executor(case, backward=True)
    dirty, _ = run_executor(case, backward=True, poison=200.0)
    check_against_truth(dirty, dense_truth(case, backward=True))
    for a, b in zip(clean, dirty):  # and bit for bit what zeroed slots give
        assert torch.equal(a.view(torch.int16) if a.dtype != torch.float32 else a.view(torch.int32),
                           b.view(torch.int16) if b.dtype != torch.float32 else b.view(torch.int32))


@pytest.mark.parametrize("head_block", [1, 8])
def test_config1_every_q_block_kv_block_pair_its_own_partial(gpu, head_block):
    """BASELINE config 1 at its full shape (seqlens 512/1024/1536/2048, 256-token blocks, 8 heads,
    D=64, causal), every (q block, kv block) pair computed as its own partial (up to 8 per q block)
    and merged; run in bf16, the types the attention kernels take (the reference's flash-attention
    has no fp32 either; the fp32 case of the merge is covered below)."""
    case = make_case(seqlens=[512, 1024, 1536, 2048], block_size=256, n_heads=8, n_groups=8, head_dim=64,
                     head_block=head_block, n_kv_groups=8)
    n_partials = [len(i.seqlens_q) for i in case["fw"].instructions if type(i).__name__ == "AttnInstr"]
    assert len(n_partials) == 8, "eight attention launches: the j-th takes every row's j-th kv block"
    assert sum(n_partials) == 70 * (8 // head_block), "70 (q block, kv block) pairs per head block"
    res, _ = run_executor(case, backward=True)
    check_against_truth(res, dense_truth(case, backward=True))


def test_config1_fp32_merge_of_up_to_eight_partials(gpu):
    """The fp32 half of config 1: the partial (out, lse) of every (q block, kv block) pair of the
    2048-token sequence computed by the oracle in fp32, merged by the HIP kernel in fp32 (1 to 8
    sources per q block) and compared with dense causal attention in fp64."""
    from dcp_amd.ops.fused_ops import flash_attn_update_out_lse

    rng = np.random.default_rng(11)
    L, bs, H, D = 2048, 256, 8, 64
    nb = L // bs
    q, k, v = (rng.standard_normal((L, H, D)).astype(np.float32) for _ in range(3))
    causal = np.tril(np.ones((L, L), dtype=bool))
    t_out, t_lse = oracle.range_attention_fwd(q, k, v, causal)
    n_slots = nb * (nb + 1) // 2
    outs = np.zeros((n_slots, bs, H, D), dtype=np.float32)
    lses = np.zeros((H, n_slots, bs), dtype=np.float32)
    table = np.full((nb, 8), -1, dtype=np.int32)
    slot = 0
    for i in range(nb):
        for j in range(i + 1):
            o, l = oracle.range_attention_fwd(q[i * bs:(i + 1) * bs], k[j * bs:(j + 1) * bs], v[j * bs:(j + 1) * bs],
                                              causal[i * bs:(i + 1) * bs, j * bs:(j + 1) * bs], dtype=np.float32)
            outs[slot], lses[:, slot] = o, l
            table[i, j] = slot
            slot += 1
    dev = lambda a: torch.from_numpy(a).to(gpu)
    dst_out = torch.zeros(L, H, D, device=gpu)
    dst_lse = torch.zeros(H, L, device=gpu)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=gpu)
    flash_attn_update_out_lse(dev(outs), dst_out, dev(lses), dst_lse, H, dev(table), i32([i * bs for i in range(nb)]),
                              i32([bs] * nb), i32([i + 1 for i in range(nb)]), bs, bs * H * D, H * D, bs, 1, n_slots * bs, L,
                              D, 8, 64)
    torch.cuda.synchronize()
    assert max_abs_err(dst_out.cpu().numpy(), t_out) <= 1e-5
    assert max_abs_err(dst_lse.cpu().numpy(), t_lse) <= 1e-5


@pytest.mark.parametrize("seed,d,bs,hq,hkv", [(21, 128, 128, 4, 2), (22, 64, 64, 2, 2), (23, 128, 64, 8, 2)])
def test_arbitrary_ranges(gpu, seed, d, bs, hq, hkv):
    """Ranges no mask generator produces: starts and ends anywhere (inside tiles, past the row's
    keys, below zero length), empty ranges beside full ones, two ranges that overlap, touch or
    nest, queries that attend a single key, rows whose queries do not fill the block.  The
    kernels classify tiles from the hull and the core of a tile's ranges and mask the rest bit by
    bit, so every row mixes skipped, unmasked and masked tiles."""
    rng = np.random.default_rng(seed)
    rows = []
    for _ in range(6):
        nblk = int(rng.integers(1, 6))
        nq = int(rng.choice([bs, bs, int(rng.integers(1, bs + 1))]))
        n_keys = nblk * bs
        n_ranges = int(rng.integers(1, 3))
        ranges = np.zeros((n_ranges, 2, nq), dtype=np.int64)
        for r in range(n_ranges):
            kind = rng.integers(0, 5, size=nq)
            s = rng.integers(0, n_keys + 1, size=nq)
            e = rng.integers(0, n_keys + bs, size=nq)            # may lie past the row's keys, or before the start
            s = np.where(kind == 0, 0, s)                         # from the first key
            e = np.where(kind == 1, s + 1, e)                     # a single key (or none, at the very end)
            e = np.where(kind == 2, s, e)                         # empty
            s, e = np.where(kind == 3, 0, s), np.where(kind == 3, n_keys, e)  # everything
            if r == 0 and rng.integers(0, 2):                     # a smooth band, so that whole tiles are unmasked
                t = np.arange(nq)
                s, e = np.maximum(t * n_keys // max(nq, 1) - bs, 0), np.minimum(t * n_keys // max(nq, 1) + bs + 1, n_keys)
            ranges[r, 0], ranges[r, 1] = s, e
        rows.append((nq, nblk, ranges))
    pr = _paged_rows(gpu, rows, bs, hq=hq, hkv=hkv, d=d, seed=seed)
    worst = _check_direct(pr, _run_direct(pr))
    assert worst["out"] <= OUT_TOL and worst["lse"] <= LSE_TOL and worst["dq"] <= GRAD_TOL and worst["dkv"] <= GRAD_TOL, worst
