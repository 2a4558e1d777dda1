"""Pins the CPU oracle before anything is compared against it.

The reference holds no stored vectors for this path (its op tests compare
random inputs with in-file torch references and mostly only print), so the
oracle is pinned by what the mathematics fixes: library routines
(scipy logsumexp, torch SDPA, torch autograd), brute force on small inputs,
closed forms and invariants -- each chosen so that a dropped term, a wrong
sign or a transposed operand fails."""

import numpy as np
import pytest
import scipy.special
import torch
import torch.nn.functional as F

from oracle import dcp_oracle as oracle


def test_round_bf16_matches_torch():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(100000, generator=g) * 37.0
    x = torch.cat([x, torch.tensor([0.0, -0.0, 1.0, 3.0e38, -3.0e38, 1e-40, float("inf")])])
    want = x.to(torch.bfloat16).float().numpy()
    got = oracle.round_bf16(x.numpy())
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # ties go to even: 1 + 2^-8 is halfway between 1 and 1 + 2^-7
    assert oracle.round_bf16(np.array([1.0 + 2.0 ** -8], dtype=np.float32))[0] == 1.0
    assert oracle.round_bf16(np.array([1.0 + 3 * 2.0 ** -8], dtype=np.float32))[0] == np.float32(1.0 + 2.0 ** -6)


def test_block_copy_is_plain_indexing():
    rng = np.random.default_rng(0)
    src = rng.integers(0, 2 ** 16, 6 * 100, dtype=np.uint16)
    dst = rng.integers(0, 2 ** 16, 8 * 100, dtype=np.uint16)
    before = dst.copy()
    src_blk, dst_blk, n = [5, 0, 3], [7, 2, 1], [100, 1, 37]
    oracle.block_copy(src, [b * 100 for b in src_blk], dst, [b * 100 for b in dst_blk], n)
    want = before.reshape(8, 100).copy()
    for s, d, k in zip(src_blk, dst_blk, n):
        want[d, :k] = src.reshape(6, 100)[s, :k]
    assert np.array_equal(dst.reshape(8, 100), want)
    # gather followed by the inverse scatter restores the source
    perm = rng.permutation(6)
    packed = np.zeros_like(src)
    oracle.block_copy(src, np.arange(6) * 100, packed, perm * 100, [100] * 6)
    back = np.zeros_like(src)
    oracle.block_copy(packed, perm * 100, back, np.arange(6) * 100, [100] * 6)
    assert np.array_equal(back, src)


def _rand_partials(seed, S=5, T=17, H=3, D=8, lo=-5.0, hi=5.0):
    rng = np.random.default_rng(seed)
    return rng.standard_normal((S, T, H, D)), rng.uniform(lo, hi, (S, H, T))


def test_blockwise_sum_is_the_exact_sum():
    """Pinned by the exactly rounded sum (math.fsum) element by element, by integer-valued blocks
    whose sum is exact in every order, and by order invariance on them; the single rounding to the
    storage type is torch's (test_round_bf16_matches_torch)."""
    import math

    rng = np.random.default_rng(5)
    srcs = [rng.standard_normal((7, 33)).astype(np.float32) * 10.0 ** rng.integers(-3, 4) for _ in range(9)]
    got = oracle.blockwise_sum(srcs)
    assert got.dtype == np.float64 and got.shape == (7, 33)
    exact = np.array([[math.fsum(float(s[i, j]) for s in srcs) for j in range(33)] for i in range(7)])
    # nine float64 additions of float32 values: within a few ulps of the exact sum's magnitude
    assert np.abs(got - exact).max() <= 16 * np.finfo(np.float64).eps * np.abs(np.stack(srcs)).sum(0).max()
    ints = [rng.integers(-1000, 1000, size=(5, 16)).astype(np.float32) for _ in range(6)]
    want = np.stack(ints).astype(np.int64).sum(0)
    assert np.array_equal(oracle.blockwise_sum(ints), want)
    assert np.array_equal(oracle.blockwise_sum(ints[::-1]), want)
    assert np.array_equal(oracle.blockwise_sum([ints[0]]), ints[0])  # one source: the block itself
    # bf16 sources are summed as the values they hold, not re-rounded in between
    b = [oracle.round_to(x * 0.37, "bf16") for x in ints]
    assert np.array_equal(oracle.blockwise_sum(b), np.stack([np.asarray(x, np.float64) for x in b]).sum(0))


def test_merge_against_scipy_logsumexp():
    outs, lses = _rand_partials(0)
    out, lse = oracle.merge_out_lse(outs, lses)
    want_lse = scipy.special.logsumexp(lses, axis=0)
    w = np.exp(lses - want_lse)  # convex weights
    assert np.allclose(w.sum(axis=0), 1.0)
    want_out = np.einsum("sht,sthd->thd", w, outs)
    assert np.allclose(lse, want_lse, rtol=0, atol=1e-12)
    assert np.allclose(out, want_out, rtol=0, atol=1e-12)


def test_merge_equals_folded_pairwise_update():
    # the reference's two-way update, folded left to right
    outs, lses = _rand_partials(1, S=6)
    a = oracle.merge_out_lse(outs, lses)
    b = oracle.merge_pairwise(outs, lses)
    assert np.allclose(a[0], b[0], atol=1e-12) and np.allclose(a[1], b[1], atol=1e-12)


def test_merge_invariants():
    outs, lses = _rand_partials(2, S=4)
    base = oracle.merge_out_lse(outs, lses)
    # permutation of sources
    p = [2, 0, 3, 1]
    perm = oracle.merge_out_lse(outs[p], lses[p])
    assert np.allclose(base[0], perm[0], atol=1e-12) and np.allclose(base[1], perm[1], atol=1e-12)
    # associativity: merge(merge(0,1), merge(2,3))
    left = oracle.merge_out_lse(outs[:2], lses[:2])
    right = oracle.merge_out_lse(outs[2:], lses[2:])
    both = oracle.merge_out_lse(np.stack([left[0], right[0]]), np.stack([left[1], right[1]]))
    assert np.allclose(base[0], both[0], atol=1e-12) and np.allclose(base[1], both[1], atol=1e-12)
    # a single source is returned unchanged
    one = oracle.merge_out_lse(outs[:1], lses[:1])
    assert np.array_equal(one[0], outs[0]) and np.array_equal(one[1], lses[0])
    # shifting every lse by c shifts the result by c and leaves out alone
    sh = oracle.merge_out_lse(outs, lses + 3.25)
    assert np.allclose(sh[1], base[1] + 3.25, atol=1e-12) and np.allclose(sh[0], base[0], atol=1e-12)


def test_merge_nonfinite_sources_are_ignored():
    outs, lses = _rand_partials(3, S=4)
    lses[1, 0, :5] = np.inf
    lses[2, 1, 3:9] = -np.inf
    outs[1, :5, 0] = 1e30  # must not leak
    lses[:, 2, 4] = [np.inf, -np.inf, np.inf, -np.inf]  # no finite source at all
    out, lse = oracle.merge_out_lse(outs, lses)
    keep = [0, 2, 3]
    ref = oracle.merge_out_lse(outs[keep], lses[keep])
    assert np.allclose(out[:5, 0], ref[0][:5, 0], atol=1e-12)
    assert np.allclose(lse[0, :5], ref[1][0, :5], atol=1e-12)
    assert lse[2, 4] == -1.0 and np.all(out[4, 2] == 0.0)
    assert np.isfinite(out).all() and np.isfinite(lse).all()


def test_merge_nan_lse_is_a_source():
    """fused_ops.py:123 tests ``lse != -inf and lse != inf``: NaN is not an empty source, so it
    poisons the merged (token, head) -- and nothing else."""
    outs, lses = _rand_partials(5, S=3)
    lses[1, 2, 7] = np.nan
    lses[0, 1, 3], lses[2, 1, 3] = np.inf, np.nan
    out, lse = oracle.merge_out_lse(outs, lses)
    assert np.isnan(lse[2, 7]) and np.isnan(out[7, 2]).all() and np.isnan(lse[1, 3]) and np.isnan(out[3, 1]).all()
    poisoned = np.zeros(lse.shape, dtype=bool)
    poisoned[2, 7] = poisoned[1, 3] = True
    assert np.isfinite(lse[~poisoned]).all() and np.isfinite(out[~poisoned.T]).all()
    clean = lses.copy()
    clean[1, 2, 7] = clean[2, 1, 3] = 0.0
    ref = oracle.merge_out_lse(outs, clean)
    assert np.array_equal(lse[~poisoned], ref[1][~poisoned]) and np.array_equal(out[~poisoned.T], ref[0][~poisoned.T])


def _torch_dense(q, k, v, allowed, dout=None):
    """Textbook softmax attention in torch fp64 with autograd."""
    q = torch.tensor(q, dtype=torch.float64, requires_grad=dout is not None)
    k = torch.tensor(k, dtype=torch.float64, requires_grad=dout is not None)
    v = torch.tensor(v, dtype=torch.float64, requires_grad=dout is not None)
    g = q.shape[1] // k.shape[1]
    ke, ve = k.repeat_interleave(g, dim=1), v.repeat_interleave(g, dim=1)
    s = torch.einsum("thd,shd->hts", q, ke) / np.sqrt(q.shape[-1])
    s = s.masked_fill(~torch.tensor(allowed)[None], float("-inf"))
    lse = torch.logsumexp(s, dim=-1)
    out = torch.einsum("hts,shd->thd", torch.softmax(s, dim=-1), ve)
    if dout is None:
        return out.detach().numpy(), lse.detach().numpy()
    out.backward(torch.tensor(dout, dtype=torch.float64))
    return out.detach().numpy(), lse.detach().numpy(), q.grad.numpy(), k.grad.numpy(), v.grad.numpy()


def test_attention_forward_causal_equals_torch_sdpa():
    rng = np.random.default_rng(4)
    T, H, Hkv, D = 37, 4, 2, 16
    q, k, v = rng.standard_normal((T, H, D)), rng.standard_normal((T, Hkv, D)), rng.standard_normal((T, Hkv, D))
    ranges = np.stack([np.zeros(T, dtype=np.int64), np.arange(T) + 1])[None]  # [1,2,T]
    out, lse = oracle.range_attention_fwd(q, k, v, oracle.ranges_to_bool(ranges, T))
    tq = torch.tensor(q).permute(1, 0, 2)[None]
    tk = torch.tensor(k).repeat_interleave(2, dim=1).permute(1, 0, 2)[None]
    tv = torch.tensor(v).repeat_interleave(2, dim=1).permute(1, 0, 2)[None]
    want = F.scaled_dot_product_attention(tq, tk, tv, is_causal=True)[0].permute(1, 0, 2).numpy()
    assert np.allclose(out, want, atol=1e-12)
    want_lse = _torch_dense(q, k, v, np.tril(np.ones((T, T), dtype=bool)))[1]
    assert np.allclose(lse, want_lse, atol=1e-12)


def test_attention_two_ranges_union_and_empty_rows():
    rng = np.random.default_rng(5)
    Tq, Tk, H, D = 9, 20, 2, 8
    q, k, v = rng.standard_normal((Tq, H, D)), rng.standard_normal((Tk, H, D)), rng.standard_normal((Tk, H, D))
    ranges = np.zeros((2, 2, Tq), dtype=np.int64)
    ranges[0, 0], ranges[0, 1] = 0, [3, 3, 3, 3, 3, 3, 3, 0, 0]
    ranges[1, 0], ranges[1, 1] = [0, 1, 2, 5, 9, 12, 3, 4, 0], [1, 4, 4, 9, 15, 20, 3, 9, 0]
    allowed = oracle.ranges_to_bool(ranges, Tk)
    brute = np.zeros((Tq, Tk), dtype=bool)
    for i in range(Tq):
        for r in range(2):
            brute[i, ranges[r, 0, i] : ranges[r, 1, i]] = True
    assert np.array_equal(allowed, brute)
    assert allowed[1].sum() == 4  # overlapping ranges [0,3) u [1,4) count once
    out, lse = oracle.range_attention_fwd(q, k, v, allowed)
    rows = allowed.any(axis=1)
    want = _torch_dense(q[rows], k, v, allowed[rows])
    assert np.allclose(out[rows], want[0], atol=1e-12) and np.allclose(lse[:, rows], want[1], atol=1e-12)
    assert not rows[8] and np.all(out[8] == 0) and np.all(np.isposinf(lse[:, 8]))


def test_attention_backward_equals_autograd_and_finite_differences():
    rng = np.random.default_rng(6)
    Tq, Tk, H, Hkv, D = 7, 11, 4, 2, 8
    q, k, v = rng.standard_normal((Tq, H, D)), rng.standard_normal((Tk, Hkv, D)), rng.standard_normal((Tk, Hkv, D))
    dout = rng.standard_normal((Tq, H, D))
    ranges = np.stack([rng.integers(0, 4, Tq), rng.integers(5, 12, Tq)])[None]
    allowed = oracle.ranges_to_bool(ranges, Tk)
    out, lse = oracle.range_attention_fwd(q, k, v, allowed)
    dq, dk, dv = oracle.range_attention_bwd(q, k, v, out, lse, dout, allowed)
    _, _, tdq, tdk, tdv = _torch_dense(q, k, v, allowed, dout)
    assert np.allclose(dq, tdq, atol=1e-11) and np.allclose(dk, tdk, atol=1e-11) and np.allclose(dv, tdv, atol=1e-11)
    # central differences of L = sum(out * dout) in a few coordinates
    def loss(q_, k_, v_):
        return (oracle.range_attention_fwd(q_, k_, v_, allowed)[0] * dout).sum()
    eps = 1e-6
    for arr, grad, idx in ((q, dq, (3, 1, 2)), (k, dk, (6, 1, 0)), (v, dv, (9, 0, 5))):
        plus, minus = arr.copy(), arr.copy()
        plus[idx] += eps
        minus[idx] -= eps
        args_p = [plus if a is arr else a for a in (q, k, v)]
        args_m = [minus if a is arr else a for a in (q, k, v)]
        fd = (loss(*args_p) - loss(*args_m)) / (2 * eps)
        assert abs(fd - grad[idx]) < 1e-6


def test_split_kv_partials_merge_to_unsplit_attention():
    rng = np.random.default_rng(7)
    T, H, D = 24, 2, 8
    q, k, v = rng.standard_normal((T, H, D)), rng.standard_normal((T, H, D)), rng.standard_normal((T, H, D))
    allowed = np.tril(np.ones((T, T), dtype=bool))
    full = oracle.range_attention_fwd(q, k, v, allowed)
    parts = []
    for cols in (slice(0, 8), slice(8, 16), slice(16, 24)):
        parts.append(oracle.range_attention_fwd(q, k[cols], v[cols], allowed[:, cols]))
    out, lse = oracle.merge_out_lse(np.stack([p[0] for p in parts]), np.stack([p[1] for p in parts]))
    assert np.allclose(out, full[0], atol=1e-12) and np.allclose(lse, full[1], atol=1e-12)


def test_flop_convention():
    # dcp/core/cost_model.py:120-127: fwd = 4*pairs*heads*dim, bwd = 2.5x
    assert oracle.attention_flops(10, 2, 8, "fwd") == 4 * 10 * 2 * 8
    assert oracle.attention_flops(10, 2, 8, "bwd") == 2.5 * 4 * 10 * 2 * 8
    assert oracle.attention_flops(10, 2, 8, "fwd+bwd") == 14 * 10 * 2 * 8


def test_torch_cpu_row_path_equals_the_numpy_oracle():
    """bench.py's CPU baseline (oracle/torch_cpu_path.py, fp32 torch on the host) against the numpy
    oracle in fp64: GQA, two ranges, a query that attends nothing."""
    from oracle.torch_cpu_path import row_attention_fwd_bwd

    rng = np.random.default_rng(9)
    Tq, Tk, H, Hkv, D = 37, 90, 4, 2, 32
    q, dout = rng.standard_normal((Tq, H, D)), rng.standard_normal((Tq, H, D))
    k, v = rng.standard_normal((Tk, Hkv, D)), rng.standard_normal((Tk, Hkv, D))
    t = np.arange(Tq)
    ranges = np.stack([np.stack([t * 0, np.minimum(t, 5)]), np.stack([t + 20, t + 41])])
    ranges[:, :, 11] = 0  # query 11 attends nothing (query 0's first range is empty too)
    allowed = oracle.ranges_to_bool(ranges, Tk)
    w_out, w_lse = oracle.range_attention_fwd(q, k, v, allowed)
    w_dq, w_dk, w_dv = oracle.range_attention_bwd(q, k, v, w_out, w_lse, dout, allowed)
    f32 = lambda x: torch.from_numpy(np.asarray(x, dtype=np.float32))
    out, lse, dq, dk, dv = row_attention_fwd_bwd(f32(q), f32(k), f32(v), f32(dout), torch.from_numpy(allowed))
    assert np.isposinf(lse.numpy()[:, 11]).all() and np.isposinf(w_lse[:, 11]).all()
    fin = np.isfinite(w_lse)
    assert np.abs(lse.numpy()[fin] - w_lse[fin]).max() <= 1e-5
    for got, want in ((out, w_out), (dq, w_dq), (dk, w_dk), (dv, w_dv)):
        assert np.abs(got.numpy() - want).max() <= 2e-5 * max(1.0, np.abs(want).max())
