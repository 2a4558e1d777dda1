"""GPU parity of the fused block operators against the CPU oracle, through the
C ABI.  Shapes and reference semantics follow the reference's own op tests
(tests/ops/test_copy.py, test_blockwise_sum.py, test_attn_update_out_lse.py);
block movement must be bit-exact."""

import numpy as np
import pytest
import torch

from oracle import dcp_oracle as oracle

pytestmark = pytest.mark.gpu

DTYPES = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


def _bits(t: torch.Tensor) -> np.ndarray:
    view = torch.int16 if t.element_size() == 2 else torch.int32
    return t.detach().view(view).cpu().numpy()


@pytest.mark.parametrize("name", ["bf16", "fp16", "fp32"])
def test_fused_copy_varlen_bit_exact(gpu, name):
    from dcp_amd.ops import fused_ops

    dtype = DTYPES[name]
    fn = getattr(fused_ops, f"fused_copy_{name}_varlen")
    rng = np.random.default_rng(0)
    g = torch.Generator().manual_seed(0)
    for block_size, n_blocks in zip([256 * 128, 512 * 128, 1024 * 128, 1000], [2, 3, 4, 5]):
        src = torch.randn(n_blocks * 2, block_size, generator=g).to(dtype).to(gpu)
        dst = torch.randn(n_blocks * 2, block_size, generator=g).to(dtype).to(gpu)
        expect = _bits(dst).copy()
        src_off = rng.choice(n_blocks * 2, n_blocks, replace=False)
        dst_off = rng.choice(n_blocks * 2, n_blocks, replace=False)
        n_elem = rng.integers(1, block_size + 1, n_blocks)
        n_elem[0] = block_size  # a full block
        n_elem[-1] = 1  # a single element
        src_bits = _bits(src)
        oracle.block_copy(src_bits.reshape(-1), src_off * block_size, expect.reshape(-1),
                          dst_off * block_size, n_elem)
        i64 = lambda v: torch.tensor(v, dtype=torch.int64, device=gpu)
        i32 = lambda v: torch.tensor(np.asarray(v), dtype=torch.int32, device=gpu)
        fn(i64([src.data_ptr()] * n_blocks), i32(src_off), i32([block_size] * n_blocks),
           i64([dst.data_ptr()] * n_blocks), i32(dst_off), i32([block_size] * n_blocks),
           i32(n_elem), block_size, 128)
        torch.cuda.synchronize()
        assert np.array_equal(_bits(dst), expect)


def test_fused_copy_full_blocks_and_unaligned(gpu):
    from dcp_amd.ops.fused_ops import fused_copy_bf16, fused_copy_bf16_varlen

    g = torch.Generator().manual_seed(1)
    src = torch.randn(6, 4096, generator=g).to(torch.bfloat16).to(gpu)
    dst = torch.zeros_like(src)
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device=gpu)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=gpu)
    fused_copy_bf16(i64([src.data_ptr()] * 3), i32([5, 0, 2]), i32([4096] * 3),
                    i64([dst.data_ptr()] * 3), i32([1, 3, 4]), i32([4096] * 3), 4096, 128)
    torch.cuda.synchronize()
    expect = torch.zeros_like(src)
    expect[[1, 3, 4]] = src[[5, 0, 2]]
    assert torch.equal(dst.view(torch.int16), expect.view(torch.int16))
    # source and destination misaligned by one element (2 bytes)
    dst.zero_()
    fused_copy_bf16_varlen(i64([src.data_ptr() + 2]), i32([0]), i32([1]), i64([dst.data_ptr() + 6]),
                           i32([0]), i32([1]), i32([777]), 4096, 128)
    torch.cuda.synchronize()
    flat_s, flat_d = src.reshape(-1), dst.reshape(-1)
    assert torch.equal(flat_d[3:780].view(torch.int16), flat_s[1:778].view(torch.int16))
    assert flat_d[:3].abs().sum() == 0 and flat_d[780:].abs().sum() == 0


def test_fused_copy_dkv_bit_exact(gpu):
    from dcp_amd.ops.fused_ops import fused_copy_bf16_varlen_dkv

    g = torch.Generator().manual_seed(2)
    max_tokens, per_token = 256, 2 * 1 * 128
    src = torch.randn(5, max_tokens, per_token, generator=g).to(torch.bfloat16).to(gpu)
    dst = torch.randn(7, max_tokens, per_token, generator=g).to(torch.bfloat16).to(gpu)
    expect = dst.clone()
    n_tokens = [256, 1, 100, 0, 255]
    dst_idx = [6, 0, 3, 2, 5]
    for s, (d, n) in enumerate(zip(dst_idx, n_tokens)):
        expect[d, :n] = src[s, :n]
    fused_copy_bf16_varlen_dkv(
        torch.tensor([src[s].data_ptr() for s in range(5)], dtype=torch.int64, device=gpu),
        torch.tensor([dst[d].data_ptr() for d in dst_idx], dtype=torch.int64, device=gpu),
        torch.tensor(n_tokens, dtype=torch.int32, device=gpu), max_tokens, per_token, 128)
    torch.cuda.synchronize()
    assert torch.equal(dst.view(torch.int16), expect.view(torch.int16))


@pytest.mark.parametrize("heads", [1, 4, 5])
def test_fused_copy_lse_bit_exact(gpu, heads):
    from dcp_amd.ops.fused_ops import fused_copy_fp32_varlen_lse

    g = torch.Generator().manual_seed(3)
    bs, n_slots = 256, 6
    n_tokens = [256, 17, 200, 1]
    total = sum(n_tokens)
    src = torch.randn(heads, total, generator=g).to(gpu)
    dst = torch.randn(heads, n_slots, bs, generator=g).to(gpu)
    expect = dst.clone()
    offs = np.concatenate(([0], np.cumsum(n_tokens)))[:-1]
    slots = [4, 0, 5, 2]
    for o, s, n in zip(offs, slots, n_tokens):
        expect[:, s, :n] = src[:, o : o + n]
    k = len(n_tokens)
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device=gpu)
    i32 = lambda v: torch.tensor(np.asarray(v), dtype=torch.int32, device=gpu)
    fused_copy_fp32_varlen_lse(i64([src.data_ptr()] * k), i32(offs), i32([total] * k),
                               i64([dst.data_ptr()] * k), i32([s * bs for s in slots]),
                               i32([n_slots * bs] * k), i32(n_tokens), heads, bs, 128)
    torch.cuda.synchronize()
    assert torch.equal(dst.view(torch.int32), expect.view(torch.int32))


def _merge_case(gpu, dtype, n_src_per_op, n_head, head_dim, block_size, seed, inf_frac=0.0,
                unpadded=True, nan_frac=0.0, min_width=1, raw=None):
    from dcp_amd.ops.fused_ops import flash_attn_update_out_lse

    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    n_ops = len(n_src_per_op)
    n_src_blocks = sum(n_src_per_op) + 3
    n_tokens = rng.integers(1, block_size + 1, n_ops)
    n_tokens[0] = block_size
    src_out = torch.randn(n_src_blocks, block_size, n_head, head_dim, generator=g).to(dtype)
    src_lse = (torch.rand(n_head, n_src_blocks, block_size, generator=g) * 10 - 5)
    if inf_frac > 0:
        u = torch.rand(src_lse.shape, generator=g)
        src_lse[u < inf_frac / 2] = float("inf")
        src_lse[(u >= inf_frac / 2) & (u < inf_frac)] = float("-inf")
    if nan_frac > 0:
        src_lse[torch.rand(src_lse.shape, generator=g) < nan_frac] = float("nan")
    blocks = rng.permutation(n_src_blocks)[: sum(n_src_per_op)]
    width = max(min_width, 1 << (max(n_src_per_op) - 1).bit_length())
    table, c = [], 0
    for n in n_src_per_op:
        table.append(list(blocks[c : c + n]) + [-1] * (width - n))
        c += n
    if unpadded:
        total = int(n_tokens.sum())
        dst_offsets = np.concatenate(([0], np.cumsum(n_tokens)))[:-1]
        dst_out = torch.zeros(total, n_head, head_dim, dtype=dtype)
        dst_lse = torch.zeros(n_head, total)
        dst_head_stride = total
    else:  # fold in place into the first source of every op
        dst_offsets = np.array([row[0] * block_size for row in table])
        dst_out, dst_lse = src_out, src_lse
        dst_head_stride = n_src_blocks * block_size
    # oracle
    exp_out, exp_lse = [], []
    for op in range(n_ops):
        n = n_tokens[op]
        idx = table[op][: n_src_per_op[op]]
        o, l = oracle.merge_out_lse(src_out[idx, :n].float().numpy(), src_lse[:, idx, :n].permute(1, 0, 2).numpy())
        exp_out.append(o)
        exp_lse.append(l)
    d_src_out, d_src_lse = src_out.to(gpu), src_lse.to(gpu)
    if unpadded:
        d_dst_out, d_dst_lse = dst_out.to(gpu), dst_lse.to(gpu)
    else:
        d_dst_out, d_dst_lse = d_src_out, d_src_lse
    i32 = lambda v: torch.tensor(np.asarray(v), dtype=torch.int32, device=gpu)
    flash_attn_update_out_lse(
        d_src_out, d_dst_out, d_src_lse, d_dst_lse, n_head, i32(table), i32(dst_offsets), i32(n_tokens),
        i32(n_src_per_op), block_size, block_size * n_head * head_dim, n_head * head_dim, block_size, 1,
        n_src_blocks * block_size, dst_head_stride, head_dim, width, 64)
    torch.cuda.synchronize()
    if raw is not None:  # the caller compares bit patterns between launches
        raw.append((d_dst_out.cpu(), d_dst_lse.cpu()))
    got_out = d_dst_out.float().cpu().numpy().reshape(-1, n_head, head_dim)
    got_lse = d_dst_lse.cpu().numpy().reshape(n_head, -1)
    max_out = max_lse = 0.0
    for op in range(n_ops):
        n, off = n_tokens[op], dst_offsets[op]
        g_out, g_lse = got_out[off : off + n], got_lse[:, off : off + n]
        if nan_frac > 0:  # NaN exactly where the oracle has it; the rest by value
            assert np.array_equal(np.isnan(g_lse), np.isnan(exp_lse[op])), f"op {op}: NaN LSEs differ"
            assert np.array_equal(np.isnan(g_out), np.isnan(exp_out[op])), f"op {op}: NaN outputs differ"
            g_out, g_lse = np.nan_to_num(g_out, nan=0.0), np.nan_to_num(g_lse, nan=0.0)
            exp_out[op], exp_lse[op] = np.nan_to_num(exp_out[op], nan=0.0), np.nan_to_num(exp_lse[op], nan=0.0)
        max_out = max(max_out, np.abs(g_out - exp_out[op]).max())
        max_lse = max(max_lse, np.abs(g_lse - exp_lse[op]).max())
    return max_out, max_lse


@pytest.mark.parametrize("name,tol", [("fp32", 2e-5), ("bf16", 2e-2), ("fp16", 4e-3)])
def test_update_out_lse_reference_shapes(gpu, name, tol):
    # the reference's own case: 5 ops with [2,4,4,2,5] sources, 4 heads, D=64, bs=256
    err_out, err_lse = _merge_case(gpu, DTYPES[name], [2, 4, 4, 2, 5], 4, 64, 256, seed=0)
    assert err_out <= tol, err_out
    assert err_lse <= 1e-3, err_lse  # tolerance on fp32 LSE


def test_update_out_lse_nan_lse_is_a_source(gpu):
    """Only +-inf marks an empty source (reference fused_ops.py:123): a NaN LSE takes part in the
    merge and turns the merged LSE and output row of its (token, head) into NaN, infinite sources
    beside it or not.  (Ops with two or more sources: a single-source op is a bit copy.)"""
    err_out, err_lse = _merge_case(gpu, torch.bfloat16, [2, 3, 8, 2, 5], 5, 128, 128, seed=11, inf_frac=0.3,
                                   nan_frac=0.02)
    assert err_out <= 2e-2 and err_lse <= 1e-3, (err_out, err_lse)
    err_out, err_lse = _merge_case(gpu, torch.float32, [4, 2], 3, 64, 64, seed=12, nan_frac=0.05)
    assert err_out <= 2e-5 and err_lse <= 1e-3, (err_out, err_lse)


def test_update_out_lse_nonfinite_sources(gpu):
    err_out, err_lse = _merge_case(gpu, torch.bfloat16, [1, 3, 8, 2], 5, 128, 128, seed=1, inf_frac=0.5)
    assert err_out <= 2e-2 and err_lse <= 1e-3


def test_update_out_lse_in_place_fold(gpu):
    err_out, err_lse = _merge_case(gpu, torch.bfloat16, [2, 2, 2], 4, 128, 256, seed=2, unpadded=False)
    assert err_out <= 2e-2 and err_lse <= 1e-3


@pytest.mark.parametrize("name,tol", [("fp32", 2e-5), ("bf16", 2e-2), ("fp16", 4e-3)])
def test_update_out_lse_wide_rows(gpu, name, tol):
    """Token rows of 4 KiB and more (16 heads x 128, the executor's layout with large head blocks)
    take the row-streaming kernel: ragged token counts, ignored sources, 1 to 9 sources per op,
    unpadded destination and the in-place fold."""
    dtype = DTYPES[name]
    heads = 16 if name != "fp32" else 8
    err_out, err_lse = _merge_case(gpu, dtype, [2, 4, 1, 9, 3], heads, 128, 64, seed=5, inf_frac=0.3)
    assert err_out <= tol and err_lse <= 1e-3, (err_out, err_lse)
    err_out, err_lse = _merge_case(gpu, dtype, [2, 2, 3], heads, 128, 128, seed=6, unpadded=False)
    assert err_out <= tol and err_lse <= 1e-3, (err_out, err_lse)


@pytest.mark.parametrize("name,tol", [("fp32", 2e-5), ("bf16", 2e-2), ("fp16", 4e-3)])
def test_update_out_lse_wide_rows_of_few_sources(gpu, name, tol):
    """Launches whose ops have at most four sources take the one-wave kernel on wide rows (the
    lanes of a quad share the exponentials): ragged token counts, ignored and NaN sources, tables
    of width 4, 2 and 1, unpadded destination; and the same ops through a table padded to eight
    columns (the workgroup kernel with its weights in LDS) give the same bits."""
    dtype = DTYPES[name]
    heads = 16 if name != "fp32" else 8
    bits = lambda t: t.view(torch.int16 if t.element_size() == 2 else torch.int32)
    # (NaN LSEs only where every op has two sources or more: a single-source op copies bits)
    for sources, seed, nan_frac in (([2, 4, 3, 4], 21, 0.01), ([2, 4, 1, 3], 24, 0.0), ([2, 1, 2], 22, 0.0), ([1, 1], 23, 0.0)):
        raw = []
        for min_width in (1, 8):
            err_out, err_lse = _merge_case(gpu, dtype, sources, heads, 128, 64, seed=seed, inf_frac=0.3, nan_frac=nan_frac,
                                           min_width=min_width, raw=raw)
            assert err_out <= tol and err_lse <= 1e-3, (sources, min_width, err_out, err_lse)
        assert torch.equal(bits(raw[0][0]), bits(raw[1][0])) and torch.equal(bits(raw[0][1]), bits(raw[1][1])), sources


def test_update_out_lse_single_source_is_exact_copy(gpu):
    # one finite source: weight exp(l - l) = 1, so the merge is the scatter-back
    err_out, err_lse = _merge_case(gpu, torch.bfloat16, [1, 1, 1, 1], 4, 128, 512, seed=3)
    assert err_out == 0.0 and err_lse == 0.0


@pytest.mark.parametrize("name", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("width", [1, 4])
@pytest.mark.parametrize("heads,d", [(3, 64), (16, 128)])  # narrow rows / rows wide enough for the row-streaming merge
def test_single_source_merge_and_sum_copy_bit_patterns(gpu, name, width, heads, d):
    """Ops with one source are the scatter-back of finished blocks: bit for bit the source,
    negative zeros and NaN payloads included (compared as integers, not as floats), also when
    the launch's table is wide enough for more sources; a source whose LSE is infinite gives
    zeros and LSE -1."""
    from dcp_amd.ops.fused_ops import flash_attn_update_out_lse, fused_blockwise_sum

    dtype = DTYPES[name]
    ibits = torch.int32 if dtype == torch.float32 else torch.int16
    g = torch.Generator().manual_seed(9)
    bs, n_blocks = 128, 5
    src = torch.randn(n_blocks, bs, heads, d, generator=g).to(dtype)
    flat = src.view(ibits).reshape(-1)
    sign = torch.tensor(-0.0, dtype=dtype).view(ibits)  # the sign bit alone = -0.0
    nan = torch.tensor(float("nan"), dtype=dtype).view(ibits) | 5  # a NaN with a payload
    flat[::7] = sign
    flat[3::11] = nan
    lse = torch.randn(heads, n_blocks, bs, generator=g)
    lse.view(torch.int32).reshape(-1)[::13] |= -2147483648  # some negative LSEs, sign set by bit
    lse[1, 2, 5] = float("inf")
    lse[2, 4, 7] = float("-inf")
    n_tok = [bs, 1, 77]
    blocks = [4, 0, 2]
    offs = [0, bs, bs + 1]
    total = sum(n_tok)
    i32 = lambda v: torch.tensor(np.asarray(v), dtype=torch.int32, device=gpu)
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device=gpu)
    table = [[b] + [-1] * (width - 1) for b in blocks]
    d_src, d_lse = src.to(gpu), lse.to(gpu)
    dst_out = torch.ones(total, heads, d, dtype=dtype, device=gpu)
    dst_lse = torch.ones(heads, total, device=gpu)
    flash_attn_update_out_lse(d_src, dst_out, d_lse, dst_lse, heads, i32(table), i32(offs), i32(n_tok), i32([1] * 3), bs,
                              bs * heads * d, heads * d, bs, 1, n_blocks * bs, total, d, width, 64)
    torch.cuda.synchronize()
    for b, o, n in zip(blocks, offs, n_tok):
        want_out, want_lse = src[b, :n].clone(), lse[:, b, :n].clone()
        dead = ~torch.isfinite(want_lse)  # [heads, n]
        want_out[dead.T] = 0.0
        want_lse[dead] = -1.0
        assert torch.equal(dst_out[o : o + n].cpu().view(ibits), want_out.view(ibits))
        assert torch.equal(dst_lse[:, o : o + n].cpu().view(torch.int32), want_lse.view(torch.int32))
    # the block sum with one source per sum
    numel = bs * heads * d
    dst = torch.ones(n_blocks, bs, heads, d, dtype=dtype, device=gpu)
    dst_idx = [1, 3, 0]
    fused_blockwise_sum(i64([d_src.data_ptr()] * 3), i32(table), i32([numel] * 3), i32([1] * 3), i64([dst.data_ptr()] * 3),
                        i32(dst_idx), i32([numel] * 3), i32([n * heads * d for n in n_tok]), dtype, width, numel, 128)
    torch.cuda.synchronize()
    for b, di, n in zip(blocks, dst_idx, n_tok):
        assert torch.equal(dst[di, :n].cpu().view(ibits), src[b, :n].view(ibits))
        assert bool((dst[di, n:] == 1).all())


def test_update_out_lse_rejects_too_many_sources(gpu):
    from dcp_amd.ops.fused_ops import flash_attn_update_out_lse

    z = torch.zeros(1, device=gpu)
    zi = torch.zeros(1, dtype=torch.int32, device=gpu)
    with pytest.raises(AssertionError):
        flash_attn_update_out_lse(z, z, z, z, 1, zi, zi, zi, zi, 64, 64, 1, 64, 1, 64, 64, 1, 128, 64)


@pytest.mark.parametrize("name,tol", [("bf16", 2e-2), ("fp16", 1e-2), ("fp32", 1e-5)])
def test_fused_blockwise_sum(gpu, name, tol):
    from dcp_amd.ops.fused_ops import fused_blockwise_sum

    dtype = DTYPES[name]
    g = torch.Generator().manual_seed(4)
    rng = np.random.default_rng(4)
    block_size, n_blocks, n_heads, head_dim, max_ops, n_reds = 512, 64, 2, 64, 8, 8
    src = torch.randn(n_blocks, block_size, n_heads, head_dim, generator=g).to(dtype).to(gpu)
    dst = torch.randn(n_blocks, block_size, n_heads, head_dim, generator=g).to(dtype).to(gpu)
    before = dst.clone()
    ops_per_red = rng.integers(1, max_ops + 1, n_reds)
    ops_per_red[0] = 1
    red_blocks = rng.choice(n_blocks, int(ops_per_red.sum()), replace=False)
    table, lists, c = [], [], 0
    for n in ops_per_red:
        lists.append(list(red_blocks[c : c + n]))
        table.append(lists[-1] + [-1] * (max_ops - n))
        c += n
    n_tok = rng.integers(1, block_size + 1, n_reds)
    n_elems = n_tok * n_heads * head_dim
    dst_idx = rng.choice(n_blocks, n_reds, replace=False)
    expect = dst.float().cpu().numpy()
    src_np = src.float().cpu().numpy()
    for lst, d, n in zip(lists, dst_idx, n_tok):
        expect[d, :n] = oracle.round_to(oracle.blockwise_sum([src_np[b, :n] for b in lst]), name)
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device=gpu)
    i32 = lambda v: torch.tensor(np.asarray(v), dtype=torch.int32, device=gpu)
    numel = block_size * n_heads * head_dim
    fused_blockwise_sum(i64([src.data_ptr()] * n_reds), i32(table), i32([numel] * n_reds), i32(ops_per_red),
                        i64([dst.data_ptr()] * n_reds), i32(dst_idx), i32([numel] * n_reds), i32(n_elems),
                        dtype, max_ops, numel, 128)
    torch.cuda.synchronize()
    got = dst.float().cpu().numpy()
    assert np.abs(got - expect).max() <= tol
    # single-source sums are copies, and untouched blocks stay as they were: compared as integers
    ibits = torch.int32 if dtype == torch.float32 else torch.int16
    d0, n0 = int(dst_idx[0]), int(n_tok[0])
    assert torch.equal(dst[d0, :n0].view(ibits), src[int(lists[0][0]), :n0].view(ibits))
    untouched = sorted(set(range(n_blocks)) - set(dst_idx.tolist()))
    assert torch.equal(dst[untouched].view(ibits).cpu(), before[untouched].view(ibits).cpu())


def test_fused_blockwise_sum_rejects_dtype(gpu):
    from dcp_amd.ops.fused_ops import fused_blockwise_sum

    z64 = torch.zeros(1, dtype=torch.int64, device=gpu)
    z32 = torch.zeros(1, dtype=torch.int32, device=gpu)
    with pytest.raises(ValueError):
        fused_blockwise_sum(z64, z32.reshape(1, 1), z32, z32, z64, z32, z32, z32, torch.int8, 1, 128, 128)


def test_roofline_probes(gpu):
    """The benchmark's two measurement-only kernels (bench_probes.hip, a library of their own):
    the streaming probe's output is the exact (wrap-around) 32-bit sum of its streams, the MFMA
    probe reports its FLOP count and clocks, and both reject what they do not support."""
    import ctypes

    from bench import call_probe

    stream = torch.cuda.current_stream().cuda_stream
    per_stream = 8192 * 64
    rng = np.random.default_rng(3)
    src = torch.from_numpy(rng.integers(-2**31, 2**31 - 1, size=4 * per_stream // 4, dtype=np.int64).astype(np.int32)).to(gpu)
    dst = torch.zeros(per_stream // 4, dtype=torch.int32, device=gpu)
    for n in (1, 2, 4):
        call_probe("bench_hbm_stream_probe", src.data_ptr(), dst.data_ptr(), n, per_stream, None, 0, stream)
        torch.cuda.synchronize()
        want = src.reshape(4, -1)[:n].to(torch.int64).sum(0).to(torch.int32)  # wraps like the 32-bit adds
        assert torch.equal(dst, want), n
    # streams made of 2 KiB blocks picked from `src` through a table: block b of stream s = table[b][s]
    block_bytes, n_blocks = 2048, per_stream // 2048
    for n in (1, 4):
        table = torch.from_numpy(rng.permutation(4 * n_blocks)[: n * n_blocks].reshape(n_blocks, n).astype(np.int32)).to(gpu)
        call_probe("bench_hbm_stream_probe", src.data_ptr(), dst.data_ptr(), n, per_stream, table.data_ptr(), block_bytes, stream)
        torch.cuda.synchronize()
        blocks = src.reshape(4 * n_blocks, block_bytes // 4).to(torch.int64)
        want = blocks[table.long()].sum(1).to(torch.int32).reshape(-1)
        assert torch.equal(dst, want), n
    with pytest.raises(ValueError):
        call_probe("bench_hbm_stream_probe", src.data_ptr(), dst.data_ptr(), 3, per_stream, None, 0, stream)
    with pytest.raises(AssertionError):
        call_probe("bench_hbm_stream_probe", src.data_ptr(), dst.data_ptr(), 1, 100, None, 0, stream)
    with pytest.raises(AssertionError):
        call_probe("bench_hbm_stream_probe", src.data_ptr(), dst.data_ptr(), 1, per_stream, dst.data_ptr(), 3000, stream)

    n_wg, iters = 8, 10
    ops = torch.full((n_wg * 256 * 16 * 8,), 0.5, device=gpu, dtype=torch.bfloat16)
    out = torch.zeros(2 + n_wg * 256, device=gpu)
    flop = ctypes.c_double()
    call_probe("bench_mfma_probe", ops.data_ptr(), out.data_ptr(), n_wg, iters, 0, ctypes.byref(flop), stream)
    torch.cuda.synchronize()
    assert flop.value == n_wg * 4 * iters * 32 * 2.0 * 32 * 32 * 16
    assert out[0].item() > 0 and out[1].item() > 0
    # every accumulator element of the probe is iters * 32 / 4 products of 16 terms 0.5 * 0.5
    assert torch.allclose(out[2:], torch.full_like(out[2:], 64 * (iters * 32 / 4) * 16 * 0.25))
    with pytest.raises(ValueError):
        call_probe("bench_mfma_probe", ops.data_ptr(), out.data_ptr(), n_wg, iters, 2, ctypes.byref(flop), stream)
