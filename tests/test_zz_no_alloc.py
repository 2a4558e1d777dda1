"""dcp_attn_bwd_static (the backward with its scratch inside the library) against dcp_attn_bwd
(caller workspace), both called through the C ABI with raw device pointers: the same bits in dQ,
dK and dV, on two calls in a row, the second with a smaller input (the scratch keeps the first
call's contents)."""

import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _problem(gpu, n_rows, block_size, n_heads_q, n_heads_kv, head_dim, kv_blocks_per_row, seed):
    """A paged causal problem laid out by hand: row b attends its first b % kv_blocks + 1 kv blocks,
    the last of them causally; the last query row of every block is padding."""
    g = torch.Generator().manual_seed(seed)
    bs = block_size
    n_kv_slots = n_rows * kv_blocks_per_row
    dt = torch.bfloat16
    rnd = lambda *shape: (torch.randn(*shape, generator=g) * 0.5).to(dt).to(gpu)
    q, out, dout = rnd(n_rows, bs, n_heads_q, head_dim), rnd(n_rows, bs, n_heads_q, head_dim), rnd(n_rows, bs, n_heads_q, head_dim)
    kv = rnd(n_kv_slots, bs, 2, n_heads_kv, head_dim)
    lse = (torch.rand(n_heads_q, n_rows, bs, generator=g) * 2 + 3).to(gpu)
    seqlens_q = torch.full((n_rows,), bs - 1, dtype=torch.int32)
    n_blocks = torch.tensor([b % kv_blocks_per_row + 1 for b in range(n_rows)], dtype=torch.int32)
    cu_q = torch.zeros(n_rows + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(seqlens_q, 0)
    cu_kv = torch.zeros(n_rows + 1, dtype=torch.int32)
    cu_kv[1:] = torch.cumsum(n_blocks * bs, 0)
    total_q = int(cu_q[-1])
    rng = torch.zeros(1, 2, total_q, dtype=torch.int32)
    for b in range(n_rows):
        first = (int(n_blocks[b]) - 1) * bs
        t = torch.arange(int(seqlens_q[b]), dtype=torch.int32)
        rng[0, 1, int(cu_q[b]):int(cu_q[b + 1])] = first + t + 1  # [0, first + t + 1)
    kv_table = torch.full((n_rows, kv_blocks_per_row), -1, dtype=torch.int32)
    dkv_table = torch.full((n_rows, kv_blocks_per_row), -1, dtype=torch.int32)
    perm = torch.randperm(n_kv_slots, generator=g).to(torch.int32)
    nxt = 0
    for b in range(n_rows):
        for j in range(int(n_blocks[b])):
            kv_table[b, j] = perm[(b * kv_blocks_per_row + j) % n_kv_slots]
            dkv_table[b, j] = nxt
            nxt += 1
    row_table = torch.arange(n_rows, dtype=torch.int32).reshape(n_rows, 1)
    dev = lambda t: t.to(gpu).contiguous()
    return dict(q=q, kv=kv, out=out, dout=dout, lse=lse, cu_q=dev(cu_q), cu_kv=dev(cu_kv), rng=dev(rng),
                q_table=dev(row_table), kv_table=dev(kv_table), dkv_table=dev(dkv_table), n_rows=n_rows, bs=bs,
                hq=n_heads_q, hkv=n_heads_kv, d=head_dim, max_kv=kv_blocks_per_row, total_q=total_q, n_dkv=nxt)


def _run(lib, pr, static):
    from dcp_amd import _lib

    gpu = pr["q"].device
    dq = torch.full_like(pr["q"], 7.0)
    dkv = torch.full((pr["n_dkv"], pr["bs"], 2, pr["hkv"], pr["d"]), 7.0, dtype=pr["q"].dtype, device=gpu)
    k, v = pr["kv"][:, :, 0], pr["kv"][:, :, 1]
    dk, dv = dkv[:, :, 0], dkv[:, :, 1]
    head = [pr["dout"].data_ptr(), pr["q"].data_ptr(), k.data_ptr(), v.data_ptr(), pr["out"].data_ptr(),
            pr["lse"].data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr()]
    tail = [pr["cu_q"].data_ptr(), pr["cu_kv"].data_ptr(), pr["rng"].data_ptr(), 1, pr["q_table"].data_ptr(),
            pr["kv_table"].data_ptr(), pr["q_table"].data_ptr(), pr["q_table"].data_ptr(), pr["dkv_table"].data_ptr(), 0,
            pr["n_rows"], pr["max_kv"], pr["total_q"], pr["bs"], pr["hq"], pr["hkv"], pr["d"],
            pr["kv"].stride(0), pr["kv"].stride(1), dkv.stride(0), dkv.stride(1), pr["n_rows"],
            float(pr["d"]) ** -0.5, 0, torch.cuda.current_stream().cuda_stream]
    if static:
        _lib.call("dcp_attn_bwd_static", *head, *tail)
    else:
        # the static entry point runs the two kernels that recompute: compare with the same backward,
        # whichever one the process has selected for its other calls
        before = lib.dcp_attn_bwd_select(0)
        try:
            need = lib.dcp_attn_bwd_workspace_bytes(pr["n_rows"], pr["total_q"], pr["bs"], pr["hq"], pr["d"])
            ws = torch.empty(need, dtype=torch.uint8, device=gpu)
            _lib.call("dcp_attn_bwd", *head, ws.data_ptr(), need, *tail)
        finally:
            lib.dcp_attn_bwd_select(before)
    torch.cuda.synchronize()
    return dq.view(torch.int16).cpu().numpy(), dkv.view(torch.int16).cpu().numpy()


def test_static_scratch_backward_equals_workspace_backward_twice_in_a_row(gpu):
    from dcp_amd import _lib

    lib = _lib.load()
    big = _problem(gpu, n_rows=24, block_size=256, n_heads_q=4, n_heads_kv=1, head_dim=128, kv_blocks_per_row=5, seed=1)
    small = _problem(gpu, n_rows=5, block_size=128, n_heads_q=2, n_heads_kv=2, head_dim=64, kv_blocks_per_row=3, seed=2)
    for pr in (big, small):  # the second call finds the first one's values in the scratch
        want_dq, want_dkv = _run(lib, pr, static=False)
        got_dq, got_dkv = _run(lib, pr, static=True)
        assert np.array_equal(got_dq, want_dq)
        assert np.array_equal(got_dkv, want_dkv)
        # something was computed: not all of dQ still holds the fill value
        assert (want_dq != torch.tensor(7.0, dtype=torch.bfloat16).view(torch.int16).item()).any()


def test_static_scratch_backward_recorded_into_a_graph(gpu):
    """The use the entry point is for: recorded into a HIP graph (after the set-up call, made outside
    the capture, has looked up the scratch address) and replayed twice with eager work and
    synchronisations in between; every replay gives the bits of dcp_attn_bwd."""
    from dcp_amd import _lib

    lib = _lib.load()
    assert lib.dcp_attn_bwd_static_scratch_bytes() == 32 << 20  # set-up: resolves the address on this device
    pr = _problem(gpu, n_rows=9, block_size=128, n_heads_q=4, n_heads_kv=2, head_dim=128, kv_blocks_per_row=4, seed=3)
    want_dq, want_dkv = _run(lib, pr, static=False)
    dq = torch.full_like(pr["q"], 7.0)
    dkv = torch.full((pr["n_dkv"], pr["bs"], 2, pr["hkv"], pr["d"]), 7.0, dtype=pr["q"].dtype, device=gpu)
    k, v = pr["kv"][:, :, 0], pr["kv"][:, :, 1]
    dk, dv = dkv[:, :, 0], dkv[:, :, 1]

    def call():
        _lib.call("dcp_attn_bwd_static", pr["dout"].data_ptr(), pr["q"].data_ptr(), k.data_ptr(), v.data_ptr(),
                  pr["out"].data_ptr(), pr["lse"].data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                  pr["cu_q"].data_ptr(), pr["cu_kv"].data_ptr(), pr["rng"].data_ptr(), 1, pr["q_table"].data_ptr(),
                  pr["kv_table"].data_ptr(), pr["q_table"].data_ptr(), pr["q_table"].data_ptr(),
                  pr["dkv_table"].data_ptr(), 0, pr["n_rows"], pr["max_kv"], pr["total_q"], pr["bs"], pr["hq"],
                  pr["hkv"], pr["d"], pr["kv"].stride(0), pr["kv"].stride(1), dkv.stride(0), dkv.stride(1),
                  pr["n_rows"], float(pr["d"]) ** -0.5, 0, torch.cuda.current_stream().cuda_stream)

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    torch.cuda.synchronize()
    for replay in range(2):
        dq.fill_(7.0)
        dkv.fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(dq.view(torch.int16).cpu().numpy(), want_dq), f"replay {replay}: dQ"
        assert np.array_equal(dkv.view(torch.int16).cpu().numpy(), want_dkv), f"replay {replay}: dK/dV"
        _run(lib, pr, static=False)  # the program's own eager work between the replays


def test_static_scratch_backward_rejects_sizes_beyond_its_scratch(gpu):
    from dcp_amd import _lib

    lib = _lib.load()
    cap = lib.dcp_attn_bwd_static_scratch_bytes()
    assert cap == 32 << 20
    total_q = 1 << 22  # 4 Mi queries x 8 heads x 2 tables x 4 bytes = 256 MiB of scratch
    assert lib.dcp_attn_bwd_workspace_bytes(4096, total_q, 1024, 8, 128) > cap
    with pytest.raises(AssertionError, match="built-in scratch"):
        _lib.call("dcp_attn_bwd_static", *([1] * 9), 1, 1, 1, 1, 1, 1, 1, 1, 1, 0, 4096, 4, total_q, 1024, 8, 8, 128,
                  1024, 8, 1024, 8, 4096, 1.0, 0, 0)
