"""BASELINE-size runs on the GPU, checked through size-independent properties
and seeded samples of the oracle (the full oracle would take hours):

* config 2 (Llama-3-8B shape, 65536 tokens, causal, bs 1024, GQA 32/8):
  sampled (sequence, head) parity against dense fp64 attention, exact
  linearity of the backward in dO, bit-reproducibility, HIP-graph replays; the same schedule
  placed on four devices whose executors share the GPU reproduces the one-device result;
* config 3 (lambda mask, sink 64 + window 4096) at 32768 tokens: sampled parity against the
  oracle; at the full 131072 tokens and config 4 (shared prefix, 98304 tokens, 40/8 heads,
  bs 512, every row's kv blocks in two partials) a whole (sequence, kv head) group is checked
  against dense fp64 attention written in plain torch on the GPU (out, LSE, dQ, dK, dV): the
  numpy oracle would need minutes per sample at these lengths;
* config 5 (262144 x 32 x 128 bf16 block movement): gather -> inverse scatter is
  the identity bit for bit, padding rows stay untouched, and the 4-way merge is
  invariant under a permutation of its sources.
"""

import numpy as np
import pytest
import torch

import bench
from oracle import dcp_oracle as oracle
from tests.plan_cases import max_abs_err, scaled_err

pytestmark = pytest.mark.gpu


def _run(wl, seed=0, graph=False):
    from dcp_amd.core.instructions import BufferType
    from dcp_amd.runtime.flash_attention.executor import get_executor

    fw, bw, layout, mask, pairs = bench.build(wl)
    ex_f, ex_b = bench.make_executors(wl, fw, bw, seed=seed)
    ex_f.execute(fw, True)
    ex_b.execute(bw, False)
    torch.cuda.synchronize()
    B = BufferType
    t = {k: ex_f.buffers[k] for k in (B.LOCAL_Q, B.LOCAL_KV, B.LOCAL_OUT, B.LOCAL_LSE)}
    t.update({k: ex_b.buffers[k] for k in (B.LOCAL_dOUT, B.LOCAL_dQ, B.LOCAL_dKV)})
    return fw, bw, layout, mask, ex_f, ex_b, t


def _sample_check(wl, layout, mask, t, samples):
    """Dense fp64 attention for a few (sequence, kv head) groups."""
    from dcp_amd.core.instructions import BufferType as B

    hb = wl["head_block"]
    group = wl["n_heads"] // wl["n_groups"]
    seq_off = np.concatenate(([0], np.cumsum(wl["seqlens"])))
    total = int(seq_off[-1])
    worst = dict(out=0.0, lse=0.0, dq=0.0, dkv=0.0)
    for s, kvh in samples:
        L = wl["seqlens"][s]
        # LOCAL order is (head block, sequence, block): a sequence is contiguous inside a head block
        hblk = kvh * group // hb  # first q head block of this kv head's group
        n_hblk = max(1, group // hb)
        sl_kv = slice(kvh * total + int(seq_off[s]), kvh * total + int(seq_off[s]) + L)
        kv = t[B.LOCAL_KV][sl_kv].float().cpu().numpy()  # [L, 2, 1, D]
        qs, douts, outs, lses, dqs = [], [], [], [], []
        for j in range(n_hblk):
            sl = slice((hblk + j) * total + int(seq_off[s]), (hblk + j) * total + int(seq_off[s]) + L)
            qs.append(t[B.LOCAL_Q][sl].float().cpu().numpy())
            douts.append(t[B.LOCAL_dOUT][sl].float().cpu().numpy())
            outs.append(t[B.LOCAL_OUT][sl].float().cpu().numpy())
            lses.append(t[B.LOCAL_LSE][:, sl].cpu().numpy())
            dqs.append(t[B.LOCAL_dQ][sl].float().cpu().numpy())
        q, dout = np.concatenate(qs, axis=1), np.concatenate(douts, axis=1)
        m = mask[int(seq_off[s]) : int(seq_off[s]) + L].numpy()
        r_out, r_lse, r_dq, r_dkv = oracle.dense_reference(q, kv, m, [L], dout=dout, dtype=np.float64)
        # max-abs for out, LSE and dQ; dK/dV (magnitudes far above 1 at these lengths) scaled by max(1, |ref|)
        worst["out"] = max(worst["out"], max_abs_err(np.concatenate(outs, axis=1), r_out))
        worst["lse"] = max(worst["lse"], max_abs_err(np.concatenate(lses, axis=0), r_lse))
        worst["dq"] = max(worst["dq"], max_abs_err(np.concatenate(dqs, axis=1), r_dq))
        worst["dkv"] = max(worst["dkv"], scaled_err(t[B.LOCAL_dKV][sl_kv].float().cpu().numpy(), r_dkv))
    return worst


def _dense_check_gpu(wl, mask, t, s, kvh, chunk=4096):
    """Dense masked attention of sequence ``s`` for the q heads of kv head ``kvh``, forward and
    backward, in fp64 with torch matmuls on the GPU, row chunk by row chunk; returns the worst
    deviations of the kernels' results.  Independent of the kernels under test and of the numpy
    oracle (whose ``dense_reference`` it restates; both are pinned against each other on a short
    sequence in ``test_dense_gpu_checker_agrees_with_oracle``)."""
    from dcp_amd.core.instructions import BufferType as B

    hb, d = wl["head_block"], wl["head_dim"]
    group = wl["n_heads"] // wl["n_groups"]
    seq_off = np.concatenate(([0], np.cumsum(wl["seqlens"])))
    total, L, o0 = int(seq_off[-1]), wl["seqlens"][s], int(seq_off[s])
    scale = d ** -0.5
    kv = t[B.LOCAL_KV][kvh * total + o0 : kvh * total + o0 + L].double()  # [L, 2, 1, D]
    k, v = kv[:, 0, 0], kv[:, 1, 0]
    m = mask[o0 : o0 + L].to("cuda", torch.int64)
    if m.dim() == 2:
        m = torch.stack([m, torch.zeros_like(m)], dim=1)
    cols = torch.arange(L, device="cuda")[None, :]
    dk = torch.zeros(L, d, dtype=torch.float64, device="cuda")
    dv = torch.zeros_like(dk)
    worst = dict(out=0.0, lse=0.0, dq=0.0, dkv=0.0)
    rel = lambda g, r: float(((g - r).abs() / r.abs().clamp(min=1.0)).max())  # dK/dV only
    mabs = lambda g, r: float((g - r).abs().max())
    hblk, n_hblk = kvh * group // hb, max(1, group // hb)
    for j in range(n_hblk):
        sl = slice((hblk + j) * total + o0, (hblk + j) * total + o0 + L)
        for hh in range(hb):
            q, do = t[B.LOCAL_Q][sl, hh].double(), t[B.LOCAL_dOUT][sl, hh].double()
            for r0 in range(0, L, chunk):
                r1 = min(r0 + chunk, L)
                mm = m[r0:r1]
                ok = ((cols >= mm[:, 0, 0:1]) & (cols < mm[:, 0, 1:2])) | ((cols >= mm[:, 1, 0:1]) & (cols < mm[:, 1, 1:2]))
                sc = (q[r0:r1] @ k.T) * scale
                sc.masked_fill_(~ok, float("-inf"))
                lse = torch.logsumexp(sc, dim=1)
                pr = torch.exp(sc - lse[:, None])
                out = pr @ v
                dp = do[r0:r1] @ v.T
                ds = pr * (dp - (do[r0:r1] * out).sum(1, keepdim=True))
                dq = (ds @ k) * scale
                dk += (ds.T @ q[r0:r1]) * scale
                dv += pr.T @ do[r0:r1]
                rs = slice(sl.start + r0, sl.start + r1)
                worst["out"] = max(worst["out"], mabs(t[B.LOCAL_OUT][rs, hh].double(), out))
                worst["lse"] = max(worst["lse"], float((t[B.LOCAL_LSE][hh, rs].double() - lse).abs().max()))
                worst["dq"] = max(worst["dq"], mabs(t[B.LOCAL_dQ][rs, hh].double(), dq))
    got = t[B.LOCAL_dKV][kvh * total + o0 : kvh * total + o0 + L].double()
    worst["dkv"] = max(rel(got[:, 0, 0], dk), rel(got[:, 1, 0], dv))
    return worst


def test_dense_gpu_checker_agrees_with_oracle(gpu):
    """The torch fp64 checker and the numpy oracle see the same deviations on a short sequence."""
    wl = bench.workload("smoke")
    fw, bw, layout, mask, ex_f, ex_b, t = _run(wl, seed=3)
    a = _sample_check(wl, layout, mask, t, [(0, 1)])
    b = _dense_check_gpu(wl, mask, t, 0, 1, chunk=256)
    for key in a:
        assert abs(a[key] - b[key]) <= 1e-6 + 1e-3 * max(a[key], b[key]), (key, a, b)
        assert b[key] <= (1e-3 if key == "lse" else 2e-2), b


def test_config2_llama_shape_sampled_parity_linearity_determinism(gpu):
    from dcp_amd.core.instructions import BufferType as B

    wl = bench.workload("llama3_8b_causal_64k")
    fw, bw, layout, mask, ex_f, ex_b, t = _run(wl)
    order = np.argsort(wl["seqlens"])
    samples = [(int(order[0]), 0), (int(order[len(order) // 2]), 5), (int(order[3]), 7)]  # short and medium sequences
    worst = _sample_check(wl, layout, mask, t, samples)
    assert worst["out"] <= 2e-2 and worst["lse"] <= 1e-3 and worst["dq"] <= 2e-2 and worst["dkv"] <= 2e-2, worst
    assert bool(torch.isfinite(t[B.LOCAL_LSE]).all()) and bool(torch.isfinite(t[B.LOCAL_dKV].float()).all())

    # bit-reproducible: no atomics anywhere on the path
    dq0, dkv0, out0 = t[B.LOCAL_dQ].clone(), t[B.LOCAL_dKV].clone(), t[B.LOCAL_OUT].clone()
    ex_f.execute(fw, True)
    ex_b.execute(bw, False)
    torch.cuda.synchronize()
    assert torch.equal(t[B.LOCAL_OUT], out0) and torch.equal(t[B.LOCAL_dQ], dq0) and torch.equal(t[B.LOCAL_dKV], dkv0)

    # the backward is linear in dO, and scaling by 2 commutes with every rounding
    t[B.LOCAL_dOUT].mul_(2)
    ex_b.execute(bw, False)
    torch.cuda.synchronize()
    assert torch.equal(t[B.LOCAL_dQ], dq0 * 2) and torch.equal(t[B.LOCAL_dKV], dkv0 * 2)


def test_config2_four_stage_round_robin_variant(gpu):
    """The same 65536-token schedule with every row's kv blocks dealt round-robin to four stages:
    four partial outputs per row merged at the end (N-way merge with up to four sources), dQ summed
    over the stages' versions, dK/dV replicas per (row, kv block) as before."""
    from dcp_amd.core.instructions import AttnReductionInstr, BufferType as B, SumInstr

    wl = dict(bench.workload("llama3_8b_causal_64k"), plan_kwargs=dict(n_kv_groups=4, kv_split="round_robin"))
    fw, bw, layout, mask, ex_f, ex_b, t = _run(wl, seed=6)
    reds = [i for i in fw.instructions if isinstance(i, AttnReductionInstr)]
    assert max(len(op.src_buffers) for r in reds for op in r.ops) == 4
    sums = [i for i in bw.instructions if isinstance(i, SumInstr)]
    assert max(len(op.src_buffers) for r in sums for op in r.ops if op.dst_buffer.buffer_type == B.BUFFER_dQ) == 4
    order = np.argsort(wl["seqlens"])
    worst = _sample_check(wl, layout, mask, t, [(int(order[1]), 2)])
    assert worst["out"] <= 2e-2 and worst["lse"] <= 1e-3 and worst["dq"] <= 2e-2 and worst["dkv"] <= 2e-2, worst
    s = int(np.argmax(wl["seqlens"]))  # the longest sequence: rows with the most kv blocks per stage
    worst = _dense_check_gpu(wl, mask, t, s, kvh=4)
    assert worst["out"] <= 2e-2 and worst["lse"] <= 1e-3 and worst["dq"] <= 2e-2 and worst["dkv"] <= 2e-2, worst


def test_config2_hip_graph_replays_match_eager(gpu):
    from dcp_amd.core.instructions import BufferType as B
    from dcp_amd.runtime.flash_attention.executor import get_executor

    wl = bench.workload("smoke")
    fw, bw, layout, mask, pairs = bench.build(wl)
    ex = get_executor(wl["head_block"], wl["head_dim"], None, fw_exec_plan=fw, bw_exec_plan=bw, use_cudagraph=True)
    ex.prepare(forward=True)
    g = torch.Generator(device="cuda").manual_seed(1)
    q = torch.randn(ex.buffers[B.LOCAL_Q].shape, generator=g, device="cuda").to(torch.bfloat16)
    kv = torch.randn(ex.buffers[B.LOCAL_KV].shape, generator=g, device="cuda").to(torch.bfloat16)
    eager_out, eager_lse = ex.forward(q, kv)
    ex.capture_cudagraph()
    assert ex.cuda_graph is not None
    for i in range(3):  # replays with eager work and synchronisation in between
        ex.buffers[B.LOCAL_OUT].zero_()
        ex.buffers[B.BUFFER_OUT].fill_(float(i))
        torch.cuda.synchronize()
        out, lse = ex.forward(q, kv)
        torch.cuda.synchronize()
        assert torch.equal(out, eager_out) and torch.equal(lse, eager_lse), i
    # new inputs through the same graph
    q2 = q * 0.5
    out2, _ = ex.forward(q2, kv)
    ex.cuda_graph = None
    ref2, _ = ex.forward(q2, kv)
    assert torch.equal(out2, ref2)


def test_config2_split_over_four_devices_matches_one_device(gpu):
    """The 65536-token schedule placed on four devices (their executors share the GPU and
    exchange Q/KV blocks, partial outputs and partial gradients over a LocalFabric) gives what one
    device owning every block gives, up to the extra roundings of partials that travel in bf16."""
    from dcp_amd.core.instructions import BufferType as B
    from dcp_amd.runtime.flash_attention.executor import get_executor
    from dcp_amd.runtime.flash_attention.fabric import LocalFabric, execute_together
    from dcp_amd.runtime.flash_attention.multi_device import build_multi_device_plans

    wl = bench.workload("llama3_8b_causal_64k")
    fw, bw, layout, mask, ex_f, ex_b, t = _run(wl)
    one = dict(q=layout.from_local_q(t[B.LOCAL_Q]), kv=layout.from_local_kv(t[B.LOCAL_KV]),
               out=layout.from_local_q(t[B.LOCAL_OUT]), lse=layout.from_local_lse(t[B.LOCAL_LSE]),
               dout=layout.from_local_q(t[B.LOCAL_dOUT]), dq=layout.from_local_q(t[B.LOCAL_dQ]),
               dkv=layout.from_local_kv(t[B.LOCAL_dKV]))
    del ex_f, ex_b, t
    torch.cuda.empty_cache()
    fws, bws, lays = build_multi_device_plans(1, 4, wl["seqlens"], wl["block_size"], wl["n_heads"], wl["n_groups"],
                                              wl["head_dim"], wl["head_block"], mask, dtype=torch.bfloat16)
    fabric = LocalFabric(1, 4)
    exs = [get_executor(wl["head_block"], wl["head_dim"], None, fw_exec_plan=f, bw_exec_plan=b, fabric=fabric)
           for f, b in zip(fws, bws)]
    print("four devices: forward", flush=True)
    for ex, lay in zip(exs, lays):
        ex.prepare(forward=True)
        ex.init_forward_input(lay.to_local_q(one["q"]), lay.to_local_kv(one["kv"]))
    execute_together(exs, forward=True)
    torch.cuda.synchronize()
    outs = [ex.buffers[B.LOCAL_OUT].clone() for ex in exs]
    lses = [ex.buffers[B.LOCAL_LSE].clone() for ex in exs]
    out = sum(lay.from_local_q(x) for lay, x in zip(lays, outs))
    lse = sum(lay.from_local_lse(x) for lay, x in zip(lays, lses))
    assert float((out.float() - one["out"].float()).abs().max()) <= 2e-2
    assert float((lse - one["lse"]).abs().max()) <= 1e-3
    print("four devices: backward", flush=True)
    for ex, lay, o, l in zip(exs, lays, outs, lses):
        ex.switch_to_backward()
        ex.set_local_out_lse(o, l)
        ex.init_forward_input(lay.to_local_q(one["q"]), lay.to_local_kv(one["kv"]))
        ex.init_backward_input(lay.to_local_q(one["dout"]))
    execute_together(exs, forward=False)
    torch.cuda.synchronize()
    dq = sum(lay.from_local_q(ex.buffers[B.LOCAL_dQ]) for lay, ex in zip(lays, exs))
    dkv = sum(lay.from_local_kv(ex.buffers[B.LOCAL_dKV]) for lay, ex in zip(lays, exs))
    # two bf16 results against each other (here the partial gradients also travel in bf16): dQ max-abs,
    # dK/dV scaled by max(1, |want|) as everywhere
    e_dq = float((dq.float() - one["dq"].float()).abs().max())
    e_dkv = float(((dkv.float() - one["dkv"].float()).abs() / one["dkv"].float().abs().clamp(min=1.0)).max())
    print("four devices vs one: dq", e_dq, "dkv (scaled)", e_dkv, flush=True)
    assert e_dq <= 2e-2 and e_dkv <= 2e-2, (e_dq, e_dkv)


def test_config3_lambda_mask_sampled_parity(gpu):
    wl = bench.workload("lambda_128k")
    wl = dict(wl, seqlens=bench.lognormal_lengths(32768, 8192, 256, 16384, seed=1))
    fw, bw, layout, mask, ex_f, ex_b, t = _run(wl, seed=2)
    order = np.argsort(wl["seqlens"])
    samples = [(int(order[-1]) if wl["seqlens"][order[-1]] <= 9000 else int(order[len(order) // 2]), 3)]
    worst = _sample_check(wl, layout, mask, t, samples)
    assert worst["out"] <= 2e-2 and worst["lse"] <= 1e-3 and worst["dq"] <= 2e-2 and worst["dkv"] <= 2e-2, worst


def test_config3_lambda_mask_full_size_dense_check(gpu):
    wl = bench.workload("lambda_128k")
    assert sum(wl["seqlens"]) == 131072
    fw, bw, layout, mask, ex_f, ex_b, t = _run(wl, seed=4)
    s = int(np.argmax(wl["seqlens"]))  # the longest sequence: most skipped tiles, both ranges in play
    worst = _dense_check_gpu(wl, mask, t, s, kvh=6)
    assert worst["out"] <= 2e-2 and worst["lse"] <= 1e-3 and worst["dq"] <= 2e-2 and worst["dkv"] <= 2e-2, worst
    from dcp_amd.core.instructions import BufferType as B
    assert bool(torch.isfinite(t[B.LOCAL_LSE]).all()) and bool(torch.isfinite(t[B.LOCAL_dQ].float()).all())


def test_config4_shared_prefix_full_size_dense_check(gpu):
    from dcp_amd.core.instructions import AttnReductionInstr

    wl = bench.workload("shared_prefix_96k")
    assert sum(wl["seqlens"]) == 98304 and wl["n_heads"] == 40 and wl["head_block"] == 5
    fw, bw, layout, mask, ex_f, ex_b, t = _run(wl, seed=5)
    # the schedule really splits every row's kv blocks over partial outputs: the merge has work to do
    reds = [i for i in fw.instructions if isinstance(i, AttnReductionInstr)]
    assert reds and max(len(op.src_buffers) for r in reds for op in r.ops) >= 2
    s = int(np.argmin(wl["seqlens"]))
    worst = _dense_check_gpu(wl, mask, t, s, kvh=3)
    assert worst["out"] <= 2e-2 and worst["lse"] <= 1e-3 and worst["dq"] <= 2e-2 and worst["dkv"] <= 2e-2, worst
    # closed form of the pair count: p(p+1)/2 + sum_k (c_k p + c_k (c_k+1)/2) per sample
    from dcp_amd.runtime.flash_attention.utils import count_attended_pairs
    want = sum(i["prefix"] * (i["prefix"] + 1) // 2 + sum(c * i["prefix"] + c * (c + 1) // 2 for c in i["continuations"])
               for i in wl["mask_info"])
    assert count_attended_pairs(mask) == want


def test_config4_head_block_of_one(gpu):
    """Config 4 with one q head per head block (five head blocks per kv head): the dK/dV sum then
    adds the replicas of five q head blocks."""
    wl = dict(bench.workload("shared_prefix_96k"), head_block=1)
    fw, bw, layout, mask, ex_f, ex_b, t = _run(wl, seed=7)
    s = int(np.argmin(wl["seqlens"]))
    worst = _dense_check_gpu(wl, mask, t, s, kvh=5)
    assert worst["out"] <= 2e-2 and worst["lse"] <= 1e-3 and worst["dq"] <= 2e-2 and worst["dkv"] <= 2e-2, worst


def test_config5_one_head_blocks_round_trip(gpu):
    """The config 5 tensor moved as one-head blocks (head block size 1: 16384 blocks of 128 KiB, ragged):
    gather through a seeded permutation, inverse scatter, bit for bit."""
    from dcp_amd.ops.fused_ops import fused_copy_bf16_varlen

    tokens, heads, d, bs = 262144, 32, 128, 512
    n_blocks, numel = tokens // bs * heads, bs * d
    rng = np.random.default_rng(1)
    perm = rng.permutation(n_blocks)
    n_tok = rng.integers(1, bs + 1, n_blocks)
    g = torch.Generator(device="cuda").manual_seed(1)
    src = torch.randn(n_blocks, bs, d, device="cuda", generator=g).to(torch.bfloat16)  # [head block x block][token][d]
    packed, back = torch.full_like(src, 7.0), torch.zeros_like(src)
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device="cuda")
    i32 = lambda v: torch.tensor(np.ascontiguousarray(v), dtype=torch.int32, device="cuda")
    ident, stride, n_el = np.arange(n_blocks), i32([numel] * n_blocks), i32(n_tok * d)
    fused_copy_bf16_varlen(i64([src.data_ptr()] * n_blocks), i32(ident), stride, i64([packed.data_ptr()] * n_blocks),
                           i32(perm), stride, n_el, numel, 128)
    fused_copy_bf16_varlen(i64([packed.data_ptr()] * n_blocks), i32(perm), stride, i64([back.data_ptr()] * n_blocks),
                           i32(ident), stride, n_el, numel, 128)
    torch.cuda.synchronize()
    valid = torch.arange(bs, device="cuda")[None, :] < torch.tensor(n_tok, device="cuda")[:, None]
    s3, b3 = src.view(torch.int16), back.view(torch.int16)
    assert torch.equal(b3[valid], s3[valid]) and bool((b3[~valid] == 0).all())
    assert torch.equal(packed.view(torch.int16)[torch.tensor(perm, device="cuda")][valid], s3[valid])


def test_config5_block_movement_full_size(gpu):
    from dcp_amd.ops.fused_ops import flash_attn_update_out_lse, fused_copy_bf16_varlen

    tokens, heads, d, bs = 262144, 32, 128, 512
    n_blocks = tokens // bs
    numel = bs * heads * d
    rng = np.random.default_rng(0)
    perm = rng.permutation(n_blocks)
    n_tok = rng.integers(1, bs + 1, n_blocks)  # ragged blocks: only the first n tokens move
    n_tok[:8] = bs
    g = torch.Generator(device="cuda").manual_seed(0)
    src = torch.randn(tokens, heads, d, device="cuda", generator=g).to(torch.bfloat16)
    packed = torch.full_like(src, 7.0)
    back = torch.zeros_like(src)
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device="cuda")
    i32 = lambda v: torch.tensor(np.ascontiguousarray(v), dtype=torch.int32, device="cuda")
    ident, stride = np.arange(n_blocks), i32([numel] * n_blocks)
    n_el = i32(n_tok * heads * d)
    fused_copy_bf16_varlen(i64([src.data_ptr()] * n_blocks), i32(ident), stride, i64([packed.data_ptr()] * n_blocks),
                           i32(perm), stride, n_el, numel, 128)
    fused_copy_bf16_varlen(i64([packed.data_ptr()] * n_blocks), i32(perm), stride, i64([back.data_ptr()] * n_blocks),
                           i32(ident), stride, n_el, numel, 128)
    torch.cuda.synchronize()
    valid = (torch.arange(bs, device="cuda")[None, :] < torch.tensor(n_tok, device="cuda")[:, None]).reshape(-1)
    s3, b3, p3 = (x.view(torch.int16).reshape(tokens, -1) for x in (src, back, packed))
    assert torch.equal(b3[valid], s3[valid])  # gather then inverse scatter: identity, bit for bit
    assert bool((b3[~valid] == 0).all())  # rows past n_tokens are never written
    inv = np.argsort(perm)
    pad_rows = ~valid.reshape(n_blocks, bs)[torch.tensor(inv, device="cuda")].reshape(-1)
    seven = torch.tensor(7.0, dtype=torch.bfloat16).view(torch.int16).item()
    assert bool((p3[pad_rows] == seven).all())
    del packed, back

    # merge: permuting the sources of every op leaves the result unchanged up to rounding
    n_src = 4
    blocks = n_blocks  # all 262144 tokens: 4 x 2 GiB of partial outputs
    outs = torch.randn(n_src * blocks, bs, heads, d, device="cuda", generator=g).to(torch.bfloat16)
    lses = torch.rand(heads, n_src * blocks, bs, device="cuda", generator=g) * 10 - 5
    table = rng.permutation(n_src * blocks).reshape(blocks, n_src)
    results = []
    for order in ([0, 1, 2, 3], [2, 0, 3, 1]):
        dst_out = torch.empty(blocks * bs, heads, d, device="cuda", dtype=torch.bfloat16)
        dst_lse = torch.empty(heads, blocks * bs, device="cuda")
        flash_attn_update_out_lse(outs, dst_out, lses, dst_lse, heads, i32(table[:, order]), i32(np.arange(blocks) * bs),
                                  i32([bs] * blocks), i32([n_src] * blocks), bs, numel, heads * d, bs, 1,
                                  n_src * blocks * bs, blocks * bs, d, n_src, 64)
        results.append((dst_out, dst_lse))
    torch.cuda.synchronize()
    assert float((results[0][1] - results[1][1]).abs().max()) <= 1e-5
    a, b = results[0][0].float(), results[1][0].float()
    assert float(((a - b).abs() / a.abs().clamp(min=1.0)).max()) <= 2e-2  # one bf16 ulp of summation order
    # and a sampled block against the oracle
    b0 = 17
    o, l = oracle.merge_out_lse(outs[table[b0]].float().cpu().numpy(), lses[:, table[b0]].permute(1, 0, 2).cpu().numpy())
    assert np.abs(results[0][0][b0 * bs : (b0 + 1) * bs].float().cpu().numpy() - o).max() <= 2e-2
    assert np.abs(results[0][1][:, b0 * bs : (b0 + 1) * bs].cpu().numpy() - l).max() <= 1e-3
