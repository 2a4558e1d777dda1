#!/usr/bin/env python3
"""Benchmark of the per-device blockwise attention path on one MI355X.

One step = one forward plus one backward pass of the executor over a synthetic
single-device block schedule (gather -> range-masked paged attention ->
merge/scatter; gather -> attention backward -> block sums/scatter), with all
inputs already resident in HBM and every argument table prepared, as the
reference's micro-benchmark times only ``executor.execute(plan)``
(benchmark/microbenchmark/benchmark_attention.py:976-1021).

Prints ONE JSON line.  ``value`` is mask-aware attention TFLOP/s for fwd+bwd,
with the reference cost model's FLOP convention (dcp/core/cost_model.py:120-127:
fwd = 4*P*H*D, bwd = 2.5*fwd, P = unmasked (q, k) pairs).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBPS = 8000.0  # MI355X HBM3E

def profile_traffic(workload, kernels):
    """HBM bytes per launch of the backward's kernels, from the committed rocprofv3 summary of this
    script (profiles/attention_<workload>_hbm_traffic.txt: a `roofline_traffic` line per kernel,
    FETCH_SIZE and WRITE_SIZE scaled by what the counters read for a copy kernel of known size).
    Counters cannot be read from inside the benchmark; the figure is only reported while the
    summary covers exactly the kernels this run launched, and with the commit it was taken at."""
    path = os.path.join(ROOT, "profiles", f"attention_{workload}_hbm_traffic.txt")
    if not os.path.exists(path):
        return None
    found, source = {}, None
    for line in open(path):
        parts = line.split()
        if len(parts) >= 3 and parts[0] == "roofline_traffic":
            found[parts[1]] = int(float(parts[2]))
        elif len(parts) >= 2 and parts[0] == "measured_at_commit":
            source = parts[1]
    big = {k for k in kernels if k not in ("bwd_tile_hull_kernel",)}
    if not big or not big <= set(found):
        return None
    return dict(bytes=sum(found[k] for k in big), source=f"profiles/{os.path.basename(path)} @ {source}")


# ---------------------------------------------------------------------------
# workloads (BASELINE.json configs)
# ---------------------------------------------------------------------------


def lognormal_lengths(total, median, lo, hi, seed, sigma=1.0):
    """Seeded lognormal sequence lengths that fill exactly ``total`` tokens."""
    rng = np.random.default_rng(seed)
    lengths, used = [], 0
    while used < total:
        n = int(np.clip(round(float(np.exp(rng.normal(np.log(median), sigma)))), lo, hi))
        if total - used - n < lo:  # the remainder would be too short: take it all
            n = total - used
            if n > hi:
                n = total - used - lo
        lengths.append(n)
        used += n
    assert sum(lengths) == total and min(lengths) >= 1
    return lengths


def workload(name):
    if name == "llama3_8b_causal_64k":
        return dict(
            seqlens=lognormal_lengths(65536, 4096, 256, 32768, seed=0),
            block_size=1024, n_heads=32, n_groups=8, head_dim=128, head_block=4, mask="causal",
            mask_info=None, mask_kwargs={},
        )
    if name == "lambda_128k":
        return dict(
            seqlens=lognormal_lengths(131072, 16384, 256, 65536, seed=0),
            block_size=1024, n_heads=32, n_groups=8, head_dim=128, head_block=4, mask="lambda",
            mask_info=None, mask_kwargs=dict(n_starting=64, l_pretrain=4096),
        )
    if name == "shared_prefix_96k":
        # one shared context of 8192 tokens followed by 4..16 independent continuations of
        # 256..2048 tokens, samples appended until 98304 tokens are filled (the last one is cut)
        rng = np.random.default_rng(0)
        seqlens, info, used, total = [], [], 0, 98304
        while used < total:
            conts = [int(c) for c in rng.integers(256, 2049, size=int(rng.integers(4, 17)))]
            room = total - used - 8192
            if room < 256:  # not even a prefix and one short continuation: lengthen the previous sample
                seqlens[-1] += total - used
                info[-1]["continuations"][-1] += total - used
                break
            kept = []
            for c in conts:
                if room <= 0:
                    break
                kept.append(min(c, room))
                room -= kept[-1]
            seqlens.append(8192 + sum(kept))
            info.append(dict(prefix=8192, continuations=kept))
            used += seqlens[-1]
        assert sum(seqlens) == total
        return dict(
            seqlens=seqlens, block_size=512, n_heads=40, n_groups=8, head_dim=128, head_block=5,
            mask="shared_prefix", mask_info=info, mask_kwargs={},
            plan_kwargs=dict(n_kv_groups=2, kv_split="contiguous"),  # every row's kv blocks in two partials: the merge runs
        )
    if name == "smoke":
        return dict(
            seqlens=[700, 300], block_size=256, n_heads=8, n_groups=2, head_dim=128, head_block=4,
            mask="causal", mask_info=None, mask_kwargs={},
        )
    raise SystemExit(f"unknown workload {name}")


def build(wl, backward=True):
    import torch
    from dcp_amd.runtime.flash_attention.single_device import build_single_device_plans
    from dcp_amd.runtime.flash_attention.utils import MASK_FNS, count_attended_pairs

    mask = MASK_FNS[wl["mask"]](wl["seqlens"], wl["seqlens"], torch.int32, wl["mask_info"], **wl["mask_kwargs"])
    fw, bw, layout = build_single_device_plans(
        wl["seqlens"], wl["block_size"], wl["n_heads"], wl["n_groups"], wl["head_dim"], wl["head_block"],
        mask, dtype=torch.bfloat16, backward=backward, **wl.get("plan_kwargs", {}))
    pairs = count_attended_pairs(mask)
    return fw, bw, layout, mask, pairs


# ---------------------------------------------------------------------------
# GPU side
# ---------------------------------------------------------------------------


def make_executors(wl, fw, bw, seed=0):
    import torch
    from dcp_amd.core.instructions import BufferType
    from dcp_amd.runtime.flash_attention.executor import get_executor

    hb, d = wl["head_block"], wl["head_dim"]
    ex_f = get_executor(hb, d, None, fw_exec_plan=fw, bw_exec_plan=bw)
    ex_f.prepare(forward=True)
    ex_b = get_executor(hb, d, None, fw_exec_plan=fw, bw_exec_plan=bw)
    ex_b.mode = "Backward"
    ex_b.prepare(forward=False)
    g = torch.Generator(device="cuda").manual_seed(seed)
    q = ex_f.buffers[BufferType.LOCAL_Q]
    kv = ex_f.buffers[BufferType.LOCAL_KV]
    q.copy_((torch.randn(q.shape, generator=g, device="cuda") * 0.5).to(q.dtype))
    kv.copy_((torch.randn(kv.shape, generator=g, device="cuda") * 0.5).to(kv.dtype))
    ex_f.execute(fw, True)
    torch.cuda.synchronize()
    ex_b.init_forward_input(q, kv)
    ex_b.set_local_out_lse(ex_f.buffers[BufferType.LOCAL_OUT], ex_f.buffers[BufferType.LOCAL_LSE])
    dout = ex_b.buffers[BufferType.LOCAL_dOUT]
    dout.copy_(torch.randn(dout.shape, generator=g, device="cuda").to(dout.dtype))
    return ex_f, ex_b


def step(ex_f, ex_b, fw, bw):
    ex_f.execute(fw, True)
    ex_b.execute(bw, False)


def time_steps(ex_f, ex_b, fw, bw, steps, warmup):
    import torch

    for _ in range(warmup):
        step(ex_f, ex_b, fw, bw)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step(ex_f, ex_b, fw, bw)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


_PROBES = None


def load_probes():
    """libbench_probes.so (bench_probes.hip, built by `python -m dcp_amd.build`): the
    measurement-only kernels this benchmark runs beside the product library."""
    global _PROBES
    if _PROBES is None:
        import ctypes

        import torch  # noqa: F401  (first: one HIP runtime per process)

        path = os.path.join(ROOT, "libbench_probes.so")
        if not os.path.exists(path):
            raise SystemExit(f"{path} is not built; run `python -m dcp_amd.build`")
        lib = ctypes.CDLL(path)
        P, I = ctypes.c_void_p, ctypes.c_int
        lib.bench_mfma_probe.argtypes = [P, P, I, I, I, P, P]
        lib.bench_mfma_mix_probe.argtypes = [P, P, I, I, I, P, P]
        lib.bench_hbm_stream_probe.argtypes = [P, P, I, ctypes.c_size_t, P, ctypes.c_size_t, P]
        lib.bench_probe_last_error.restype = ctypes.c_char_p
        _PROBES = lib
    return _PROBES


def call_probe(name, *args):
    """Status 1 (argument) -> AssertionError, 2 (unsupported) -> ValueError, as the product library's calls."""
    lib = load_probes()
    status = getattr(lib, name)(*args)
    if status != 0:
        message = f"{name}: {lib.bench_probe_last_error().decode(errors='replace')}"
        raise {1: AssertionError, 2: ValueError}.get(status, RuntimeError)(message)


def mfma_sustained(iters=60000):
    """What the matrix cores sustain on this device when a kernel does nothing but bf16
    32x32x16 MFMAs, one wave per SIMD: with constant operands (full shader clock) and with
    random N(0,1) operands (the chip lowers its clock under the switching power of real data).
    The second figure is the practical ceiling the attention kernels can be held against; the
    roofline `peak` stays the published 2.5 PFLOP/s."""
    import ctypes

    import torch

    n_wg = torch.cuda.get_device_properties(0).multi_processor_count
    n_words = n_wg * 256 * 16 * 8  # 16 x 16 bytes per thread, as bf16
    out = torch.empty(2 + n_wg * 256, device="cuda", dtype=torch.float32)
    res = {}
    g = torch.Generator(device="cuda").manual_seed(0)
    stream = torch.cuda.current_stream().cuda_stream
    for name in ("constant_operands", "random_operands"):
        ops = (torch.full((n_words,), 0.5, device="cuda") if name == "constant_operands"
               else torch.randn(n_words, device="cuda", generator=g)).to(torch.bfloat16)
        flop = ctypes.c_double()
        args = (ops.data_ptr(), out.data_ptr(), n_wg, iters, 0, ctypes.byref(flop), stream)
        call_probe("bench_mfma_probe", *args)  # warm-up
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        call_probe("bench_mfma_probe", *args)
        e1.record()
        torch.cuda.synchronize()
        clocks, ticks = out[:2].tolist()
        res[name] = dict(TFLOPs=round(flop.value / (e0.elapsed_time(e1) * 1e-3) / 1e12, 1),
                         shader_MHz=round(clocks / ticks * 100.0))
    return res


def mfma_with_instruction_mix(iters=4000):
    """The MFMA probe again, two waves per SIMD and random operands, with every wave also issuing
    what an attention kernel issues beside its MFMAs (vector instructions, exponentials, LDS
    reads in the kernel's own proportions), evenly spread and free of dependencies, tile loads
    and barriers: what no schedule of that instruction mix can exceed on this device."""
    import ctypes

    import torch

    n_wg = 2 * torch.cuda.get_device_properties(0).multi_processor_count
    n_words = n_wg * 256 * 16 * 8
    g = torch.Generator(device="cuda").manual_seed(0)
    ops = torch.randn(n_words, device="cuda", generator=g).to(torch.bfloat16)
    out = torch.empty(2 + n_wg * 256, device="cuda", dtype=torch.float32)
    stream = torch.cuda.current_stream().cuda_stream
    res = {}
    for mix, name in enumerate(("attn_fwd_kernel", "attn_bwd_dkv_kernel", "attn_bwd_dq_kernel")):
        flop = ctypes.c_double()
        args = (ops.data_ptr(), out.data_ptr(), n_wg, iters, mix, ctypes.byref(flop), stream)
        call_probe("bench_mfma_mix_probe", *args)  # warm-up
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        call_probe("bench_mfma_mix_probe", *args)
        e1.record()
        torch.cuda.synchronize()
        res[name] = round(flop.value / (e0.elapsed_time(e1) * 1e-3) / 1e12, 1)
    return res


def kernel_times(ex_f, ex_b, fw, bw, steps):
    """Average duration of every kernel of the library over ``steps`` steps,
    from events recorded on the launch stream by the library itself."""
    import torch
    from dcp_amd import _lib

    torch.cuda.synchronize()
    _lib.profile_enable(True)
    for _ in range(steps):
        step(ex_f, ex_b, fw, bw)
    torch.cuda.synchronize()
    _lib.profile_enable(False)
    rep = _lib.profile_report()
    return {name: dict(launches=n, avg_ms=total / n, ms_per_step=total / steps) for name, (n, total) in rep.items()}


def movement_microbench(iters=5, bs=512):
    """BASELINE config 5: 262144 tokens x 32 heads x 128, bf16, 512-token
    blocks; gather through a seeded block permutation, inverse scatter, then a
    4-way (out, lse) merge.  Returns GB/s from events on the launch stream."""
    import torch
    from dcp_amd import _lib
    from dcp_amd.ops.fused_ops import flash_attn_update_out_lse, fused_blockwise_sum, fused_copy_bf16_varlen

    tokens, heads, d = 262144, 32, 128
    n_blocks = tokens // bs
    numel = bs * heads * d
    rng = np.random.default_rng(0)
    perm = rng.permutation(n_blocks)
    src = torch.randn(tokens, heads, d, device="cuda", dtype=torch.bfloat16)
    packed = torch.empty_like(src)
    back = torch.empty_like(src)
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device="cuda")
    i32 = lambda v: torch.tensor(np.asarray(v), dtype=torch.int32, device="cuda")
    ident = np.arange(n_blocks)
    full = i32([numel] * n_blocks)
    stride = i32([numel] * n_blocks)
    gather = (i64([src.data_ptr()] * n_blocks), i32(ident), stride, i64([packed.data_ptr()] * n_blocks), i32(perm), stride, full)
    scatter = (i64([packed.data_ptr()] * n_blocks), i32(perm), stride, i64([back.data_ptr()] * n_blocks), i32(ident), stride, full)
    fused_copy_bf16_varlen(*gather, numel, 128)
    fused_copy_bf16_varlen(*scatter, numel, 128)
    torch.cuda.synchronize()
    exact = bool(torch.equal(back, src))
    _lib.profile_enable(True)
    for _ in range(iters):
        fused_copy_bf16_varlen(*gather, numel, 128)
        fused_copy_bf16_varlen(*scatter, numel, 128)
    torch.cuda.synchronize()
    _lib.profile_enable(False)
    n, total = _lib.profile_report()["copy_varlen_kernel"]
    copy_bytes = 2 * tokens * heads * d * 2
    copy_gbps = copy_bytes / (total / n * 1e-3) / 1e9

    # the same bytes as one-head blocks (head block size 1: 16384 blocks of 128 KiB)
    n1, numel1 = n_blocks * heads, bs * d
    perm1 = rng.permutation(n1)
    ident1, stride1 = np.arange(n1), i32([numel1] * n1)
    gather1 = (i64([src.data_ptr()] * n1), i32(ident1), stride1, i64([packed.data_ptr()] * n1), i32(perm1), stride1, stride1)
    scatter1 = (i64([packed.data_ptr()] * n1), i32(perm1), stride1, i64([back.data_ptr()] * n1), i32(ident1), stride1, stride1)
    back.zero_()
    fused_copy_bf16_varlen(*gather1, numel1, 128)
    fused_copy_bf16_varlen(*scatter1, numel1, 128)
    torch.cuda.synchronize()
    exact = exact and bool(torch.equal(back, src))
    # every launch timed by itself (events on the launch stream): the first launch after another
    # kernel has been through other memory (here torch.equal over both tensors) takes about 0.3 ms
    # longer than the ones that follow -- idle time before it does not matter, a fresh destination
    # hardly -- so both rates are reported
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(2 * max(iters, 8) + 1)]
    marks[0].record()
    for i in range(max(iters, 8)):
        fused_copy_bf16_varlen(*gather1, numel1, 128)
        marks[2 * i + 1].record()
        fused_copy_bf16_varlen(*scatter1, numel1, 128)
        marks[2 * i + 2].record()
    torch.cuda.synchronize()
    launch_ms = [marks[i].elapsed_time(marks[i + 1]) for i in range(len(marks) - 1)]
    one_launch_bytes = copy_bytes  # (one launch reads 2 GiB and writes 2 GiB)
    copy1_gbps = one_launch_bytes / (sum(launch_ms) / len(launch_ms) * 1e-3) / 1e9
    copy1_first_gbps = one_launch_bytes / (launch_ms[0] * 1e-3) / 1e9
    steady = sorted(launch_ms[2:])
    copy1_steady_gbps = one_launch_bytes / (steady[len(steady) // 2] * 1e-3) / 1e9
    del packed, back

    # merge: 4 partial outs per q block
    n_src = 4
    outs = torch.randn(n_src * n_blocks, bs, heads, d, device="cuda", dtype=torch.bfloat16)
    lses = torch.rand(heads, n_src * n_blocks, bs, device="cuda") * 10 - 5
    dst_out = torch.empty(tokens, heads, d, device="cuda", dtype=torch.bfloat16)
    dst_lse = torch.empty(heads, tokens, device="cuda")
    table = i32(rng.permutation(n_src * n_blocks).reshape(n_blocks, n_src))
    args = (outs, dst_out, lses, dst_lse, heads, table, i32(ident * bs), i32([bs] * n_blocks), i32([n_src] * n_blocks),
            bs, numel, heads * d, bs, 1, n_src * n_blocks * bs, tokens, d, n_src, 64)
    flash_attn_update_out_lse(*args)
    torch.cuda.synchronize()
    _lib.profile_enable(True)
    for _ in range(iters):
        flash_attn_update_out_lse(*args)
    torch.cuda.synchronize()
    _lib.profile_enable(False)
    n, total = _lib.profile_report()["merge_out_lse_kernel"]
    merge_bytes = (n_src + 1) * (d * 2 + 4) * tokens * heads
    merge_gbps = merge_bytes / (total / n * 1e-3) / 1e9

    # block sum: the same four sources per block added up (fp32 accumulation, one rounding)
    sum_args = (i64([outs.data_ptr()] * n_blocks), table, stride, i32([n_src] * n_blocks), i64([dst_out.data_ptr()] * n_blocks),
                i32(ident), stride, full, torch.bfloat16, n_src, numel, 128)
    fused_blockwise_sum(*sum_args)
    torch.cuda.synchronize()
    _lib.profile_enable(True)
    for _ in range(iters):
        fused_blockwise_sum(*sum_args)
    torch.cuda.synchronize()
    _lib.profile_enable(False)
    n, total = _lib.profile_report()["blockwise_sum_kernel"]
    sum_bytes = (n_src + 1) * tokens * heads * d * 2
    sum_gbps = sum_bytes / (total / n * 1e-3) / 1e9

    # what a plain streaming kernel reaches at the same read : write mixes on the same buffers
    # (1 read + 1 write like the copy, 4 reads + 1 write like the merge): the practical ceiling
    stream_gbps = {}
    stream = torch.cuda.current_stream().cuda_stream
    per_stream = tokens * heads * d * 2  # 2 GiB
    # (1 read: the copy's permutation of 4 MiB blocks; 4 reads: the very table of the merge and the sum)
    tables = {1: i32(perm), 4: table}
    for ns in (1, 4):
        call = lambda: call_probe("bench_hbm_stream_probe", outs.data_ptr(), dst_out.data_ptr(), ns, per_stream,
                                  tables[ns].data_ptr(), numel * 2, stream)
        call()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            call()
        e1.record()
        torch.cuda.synchronize()
        stream_gbps[ns] = (ns + 1) * per_stream / (e0.elapsed_time(e1) / iters * 1e-3) / 1e9
    return dict(
        workload="block movement: 262144 tok x 32 heads x 128 bf16, 512-token blocks (512 blocks of 4 MiB; as one-head blocks 16384 of 128 KiB), seeded permutation",
        gather_scatter_GBps=round(copy_gbps, 1),
        gather_scatter_frac_of_8TBps=round(copy_gbps / PEAK_HBM_GBPS, 4),
        gather_scatter_one_head_blocks_GBps=round(copy1_gbps, 1),
        gather_scatter_one_head_blocks_first_launch_GBps=round(copy1_first_gbps, 1),
        gather_scatter_one_head_blocks_steady_GBps=round(copy1_steady_gbps, 1),
        gather_scatter_one_head_blocks_steady_frac_of_8TBps=round(copy1_steady_gbps / PEAK_HBM_GBPS, 4),
        gather_scatter_roundtrip_bit_exact=exact,
        copy_bytes_per_launch=copy_bytes,
        merge4_GBps=round(merge_gbps, 1),
        merge4_frac_of_8TBps=round(merge_gbps / PEAK_HBM_GBPS, 4),
        merge_bytes_per_launch=merge_bytes,
        block_sum4_GBps=round(sum_gbps, 1),
        block_sum4_frac_of_8TBps=round(sum_gbps / PEAK_HBM_GBPS, 4),
        block_sum_bytes_per_launch=sum_bytes,
        plain_stream_1r1w_GBps=round(stream_gbps[1], 1),
        plain_stream_4r1w_GBps=round(stream_gbps[4], 1),
    )


def exchange_microbench(n_devices=4, blocks_per_pair=64, bs=1024, hb=4, d=128, iters=5):
    """Block exchange between devices' executors that share the GPU (LocalFabric): every device
    sends ``blocks_per_pair`` Q blocks of [bs, hb, d] bf16 (1 MiB at the defaults) to every other
    device; the sender's copy writes into the receiver's staging buffer, the receiver unpacks
    into its slots.  Each block is read and written once per pass, two passes."""
    import torch
    from dcp_amd.core.instructions import (BufferBlock, BufferInfo, BufferType, CommLaunchInstr, CommOp,
                                            CommType, CommWaitInstr, DType, ExecutionPlan)
    from dcp_amd.runtime.flash_attention.executor import get_executor
    from dcp_amd.runtime.flash_attention.fabric import LocalFabric, execute_together

    n_send = blocks_per_pair * (n_devices - 1)
    numel = bs * hb * d
    info = {
        BufferType.LOCAL_Q: BufferInfo(n_send, bs, numel, DType.BFLOAT16, (n_send * bs, hb, d), (hb, d)),
        BufferType.BUFFER_Q: BufferInfo(n_send, bs, numel, DType.BFLOAT16, (n_send, bs, hb, d), (hb, d)),
    }
    cu = [i * bs for i in range(n_send + 1)]
    plans = []
    for r in range(n_devices):
        peers = [p for p in range(n_devices) if p != r]
        ops = []
        for k, p in enumerate(peers):
            for i in range(blocks_per_pair):
                ops.append(CommOp(CommType.SEND, (0, p), BufferBlock(BufferType.LOCAL_Q, k * blocks_per_pair + i, bs)))
                ops.append(CommOp(CommType.RECV, (0, p), BufferBlock(BufferType.BUFFER_Q, k * blocks_per_pair + i, bs)))
        plans.append(ExecutionPlan([CommLaunchInstr("S0", ops), CommWaitInstr("S0")], 1, n_devices, 0, r, 1, cu, info))
    fabric = LocalFabric(1, n_devices)
    exs = [get_executor(hb, d, None, fw_exec_plan=p, fabric=fabric) for p in plans]
    g = torch.Generator(device="cuda").manual_seed(0)
    for ex in exs:
        ex.prepare(forward=True)
        ex.buffers[BufferType.LOCAL_Q].copy_(torch.randn(n_send * bs, hb, d, device="cuda", generator=g))
    execute_together(exs)
    torch.cuda.synchronize()
    exact = True
    for r, ex in enumerate(exs):  # slot k*bpp+i of r came from peer p's block (index of r among p's peers)*bpp+i
        for k, p in enumerate([p for p in range(n_devices) if p != r]):
            kp = [q for q in range(n_devices) if q != p].index(r)
            got = ex.buffers[BufferType.BUFFER_Q][k * blocks_per_pair : (k + 1) * blocks_per_pair]
            want = exs[p].buffers[BufferType.LOCAL_Q][kp * blocks_per_pair * bs : (kp + 1) * blocks_per_pair * bs]
            exact &= bool(torch.equal(got.reshape(-1), want.reshape(-1)))
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        execute_together(exs)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / iters
    moved = n_devices * n_send * numel * 2  # bytes that change device per exchange
    return dict(
        workload=f"{n_devices} devices' executors on one GPU, {blocks_per_pair} blocks of {numel * 2 >> 10} KiB to every peer",
        ms_per_exchange=round(ms, 3),
        moved_GB_per_exchange=round(moved / 1e9, 3),
        hbm_GBps=round(4 * moved / (ms * 1e-3) / 1e9, 1),  # pack + unpack, each a read and a write
        bit_exact=exact,
    )


# ---------------------------------------------------------------------------
# CPU baseline: dense masked attention in torch on a bounded, seeded sample of q-block rows
# ---------------------------------------------------------------------------


def cpu_baseline(wl, fw, bw, budget_s=20.0, seed=0):
    """Times dense masked attention, forward and backward, of whole q-block rows (all heads of the
    row's head block against the row's keys) drawn from the workload's plan, in fp32 torch on the
    host cores (oracle/torch_cpu_path.py: the form of the reference's own dense check, the only
    CPU-expressible statement of this path it holds), until about ``budget_s`` seconds of CPU
    work are done.  One untimed row first."""
    import torch

    from oracle import dcp_oracle as oracle
    from oracle.torch_cpu_path import row_attention_fwd_bwd

    threads = torch.get_num_threads()  # the intra-op pool torch's CPU kernels run on (OMP_NUM_THREADS honoured)
    if not threads or threads < 1:
        raise SystemExit("bench.py: torch reports no CPU threads")
    instr = next(i for i in fw.instructions if type(i).__name__ == "AttnInstr")
    mask = np.asarray(instr.attn_mask)
    if mask.ndim == 2:
        mask = mask[None]
    rng = np.random.default_rng(seed)
    order = rng.permutation(len(instr.seqlens_q))
    hb, d, bs = wl["head_block"], wl["head_dim"], wl["block_size"]
    hkv = max(1, hb // (wl["n_heads"] // wl["n_groups"]))
    cu = np.concatenate(([0], np.cumsum(instr.seqlens_q)))
    pairs, rows, elapsed = 0, 0, 0.0
    f32 = lambda *shape: torch.from_numpy(rng.standard_normal(shape).astype(np.float32))
    for n, b in enumerate([order[0]] + list(order)):
        n_kv = instr.seqlens_kv[b]
        q, k, v, dout = f32(bs, hb, d) * 0.5, f32(n_kv, hkv, d) * 0.5, f32(n_kv, hkv, d) * 0.5, f32(bs, hb, d)
        allowed = torch.from_numpy(oracle.ranges_to_bool(mask[:, :, cu[b] : cu[b + 1]], n_kv))
        t0 = time.perf_counter()
        row_attention_fwd_bwd(q, k, v, dout, allowed)
        if n == 0:
            continue  # warm-up
        elapsed += time.perf_counter() - t0
        pairs += int(allowed.sum())
        rows += 1
        if elapsed >= budget_s:
            break
    flops = oracle.attention_flops(pairs, hb, d, "fwd+bwd")
    return dict(
        value=round(flops / elapsed / 1e12, 5), unit="TFLOP/s", cores=int(threads), kind="port",
        sample=f"{rows} seeded q-block rows of the same schedule, their shapes and masks with random N(0, 1) data "
               f"(not the GPU run's tensors): fwd+bwd, dense masked attention in fp32 torch on the host, {elapsed:.1f} s",
    )


# ---------------------------------------------------------------------------


def stage_packer_timing(n_blocks=96, n_nodes=2, ranks=8, n_stages=4):
    """Host side of the planner: one backward-style planning problem (causal block pairs of
    `n_blocks` query/key blocks over n_nodes x ranks devices) grouped into `n_stages` stages by the
    native stage packer (dcp_greedy_stage_selection) and, where it has been built from the
    reference sources into oracle/_ref, by the reference's own C++ module, on the host cores.
    Reported per greedy-selection call, conversion of the Python containers included for both."""
    import importlib.util

    from dcp_amd.core import pipeline
    from oracle import build_ref

    devices = [(n, r) for n in range(n_nodes) for r in range(ranks)]
    types = ["Q"] * n_blocks + ["KV"] * n_blocks
    sizes = [1.0 + (i % 7) * 0.25 for i in range(n_blocks)] + [2.0 + (i % 5) * 0.5 for i in range(n_blocks)]
    for q in range(n_blocks):
        types += ["OUT", "LSE", "dOUT"]
        sizes += [sizes[q], sizes[q] / 64, sizes[q]]
    win, costs = [], []
    for q in range(n_blocks):
        for k in range(q + 1):
            win.append([q, n_blocks + k, 2 * n_blocks + 3 * q, 2 * n_blocks + 3 * q + 1, 2 * n_blocks + 3 * q + 2])
            costs.append(1.0 + ((q * 31 + k * 17) % 97) / 97.0)
    home = {i: devices[(i % n_blocks) % len(devices)] for i in range(2 * n_blocks)}
    for q in range(n_blocks):
        for j in range(3):
            home[2 * n_blocks + 3 * q + j] = home[q]
    w_home = {w: devices[(w * 7) % len(devices)] for w in range(len(win))}
    dev_work = {d: [] for d in devices}
    for w, d in w_home.items():
        dev_work[d].append(w)
    local0 = {d: {} for d in devices}
    for i, d in home.items():
        local0[d][i] = -1
    total = sum(sizes)
    target = {d: total / len(devices) / n_stages * 1.2 for d in devices}

    def run(select):
        scheduled, local = set(), local0
        t0 = time.perf_counter()
        for stage in range(n_stages):
            tgt = target if stage < n_stages - 1 else {d: float("inf") for d in devices}
            unlocked, _, local = select(set(devices), scheduled, costs, sizes, win, types, dev_work, local, tgt, True,
                                        stage, None)
            for ws in unlocked.values():
                scheduled |= ws
        assert len(scheduled) == len(win)
        return (time.perf_counter() - t0) / n_stages * 1e3

    res = {"problem": f"{len(win)} workloads, {len(sizes)} blocks, {len(devices)} devices, {n_stages} stages",
           "native_ms_per_call": round(min(run(pipeline.greedy_selection_per_device) for _ in range(3)), 3)}
    ref_path = build_ref.module_path()
    if ref_path.exists():
        spec = importlib.util.spec_from_file_location("dcp_cpp", ref_path)
        ref = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(ref)
        res["reference_cpp_ms_per_call"] = round(min(run(ref.greedy_selection_per_device) for _ in range(3)), 3)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="llama3_8b_causal_64k")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-movement", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit(
            "bench.py: this build runs on exactly one GPU (no collectives, no sharding); use --gpus 1")

    import torch

    if not torch.cuda.is_available():
        raise SystemExit("bench.py: no GPU visible")
    from dcp_amd import _lib

    _lib.load()
    torch.cuda.set_device(0)
    wl = workload(args.workload)
    fw, bw, layout, mask, pairs = build(wl)
    flops_fwd = 4.0 * pairs * wl["n_heads"] * wl["head_dim"]
    flops_step = 3.5 * flops_fwd

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(wl, fw, bw, budget_s=args.cpu_seconds)

    ex_f, ex_b = make_executors(wl, fw, bw)
    sec = time_steps(ex_f, ex_b, fw, bw, args.steps, args.warmup)
    kt = kernel_times(ex_f, ex_b, fw, bw, max(2, min(args.steps, 5)))
    value = flops_step / sec / 1e12

    # The backward is a group of kernels that together do the algorithmic backward work
    # 2.5 * fwd and are priced as one unit: the key-outer dK/dV kernel, a dQ kernel (one that
    # recomputes S and dP, or one that reads the dS the dK/dV kernel stored) and the small kernel
    # before them (range hulls; with stored dS also -delta and the base-2 log-sum-exp).
    # Executed matrix products per kernel, of the backward's five:
    products = {"attn_bwd_dkv_kernel": 4, "attn_bwd_dq_kernel": 3, "attn_bwd_dq_ds_kernel": 1, "attn_bwd_fused_kernel": 5,
                "bwd_tile_hull_kernel": 0, "bwd_prepare_kernel": 0}
    bwd = {k: v for k, v in kt.items() if k in products}
    fwd = kt["attn_fwd_kernel"]
    # A plan that splits every row's kv blocks over several partials launches each kernel that
    # many times per step; a launch then does 1/n of the step's work on average.
    n_launch = max(1, round(fwd["ms_per_step"] / fwd["avg_ms"]))
    bwd_ms = sum(v["avg_ms"] for v in bwd.values())
    bwd_tflops = 2.5 * flops_fwd / n_launch / (bwd_ms * 1e-3) / 1e12
    fwd_tflops = flops_fwd / n_launch / (fwd["avg_ms"] * 1e-3) / 1e12
    traffic = profile_traffic(args.workload, set(bwd))
    roofline = dict(
        bound="mfma", kernel="+".join(sorted(bwd)), achieved=round(bwd_tflops, 2),
        peak=PEAK_BF16_TFLOPS, unit="TFLOP/s", frac=round(bwd_tflops / PEAK_BF16_TFLOPS, 4),
        traffic=traffic["bytes"] if traffic else None, traffic_source=traffic["source"] if traffic else None,
        flops_per_launch=2.5 * flops_fwd / n_launch, avg_launch_ms=round(bwd_ms, 4),
    )
    extra = dict(
        attn_fwd_kernel=dict(achieved_TFLOPs=round(fwd_tflops, 2), frac_of_peak=round(fwd_tflops / PEAK_BF16_TFLOPS, 4),
                             avg_launch_ms=round(fwd["avg_ms"], 4)),
        kernel_ms_per_step={k: round(v["ms_per_step"], 4) for k, v in sorted(kt.items())},
        mfma_only_kernel=mfma_sustained(),
    )
    for k, v in bwd.items():
        if products[k]:
            extra[k] = dict(executed_TFLOPs=round(products[k] * 0.5 * flops_fwd / n_launch / (v["avg_ms"] * 1e-3) / 1e12, 2),
                            matrix_products=products[k], avg_launch_ms=round(v["avg_ms"], 4))
    # executed MFMA rate of each attention kernel against what MFMAs sustain beside that kernel's
    # own mix of other instructions (dependency-free, no loads, no barriers)
    mix = mfma_with_instruction_mix()
    executed = dict(attn_fwd_kernel=fwd_tflops, **{k: extra[k]["executed_TFLOPs"] for k in bwd if k in extra})
    extra["mfma_with_kernel_instruction_mix"] = {
        k: dict(bound_TFLOPs=v, kernel_executed_frac_of_bound=round(executed[k] / v, 3)) for k, v in mix.items() if k in executed}
    if not args.no_movement:
        del ex_f, ex_b
        torch.cuda.empty_cache()
        extra["block_movement"] = movement_microbench()
        torch.cuda.empty_cache()
        extra["block_exchange"] = exchange_microbench()
    if not args.no_cpu:
        extra["stage_packer"] = stage_packer_timing()

    line = {
        "metric": "mask-aware attn fwd+bwd TFLOP/s @1 MI355X; block merge/gather HBM GB/s",
        "value": round(value, 3),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": args.workload,
            "tokens": int(sum(wl["seqlens"])), "n_sequences": len(wl["seqlens"]),
            "max_seqlen": int(max(wl["seqlens"])), "block_size": wl["block_size"],
            "q_heads": wl["n_heads"], "kv_heads": wl["n_groups"], "head_dim": wl["head_dim"],
            "head_block": wl["head_block"], "mask": wl["mask"], "unmasked_pairs_per_head": int(pairs),
            "flops_per_step": flops_step,
        },
        "roofline": roofline,
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
