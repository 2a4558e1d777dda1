"""Shared builders for plan-level tests: seeded inputs, the oracle run and the
executor run of one synthetic single-device schedule."""

import numpy as np
import torch

from dcp_amd.runtime.flash_attention.single_device import build_single_device_plans
from dcp_amd.runtime.flash_attention.utils import MASK_FNS
from oracle import dcp_oracle as oracle

TORCH_DTYPE = {"bf16": torch.bfloat16, "fp16": torch.float16}

# Parity bounds against the fp64 oracle fed the same (already rounded) inputs: max-abs 2e-2 on
# out and dQ, 1e-3 on the fp32 LSE.  dK/dV sum thousands of queries and reach magnitudes (5..13
# in these cases) where one bf16 ulp exceeds 2e-2, so for them the bound is 2e-2 * max(1, |ref|).
OUT_TOL = 2e-2
LSE_TOL = 1e-3
GRAD_TOL = 2e-2


def max_abs_err(got, ref):
    return float(np.abs(np.asarray(got, dtype=np.float64) - np.asarray(ref, dtype=np.float64)).max())


def scaled_err(got, ref):
    """Largest |got - ref| / max(1, |ref|) (dK/dV only)."""
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    return float((np.abs(got - ref) / np.maximum(1.0, np.abs(ref))).max())


def check_against_truth(res, truth, out_tol=OUT_TOL):
    """Asserts the bounds above on (out, lse[, dq, dkv]); returns the errors."""
    errs = dict(out=max_abs_err(res[0].float().numpy(), truth[0]), lse=max_abs_err(res[1].numpy(), truth[1]))
    assert np.isfinite(res[1].numpy()).all()
    assert errs["out"] <= out_tol, errs
    assert errs["lse"] <= LSE_TOL, errs
    if len(truth) > 2:
        errs["dq"] = max_abs_err(res[2].float().numpy(), truth[2])
        errs["dkv"] = scaled_err(res[3].float().numpy(), truth[3])
        assert errs["dq"] <= GRAD_TOL, errs
        assert errs["dkv"] <= GRAD_TOL, errs
    return errs


def make_case(seqlens, block_size, n_heads, n_groups, head_dim, head_block, mask="causal",
              mask_info=None, dtype="bf16", n_kv_groups=1, kv_split="round_robin", fold=False,
              seed=0, qkv_scale=1.0, mask_kwargs=None, work_units="overlap"):
    mask_t = MASK_FNS[mask](list(seqlens), list(seqlens), torch.int32, mask_info, **(mask_kwargs or {}))
    fw, bw, layout = build_single_device_plans(
        seqlens, block_size, n_heads, n_groups, head_dim, head_block, mask_t,
        dtype=TORCH_DTYPE[dtype], n_kv_groups=n_kv_groups, kv_split=kv_split, fold_stages=fold,
        work_units=work_units)
    g = torch.Generator().manual_seed(seed)
    T = sum(seqlens)
    q = (torch.randn(T, n_heads, head_dim, generator=g) * qkv_scale).to(TORCH_DTYPE[dtype])
    kv = (torch.randn(T, 2, n_groups, head_dim, generator=g) * qkv_scale).to(TORCH_DTYPE[dtype])
    dout = torch.randn(T, n_heads, head_dim, generator=g).to(TORCH_DTYPE[dtype])
    return dict(fw=fw, bw=bw, layout=layout, mask=mask_t, q=q, kv=kv, dout=dout, seqlens=list(seqlens),
                head_block=head_block, head_dim=head_dim, dtype=dtype)


def dense_truth(case, backward=False):
    """Whole-sequence fp64 attention on the (already rounded) inputs."""
    q = case["q"].float().numpy()
    kv = case["kv"].float().numpy()
    m = case["mask"].numpy()
    if backward:
        return oracle.dense_reference(q, kv, m, case["seqlens"], dout=case["dout"].float().numpy())
    return oracle.dense_reference(q, kv, m, case["seqlens"])


def poison_slot_buffers(ex, value):
    """Fills every padded slot buffer of a prepared executor with +-``value`` (LSE slots: +value):
    what a caller's recycled memory may hold in the rows the gather does not overwrite."""
    for name, buf in ex.buffers.items():
        if not name.startswith("Buffer"):
            continue
        if buf.dtype == torch.float32:
            buf.fill_(value)
        else:
            sign = (torch.arange(buf.numel(), device=buf.device) % 3 == 0).to(buf.dtype) * 2 - 1
            buf.copy_((sign * value).reshape(buf.shape))


def run_executor(case, backward=False, use_graph=False, synchronous=False, poison=None):
    """Run the plans through the HIP executor.  Returns global-layout tensors
    on the CPU: (out, lse) or (out, lse, dq, dkv).  ``poison``: fill the padded slot buffers
    with +-that value instead of the zeros they are created with."""
    from dcp_amd.runtime.flash_attention.executor import get_executor

    layout = case["layout"]
    ex = get_executor(case["head_block"], case["head_dim"], None, fw_exec_plan=case["fw"],
                      bw_exec_plan=case["bw"], synchronous=synchronous, use_cudagraph=use_graph)
    ex.prepare(forward=True)
    if poison is not None:
        poison_slot_buffers(ex, poison)
    lq = layout.to_local_q(case["q"]).cuda()
    lkv = layout.to_local_kv(case["kv"]).cuda()
    if use_graph:
        ex.init_forward_input(lq, lkv)
        ex.execute(case["fw"], True)  # eager once
        ex.capture_cudagraph()
    out, lse = ex.forward(lq, lkv)
    torch.cuda.synchronize()
    res = [layout.from_local_q(out.cpu()), layout.from_local_lse(lse.cpu())]
    if backward:
        ex.switch_to_backward()
        if poison is not None:
            poison_slot_buffers(ex, poison)
        ldout = layout.to_local_q(case["dout"]).cuda()
        if use_graph:
            ex.capture_cudagraph()
        dq, dkv = ex.backward(lq, lkv, out, ldout, lse)
        torch.cuda.synchronize()
        res += [layout.from_local_q(dq.cpu()), layout.from_local_kv(dkv.cpu())]
    return res, ex


def storage_ulp(x, dtype="bf16"):
    """Spacing of the 16-bit storage type at |x| (bf16: 8 significand bits, fp16: 11)."""
    x = np.maximum(np.abs(np.asarray(x, dtype=np.float64)), 2.0 ** -126 if dtype == "bf16" else 2.0 ** -14)
    return 2.0 ** (np.floor(np.log2(x)) - (7 if dtype == "bf16" else 10))


class SlackPlanOracle(oracle.PlanOracle):
    """The plan interpreter, which also keeps for every element of the 16-bit buffers how far a second
    exact run of the same plan may end up from this one through rounding alone: wherever the plan
    stores a value in 16 bits, a difference in the last bits of the value before rounding can move
    the stored value by one step of the type AT THAT VALUE's magnitude; a sum passes its sources'
    steps on and adds its own, a merge (a convex combination) passes on the largest.  This is what
    makes a bound of "a few steps of the result" wrong for a dK that is the small sum of large
    replicas, and it is all the slack a comparison of the kernels with the interpreter needs
    beyond the kernels' own arithmetic."""

    def __init__(self, plan, hb, head_dim, dtype="bf16"):
        super().__init__(plan, hb, head_dim)
        self.dtype = dtype
        self.slack = {name: np.zeros(buf.shape) for name, buf in self.buffers.items()
                      if self.store_dtype[name] != "fp32"}
        self._carried = 0.0

    def _store(self, name, index, value):
        super()._store(name, index, value)
        if name in self.slack:
            # (the step just above the value: the other run may land across a power of two)
            self.slack[name][index] = self._carried + storage_ulp(1.01 * self.buffers[name][index], self.dtype)

    def _MemcpyInstr(self, instr):
        super()._MemcpyInstr(instr)
        cu = self.plan.local_cu_seqlens
        for src, dst in instr.src_dst_pairs:
            if dst.buffer_type in self.slack and src.buffer_type in self.slack:
                off = cu[src.index]
                self.slack[dst.buffer_type][dst.index, : src.n_tokens] = self.slack[src.buffer_type][off : off + src.n_tokens]

    def _AttnReductionInstr(self, instr):
        for op in instr.ops:
            n = op.dst_buffer[0].n_tokens
            self._carried = np.max([self.slack[o.buffer_type][o.index, :n] for o, _ in op.src_buffers], axis=0)
            super()._AttnReductionInstr(type("One", (), dict(ops=[op], output_is_unpadded=instr.output_is_unpadded))())
        self._carried = 0.0

    def _SumInstr(self, instr):
        for op in instr.ops:
            n = op.dst_buffer.n_tokens
            self._carried = np.sum([self.slack[s.buffer_type][s.index, :n] for s in op.src_buffers], axis=0)
            if len(op.src_buffers) == 1:  # a copy rounds nothing
                self._carried = self._carried - storage_ulp(1.01 * self.buffers[op.src_buffers[0].buffer_type][op.src_buffers[0].index, :n], self.dtype)
            super()._SumInstr(type("One", (), dict(ops=[op], output_is_unpadded=instr.output_is_unpadded))())
        self._carried = 0.0


def run_plan_oracle(case, backward=False, with_slack=False):
    """The plans on the oracle's interpreter; global-layout results like run_executor.  With
    ``with_slack`` also the rounding slack of out, dq and dkv (see SlackPlanOracle), in the same layout."""
    if with_slack:
        return _run_plan_oracle_with_slack(case)
    layout = case["layout"]
    po = oracle.PlanOracle(case["fw"], case["head_block"], case["head_dim"])
    po.set("LocalQ", layout.to_local_q(case["q"]).float().numpy())
    po.set("LocalKV", layout.to_local_kv(case["kv"]).float().numpy())
    bufs = po.run()
    out_l = torch.from_numpy(bufs["LocalOut"].copy())
    lse_l = torch.from_numpy(bufs["LocalLSE"].copy())
    res = [layout.from_local_q(out_l), layout.from_local_lse(lse_l)]
    if backward:
        pb = oracle.PlanOracle(case["bw"], case["head_block"], case["head_dim"])
        pb.set("LocalQ", layout.to_local_q(case["q"]).float().numpy())
        pb.set("LocalKV", layout.to_local_kv(case["kv"]).float().numpy())
        pb.set("LocalOut", bufs["LocalOut"])
        pb.buffers["LocalLSE"][...] = bufs["LocalLSE"]
        pb.set("LocaldOut", layout.to_local_q(case["dout"]).float().numpy())
        b2 = pb.run()
        res += [layout.from_local_q(torch.from_numpy(b2["LocaldQ"].copy())),
                layout.from_local_kv(torch.from_numpy(b2["LocaldKV"].copy()))]
    return res


def _run_plan_oracle_with_slack(case):
    layout = case["layout"]
    po = SlackPlanOracle(case["fw"], case["head_block"], case["head_dim"], case["dtype"])
    po.set("LocalQ", layout.to_local_q(case["q"]).float().numpy())
    po.set("LocalKV", layout.to_local_kv(case["kv"]).float().numpy())
    po.slack["LocalQ"][...] = 0.0  # inputs are given, not computed
    po.slack["LocalKV"][...] = 0.0
    bufs = po.run()
    pb = SlackPlanOracle(case["bw"], case["head_block"], case["head_dim"], case["dtype"])
    pb.set("LocalQ", layout.to_local_q(case["q"]).float().numpy())
    pb.set("LocalKV", layout.to_local_kv(case["kv"]).float().numpy())
    pb.set("LocalOut", bufs["LocalOut"])
    pb.buffers["LocalLSE"][...] = bufs["LocalLSE"]
    pb.set("LocaldOut", layout.to_local_q(case["dout"]).float().numpy())
    for name in ("LocalQ", "LocalKV", "LocalOut", "LocaldOut"):
        pb.slack[name][...] = 0.0
    b2 = pb.run()
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32))
    res = [layout.from_local_q(t(bufs["LocalOut"])), layout.from_local_lse(t(bufs["LocalLSE"])),
           layout.from_local_q(t(b2["LocaldQ"])), layout.from_local_kv(t(b2["LocaldKV"]))]
    slack = [layout.from_local_q(t(po.slack["LocalOut"])), None, layout.from_local_q(t(pb.slack["LocaldQ"])),
             layout.from_local_kv(t(pb.slack["LocaldKV"]))]
    return res, slack


# ---------------------------------------------------------------------------
# several devices (their executors share the one GPU; blocks travel over a LocalFabric)
# ---------------------------------------------------------------------------


def make_multi_case(n_nodes, n_devices_per_node, seqlens, block_size, n_heads, n_groups, head_dim, head_block,
                    mask="causal", mask_info=None, dtype="bf16", seed=0, mask_kwargs=None, n_stages=None,
                    disable_two_phase_comm=False):
    """``n_stages`` = None: one input exchange (build_multi_device_plans); a number: the stage
    packer groups the work units into that many stages (build_staged_multi_device_plans)."""
    from dcp_amd.runtime.flash_attention.multi_device import build_multi_device_plans, build_staged_multi_device_plans

    mask_t = MASK_FNS[mask](list(seqlens), list(seqlens), torch.int32, mask_info, **(mask_kwargs or {}))
    if n_stages is None:
        fw, bw, layouts = build_multi_device_plans(n_nodes, n_devices_per_node, seqlens, block_size, n_heads, n_groups,
                                                   head_dim, head_block, mask_t, dtype=TORCH_DTYPE[dtype])
    else:
        fw, bw, layouts = build_staged_multi_device_plans(
            n_nodes, n_devices_per_node, seqlens, block_size, n_heads, n_groups, head_dim, head_block, mask_t,
            dtype=TORCH_DTYPE[dtype], n_stages=n_stages, disable_two_phase_comm=disable_two_phase_comm)
    g = torch.Generator().manual_seed(seed)
    T = sum(seqlens)
    q = torch.randn(T, n_heads, head_dim, generator=g).to(TORCH_DTYPE[dtype])
    kv = torch.randn(T, 2, n_groups, head_dim, generator=g).to(TORCH_DTYPE[dtype])
    dout = torch.randn(T, n_heads, head_dim, generator=g).to(TORCH_DTYPE[dtype])
    return dict(fw=fw, bw=bw, layouts=layouts, mask=mask_t, q=q, kv=kv, dout=dout, seqlens=list(seqlens),
                head_block=head_block, head_dim=head_dim, dtype=dtype, n_nodes=n_nodes,
                n_devices_per_node=n_devices_per_node)


def _sum_over_ranks(parts):
    total = parts[0].clone()
    for p in parts[1:]:
        total += p
    return total


def run_multi_oracle(case, backward=False):
    """All devices' plans on the numpy oracle.  Global-layout (out, lse[, dq, dkv])."""
    lays = case["layouts"]
    fw = [oracle.PlanOracle(p, case["head_block"], case["head_dim"]) for p in case["fw"]]
    for o, lay in zip(fw, lays):
        o.set("LocalQ", lay.to_local_q(case["q"]).float().numpy())
        o.set("LocalKV", lay.to_local_kv(case["kv"]).float().numpy())
    oracle.run_plans_together(fw, case["n_devices_per_node"])
    outs = [torch.from_numpy(o.buffers["LocalOut"].copy()) for o in fw]
    lses = [torch.from_numpy(o.buffers["LocalLSE"].copy()) for o in fw]
    res = [_sum_over_ranks([lay.from_local_q(x) for lay, x in zip(lays, outs)]),
           _sum_over_ranks([lay.from_local_lse(x) for lay, x in zip(lays, lses)])]
    if backward:
        bw = [oracle.PlanOracle(p, case["head_block"], case["head_dim"]) for p in case["bw"]]
        for o, f, lay in zip(bw, fw, lays):
            o.set("LocalQ", lay.to_local_q(case["q"]).float().numpy())
            o.set("LocalKV", lay.to_local_kv(case["kv"]).float().numpy())
            o.set("LocalOut", f.buffers["LocalOut"])
            o.buffers["LocalLSE"][...] = f.buffers["LocalLSE"]
            o.set("LocaldOut", lay.to_local_q(case["dout"]).float().numpy())
        oracle.run_plans_together(bw, case["n_devices_per_node"])
        res += [_sum_over_ranks([lay.from_local_q(torch.from_numpy(o.buffers["LocaldQ"].copy())) for lay, o in zip(lays, bw)]),
                _sum_over_ranks([lay.from_local_kv(torch.from_numpy(o.buffers["LocaldKV"].copy())) for lay, o in zip(lays, bw)])]
    return res


def run_multi_executor(case, backward=False, repeats=1):
    """All devices' plans through HIP executors that share the GPU and one LocalFabric."""
    from dcp_amd.runtime.flash_attention.executor import get_executor
    from dcp_amd.runtime.flash_attention.fabric import LocalFabric, execute_together

    fabric = LocalFabric(case["n_nodes"], case["n_devices_per_node"])
    lays = case["layouts"]
    exs = [get_executor(case["head_block"], case["head_dim"], None, fw_exec_plan=f, bw_exec_plan=b, fabric=fabric)
           for f, b in zip(case["fw"], case["bw"])]
    for ex in exs:
        ex.prepare(forward=True)
    for ex, lay in zip(exs, lays):
        ex.init_forward_input(lay.to_local_q(case["q"]).cuda(), lay.to_local_kv(case["kv"]).cuda())
    for _ in range(repeats):
        execute_together(exs, forward=True)
    torch.cuda.synchronize()
    outs = [ex.buffers["LocalOut"].clone() for ex in exs]
    lses = [ex.buffers["LocalLSE"].clone() for ex in exs]
    res = [_sum_over_ranks([lay.from_local_q(x.cpu()) for lay, x in zip(lays, outs)]),
           _sum_over_ranks([lay.from_local_lse(x.cpu()) for lay, x in zip(lays, lses)])]
    if backward:
        for ex in exs:
            ex.switch_to_backward()
        for ex, lay, o, l in zip(exs, lays, outs, lses):
            ex.set_local_out_lse(o, l)
            ex.init_forward_input(lay.to_local_q(case["q"]).cuda(), lay.to_local_kv(case["kv"]).cuda())
            ex.init_backward_input(lay.to_local_q(case["dout"]).cuda())
        for _ in range(repeats):
            execute_together(exs, forward=False)
        torch.cuda.synchronize()
        res += [_sum_over_ranks([lay.from_local_q(ex.buffers["LocaldQ"].cpu()) for lay, ex in zip(lays, exs)]),
                _sum_over_ranks([lay.from_local_kv(ex.buffers["LocaldKV"].cpu()) for lay, ex in zip(lays, exs)])]
    return res, exs
