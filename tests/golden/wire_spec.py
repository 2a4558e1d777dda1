"""Plain-data description of DCP instructions and plans, and its conversion to and from the
objects of an instruction module.  `isa` is any module with the instruction set's class names
(BufferBlock, MemcpyInstr, ... ExecutionPlan): the fixture generator passes the reference's
dcp.core.instructions, the tests pass dcp_amd.core.instructions.  Nothing here encodes bytes.

block            [buffer_type, index, n_tokens]
MemcpyInstr      {"op", "src_dst_pairs": [[block, block], ...]}
CommLaunchInstr  {"op", "key", "comm_ops": [[comm_type, [node, device], block], ...], "stream"}
CommWaitInstr    {"op", "key", "stream"}     BarrierInstr  {"op"}
AttnInstr        {"op", "stage_id", "seqlens_q", "seqlens_kv", "max_seqlen_q", "max_seqlen_kv",
                  "attn_mask": nested ints [2][T] or [2][2][T], "q_block_table": [[block, ...], ...],
                  "kv_block_table", "out_block_table", "lse_block_table"}
AttnBackwardInstr  as AttnInstr with "dq_block_table", "dkv_block_table" instead of "lse_block_table"
AttnReductionInstr {"op", "ops": [{"src": [[out block, lse block], ...], "dst": [out block, lse block]}], "output_is_unpadded"}
SumInstr         {"op", "ops": [{"src": [block, ...], "dst": block}], "output_is_unpadded"}
plan             {"instructions": [...], "n_nodes", "n_devices_per_node", "node_id", "local_device_id",
                  "n_stages", "local_cu_seqlens", "buffer_info": {buffer_type: [n_blocks, block_size,
                  block_numel, dtype, buffer_shape, per_token_shape]}}
"""

import torch

_TABLES = ("q_block_table", "kv_block_table", "out_block_table", "lse_block_table", "dq_block_table", "dkv_block_table")
_ATTN_SCALARS = ("stage_id", "seqlens_q", "seqlens_kv", "max_seqlen_q", "max_seqlen_kv")


def _blk(isa, b):
    return isa.BufferBlock(b[0], int(b[1]), int(b[2]))


def _unblk(b):
    return [b.buffer_type, int(b.index), int(b.n_tokens)]


def instr_from_spec(isa, s, mask_as_planes):
    """``mask_as_planes``: hand the ranges over as a list of int32 tensors, one per entry of the
    first axis (what the reference's codec iterates over), instead of as one tensor."""
    op = s["op"]
    if op == "MemcpyInstr":
        return isa.MemcpyInstr([(_blk(isa, a), _blk(isa, b)) for a, b in s["src_dst_pairs"]])
    if op == "CommLaunchInstr":
        ops = [isa.CommOp(int(t), (int(peer[0]), int(peer[1])), _blk(isa, b)) for t, peer, b in s["comm_ops"]]
        return isa.CommLaunchInstr(s["key"], ops, stream=s["stream"])
    if op == "CommWaitInstr":
        return isa.CommWaitInstr(s["key"], stream=s["stream"])
    if op == "BarrierInstr":
        return isa.BarrierInstr()
    if op in ("AttnInstr", "AttnBackwardInstr"):
        mask = torch.tensor(s["attn_mask"], dtype=torch.int32)
        kw = {k: s[k] for k in _ATTN_SCALARS}
        kw["attn_mask"] = [m.contiguous() for m in mask] if mask_as_planes else mask
        for t in _TABLES:
            if t in s:
                kw[t] = [[_blk(isa, b) for b in row] for row in s[t]]
        return getattr(isa, op)(**kw)
    if op == "AttnReductionInstr":
        ops = [isa.ReductionOp([(_blk(isa, o), _blk(isa, l)) for o, l in r["src"]], (_blk(isa, r["dst"][0]), _blk(isa, r["dst"][1])))
               for r in s["ops"]]
        return isa.AttnReductionInstr(ops, int(s["output_is_unpadded"]))
    if op == "SumInstr":
        ops = [isa.SumOp([_blk(isa, b) for b in r["src"]], _blk(isa, r["dst"])) for r in s["ops"]]
        return isa.SumInstr(ops, int(s["output_is_unpadded"]))
    raise ValueError(f"unknown instruction {op}")


def plan_from_spec(isa, s, mask_as_planes):
    info = {k: isa.BufferInfo(int(v[0]), int(v[1]), int(v[2]), int(v[3]), tuple(v[4]), tuple(v[5]))
            for k, v in s["buffer_info"].items()}
    return isa.ExecutionPlan([instr_from_spec(isa, i, mask_as_planes) for i in s["instructions"]], s["n_nodes"],
                             s["n_devices_per_node"], s["node_id"], s["local_device_id"], s["n_stages"],
                             list(s["local_cu_seqlens"]), info)


def instr_to_spec(instr):
    """The plain description of an instruction object (of either module)."""
    op = type(instr).__name__
    s = {"op": op}
    if op == "MemcpyInstr":
        s["src_dst_pairs"] = [[_unblk(a), _unblk(b)] for a, b in instr.src_dst_pairs]
    elif op == "CommLaunchInstr":
        s.update(key=instr.key, stream=instr.stream,
                 comm_ops=[[int(o.comm_type), [int(o.peer[0]), int(o.peer[1])], _unblk(o.buffer_block)] for o in instr.comm_ops])
    elif op == "CommWaitInstr":
        s.update(key=instr.key, stream=instr.stream)
    elif op in ("AttnInstr", "AttnBackwardInstr"):
        for k in _ATTN_SCALARS:
            v = getattr(instr, k)
            s[k] = [int(x) for x in v] if isinstance(v, (list, tuple)) else int(v)
        mask = instr.attn_mask
        mask = torch.stack(list(mask)) if isinstance(mask, (list, tuple)) else mask
        s["attn_mask"] = mask.tolist()
        for t in _TABLES:
            if hasattr(instr, t):
                s[t] = [[_unblk(b) for b in row] for row in getattr(instr, t)]
    elif op == "AttnReductionInstr":
        s.update(output_is_unpadded=int(instr.output_is_unpadded),
                 ops=[{"src": [[_unblk(o), _unblk(l)] for o, l in r.src_buffers], "dst": [_unblk(r.dst_buffer[0]), _unblk(r.dst_buffer[1])]}
                      for r in instr.ops])
    elif op == "SumInstr":
        s.update(output_is_unpadded=int(instr.output_is_unpadded),
                 ops=[{"src": [_unblk(b) for b in r.src_buffers], "dst": _unblk(r.dst_buffer)} for r in instr.ops])
    elif op != "BarrierInstr":
        raise ValueError(f"unknown instruction {op}")
    return s


def plan_to_spec(plan):
    return dict(instructions=[instr_to_spec(i) for i in plan.instructions], n_nodes=int(plan.n_nodes),
                n_devices_per_node=int(plan.n_devices_per_node), node_id=int(plan.node_id),
                local_device_id=int(plan.local_device_id), n_stages=int(plan.n_stages),
                local_cu_seqlens=[int(x) for x in plan.local_cu_seqlens],
                buffer_info={k: [int(v.n_blocks), int(v.block_size), int(v.block_numel), int(v.dtype), list(v.buffer_shape),
                                 list(v.per_token_shape)] for k, v in plan.buffer_info.items()})
