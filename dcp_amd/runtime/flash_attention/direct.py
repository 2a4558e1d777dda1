"""Which copies of a plan the executor need not make.

A plan spells out every block movement: a ``MemcpyInstr`` gathers the device's own blocks from the
unpadded ``LOCAL_*`` tensors into padded ``BUFFER_*`` slots before the attention kernels read them
(reference ``_copy_input_to_local_buffer``, ``dcp/core/scheduler.py:870-892``), and the final
``AttnReductionInstr`` / ``SumInstr`` with ``output_is_unpadded=1`` moves results back
(``scheduler.py:1764-1940``).  Where such a movement is a plain copy -- a slot that holds nothing but
a local block and is read by attention kernels only; a partial output, dQ or summed dK/dV that a
single-source op scatters back unchanged -- the kernels can address the unpadded tensor itself: a
block table entry becomes a token offset (``local_cu_seqlens``) instead of a slot number, the stride
of a table entry a token instead of a block (``dcp_attn_fwd_strided`` / ``dcp_attn_bwd_strided``).
The bytes that reach ``LOCAL_OUT``, ``LOCAL_LSE``, ``LOCAL_dQ`` and ``LOCAL_dKV`` are the same: the
skipped operations are bit copies (and a sum that is rounded once is rounded once either way).

``analyse`` only looks at the instruction list; it changes nothing in the plan.  Plans that exchange
blocks with other devices are left alone (their slots are also read and written by the exchange).
"""

from __future__ import annotations

from collections import defaultdict
from dataclasses import dataclass, field
from typing import Dict, List, Set, Tuple

from dcp_amd.core.instructions import (
    AttnBackwardInstr,
    AttnInstr,
    AttnReductionInstr,
    BarrierInstr,
    BufferBlock,
    BufferType,
    CommLaunchInstr,
    CommWaitInstr,
    ExecutionPlan,
    MemcpyInstr,
    SumInstr,
)


@dataclass
class DirectPlan:
    """Per instruction index, what the executor does differently."""

    # MemcpyInstr: positions of the (src, dst) pairs that are not copied
    skip_pairs: Dict[int, Set[int]] = field(default_factory=dict)
    # AttnInstr / AttnBackwardInstr: operand name ("q", "kv", "out", "dq") -> per row, the index (q, out,
    # dq) or the list of indices (kv) of the LOCAL block(s) the kernel addresses instead of slots.
    # "out" of a forward instruction is where it WRITES; of a backward one where it reads out, lse, dout.
    operands: Dict[int, Dict[str, list]] = field(default_factory=dict)
    # AttnReductionInstr / SumInstr: positions of the ops that are not run
    skip_ops: Dict[int, Set[int]] = field(default_factory=dict)
    # SumInstr: op position -> the LOCAL block the sum is written to instead of its slot
    redirect_ops: Dict[int, Dict[int, BufferBlock]] = field(default_factory=dict)

    def anything(self) -> bool:
        return bool(self.skip_pairs or self.operands or self.skip_ops or self.redirect_ops)


_LOCAL_OF = {
    BufferType.BUFFER_Q: BufferType.LOCAL_Q,
    BufferType.BUFFER_KV: BufferType.LOCAL_KV,
    BufferType.BUFFER_OUT: BufferType.LOCAL_OUT,
    BufferType.BUFFER_LSE: BufferType.LOCAL_LSE,
    BufferType.BUFFER_dOUT: BufferType.LOCAL_dOUT,
}


def analyse(plan: ExecutionPlan) -> DirectPlan:
    result = DirectPlan()
    instrs = plan.instructions
    if any(isinstance(i, (CommLaunchInstr, CommWaitInstr, BarrierInstr)) for i in instrs):
        return result

    # A slot that holds a copy of a local block: (buffer type, slot) -> (memcpy index, pair position, source)
    origin: Dict[Tuple[str, int], Tuple[int, int, BufferBlock]] = {}
    # per copied pair: does every reader address it through an operand that can go to the source?
    pair_readers: Dict[Tuple[int, int], List[bool]] = defaultdict(list)
    all_pairs: Set[Tuple[int, int]] = set()
    # kernel outputs: (buffer type, slot) -> producer, and the readers of each produced block
    produced: Dict[Tuple[str, int], tuple] = {}
    readers: Dict[tuple, list] = defaultdict(list)

    def local_blocks(idx: int, blocks: List[BufferBlock]):
        """The local blocks behind ``blocks`` if every one of them is a fresh copy of the matching
        LOCAL_* type; the copied pairs get a reader each, direct or not."""
        hits = [origin.get((blk.buffer_type, blk.index)) for blk in blocks]
        ok = all(h is not None and h[2].buffer_type == _LOCAL_OF.get(blk.buffer_type) and h[2].n_tokens == blk.n_tokens
                 for h, blk in zip(hits, blocks))
        for h in hits:
            if h is not None:
                pair_readers[(h[0], h[1])].append(ok)
        return [h[2].index for h in hits] if ok else None

    def overwritten(blk: BufferBlock):
        origin.pop((blk.buffer_type, blk.index), None)
        produced.pop((blk.buffer_type, blk.index), None)

    candidates: Dict[int, Dict[str, list]] = defaultdict(dict)
    for idx, instr in enumerate(instrs):
        if isinstance(instr, MemcpyInstr):
            for pos, (src, dst) in enumerate(instr.src_dst_pairs):
                overwritten(dst)
                if _LOCAL_OF.get(dst.buffer_type) == src.buffer_type:
                    origin[(dst.buffer_type, dst.index)] = (idx, pos, src)
                    all_pairs.add((idx, pos))
        elif isinstance(instr, (AttnInstr, AttnBackwardInstr)):
            q_local = local_blocks(idx, [row[0] for row in instr.q_block_table])
            kv_rows = [local_blocks(idx, list(row)) for row in instr.kv_block_table]
            if q_local is not None:
                candidates[idx]["q"] = q_local
            if all(r is not None for r in kv_rows):
                candidates[idx]["kv"] = kv_rows
            elif any(r is not None for r in kv_rows):  # some rows could, the launch as a whole cannot
                for row in instr.kv_block_table:
                    for blk in row:
                        h = origin.get((blk.buffer_type, blk.index))
                        if h is not None:
                            pair_readers[(h[0], h[1])].append(False)
            if isinstance(instr, AttnInstr):
                for b, row in enumerate(instr.out_block_table):
                    for t in (BufferType.BUFFER_OUT, BufferType.BUFFER_LSE):
                        overwritten(BufferBlock(t, row[0].index, row[0].n_tokens))
                    produced[(BufferType.BUFFER_OUT, row[0].index)] = ("out", idx, b)
            else:
                # out, lse and dout of a row share the slot number: all three must be copies of the same local block
                per_type = [local_blocks(idx, [BufferBlock(t, row[0].index, row[0].n_tokens) for row in instr.out_block_table])
                            for t in (BufferType.BUFFER_OUT, BufferType.BUFFER_LSE, BufferType.BUFFER_dOUT)]
                if all(x is not None for x in per_type) and per_type[0] == per_type[1] == per_type[2]:
                    candidates[idx]["out"] = per_type[0]
                else:
                    for t in (BufferType.BUFFER_OUT, BufferType.BUFFER_LSE, BufferType.BUFFER_dOUT):
                        for row in instr.out_block_table:
                            h = origin.get((t, row[0].index))
                            if h is not None:
                                pair_readers[(h[0], h[1])].append(False)
                for b, row in enumerate(instr.dq_block_table):
                    overwritten(row[0])
                    produced[(row[0].buffer_type, row[0].index)] = ("dq", idx, b)
                for b, row in enumerate(instr.dkv_block_table):
                    for blk in row:
                        overwritten(blk)
                        produced[(blk.buffer_type, blk.index)] = ("dkv", idx, b)
        elif isinstance(instr, AttnReductionInstr):
            for pos, op in enumerate(instr.ops):
                for src_out, src_lse in op.src_buffers:
                    for blk in (src_out, src_lse):
                        h = origin.get((blk.buffer_type, blk.index))
                        if h is not None:
                            pair_readers[(h[0], h[1])].append(False)
                    who = produced.get((src_out.buffer_type, src_out.index))
                    if who is not None:
                        readers[who].append((idx, pos, len(op.src_buffers), bool(instr.output_is_unpadded)))
                if not instr.output_is_unpadded:
                    for blk in op.dst_buffer:
                        overwritten(blk)
                    produced[(op.dst_buffer[0].buffer_type, op.dst_buffer[0].index)] = ("merged", idx, pos)
        elif isinstance(instr, SumInstr):
            for pos, op in enumerate(instr.ops):
                for blk in op.src_buffers:
                    h = origin.get((blk.buffer_type, blk.index))
                    if h is not None:
                        pair_readers[(h[0], h[1])].append(False)
                    who = produced.get((blk.buffer_type, blk.index))
                    if who is not None:
                        readers[who].append((idx, pos, len(op.src_buffers), bool(instr.output_is_unpadded)))
                if not instr.output_is_unpadded:
                    overwritten(op.dst_buffer)
                    produced[(op.dst_buffer.buffer_type, op.dst_buffer.index)] = ("summed", idx, pos)
        else:  # an instruction this analysis does not know: leave the plan alone
            return DirectPlan()

    def sole_scatter(who):
        """The single-source, unpadded op that is the only reader of a produced block, if that is so."""
        r = readers.get(who, [])
        if len(r) == 1 and r[0][2] == 1 and r[0][3]:
            return r[0][0], r[0][1]
        return None

    for idx, instr in enumerate(instrs):
        if isinstance(instr, AttnInstr):
            hits = [sole_scatter(("out", idx, b)) for b in range(len(instr.out_block_table))]
            if hits and all(h is not None for h in hits):
                dsts = [instrs[j].ops[pos].dst_buffer for j, pos in hits]
                if all(d[0].buffer_type == BufferType.LOCAL_OUT and d[1].buffer_type == BufferType.LOCAL_LSE and
                       d[0].n_tokens == row[0].n_tokens for d, row in zip(dsts, instr.out_block_table)):
                    candidates[idx]["out"] = [d[0].index for d in dsts]
                    for j, pos in hits:
                        result.skip_ops.setdefault(j, set()).add(pos)
        elif isinstance(instr, AttnBackwardInstr):
            hits = [sole_scatter(("dq", idx, b)) for b in range(len(instr.dq_block_table))]
            if hits and all(h is not None for h in hits):
                dsts = [instrs[j].ops[pos].dst_buffer for j, pos in hits]
                if all(d.buffer_type == BufferType.LOCAL_dQ and d.n_tokens == row[0].n_tokens
                       for d, row in zip(dsts, instr.dq_block_table)):
                    candidates[idx]["dq"] = [d.index for d in dsts]
                    for j, pos in hits:
                        result.skip_ops.setdefault(j, set()).add(pos)
        elif isinstance(instr, SumInstr) and not instr.output_is_unpadded:
            # a sum into a slot whose only reader scatters it back unchanged: sum straight to where that goes
            for pos, op in enumerate(instr.ops):
                hit = sole_scatter(("summed", idx, pos))
                if hit is None:
                    continue
                dst = instrs[hit[0]].ops[hit[1]].dst_buffer
                if dst.buffer_type.startswith("Local") and dst.n_tokens == op.dst_buffer.n_tokens:
                    result.redirect_ops.setdefault(idx, {})[pos] = dst
                    result.skip_ops.setdefault(hit[0], set()).add(hit[1])

    result.operands = {idx: ops for idx, ops in candidates.items() if ops}
    for key in all_pairs:
        if all(pair_readers.get(key, [])):  # (a slot nobody reads is not worth filling either)
            result.skip_pairs.setdefault(key[0], set()).add(key[1])
    return result
