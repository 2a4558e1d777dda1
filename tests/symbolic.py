"""Symbolic run of execution plans: every buffer slot holds the *name* of what it contains
instead of numbers, so a plan can be checked for structure alone -- the approach of the
reference's DummyExecutor (tests/core/test_compiler.py:137-765: copies need a filled source and
equal block geometry, communication ops must pair up in order with equal block numel and dtype
(:24-125), attention tables must point at slots holding the right kind of block with the stated
lengths, range masks must stay inside the row's keys (:238-300), reductions must combine partials
of one block).  On top of that this checker follows *which* (q block, kv block) work units each
partial contains, so that at the end every output block must hold each of its units exactly once.

Names: ("Q"|"KV"|"OUT"|"LSE"|"dOUT", head block, sequence, block) for inputs;
("out"|"lse"|"dq", g, s, i, frozenset of kv blocks) and ("dkv", g_kv, s, j, frozenset of
(q head block, q block)) for results."""

from collections import defaultdict

import numpy as np

from dcp_amd.core.instructions import (AttnBackwardInstr, AttnInstr, AttnReductionInstr, BarrierInstr, CommLaunchInstr,
                                        CommWaitInstr, MemcpyInstr, SumInstr)
from dcp_amd.runtime.flash_attention.single_device import _block_overlaps

_LOCAL_INPUTS = {"LocalQ": "Q", "LocalKV": "KV", "LocalOut": "OUT", "LocalLSE": "LSE", "LocaldOut": "dOUT"}


class SymbolicDevice:
    def __init__(self, plan, layout, backward):
        self.plan, self.layout = plan, layout
        self.slots = {name: [None] * info.n_blocks for name, info in plan.buffer_info.items()}
        for i, (g, s, b, n) in enumerate(layout.q_blocks):
            self.slots["LocalQ"][i] = ("Q", g, s, b)
            if backward:
                for name in ("LocalOut", "LocalLSE", "LocaldOut"):
                    self.slots[name][i] = (_LOCAL_INPUTS[name], g, s, b)
        for i, (g, s, b, n) in enumerate(layout.kv_blocks):
            self.slots["LocalKV"][i] = ("KV", g, s, b)
        self.pending = {}
        # slot recycling: what every slot has held, in order, and how often each content was read,
        # so that a read of recycled contents can say what happened and the run can report reuse
        self.history = defaultdict(list)  # (buffer type, index) -> [name, ...]
        self.overwritten = 0              # writes that replaced contents of another block
        self.reads = defaultdict(int)     # (buffer type, index) -> reads of the present contents

    def get(self, block):
        assert block.index < len(self.slots[block.buffer_type]), f"{block} outside its buffer"
        self.reads[(block.buffer_type, block.index)] += 1
        return self.slots[block.buffer_type][block.index]

    def expect(self, block, name):
        """A read that must find ``name``: fails with the slot's history when the slot was recycled
        (overwritten while the block was still live) or never filled."""
        got = self.get(block)
        if got != name:
            past = self.history[(block.buffer_type, block.index)]
            why = "was overwritten while still live" if name in past else "was never put there"
            raise AssertionError(f"{block} should hold {name} but holds {got}: it {why} (slot history {past})")
        return got

    def put(self, block, name):
        assert block.index < len(self.slots[block.buffer_type]), f"{block} outside its buffer"
        old = self.slots[block.buffer_type][block.index]
        if old is not None and old[:4] != name[:4]:
            self.overwritten += 1
            # An input block (a gathered or received Q, KV, OUT, LSE or dOUT block) is put into a slot
            # for some instruction to read.  Replaced before anything has read it, its slot was given
            # away too early: the instruction it was meant for will find the newcomer (which a check
            # of what that instruction reads cannot tell when the newcomer looks just as plausible).
            if old[0] in _LOCAL_INPUTS.values() and block.buffer_type.startswith("Buffer"):
                assert self.reads[(block.buffer_type, block.index)] > 0, (
                    f"{block}: {old} is overwritten by {name} before any instruction read it "
                    f"(slot history {self.history[(block.buffer_type, block.index)]})")
        self.reads[(block.buffer_type, block.index)] = 0
        self.history[(block.buffer_type, block.index)].append(name)
        self.slots[block.buffer_type][block.index] = name


def _n_tok(layout, s, b):
    return min(layout.block_size, layout.raw_seqlens[s] - b * layout.block_size)


def _check_tokens(layout, block, name):
    assert name is not None, f"{block} is read before anything was put there"
    assert block.n_tokens == _n_tok(layout, name[2], name[3]), f"{block} holds {name}"


def _geometry(plan, a, b):
    ia, ib = plan.buffer_info[a.buffer_type], plan.buffer_info[b.buffer_type]
    return (ia.block_size, ia.block_numel, ia.dtype) == (ib.block_size, ib.block_numel, ib.dtype)


def _check_mask(instr):
    m = np.asarray(instr.attn_mask)
    total = sum(instr.seqlens_q)
    assert m.shape in ((2, total), (2, 2, total)), m.shape
    m = m.reshape(-1, 2, total)
    assert (m[:, 0] <= m[:, 1]).all() and (m >= 0).all()
    q0 = 0
    for b, n_q in enumerate(instr.seqlens_q):
        assert (m[:, :, q0 : q0 + n_q] <= instr.seqlens_kv[b]).all(), "a range reaches past the row's keys"
        q0 += n_q


def _attention(dev, instr, group_of, backward):
    lay, bs = dev.layout, dev.layout.block_size
    tables = [instr.seqlens_q, instr.seqlens_kv, instr.q_block_table, instr.kv_block_table, instr.out_block_table]
    tables += [instr.dq_block_table, instr.dkv_block_table] if backward else [instr.lse_block_table]
    assert len({len(t) for t in tables}) == 1, "tables of different lengths"
    _check_mask(instr)
    for b in range(len(instr.seqlens_q)):
        (q_block,) = instr.q_block_table[b]
        assert q_block.buffer_type == "BufferQ" and instr.seqlens_q[b] == bs
        q = dev.get(q_block)
        _check_tokens(lay, q_block, q)
        assert q[0] == "Q"
        _, g, s, i = q
        kv_ids = []
        assert instr.seqlens_kv[b] == bs * len(instr.kv_block_table[b])
        for kv_block in instr.kv_block_table[b]:
            assert kv_block.buffer_type == "BufferKV"
            kv = dev.get(kv_block)
            _check_tokens(lay, kv_block, kv)
            assert kv[0] == "KV" and kv[2] == s and kv[1] == group_of(g), f"row of {q} reads {kv}"
            kv_ids.append(kv[3])
        assert kv_ids == sorted(set(kv_ids)), "kv blocks of a row in sequence order, each once"
        (o_block,) = instr.out_block_table[b]
        assert o_block.buffer_type == "BufferOut" and o_block.n_tokens == q_block.n_tokens
        if not backward:
            (l_block,) = instr.lse_block_table[b]
            assert l_block.buffer_type == "BufferLSE" and l_block.index == o_block.index
            dev.put(o_block, ("out", g, s, i, frozenset(kv_ids)))
            dev.put(l_block, ("lse", g, s, i, frozenset(kv_ids)))
            continue
        dev.expect(o_block, ("OUT", g, s, i))
        dev.expect(type(o_block)("BufferLSE", o_block.index, o_block.n_tokens), ("LSE", g, s, i))
        dev.expect(type(o_block)("BufferdOut", o_block.index, o_block.n_tokens), ("dOUT", g, s, i))
        (dq_block,) = instr.dq_block_table[b]
        assert dq_block.buffer_type == "BufferdQ" and dq_block.n_tokens == q_block.n_tokens
        dev.put(dq_block, ("dq", g, s, i, frozenset(kv_ids)))
        assert len(instr.dkv_block_table[b]) == len(kv_ids)
        for j, kv_block, dkv_block in zip(kv_ids, instr.kv_block_table[b], instr.dkv_block_table[b]):
            assert dkv_block.buffer_type == "BufferdKV" and dkv_block.n_tokens == kv_block.n_tokens
            dev.put(dkv_block, ("dkv", group_of(g), s, j, frozenset({(g, i)})))


def _combine(names, what):
    assert all(n is not None and n[0] == what for n in names), f"expected {what} partials, got {names}"
    assert len({n[1:4] for n in names}) == 1, f"partials of different blocks combined: {names}"
    units = [u for n in names for u in n[4]]
    assert len(units) == len(set(units)), f"a work unit is counted twice in {names}"
    return (*names[0][:4], frozenset(units))


def run_symbolic(plans, layouts, n_devices_per_node, backward, mask, q_per_kv):
    """Runs the devices' plans in turns (a device stops at a wait whose peers have not launched)
    and returns the devices.  ``mask`` is the global range mask, for the final completeness check."""
    devs = [SymbolicDevice(p, lay, backward) for p, lay in zip(plans, layouts)]
    group_of = lambda g: g // q_per_kv
    mailbox = defaultdict(list)
    cursor = [0] * len(devs)
    while any(c < len(d.plan.instructions) for c, d in zip(cursor, devs)):
        progressed = False
        for rank, dev in enumerate(devs):
            while cursor[rank] < len(dev.plan.instructions):
                instr = dev.plan.instructions[cursor[rank]]
                if isinstance(instr, CommWaitInstr):
                    need = defaultdict(int)
                    for peer, _ in dev.pending[instr.key]:
                        need[peer] += 1
                    if any(len(mailbox[(peer, rank, instr.key)]) < n for peer, n in need.items()):
                        break
                    for peer, block in dev.pending.pop(instr.key):
                        name, n_tokens, geometry = mailbox[(peer, rank, instr.key)].pop(0)
                        info = dev.plan.buffer_info[block.buffer_type]
                        assert (info.block_numel, info.dtype) == geometry, "send and receive of different block numel or dtype"
                        assert n_tokens == block.n_tokens
                        dev.put(block, name)
                elif isinstance(instr, CommLaunchInstr):
                    assert instr.key not in dev.pending, "key launched twice without a wait"
                    recvs = []
                    for op in instr.comm_ops:
                        peer = op.peer[0] * n_devices_per_node + op.peer[1]
                        if op.comm_type == 0:
                            name = dev.get(op.buffer_block)
                            _check_tokens(dev.layout, op.buffer_block, name)
                            info = dev.plan.buffer_info[op.buffer_block.buffer_type]
                            mailbox[(rank, peer, instr.key)].append((name, op.buffer_block.n_tokens, (info.block_numel, info.dtype)))
                        else:
                            recvs.append((peer, op.buffer_block))
                    dev.pending[instr.key] = recvs
                elif isinstance(instr, MemcpyInstr):
                    for src, dst in instr.src_dst_pairs:
                        assert _geometry(dev.plan, src, dst) and src.n_tokens == dst.n_tokens
                        _check_tokens(dev.layout, src, dev.get(src))
                        dev.put(dst, dev.get(src))
                elif isinstance(instr, (AttnInstr, AttnBackwardInstr)):
                    _attention(dev, instr, group_of, isinstance(instr, AttnBackwardInstr))
                elif isinstance(instr, AttnReductionInstr):
                    for op in instr.ops:
                        out = _combine([dev.get(o) for o, _ in op.src_buffers], "out")
                        lse = _combine([dev.get(l) for _, l in op.src_buffers], "lse")
                        assert out[1:] == lse[1:]
                        dev.put(op.dst_buffer[0], out)
                        dev.put(op.dst_buffer[1], lse)
                elif isinstance(instr, SumInstr):
                    for op in instr.ops:
                        names = [dev.get(b) for b in op.src_buffers]
                        dev.put(op.dst_buffer, _combine(names, names[0][0]))
                else:
                    assert isinstance(instr, BarrierInstr), instr
                cursor[rank] += 1
                progressed = True
        assert progressed, "the plans wait for each other"
    assert all(len(v) == 0 for v in mailbox.values()), "blocks sent but never received"
    assert all(not d.pending for d in devs), "a launch without its wait"
    # every output block holds each of its work units exactly once
    lay0 = layouts[0]
    bs, off = lay0.block_size, np.concatenate(([0], np.cumsum(lay0.raw_seqlens)))
    m = np.asarray(mask)
    n_blocks = [(L + bs - 1) // bs for L in lay0.raw_seqlens]
    attended = {(s, i): frozenset(_block_overlaps(m[off[s] : off[s + 1]], i * bs, _n_tok(lay0, s, i), bs, n_blocks[s], lay0.raw_seqlens[s]))
                for s in range(len(n_blocks)) for i in range(n_blocks[s])}
    for dev in devs:
        for idx, (g, s, b, _) in enumerate(dev.layout.q_blocks):
            if not attended[(s, b)]:
                continue
            for name, what in ((("LocaldQ", "dq"),) if backward else (("LocalOut", "out"), ("LocalLSE", "lse"))):
                assert dev.slots[name][idx] == (what, g, s, b, attended[(s, b)]), (name, idx, dev.slots[name][idx])
        if backward:
            for idx, (gk, s, b, _) in enumerate(dev.layout.kv_blocks):
                want = frozenset((g, i) for g in range(gk * q_per_kv, (gk + 1) * q_per_kv)
                                 for i in range(n_blocks[s]) if b in attended[(s, i)])
                if want:
                    assert dev.slots["LocaldKV"][idx] == ("dkv", gk, s, b, want), (idx, dev.slots["LocaldKV"][idx])
    return devs
