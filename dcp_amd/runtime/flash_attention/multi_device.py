"""Plan builders for several devices with a fixed placement rule.

NOT the reference's planner (no hypergraph partitioning, no cost-model-driven placement, no slot
reuse): a simple context-parallel placement that produces per-device forward and backward
``ExecutionPlan``s with the same instruction structure the reference scheduler emits for a
device that exchanges blocks with others (``dcp/core/scheduler.py:894-1049`` input exchange,
``:1702-1762`` output exchange, ``:1764-1940`` final merges and sums), so that the
communication instructions can be run and checked.  ``build_multi_device_plans`` exchanges all
inputs at once; ``build_staged_multi_device_plans`` lets the stage packer group the work into
pipeline stages.  The placement:

* token block ``b`` of sequence ``s`` (its Q and its KV, every head block) lives on device
  ``(s + b) % n_devices``;
* the work unit (q block ``i``, kv block ``j``) of a sequence runs on the owner of the q block
  if ``i + j`` is even and on the owner of the kv block otherwise, so both kinds of traffic
  occur: KV (and Q) blocks travel to where they are multiplied, and partial results travel back
  -- (out, lse) partials to the q block's owner, which merges them, dQ partials to the q block's
  owner and dKV partials to the kv block's owner, which sum them;
* one input exchange (key ``S0``; ``S1``, ``S2``, ... when staged) and one output exchange
  (key ``O``) per pass.

Each device's LOCAL_* buffers hold its own blocks in (head block, sequence, block) order.
"""

from __future__ import annotations

from collections import defaultdict
from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch

from dcp_amd.core.instructions import (
    AttnBackwardInstr,
    AttnInstr,
    AttnReductionInstr,
    BufferBlock,
    BufferInfo,
    BufferType,
    CommLaunchInstr,
    CommOp,
    CommType,
    CommWaitInstr,
    DType,
    ExecutionPlan,
    MemcpyInstr,
    ReductionOp,
    SumInstr,
    SumOp,
)
from dcp_amd.core.serialization import torch_dtype_to_int
from dcp_amd.runtime.flash_attention.single_device import LocalLayout, _block_overlaps, _row_ranges, _Slots

Key = Tuple[int, int, int]  # (head block, sequence, token block)


class _Placement:
    """What both builders share: the head blocking, the block grid of every sequence, who owns
    which token block, each rank's LOCAL layout and the buffer descriptions."""

    def __init__(self, n_nodes, n_devices_per_node, raw_seqlens, block_size, n_heads, n_query_groups, head_dim,
                 head_block_size, attn_mask, dtype):
        self.n_nodes, self.n_devices_per_node = n_nodes, n_devices_per_node
        self.n_dev = n_nodes * n_devices_per_node
        self.raw_seqlens = [int(x) for x in raw_seqlens]
        self.block_size, self.head_dim = block_size, head_dim
        group = n_heads // n_query_groups
        assert n_heads % n_query_groups == 0 and n_heads % head_block_size == 0
        if group > 1:
            assert head_block_size <= group and group % head_block_size == 0
        self.hb = head_block_size
        self.hkv = 1 if group > 1 else head_block_size
        self.n_hb_q, self.n_hb_kv = n_heads // self.hb, n_query_groups // self.hkv
        self.q_per_kv = self.n_hb_q // self.n_hb_kv  # q head blocks sharing one kv head block
        self.mask_np = attn_mask.cpu().numpy()
        assert self.mask_np.shape[0] == sum(self.raw_seqlens)
        self.seq_off = np.concatenate(([0], np.cumsum(self.raw_seqlens)))
        self.n_blocks_of = [(L + block_size - 1) // block_size for L in self.raw_seqlens]
        self.wire_dtype = torch_dtype_to_int(dtype)
        self.elem_bytes = 4 if dtype == torch.float32 else 2
        self.q_tok_shape, self.kv_tok_shape = (self.hb, head_dim), (2, self.hkv, head_dim)
        self.q_numel, self.kv_numel = block_size * self.hb * head_dim, block_size * 2 * self.hkv * head_dim
        # LOCAL order on every rank: (head block, sequence, block) over the blocks it owns
        self.layouts: List[LocalLayout] = []
        self.local_q: List[Dict[Key, int]] = []
        self.local_kv: List[Dict[Key, int]] = []
        for r in range(self.n_dev):
            lay = LocalLayout(self.raw_seqlens, block_size, n_heads, n_query_groups, head_dim, self.hb, self.hkv)
            iq, ikv = {}, {}
            for index, n_hb, blocks in ((iq, self.n_hb_q, lay.q_blocks), (ikv, self.n_hb_kv, lay.kv_blocks)):
                for g in range(n_hb):
                    for s in range(len(self.raw_seqlens)):
                        for b in range(self.n_blocks_of[s]):
                            if self.owner(s, b) == r:
                                index[(g, s, b)] = len(blocks)
                                blocks.append((g, s, b, self.n_tok(s, b)))
            cu = [0]
            for _, _, _, n in lay.q_blocks:
                cu.append(cu[-1] + n)
            lay.local_cu_seqlens = cu
            self.layouts.append(lay)
            self.local_q.append(iq)
            self.local_kv.append(ikv)

    def n_tok(self, s, b):
        return min(self.block_size, self.raw_seqlens[s] - b * self.block_size)

    def owner(self, s, b) -> int:
        """Rank that holds token block b of sequence s."""
        return (s + b) % self.n_dev

    def device(self, rank) -> Tuple[int, int]:
        return divmod(rank, self.n_devices_per_node)

    def unit_rank(self, s, i, j) -> int:
        """Rank that computes (q block i, kv block j) of sequence s."""
        return self.owner(s, i) if (i + j) % 2 == 0 else self.owner(s, j)

    def attended_blocks(self, s, i) -> List[int]:
        seq_mask = self.mask_np[self.seq_off[s] : self.seq_off[s + 1]]
        return _block_overlaps(seq_mask, i * self.block_size, self.n_tok(s, i), self.block_size, self.n_blocks_of[s],
                               self.raw_seqlens[s])

    def rows_mask(self, rows):
        """Range planes of attention rows ``[((g, s, i), kv block ids)]`` in their concatenated kv coordinates."""
        planes = []
        for (g, s, i), ids in rows:
            seq_mask = self.mask_np[self.seq_off[s] : self.seq_off[s + 1]]
            planes.append(_row_ranges(seq_mask, i * self.block_size, self.n_tok(s, i), self.block_size, ids,
                                      [self.n_tok(s, j) for j in ids]))
        t = torch.from_numpy(np.concatenate(planes, axis=2))
        return t[0] if t.shape[0] == 1 else t

    def block(self, buffer_type, index, key: Key) -> BufferBlock:
        return BufferBlock(buffer_type, index, self.n_tok(key[1], key[2]))

    def local_info(self, n_blocks, total, tok_shape, numel):
        return BufferInfo(n_blocks, self.block_size, numel, self.wire_dtype, (total, *tok_shape), tok_shape)

    def slot_info(self, n_blocks, tok_shape, numel):
        n = max(n_blocks, 1)
        return BufferInfo(n, self.block_size, numel, self.wire_dtype, (n, self.block_size, *tok_shape), tok_shape)

    def lse_slot_info(self, n_blocks):
        n = max(n_blocks, 1)
        return BufferInfo(n, self.block_size, self.block_size * self.hb, DType.FLOAT32, (self.hb, n, self.block_size), (1,))

    def buffer_info(self, r, n_q, n_kv, n_out, backward_slots=None):
        """Buffer descriptions of rank r: ``n_q`` / ``n_kv`` / ``n_out`` padded slots; in the
        backward ``backward_slots = (n_dq, n_dkv)`` and BUFFER_OUT / LSE / dOUT share ``n_out``."""
        lay = self.layouts[r]
        total_q, total_kv = lay.local_cu_seqlens[-1], sum(n for _, _, _, n in lay.kv_blocks)
        nq, nkv = len(lay.q_blocks), len(lay.kv_blocks)
        info = {
            BufferType.LOCAL_Q: self.local_info(nq, total_q, self.q_tok_shape, self.q_numel),
            BufferType.LOCAL_KV: self.local_info(nkv, total_kv, self.kv_tok_shape, self.kv_numel),
            BufferType.LOCAL_OUT: self.local_info(nq, total_q, self.q_tok_shape, self.q_numel),
            BufferType.LOCAL_LSE: BufferInfo(nq, self.block_size, self.block_size * self.hb, DType.FLOAT32, (self.hb, total_q), (1,)),
            BufferType.BUFFER_Q: self.slot_info(n_q, self.q_tok_shape, self.q_numel),
            BufferType.BUFFER_KV: self.slot_info(n_kv, self.kv_tok_shape, self.kv_numel),
            BufferType.BUFFER_OUT: self.slot_info(n_out, self.q_tok_shape, self.q_numel),
            BufferType.BUFFER_LSE: self.lse_slot_info(n_out),
        }
        if backward_slots is not None:
            n_dq, n_dkv = backward_slots
            info.update({
                BufferType.LOCAL_dOUT: self.local_info(nq, total_q, self.q_tok_shape, self.q_numel),
                BufferType.LOCAL_dQ: self.local_info(nq, total_q, self.q_tok_shape, self.q_numel),
                BufferType.LOCAL_dKV: self.local_info(nkv, total_kv, self.kv_tok_shape, self.kv_numel),
                BufferType.BUFFER_dOUT: self.slot_info(n_out, self.q_tok_shape, self.q_numel),
                BufferType.BUFFER_dQ: self.slot_info(n_dq, self.q_tok_shape, self.q_numel),
                BufferType.BUFFER_dKV: self.slot_info(n_dkv, self.kv_tok_shape, self.kv_numel),
            })
        return info


_BY_SEQUENCE = lambda kv: (kv[0][1], kv[0][0], kv[0][2])  # rows in (sequence, head block, block) order


def build_multi_device_plans(
    n_nodes: int,
    n_devices_per_node: int,
    raw_seqlens: Sequence[int],
    block_size: int,
    n_heads: int,
    n_query_groups: int,
    head_dim: int,
    head_block_size: int,
    attn_mask: torch.Tensor,
    dtype: torch.dtype = torch.bfloat16,
):
    """Returns ``(fw_plans, bw_plans, layouts)``, one entry per rank
    (``rank = node * n_devices_per_node + device``).  ``attn_mask`` as for
    ``build_single_device_plans``.  ``layouts[rank]`` maps between global tensors and the rank's
    LOCAL buffers; blocks a rank does not own come out of its ``from_local_*`` as zeros, so the
    global result is the sum over ranks."""
    pl = _Placement(n_nodes, n_devices_per_node, raw_seqlens, block_size, n_heads, n_query_groups, head_dim,
                    head_block_size, attn_mask, dtype)
    n_dev, q_per_kv, layouts, local_q, local_kv = pl.n_dev, pl.q_per_kv, pl.layouts, pl.local_q, pl.local_kv
    owner, peer_of, blk = pl.owner, pl.device, pl.block

    # ---- where every work unit runs: rows[rank][(g, s, i)] = kv block ids ----------------
    rows: List[Dict[Key, List[int]]] = [defaultdict(list) for _ in range(n_dev)]
    for s in range(len(pl.raw_seqlens)):
        for i in range(pl.n_blocks_of[s]):
            for j in pl.attended_blocks(s, i):
                for g in range(pl.n_hb_q):
                    rows[pl.unit_rank(s, i, j)][(g, s, i)].append(j)

    def ordered_rows(r):
        return sorted(rows[r].items(), key=_BY_SEQUENCE)

    def row_mask(r):
        return pl.rows_mask(ordered_rows(r))

    # A transfer list is built once, in one order, and read by both ends: entry
    # (src rank, dst rank, what, key) becomes a SEND in src's launch and a RECV in dst's.
    def exchange(transfers, send_block, recv_block):
        ops = [[] for _ in range(n_dev)]
        for src, dst, what, key in transfers:
            ops[src].append(CommOp(CommType.SEND, peer_of(dst), send_block(src, dst, what, key)))
            ops[dst].append(CommOp(CommType.RECV, peer_of(src), recv_block(src, dst, what, key)))
        return ops

    # ---- inputs every rank needs -------------------------------------------------------------
    need_q = [sorted(rows[r].keys(), key=lambda k: (k[1], k[0], k[2])) for r in range(n_dev)]
    need_kv = []
    for r in range(n_dev):
        ks = {(g // q_per_kv, s, j) for (g, s, i), ids in rows[r].items() for j in ids}
        need_kv.append(sorted(ks, key=lambda k: (k[1], k[0], k[2])))

    def input_phase(r, with_out):
        """Slots, the gather of own blocks and the S0 transfer list entries that end on r."""
        slots = {t: _Slots() for t in ("q", "kv", "o")}
        buf_q = {k: slots["q"].take() for k in need_q[r]}
        buf_kv = {k: slots["kv"].take() for k in need_kv[r]}
        buf_o = {k: slots["o"].take() for k in need_q[r]} if with_out else {}
        pairs, incoming = [], []
        for k, slot in buf_q.items():
            o = owner(k[1], k[2])
            if o == r:
                pairs.append((blk(BufferType.LOCAL_Q, local_q[r][k], k), blk(BufferType.BUFFER_Q, slot, k)))
            else:
                incoming.append((o, r, "q", k))
        for k, slot in buf_kv.items():
            o = owner(k[1], k[2])
            if o == r:
                pairs.append((blk(BufferType.LOCAL_KV, local_kv[r][k], k), blk(BufferType.BUFFER_KV, slot, k)))
            else:
                incoming.append((o, r, "kv", k))
        for k, slot in buf_o.items():
            o = owner(k[1], k[2])
            if o == r:
                li = local_q[r][k]
                pairs.append((blk(BufferType.LOCAL_OUT, li, k), blk(BufferType.BUFFER_OUT, slot, k)))
                pairs.append((blk(BufferType.LOCAL_LSE, li, k), blk(BufferType.BUFFER_LSE, slot, k)))
                pairs.append((blk(BufferType.LOCAL_dOUT, li, k), blk(BufferType.BUFFER_dOUT, slot, k)))
            else:
                incoming += [(o, r, "out", k), (o, r, "lse", k), (o, r, "dout", k)]
        return slots, buf_q, buf_kv, buf_o, pairs, incoming

    _LOCAL_OF = {"q": BufferType.LOCAL_Q, "kv": BufferType.LOCAL_KV, "out": BufferType.LOCAL_OUT,
                 "lse": BufferType.LOCAL_LSE, "dout": BufferType.LOCAL_dOUT}
    _SLOT_OF = {"q": BufferType.BUFFER_Q, "kv": BufferType.BUFFER_KV, "out": BufferType.BUFFER_OUT,
                "lse": BufferType.BUFFER_LSE, "dout": BufferType.BUFFER_dOUT}

    def build(with_backward):
        phase = [input_phase(r, with_backward) for r in range(n_dev)]
        transfers = [t for r in range(n_dev) for t in phase[r][5]]

        def send_input(src, dst, what, k):  # straight from the owner's unpadded buffer
            index = local_kv[src][k] if what == "kv" else local_q[src][k]
            return blk(_LOCAL_OF[what], index, k)

        def recv_input(src, dst, what, k):
            table = {"q": phase[dst][1], "kv": phase[dst][2]}.get(what, phase[dst][3])
            return blk(_SLOT_OF[what], table[k], k)

        s0 = exchange(transfers, send_input, recv_input)
        plans = []
        # results: slot bookkeeping per rank, then the O exchange, then the final instructions
        state = []
        for r in range(n_dev):
            slots, buf_q, buf_kv, buf_o, pairs, _ = phase[r]
            instrs = [MemcpyInstr(pairs)] if pairs else []
            if s0[r]:
                instrs += [CommLaunchInstr("S0", s0[r]), CommWaitInstr("S0")]
            my_rows = ordered_rows(r)
            res = {t: _Slots() for t in ("out", "dq", "dkv")}
            st = dict(instrs=instrs, res=res, partial_out={}, partial_dq={}, dkv_sum={}, outgoing=[])
            if my_rows:
                seq_q = [block_size] * len(my_rows)
                seq_kv = [block_size * len(ids) for _, ids in my_rows]
                q_tab = [[blk(BufferType.BUFFER_Q, buf_q[k], k)] for k, _ in my_rows]
                kv_tab = [[blk(BufferType.BUFFER_KV, buf_kv[(k[0] // q_per_kv, k[1], j)], (0, k[1], j)) for j in ids]
                          for k, ids in my_rows]
                if not with_backward:
                    out_tab, lse_tab = [], []
                    for k, _ in my_rows:
                        slot = res["out"].take()
                        st["partial_out"][k] = slot
                        out_tab.append([blk(BufferType.BUFFER_OUT, slot, k)])
                        lse_tab.append([blk(BufferType.BUFFER_LSE, slot, k)])
                        if owner(k[1], k[2]) != r:
                            st["outgoing"] += [(r, owner(k[1], k[2]), "out", k), (r, owner(k[1], k[2]), "lse", k)]
                    instrs.append(AttnInstr(0, seq_q, seq_kv, block_size, max(seq_kv), row_mask(r),
                                            q_tab, kv_tab, out_tab, lse_tab))
                else:
                    o_tab = [[blk(BufferType.BUFFER_OUT, buf_o[k], k)] for k, _ in my_rows]
                    dq_tab, dkv_tab = [], []
                    replicas = defaultdict(list)
                    for k, ids in my_rows:
                        slot = res["dq"].take()
                        st["partial_dq"][k] = slot
                        dq_tab.append([blk(BufferType.BUFFER_dQ, slot, k)])
                        if owner(k[1], k[2]) != r:
                            st["outgoing"].append((r, owner(k[1], k[2]), "dq", k))
                        row = []
                        for j in ids:
                            slot = res["dkv"].take()
                            kk = (k[0] // q_per_kv, k[1], j)
                            replicas[kk].append(slot)
                            row.append(blk(BufferType.BUFFER_dKV, slot, kk))
                        dkv_tab.append(row)
                    instrs.append(AttnBackwardInstr(0, seq_q, seq_kv, block_size, max(seq_kv), row_mask(r),
                                                    q_tab, kv_tab, o_tab, dq_tab, dkv_tab))
                    presum = [SumOp([blk(BufferType.BUFFER_dKV, s_, kk) for s_ in sl], blk(BufferType.BUFFER_dKV, sl[0], kk))
                              for kk, sl in replicas.items() if len(sl) > 1]
                    if presum:
                        instrs.append(SumInstr(presum, output_is_unpadded=0))
                    for kk, sl in sorted(replicas.items(), key=lambda kv: (kv[0][1], kv[0][0], kv[0][2])):
                        st["dkv_sum"][kk] = sl[0]
                        if owner(kk[1], kk[2]) != r:
                            st["outgoing"].append((r, owner(kk[1], kk[2]), "dkv", kk))
            state.append(st)

        # the O exchange: partial results go to the owners of the blocks they belong to
        arrivals = [defaultdict(list) for _ in range(n_dev)]  # dst: (what, key) -> [slot]
        out_transfers = [t for r in range(n_dev) for t in state[r]["outgoing"]]
        recv_slot = {}
        for src, dst, what, k in out_transfers:
            if what == "lse":  # shares the slot index of its out block
                recv_slot[(src, dst, what, k)] = recv_slot[(src, dst, "out", k)]
                continue
            slot = state[dst]["res"]["out" if what == "out" else what].take()
            recv_slot[(src, dst, what, k)] = slot
            arrivals[dst][(what, k)].append(slot)
        _RES = {"out": BufferType.BUFFER_OUT, "lse": BufferType.BUFFER_LSE, "dq": BufferType.BUFFER_dQ, "dkv": BufferType.BUFFER_dKV}

        def send_result(src, dst, what, k):
            table = {"out": "partial_out", "lse": "partial_out", "dq": "partial_dq", "dkv": "dkv_sum"}[what]
            return blk(_RES[what], state[src][table][k], k)

        def recv_result(src, dst, what, k):
            return blk(_RES[what], recv_slot[(src, dst, what, k)], k)

        o_ops = exchange(out_transfers, send_result, recv_result)
        for r in range(n_dev):
            st, lay = state[r], layouts[r]
            instrs = st["instrs"]
            if o_ops[r]:
                instrs += [CommLaunchInstr("O", o_ops[r]), CommWaitInstr("O")]
            slots = phase[r][0]
            if not with_backward:
                ops = []
                for k, li in local_q[r].items():
                    srcs = ([st["partial_out"][k]] if k in st["partial_out"] else []) + arrivals[r][("out", k)]
                    if srcs:
                        ops.append(ReductionOp([(blk(BufferType.BUFFER_OUT, s_, k), blk(BufferType.BUFFER_LSE, s_, k)) for s_ in srcs],
                                               (blk(BufferType.LOCAL_OUT, li, k), blk(BufferType.LOCAL_LSE, li, k))))
                if ops:
                    instrs.append(AttnReductionInstr(ops, output_is_unpadded=1))
                info = pl.buffer_info(r, slots["q"].n, slots["kv"].n, st["res"]["out"].n)
            else:
                ops = []
                for k, li in local_q[r].items():
                    srcs = ([st["partial_dq"][k]] if k in st["partial_dq"] else []) + arrivals[r][("dq", k)]
                    if srcs:
                        ops.append(SumOp([blk(BufferType.BUFFER_dQ, s_, k) for s_ in srcs], blk(BufferType.LOCAL_dQ, li, k)))
                if ops:
                    instrs.append(SumInstr(ops, output_is_unpadded=1))
                ops = []
                for k, li in local_kv[r].items():
                    srcs = ([st["dkv_sum"][k]] if k in st["dkv_sum"] else []) + arrivals[r][("dkv", k)]
                    if srcs:
                        ops.append(SumOp([blk(BufferType.BUFFER_dKV, s_, k) for s_ in srcs], blk(BufferType.LOCAL_dKV, li, k)))
                if ops:
                    instrs.append(SumInstr(ops, output_is_unpadded=1))
                info = pl.buffer_info(r, slots["q"].n, slots["kv"].n, slots["o"].n, (st["res"]["dq"].n, st["res"]["dkv"].n))
            node, dev = peer_of(r)
            plans.append(ExecutionPlan(instrs, n_nodes, n_devices_per_node, node, dev, 1, lay.local_cu_seqlens, info))
        return plans

    return build(False), build(True), layouts


def build_staged_multi_device_plans(
    n_nodes: int,
    n_devices_per_node: int,
    raw_seqlens: Sequence[int],
    block_size: int,
    n_heads: int,
    n_query_groups: int,
    head_dim: int,
    head_block_size: int,
    attn_mask: torch.Tensor,
    dtype: torch.dtype = torch.bfloat16,
    n_stages: int = 2,
    disable_two_phase_comm: bool = False,
):
    """The same placement as ``build_multi_device_plans``, but the work units are grouped into
    pipeline stages by the stage packer (``dcp_amd.core.pipeline.generate_pipelines_n_stages``):
    stage 0 holds what needs no transfer, the blocks of stage k+1 travel (key ``S{k+1}``) while
    stage k is computed, and a remote block wanted by several devices of a node is received by
    one of them and forwarded inside the node on the second-phase stream (key ``S{k+1}P2``), in
    the instruction order of ``dcp/core/scheduler.py:894-1049``.  A stage's partial of a block that
    already has one on the device is folded into the older one right after the stage (merge for
    out / LSE, sum for dQ; a kv block's private dK/dV replicas are summed into the first) and its
    slot is returned (``scheduler.py:1324-1363,1656-1700``); the devices' partials meet at the owner
    of their block through the output exchange ``O``.
    Input slots are recycled as in the reference's scheduler (``scheduler.py:826-857,2167-2199``
    with the first-free rule of ``block_table.py:434-460``): an input block is live on a device
    from the first to the last stage that uses it there (a work unit reads it, it arrives for
    that stage, or it is sent for the next one), its slot is returned after the last such stage
    has been computed, and blocks that arrive later take the lowest free slot.
    Returns ``(fw_plans, bw_plans, layouts)`` as the unstaged builder."""
    from types import SimpleNamespace

    from dcp_amd.core.pipeline import generate_pipelines_n_stages

    pl = _Placement(n_nodes, n_devices_per_node, raw_seqlens, block_size, n_heads, n_query_groups, head_dim,
                    head_block_size, attn_mask, dtype)
    n_dev, n_hb_q, n_hb_kv, q_per_kv, layouts, n_tok = pl.n_dev, pl.n_hb_q, pl.n_hb_kv, pl.q_per_kv, pl.layouts, pl.n_tok
    devices = [pl.device(r) for r in range(n_dev)]
    # blocks a rank owns: ("q" | "kv", head block, sequence, block) -> LOCAL index
    local_index = [{**{("q", *k): v for k, v in pl.local_q[r].items()}, **{("kv", *k): v for k, v in pl.local_kv[r].items()}}
                   for r in range(n_dev)]

    def owner(s, b):
        return devices[pl.owner(s, b)]

    def rank_of(device):
        return device[0] * n_devices_per_node + device[1]

    _LOCAL = {"Q": BufferType.LOCAL_Q, "KV": BufferType.LOCAL_KV, "OUT": BufferType.LOCAL_OUT,
              "LSE": BufferType.LOCAL_LSE, "dOUT": BufferType.LOCAL_dOUT}
    _SLOT = {"Q": BufferType.BUFFER_Q, "KV": BufferType.BUFFER_KV, "OUT": BufferType.BUFFER_OUT,
             "LSE": BufferType.BUFFER_LSE, "dOUT": BufferType.BUFFER_dOUT}

    def build(is_bw):
        # ---- the planning problem: data blocks, work units, where they are ----------------
        inputs: List[Tuple[str, int, int, int]] = []  # (type, head block, sequence, block)
        input_id: Dict[Tuple[str, int, int, int], int] = {}

        def add_input(kind, g, s, b):
            input_id[(kind, g, s, b)] = len(inputs)
            inputs.append((kind, g, s, b))

        for s in range(len(pl.raw_seqlens)):
            for b in range(pl.n_blocks_of[s]):
                for g in range(n_hb_q):
                    add_input("Q", g, s, b)
                    if is_bw:
                        for kind in ("OUT", "LSE", "dOUT"):
                            add_input(kind, g, s, b)
                for g in range(n_hb_kv):
                    add_input("KV", g, s, b)
        q_bytes, kv_bytes = pl.q_numel * pl.elem_bytes, pl.kv_numel * pl.elem_bytes
        size_of = {"Q": q_bytes, "OUT": q_bytes, "dOUT": q_bytes, "KV": kv_bytes, "LSE": block_size * pl.hb * 4}
        input_sizes = [float(size_of[kind]) for kind, _, _, _ in inputs]
        input_device = {i: owner(s, b) for i, (_, _, s, b) in enumerate(inputs)}
        units: List[Tuple[int, int, int, int]] = []  # (q head block, sequence, q block, kv block)
        unit_inputs, unit_device, unit_cost = [], {}, []
        for s in range(len(pl.raw_seqlens)):
            for i in range(pl.n_blocks_of[s]):
                for j in pl.attended_blocks(s, i):
                    for g in range(n_hb_q):
                        w = len(units)
                        units.append((g, s, i, j))
                        ins = [input_id[("Q", g, s, i)], input_id[("KV", g // q_per_kv, s, j)]]
                        if is_bw:
                            ins += [input_id[(kind, g, s, i)] for kind in ("OUT", "LSE", "dOUT")]
                        unit_inputs.append(ins)
                        unit_device[w] = devices[pl.unit_rank(s, i, j)]
                        unit_cost.append(float(n_tok(s, i) * n_tok(s, j)))
        meta = {i: SimpleNamespace(type=kind) for i, (kind, _, _, _) in enumerate(inputs)}
        work_per_stage, first_phase, second_phase = generate_pipelines_n_stages(
            n_stages, set(devices), unit_cost, unit_inputs, meta, input_sizes, unit_device, input_device, is_bw,
            disable_two_phase_comm=disable_two_phase_comm)

        # ---- how long a device needs each input block (scheduler.py:826-857) --------------------
        last_live: List[Dict[int, int]] = [defaultdict(int) for _ in range(n_dev)]  # input id -> last stage it is live in
        for stage_id, stage in enumerate(work_per_stage):
            for d, ws in stage.items():
                for w in ws:
                    for i in unit_inputs[w]:
                        last_live[rank_of(d)][i] = max(last_live[rank_of(d)][i], stage_id)
        for phase in (first_phase, second_phase):
            for stage_id, per_dst in enumerate(phase):
                for dst, comms in per_dst.items():
                    for i, src in comms:
                        last_live[rank_of(dst)][i] = max(last_live[rank_of(dst)][i], stage_id)
                        last_live[rank_of(src)][i] = max(last_live[rank_of(src)][i], stage_id - 1)

        # ---- per device: where each block it holds sits ----------------------------------------
        slots = [{t: _Slots() for t in ("Q", "KV", "O", "out", "dq", "dkv")} for _ in range(n_dev)]
        held: List[Dict[int, BufferBlock]] = [{} for _ in range(n_dev)]  # input id -> the block to read it from
        o_slot: List[Dict[Key, int]] = [{} for _ in range(n_dev)]         # OUT / LSE / dOUT of a q block share a slot index

        def block_of(i, buffer_type, index):
            _, _, s, b = inputs[i]
            return BufferBlock(buffer_type, index, n_tok(s, b))

        def take_slot(r, i):
            kind, g, s, b = inputs[i]
            if kind in ("OUT", "LSE", "dOUT"):
                if (g, s, b) not in o_slot[r]:
                    o_slot[r][(g, s, b)] = slots[r]["O"].take()
                return o_slot[r][(g, s, b)]
            return slots[r][kind].take()

        def local_block(r, i):
            kind, g, s, b = inputs[i]
            return block_of(i, _LOCAL[kind], local_index[r][("kv" if kind == "KV" else "q", g, s, b)])

        def release_dead_inputs(r, stage_id):
            """After stage ``stage_id`` has been computed: the slots of the inputs the device needs no longer
            (scheduler.py:2167-2199).  OUT / LSE / dOUT of a q block live and die together and share one index."""
            for i in [i for i in held[r] if last_live[r][i] <= stage_id]:
                kind, g, s, b = inputs[i]
                block = held[r].pop(i)
                if kind in ("OUT", "LSE", "dOUT"):
                    if not any(inputs[j][0] in ("OUT", "LSE", "dOUT") and inputs[j][1:] == (g, s, b) for j in held[r]):
                        slots[r]["O"].free(o_slot[r].pop((g, s, b)))
                else:
                    slots[r][kind].free(block.index)

        instrs: List[list] = [[] for _ in range(n_dev)]
        used = [set() for _ in range(n_dev)]  # inputs some work unit on the device reads
        for stage in work_per_stage:
            for d, ws in stage.items():
                for w in ws:
                    used[rank_of(d)].update(unit_inputs[w])
        for r in range(n_dev):
            pairs = []
            for i in sorted(used[r]):
                if rank_of(input_device[i]) == r:
                    dst = block_of(i, _SLOT[inputs[i][0]], take_slot(r, i))
                    pairs.append((local_block(r, i), dst))
                    held[r][i] = dst
            if pairs:
                instrs[r].append(MemcpyInstr(pairs))

        def source_block(r, i):
            """What a device sends for input i: its own unpadded block, or the slot it received it in."""
            return local_block(r, i) if rank_of(input_device[i]) == r else held[r][i]

        def exchange_ops(transfers):
            """transfers: (src rank, dst rank, input id) in one global order -> ops per rank."""
            ops = [[] for _ in range(n_dev)]
            arrivals = []
            for src, dst, i in transfers:
                ops[src].append(CommOp(CommType.SEND, devices[dst], source_block(src, i)))
                slot = block_of(i, _SLOT[inputs[i][0]], take_slot(dst, i))
                ops[dst].append(CommOp(CommType.RECV, devices[src], slot))
                arrivals.append((dst, i, slot))
            return ops, arrivals

        partial_out = [defaultdict(list) for _ in range(n_dev)]  # q block key -> partial slots on this device
        partial_dq = [defaultdict(list) for _ in range(n_dev)]
        replicas = [defaultdict(list) for _ in range(n_dev)]     # kv block key -> private dKV slots

        def compute(r, stage_id):
            ws = sorted(work_per_stage[stage_id].get(devices[r], ()))
            if not ws:
                return
            rows = defaultdict(list)
            for w in ws:
                g, s, i, j = units[w]
                rows[(g, s, i)].append(j)
            rows = sorted(((k, sorted(ids)) for k, ids in rows.items()), key=_BY_SEQUENCE)
            m = pl.rows_mask(rows)
            seq_q = [block_size] * len(rows)
            seq_kv = [block_size * len(ids) for _, ids in rows]
            q_tab = [[held[r][input_id[("Q", *k)]]] for k, _ in rows]
            kv_tab = [[held[r][input_id[("KV", k[0] // q_per_kv, k[1], j)]] for j in ids] for k, ids in rows]

            def row_block(buffer_type, slot, k):
                return BufferBlock(buffer_type, slot, n_tok(k[1], k[2]))

            if not is_bw:
                out_tab, lse_tab, folds = [], [], []
                for k, _ in rows:
                    slot = slots[r]["out"].take()
                    out_tab.append([row_block(BufferType.BUFFER_OUT, slot, k)])
                    lse_tab.append([row_block(BufferType.BUFFER_LSE, slot, k)])
                    if partial_out[r][k]:
                        # the block has a partial from an earlier stage: fold the new one into it and
                        # give the new one's slot back (scheduler.py:1324-1363)
                        old = partial_out[r][k][0]
                        pair = lambda sl: (row_block(BufferType.BUFFER_OUT, sl, k), row_block(BufferType.BUFFER_LSE, sl, k))
                        folds.append((ReductionOp([pair(old), pair(slot)], pair(old)), slot))
                    else:
                        partial_out[r][k].append(slot)
                instrs[r].append(AttnInstr(stage_id, seq_q, seq_kv, block_size, max(seq_kv), m, q_tab, kv_tab, out_tab, lse_tab))
                if folds:
                    instrs[r].append(AttnReductionInstr([op for op, _ in folds], output_is_unpadded=0))
                    for _, slot in folds:
                        slots[r]["out"].free(slot)
                return
            o_tab = [[row_block(BufferType.BUFFER_OUT, o_slot[r][k], k)] for k, _ in rows]
            dq_tab, dkv_tab, touched = [], [], []
            for k, ids in rows:
                slot = slots[r]["dq"].take()
                partial_dq[r][k].append(slot)
                dq_tab.append([row_block(BufferType.BUFFER_dQ, slot, k)])
                row = []
                for j in ids:
                    kk = (k[0] // q_per_kv, k[1], j)
                    slot = slots[r]["dkv"].take()
                    if kk not in touched:
                        touched.append(kk)
                    replicas[r][kk].append(slot)
                    row.append(row_block(BufferType.BUFFER_dKV, slot, kk))
                dkv_tab.append(row)
            instrs[r].append(AttnBackwardInstr(stage_id, seq_q, seq_kv, block_size, max(seq_kv), m, q_tab, kv_tab, o_tab, dq_tab, dkv_tab))
            # what the stage added to blocks that already had a partial, and all of a kv block's private
            # replicas, are summed into the oldest slot and their slots given back (scheduler.py:1656-1700)
            sums, freed = [], []
            for what, table, keys, buffer_type in (("dq", partial_dq[r], [k for k, _ in rows], BufferType.BUFFER_dQ),
                                                   ("dkv", replicas[r], touched, BufferType.BUFFER_dKV)):
                for key in keys:
                    sl = table[key]
                    if len(sl) > 1:
                        sums.append(SumOp([row_block(buffer_type, s_, key) for s_ in sl], row_block(buffer_type, sl[0], key)))
                        freed += [(what, s_) for s_ in sl[1:]]
                        del sl[1:]
            if sums:
                instrs[r].append(SumInstr(sums, output_is_unpadded=0))
                for what, s_ in freed:
                    slots[r][what].free(s_)

        # ---- stages: the transfers of stage k+1 are launched before stage k is computed ---------
        for k in range(n_stages + 1):
            nxt = k + 1
            waits = [[] for _ in range(n_dev)]
            if nxt <= n_stages:
                first = [(rank_of(src), rank_of(dst), i) for dst in sorted(first_phase[nxt]) for i, src in first_phase[nxt][dst]]
                second = [(rank_of(src), rank_of(dst), i) for dst in sorted(second_phase[nxt]) for i, src in second_phase[nxt][dst]]
                ops1, arrived1 = exchange_ops(first)
                relays = {src for src, _, _ in second}
                for r in range(n_dev):
                    if ops1[r]:
                        instrs[r].append(CommLaunchInstr(f"S{nxt}", ops1[r]))
                # a relay forwards what it has just received: its receive must be booked first
                for dst, i, slot in arrived1:
                    held[dst][i] = slot
                ops2, arrived2 = exchange_ops(second)
                for r in range(n_dev):
                    if ops2[r]:
                        if ops1[r] and r in relays:
                            instrs[r].append(CommWaitInstr(f"S{nxt}", stream="second_phase"))
                        elif ops1[r]:
                            waits[r].append(f"S{nxt}")
                        instrs[r].append(CommLaunchInstr(f"S{nxt}P2", ops2[r], stream="second_phase"))
                        waits[r].append(f"S{nxt}P2")
                    elif ops1[r]:
                        waits[r].append(f"S{nxt}")
                for dst, i, slot in arrived2:
                    held[dst][i] = slot
            # stage k reads only blocks booked before this iteration's transfers: compute it now
            # (held already names the stage k+1 arrivals, but no work unit of stage k uses them)
            for r in range(n_dev):
                compute(r, k)
                release_dead_inputs(r, k)
                for key in waits[r]:
                    instrs[r].append(CommWaitInstr(key))

        # ---- results travel to the owners of their blocks -------------------------------------
        _RES = {"out": BufferType.BUFFER_OUT, "lse": BufferType.BUFFER_LSE, "dq": BufferType.BUFFER_dQ, "dkv": BufferType.BUFFER_dKV}

        def res_block(what, slot, key):
            return BufferBlock(_RES[what], slot, n_tok(key[1], key[2]))

        if is_bw:  # one partial per block and device: sum the device's own first
            for r in range(n_dev):
                pre = [SumOp([res_block("dq", s_, k) for s_ in sl], res_block("dq", sl[0], k)) for k, sl in partial_dq[r].items() if len(sl) > 1]
                pre += [SumOp([res_block("dkv", s_, k) for s_ in sl], res_block("dkv", sl[0], k)) for k, sl in replicas[r].items() if len(sl) > 1]
                if pre:
                    instrs[r].append(SumInstr(pre, output_is_unpadded=0))
        o_ops = [[] for _ in range(n_dev)]
        gathered = [defaultdict(list) for _ in range(n_dev)]  # owner: (what, key) -> slots to merge / sum
        for r in range(n_dev):
            tables = [("dq", partial_dq[r]), ("dkv", replicas[r])] if is_bw else [("out", partial_out[r])]
            for what, table in tables:
                for key, sl in sorted(table.items(), key=_BY_SEQUENCE):
                    dst = rank_of(owner(key[1], key[2]))
                    for slot in (sl[:1] if is_bw else sl):
                        if dst == r:
                            gathered[r][(what, key)].append(slot)
                            continue
                        there = slots[dst][what].take()
                        gathered[dst][(what, key)].append(there)
                        for part in (("out", "lse") if what == "out" else (what,)):
                            o_ops[r].append(CommOp(CommType.SEND, devices[dst], res_block(part, slot, key)))
                            o_ops[dst].append(CommOp(CommType.RECV, devices[r], res_block(part, there, key)))
        plans = []
        for r in range(n_dev):
            lay = layouts[r]
            if o_ops[r]:
                instrs[r] += [CommLaunchInstr("O", o_ops[r]), CommWaitInstr("O")]
            finals = []
            for (kind, g, s, b), li in local_index[r].items():
                key = (g, s, b)
                if kind == "q" and not is_bw and gathered[r][("out", key)]:
                    finals.append(ReductionOp([(res_block("out", s_, key), res_block("lse", s_, key)) for s_ in gathered[r][("out", key)]],
                                              (BufferBlock(BufferType.LOCAL_OUT, li, n_tok(s, b)), BufferBlock(BufferType.LOCAL_LSE, li, n_tok(s, b)))))
            if finals:
                instrs[r].append(AttnReductionInstr(finals, output_is_unpadded=1))
            if is_bw:
                for kind, what, local in (("q", "dq", BufferType.LOCAL_dQ), ("kv", "dkv", BufferType.LOCAL_dKV)):
                    sums = [SumOp([res_block(what, s_, (g, s, b)) for s_ in gathered[r][(what, (g, s, b))]],
                                  BufferBlock(local, li, n_tok(s, b)))
                            for (k2, g, s, b), li in local_index[r].items() if k2 == kind and gathered[r][(what, (g, s, b))]]
                    if sums:
                        instrs[r].append(SumInstr(sums, output_is_unpadded=1))
            if is_bw:
                info = pl.buffer_info(r, slots[r]["Q"].n, slots[r]["KV"].n, slots[r]["O"].n, (slots[r]["dq"].n, slots[r]["dkv"].n))
            else:
                info = pl.buffer_info(r, slots[r]["Q"].n, slots[r]["KV"].n, slots[r]["out"].n)
            node, dev = devices[r]
            plans.append(ExecutionPlan(instrs[r], n_nodes, n_devices_per_node, node, dev, n_stages + 1, lay.local_cu_seqlens, info))
        return plans

    return build(False), build(True), layouts
