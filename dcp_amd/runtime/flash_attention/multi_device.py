"""Plan builder for several devices with a fixed placement rule.

NOT the reference's planner (hypergraph partitioning and stage packing are out of this file's
reach): a simple context-parallel placement that produces per-device forward and backward
``ExecutionPlan``s with the same instruction structure the reference scheduler emits for a
device that exchanges blocks with others (``dcp/core/scheduler.py:894-1049`` input exchange,
``:1702-1762`` output exchange, ``:1764-1940`` final merges and sums), so that the
communication instructions can be run and checked:

* token block ``b`` of sequence ``s`` (its Q and its KV, every head block) lives on device
  ``(s + b) % n_devices``;
* the work unit (q block ``i``, kv block ``j``) of a sequence runs on the owner of the q block
  if ``i + j`` is even and on the owner of the kv block otherwise, so both kinds of traffic
  occur: KV (and Q) blocks travel to where they are multiplied, and partial results travel back
  -- (out, lse) partials to the q block's owner, which merges them, dQ partials to the q block's
  owner and dKV partials to the kv block's owner, which sum them;
* one input exchange (key ``S0``) and one output exchange (key ``O``) per pass.

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
    raw_seqlens = [int(x) for x in raw_seqlens]
    n_dev = n_nodes * n_devices_per_node
    group = n_heads // n_query_groups
    assert n_heads % n_query_groups == 0 and n_heads % head_block_size == 0
    if group > 1:
        assert head_block_size <= group and group % head_block_size == 0
    hb = head_block_size
    hkv = 1 if group > 1 else head_block_size
    n_hb_q, n_hb_kv = n_heads // hb, n_query_groups // hkv
    q_per_kv = n_hb_q // n_hb_kv
    mask_np = attn_mask.cpu().numpy()
    assert mask_np.shape[0] == sum(raw_seqlens)
    seq_off = np.concatenate(([0], np.cumsum(raw_seqlens)))
    n_blocks_of = [(L + block_size - 1) // block_size for L in raw_seqlens]
    wire_dtype = torch_dtype_to_int(dtype)

    def n_tok(s, b):
        return min(block_size, raw_seqlens[s] - b * block_size)

    def owner(s, b):
        return (s + b) % n_dev

    def peer_of(rank):
        return divmod(rank, n_devices_per_node)

    # ---- where every work unit runs: rows[rank][(g, s, i)] = kv block ids ----------------
    rows: List[Dict[Key, List[int]]] = [defaultdict(list) for _ in range(n_dev)]
    for s, L in enumerate(raw_seqlens):
        seq_mask = mask_np[seq_off[s] : seq_off[s + 1]]
        for i in range(n_blocks_of[s]):
            for j in _block_overlaps(seq_mask, i * block_size, n_tok(s, i), block_size, n_blocks_of[s], L):
                where = owner(s, i) if (i + j) % 2 == 0 else owner(s, j)
                for g in range(n_hb_q):
                    rows[where][(g, s, i)].append(j)

    # ---- LOCAL layouts --------------------------------------------------------------------
    layouts, local_q, local_kv = [], [], []
    for r in range(n_dev):
        lay = LocalLayout(raw_seqlens, block_size, n_heads, n_query_groups, head_dim, hb, hkv)
        iq, ikv = {}, {}
        for g in range(n_hb_q):
            for s in range(len(raw_seqlens)):
                for b in range(n_blocks_of[s]):
                    if owner(s, b) == r:
                        iq[(g, s, b)] = len(lay.q_blocks)
                        lay.q_blocks.append((g, s, b, n_tok(s, b)))
        for g in range(n_hb_kv):
            for s in range(len(raw_seqlens)):
                for b in range(n_blocks_of[s]):
                    if owner(s, b) == r:
                        ikv[(g, s, b)] = len(lay.kv_blocks)
                        lay.kv_blocks.append((g, s, b, n_tok(s, b)))
        cu = [0]
        for _, _, _, n in lay.q_blocks:
            cu.append(cu[-1] + n)
        lay.local_cu_seqlens = cu
        layouts.append(lay)
        local_q.append(iq)
        local_kv.append(ikv)

    def blk(buffer_type, index, key: Key):
        return BufferBlock(buffer_type, index, n_tok(key[1], key[2]))

    def row_mask(r):
        planes = []
        for (g, s, i), ids in sorted(rows[r].items(), key=lambda kv: (kv[0][1], kv[0][0], kv[0][2])):
            seq_mask = mask_np[seq_off[s] : seq_off[s + 1]]
            planes.append(_row_ranges(seq_mask, i * block_size, n_tok(s, i), block_size, ids, [n_tok(s, j) for j in ids]))
        t = torch.from_numpy(np.concatenate(planes, axis=2))
        return t[0] if t.shape[0] == 1 else t

    def ordered_rows(r):
        return sorted(rows[r].items(), key=lambda kv: (kv[0][1], kv[0][0], kv[0][2]))

    q_tok_shape, kv_tok_shape = (hb, head_dim), (2, hkv, head_dim)
    q_numel, kv_numel = block_size * hb * head_dim, block_size * 2 * hkv * head_dim

    def local_info(n_blocks, total, tok_shape, numel):
        return BufferInfo(n_blocks, block_size, numel, wire_dtype, (total, *tok_shape), tok_shape)

    def slot_info(n_blocks, tok_shape, numel):
        return BufferInfo(n_blocks, block_size, numel, wire_dtype, (n_blocks, block_size, *tok_shape), tok_shape)

    def lse_slot_info(n_blocks):
        return BufferInfo(n_blocks, block_size, block_size * hb, DType.FLOAT32, (hb, n_blocks, block_size), (1,))

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
            total_q, total_kv = lay.local_cu_seqlens[-1], sum(n for _, _, _, n in lay.kv_blocks)
            slots = phase[r][0]
            info = {
                BufferType.LOCAL_Q: local_info(len(lay.q_blocks), total_q, q_tok_shape, q_numel),
                BufferType.LOCAL_KV: local_info(len(lay.kv_blocks), total_kv, kv_tok_shape, kv_numel),
                BufferType.LOCAL_OUT: local_info(len(lay.q_blocks), total_q, q_tok_shape, q_numel),
                BufferType.LOCAL_LSE: BufferInfo(len(lay.q_blocks), block_size, block_size * hb, DType.FLOAT32, (hb, total_q), (1,)),
                BufferType.BUFFER_Q: slot_info(max(slots["q"].n, 1), q_tok_shape, q_numel),
                BufferType.BUFFER_KV: slot_info(max(slots["kv"].n, 1), kv_tok_shape, kv_numel),
            }
            if not with_backward:
                ops = []
                for k, li in local_q[r].items():
                    srcs = ([st["partial_out"][k]] if k in st["partial_out"] else []) + arrivals[r][("out", k)]
                    if srcs:
                        ops.append(ReductionOp([(blk(BufferType.BUFFER_OUT, s_, k), blk(BufferType.BUFFER_LSE, s_, k)) for s_ in srcs],
                                               (blk(BufferType.LOCAL_OUT, li, k), blk(BufferType.LOCAL_LSE, li, k))))
                if ops:
                    instrs.append(AttnReductionInstr(ops, output_is_unpadded=1))
                n_out = max(st["res"]["out"].n, 1)
                info[BufferType.BUFFER_OUT] = slot_info(n_out, q_tok_shape, q_numel)
                info[BufferType.BUFFER_LSE] = lse_slot_info(n_out)
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
                n_o = max(slots["o"].n, 1)
                info.update({
                    BufferType.LOCAL_dOUT: local_info(len(lay.q_blocks), total_q, q_tok_shape, q_numel),
                    BufferType.LOCAL_dQ: local_info(len(lay.q_blocks), total_q, q_tok_shape, q_numel),
                    BufferType.LOCAL_dKV: local_info(len(lay.kv_blocks), total_kv, kv_tok_shape, kv_numel),
                    BufferType.BUFFER_OUT: slot_info(n_o, q_tok_shape, q_numel),
                    BufferType.BUFFER_LSE: lse_slot_info(n_o),
                    BufferType.BUFFER_dOUT: slot_info(n_o, q_tok_shape, q_numel),
                    BufferType.BUFFER_dQ: slot_info(max(st["res"]["dq"].n, 1), q_tok_shape, q_numel),
                    BufferType.BUFFER_dKV: slot_info(max(st["res"]["dkv"].n, 1), kv_tok_shape, kv_numel),
                })
            node, dev = peer_of(r)
            plans.append(ExecutionPlan(instrs, n_nodes, n_devices_per_node, node, dev, 1, lay.local_cu_seqlens, info))
        return plans

    return build(False), build(True), layouts
