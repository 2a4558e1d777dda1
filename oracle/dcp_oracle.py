"""CPU oracle of DCP's per-device blockwise attention path.  TEST INFRASTRUCTURE
ONLY: imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
leg as the checker; the product (dcp_amd/) never imports it.

A numpy restatement of what the reference computes on this path.  Each
function cites the reference code it follows (paths relative to the reference
repository root):

  block_copy              commented torch fallback of _handle_memcpy
                          (dcp/runtime/flash_attention/executor.py:814-831),
                          kernels dcp/ops/fused_ops.py:290-335, 370-429
  merge_out_lse           _flash_attn_update_out_lse (fused_ops.py:15-146);
                          pairwise form _update_out_and_lse
                          (executor.py:1197-1215)
  blockwise_sum           commented torch fallback of _handle_sum
                          (executor.py:1549-1580), kernel fused_ops.py:1087-1151
  range_attention_fwd/bwd attention_ref with attn_range
                          (tests/runtime/test_flash_attention.py:127-279); the
                          arithmetic itself lives in the external dcp_flash_attn
                          fork of flash-attention 2.6.3 (docker/Dockerfile:63-65),
                          whose source is not in the reference tree: its
                          published algorithm (softmax(scale*QK^T + mask)V with
                          LSE = logsumexp, out=0 / lse=+inf for empty rows) is
                          restated here
  run_plan                instruction semantics of
                          dcp/runtime/flash_attention/executor.py:606-1546;
                          block exchange between devices (CommLaunchInstr /
                          CommWaitInstr) executor.py:1583-2074

Pinning (tests/test_oracle.py): block movement against numpy fancy indexing
and gather/scatter round trips; the block sum against math.fsum (the exactly
rounded sum) and exact integer sums; merge against scipy.special.logsumexp, the
folded pairwise sigmoid form and its invariants; attention forward against
torch.nn.functional.scaled_dot_product_attention and a dense boolean mask;
backward against torch.autograd and central finite differences; masks against
O(L^2) brute force and closed-form pair counts.  The exact rounding order of
the reference's in-dtype block sum and the bit-level behaviour of the external
flash-attention fork are "parity unpinned": nothing in the reference tree
fixes them, so those comparisons are toleranced.

All arithmetic is float64 unless stated; ``round_to`` models the single
rounding a kernel performs when it stores bf16/fp16.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

NEG_INF = -np.inf


# ---------------------------------------------------------------------------
# storage rounding
# ---------------------------------------------------------------------------


def round_bf16(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even to bfloat16, returned as float32."""
    f = np.ascontiguousarray(x, dtype=np.float32)
    u = f.view(np.uint32).astype(np.uint64)
    rounded = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    out = rounded.astype(np.uint32).view(np.float32)
    return np.where(np.isnan(f), f, out).reshape(f.shape)


def round_to(x: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "bf16":
        return round_bf16(x)
    if dtype == "fp16":
        return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)
    if dtype == "fp32":
        return np.asarray(x, dtype=np.float32)
    raise ValueError(f"Unsupported dtype {dtype}")


# ---------------------------------------------------------------------------
# block movement (bit-exact; works on any numpy dtype, incl. uint16 views)
# ---------------------------------------------------------------------------


def block_copy(src_flat, src_elem_offsets, dst_flat, dst_elem_offsets, n_elements):
    """dst[dst_off : dst_off+n] = src[src_off : src_off+n] for every pair."""
    for so, do, n in zip(src_elem_offsets, dst_elem_offsets, n_elements):
        dst_flat[do : do + n] = src_flat[so : so + n]


# ---------------------------------------------------------------------------
# N-way online-softmax merge
# ---------------------------------------------------------------------------


def merge_out_lse(outs: np.ndarray, lses: np.ndarray):
    """outs [S, T, H, D], lses [S, H, T] -> (out [T, H, D], lse [H, T]).

    Sources with lse = +-inf are ignored; with no other source lse = -1 and
    out = 0 (fused_ops.py:118-143).  Only the two infinities mark an empty source
    (fused_ops.py:123: ``lse != -inf and lse != inf``): a NaN lse counts as a source and
    makes the merged lse and out of its (token, head) NaN."""
    outs = np.asarray(outs, dtype=np.float64)
    lses = np.asarray(lses, dtype=np.float64)
    finite = ~np.isinf(lses)
    masked = np.where(finite, lses, NEG_INF)
    m = masked.max(axis=0)
    any_finite = finite.any(axis=0)
    m_safe = np.where(any_finite, m, 0.0)
    with np.errstate(divide="ignore"):
        new_lse = m_safe + np.log(np.where(finite, np.exp(masked - m_safe), 0.0).sum(axis=0))
    new_lse = np.where(any_finite, new_lse, -1.0)
    w = np.where(finite, np.exp(masked - np.where(any_finite, new_lse, 0.0)), 0.0)  # [S,H,T]
    w = np.transpose(w, (0, 2, 1))[..., None]  # [S,T,H,1]
    out = (np.where(w > 0, outs, 0.0) * w).sum(axis=0)
    return out, new_lse


def merge_pairwise(outs: np.ndarray, lses: np.ndarray):
    """Left fold with the reference's two-way update
    (executor.py:1212-1213): out -= sigmoid(l_b - l)*(out - out_b);
    l -= logsigmoid(l - l_b).  Finite LSEs only."""
    out = np.asarray(outs[0], dtype=np.float64)
    lse = np.asarray(lses[0], dtype=np.float64)  # [H,T]
    for j in range(1, len(outs)):
        blk_lse = np.asarray(lses[j], dtype=np.float64)
        d = (blk_lse - lse).T[..., None]  # [T,H,1]
        sig = 1.0 / (1.0 + np.exp(-d))
        out = out - sig * (out - np.asarray(outs[j], dtype=np.float64))
        x = lse - blk_lse
        lse = lse + np.logaddexp(0.0, -x)  # - logsigmoid(x) = log(1+exp(-x))
    return out, lse


def blockwise_sum(srcs: Sequence[np.ndarray]) -> np.ndarray:
    """Element-wise sum in float64."""
    acc = np.zeros_like(np.asarray(srcs[0], dtype=np.float64))
    for s in srcs:
        acc += np.asarray(s, dtype=np.float64)
    return acc


# ---------------------------------------------------------------------------
# range-masked attention (one row: Tq queries against Tk keys)
# ---------------------------------------------------------------------------


def ranges_to_bool(ranges: np.ndarray, n_keys: int) -> np.ndarray:
    """ranges [n_ranges, 2, Tq] -> bool [Tq, Tk]: union of [start, end)."""
    ranges = np.asarray(ranges)
    if ranges.ndim == 2:
        ranges = ranges[None]
    k = np.arange(n_keys)[None, :]
    allowed = np.zeros((ranges.shape[2], n_keys), dtype=bool)
    for r in range(ranges.shape[0]):
        allowed |= (k >= ranges[r, 0][:, None]) & (k < ranges[r, 1][:, None])
    return allowed


def range_attention_fwd(q, k, v, allowed, scale=None, dtype=np.float64):
    """q [Tq,H,D], k/v [Tk,Hkv,D], allowed bool [Tq,Tk].
    Returns out [Tq,H,D], lse [H,Tq].  q head h uses kv head h // (H//Hkv).
    Rows with no allowed key: out = 0, lse = +inf."""
    q = np.asarray(q, dtype=dtype)
    k = np.asarray(k, dtype=dtype)
    v = np.asarray(v, dtype=dtype)
    Tq, H, D = q.shape
    Hkv = k.shape[1]
    g = H // Hkv
    if scale is None:
        scale = D ** -0.5
    out = np.zeros((Tq, H, D), dtype=dtype)
    lse = np.full((H, Tq), np.inf, dtype=dtype)
    has_key = allowed.any(axis=1)
    for h in range(H):
        s = (q[:, h] @ k[:, h // g].T) * scale
        s = np.where(allowed, s, NEG_INF)
        m = np.where(has_key, s.max(axis=1, initial=NEG_INF), 0.0)
        p = np.exp(s - m[:, None])
        l = p.sum(axis=1)
        with np.errstate(divide="ignore", invalid="ignore"):
            out[:, h] = np.where(has_key[:, None], (p @ v[:, h // g]) / l[:, None], 0.0)
            lse[h] = np.where(has_key, m + np.log(l), np.inf)
    return out, lse


def range_attention_bwd(q, k, v, out, lse, dout, allowed, scale=None, dtype=np.float64):
    """Analytic gradient of range_attention_fwd.  Returns dq [Tq,H,D],
    dk, dv [Tk,Hkv,D] (summed over the q heads of each kv head's group)."""
    q = np.asarray(q, dtype=dtype)
    k = np.asarray(k, dtype=dtype)
    v = np.asarray(v, dtype=dtype)
    out = np.asarray(out, dtype=dtype)
    dout = np.asarray(dout, dtype=dtype)
    lse = np.asarray(lse, dtype=dtype)
    Tq, H, D = q.shape
    Hkv = k.shape[1]
    g = H // Hkv
    if scale is None:
        scale = D ** -0.5
    dq = np.zeros_like(q)
    dk = np.zeros_like(k)
    dv = np.zeros_like(v)
    for h in range(H):
        kh, vh = k[:, h // g], v[:, h // g]
        s = (q[:, h] @ kh.T) * scale
        row_lse = np.where(np.isfinite(lse[h]), lse[h], 0.0)
        p = np.where(allowed, np.exp(np.where(allowed, s, 0.0) - row_lse[:, None]), 0.0)
        p = np.where(np.isfinite(lse[h])[:, None], p, 0.0)
        dv[:, h // g] += p.T @ dout[:, h]
        dp = dout[:, h] @ vh.T
        delta = (dout[:, h] * out[:, h]).sum(axis=1)
        ds = p * (dp - delta[:, None]) * scale
        dq[:, h] = ds @ kh
        dk[:, h // g] += ds.T @ q[:, h]
    return dq, dk, dv


# ---------------------------------------------------------------------------
# plan interpreter
# ---------------------------------------------------------------------------

_LSE_TYPES = ("BufferLSE", "LocalLSE")
_DTYPE_NAME = {0: "bf16", 1: "fp16", 2: "fp32"}


class PlanOracle:
    """Runs an ExecutionPlan on numpy buffers with the semantics of the
    reference handlers.  Buffers hold float32 values that are exactly
    representable in the buffer's storage type."""

    def __init__(self, plan, n_heads_per_block: int, head_dim: int, compute_dtype=np.float64):
        self.plan = plan
        self.hb = n_heads_per_block
        self.head_dim = head_dim
        self.compute_dtype = compute_dtype
        self.buffers: Dict[str, np.ndarray] = {}
        self.store_dtype: Dict[str, str] = {}
        for name, info in plan.buffer_info.items():
            self.buffers[name] = np.zeros(tuple(info.buffer_shape), dtype=np.float32)
            self.store_dtype[name] = _DTYPE_NAME[info.dtype]

    # -- helpers -------------------------------------------------------------
    def set(self, name: str, value) -> None:
        self.buffers[name][...] = round_to(np.asarray(value, dtype=np.float32), self.store_dtype[name])

    def _store(self, name: str, index, value) -> None:
        self.buffers[name][index] = round_to(value, self.store_dtype[name])

    def run(self):
        for instr in self.plan.instructions:
            getattr(self, "_" + type(instr).__name__)(instr)
        return self.buffers

    # -- communication (several devices' plans run together, see run_plans_together) ----------
    def attach(self, mailbox: dict, rank: int, n_devices_per_node: int) -> None:
        self.mailbox, self.rank, self.n_devices_per_node = mailbox, rank, n_devices_per_node
        self.expected: Dict[str, list] = {}

    def _block_view(self, block):
        """The elements a communication op moves for ``block``: the same views as
        _prepare_comm_launch builds (executor.py:1617-1640)."""
        buf, n = self.buffers[block.buffer_type], block.n_tokens
        if block.buffer_type.startswith("Local"):
            off = self.plan.local_cu_seqlens[block.index]
            return buf[:, off : off + n] if block.buffer_type in _LSE_TYPES else buf[off : off + n]
        return buf[:, block.index, :n] if block.buffer_type in _LSE_TYPES else buf[block.index, :n]

    def _CommLaunchInstr(self, instr):
        """Sends are snapshotted at launch, in op order per peer (the send buffer of
        executor.py:1949-1976); receives land at the matching wait (:2043-2073)."""
        recvs = []
        for op in instr.comm_ops:
            peer = op.peer[0] * self.n_devices_per_node + op.peer[1]
            if op.comm_type == 0:  # CommType.SEND
                self.mailbox.setdefault((self.rank, peer, instr.key), []).append(self._block_view(op.buffer_block).copy())
            else:
                recvs.append((peer, op.buffer_block))
        self.expected[instr.key] = recvs

    def comm_ready(self, key: str) -> bool:
        need: Dict[int, int] = {}
        for peer, _ in self.expected[key]:
            need[peer] = need.get(peer, 0) + 1
        return all(len(self.mailbox.get((peer, self.rank, key), [])) >= n for peer, n in need.items())

    def _CommWaitInstr(self, instr):
        assert self.comm_ready(instr.key), "wait before the peers' launches"
        for peer, block in self.expected.pop(instr.key):
            data = self.mailbox[(peer, self.rank, instr.key)].pop(0)
            view = self._block_view(block)
            assert view.shape == data.shape, (view.shape, data.shape)
            view[...] = data

    # -- instructions --------------------------------------------------------
    def _MemcpyInstr(self, instr):
        cu = self.plan.local_cu_seqlens
        for src, dst in instr.src_dst_pairs:
            n = src.n_tokens
            off = cu[src.index]
            if src.buffer_type in _LSE_TYPES:
                self.buffers[dst.buffer_type][:, dst.index, :n] = self.buffers[src.buffer_type][:, off : off + n]
            else:
                self.buffers[dst.buffer_type][dst.index, :n] = self.buffers[src.buffer_type][off : off + n]

    def _rows(self, instr):
        """Yield (b, q slot, n_q, kv slots, ranges [n_ranges,2,n_q])."""
        mask = np.asarray(instr.attn_mask)
        if mask.ndim == 2:
            mask = mask[None]
        q0 = 0
        for b, n_q in enumerate(instr.seqlens_q):
            yield b, instr.q_block_table[b][0].index, n_q, [x.index for x in instr.kv_block_table[b]], mask[:, :, q0 : q0 + n_q]
            q0 += n_q

    def _AttnInstr(self, instr):
        Q, KV = self.buffers["BufferQ"], self.buffers["BufferKV"]
        for b, q_slot, n_q, kv_slots, ranges in self._rows(instr):
            kv = np.concatenate([KV[s] for s in kv_slots], axis=0)  # [Tk,2,hkv,D]
            allowed = ranges_to_bool(ranges, kv.shape[0])
            out, lse = range_attention_fwd(Q[q_slot, :n_q], kv[:, 0], kv[:, 1], allowed,
                                           dtype=self.compute_dtype)
            o_slot = instr.out_block_table[b][0].index
            self._store("BufferOut", (o_slot, slice(0, n_q)), out)
            self.buffers["BufferLSE"][:, o_slot, :n_q] = lse.astype(np.float32)

    def _AttnBackwardInstr(self, instr):
        Q, KV = self.buffers["BufferQ"], self.buffers["BufferKV"]
        O, LSE, dO = self.buffers["BufferOut"], self.buffers["BufferLSE"], self.buffers["BufferdOut"]
        bs = Q.shape[1]
        for b, q_slot, n_q, kv_slots, ranges in self._rows(instr):
            kv = np.concatenate([KV[s] for s in kv_slots], axis=0)
            allowed = ranges_to_bool(ranges, kv.shape[0])
            o_slot = instr.out_block_table[b][0].index
            dq, dk, dv = range_attention_bwd(
                Q[q_slot, :n_q], kv[:, 0], kv[:, 1], O[o_slot, :n_q], LSE[:, o_slot, :n_q],
                dO[o_slot, :n_q], allowed, dtype=self.compute_dtype)
            self._store("BufferdQ", (instr.dq_block_table[b][0].index, slice(0, n_q)), dq)
            for j, blk in enumerate(instr.dkv_block_table[b]):
                self._store("BufferdKV", (blk.index, slice(None), 0), dk[j * bs : (j + 1) * bs])
                self._store("BufferdKV", (blk.index, slice(None), 1), dv[j * bs : (j + 1) * bs])

    def _AttnReductionInstr(self, instr):
        cu = self.plan.local_cu_seqlens
        for op in instr.ops:
            n = op.dst_buffer[0].n_tokens
            outs = np.stack([self.buffers[o.buffer_type][o.index, :n] for o, _ in op.src_buffers])
            lses = np.stack([self.buffers[l.buffer_type][:, l.index, :n] for _, l in op.src_buffers])
            out, lse = merge_out_lse(outs, lses)
            d_out, d_lse = op.dst_buffer
            if instr.output_is_unpadded:
                off = cu[d_out.index]
                self._store(d_out.buffer_type, slice(off, off + n), out)
                self.buffers[d_lse.buffer_type][:, off : off + n] = lse.astype(np.float32)
            else:
                self._store(d_out.buffer_type, (d_out.index, slice(0, n)), out)
                self.buffers[d_lse.buffer_type][:, d_lse.index, :n] = lse.astype(np.float32)

    def _SumInstr(self, instr):
        cu = self.plan.local_cu_seqlens
        for op in instr.ops:
            n = op.dst_buffer.n_tokens
            total = blockwise_sum([self.buffers[s.buffer_type][s.index, :n] for s in op.src_buffers])
            d = op.dst_buffer
            if instr.output_is_unpadded:
                off = cu[d.index]
                self._store(d.buffer_type, slice(off, off + n), total)
            else:
                self._store(d.buffer_type, (d.index, slice(0, n)), total)


def run_plans_together(oracles: Sequence["PlanOracle"], n_devices_per_node: int) -> None:
    """Runs the plans of several devices (``oracles[rank]``) to the end, each as far as its
    next wait whose peers have not launched yet, in turns: a device's sends are visible to its
    peers from its CommLaunchInstr on, as with the asynchronous all-to-all of
    executor.py:1977-1999."""
    mailbox: dict = {}
    for rank, o in enumerate(oracles):
        o.attach(mailbox, rank, n_devices_per_node)
    cursor = [0] * len(oracles)
    while any(c < len(o.plan.instructions) for c, o in zip(cursor, oracles)):
        progressed = False
        for rank, o in enumerate(oracles):
            instrs = o.plan.instructions
            while cursor[rank] < len(instrs):
                instr = instrs[cursor[rank]]
                if type(instr).__name__ == "CommWaitInstr" and not o.comm_ready(instr.key):
                    break
                getattr(o, "_" + type(instr).__name__)(instr)
                cursor[rank] += 1
                progressed = True
        assert progressed, "the plans wait for each other"
    assert all(len(v) == 0 for v in mailbox.values()), "blocks sent but never received"


# ---------------------------------------------------------------------------
# whole-sequence truth (what any correct schedule must reproduce)
# ---------------------------------------------------------------------------


def dense_reference(q, kv, seq_mask, raw_seqlens, dout=None, dtype=np.float64):
    """q [T,H,D], kv [T,2,Hkv,D], seq_mask [T,2] or [T,2,2] in sequence-local
    key positions.  Returns out [T,H,D], lse [H,T] and, if dout is given,
    dq [T,H,D], dkv [T,2,Hkv,D]."""
    q = np.asarray(q, dtype=dtype)
    kv = np.asarray(kv, dtype=dtype)
    T, H, D = q.shape
    out = np.zeros((T, H, D), dtype=dtype)
    lse = np.zeros((H, T), dtype=dtype)
    dq = np.zeros_like(q) if dout is not None else None
    dkv = np.zeros_like(kv) if dout is not None else None
    seq_mask = np.asarray(seq_mask)
    t0 = 0
    for L in raw_seqlens:
        sl = slice(t0, t0 + L)
        m = seq_mask[sl]
        ranges = m.T[None] if m.ndim == 2 else np.transpose(m, (1, 2, 0))
        allowed = ranges_to_bool(ranges, L)
        o, l = range_attention_fwd(q[sl], kv[sl, 0], kv[sl, 1], allowed, dtype=dtype)
        out[sl], lse[:, sl] = o, l
        if dout is not None:
            a, b, c = range_attention_bwd(q[sl], kv[sl, 0], kv[sl, 1], o, l,
                                          np.asarray(dout, dtype=dtype)[sl], allowed, dtype=dtype)
            dq[sl], dkv[sl, 0], dkv[sl, 1] = a, b, c
        t0 += L
    if dout is None:
        return out, lse
    return out, lse, dq, dkv


def attention_flops(n_pairs: int, n_heads: int, head_dim: int, mode: str = "fwd") -> float:
    """FLOP convention of the reference cost model (dcp/core/cost_model.py:108-127):
    fwd = 4*pairs*heads*head_dim, bwd = 2.5*fwd."""
    f = 4.0 * n_pairs * n_heads * head_dim
    return {"fwd": f, "bwd": 2.5 * f, "fwd+bwd": 3.5 * f}[mode]
