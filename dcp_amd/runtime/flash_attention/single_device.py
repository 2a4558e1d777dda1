"""Plan builder for one device that owns every block.

Given raw sequence lengths, a block size, a head blocking and a range mask it
emits the forward and backward ``ExecutionPlan`` a single device runs: gather
into padded slots, one attention instruction per stage, merges / sums, scatter
back.  The plans have the structure the reference scheduler produces when all
inputs are local (every work unit lands in stage 0:
``dcp/core/pipeline.py:614-646``; gather ``dcp/core/scheduler.py:870-892``;
attention rows and concatenated range masks ``:1051-1322``; per-stage folds
``:1324-1363``; backward rows and private dKV replicas ``:1365-1700``; final
merges and sums ``:1764-1940``; buffer shapes ``:1998-2102``; LOCAL ordering
and ``local_cu_seqlens`` ``dcp/core/compiler.py:197-263``).

A multi-device share is emulated by ``n_kv_groups > 1``: each row's kv blocks
are dealt round-robin (or contiguously) into groups, one attention instruction
runs per group into its own out/lse (or dQ/dKV) slots, and the partials are
merged (summed) exactly as partials received from other devices would be.
"""

from __future__ import annotations

import heapq

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from dcp_amd.core.instructions import (
    AttnBackwardInstr,
    AttnInstr,
    AttnReductionInstr,
    BufferBlock,
    BufferInfo,
    BufferType,
    DType,
    ExecutionPlan,
    MemcpyInstr,
    ReductionOp,
    SumInstr,
    SumOp,
)
from dcp_amd.core.serialization import torch_dtype_to_int
from dcp_amd.runtime.flash_attention.workload import concat_local_attn_masks, generate_work_units, rows_of_work_units


@dataclass
class LocalLayout:
    """Where each (head block, sequence, token block) lives in the unpadded
    LOCAL_* buffers.  ``q_blocks[i]`` / ``kv_blocks[i]`` are
    ``(head_block, seq, block, n_tokens)`` for local index ``i``; tokens of
    local block ``i`` occupy ``local_cu_seqlens[i] : +n_tokens``."""

    raw_seqlens: List[int]
    block_size: int
    n_heads: int
    n_query_groups: int
    head_dim: int
    head_block_size: int
    head_block_size_kv: int
    q_blocks: List[Tuple[int, int, int, int]] = field(default_factory=list)
    kv_blocks: List[Tuple[int, int, int, int]] = field(default_factory=list)
    local_cu_seqlens: List[int] = field(default_factory=list)

    @property
    def total_tokens(self) -> int:
        return int(sum(self.raw_seqlens))

    @property
    def n_head_blocks_q(self) -> int:
        return self.n_heads // self.head_block_size

    @property
    def n_head_blocks_kv(self) -> int:
        return self.n_query_groups // self.head_block_size_kv

    def _seq_offsets(self) -> np.ndarray:
        return np.concatenate(([0], np.cumsum(self.raw_seqlens)))

    def _gather(self, x: torch.Tensor, blocks, hb: int, head_axis: int):
        """x is global ``[total_tokens, ...heads..., D]``; returns the local
        concatenation over blocks of the head-block slice."""
        off = self._seq_offsets()
        parts = []
        for head_block, seq, blk, n_tok in blocks:
            t0 = int(off[seq]) + blk * self.block_size
            sl = [slice(t0, t0 + n_tok)] + [slice(None)] * (x.dim() - 1)
            sl[head_axis] = slice(head_block * hb, (head_block + 1) * hb)
            parts.append(x[tuple(sl)])
        if not parts:  # a device that owns no block
            shape = list(x.shape)
            shape[0], shape[head_axis] = 0, hb
            return x.new_zeros(shape)
        return torch.cat(parts, dim=0).contiguous()

    def to_local_q(self, q: torch.Tensor) -> torch.Tensor:
        """Global ``[T, n_heads, D]`` -> LOCAL_Q ``[n_head_blocks*T, hb, D]``
        (also for out / dout / dq)."""
        return self._gather(q, self.q_blocks, self.head_block_size, 1)

    def to_local_kv(self, kv: torch.Tensor) -> torch.Tensor:
        """Global ``[T, 2, n_query_groups, D]`` -> LOCAL_KV."""
        return self._gather(kv, self.kv_blocks, self.head_block_size_kv, 2)

    def _scatter(self, local: torch.Tensor, blocks, hb: int, head_axis: int, shape):
        off = self._seq_offsets()
        out = local.new_zeros(shape)
        pos = 0
        for head_block, seq, blk, n_tok in blocks:
            t0 = int(off[seq]) + blk * self.block_size
            sl = [slice(t0, t0 + n_tok)] + [slice(None)] * (len(shape) - 1)
            sl[head_axis] = slice(head_block * hb, (head_block + 1) * hb)
            out[tuple(sl)] = local[pos : pos + n_tok]
            pos += n_tok
        return out

    def from_local_q(self, local: torch.Tensor) -> torch.Tensor:
        shape = (self.total_tokens, self.n_heads, self.head_dim)
        return self._scatter(local, self.q_blocks, self.head_block_size, 1, shape)

    def from_local_kv(self, local: torch.Tensor) -> torch.Tensor:
        shape = (self.total_tokens, 2, self.n_query_groups, self.head_dim)
        return self._scatter(local, self.kv_blocks, self.head_block_size_kv, 2, shape)

    def from_local_lse(self, local_lse: torch.Tensor) -> torch.Tensor:
        """LOCAL_LSE ``[hb, n_head_blocks*T]`` -> global ``[n_heads, T]``."""
        off = self._seq_offsets()
        out = local_lse.new_zeros((self.n_heads, self.total_tokens))
        pos = 0
        hb = self.head_block_size
        for head_block, seq, blk, n_tok in self.q_blocks:
            t0 = int(off[seq]) + blk * self.block_size
            out[head_block * hb : (head_block + 1) * hb, t0 : t0 + n_tok] = local_lse[
                :, pos : pos + n_tok
            ]
            pos += n_tok
        return out

    def to_local_lse(self, lse: torch.Tensor) -> torch.Tensor:
        off = self._seq_offsets()
        hb = self.head_block_size
        parts = []
        for head_block, seq, blk, n_tok in self.q_blocks:
            t0 = int(off[seq]) + blk * self.block_size
            parts.append(lse[head_block * hb : (head_block + 1) * hb, t0 : t0 + n_tok])
        if not parts:
            return lse.new_zeros((hb, 0))
        return torch.cat(parts, dim=1).contiguous()


class _Slots:
    """First-free slot allocator of one padded buffer: ``take`` hands out the lowest slot that is
    not in use, ``free`` returns one (the allocation rule of the reference's BlockManager,
    dcp/core/block_table.py:434-460).  ``n`` = slots the buffer needs."""

    def __init__(self):
        self.n = 0
        self._free: List[int] = []

    def take(self) -> int:
        if self._free:
            return heapq.heappop(self._free)
        self.n += 1
        return self.n - 1

    def free(self, index: int) -> None:
        assert 0 <= index < self.n and index not in self._free, f"slot {index} is not in use"
        heapq.heappush(self._free, index)


def _row_ranges(seq_mask: np.ndarray, q0: int, n_q: int, block_size: int,
                kv_block_ids: Sequence[int], kv_n_tokens: Sequence[int]):
    """Ranges of the ``n_q`` query tokens starting at sequence position ``q0``
    re-expressed in the coordinates of the concatenation of ``kv_block_ids``
    (each occupying ``block_size`` positions).  Returns int32
    ``[n_ranges, 2, block_size]``; padding query rows and empty ranges are
    ``[0, 0)``."""
    n_ranges = 1 if seq_mask.ndim == 2 else 2
    out = np.zeros((n_ranges, 2, block_size), dtype=np.int32)
    for r in range(n_ranges):
        rng = seq_mask[q0 : q0 + n_q] if n_ranges == 1 else seq_mask[q0 : q0 + n_q, r]
        s, e = rng[:, 0].astype(np.int64), rng[:, 1].astype(np.int64)
        start = np.full(n_q, -1, dtype=np.int64)
        end = np.zeros(n_q, dtype=np.int64)
        for k, (j, n_tok) in enumerate(zip(kv_block_ids, kv_n_tokens)):
            lo = np.maximum(s, j * block_size)
            hi = np.minimum(e, j * block_size + n_tok)
            valid = hi > lo
            c_lo = k * block_size + (lo - j * block_size)
            c_hi = k * block_size + (hi - j * block_size)
            contiguous = (start == -1) | (c_lo == end) | ~valid
            assert contiguous.all(), "Discontinuous attn mask"
            first = valid & (start == -1)
            start[first] = c_lo[first]
            end[valid] = c_hi[valid]
        start[start == -1] = 0
        out[r, 0, :n_q] = start
        out[r, 1, :n_q] = end
    return out


def _block_overlaps(seq_mask: np.ndarray, q0: int, n_q: int, block_size: int,
                    n_blocks: int, seqlen: int) -> List[int]:
    """kv block ids that at least one of the query tokens attends."""
    hit = np.zeros(n_blocks, dtype=bool)
    rows = seq_mask[q0 : q0 + n_q].reshape(n_q, -1, 2)
    for r in range(rows.shape[1]):
        s = rows[:, r, 0].astype(np.int64)
        e = np.minimum(rows[:, r, 1].astype(np.int64), seqlen)
        ok = e > s
        if not ok.any():
            continue
        b0 = s[ok] // block_size
        b1 = (e[ok] - 1) // block_size
        delta = np.zeros(n_blocks + 1, dtype=np.int64)
        np.add.at(delta, b0, 1)
        np.add.at(delta, b1 + 1, -1)
        hit |= np.cumsum(delta[:-1]) > 0
    return [int(b) for b in np.nonzero(hit)[0]]


def build_single_device_plans(
    raw_seqlens: Sequence[int],
    block_size: int,
    n_heads: int,
    n_query_groups: int,
    head_dim: int,
    head_block_size: int,
    attn_mask: torch.Tensor,
    dtype: torch.dtype = torch.bfloat16,
    n_kv_groups: int = 1,
    kv_split: str = "round_robin",
    fold_stages: bool = False,
    backward: bool = True,
    work_units: str = "overlap",
):
    """Returns ``(fw_plan, bw_plan, layout)`` (``bw_plan`` is ``None`` when
    ``backward`` is false).

    ``attn_mask`` is the output of a mask generator over *unpadded* sequences
    (``padded_seqlens == raw_seqlens``): ``[sum(raw_seqlens), 2]`` or
    ``[sum(raw_seqlens), 2, 2]``.
    ``n_kv_groups``/``kv_split`` split each row's kv blocks into partials;
    ``fold_stages`` merges each later stage's partial into the stage-0 partial
    in place (padded destination) instead of one N-way merge at the end.
    ``work_units`` chooses which (q block, kv block) pairs a row holds:
    ``"overlap"`` keeps the pairs in which some query attends some key;
    ``"reference"`` goes the reference's way through block-local masks
    (``workload.generate_work_units`` / ``concat_local_attn_masks``), which also
    keeps pairs that only the hull of the block's ranges touches (all their
    ranges are empty; same results, a few more kv blocks per row).
    """
    assert work_units in ("overlap", "reference")
    raw_seqlens = [int(x) for x in raw_seqlens]
    assert n_heads % n_query_groups == 0
    group = n_heads // n_query_groups
    is_gqa = group > 1
    if is_gqa:
        assert head_block_size <= group and group % head_block_size == 0
    assert n_heads % head_block_size == 0
    hb = head_block_size
    hkv = 1 if is_gqa else head_block_size
    n_hb_q = n_heads // hb
    n_hb_kv = n_query_groups // hkv
    q_per_kv_block = n_hb_q // n_hb_kv  # q head blocks sharing one kv head block
    assert kv_split in ("round_robin", "contiguous")
    assert n_kv_groups >= 1
    mask_np = attn_mask.cpu().numpy()
    assert mask_np.shape[0] == sum(raw_seqlens)
    wire_dtype = torch_dtype_to_int(dtype)

    n_blocks_of = [(L + block_size - 1) // block_size for L in raw_seqlens]

    def n_tok(seq, blk):
        return min(block_size, raw_seqlens[seq] - blk * block_size)

    layout = LocalLayout(raw_seqlens, block_size, n_heads, n_query_groups, head_dim, hb, hkv)
    # LOCAL order: (head block, sequence, block)
    local_q_index: Dict[Tuple[int, int, int], int] = {}
    for g in range(n_hb_q):
        for s in range(len(raw_seqlens)):
            for b in range(n_blocks_of[s]):
                local_q_index[(g, s, b)] = len(layout.q_blocks)
                layout.q_blocks.append((g, s, b, n_tok(s, b)))
    local_kv_index: Dict[Tuple[int, int, int], int] = {}
    for g in range(n_hb_kv):
        for s in range(len(raw_seqlens)):
            for b in range(n_blocks_of[s]):
                local_kv_index[(g, s, b)] = len(layout.kv_blocks)
                layout.kv_blocks.append((g, s, b, n_tok(s, b)))
    cu = [0]
    for _, _, _, n in layout.q_blocks:
        cu.append(cu[-1] + n)
    layout.local_cu_seqlens = cu

    # BUFFER order: (sequence, head block, block), Q and KV in their own buffers
    q_slots, kv_slots = _Slots(), _Slots()
    buf_q: Dict[Tuple[int, int, int], int] = {}
    buf_kv: Dict[Tuple[int, int, int], int] = {}
    for s in range(len(raw_seqlens)):
        for g in range(n_hb_q):
            for b in range(n_blocks_of[s]):
                buf_q[(g, s, b)] = q_slots.take()
        for g in range(n_hb_kv):
            for b in range(n_blocks_of[s]):
                buf_kv[(g, s, b)] = kv_slots.take()

    seq_off = np.concatenate(([0], np.cumsum(raw_seqlens)))

    # rows: one per (sequence, q head block, q block) that attends anything
    @dataclass
    class Row:
        g: int
        s: int
        b: int
        kv_ids: List[int]

    rows: List[Row] = []
    local_masks: Dict[Tuple[int, int, int], np.ndarray] = {}  # (sequence, q block, kv block), "reference" only
    for s, L in enumerate(raw_seqlens):
        seq_mask = mask_np[seq_off[s] : seq_off[s + 1]]
        if work_units == "reference":
            units = generate_work_units(seq_mask, L, block_size)
            local_masks.update({(s, i, j): m for (i, j), m in units.items()})
            kv_of = rows_of_work_units(units)
        for b in range(n_blocks_of[s]):
            if work_units == "reference":
                kv_ids = kv_of.get(b, [])
            else:
                kv_ids = _block_overlaps(seq_mask, b * block_size, n_tok(s, b), block_size,
                                         n_blocks_of[s], L)
            for g in range(n_hb_q):
                rows.append(Row(g, s, b, kv_ids))
    rows.sort(key=lambda r: (r.s, r.g, r.b))

    def split(kv_ids: List[int]) -> List[List[int]]:
        if n_kv_groups == 1:
            return [kv_ids]
        if kv_split == "round_robin":
            return [kv_ids[i::n_kv_groups] for i in range(n_kv_groups)]
        per = (len(kv_ids) + n_kv_groups - 1) // n_kv_groups
        return [kv_ids[i * per : (i + 1) * per] for i in range(n_kv_groups)]

    def q_block(buffer_type, r: Row, slot):
        return BufferBlock(buffer_type, slot, n_tok(r.s, r.b))

    def attn_tables(stage: int):
        """Rows of one stage: (row, kv ids of the stage, mask planes)."""
        stage_rows = []
        for r in rows:
            ids = split(r.kv_ids)[stage]
            if ids:
                stage_rows.append((r, ids))
        return stage_rows

    def build_mask(stage_rows):
        planes = []
        for r, ids in stage_rows:
            seq_mask = mask_np[seq_off[r.s] : seq_off[r.s + 1]]
            if work_units == "reference":
                joined = concat_local_attn_masks([local_masks[(r.s, r.b, j)] for j in ids],
                                                 [n_tok(r.s, j) for j in ids], n_tok(r.s, r.b))
                plane = np.zeros(joined.shape[:2] + (block_size,), dtype=np.int32)
                plane[..., : joined.shape[2]] = joined
                planes.append(plane)
                continue
            planes.append(
                _row_ranges(seq_mask, r.b * block_size, n_tok(r.s, r.b), block_size, ids,
                            [n_tok(r.s, j) for j in ids])
            )
        m = np.concatenate(planes, axis=2)  # [n_ranges, 2, total_q]
        t = torch.from_numpy(m)
        return t[0] if t.shape[0] == 1 else t

    def kv_head_block(r: Row) -> int:
        return r.g // q_per_kv_block

    # ------------------------------------------------------------------ forward
    fw_instrs = []
    fw_instrs.append(
        MemcpyInstr(
            [
                (
                    BufferBlock(BufferType.LOCAL_Q, local_q_index[key], n_tok(key[1], key[2])),
                    BufferBlock(BufferType.BUFFER_Q, slot, n_tok(key[1], key[2])),
                )
                for key, slot in sorted(buf_q.items(), key=lambda kv: kv[1])
            ]
            + [
                (
                    BufferBlock(BufferType.LOCAL_KV, local_kv_index[key], n_tok(key[1], key[2])),
                    BufferBlock(BufferType.BUFFER_KV, slot, n_tok(key[1], key[2])),
                )
                for key, slot in sorted(buf_kv.items(), key=lambda kv: kv[1])
            ]
        )
    )
    out_slots = _Slots()
    partials: Dict[Tuple[int, int, int], List[int]] = {}
    for stage in range(n_kv_groups):
        stage_rows = attn_tables(stage)
        if not stage_rows:
            continue
        q_tab, kv_tab, out_tab, lse_tab = [], [], [], []
        fold_ops = []
        for r, ids in stage_rows:
            slot = out_slots.take()
            key = (r.g, r.s, r.b)
            q_tab.append([q_block(BufferType.BUFFER_Q, r, buf_q[key])])
            kv_tab.append(
                [
                    BufferBlock(BufferType.BUFFER_KV, buf_kv[(kv_head_block(r), r.s, j)], n_tok(r.s, j))
                    for j in ids
                ]
            )
            out_tab.append([q_block(BufferType.BUFFER_OUT, r, slot)])
            lse_tab.append([q_block(BufferType.BUFFER_LSE, r, slot)])
            if fold_stages and key in partials:
                first = partials[key][0]
                fold_ops.append(
                    ReductionOp(
                        [
                            (q_block(BufferType.BUFFER_OUT, r, first), q_block(BufferType.BUFFER_LSE, r, first)),
                            (q_block(BufferType.BUFFER_OUT, r, slot), q_block(BufferType.BUFFER_LSE, r, slot)),
                        ],
                        (q_block(BufferType.BUFFER_OUT, r, first), q_block(BufferType.BUFFER_LSE, r, first)),
                    )
                )
            else:
                partials.setdefault(key, []).append(slot)
        fw_instrs.append(
            AttnInstr(
                stage,
                [block_size] * len(stage_rows),
                [block_size * len(ids) for _, ids in stage_rows],
                block_size,
                block_size * max(len(ids) for _, ids in stage_rows),
                build_mask(stage_rows),
                q_tab,
                kv_tab,
                out_tab,
                lse_tab,
            )
        )
        if fold_ops:
            fw_instrs.append(AttnReductionInstr(fold_ops, output_is_unpadded=0))
    final_ops = []
    for r in rows:
        key = (r.g, r.s, r.b)
        srcs = partials.get(key, [])
        if not srcs:
            continue
        idx = local_q_index[key]
        final_ops.append(
            ReductionOp(
                [(q_block(BufferType.BUFFER_OUT, r, s_), q_block(BufferType.BUFFER_LSE, r, s_)) for s_ in srcs],
                (q_block(BufferType.LOCAL_OUT, r, idx), q_block(BufferType.LOCAL_LSE, r, idx)),
            )
        )
    fw_instrs.append(AttnReductionInstr(final_ops, output_is_unpadded=1))

    total_q_tokens = cu[-1]
    total_kv_tokens = sum(n for _, _, _, n in layout.kv_blocks)
    q_tok_shape = (hb, head_dim)
    kv_tok_shape = (2, hkv, head_dim)
    q_numel = block_size * hb * head_dim
    kv_numel = block_size * 2 * hkv * head_dim

    def local_info(n_blocks, total, tok_shape, numel, dt=wire_dtype):
        return BufferInfo(n_blocks, block_size, numel, dt, (total, *tok_shape), tok_shape)

    def slot_info(n_blocks, tok_shape, numel, dt=wire_dtype):
        return BufferInfo(n_blocks, block_size, numel, dt, (n_blocks, block_size, *tok_shape), tok_shape)

    def lse_local_info():
        return BufferInfo(len(layout.q_blocks), block_size, block_size * hb, DType.FLOAT32,
                          (hb, total_q_tokens), (1,))

    def lse_slot_info(n_blocks):
        return BufferInfo(n_blocks, block_size, block_size * hb, DType.FLOAT32,
                          (hb, n_blocks, block_size), (1,))

    fw_info = {
        BufferType.LOCAL_Q: local_info(len(layout.q_blocks), total_q_tokens, q_tok_shape, q_numel),
        BufferType.LOCAL_KV: local_info(len(layout.kv_blocks), total_kv_tokens, kv_tok_shape, kv_numel),
        BufferType.LOCAL_OUT: local_info(len(layout.q_blocks), total_q_tokens, q_tok_shape, q_numel),
        BufferType.LOCAL_LSE: lse_local_info(),
        BufferType.BUFFER_Q: slot_info(q_slots.n, q_tok_shape, q_numel),
        BufferType.BUFFER_KV: slot_info(kv_slots.n, kv_tok_shape, kv_numel),
        BufferType.BUFFER_OUT: slot_info(out_slots.n, q_tok_shape, q_numel),
        BufferType.BUFFER_LSE: lse_slot_info(out_slots.n),
    }
    fw_plan = ExecutionPlan(fw_instrs, 1, 1, 0, 0, n_kv_groups, cu, fw_info)
    if not backward:
        return fw_plan, None, layout

    # ----------------------------------------------------------------- backward
    bw_instrs = []
    # out / lse / dout of a q block share one slot index
    o_slots = _Slots()
    buf_o = {key: o_slots.take() for key, _ in sorted(buf_q.items(), key=lambda kv: kv[1])}
    pairs = []
    for key, slot in sorted(buf_q.items(), key=lambda kv: kv[1]):
        n = n_tok(key[1], key[2])
        li = local_q_index[key]
        pairs.append((BufferBlock(BufferType.LOCAL_Q, li, n), BufferBlock(BufferType.BUFFER_Q, slot, n)))
    for key, slot in sorted(buf_kv.items(), key=lambda kv: kv[1]):
        n = n_tok(key[1], key[2])
        pairs.append((BufferBlock(BufferType.LOCAL_KV, local_kv_index[key], n),
                      BufferBlock(BufferType.BUFFER_KV, slot, n)))
    for key, slot in sorted(buf_o.items(), key=lambda kv: kv[1]):
        n = n_tok(key[1], key[2])
        li = local_q_index[key]
        pairs.append((BufferBlock(BufferType.LOCAL_OUT, li, n), BufferBlock(BufferType.BUFFER_OUT, slot, n)))
        pairs.append((BufferBlock(BufferType.LOCAL_LSE, li, n), BufferBlock(BufferType.BUFFER_LSE, slot, n)))
        pairs.append((BufferBlock(BufferType.LOCAL_dOUT, li, n), BufferBlock(BufferType.BUFFER_dOUT, slot, n)))
    bw_instrs.append(MemcpyInstr(pairs))

    dq_slots, dkv_slots = _Slots(), _Slots()
    dq_versions: Dict[Tuple[int, int, int], List[int]] = {}
    dkv_replicas: Dict[Tuple[int, int, int], List[int]] = {}
    for stage in range(n_kv_groups):
        stage_rows = attn_tables(stage)
        if not stage_rows:
            continue
        q_tab, kv_tab, o_tab, dq_tab, dkv_tab = [], [], [], [], []
        for r, ids in stage_rows:
            key = (r.g, r.s, r.b)
            q_tab.append([q_block(BufferType.BUFFER_Q, r, buf_q[key])])
            kv_tab.append(
                [
                    BufferBlock(BufferType.BUFFER_KV, buf_kv[(kv_head_block(r), r.s, j)], n_tok(r.s, j))
                    for j in ids
                ]
            )
            o_tab.append([q_block(BufferType.BUFFER_OUT, r, buf_o[key])])
            dq_slot = dq_slots.take()
            dq_versions.setdefault(key, []).append(dq_slot)
            dq_tab.append([q_block(BufferType.BUFFER_dQ, r, dq_slot)])
            dkv_row = []
            for j in ids:
                slot = dkv_slots.take()
                dkv_replicas.setdefault((kv_head_block(r), r.s, j), []).append(slot)
                dkv_row.append(BufferBlock(BufferType.BUFFER_dKV, slot, n_tok(r.s, j)))
            dkv_tab.append(dkv_row)
        bw_instrs.append(
            AttnBackwardInstr(
                stage,
                [block_size] * len(stage_rows),
                [block_size * len(ids) for _, ids in stage_rows],
                block_size,
                block_size * max(len(ids) for _, ids in stage_rows),
                build_mask(stage_rows),
                q_tab,
                kv_tab,
                o_tab,
                dq_tab,
                dkv_tab,
            )
        )
    # in-buffer accumulation of replicas into the first one
    inner = []
    for key, slots in dq_versions.items():
        if len(slots) > 1:
            n = n_tok(key[1], key[2])
            inner.append(SumOp([BufferBlock(BufferType.BUFFER_dQ, s_, n) for s_ in slots],
                               BufferBlock(BufferType.BUFFER_dQ, slots[0], n)))
    if inner:
        bw_instrs.append(SumInstr(inner, output_is_unpadded=0))
    inner = []
    for key, slots in dkv_replicas.items():
        if len(slots) > 1:
            n = n_tok(key[1], key[2])
            inner.append(SumOp([BufferBlock(BufferType.BUFFER_dKV, s_, n) for s_ in slots],
                               BufferBlock(BufferType.BUFFER_dKV, slots[0], n)))
    if inner:
        bw_instrs.append(SumInstr(inner, output_is_unpadded=0))
    # scatter back
    final = []
    for key, li in local_q_index.items():
        n = n_tok(key[1], key[2])
        if key in dq_versions:
            final.append(SumOp([BufferBlock(BufferType.BUFFER_dQ, dq_versions[key][0], n)],
                               BufferBlock(BufferType.LOCAL_dQ, li, n)))
    if final:
        bw_instrs.append(SumInstr(final, output_is_unpadded=1))
    final = []
    for key, li in local_kv_index.items():
        n = n_tok(key[1], key[2])
        if key in dkv_replicas:
            final.append(SumOp([BufferBlock(BufferType.BUFFER_dKV, dkv_replicas[key][0], n)],
                               BufferBlock(BufferType.LOCAL_dKV, li, n)))
    if final:
        bw_instrs.append(SumInstr(final, output_is_unpadded=1))

    bw_info = {
        BufferType.LOCAL_Q: fw_info[BufferType.LOCAL_Q],
        BufferType.LOCAL_KV: fw_info[BufferType.LOCAL_KV],
        BufferType.LOCAL_OUT: fw_info[BufferType.LOCAL_OUT],
        BufferType.LOCAL_LSE: fw_info[BufferType.LOCAL_LSE],
        BufferType.LOCAL_dOUT: local_info(len(layout.q_blocks), total_q_tokens, q_tok_shape, q_numel),
        BufferType.LOCAL_dQ: local_info(len(layout.q_blocks), total_q_tokens, q_tok_shape, q_numel),
        BufferType.LOCAL_dKV: local_info(len(layout.kv_blocks), total_kv_tokens, kv_tok_shape, kv_numel),
        BufferType.BUFFER_Q: slot_info(q_slots.n, q_tok_shape, q_numel),
        BufferType.BUFFER_KV: slot_info(kv_slots.n, kv_tok_shape, kv_numel),
        BufferType.BUFFER_OUT: slot_info(o_slots.n, q_tok_shape, q_numel),
        BufferType.BUFFER_LSE: lse_slot_info(o_slots.n),
        BufferType.BUFFER_dOUT: slot_info(o_slots.n, q_tok_shape, q_numel),
        BufferType.BUFFER_dQ: slot_info(dq_slots.n, q_tok_shape, q_numel),
        BufferType.BUFFER_dKV: slot_info(dkv_slots.n, kv_tok_shape, kv_numel),
    }
    bw_plan = ExecutionPlan(bw_instrs, 1, 1, 0, 0, n_kv_groups, cu, bw_info)
    return fw_plan, bw_plan, layout
