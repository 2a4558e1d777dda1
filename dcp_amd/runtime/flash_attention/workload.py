"""Work units of one sequence and their block-local masks: the form in which the
reference's dataloader hands attention work to its scheduler, and the scheduler's way
back from block-local masks to the per-row ranges an ``AttnInstr`` carries.

A work unit is one (q block i, kv block j) pair of a sequence.  Its mask holds, per
query token of block i, the token's range(s) clipped to kv block j and counted from
the block's first key; pairs that no query of the block can attend are not work
units at all (``dcp/data/dataloader.py:1384-1546``, ``_generate_workload``).  A row of
an attention instruction is a q block with the kv blocks of its work units
concatenated in block order; the row's ranges are the work units' masks shifted by
the keys before them and joined, which must give one contiguous range per plane
(``dcp/core/scheduler.py:1143-1185``, ``_concat_attn_mask``).

``single_device.py`` goes from the sequence mask to the row ranges in one step
(``_block_overlaps``, ``_row_ranges``); the two routes are checked against each other
and against a dense boolean mask in ``tests/test_workload.py``.  One difference is
kept on purpose and tested: the reference decides whether a pair is a work unit from
the HULL of the block's ranges (smallest start, largest end), so it keeps pairs whose
every query is masked out when ranges of different queries straddle the kv block;
such a unit has only empty ranges and adds nothing to the result.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np


def local_attn_mask(seq_mask: np.ndarray, i: int, j: int, block_size: int, padded_seqlen: int) -> Optional[np.ndarray]:
    """Mask of work unit (q block ``i``, kv block ``j``) of a sequence whose
    per-token ranges are ``seq_mask`` (``[L, 2]`` or ``[L, 2, 2]``: token, [range,]
    start/end), or ``None`` when the pair is no work unit.  int32
    ``[2, block_size]`` (start plane, end plane) or ``[2, 2, block_size]`` (range,
    plane); entries past the q block's tokens stay -1, as in the reference."""
    rows = np.asarray(seq_mask)[i * block_size : min((i + 1) * block_size, padded_seqlen)].astype(np.int64)
    n_q = rows.shape[0]
    lo, hi = j * block_size, min((j + 1) * block_size, padded_seqlen)
    if rows.ndim == 2:
        if n_q == 0 or rows[:, 0].min() >= hi or rows[:, 1].max() <= lo:
            return None
        out = np.full((2, block_size), -1, dtype=np.int32)
        # the start is only raised to the block's first key (a start past the block then lies
        # past the clipped end: an empty range), the end only lowered to its last
        out[0, :n_q] = np.maximum(np.maximum(rows[:, 0], lo) - lo, 0)
        out[1, :n_q] = np.maximum(np.minimum(rows[:, 1], hi) - lo, 0)
        return out
    assert rows.ndim == 3 and rows.shape[1:] == (2, 2), "ranges are [L, 2] or [L, 2, 2]"
    overlaps = False
    for r in range(2):
        valid = rows[:, r, 0] < rows[:, r, 1]
        if valid.any():
            overlaps |= min(hi, rows[valid, r, 1].max()) > max(lo, rows[valid, r, 0].min())
    if not overlaps:
        return None
    out = np.full((2, 2, block_size), -1, dtype=np.int32)
    for r in range(2):
        out[r, 0, :n_q] = np.clip(rows[:, r, 0], lo, hi) - lo
        out[r, 1, :n_q] = np.clip(rows[:, r, 1], lo, hi) - lo
    return out


def generate_work_units(seq_mask: np.ndarray, seqlen: int, block_size: int,
                        causal: bool = False) -> Dict[Tuple[int, int], np.ndarray]:
    """All work units of one sequence: ``{(i, j): local mask}`` in the reference's
    order (q blocks outermost; ``causal`` restricts j to 0..i before looking at the
    mask, as ``_generate_workload`` does)."""
    n_blocks = (seqlen + block_size - 1) // block_size
    units: Dict[Tuple[int, int], np.ndarray] = {}
    for i in range(n_blocks):
        for j in range(i + 1 if causal else n_blocks):
            m = local_attn_mask(seq_mask, i, j, block_size, seqlen)
            if m is not None:
                units[(i, j)] = m
    return units


def concat_local_attn_masks(local_masks: Sequence[np.ndarray], kv_n_tokens: Sequence[int], q_seqlen: int) -> np.ndarray:
    """Row ranges from the masks of a row's work units, given in kv block order with
    the number of keys each kv block contributes: int32 ``[n_ranges, 2, q_seqlen]``,
    queries that attend nothing get ``[0, 0)``.  Raises ``AssertionError``
    ("Discontinuous attn mask") when a query's pieces do not join up."""
    assert len(local_masks) == len(kv_n_tokens) and len(local_masks) > 0
    planes = [np.asarray(m)[None] if np.asarray(m).ndim == 2 else np.asarray(m) for m in local_masks]
    n_ranges = planes[0].shape[0]
    out = np.zeros((n_ranges, 2, q_seqlen), dtype=np.int32)
    for r in range(n_ranges):
        start = np.full(q_seqlen, -1, dtype=np.int64)
        end = np.full(q_seqlen, -1, dtype=np.int64)
        before = 0
        for m, n_keys in zip(planes, kv_n_tokens):
            s, e = m[r, 0, :q_seqlen].astype(np.int64), m[r, 1, :q_seqlen].astype(np.int64)
            valid = e > s
            assert ((start == -1) | (s + before == end) | ~valid).all(), "Discontinuous attn mask"
            first = valid & (start == -1)
            start[first] = s[first] + before
            end[valid] = e[valid] + before
            before += int(n_keys)
        nothing = start == -1
        start[nothing] = 0
        end[nothing] = 0
        out[r, 0], out[r, 1] = start, end
    return out


def rows_of_work_units(units: Dict[Tuple[int, int], np.ndarray]) -> Dict[int, List[int]]:
    """``{q block: kv blocks of its work units, ascending}``."""
    rows: Dict[int, List[int]] = {}
    for i, j in units:
        rows.setdefault(i, []).append(j)
    return {i: sorted(js) for i, js in rows.items()}
