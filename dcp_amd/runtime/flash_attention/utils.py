"""Attention-mask generators: per-token ``[start, end)`` range lists.

Same outputs as the reference's generators in
``dcp/runtime/flash_attention/utils.py`` (``lambda_mask_fn`` :501-525,
``causal_range_mask_fn`` :528-542, ``shared_question_mask_fn`` :545-592,
``causal_blockwise_mask_fn`` :595-633, ``modality_specific_mask_fn``
:636-683), computed with closed forms over ``arange`` instead of a Python
loop per token.  A mask is an integer tensor ``[sum(padded_seqlens), 2]`` (one
range per token) or ``[sum(padded_seqlens), 2, 2]`` (two ranges; axis 1 is the
range, axis 2 start/end) in sequence-local key positions; rows of padding
tokens stay ``[0, 0)``.  A token attends to the union of its ranges.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import numpy as np
import torch


def _offsets(padded_seqlens: Sequence[int]) -> np.ndarray:
    return np.concatenate(([0], np.cumsum(np.asarray(padded_seqlens, dtype=np.int64))))


def _finish(mask: np.ndarray, mask_dtype: torch.dtype) -> torch.Tensor:
    return torch.from_numpy(mask).to(mask_dtype)


def causal_range_mask_fn(
    raw_seqlens: List[int],
    padded_seqlens: List[int],
    mask_dtype: torch.dtype,
    mask_fn_info: Optional[List[Dict]] = None,
):
    """Token i attends ``[0, i+1)``."""
    off = _offsets(padded_seqlens)
    mask = np.zeros((int(off[-1]), 2), dtype=np.int64)
    for seq_id, seqlen in enumerate(raw_seqlens):
        i = np.arange(seqlen)
        mask[off[seq_id] + i, 1] = i + 1
    return _finish(mask, mask_dtype)


def lambda_mask_fn(
    raw_seqlens: List[int],
    padded_seqlens: List[int],
    mask_dtype: torch.dtype,
    mask_fn_info: Optional[List[Dict]] = None,
    n_starting: int = 64,
    l_pretrain: int = 4096,
):
    """Attention sink plus sliding window: token i attends
    ``[0, min(n_starting, i+1))`` and ``[max(0, i-l_pretrain+1), i+1)``."""
    off = _offsets(padded_seqlens)
    mask = np.zeros((int(off[-1]), 2, 2), dtype=np.int64)
    for seq_id, seqlen in enumerate(raw_seqlens):
        i = np.arange(seqlen)
        rows = off[seq_id] + i
        mask[rows, 0, 1] = np.minimum(n_starting, i + 1)
        mask[rows, 1, 0] = np.maximum(0, i - l_pretrain + 1)
        mask[rows, 1, 1] = i + 1
    return _finish(mask, mask_dtype)


def shared_question_mask_fn(
    raw_seqlens: List[int],
    padded_seqlens: List[int],
    mask_dtype: torch.dtype,
    mask_fn_info: Optional[List[Dict]] = None,
    question_proportion: float = 0.2,
    n_answers: int = 4,
):
    """One question followed by ``n_answers`` independent answers: question
    tokens are causal (second range empty at ``[i+1, i+1)``); an answer token
    sees the whole question and its own answer causally."""
    off = _offsets(padded_seqlens)
    mask = np.zeros((int(off[-1]), 2, 2), dtype=np.int64)
    for seq_id, seqlen in enumerate(raw_seqlens):
        n_q = int(seqlen * question_proportion)
        per_answer = (seqlen - n_q) // n_answers
        i = np.arange(seqlen)
        rows = off[seq_id] + i
        is_q = i < n_q
        last_start = n_q + (n_answers - 1) * per_answer
        if per_answer > 0:
            regular = (i - n_q) // per_answer * per_answer + n_q
        else:
            regular = np.full_like(i, last_start)
        answer_start = np.where(i < last_start, regular, last_start)
        mask[rows, 0, 0] = 0
        mask[rows, 0, 1] = np.where(is_q, i + 1, n_q)
        mask[rows, 1, 0] = np.where(is_q, i + 1, answer_start)
        mask[rows, 1, 1] = i + 1
    return _finish(mask, mask_dtype)


def causal_blockwise_mask_fn(
    raw_seqlens: List[int],
    padded_seqlens: List[int],
    mask_dtype: torch.dtype,
    mask_fn_info: Optional[List[Dict]] = None,
    block_size: int = 256,
    k_local: int = 2,
):
    """First block causal; last block sees everything before it; blocks in
    between see the first block plus a local window of ``k_local`` blocks."""
    off = _offsets(padded_seqlens)
    mask = np.zeros((int(off[-1]), 2, 2), dtype=np.int64)
    for seq_id, seqlen in enumerate(raw_seqlens):
        i = np.arange(seqlen)
        rows = off[seq_id] + i
        blk = i // block_size
        n_blocks = (seqlen + block_size - 1) // block_size
        first = blk == 0
        last = (blk == n_blocks - 1) & ~first
        prev_end_last = (blk - 1) * block_size
        prev_end_mid = np.maximum(block_size, i - k_local * block_size)
        mask[rows, 0, 0] = 0
        mask[rows, 0, 1] = np.where(first, i + 1, np.where(last, prev_end_last, block_size))
        mask[rows, 1, 0] = np.where(first, i + 1, np.where(last, prev_end_last, prev_end_mid))
        mask[rows, 1, 1] = i + 1
    return _finish(mask, mask_dtype)


def modality_specific_mask_fn(
    raw_seqlens: List[int],
    padded_seqlens: List[int],
    mask_dtype: torch.dtype,
    mask_fn_info: Optional[List[Dict]] = None,
    limit_image_attn_to_self: bool = False,
):
    """Text tokens are causal; the tokens of an image (inserted between text
    segments) attend bidirectionally inside the image and, unless
    ``limit_image_attn_to_self``, causally to everything before it."""
    assert mask_fn_info is not None
    assert len(mask_fn_info) == len(raw_seqlens)
    off = _offsets(padded_seqlens)
    mask = np.zeros((int(off[-1]), 2), dtype=np.int64)
    for seq_id in range(len(raw_seqlens)):
        info = mask_fn_info[seq_id]
        image_size = info["image_size"]
        text_lengths = info["text_lengths"]
        pos = 0
        for idx, text_len in enumerate(text_lengths):
            i = np.arange(text_len)
            mask[off[seq_id] + pos + i, 1] = pos + i + 1
            pos += text_len
            if idx < len(text_lengths) - 1:
                rows = off[seq_id] + pos + np.arange(image_size)
                mask[rows, 0] = pos if limit_image_attn_to_self else 0
                mask[rows, 1] = pos + image_size
                pos += image_size
    return _finish(mask, mask_dtype)


def shared_prefix_mask_fn(
    raw_seqlens: List[int],
    padded_seqlens: List[int],
    mask_dtype: torch.dtype,
    mask_fn_info: Optional[List[Dict]] = None,
):
    """One shared prefix followed by independent continuations of given
    lengths (``mask_fn_info[s] = {"prefix": p, "continuations": [c0, ...]}``,
    ``p + sum(c) == raw_seqlens[s]``).  Prefix tokens are causal; a
    continuation token sees the whole prefix and its own continuation
    causally.  This is the shared-question mask of the reference
    (``utils.py:545-592``) with explicit, unequal answer lengths."""
    assert mask_fn_info is not None
    off = _offsets(padded_seqlens)
    mask = np.zeros((int(off[-1]), 2, 2), dtype=np.int64)
    for seq_id, seqlen in enumerate(raw_seqlens):
        info = mask_fn_info[seq_id]
        prefix = int(info["prefix"])
        conts = [int(c) for c in info["continuations"]]
        assert prefix + sum(conts) == seqlen, (prefix, conts, seqlen)
        i = np.arange(prefix)
        rows = off[seq_id] + i
        mask[rows, 0, 1] = i + 1
        mask[rows, 1, 0] = i + 1
        mask[rows, 1, 1] = i + 1
        start = prefix
        for c in conts:
            i = start + np.arange(c)
            rows = off[seq_id] + i
            mask[rows, 0, 1] = prefix
            mask[rows, 1, 0] = start
            mask[rows, 1, 1] = i + 1
            start += c
    return _finish(mask, mask_dtype)


MASK_FNS = {
    "causal": causal_range_mask_fn,
    "lambda": lambda_mask_fn,
    "shared_question": shared_question_mask_fn,
    "causal_blockwise": causal_blockwise_mask_fn,
    "modality_specific": modality_specific_mask_fn,
    "shared_prefix": shared_prefix_mask_fn,
}


def count_attended_pairs(mask: torch.Tensor) -> int:
    """Number of (query, key) pairs a range mask lets through (size of the
    union of the token's ranges, summed over tokens)."""
    m = mask.to(torch.int64)
    if m.dim() == 2:
        return int(torch.clamp(m[:, 1] - m[:, 0], min=0).sum())
    s0, e0, s1, e1 = m[:, 0, 0], m[:, 0, 1], m[:, 1, 0], m[:, 1, 1]
    l0 = torch.clamp(e0 - s0, min=0)
    l1 = torch.clamp(e1 - s1, min=0)
    inter = torch.clamp(torch.minimum(e0, e1) - torch.maximum(s0, s1), min=0)
    inter = torch.where((l0 > 0) & (l1 > 0), inter, torch.zeros_like(inter))
    return int((l0 + l1 - inter).sum())
