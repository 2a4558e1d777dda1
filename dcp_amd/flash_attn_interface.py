"""Range-masked paged variable-length attention: the two functions the
reference executor imports from its flash-attention fork
(``dcp_flash_attn.flash_attn_interface._flash_attn_varlen_forward`` /
``_flash_attn_varlen_backward``, called at
``dcp/runtime/flash_attention/executor.py:161-184`` and ``:303-334``), with the
same argument order, backed by the gfx950 kernels of ``libdcp_hip.so``.

Only the configuration the executor uses is implemented: no dropout, no causal
flag, no sliding window, no softcap, no alibi; masking comes from
``attn_range`` and all tensors are paged through block tables.  Anything else
raises ``NotImplementedError`` rather than computing something different.
"""

from __future__ import annotations

from typing import Optional

import torch

from dcp_amd import _lib
from dcp_amd.ops.fused_ops import dtype_code

__all__ = [
    "_flash_attn_varlen_forward",
    "forward_workspace",
    "_flash_attn_varlen_backward",
    "backward_workspace_bytes",
]


def backward_workspace_bytes(batch, total_q, block_size, n_heads_q, head_dim, total_k=0) -> int:
    """Scratch bytes ``_flash_attn_varlen_backward`` needs for these sizes with the backward that is
    selected now (``dcp_attn_bwd_select``).  ``total_k``: the sum of the rows' key counts; without
    it the backward that keeps dS in memory cannot be taken (the call then recomputes instead)."""
    return int(_lib.load().dcp_attn_bwd_workspace_bytes_kv(
        int(batch), int(total_q), int(total_k), int(block_size), int(n_heads_q), int(head_dim)))


def forward_workspace(device="cuda") -> torch.Tensor:
    """A work-counter buffer for ``_flash_attn_varlen_forward`` (contents are overwritten by
    every launch); one buffer serves all launches that follow each other on one stream."""
    n = int(_lib.load().dcp_attn_fwd_workspace_bytes())
    return torch.empty((n + 3) // 4, dtype=torch.int32, device=device)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _check_plain(dropout_p, causal, window_size_left, window_size_right, softcap,
                 alibi_slopes, return_softmax=False):
    if dropout_p != 0.0:
        raise NotImplementedError("dropout is not supported")
    if causal:
        raise NotImplementedError("use attn_range instead of the causal flag")
    if window_size_left != -1 or window_size_right != -1:
        raise NotImplementedError("use attn_range instead of window_size")
    if softcap != 0.0:
        raise NotImplementedError("softcap is not supported")
    if alibi_slopes is not None:
        raise NotImplementedError("alibi is not supported")
    if return_softmax:
        raise NotImplementedError("return_softmax is not supported")


def _i32(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.dtype != torch.int32 or not t.is_cuda or not t.is_contiguous():
        raise ValueError(f"{name} must be a contiguous int32 device tensor")
    return t


def _kv_strides(k: torch.Tensor, v: torch.Tensor, name: str):
    """k and v are [n_slots, block_size, n_heads_kv, D] views (typically the
    two halves of a [n_slots, block_size, 2, n_heads_kv, D] buffer)."""
    if k.shape != v.shape or k.stride() != v.stride():
        raise ValueError(f"{name}: k and v must have the same shape and strides")
    if k.dim() == 3:  # unpadded [tokens, n_heads_kv, D]: a table entry is a token offset
        if k.stride(2) != 1 or k.stride(1) != k.shape[2]:
            raise ValueError(f"{name}: k/v head and feature axes must be dense")
        return k.stride(0), k.stride(0)
    if k.dim() != 4:
        raise ValueError(f"{name}: k/v must be paged [n_slots, block_size, n_heads_kv, D] or unpadded [tokens, n_heads_kv, D]")
    if k.stride(3) != 1 or k.stride(2) != k.shape[3]:
        raise ValueError(f"{name}: k/v head and feature axes must be dense")
    return k.stride(0), k.stride(1)


def _paged_or_tokens(t: torch.Tensor, name: str, block_size):
    """``(block_size, stride of a table entry in elements)`` of a q-like tensor: paged
    ``[n_slots, block_size, H, D]`` (a table entry is a slot) or unpadded ``[tokens, H, D]`` (a table
    entry is a token offset; ``block_size`` then has to be given)."""
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if t.dim() == 4:
        if block_size is not None and block_size != t.shape[1]:
            raise ValueError(f"{name}: block size {t.shape[1]} differs from {block_size}")
        return t.shape[1], t.shape[1] * t.shape[2] * t.shape[3]
    if t.dim() == 3:
        if block_size is None:
            raise ValueError(f"{name} is unpadded [tokens, H, D]: block_size must be given")
        return block_size, t.shape[1] * t.shape[2]
    raise ValueError(f"{name} must be [n_slots, block_size, H, D] or [tokens, H, D]")


def _lse_strides(lse: torch.Tensor, out: torch.Tensor, block_size: int, name: str):
    """``(head stride, entry stride)`` of an LSE tensor that goes with ``out``: ``[H, n_slots,
    block_size]`` beside a paged out, ``[H, tokens]`` beside an unpadded one."""
    if lse.dtype != torch.float32 or not lse.is_contiguous():
        raise ValueError(f"{name} must be contiguous float32")
    n_heads = out.shape[-2]
    if out.dim() == 4:
        if tuple(lse.shape) != (n_heads, out.shape[0], block_size):
            raise ValueError(f"{name} shape {tuple(lse.shape)} does not match out")
        return out.shape[0] * block_size, block_size
    if tuple(lse.shape) != (n_heads, out.shape[0]):
        raise ValueError(f"{name} shape {tuple(lse.shape)} does not match the unpadded out")
    return out.shape[0], 1


def _check_tables(batch, cu_seqlens_k, row_order, single, wide):
    """The kernels index the block tables by row and, for the wide ones, with one common width:
    a table of another shape would be read out of bounds or at the wrong slots."""
    if cu_seqlens_k.numel() != batch + 1:
        raise ValueError(f"cu_seqlens_k must have {batch + 1} entries like cu_seqlens_q, got {cu_seqlens_k.numel()}")
    for name, t in single.items():
        if tuple(t.shape) != (batch, 1):
            raise ValueError(f"{name} must be [{batch}, 1], got {tuple(t.shape)}")
    width = None
    for name, t in wide.items():
        if t.dim() != 2 or t.shape[0] != batch or t.shape[1] < 1:
            raise ValueError(f"{name} must be [{batch}, max_blocks], got {tuple(t.shape)}")
        if width is not None and t.shape[1] != width:
            raise ValueError(f"{name} must have the width of kv_block_table ({width}), got {tuple(t.shape)}")
        width = t.shape[1]
    if row_order is not None and row_order.numel() != batch:
        raise ValueError(f"row_order must have {batch} entries, got {row_order.numel()}")


KERNEL_HEAD_DIMS = (64, 128)


def _kernel_head_dim(head_dim: int) -> int:
    """The head size the kernels run a given head size at."""
    for d in KERNEL_HEAD_DIMS:
        if head_dim <= d:
            return d
    raise ValueError(f"head size {head_dim} is above the largest supported one ({KERNEL_HEAD_DIMS[-1]})")


def _widen(t: torch.Tensor, d: int, slack_tokens: int = 0) -> torch.Tensor:
    """A dense copy of ``t`` with its last axis zero-padded to ``d``.  An unpadded tensor
    (``[tokens, H, D]``) also gets ``slack_tokens`` zeroed tokens of storage behind its last one,
    which the result does not show: the kernels load whole tiles past a ragged last block."""
    if t.dim() == 3 and slack_tokens > 0:
        wide = torch.nn.functional.pad(t, (0, d - t.shape[-1], 0, 0, 0, slack_tokens))
        return wide[: t.shape[0]]
    return torch.nn.functional.pad(t, (0, d - t.shape[-1]))


def _range_arg(attn_range: torch.Tensor, total_q: int):
    _i32(attn_range, "attn_range")
    if attn_range.dim() == 2 and tuple(attn_range.shape) == (2, total_q):
        return 1
    if attn_range.dim() == 3 and tuple(attn_range.shape) == (2, 2, total_q):
        return 2
    raise ValueError(
        f"attn_range must be [2, {total_q}] or [2, 2, {total_q}], got {tuple(attn_range.shape)}"
    )


def _flash_attn_varlen_forward(
    q,
    k,
    v,
    cu_seqlens_q,
    cu_seqlens_k,
    total_q,
    max_seqlen_q,
    max_seqlen_k,
    dropout_p,
    softmax_scale,
    causal=False,
    window_size_left=-1,
    window_size_right=-1,
    softcap=0.0,
    alibi_slopes=None,
    return_softmax=False,
    attn_range=None,
    q_block_table=None,
    kv_block_table=None,
    out_block_table=None,
    out_=None,
    lse_=None,
    row_order: Optional[torch.Tensor] = None,
    workspace: Optional[torch.Tensor] = None,
    block_size: Optional[int] = None,
    merged_form: bool = False,
):
    """Writes the row outputs into ``out_`` / ``lse_`` in place and returns
    ``(out_, lse_, None, None)`` (the reference returns
    ``out_padded, softmax_lse, S_dmask, rng_state``).

    q ``[n_slots, bs, H, D]``; k, v ``[n_slots, bs, Hkv, D]`` views; block
    tables int32 ``[B, 1]`` (q, out) and ``[B, max_blocks]`` (kv, padded with
    -1); ``attn_range`` int32 ``[2, total_q]`` or ``[2, 2, total_q]``;
    ``out_`` like q; ``lse_`` fp32 ``[H, n_out_slots, bs]``.
    ``row_order`` (extension): launch order of the rows, longest first.
    ``workspace`` (extension): a buffer from ``forward_workspace()``; pass one to keep the call
    allocation-free (e.g. under graph capture), otherwise it is allocated here.
    ``block_size`` (extension): any of q, k/v, out_ (with lse_) may instead be the UNPADDED tensor
    (``[tokens, H, D]``; lse_ ``[H, tokens]``), its block table then holding token offsets; the
    block size, which no paged tensor may be left to tell, is then given here.  k/v must be
    readable for ``block_size`` tokens from every table entry on (the kernel loads whole blocks).
    ``merged_form`` (extension): queries without a visible key get ``lse = -1`` (what the merge
    leaves for a row with no finite source) instead of ``+inf``.
    """
    _check_plain(dropout_p, causal, window_size_left, window_size_right, softcap,
                 alibi_slopes, return_softmax)
    if attn_range is None or q_block_table is None or kv_block_table is None \
            or out_block_table is None or out_ is None or lse_ is None:
        raise NotImplementedError(
            "only the paged, range-masked, in-place form is implemented")
    if k.dim() == 4:
        block_size = k.shape[1] if block_size is None else block_size
        if block_size != k.shape[1]:
            raise ValueError(f"k/v: block size {k.shape[1]} differs from {block_size}")
    block_size, q_entry = _paged_or_tokens(q, "q", block_size)
    _, out_entry = _paged_or_tokens(out_, "out_", block_size)
    n_heads_q, head_dim = q.shape[-2], q.shape[-1]
    n_heads_kv = k.shape[-2]
    lse_head_stride, lse_entry = _lse_strides(lse_, out_, block_size, "lse_")
    kv_slot_stride, kv_token_stride = _kv_strides(k, v, "forward")
    n_ranges = _range_arg(attn_range, total_q)
    batch = cu_seqlens_q.numel() - 1
    _check_tables(batch, cu_seqlens_k, row_order, dict(q_block_table=q_block_table, out_block_table=out_block_table),
                  dict(kv_block_table=kv_block_table))
    if softmax_scale is None:
        softmax_scale = head_dim ** (-0.5)
    if head_dim not in KERNEL_HEAD_DIMS:
        # Any other head size runs at the next kernel head size on zero-padded copies, like the
        # reference pads head sizes that are not multiples of 8 (dcp/runtime/flash_attention/
        # executor.py:156-160): zero columns add nothing to a score, and the scale is already
        # fixed.  A compatibility path: it allocates and copies whole buffers on every call.
        d = _kernel_head_dim(head_dim)
        out_wide = _widen(out_, d)  # carries the slots this call does not write
        _flash_attn_varlen_forward(
            _widen(q, d, block_size), _widen(k, d, block_size), _widen(v, d, block_size), cu_seqlens_q, cu_seqlens_k, total_q, max_seqlen_q, max_seqlen_k,
            dropout_p, softmax_scale, attn_range=attn_range, q_block_table=q_block_table, kv_block_table=kv_block_table,
            out_block_table=out_block_table, out_=out_wide, lse_=lse_, row_order=row_order, workspace=workspace,
            block_size=block_size, merged_form=merged_form)
        out_.copy_(out_wide[..., :head_dim])
        return out_, lse_, None, None
    if workspace is None:
        workspace = forward_workspace(q.device)
    if workspace.dtype != torch.int32 or not workspace.is_contiguous():
        raise ValueError("workspace must be a contiguous int32 tensor from forward_workspace()")
    _lib.call(
        "dcp_attn_fwd_strided",
        q.data_ptr(), k.data_ptr(), v.data_ptr(), out_.data_ptr(), lse_.data_ptr(),
        _i32(cu_seqlens_q, "cu_seqlens_q").data_ptr(),
        _i32(cu_seqlens_k, "cu_seqlens_k").data_ptr(),
        attn_range.data_ptr(), n_ranges,
        _i32(q_block_table, "q_block_table").data_ptr(),
        _i32(kv_block_table, "kv_block_table").data_ptr(),
        _i32(out_block_table, "out_block_table").data_ptr(),
        0 if row_order is None else _i32(row_order, "row_order").data_ptr(),
        batch, kv_block_table.shape[1], int(total_q), block_size,
        n_heads_q, n_heads_kv, head_dim,
        kv_slot_stride, kv_token_stride, q_entry, out_entry, lse_head_stride, lse_entry,
        1 if merged_form else 0, float(softmax_scale), dtype_code(q.dtype),
        workspace.data_ptr(), workspace.numel() * 4, _stream(),
    )
    return out_, lse_, None, None


def _flash_attn_varlen_backward(
    dout,
    q,
    k,
    v,
    out,
    softmax_lse,
    dq,
    dk,
    dv,
    cu_seqlens_q,
    cu_seqlens_k,
    total_q,
    total_k,
    max_seqlen_q,
    max_seqlen_k,
    dropout_p,
    softmax_scale,
    causal,
    window_size_left,
    window_size_right,
    softcap,
    alibi_slopes,
    deterministic,
    attn_range=None,
    q_block_table=None,
    kv_block_table=None,
    out_block_table=None,
    dq_block_table=None,
    dkv_block_table=None,
    rng_state=None,
    workspace: Optional[torch.Tensor] = None,
    row_order: Optional[torch.Tensor] = None,
    block_size: Optional[int] = None,
):
    """Writes dQ into ``dq`` (slots ``dq_block_table``) and dK/dV into
    ``dk``/``dv`` (one slot per (row, kv block), ``dkv_block_table``).
    dK/dV of a kv head are summed over the q heads of its group inside the
    kernel, and the slots of a row's kv positions below its key count rounded up
    to 32 are written whole (zeros where no query attends), so ``dk``/``dv`` need
    not be zeroed when the key count is a multiple of the block size, as in
    every plan.  Slot padding of q/k/v/out/dout may hold anything finite whose
    dot products with the data stay finite; it is masked, not read as zero.

    ``workspace`` is scratch of ``backward_workspace_bytes(...)`` bytes (any
    dtype, contiguous); pass a preallocated tensor to keep the call
    allocation-free (e.g. under graph capture), otherwise it is allocated
    here.
    ``block_size`` (extension): as in the forward, q, k/v, out with dout and softmax_lse, and dq may
    each be the unpadded tensor, addressed by token offsets in its block table.  q and dout must
    then be readable for 64 tokens past the last row's queries (the dK/dV kernel loads whole
    64-query tiles).  dk/dv are always paged.
    """
    _check_plain(dropout_p, causal, window_size_left, window_size_right, softcap, alibi_slopes)
    if attn_range is None or q_block_table is None or kv_block_table is None \
            or out_block_table is None or dq_block_table is None or dkv_block_table is None:
        raise NotImplementedError(
            "only the paged, range-masked form is implemented")
    if dk.dim() != 4:
        raise ValueError("dk/dv must be paged [n_slots, block_size, n_heads_kv, D]")
    block_size = dk.shape[1] if block_size is None else block_size
    if block_size != dk.shape[1] or (k.dim() == 4 and k.shape[1] != block_size):
        raise ValueError(f"k/v/dk/dv: block sizes differ from {block_size}")
    _, q_entry = _paged_or_tokens(q, "q", block_size)
    _, out_entry = _paged_or_tokens(out, "out", block_size)
    _, dq_entry = _paged_or_tokens(dq, "dq", block_size)
    if dout.shape != out.shape or not dout.is_contiguous():
        raise ValueError("dout must be contiguous and shaped like out (they share out_block_table)")
    n_heads_q, head_dim = q.shape[-2], q.shape[-1]
    n_heads_kv = k.shape[-2]
    lse_head_stride, lse_entry = _lse_strides(softmax_lse, out, block_size, "softmax_lse")
    kv_slot_stride, kv_token_stride = _kv_strides(k, v, "backward k/v")
    dkv_slot_stride, dkv_token_stride = _kv_strides(dk, dv, "backward dk/dv")
    n_ranges = _range_arg(attn_range, total_q)
    batch = cu_seqlens_q.numel() - 1
    _check_tables(batch, cu_seqlens_k, row_order,
                  dict(q_block_table=q_block_table, out_block_table=out_block_table, dq_block_table=dq_block_table),
                  dict(kv_block_table=kv_block_table, dkv_block_table=dkv_block_table))
    if softmax_scale is None:
        softmax_scale = head_dim ** (-0.5)
    if head_dim not in KERNEL_HEAD_DIMS:
        # as in the forward: zero-padded copies at the next kernel head size; the gradients'
        # padded columns come out zero and are dropped, slots this call leaves alone are carried
        d = _kernel_head_dim(head_dim)
        dq_wide, dk_wide, dv_wide = _widen(dq, d, block_size), _widen(dk, d), _widen(dv, d)
        _flash_attn_varlen_backward(
            _widen(dout, d, block_size), _widen(q, d, block_size), _widen(k, d, block_size), _widen(v, d, block_size),
            _widen(out, d, block_size), softmax_lse, dq_wide, dk_wide,
            dv_wide, cu_seqlens_q, cu_seqlens_k, total_q, total_k, max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale,
            causal, window_size_left, window_size_right, softcap, alibi_slopes, deterministic, attn_range=attn_range,
            q_block_table=q_block_table, kv_block_table=kv_block_table, out_block_table=out_block_table,
            dq_block_table=dq_block_table, dkv_block_table=dkv_block_table, workspace=workspace, row_order=row_order,
            block_size=block_size)
        dq.copy_(dq_wide[..., :head_dim])
        dk.copy_(dk_wide[..., :head_dim])
        dv.copy_(dv_wide[..., :head_dim])
        return dq, dk, dv, None
    # (a caller's workspace may be the smaller one of the recomputing backward: the call then takes that one)
    need = backward_workspace_bytes(batch, int(total_q), block_size, n_heads_q, head_dim)
    if workspace is None:
        workspace = torch.empty(backward_workspace_bytes(batch, int(total_q), block_size, n_heads_q, head_dim, int(total_k or 0)),
                                dtype=torch.uint8, device=q.device)
    ws_bytes = workspace.numel() * workspace.element_size()
    if not workspace.is_contiguous() or ws_bytes < need:
        raise ValueError(f"workspace must be contiguous with at least {need} bytes")
    _lib.call(
        "dcp_attn_bwd_strided",
        dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
        softmax_lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
        workspace.data_ptr(), ws_bytes,
        _i32(cu_seqlens_q, "cu_seqlens_q").data_ptr(),
        _i32(cu_seqlens_k, "cu_seqlens_k").data_ptr(),
        attn_range.data_ptr(), n_ranges,
        _i32(q_block_table, "q_block_table").data_ptr(),
        _i32(kv_block_table, "kv_block_table").data_ptr(),
        _i32(out_block_table, "out_block_table").data_ptr(),
        _i32(dq_block_table, "dq_block_table").data_ptr(),
        _i32(dkv_block_table, "dkv_block_table").data_ptr(),
        0 if row_order is None else _i32(row_order, "row_order").data_ptr(),
        batch, kv_block_table.shape[1], int(total_q), block_size,
        n_heads_q, n_heads_kv, head_dim,
        kv_slot_stride, kv_token_stride, dkv_slot_stride, dkv_token_stride,
        q_entry, out_entry, dq_entry, lse_head_stride, lse_entry, int(total_k or 0),
        float(softmax_scale), dtype_code(q.dtype), _stream(),
    )
    return dq, dk, dv, None
