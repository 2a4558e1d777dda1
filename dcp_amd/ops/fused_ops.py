"""Fused block operators: the call surface of the reference's
``dcp/ops/fused_ops.py`` backed by the gfx950 kernels of ``libdcp_hip.so``.

Every function keeps the reference's name, argument order and meaning
(wrappers at ``fused_ops.py:149-247, 796-1084, 1288-1360``); arguments that
only tuned the Triton launch (``triton_block_size``, ``require_cached``) are
accepted, validated the same way and otherwise ignored.  Index and pointer
tables are device tensors; work is enqueued on torch's current stream.

There is no fallback: without the built library these raise.
"""

from __future__ import annotations

import torch

from dcp_amd import _lib

__all__ = [
    "flash_attn_update_out_lse",
    "fused_copy_bf16",
    "fused_copy_fp16",
    "fused_copy_fp32",
    "fused_copy_bf16_varlen",
    "fused_copy_fp16_varlen",
    "fused_copy_fp32_varlen",
    "fused_copy_bf16_varlen_dkv",
    "fused_copy_fp16_varlen_dkv",
    "fused_copy_fp32_varlen_dkv",
    "fused_copy_bf16_varlen_lse",
    "fused_copy_fp16_varlen_lse",
    "fused_copy_fp32_varlen_lse",
    "fused_blockwise_sum",
    "warmup_triton_ops",
]

_DTYPE_CODE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}


def dtype_code(dtype) -> int:
    """Wire integer of a torch dtype (or of its ``str``)."""
    if isinstance(dtype, str):
        for k, v in _DTYPE_CODE.items():
            if str(k) == dtype:
                return v
        raise ValueError(f"Unsupported dtype: {dtype}")
    if dtype not in _DTYPE_CODE:
        raise ValueError(f"Unsupported dtype: {dtype}")
    return _DTYPE_CODE[dtype]


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _table(t: torch.Tensor, dtype: torch.dtype, name: str) -> int:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a tensor, got {type(t).__name__}")
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_cuda:
        raise ValueError(f"{name} must be a device tensor")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    return t.data_ptr()


def _i32(t, name):
    return _table(t, torch.int32, name)


def _i64(t, name):
    return _table(t, torch.int64, name)


# ---------------------------------------------------------------------------
# block copies
# ---------------------------------------------------------------------------


def _copy_varlen(elem_size, src_ptrs, src_offsets, src_strides, dst_ptrs,
                 dst_offsets, dst_strides, n_elements, block_size):
    _lib.call(
        "dcp_fused_copy_varlen",
        _i64(src_ptrs, "src_ptrs"),
        _i32(src_offsets, "src_offsets"),
        _i32(src_strides, "src_strides"),
        _i64(dst_ptrs, "dst_ptrs"),
        _i32(dst_offsets, "dst_offsets"),
        _i32(dst_strides, "dst_strides"),
        _i32(n_elements, "n_elements"),
        len(src_ptrs),
        int(block_size),
        elem_size,
        _stream(),
    )


def _copy_full(elem_size, src_ptrs, src_offsets, src_strides, dst_ptrs,
               dst_offsets, dst_strides, block_size, triton_block_size):
    assert block_size % triton_block_size == 0
    n_elements = torch.full(
        (len(src_ptrs),), int(block_size), dtype=torch.int32,
        device=src_ptrs.device,
    )
    _copy_varlen(elem_size, src_ptrs, src_offsets, src_strides, dst_ptrs,
                 dst_offsets, dst_strides, n_elements, block_size)


def fused_copy_bf16(src_ptrs, src_offsets, src_strides, dst_ptrs, dst_offsets,
                    dst_strides, block_size: int, triton_block_size: int):
    """Whole-block copy (reference ``fused_ops.py:796-816``)."""
    _copy_full(2, src_ptrs, src_offsets, src_strides, dst_ptrs, dst_offsets,
               dst_strides, block_size, triton_block_size)


def fused_copy_fp16(src_ptrs, src_offsets, src_strides, dst_ptrs, dst_offsets,
                    dst_strides, block_size: int, triton_block_size: int):
    _copy_full(2, src_ptrs, src_offsets, src_strides, dst_ptrs, dst_offsets,
               dst_strides, block_size, triton_block_size)


def fused_copy_fp32(src_ptrs, src_offsets, src_strides, dst_ptrs, dst_offsets,
                    dst_strides, block_size: int, triton_block_size: int):
    _copy_full(4, src_ptrs, src_offsets, src_strides, dst_ptrs, dst_offsets,
               dst_strides, block_size, triton_block_size)


def fused_copy_bf16_varlen(src_ptrs, src_offsets, src_strides, dst_ptrs,
                           dst_offsets, dst_strides, n_elements,
                           block_size: int, triton_block_size: int):
    """``dst[p][dst_off*dst_stride + i] = src[p][src_off*src_stride + i]`` for
    ``i < n_elements[p]`` (reference ``fused_ops.py:842-864``)."""
    _copy_varlen(2, src_ptrs, src_offsets, src_strides, dst_ptrs, dst_offsets,
                 dst_strides, n_elements, block_size)


def fused_copy_fp16_varlen(src_ptrs, src_offsets, src_strides, dst_ptrs,
                           dst_offsets, dst_strides, n_elements,
                           block_size: int, triton_block_size: int):
    _copy_varlen(2, src_ptrs, src_offsets, src_strides, dst_ptrs, dst_offsets,
                 dst_strides, n_elements, block_size)


def fused_copy_fp32_varlen(src_ptrs, src_offsets, src_strides, dst_ptrs,
                           dst_offsets, dst_strides, n_elements,
                           block_size: int, triton_block_size: int):
    _copy_varlen(4, src_ptrs, src_offsets, src_strides, dst_ptrs, dst_offsets,
                 dst_strides, n_elements, block_size)


def _copy_dkv(elem_size, src_ptrs, dst_ptrs, n_tokens, max_n_tokens,
              per_token_size, triton_block_size):
    assert per_token_size % triton_block_size == 0
    _lib.call(
        "dcp_fused_copy_varlen_dkv",
        _i64(src_ptrs, "src_ptrs"),
        _i64(dst_ptrs, "dst_ptrs"),
        _i32(n_tokens, "n_tokens"),
        len(src_ptrs),
        int(max_n_tokens),
        int(per_token_size),
        elem_size,
        _stream(),
    )


def fused_copy_bf16_varlen_dkv(src_ptrs, dst_ptrs, n_tokens, max_n_tokens: int,
                               per_token_size: int, triton_block_size: int):
    """Copy the first ``n_tokens[p]`` tokens of block p (reference
    ``fused_ops.py:867-885``)."""
    _copy_dkv(2, src_ptrs, dst_ptrs, n_tokens, max_n_tokens, per_token_size,
              triton_block_size)


def fused_copy_fp16_varlen_dkv(src_ptrs, dst_ptrs, n_tokens, max_n_tokens: int,
                               per_token_size: int, triton_block_size: int):
    _copy_dkv(2, src_ptrs, dst_ptrs, n_tokens, max_n_tokens, per_token_size,
              triton_block_size)


def fused_copy_fp32_varlen_dkv(src_ptrs, dst_ptrs, n_tokens, max_n_tokens: int,
                               per_token_size: int, triton_block_size: int):
    _copy_dkv(4, src_ptrs, dst_ptrs, n_tokens, max_n_tokens, per_token_size,
              triton_block_size)


def _copy_lse(elem_size, src_ptrs, src_token_offsets, src_head_strides,
              dst_ptrs, dst_token_offsets, dst_head_strides, n_tokens,
              head_block_size, block_size, triton_block_size):
    assert block_size % triton_block_size == 0
    _lib.call(
        "dcp_fused_copy_varlen_lse",
        _i64(src_ptrs, "src_ptrs"),
        _i32(src_token_offsets, "src_token_offsets"),
        _i32(src_head_strides, "src_head_strides"),
        _i64(dst_ptrs, "dst_ptrs"),
        _i32(dst_token_offsets, "dst_token_offsets"),
        _i32(dst_head_strides, "dst_head_strides"),
        _i32(n_tokens, "n_tokens"),
        len(src_ptrs),
        int(head_block_size),
        int(block_size),
        elem_size,
        _stream(),
    )


def fused_copy_bf16_varlen_lse(src_ptrs, src_token_offsets, src_head_strides,
                               dst_ptrs, dst_token_offsets, dst_head_strides,
                               n_tokens, head_block_size: int, block_size: int,
                               triton_block_size: int):
    _copy_lse(2, src_ptrs, src_token_offsets, src_head_strides, dst_ptrs,
              dst_token_offsets, dst_head_strides, n_tokens, head_block_size,
              block_size, triton_block_size)


def fused_copy_fp16_varlen_lse(src_ptrs, src_token_offsets, src_head_strides,
                               dst_ptrs, dst_token_offsets, dst_head_strides,
                               n_tokens, head_block_size: int, block_size: int,
                               triton_block_size: int):
    _copy_lse(2, src_ptrs, src_token_offsets, src_head_strides, dst_ptrs,
              dst_token_offsets, dst_head_strides, n_tokens, head_block_size,
              block_size, triton_block_size)


def fused_copy_fp32_varlen_lse(src_ptrs, src_token_offsets, src_head_strides,
                               dst_ptrs, dst_token_offsets, dst_head_strides,
                               n_tokens, head_block_size: int, block_size: int,
                               triton_block_size: int):
    """Head-strided LSE block copy, ``[head_block_size, n_tokens[p]]`` per
    block (reference ``fused_ops.py:1059-1084``)."""
    _copy_lse(4, src_ptrs, src_token_offsets, src_head_strides, dst_ptrs,
              dst_token_offsets, dst_head_strides, n_tokens, head_block_size,
              block_size, triton_block_size)


# ---------------------------------------------------------------------------
# (out, lse) merge
# ---------------------------------------------------------------------------


def flash_attn_update_out_lse(
    src_out_buffer,  # [src_n_total_blocks, block_size, n_head, head_dim]
    dst_out_buffer,  # [sum(n_tokens_per_block), n_head, head_dim] or padded
    src_lse_buffer,  # [n_head, src_n_total_blocks, block_size]
    dst_lse_buffer,  # [n_head, sum(n_tokens_per_block)] or padded
    n_head,
    src_block_table,  # [n_red_ops, max_n_blocks_per_op] int32
    dst_token_offsets,  # [n_red_ops] int32
    n_tokens_per_block,  # [n_red_ops] int32
    block_lengths,  # [n_red_ops] int32: sources per op
    block_size,
    out_block_stride,
    out_token_stride,
    lse_block_stride,
    lse_token_stride,
    src_lse_head_stride,
    dst_lse_head_stride,
    HEAD_DIM: int,
    max_n_blocks_per_op: int,
    triton_block_size: int,
    require_cached: bool = False,
    return_key: bool = False,
):
    """N-way online-softmax merge of partial outputs and their LSEs, written
    at ``dst_token_offsets`` (reference ``fused_ops.py:149-247``).  Sources
    whose LSE is +-inf are skipped; with no finite source the result is
    ``out = 0``, ``lse = -1``."""
    assert max_n_blocks_per_op <= 64, "Too many blocks for reduction"
    assert block_size % triton_block_size == 0
    if src_out_buffer.dtype != dst_out_buffer.dtype:
        raise ValueError(
            f"src/dst out dtypes differ: {src_out_buffer.dtype} vs "
            f"{dst_out_buffer.dtype}"
        )
    if src_lse_buffer.dtype != torch.float32 or dst_lse_buffer.dtype != torch.float32:
        raise ValueError("LSE buffers must be float32")
    _lib.call(
        "dcp_update_out_lse",
        src_out_buffer.data_ptr(),
        dst_out_buffer.data_ptr(),
        src_lse_buffer.data_ptr(),
        dst_lse_buffer.data_ptr(),
        int(n_head),
        _i32(src_block_table, "src_block_table"),
        _i32(dst_token_offsets, "dst_token_offsets"),
        _i32(n_tokens_per_block, "n_tokens_per_block"),
        _i32(block_lengths, "block_lengths"),
        len(block_lengths),
        int(block_size),
        int(out_block_stride),
        int(out_token_stride),
        int(lse_block_stride),
        int(lse_token_stride),
        int(src_lse_head_stride),
        int(dst_lse_head_stride),
        int(HEAD_DIM),
        int(max_n_blocks_per_op),
        dtype_code(src_out_buffer.dtype),
        _stream(),
    )
    if return_key:
        return "hip", torch.cuda.current_device()


# ---------------------------------------------------------------------------
# block sum
# ---------------------------------------------------------------------------


def fused_blockwise_sum(
    src_ptrs,  # [n_sums] int64
    src_offsets,  # [n_sums, max_n_ops_per_block] int32 (block indices)
    src_strides,  # [n_sums] int32
    n_ops_per_block,  # [n_sums] int32
    dst_ptrs,  # [n_sums] int64
    dst_offsets,  # [n_sums] int32
    dst_strides,  # [n_sums] int32
    n_elements,  # [n_sums] int32
    dtype,
    max_n_ops_per_block: int,
    block_size: int,
    triton_block_size: int,
    require_cached: bool = False,
):
    """``dst[s] = sum_j src[s][j]`` over ``n_elements[s]`` elements (reference
    ``fused_ops.py:1288-1360``); accumulated in fp32."""
    assert block_size % triton_block_size == 0
    code = dtype_code(dtype if isinstance(dtype, str) else str(dtype))
    if src_offsets.dim() != 2 or src_offsets.shape[1] != max_n_ops_per_block:
        raise ValueError(
            "src_offsets must be [n_sums, max_n_ops_per_block], got "
            f"{tuple(src_offsets.shape)}"
        )
    _lib.call(
        "dcp_blockwise_sum",
        _i64(src_ptrs, "src_ptrs"),
        _i32(src_offsets, "src_offsets"),
        _i32(src_strides, "src_strides"),
        _i32(n_ops_per_block, "n_ops_per_block"),
        _i64(dst_ptrs, "dst_ptrs"),
        _i32(dst_offsets, "dst_offsets"),
        _i32(dst_strides, "dst_strides"),
        _i32(n_elements, "n_elements"),
        len(src_ptrs),
        int(max_n_ops_per_block),
        int(block_size),
        code,
        _stream(),
    )


def warmup_triton_ops(*args, **kwargs):
    """The reference pre-compiles its Triton kernels here
    (``fused_ops.py:1690-1817``); the HIP kernels are compiled ahead of time,
    so this only checks that the library loads."""
    _lib.load()
