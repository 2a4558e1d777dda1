"""Concrete executor of one device's blockwise attention plan on MI355X.

Keeps the interface of the reference's
``dcp/runtime/flash_attention/executor.py``: ``AttentionExecutor`` (:340-533)
with ``prepare`` / ``execute`` / ``forward`` / ``backward`` /
``switch_to_backward`` / ``capture_cudagraph``, the autograd wrapper
``DCPAttention`` (:536-587), prep handlers that build device argument tables
once per plan (``_prepare_*``) and execute handlers that only launch kernels
(``_handle_*``), and the factory ``get_executor`` (:2077-2133).

Differences that follow from the kernels, not from the interface:

* the backward kernel sums dK/dV over a kv head's q-head group itself and
  writes whole dKV slots, so the grouped-query path needs no zeroed temporary
  dKV buffer and no copy pass (reference :954-1035, :1074-1114);
* attention rows are launched longest-first (a ``row_order`` table built in
  ``prepare``) so that ragged rows balance across the 256 CUs;
* communication instructions are rejected: this build runs one GPU.
"""

from __future__ import annotations

from collections import defaultdict
from typing import Dict, List, Optional, Tuple

import math
import numpy as np
import torch

from dcp_amd.core.executor import DCPExecutor
from dcp_amd.core.instructions import *  # noqa: F401,F403
from dcp_amd.core.instructions import (
    AttnBackwardInstr,
    AttnInstr,
    AttnReductionInstr,
    BarrierInstr,
    BlockInstrBase,
    BufferBlock,
    BufferType,
    CommLaunchInstr,
    CommWaitInstr,
    ExecutionPlan,
    MemcpyInstr,
    SumInstr,
)
from dcp_amd.core.serialization import int_to_torch_dtype
from dcp_amd.flash_attn_interface import (
    _flash_attn_varlen_backward,
    _flash_attn_varlen_forward,
    backward_workspace_bytes,
    forward_workspace,
)
from dcp_amd.ops.fused_ops import (
    flash_attn_update_out_lse,
    fused_blockwise_sum,
    fused_copy_bf16_varlen,
    fused_copy_fp16_varlen,
    fused_copy_fp32_varlen,
    fused_copy_fp32_varlen_lse,
)

_LSE_BUFFER_TYPES = {BufferType.BUFFER_LSE, BufferType.LOCAL_LSE}

_COPY_FN = {
    torch.float32: fused_copy_fp32_varlen,
    torch.float16: fused_copy_fp16_varlen,
    torch.bfloat16: fused_copy_bf16_varlen,
}


def _dev(values, dtype) -> torch.Tensor:
    return torch.tensor(values, dtype=dtype, device="cuda")


class AttentionExecutor(DCPExecutor):
    def __init__(
        self,
        fw_exec_plan: Optional[ExecutionPlan] = None,
        fw_workload=None,
        bw_exec_plan: Optional[ExecutionPlan] = None,
        bw_workload=None,
        node_id: int = None,
        local_device_id: int = None,
        n_devices_per_node: int = None,
        n_nodes: int = None,
        n_heads_per_block: int = 1,
        head_dim: int = None,
        synchronous: bool = False,
        process_group=None,
        iteration_idx: Optional[int] = None,
        tp_rank: Optional[int] = None,
        use_cudagraph: bool = False,
    ):
        super().__init__(
            node_id=node_id,
            local_device_id=local_device_id,
            n_devices_per_node=n_devices_per_node,
            n_nodes=n_nodes,
            synchronous=synchronous,
            iteration_idx=iteration_idx,
            tp_rank=tp_rank,
        )
        self.process_group = process_group
        self.n_heads_per_block = n_heads_per_block
        self.head_dim = head_dim
        self.main_stream = torch.cuda.Stream()
        self.streams: Dict[str, torch.cuda.Stream] = {}
        self._prep_handlers = {}
        self._args_cache = {}
        self.register_synchronization_handler(torch.cuda.synchronize)
        self.fw_exec_plan = fw_exec_plan
        self.bw_exec_plan = bw_exec_plan
        self.fw_workload = fw_workload
        self.bw_workload = bw_workload
        self.mode = "Forward"
        self.use_cudagraph = use_cudagraph
        self.cuda_graph = None

    # -- buffers ---------------------------------------------------------------
    def _create_buffer(self, buffer_shape: Tuple[int, ...], buffer_dtype: int):
        return torch.zeros(*buffer_shape, dtype=int_to_torch_dtype(buffer_dtype), device="cuda")

    def log_memory_usage(self):
        total = 0.0
        for buffer_type, buffer in self.buffers.items():
            if buffer is None:
                continue
            size = buffer.element_size() * buffer.numel() / 1e6
            total += size
            if self.logger:
                self.logger.debug(f"Buffer {buffer_type}: {size:.2f} MB")
        if self.logger:
            self.logger.debug(f"Total memory: {total:.2f} MB")
        return total

    def set_local_out_lse(self, out, lse):
        self.buffers[BufferType.LOCAL_OUT].copy_(out)
        self.buffers[BufferType.LOCAL_LSE].copy_(lse)

    def deallocate_all_buffers(self):
        self.buffers = {}
        self.streams = {}
        self._args_cache = {}

    # -- prepare / execute -------------------------------------------------------
    def register_prep_handler(self, instruction_type, handler):
        if not (isinstance(instruction_type, type) and issubclass(instruction_type, BlockInstrBase)):
            raise TypeError(
                "Instruction type must be a subclass of BlockInstrBase, got "
                f"{getattr(instruction_type, '__name__', instruction_type)}"
            )
        if instruction_type in self._prep_handlers:
            raise ValueError(f"Prep handler for {instruction_type.__name__} already registered.")
        self._prep_handlers[instruction_type] = handler

    def prepare(self, forward=True):
        """Allocate the plan's buffers and build every instruction's device
        argument tables; after this ``execute`` allocates nothing and never
        touches the host."""
        torch.cuda.nvtx.range_push("AttentionExecutor prepare")
        self._args_cache = {}
        self.execution_plan = self.fw_exec_plan if forward else self.bw_exec_plan
        self.init_buffers(self.execution_plan)
        for instr_index, instr in enumerate(self.execution_plan.instructions):
            self.instr_index = instr_index
            prep = self._prep_handlers.get(type(instr))
            if prep is not None:
                prep(self, instr)
        torch.cuda.nvtx.range_pop()

    def switch_to_backward(self):
        self.mode = "Backward"
        self.cuda_graph = None
        self.deallocate_buffers()
        self.prepare(forward=False)
        self.log_memory_usage()

    def capture_cudagraph(self):
        """Capture ``execute`` of the current mode's plan into a HIP graph
        (call after ``prepare``)."""
        if not self.use_cudagraph:
            return
        plan, is_forward = (
            (self.fw_exec_plan, True) if self.mode == "Forward" else (self.bw_exec_plan, False)
        )
        self.cuda_graph = None
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            self.execute(plan, is_forward=is_forward)
        torch.cuda.synchronize()
        self.cuda_graph = graph

    def execute(self, execution_plan, is_forward=True):
        torch.cuda.nvtx.range_push("AttentionExecutor execute")
        prev_stream = torch.cuda.current_stream()
        self.main_stream.wait_stream(prev_stream)
        with torch.cuda.stream(self.main_stream):
            if self.cuda_graph is not None:
                self.cuda_graph.replay()
            else:
                super().execute(execution_plan, is_forward)
        prev_stream.wait_stream(self.main_stream)
        torch.cuda.nvtx.range_pop()
        if is_forward:
            return self.buffers[BufferType.LOCAL_OUT], self.buffers[BufferType.LOCAL_LSE]
        return self.buffers[BufferType.LOCAL_dQ], self.buffers[BufferType.LOCAL_dKV]

    def forward(self, q, kv):
        self.init_forward_input(q, kv)
        self.execute(self.fw_exec_plan, is_forward=True)
        return (
            self.buffers[BufferType.LOCAL_OUT].detach().clone(),
            self.buffers[BufferType.LOCAL_LSE].detach().clone(),
        )

    def backward(self, q, kv, out, dout, lse):
        self.set_local_out_lse(out, lse)
        self.init_forward_input(q, kv)
        self.init_backward_input(dout)
        self.execute(self.bw_exec_plan, is_forward=False)
        return (
            self.buffers[BufferType.LOCAL_dQ].detach().clone(),
            self.buffers[BufferType.LOCAL_dKV].detach().clone(),
        )


class DCPAttention(torch.autograd.Function):
    """``out = DCPAttention.apply(executor, capture_fwd_graph,
    capture_bwd_graph, q, kv)`` with q, kv in LOCAL layout."""

    @staticmethod
    def forward(ctx, executor: AttentionExecutor, capture_fwd_graph: bool,
                capture_bwd_graph: bool, q: torch.Tensor, kv: torch.Tensor):
        ctx.executor = executor
        ctx.capture_bwd_graph = capture_bwd_graph
        if capture_fwd_graph:
            executor.capture_cudagraph()
        out, lse = executor.forward(q, kv)
        ctx.save_for_backward(q, kv, out, lse)
        return out

    @staticmethod
    def backward(ctx, dout: torch.Tensor):
        q, kv, out, lse = ctx.saved_tensors
        executor: AttentionExecutor = ctx.executor
        if executor.mode == "Forward":
            executor.switch_to_backward()
        if ctx.capture_bwd_graph:
            executor.capture_cudagraph()
        dq, dkv = executor.backward(q, kv, out, dout, lse)
        return None, None, None, dq, dkv


# ---------------------------------------------------------------------------
# MemcpyInstr: gather LOCAL_* blocks into BUFFER_* slots
# ---------------------------------------------------------------------------


def _prepare_memcpy(exec: AttentionExecutor, instr: MemcpyInstr):
    """One argument table per (dtype, block numel) for data blocks and one for
    LSE blocks.  The source is the unpadded buffer, addressed by
    ``local_cu_seqlens`` (reference ``_prepare_memcpy`` :606-790)."""
    cu = exec.execution_plan.local_cu_seqlens
    data = defaultdict(lambda: [[] for _ in range(7)])
    lse = defaultdict(lambda: [[] for _ in range(7)])
    head_block_size = None
    for src, dst in instr.src_dst_pairs:
        src_buf, dst_buf = exec.buffers[src.buffer_type], exec.buffers[dst.buffer_type]
        key = (src_buf.dtype, exec.buffer_block_strides[src.buffer_type])
        src_off = cu[src.index]
        if src.buffer_type in _LSE_BUFFER_TYPES:
            assert dst.buffer_type in _LSE_BUFFER_TYPES
            cols = lse[key]
            cols[0].append(src_buf.data_ptr())
            cols[1].append(src_off)
            cols[2].append(src_buf.shape[1])
            cols[3].append(dst_buf.data_ptr())
            cols[4].append(dst.index * dst_buf.shape[2])
            cols[5].append(dst_buf.shape[1] * dst_buf.shape[2])
            cols[6].append(src.n_tokens)
            head_block_size = src_buf.shape[0] if head_block_size is None else head_block_size
            continue
        assert src_buf.dtype == dst_buf.dtype, f"{src_buf.dtype} != {dst_buf.dtype} in MemcpyInstr"
        assert src_buf.dtype in _COPY_FN, f"Unsupported dtype {src_buf.dtype}"
        assert (
            exec.buffer_block_strides[src.buffer_type] == exec.buffer_block_strides[dst.buffer_type]
        ), "block numel mismatch in MemcpyInstr"
        assert src.n_tokens == dst.n_tokens, f"{src.n_tokens} != {dst.n_tokens} in MemcpyInstr"
        per_token = int(np.prod(exec.buffer_per_token_shape[src.buffer_type]))
        cols = data[key]
        cols[0].append(src_buf.data_ptr() + src_off * src_buf.stride(0) * src_buf.element_size())
        cols[1].append(0)
        cols[2].append(1)
        cols[3].append(dst_buf.data_ptr())
        cols[4].append(dst.index)
        cols[5].append(exec.buffer_block_strides[dst.buffer_type])
        cols[6].append(src.n_tokens * per_token)

    def tables(cols):
        kinds = (torch.int64, torch.int32, torch.int32, torch.int64, torch.int32, torch.int32, torch.int32)
        return tuple(_dev(c, k) for c, k in zip(cols, kinds))

    exec._args_cache[exec.instr_index] = {
        "other": {key: tables(cols) for key, cols in data.items()},
        "lse": {key: tables(cols) + (head_block_size,) for key, cols in lse.items()},
    }


def _handle_memcpy(exec: AttentionExecutor, instr: MemcpyInstr):
    torch.cuda.nvtx.range_push("MemcpyInstr")
    args_cache = exec._args_cache[exec.instr_index]
    for (dtype, block_numel), args in args_cache["other"].items():
        if dtype not in _COPY_FN:
            raise ValueError(f"Unsupported dtype {dtype}")
        _COPY_FN[dtype](*args, block_numel, 128)
    for (dtype, block_numel), args in args_cache["lse"].items():
        if dtype != torch.float32:
            raise ValueError(f"Unsupported dtype {dtype}")
        # the tile argument only has to divide the block (the reference fixes 128, :808)
        fused_copy_fp32_varlen_lse(*args, block_numel, math.gcd(block_numel, 128))
    torch.cuda.nvtx.range_pop()


# ---------------------------------------------------------------------------
# AttnInstr / AttnBackwardInstr
# ---------------------------------------------------------------------------


def _pad_block_table(table: List[List[BufferBlock]]) -> List[List[int]]:
    width = max(len(row) for row in table)
    return [[blk.index for blk in row] + [-1] * (width - len(row)) for row in table]


def _cu(seqlens: List[int]) -> torch.Tensor:
    return _dev(np.concatenate(([0], np.cumsum(seqlens))).tolist(), torch.int32)


def _mask_tensor(attn_mask) -> torch.Tensor:
    if not isinstance(attn_mask, torch.Tensor):
        attn_mask = torch.stack([torch.as_tensor(m) for m in attn_mask], dim=0)
    return attn_mask.to(torch.int32).contiguous().cuda()


def _longest_first(seqlens_kv: List[int]) -> torch.Tensor:
    order = np.argsort(-np.asarray(seqlens_kv, dtype=np.int64), kind="stable")
    return _dev(order.tolist(), torch.int32)


def _prepare_attn(exec: AttentionExecutor, instr: AttnInstr):
    exec._args_cache[exec.instr_index] = (
        sum(instr.seqlens_q),
        _cu(instr.seqlens_q),
        _cu(instr.seqlens_kv),
        _dev(_pad_block_table(instr.q_block_table), torch.int32),
        _dev(_pad_block_table(instr.kv_block_table), torch.int32),
        _dev(_pad_block_table(instr.out_block_table), torch.int32),
        _mask_tensor(instr.attn_mask),
        _longest_first(instr.seqlens_kv),
        forward_workspace(),
    )


def _kv_views(kv: torch.Tensor):
    return kv[:, :, 0], kv[:, :, 1]


def _handle_attn(exec: AttentionExecutor, instr: AttnInstr):
    torch.cuda.nvtx.range_push("AttnInstr")
    (total_q, cu_q, cu_kv, q_table, kv_table, out_table, attn_mask, row_order, workspace) = exec._args_cache[
        exec.instr_index
    ]
    k, v = _kv_views(exec.buffers[BufferType.BUFFER_KV])
    _flash_attn_varlen_forward(
        exec.buffers[BufferType.BUFFER_Q],
        k,
        v,
        cu_q,
        cu_kv,
        total_q,
        instr.max_seqlen_q,
        instr.max_seqlen_kv,
        0.0,
        exec.head_dim ** (-0.5),
        causal=False,
        attn_range=attn_mask,
        q_block_table=q_table,
        kv_block_table=kv_table,
        out_block_table=out_table,
        out_=exec.buffers[BufferType.BUFFER_OUT],
        lse_=exec.buffers[BufferType.BUFFER_LSE],
        row_order=row_order,
        workspace=workspace,
    )
    torch.cuda.nvtx.range_pop()


def _prepare_attn_bw(exec: AttentionExecutor, instr: AttnBackwardInstr):
    total_q = sum(instr.seqlens_q)
    hb = exec.buffer_per_token_shape[BufferType.BUFFER_dQ][-2]
    d = exec.buffer_per_token_shape[BufferType.BUFFER_dQ][-1]
    bs = exec.buffer_block_sizes[BufferType.BUFFER_dQ]
    exec._args_cache[exec.instr_index] = (
        total_q,
        sum(instr.seqlens_kv),
        _cu(instr.seqlens_q),
        _cu(instr.seqlens_kv),
        _dev(_pad_block_table(instr.q_block_table), torch.int32),
        _dev(_pad_block_table(instr.kv_block_table), torch.int32),
        _dev(_pad_block_table(instr.out_block_table), torch.int32),
        _mask_tensor(instr.attn_mask),
        _dev(_pad_block_table(instr.dq_block_table), torch.int32),
        _dev(_pad_block_table(instr.dkv_block_table), torch.int32),
        torch.empty(
            backward_workspace_bytes(len(instr.seqlens_q), total_q, bs, hb, d),
            dtype=torch.uint8,
            device="cuda",
        ),
        _longest_first(instr.seqlens_kv),
    )


def _handle_attn_bw(exec: AttentionExecutor, instr: AttnBackwardInstr):
    torch.cuda.nvtx.range_push("AttnBackwardInstr")
    (total_q, total_kv, cu_q, cu_kv, q_table, kv_table, out_table, attn_mask, dq_table, dkv_table,
     workspace, row_order) = exec._args_cache[exec.instr_index]
    k, v = _kv_views(exec.buffers[BufferType.BUFFER_KV])
    dk, dv = _kv_views(exec.buffers[BufferType.BUFFER_dKV])
    _flash_attn_varlen_backward(
        exec.buffers[BufferType.BUFFER_dOUT],
        exec.buffers[BufferType.BUFFER_Q],
        k,
        v,
        exec.buffers[BufferType.BUFFER_OUT],
        exec.buffers[BufferType.BUFFER_LSE],
        exec.buffers[BufferType.BUFFER_dQ],
        dk,
        dv,
        cu_q,
        cu_kv,
        total_q,
        total_kv,
        instr.max_seqlen_q,
        instr.max_seqlen_kv,
        0.0,
        exec.head_dim ** (-0.5),
        False,
        -1,
        -1,
        0.0,
        None,
        False,
        attn_range=attn_mask,
        q_block_table=q_table,
        kv_block_table=kv_table,
        out_block_table=out_table,
        dq_block_table=dq_table,
        dkv_block_table=dkv_table,
        workspace=workspace,
        row_order=row_order,
    )
    torch.cuda.nvtx.range_pop()


# ---------------------------------------------------------------------------
# AttnReductionInstr: N-way (out, lse) merge (+ scatter when unpadded)
# ---------------------------------------------------------------------------


def _round_to_pow_2(x: int):
    return 1 << (x - 1).bit_length()


def _prepare_reduction(exec: AttentionExecutor, instr: AttnReductionInstr):
    first = instr.ops[0]
    types = (
        first.src_buffers[0][0].buffer_type,
        first.src_buffers[0][1].buffer_type,
        first.dst_buffer[0].buffer_type,
        first.dst_buffer[1].buffer_type,
    )
    unpadded = bool(instr.output_is_unpadded)
    cu = exec.execution_plan.local_cu_seqlens
    width = _round_to_pow_2(max(len(op.src_buffers) for op in instr.ops))
    table, dst_offsets, n_tokens, n_srcs = [], [], [], []
    for op in instr.ops:
        srcs = [out_blk.index for out_blk, _ in op.src_buffers]
        table.append(srcs + [-1] * (width - len(srcs)))
        idx = op.dst_buffer[0].index
        dst_offsets.append(cu[idx] if unpadded else idx * exec.buffer_block_sizes[types[2]])
        n_tokens.append(op.dst_buffer[0].n_tokens)
        n_srcs.append(len(srcs))
    dst_lse = exec.buffers[types[3]]
    exec._args_cache[exec.instr_index] = (
        types,
        _dev(table, torch.int32),
        _dev(dst_offsets, torch.int32),
        _dev(n_tokens, torch.int32),
        _dev(n_srcs, torch.int32),
        width,
        # head stride of the destination LSE: its token axis length
        dst_lse.shape[1] if unpadded else dst_lse.shape[1] * dst_lse.shape[2],
    )


def _handle_reduction(exec: AttentionExecutor, instr: AttnReductionInstr):
    torch.cuda.nvtx.range_push("AttnReductionInstr")
    (types, table, dst_offsets, n_tokens, n_srcs, width, dst_lse_head_stride) = exec._args_cache[
        exec.instr_index
    ]
    src_out_t, src_lse_t, dst_out_t, dst_lse_t = types
    flash_attn_update_out_lse(
        exec.buffers[src_out_t],
        exec.buffers[dst_out_t],
        exec.buffers[src_lse_t],
        exec.buffers[dst_lse_t],
        exec.n_heads_per_block,
        table,
        dst_offsets,
        n_tokens,
        n_srcs,
        exec.buffer_block_sizes[src_out_t],
        exec.buffer_block_strides[src_out_t],
        exec.n_heads_per_block * exec.head_dim,
        exec.buffer_block_sizes[src_lse_t],
        1,
        exec.buffer_n_blocks[src_lse_t] * exec.buffer_block_sizes[src_lse_t],
        dst_lse_head_stride,
        exec.head_dim,
        width,
        64,
    )
    torch.cuda.nvtx.range_pop()


# ---------------------------------------------------------------------------
# SumInstr: N-way block sum (+ scatter when unpadded)
# ---------------------------------------------------------------------------


def _prepare_sum(exec: AttentionExecutor, instr: SumInstr):
    groups = defaultdict(lambda: defaultdict(list))
    cu = exec.execution_plan.local_cu_seqlens
    for op in instr.ops:
        src_type = op.src_buffers[0].buffer_type
        dst_type = op.dst_buffer.buffer_type
        key = (exec.buffers[src_type].dtype, exec.buffer_block_strides[src_type])
        g = groups[key]
        per_token = int(np.prod(exec.buffer_per_token_shape[src_type]))
        g["src_ptrs"].append(exec.buffers[src_type].data_ptr())
        g["src_offsets"].append([blk.index for blk in op.src_buffers])
        g["src_strides"].append(exec.buffer_block_strides[src_type])
        g["n_ops"].append(len(op.src_buffers))
        g["dst_ptrs"].append(exec.buffers[dst_type].data_ptr())
        if instr.output_is_unpadded:
            g["dst_offsets"].append(cu[op.dst_buffer.index])
            g["dst_strides"].append(per_token)
        else:
            g["dst_offsets"].append(op.dst_buffer.index)
            g["dst_strides"].append(exec.buffer_block_strides[dst_type])
        g["n_elems"].append(op.dst_buffer.n_tokens * per_token)
    prepared = {}
    for key, g in groups.items():
        width = _round_to_pow_2(max(g["n_ops"]))
        padded = [row + [-1] * (width - len(row)) for row in g["src_offsets"]]
        prepared[key] = (
            _dev(g["src_ptrs"], torch.int64),
            _dev(padded, torch.int32),
            _dev(g["src_strides"], torch.int32),
            _dev(g["n_ops"], torch.int32),
            _dev(g["dst_ptrs"], torch.int64),
            _dev(g["dst_offsets"], torch.int32),
            _dev(g["dst_strides"], torch.int32),
            _dev(g["n_elems"], torch.int32),
            width,
        )
    exec._args_cache[exec.instr_index] = prepared


def _handle_sum(exec: AttentionExecutor, instr: SumInstr):
    torch.cuda.nvtx.range_push("SumInstr")
    for (dtype, block_numel), args in exec._args_cache[exec.instr_index].items():
        *tables, width = args
        fused_blockwise_sum(*tables, dtype, width, block_numel, 128)
    torch.cuda.nvtx.range_pop()


# ---------------------------------------------------------------------------
# communication: not part of a one-GPU build
# ---------------------------------------------------------------------------


def _reject_comm(exec: AttentionExecutor, instr: BlockInstrBase):
    raise NotImplementedError(
        f"{type(instr).__name__}: inter-GPU communication is not available in this build "
        "(one GPU owns every block of the plan)"
    )


def get_executor(
    n_heads_per_block: int,
    head_dim: int,
    exec_context=None,
    fw_exec_plan: Optional[ExecutionPlan] = None,
    fw_workload=None,
    bw_exec_plan: Optional[ExecutionPlan] = None,
    bw_workload=None,
    executor_impl="python",
    process_group=None,
    synchronous: bool = False,
    iteration_idx: Optional[int] = None,
    tp_rank: Optional[int] = None,
    use_cudagraph: bool = False,
):
    """Factory with the reference's signature (:2077-2133).  ``exec_context``
    only supplies ``n_devices_per_node`` / ``n_nodes`` and may be ``None``."""
    if executor_impl != "python":
        raise ValueError(f"Unsupported executor_impl: {executor_impl}")
    n_devices_per_node = getattr(exec_context, "n_devices_per_node", 1)
    n_nodes = getattr(exec_context, "n_nodes", 1)
    rank = 0
    if torch.distributed.is_available() and torch.distributed.is_initialized():
        rank = torch.distributed.get_rank(group=process_group)
    executor = AttentionExecutor(
        fw_exec_plan=fw_exec_plan,
        bw_exec_plan=bw_exec_plan,
        fw_workload=fw_workload,
        bw_workload=bw_workload,
        node_id=rank // n_devices_per_node,
        local_device_id=rank % n_devices_per_node,
        n_devices_per_node=n_devices_per_node,
        n_nodes=n_nodes,
        n_heads_per_block=n_heads_per_block,
        head_dim=head_dim,
        synchronous=synchronous,
        process_group=process_group,
        iteration_idx=iteration_idx,
        tp_rank=tp_rank,
        use_cudagraph=use_cudagraph,
    )
    executor.register_handler(MemcpyInstr, _handle_memcpy)
    executor.register_handler(AttnInstr, _handle_attn)
    executor.register_handler(AttnBackwardInstr, _handle_attn_bw)
    executor.register_handler(AttnReductionInstr, _handle_reduction)
    executor.register_handler(SumInstr, _handle_sum)
    executor.register_handler(CommLaunchInstr, _reject_comm)
    executor.register_handler(CommWaitInstr, _reject_comm)
    executor.register_handler(BarrierInstr, _reject_comm)
    executor.register_prep_handler(MemcpyInstr, _prepare_memcpy)
    executor.register_prep_handler(AttnInstr, _prepare_attn)
    executor.register_prep_handler(AttnBackwardInstr, _prepare_attn_bw)
    executor.register_prep_handler(AttnReductionInstr, _prepare_reduction)
    executor.register_prep_handler(SumInstr, _prepare_sum)
    executor.check_all_handlers_registered()
    return executor
