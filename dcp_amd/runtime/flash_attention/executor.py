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
* where a plan's block movements are plain copies (the gather of the device's own blocks into
  slots that only the attention kernels read; a single-source scatter of a partial output, dQ or
  summed dK/dV back into the unpadded tensors) the kernels address the unpadded ``LOCAL_*``
  tensors themselves and the copies are not made (``direct.py``; ``direct_local`` of the
  executor, on by default, ``DCP_DIRECT_LOCAL=0`` in the environment turns it off).  The bytes
  in the ``LOCAL_*`` results are the same either way;
* communication instructions run over a ``LocalFabric`` (``fabric.py``): the
  executors of several devices share one GPU and one process, the sender's
  copy kernel writes into the receiver's staging buffer and signals with a
  stream event (two passes instead of the reference's pack, all-to-all and
  unpack, :1583-2074).  Without a fabric they raise: an exchange between
  GPUs is not part of this build.
"""

from __future__ import annotations

from collections import defaultdict
from typing import Dict, List, Optional, Tuple

import math
import os
import numpy as np
import torch

from dcp_amd.core.executor import DCPExecutor, HandlerTable
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
    CommType,
    CommWaitInstr,
    ExecutionPlan,
    MemcpyInstr,
    SumInstr,
)
from dcp_amd.core.serialization import int_to_torch_dtype
from dcp_amd.runtime.flash_attention.direct import DirectPlan, analyse as _analyse_direct
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
        fabric=None,
        direct_local: Optional[bool] = None,
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
        self.fabric = fabric
        self.pending_comm_ops: Dict[str, dict] = {}
        self._barrier_generation: Dict[int, int] = {}
        self.n_heads_per_block = n_heads_per_block
        self.head_dim = head_dim
        # The kernels exist for head sizes 64 and 128.  Another head size (up to 128) is stored at the
        # next of the two in every buffer this executor owns, the added columns zero (zero q and k
        # columns leave the scores unchanged; zero v and dout columns give zero out, dq, dk, dv
        # columns), so that no call pads or copies anything: the reference pads head sizes to what
        # its kernels take, too (dcp/runtime/flash_attention/executor.py:156-160).
        self.kernel_head_dim = head_dim if head_dim is None or head_dim > 128 else (64 if head_dim <= 64 else 128)
        self.main_stream = torch.cuda.Stream()
        self.streams: Dict[str, torch.cuda.Stream] = {}
        self._prep_handlers = HandlerTable("Prep handler")
        self._args_cache = {}
        self.register_synchronization_handler(torch.cuda.synchronize)
        self.fw_exec_plan = fw_exec_plan
        self.bw_exec_plan = bw_exec_plan
        self.fw_workload = fw_workload
        self.bw_workload = bw_workload
        self.mode = "Forward"
        self.use_cudagraph = use_cudagraph
        self.cuda_graph = None
        # let the kernels address the unpadded LOCAL_* tensors where the plan only copies (direct.py)
        self.direct_local = (os.environ.get("DCP_DIRECT_LOCAL", "1") != "0") if direct_local is None else bool(direct_local)
        self._direct = DirectPlan()

    # -- buffers ---------------------------------------------------------------
    def _create_buffer(self, buffer_shape: Tuple[int, ...], buffer_dtype: int):
        return torch.zeros(*buffer_shape, dtype=int_to_torch_dtype(buffer_dtype), device="cuda")

    def init_buffers(self, execution_plan: ExecutionPlan):
        """As the base class, with two differences.  The unpadded token-major tensors get one block of
        zeroed tokens behind their last one: kernels that address them directly load whole tiles,
        i.e. up to a block past a ragged last block (masked, but it has to be readable and finite).
        And a head size the kernels do not have is stored at the next one they have (see
        ``kernel_head_dim``): shapes, per-token sizes and block strides are those of the wider rows."""
        d, dk = self.head_dim, self.kernel_head_dim
        for buffer_type, info in execution_plan.buffer_info.items():
            shape, per_token_shape, numel = tuple(info.buffer_shape), tuple(info.per_token_shape), info.block_numel
            if dk != d and buffer_type not in _LSE_BUFFER_TYPES and shape and shape[-1] == d:
                shape, per_token_shape, numel = shape[:-1] + (dk,), per_token_shape[:-1] + (dk,), numel // d * dk
            self.buffer_n_blocks[buffer_type] = info.n_blocks
            self.buffer_block_strides[buffer_type] = numel
            self.buffer_block_sizes[buffer_type] = info.block_size
            self.buffer_per_token_shape[buffer_type] = per_token_shape
            if self.buffers.get(buffer_type) is not None:
                continue
            if buffer_type.startswith("Local") and buffer_type not in _LSE_BUFFER_TYPES and len(shape) >= 2:
                per_token = int(np.prod(shape[1:]))
                flat = torch.zeros((shape[0] + info.block_size) * per_token, dtype=int_to_torch_dtype(info.dtype), device="cuda")
                self.buffers[buffer_type] = flat[: shape[0] * per_token].view(shape)
            else:
                self.buffers[buffer_type] = self._create_buffer(shape, info.dtype)

    def _user_view(self, buffer_type):
        """The caller's view of a buffer: without the columns added for the kernels' head size."""
        buf = self.buffers[buffer_type]
        if self.kernel_head_dim != self.head_dim and buffer_type not in _LSE_BUFFER_TYPES:
            return buf[..., : self.head_dim]
        return buf

    def init_forward_input(self, local_q, local_kv):
        self._user_view(BufferType.LOCAL_Q).copy_(local_q)
        self._user_view(BufferType.LOCAL_KV).copy_(local_kv)

    def init_backward_input(self, local_dout):
        self._user_view(BufferType.LOCAL_dOUT).copy_(local_dout)

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
        self._user_view(BufferType.LOCAL_OUT).copy_(out)
        self.buffers[BufferType.LOCAL_LSE].copy_(lse)

    def deallocate_all_buffers(self):
        self.buffers = {}
        self.streams = {}
        self._args_cache = {}

    # -- prepare / execute -------------------------------------------------------
    def register_prep_handler(self, instruction_type, handler):
        self._prep_handlers.register(instruction_type, handler)

    def prepare(self, forward=True):
        """Allocate the plan's buffers and build every instruction's device
        argument tables; after this ``execute`` allocates nothing and never
        touches the host."""
        torch.cuda.nvtx.range_push("AttentionExecutor prepare")
        self._args_cache = {}
        self.pending_comm_ops = {}
        if self.fabric is not None:
            self.fabric.forget(self.rank)
        self.execution_plan = self.fw_exec_plan if forward else self.bw_exec_plan
        self.init_buffers(self.execution_plan)
        self._direct = _analyse_direct(self.execution_plan) if self.direct_local and self.fabric is None else DirectPlan()
        self._bwd_workspace_bytes = 0
        self._bwd_workspace = None
        for instr_index, instr in enumerate(self.execution_plan.instructions):
            self.instr_index = instr_index
            prep = self._prep_handlers.get(type(instr))
            if prep is not None:
                prep(self, instr)
        if self._bwd_workspace_bytes:
            self._bwd_workspace = torch.empty(self._bwd_workspace_bytes, dtype=torch.uint8, device="cuda")
        torch.cuda.nvtx.range_pop()

    def _reserve_backward_workspace(self, batch, total_q, block_size, n_heads, head_dim, total_kv) -> int:
        """Bytes of the backward scratch one instruction uses.  The plan's backward instructions run one
        after another on one stream and share a single buffer, sized for the largest.  The backward
        that keeps dS in memory needs 2 * block_size * n_heads bytes per key of the launch; past
        ``DCP_BWD_DS_MAX_BYTES`` (default: a quarter of the device's memory) the instruction gets the
        small scratch instead and the library recomputes."""
        nbytes = backward_workspace_bytes(batch, total_q, block_size, n_heads, head_dim, total_kv)
        limit = os.environ.get("DCP_BWD_DS_MAX_BYTES")
        limit = int(limit) if limit else torch.cuda.get_device_properties(torch.cuda.current_device()).total_memory // 4
        if nbytes > limit:
            nbytes = backward_workspace_bytes(batch, total_q, block_size, n_heads, head_dim, 0)
        self._bwd_workspace_bytes = max(self._bwd_workspace_bytes, nbytes)
        return nbytes

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
        if any(isinstance(i, (CommLaunchInstr, CommWaitInstr, BarrierInstr)) for i in plan.instructions):
            raise NotImplementedError("plans that exchange blocks with other devices are not captured into graphs")
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
            for stream in self.streams.values():
                self.main_stream.wait_stream(stream)
        prev_stream.wait_stream(self.main_stream)
        torch.cuda.nvtx.range_pop()
        if is_forward:
            return self._user_view(BufferType.LOCAL_OUT), self.buffers[BufferType.LOCAL_LSE]
        return self._user_view(BufferType.LOCAL_dQ), self._user_view(BufferType.LOCAL_dKV)

    # -- one instruction at a time (several devices' plans run in turns: fabric.execute_together) --
    def begin(self, execution_plan):
        self.execution_plan = execution_plan
        self.init_buffers(execution_plan)
        self._prev_stream = torch.cuda.current_stream()
        self.main_stream.wait_stream(self._prev_stream)

    def step(self, instr_index: int):
        with torch.cuda.stream(self.main_stream):
            self.instr_index = instr_index
            self._execute_instruction(self.execution_plan.instructions[instr_index])

    def finish(self):
        for stream in self.streams.values():
            self.main_stream.wait_stream(stream)
        self._prev_stream.wait_stream(self.main_stream)

    def comm_ready(self, key: str) -> bool:
        """Have all peers this device receives from under ``key`` launched their sends?"""
        pending = self.pending_comm_ops.get(key)
        if pending is None:
            raise RuntimeError(f"CommWaitInstr {key!r} without a CommLaunchInstr before it")
        return all(self.fabric.posted(peer, self.rank, key) is not None for peer in pending["recv_peers"])

    def barrier_ready(self, instr_index: int) -> bool:
        if instr_index not in self._barrier_generation:
            self._barrier_generation[instr_index] = self.fabric.barrier_arrive(self.rank)
        if not self.fabric.barrier_passed(self._barrier_generation[instr_index]):
            return False
        del self._barrier_generation[instr_index]
        return True

    def forward(self, q, kv):
        self.init_forward_input(q, kv)
        self.execute(self.fw_exec_plan, is_forward=True)
        return (
            self._user_view(BufferType.LOCAL_OUT).detach().clone(),
            self.buffers[BufferType.LOCAL_LSE].detach().clone(),
        )

    def backward(self, q, kv, out, dout, lse):
        self.set_local_out_lse(out, lse)
        self.init_forward_input(q, kv)
        self.init_backward_input(dout)
        self.execute(self.bw_exec_plan, is_forward=False)
        return (
            self._user_view(BufferType.LOCAL_dQ).detach().clone(),
            self._user_view(BufferType.LOCAL_dKV).detach().clone(),
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


def _size_classes(block_numels) -> dict:
    """``{block numel: class}`` such that blocks within a factor of four of a class's largest share
    a launch: its grid is sized for the largest of them, so at most three in four workgroups of
    the smallest find nothing to do, whereas a 64 KiB block in a grid sized for 4 MiB blocks would
    idle 63 in 64.  (Q and KV blocks of one plan, a factor 2 to 5 apart at most head layouts, land
    in one class.)"""
    classes, top = {}, None
    for n in sorted(set(int(x) for x in block_numels), reverse=True):
        if top is None or n * 4 < top:
            top = n
        classes[n] = top
    return classes


def _prepare_memcpy(exec: AttentionExecutor, instr: MemcpyInstr):
    """One argument table per (dtype, size class) for data blocks and one for LSE blocks.  The source
    is the unpadded buffer, addressed by ``local_cu_seqlens`` (reference ``_prepare_memcpy`` :606-790,
    which makes one table, and one launch, per (dtype, block numel): here blocks of similar
    sizes share a launch, whose grid is sized for the largest -- every block carries its own
    element count and stride, and the workgroups past a smaller block's end leave at once)."""
    cu = exec.execution_plan.local_cu_seqlens
    data = defaultdict(lambda: [[] for _ in range(7)])
    lse = defaultdict(lambda: [[] for _ in range(7)])
    head_block_size = None
    size_class = _size_classes(exec.buffer_block_strides[src.buffer_type] for src, _ in instr.src_dst_pairs
                               if src.buffer_type not in _LSE_BUFFER_TYPES)
    skipped = exec._direct.skip_pairs.get(exec.instr_index, ())
    for pos, (src, dst) in enumerate(instr.src_dst_pairs):
        if pos in skipped:  # the kernels read the source where it lies
            continue
        src_buf, dst_buf = exec.buffers[src.buffer_type], exec.buffers[dst.buffer_type]
        src_off = cu[src.index]
        key = ((src_buf.dtype, exec.buffer_block_strides[src.buffer_type]) if src.buffer_type in _LSE_BUFFER_TYPES
               else (src_buf.dtype, size_class[exec.buffer_block_strides[src.buffer_type]]))
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
        # key: (dtype, the largest block numel of the launch)
        "other": {(dtype, max(cols[5])): tables(cols) for (dtype, _), cols in data.items()},
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


def _compact_rows(instr, attn_mask: torch.Tensor):
    """Row lengths and ranges without the rows' padding: the plan gives every row ``seqlens_q`` =
    the padded block size and ``[0, 0)`` ranges for the padding; a kernel that writes into an
    unpadded tensor must not see the padding as queries at all."""
    n_tokens = [row[0].n_tokens for row in instr.q_block_table]
    keep = np.concatenate([np.arange(n, dtype=np.int64) + start for n, start in
                           zip(n_tokens, np.concatenate(([0], np.cumsum(instr.seqlens_q)[:-1])))]
                          or [np.zeros(0, dtype=np.int64)])
    return n_tokens, attn_mask[..., torch.from_numpy(keep).to(attn_mask.device)].contiguous()


def _token_table(cu, rows, width: int = 1) -> List[List[int]]:
    """Block table of token offsets (local block ``i`` starts at token ``local_cu_seqlens[i]``): one
    row per attention row, from its local block index or list of indices, padded with -1."""
    table = []
    for row in rows:
        blocks = row if isinstance(row, list) else [row]
        table.append([cu[i] for i in blocks] + [-1] * (width - len(blocks)))
    return table


def _prepare_attn(exec: AttentionExecutor, instr: AttnInstr):
    direct = exec._direct.operands.get(exec.instr_index, {})
    cu = exec.execution_plan.local_cu_seqlens
    seqlens_q, mask = instr.seqlens_q, _mask_tensor(instr.attn_mask)
    if direct:
        seqlens_q, mask = _compact_rows(instr, mask)
    width = max(len(row) for row in instr.kv_block_table)
    exec._args_cache[exec.instr_index] = (
        sum(seqlens_q),
        _cu(seqlens_q),
        _cu(instr.seqlens_kv),
        _dev(_token_table(cu, direct["q"]) if "q" in direct else _pad_block_table(instr.q_block_table), torch.int32),
        _dev(_token_table(cu, direct["kv"], width) if "kv" in direct else _pad_block_table(instr.kv_block_table), torch.int32),
        _dev(_token_table(cu, direct["out"]) if "out" in direct else _pad_block_table(instr.out_block_table), torch.int32),
        mask,
        _longest_first(instr.seqlens_kv),
        frozenset(direct),
        forward_workspace(),
    )


def _kv_views(kv: torch.Tensor):
    """K and V of a paged ``[slots, block, 2, heads, D]`` or unpadded ``[tokens, 2, heads, D]`` buffer."""
    return (kv[:, :, 0], kv[:, :, 1]) if kv.dim() == 5 else (kv[:, 0], kv[:, 1])


def _handle_attn(exec: AttentionExecutor, instr: AttnInstr):
    torch.cuda.nvtx.range_push("AttnInstr")
    (total_q, cu_q, cu_kv, q_table, kv_table, out_table, attn_mask, row_order, direct, workspace) = exec._args_cache[
        exec.instr_index
    ]
    # an operand the plan only copies is read (written) in the unpadded tensor, by token offset
    k, v = _kv_views(exec.buffers[BufferType.LOCAL_KV if "kv" in direct else BufferType.BUFFER_KV])
    _flash_attn_varlen_forward(
        exec.buffers[BufferType.LOCAL_Q if "q" in direct else BufferType.BUFFER_Q],
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
        out_=exec.buffers[BufferType.LOCAL_OUT if "out" in direct else BufferType.BUFFER_OUT],
        lse_=exec.buffers[BufferType.LOCAL_LSE if "out" in direct else BufferType.BUFFER_LSE],
        row_order=row_order,
        workspace=workspace,
        block_size=exec.buffer_block_sizes[BufferType.BUFFER_Q],
        merged_form="out" in direct,  # the scatter this replaces leaves lse = -1 where no key is visible
    )
    torch.cuda.nvtx.range_pop()


def _prepare_attn_bw(exec: AttentionExecutor, instr: AttnBackwardInstr):
    direct = exec._direct.operands.get(exec.instr_index, {})
    cu = exec.execution_plan.local_cu_seqlens
    seqlens_q, mask = instr.seqlens_q, _mask_tensor(instr.attn_mask)
    if direct:
        seqlens_q, mask = _compact_rows(instr, mask)
    total_q = sum(seqlens_q)
    hb = exec.buffer_per_token_shape[BufferType.BUFFER_dQ][-2]
    d = exec.buffer_per_token_shape[BufferType.BUFFER_dQ][-1]
    bs = exec.buffer_block_sizes[BufferType.BUFFER_dQ]
    width = max(len(row) for row in instr.kv_block_table)
    exec._args_cache[exec.instr_index] = (
        total_q,
        sum(instr.seqlens_kv),
        _cu(seqlens_q),
        _cu(instr.seqlens_kv),
        _dev(_token_table(cu, direct["q"]) if "q" in direct else _pad_block_table(instr.q_block_table), torch.int32),
        _dev(_token_table(cu, direct["kv"], width) if "kv" in direct else _pad_block_table(instr.kv_block_table), torch.int32),
        _dev(_token_table(cu, direct["out"]) if "out" in direct else _pad_block_table(instr.out_block_table), torch.int32),
        mask,
        _dev(_token_table(cu, direct["dq"]) if "dq" in direct else _pad_block_table(instr.dq_block_table), torch.int32),
        _dev(_pad_block_table(instr.dkv_block_table), torch.int32),
        exec._reserve_backward_workspace(len(instr.seqlens_q), total_q, bs, hb, d, sum(instr.seqlens_kv)),
        _longest_first(instr.seqlens_kv),
        frozenset(direct),
    )


def _handle_attn_bw(exec: AttentionExecutor, instr: AttnBackwardInstr):
    torch.cuda.nvtx.range_push("AttnBackwardInstr")
    (total_q, total_kv, cu_q, cu_kv, q_table, kv_table, out_table, attn_mask, dq_table, dkv_table,
     workspace_bytes, row_order, direct) = exec._args_cache[exec.instr_index]
    workspace = exec._bwd_workspace[:workspace_bytes]
    buf = exec.buffers
    k, v = _kv_views(buf[BufferType.LOCAL_KV if "kv" in direct else BufferType.BUFFER_KV])
    dk, dv = _kv_views(buf[BufferType.BUFFER_dKV])
    _flash_attn_varlen_backward(
        buf[BufferType.LOCAL_dOUT if "out" in direct else BufferType.BUFFER_dOUT],
        buf[BufferType.LOCAL_Q if "q" in direct else BufferType.BUFFER_Q],
        k,
        v,
        buf[BufferType.LOCAL_OUT if "out" in direct else BufferType.BUFFER_OUT],
        buf[BufferType.LOCAL_LSE if "out" in direct else BufferType.BUFFER_LSE],
        buf[BufferType.LOCAL_dQ if "dq" in direct else BufferType.BUFFER_dQ],
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
        block_size=exec.buffer_block_sizes[BufferType.BUFFER_dKV],
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
    skipped = exec._direct.skip_ops.get(exec.instr_index, ())
    for pos, op in enumerate(instr.ops):
        if pos in skipped:  # the attention kernel wrote this block where the op would have put it
            continue
        srcs = [out_blk.index for out_blk, _ in op.src_buffers]
        table.append(srcs + [-1] * (width - len(srcs)))
        idx = op.dst_buffer[0].index
        dst_offsets.append(cu[idx] if unpadded else idx * exec.buffer_block_sizes[types[2]])
        n_tokens.append(op.dst_buffer[0].n_tokens)
        n_srcs.append(len(srcs))
    dst_lse = exec.buffers[types[3]]
    if not table:
        exec._args_cache[exec.instr_index] = None
        return
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
    if exec._args_cache[exec.instr_index] is None:  # every op of the plan's was a scatter the kernels made themselves
        return
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
        exec.n_heads_per_block * exec.kernel_head_dim,
        exec.buffer_block_sizes[src_lse_t],
        1,
        exec.buffer_n_blocks[src_lse_t] * exec.buffer_block_sizes[src_lse_t],
        dst_lse_head_stride,
        exec.kernel_head_dim,
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
    # one launch per (dtype, size class): sums over blocks of similar sizes share it (its grid is
    # sized for the largest block, every sum carries its own element count and strides)
    size_class = _size_classes(exec.buffer_block_strides[op.src_buffers[0].buffer_type] for op in instr.ops)
    skipped = exec._direct.skip_ops.get(exec.instr_index, ())
    redirected = exec._direct.redirect_ops.get(exec.instr_index, {})
    for pos, op in enumerate(instr.ops):
        if pos in skipped:  # a kernel or an earlier sum wrote this block where the op would have put it
            continue
        src_type = op.src_buffers[0].buffer_type
        # a sum whose slot the plan only scatters back afterwards goes straight to the unpadded tensor
        dst_block = redirected.get(pos, op.dst_buffer)
        unpadded = bool(instr.output_is_unpadded) or pos in redirected
        dst_type = dst_block.buffer_type
        g = groups[(exec.buffers[src_type].dtype, size_class[exec.buffer_block_strides[src_type]])]
        per_token = int(np.prod(exec.buffer_per_token_shape[src_type]))
        g["src_ptrs"].append(exec.buffers[src_type].data_ptr())
        g["src_offsets"].append([blk.index for blk in op.src_buffers])
        g["src_strides"].append(exec.buffer_block_strides[src_type])
        g["n_ops"].append(len(op.src_buffers))
        g["dst_ptrs"].append(exec.buffers[dst_type].data_ptr())
        if unpadded:
            g["dst_offsets"].append(cu[dst_block.index])
            g["dst_strides"].append(per_token)
        else:
            g["dst_offsets"].append(dst_block.index)
            g["dst_strides"].append(exec.buffer_block_strides[dst_type])
        g["n_elems"].append(dst_block.n_tokens * per_token)
    prepared = {}
    for (dtype, _), g in groups.items():
        width = _round_to_pow_2(max(g["n_ops"]))
        padded = [row + [-1] * (width - len(row)) for row in g["src_offsets"]]
        prepared[(dtype, max(g["src_strides"]))] = (
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
# CommLaunchInstr / CommWaitInstr / BarrierInstr over a LocalFabric
# ---------------------------------------------------------------------------

_DATA_KINDS = (torch.int64, torch.int32, torch.int32, torch.int64, torch.int32, torch.int32, torch.int32)


def _require_fabric(exec: AttentionExecutor, instr: BlockInstrBase):
    if exec.fabric is None:
        raise NotImplementedError(
            f"{type(instr).__name__}: this executor has no fabric.  Blocks are exchanged between executors "
            "that share one GPU (get_executor(..., fabric=LocalFabric(...))); an exchange between GPUs is "
            "not part of this build"
        )


def _comm_block(exec: AttentionExecutor, block: BufferBlock):
    """What a communication op moves for ``block`` (the views of the reference's
    ``_prepare_comm_launch`` :1617-1640): ``("data", address, numel)`` for a contiguous run of
    tokens, ``("lse", base address, token offset, head stride, n_tokens)`` for the
    ``[head block, n_tokens]`` slice of an LSE buffer."""
    buf = exec.buffers[block.buffer_type]
    local = block.buffer_type.startswith("Local")
    if block.buffer_type in _LSE_BUFFER_TYPES:
        if local:
            return ("lse", buf.data_ptr(), exec.execution_plan.local_cu_seqlens[block.index], buf.stride(0), block.n_tokens)
        return ("lse", buf.data_ptr(), block.index * buf.shape[2], buf.stride(0), block.n_tokens)
    first = exec.execution_plan.local_cu_seqlens[block.index] if local else block.index
    per_token = int(np.prod(exec.buffer_per_token_shape[block.buffer_type]))
    return ("data", buf.data_ptr() + first * buf.stride(0) * buf.element_size(), block.n_tokens * per_token)


class _CopyTables:
    """Argument tables of the copy launches that move a list of blocks between their buffers
    and a staging buffer: one launch per (dtype, block numel) for data blocks, one for LSE
    blocks."""

    def __init__(self):
        self.data = defaultdict(lambda: [[] for _ in range(7)])
        self.lse = [[] for _ in range(7)]
        self.hb = None

    def add(self, exec: AttentionExecutor, block: BufferBlock, desc, dtype, staging_address: int, to_staging: bool):
        if desc[0] == "data":
            cols = self.data[(dtype, exec.buffer_block_strides[block.buffer_type])]
            src, dst = (desc[1], staging_address) if to_staging else (staging_address, desc[1])
            for col, v in zip(cols, (src, 0, 1, dst, 0, 1, desc[2])):
                col.append(v)
            return
        _, base, token_offset, head_stride, n_tokens = desc
        self.hb = exec.buffers[block.buffer_type].shape[0]
        mine = (base, token_offset, head_stride)
        theirs = (staging_address, 0, n_tokens)  # [head block, n_tokens], contiguous
        src, dst = (mine, theirs) if to_staging else (theirs, mine)
        for col, v in zip(self.lse, (*src, *dst, n_tokens)):
            col.append(v)

    def freeze(self):
        data = {key: tuple(_dev(c, k) for c, k in zip(cols, _DATA_KINDS)) for key, cols in self.data.items()}
        lse = None
        if self.lse[0]:
            lse = tuple(_dev(c, k) for c, k in zip(self.lse, _DATA_KINDS)) + (self.hb, max(self.lse[6]))
        return data, lse


def _launch_copies(frozen):
    data, lse = frozen
    for (dtype, block_numel), args in data.items():
        _COPY_FN[dtype](*args, block_numel, 128)
    if lse is not None:
        *tables, hb, max_tokens = lse
        fused_copy_fp32_varlen_lse(*tables, hb, max_tokens, 1)


def _block_numel(exec: AttentionExecutor, block: BufferBlock, desc) -> int:
    if desc[0] == "data":
        return desc[2]
    return exec.buffers[block.buffer_type].shape[0] * desc[4]


def _comm_stream(exec: AttentionExecutor, name: Optional[str]):
    if name is None:
        return torch.cuda.current_stream()
    return exec.streams[name]


def _prepare_comm_launch(exec: AttentionExecutor, instr: CommLaunchInstr):
    """Receives: one staging buffer per dtype, the peers' segments in rank order and each
    peer's blocks in op order (the recv buffer of the reference, :1752-1776), registered with
    the fabric, and the unpack tables.  Sends: only described here; their tables need the
    receivers' staging addresses, which exist once every device has prepared, so they are
    built at the first launch."""
    _require_fabric(exec, instr)
    if instr.stream is not None and instr.stream not in exec.streams:
        exec.streams[instr.stream] = torch.cuda.Stream()
    sends = []  # (peer, dtype, block, desc)
    recvs = defaultdict(lambda: defaultdict(list))  # dtype -> peer -> [(block, desc)]
    for op in instr.comm_ops:
        peer = exec.get_rank(*op.peer)
        desc = _comm_block(exec, op.buffer_block)
        dtype = exec.buffers[op.buffer_block.buffer_type].dtype
        if dtype not in _COPY_FN:
            raise ValueError(f"Unsupported dtype {dtype}")
        if desc[0] == "lse" and dtype != torch.float32:
            raise ValueError(f"Unsupported LSE dtype {dtype}")
        if op.comm_type == CommType.SEND:
            sends.append((peer, dtype, op.buffer_block, desc))
        else:
            recvs[dtype][peer].append((op.buffer_block, desc))
    unpack = _CopyTables()
    staging_buffers = []
    for dtype, per_peer in recvs.items():
        segments, total = {}, 0
        for peer in sorted(per_peer):
            numels = [_block_numel(exec, block, desc) for block, desc in per_peer[peer]]
            segments[peer] = (total, numels)
            total += sum(numels)
        staging = torch.empty(total, dtype=dtype, device="cuda")
        staging_buffers.append(staging)
        exec.fabric.register_staging(exec.rank, instr.key, dtype, staging, segments)
        for peer in sorted(per_peer):
            at = segments[peer][0]
            for (block, desc), numel in zip(per_peer[peer], segments[peer][1]):
                unpack.add(exec, block, desc, dtype, staging.data_ptr() + at * staging.element_size(), to_staging=False)
                at += numel
    exec._args_cache[exec.instr_index] = {
        "sends": sends,
        "pack": None,
        "epoch": None,
        "send_peers": sorted({peer for peer, _, _, _ in sends}),
        "recv_peers": sorted({peer for per_peer in recvs.values() for peer in per_peer}),
        "unpack": unpack.freeze(),
        "staging": staging_buffers,
    }


def _resolve_sends(exec: AttentionExecutor, instr: CommLaunchInstr, cache: dict):
    pack = _CopyTables()
    at: Dict[Tuple[int, torch.dtype], int] = {}
    seen: Dict[Tuple[int, torch.dtype], int] = {}
    for peer, dtype, block, desc in cache["sends"]:
        staging, offset, numels = exec.fabric.staging_segment(peer, instr.key, dtype, exec.rank)
        k = (peer, dtype)
        i = seen.get(k, 0)
        numel = _block_numel(exec, block, desc)
        if i >= len(numels) or numels[i] != numel:
            raise RuntimeError(
                f"key {instr.key!r}: send {i} of rank {exec.rank} to rank {peer} has {numel} elements, "
                f"the receiver expects {numels[i] if i < len(numels) else 'no such block'}"
            )
        pos = at.get(k, offset)
        pack.add(exec, block, desc, dtype, staging.data_ptr() + pos * staging.element_size(), to_staging=True)
        at[k] = pos + numel
        seen[k] = i + 1
    for (peer, dtype), n in seen.items():
        expected = len(exec.fabric.staging_segment(peer, instr.key, dtype, exec.rank)[2])
        if n != expected:
            raise RuntimeError(f"key {instr.key!r}: rank {exec.rank} sends {n} blocks to rank {peer}, which expects {expected}")
    cache["pack"] = pack.freeze()


def _handle_comm_launch(exec: AttentionExecutor, instr: CommLaunchInstr):
    torch.cuda.nvtx.range_push("CommLaunchInstr")
    _require_fabric(exec, instr)
    cache = exec._args_cache[exec.instr_index]
    if cache["pack"] is None or cache["epoch"] != exec.fabric.epoch:
        # first launch, or a peer has prepared again since: its staging buffers are new ones
        _resolve_sends(exec, instr, cache)
        cache["epoch"] = exec.fabric.epoch
    issuing = torch.cuda.current_stream()
    stream = _comm_stream(exec, instr.stream)
    stream.wait_stream(issuing)  # the blocks to send were produced by what came before on this device
    with torch.cuda.stream(stream):
        for peer in cache["send_peers"]:
            done = exec.fabric.consumed(peer, instr.key)
            if done is not None:
                stream.wait_event(done)  # the receiver's last unpack of this staging buffer
        _launch_copies(cache["pack"])
        launched = torch.cuda.Event()
        launched.record(stream)
        for peer in cache["send_peers"]:
            exec.fabric.post(exec.rank, peer, instr.key, launched)
    exec.pending_comm_ops[instr.key] = {"recv_peers": cache["recv_peers"], "unpack": cache["unpack"], "launched": launched}
    torch.cuda.nvtx.range_pop()


def _prepare_comm_wait(exec: AttentionExecutor, instr: CommWaitInstr):
    _require_fabric(exec, instr)
    if instr.stream is not None and instr.stream not in exec.streams:
        exec.streams[instr.stream] = torch.cuda.Stream()


def _handle_comm_wait(exec: AttentionExecutor, instr: CommWaitInstr):
    torch.cuda.nvtx.range_push("CommWaitInstr")
    _require_fabric(exec, instr)
    if not exec.comm_ready(instr.key):
        raise RuntimeError(
            f"CommWaitInstr {instr.key!r} on rank {exec.rank}: a peer has not launched its sends yet "
            "(run the devices' plans with fabric.execute_together)"
        )
    pending = exec.pending_comm_ops.pop(instr.key)
    stream = _comm_stream(exec, instr.stream)
    with torch.cuda.stream(stream):
        # the wait covers this device's own part of the exchange too, as waiting for the
        # reference's all-to-all does: what the launch's stream did before it is done
        stream.wait_event(pending["launched"])
        for peer in pending["recv_peers"]:
            stream.wait_event(exec.fabric.take(peer, exec.rank, instr.key))
        _launch_copies(pending["unpack"])
        if pending["recv_peers"]:
            event = torch.cuda.Event()
            event.record(stream)
            exec.fabric.set_consumed(exec.rank, instr.key, event)
    torch.cuda.nvtx.range_pop()


def _handle_barrier(exec: AttentionExecutor, instr: BarrierInstr):
    """All devices have reached the barrier when this runs (``execute_together`` holds a device
    back until then): what is left of the reference's all-reduce (:2006-2012) is to wait for
    the device's own work."""
    _require_fabric(exec, instr)
    torch.cuda.current_stream().synchronize()


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
    fabric=None,
):
    """Factory with the reference's signature (:2077-2133) plus ``fabric``.  ``exec_context``
    only supplies ``n_devices_per_node`` / ``n_nodes`` and may be ``None``.  With a
    ``LocalFabric`` the executor is one of several devices sharing this GPU: the fabric gives
    the device grid and the plan says which device it is."""
    if executor_impl != "python":
        raise ValueError(f"Unsupported executor_impl: {executor_impl}")
    n_devices_per_node = getattr(exec_context, "n_devices_per_node", 1)
    n_nodes = getattr(exec_context, "n_nodes", 1)
    rank = 0
    if fabric is not None:
        plan = fw_exec_plan if fw_exec_plan is not None else bw_exec_plan
        n_devices_per_node, n_nodes = fabric.n_devices_per_node, fabric.n_nodes
        rank = plan.node_id * n_devices_per_node + plan.local_device_id
    elif torch.distributed.is_available() and torch.distributed.is_initialized():
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
        fabric=fabric,
    )
    executor.register_handler(MemcpyInstr, _handle_memcpy)
    executor.register_handler(AttnInstr, _handle_attn)
    executor.register_handler(AttnBackwardInstr, _handle_attn_bw)
    executor.register_handler(AttnReductionInstr, _handle_reduction)
    executor.register_handler(SumInstr, _handle_sum)
    executor.register_handler(CommLaunchInstr, _handle_comm_launch)
    executor.register_handler(CommWaitInstr, _handle_comm_wait)
    executor.register_handler(BarrierInstr, _handle_barrier)
    executor.register_prep_handler(MemcpyInstr, _prepare_memcpy)
    executor.register_prep_handler(AttnInstr, _prepare_attn)
    executor.register_prep_handler(AttnBackwardInstr, _prepare_attn_bw)
    executor.register_prep_handler(AttnReductionInstr, _prepare_reduction)
    executor.register_prep_handler(SumInstr, _prepare_sum)
    executor.register_prep_handler(CommLaunchInstr, _prepare_comm_launch)
    executor.register_prep_handler(CommWaitInstr, _prepare_comm_wait)
    executor.check_all_handlers_registered()
    return executor
