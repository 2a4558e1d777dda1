"""Handler registry and instruction loop of the abstract executor (no GPU):
the error behaviour of the reference's dcp/core/executor.py."""

import pytest

from dcp_amd.core.executor import DCPExecutor
from dcp_amd.core.instructions import (
    BarrierInstr,
    BlockInstrBase,
    BufferBlock,
    BufferInfo,
    BufferType,
    ExecutionPlan,
    MemcpyInstr,
)


class RecordingExecutor(DCPExecutor):
    def _create_buffer(self, shape, dtype):
        return ("buffer", tuple(shape), dtype)


def _plan(instrs):
    info = {BufferType.LOCAL_Q: BufferInfo(1, 4, 32, 0, (4, 1, 8), (1, 8))}
    return ExecutionPlan(instrs, 1, 1, 0, 0, 1, [0, 4], info)


def test_all_leaf_instructions_need_a_handler():
    ex = RecordingExecutor(node_id=0, local_device_id=0, n_devices_per_node=1, n_nodes=1)
    needed = ex.get_all_needed_handlers()
    assert set(needed) == {"MemcpyInstr", "CommLaunchInstr", "BarrierInstr", "CommWaitInstr", "AttnInstr",
                           "AttnBackwardInstr", "AttnReductionInstr", "SumInstr"}
    with pytest.raises(ValueError, match="No handler registered"):
        ex.check_all_handlers_registered()
    with pytest.raises(TypeError):
        ex.register_handler(int, lambda e, i: None)
    ex.register_handler(MemcpyInstr, lambda e, i: None)
    with pytest.raises(ValueError, match="already registered"):
        ex.register_handler(MemcpyInstr, lambda e, i: None)


def test_execute_dispatches_in_order_and_creates_buffers():
    ex = RecordingExecutor(node_id=0, local_device_id=1, n_devices_per_node=4, n_nodes=2, synchronous=True)
    seen, syncs = [], []
    ex.register_handler(MemcpyInstr, lambda e, i: seen.append((e.instr_index, type(i).__name__)))
    ex.register_synchronization_handler(lambda: syncs.append(1))
    m = MemcpyInstr([(BufferBlock(BufferType.LOCAL_Q, 0, 4), BufferBlock(BufferType.BUFFER_Q, 0, 4))])
    ex.execute(_plan([m, m]))
    assert seen == [(0, "MemcpyInstr"), (1, "MemcpyInstr")] and len(syncs) == 2
    assert ex.buffers[BufferType.LOCAL_Q] == ("buffer", (4, 1, 8), 0)
    assert ex.buffer_block_strides[BufferType.LOCAL_Q] == 32 and ex.buffer_block_sizes[BufferType.LOCAL_Q] == 4
    assert ex.rank == 1 and ex.reverse_get_rank(5) == (1, 1)
    with pytest.raises(ValueError, match="No handler registered for instruction BarrierInstr"):
        ex.execute(_plan([BarrierInstr()]))


def test_synchronize_must_be_registered():
    ex = RecordingExecutor(synchronous=True)
    ex.register_handler(MemcpyInstr, lambda e, i: None)
    m = MemcpyInstr([])
    with pytest.raises(NotImplementedError):
        ex.execute(_plan([m]))
    with pytest.raises(NotImplementedError):
        DCPExecutor()._create_buffer((1,), 0)


def test_attention_wrappers_reject_block_tables_of_the_wrong_shape():
    """The kernels index every wide table with kv_block_table's width and every table by row:
    a mismatch is a ValueError on the host, not an out-of-bounds read on the device."""
    import torch

    from dcp_amd.flash_attn_interface import _check_tables

    i32 = lambda *shape: torch.zeros(*shape, dtype=torch.int32)
    ok = dict(q_block_table=i32(3, 1), out_block_table=i32(3, 1))
    _check_tables(3, i32(4), None, ok, dict(kv_block_table=i32(3, 5), dkv_block_table=i32(3, 5)))
    with pytest.raises(ValueError, match="width of kv_block_table"):
        _check_tables(3, i32(4), None, ok, dict(kv_block_table=i32(3, 5), dkv_block_table=i32(3, 8)))
    with pytest.raises(ValueError, match=r"q_block_table must be \[3, 1\]"):
        _check_tables(3, i32(4), None, dict(q_block_table=i32(4, 1)), dict(kv_block_table=i32(3, 5)))
    with pytest.raises(ValueError, match="kv_block_table must be"):
        _check_tables(3, i32(4), None, ok, dict(kv_block_table=i32(2, 5)))
    with pytest.raises(ValueError, match="cu_seqlens_k"):
        _check_tables(3, i32(5), None, ok, dict(kv_block_table=i32(3, 5)))
    with pytest.raises(ValueError, match="row_order"):
        _check_tables(3, i32(4), i32(2), ok, dict(kv_block_table=i32(3, 5)))


def test_blocks_share_a_launch_only_within_a_factor_of_four():
    from dcp_amd.runtime.flash_attention.executor import _size_classes

    c = _size_classes([524288, 262144, 327680, 131072, 131071, 4096, 1 << 22, 65536, 16385])
    assert c[524288] == c[262144] == c[327680] == c[131072] == 524288  # Q and KV blocks of one plan
    assert c[131071] == 131071 and c[65536] == 131071  # just under a quarter of the largest: the next class starts
    assert c[1 << 22] == 1 << 22 and c[4096] == 4096 and c[16385] == 16385
    for n, top in c.items():
        assert n <= top <= 4 * n
