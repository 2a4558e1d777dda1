"""Wire format and data model of the instruction set: every instruction type
and a whole ExecutionPlan survive serialize -> deserialize, the byte layout is
the reference's (little-endian 4-byte fields, 1-byte opcodes in definition
order), and malformed input fails loudly.  Mirrors the reference's
tests/core/test_instructions.py."""

import struct

import pytest
import torch

from dcp_amd.core.instructions import (
    AttnBackwardInstr,
    AttnInstr,
    AttnReductionInstr,
    BarrierInstr,
    BlockInstrBase,
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
    deserialize_list_of_execution_plans,
    serialize_list_of_execution_plans,
)
from dcp_amd.core.serialization import (
    bytes_to_int_meta,
    deserialize_float,
    deserialize_int_tuple,
    deserialize_list_of_ints,
    deserialize_str,
    int_meta_to_bytes,
    int_to_torch_dtype,
    serialize_float,
    serialize_int_tuple,
    serialize_list_of_ints,
    serialize_str,
    torch_dtype_to_int,
)


def blk(t, i, n=256):
    return BufferBlock(t, i, n)


def roundtrip(instr):
    data = instr.serialize()
    back, rest = BlockInstrBase.deserialize(data)
    assert rest == b""
    assert type(back) is type(instr)
    assert back == instr
    assert back.serialize() == data
    return data


def test_opcodes_follow_definition_order():
    order = [MemcpyInstr, CommLaunchInstr, BarrierInstr, CommWaitInstr, AttnInstr, AttnBackwardInstr,
             AttnReductionInstr, SumInstr]
    assert [c._instr_index for c in order] == list(range(8))


def test_scalar_codecs_are_little_endian_4_byte():
    assert int_meta_to_bytes(0x01020304) == bytes([4, 3, 2, 1])
    assert bytes_to_int_meta(bytes([4, 3, 2, 1, 9])) == (0x01020304, bytes([9]))
    assert serialize_list_of_ints([1, 2]) == struct.pack("<3I", 2, 1, 2)
    assert deserialize_list_of_ints(struct.pack("<3I", 2, 7, 8) + b"x") == ([7, 8], b"x")
    assert deserialize_int_tuple(serialize_int_tuple((3, 4, 5))) == ((3, 4, 5), b"")
    assert serialize_str("ab") == struct.pack("<I", 2) + b"ab"
    assert serialize_str("") == serialize_str(None) == struct.pack("<I", 0)
    assert deserialize_str(serialize_str("LocalQ") + b"!") == ("LocalQ", b"!")
    assert deserialize_float(serialize_float(-1.5)) == (-1.5, b"")
    assert serialize_float(1.0) == struct.pack("<d", 1.0)


def test_dtype_tables():
    for i, t in enumerate((torch.bfloat16, torch.float16, torch.float32, torch.int32, torch.int64)):
        assert torch_dtype_to_int(t) == i and int_to_torch_dtype(i) is t
    with pytest.raises(ValueError):
        torch_dtype_to_int(torch.float64)
    with pytest.raises(ValueError):
        int_to_torch_dtype(9)
    assert DType.as_str(DType.BFLOAT16) == "bf16" and DType.element_size(DType.FLOAT32) == 4
    with pytest.raises(ValueError):
        DType.from_num(7)


def test_memcpy_roundtrip_and_bytes():
    instr = MemcpyInstr([(blk(BufferType.LOCAL_Q, 0, 100), blk(BufferType.BUFFER_Q, 5, 100)),
                         (blk(BufferType.LOCAL_KV, 3), blk(BufferType.BUFFER_KV, 1))])
    data = roundtrip(instr)
    # opcode, pair count, then (name, index, n_tokens) x2 per pair
    assert data[0] == 0 and data[1:5] == struct.pack("<I", 2)
    assert data[5:9] == struct.pack("<I", len("LocalQ")) and data[9:15] == b"LocalQ"


def test_comm_instructions_roundtrip():
    ops = [CommOp(CommType.SEND, (0, 1), blk(BufferType.BUFFER_Q, 2)),
           CommOp(CommType.RECV, (1, 3), blk(BufferType.BUFFER_KV, 7, 12))]
    roundtrip(CommLaunchInstr("stage1", ops, stream="comm"))
    back, _ = BlockInstrBase.deserialize(CommLaunchInstr("k", ops).serialize())
    assert back.stream is None  # empty string on the wire reads back as None
    roundtrip(CommWaitInstr("stage1", stream=None))
    roundtrip(BarrierInstr())
    with pytest.raises(ValueError):
        CommType.from_num(5)


def _attn_args(two_ranges):
    total_q = 8
    if two_ranges:
        mask = torch.arange(2 * 2 * total_q, dtype=torch.int32).reshape(2, 2, total_q)
    else:
        mask = torch.arange(2 * total_q, dtype=torch.int32).reshape(2, total_q)
    return dict(
        stage_id=1, seqlens_q=[4, 4], seqlens_kv=[8, 4], max_seqlen_q=4, max_seqlen_kv=8, attn_mask=mask,
        q_block_table=[[blk(BufferType.BUFFER_Q, 0, 4)], [blk(BufferType.BUFFER_Q, 1, 3)]],
        kv_block_table=[[blk(BufferType.BUFFER_KV, 0, 4), blk(BufferType.BUFFER_KV, 2, 4)], [blk(BufferType.BUFFER_KV, 1, 3)]],
        out_block_table=[[blk(BufferType.BUFFER_OUT, 4, 4)], [blk(BufferType.BUFFER_OUT, 5, 3)]],
    )


@pytest.mark.parametrize("two_ranges", [False, True])
def test_attn_instr_roundtrip(two_ranges):
    args = _attn_args(two_ranges)
    lse = [[blk(BufferType.BUFFER_LSE, 4, 4)], [blk(BufferType.BUFFER_LSE, 5, 3)]]
    instr = AttnInstr(lse_block_table=lse, **args)
    roundtrip(instr)
    other = AttnInstr(lse_block_table=lse, **{**args, "attn_mask": args["attn_mask"] + 1})
    assert other != instr
    # a mask given as a list of planes (what a decoded reference plan holds) is the same mask
    planes = AttnInstr(lse_block_table=lse, **{**args, "attn_mask": [p for p in args["attn_mask"]]})
    assert planes == instr and planes.serialize() == instr.serialize()
    with pytest.raises(AssertionError):  # out and lse slots must agree
        AttnInstr(lse_block_table=[[blk(BufferType.BUFFER_LSE, 9, 4)], [blk(BufferType.BUFFER_LSE, 5, 3)]], **args)


@pytest.mark.parametrize("two_ranges", [False, True])
def test_attn_backward_instr_roundtrip(two_ranges):
    args = _attn_args(two_ranges)
    instr = AttnBackwardInstr(
        dq_block_table=[[blk(BufferType.BUFFER_dQ, 0, 4)], [blk(BufferType.BUFFER_dQ, 1, 3)]],
        dkv_block_table=[[blk(BufferType.BUFFER_dKV, 0, 4), blk(BufferType.BUFFER_dKV, 1, 4)],
                         [blk(BufferType.BUFFER_dKV, 2, 3)]],
        **args)
    roundtrip(instr)
    assert "attn_mask" not in repr(instr) and "BufferdKV[[0, 1], [2]]" in repr(instr)


def test_reduction_and_sum_roundtrip():
    red = AttnReductionInstr(
        [ReductionOp([(blk(BufferType.BUFFER_OUT, 0), blk(BufferType.BUFFER_LSE, 0)),
                      (blk(BufferType.BUFFER_OUT, 3), blk(BufferType.BUFFER_LSE, 3))],
                     (blk(BufferType.LOCAL_OUT, 1), blk(BufferType.LOCAL_LSE, 1)))],
        output_is_unpadded=1)
    roundtrip(red)
    with pytest.raises(ValueError):
        ReductionOp([(blk(BufferType.BUFFER_OUT, 0), blk(BufferType.BUFFER_LSE, 1))],
                    (blk(BufferType.LOCAL_OUT, 1), blk(BufferType.LOCAL_LSE, 1)))
    roundtrip(SumInstr([SumOp([blk(BufferType.BUFFER_dKV, 2), blk(BufferType.BUFFER_dKV, 6)],
                              blk(BufferType.BUFFER_dKV, 2))], output_is_unpadded=0))


def _plan():
    args = _attn_args(True)
    instrs = [
        MemcpyInstr([(blk(BufferType.LOCAL_Q, 0, 4), blk(BufferType.BUFFER_Q, 0, 4))]),
        AttnInstr(lse_block_table=[[blk(BufferType.BUFFER_LSE, 4, 4)], [blk(BufferType.BUFFER_LSE, 5, 3)]], **args),
        AttnReductionInstr([ReductionOp([(blk(BufferType.BUFFER_OUT, 4), blk(BufferType.BUFFER_LSE, 4))],
                                        (blk(BufferType.LOCAL_OUT, 0), blk(BufferType.LOCAL_LSE, 0)))], 1),
    ]
    info = {
        BufferType.LOCAL_Q: BufferInfo(2, 4, 4 * 2 * 8, 0, (7, 2, 8), (2, 8)),
        BufferType.BUFFER_LSE: BufferInfo(6, 4, 8, 2, (2, 6, 4), (1,)),
    }
    return ExecutionPlan(instrs, 1, 1, 0, 0, 2, [0, 4, 7], info)


def test_execution_plan_roundtrip():
    plan = _plan()
    data = plan.serialize()
    back, rest = ExecutionPlan.deserialize(data + b"tail")
    assert rest == b"tail" and back == plan and back.serialize() == data
    assert back.buffer_info[BufferType.LOCAL_Q].per_token_shape == (2, 8)
    assert "MemcpyInstr" in str(plan)
    changed = _plan()
    changed.local_cu_seqlens = [0, 4, 8]
    assert changed != plan
    plans, rest = deserialize_list_of_execution_plans(serialize_list_of_execution_plans([plan, changed]))
    assert rest == b"" and plans == [plan, changed]


def test_truncated_input_raises():
    data = _plan().serialize()
    with pytest.raises(ValueError):
        ExecutionPlan.deserialize(data[: len(data) // 2])
    with pytest.raises(KeyError):
        BlockInstrBase.deserialize(bytes([200]))
