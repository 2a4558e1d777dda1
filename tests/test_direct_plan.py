"""Host logic of dcp_amd/runtime/flash_attention/direct.py (no GPU): which of a plan's copies the
executor may skip.  The analysis only reads the instruction list; these tests pin what it finds on
the plan families the builders produce, that it leaves alone what it must (slots that something other
than an attention kernel reads, plans that exchange blocks), and -- by replaying the plan on names
instead of data -- that every block an attention instruction would read directly is the block the
copy it skips would have put into the slot, and every result written directly lands where the
skipped scatter would have moved it."""

import copy

import pytest

from dcp_amd.core.instructions import AttnReductionInstr, BufferBlock, BufferType, MemcpyInstr, ReductionOp
from dcp_amd.runtime.flash_attention.direct import analyse
from tests.plan_cases import make_case, make_multi_case

SINGLE_STAGE = dict(seqlens=[200, 330], block_size=64, n_heads=4, n_groups=4, head_dim=16, head_block=2)
THREE_PARTIALS = dict(seqlens=[500, 130], block_size=64, n_heads=8, n_groups=2, head_dim=16, head_block=2, n_kv_groups=3)
FOLDED = dict(seqlens=[700], block_size=64, n_heads=2, n_groups=2, head_dim=16, head_block=1, mask="lambda",
              mask_info=[16, 96], n_kv_groups=2, kv_split="contiguous", fold=True)


def _kinds(plan):
    return [type(i).__name__ for i in plan.instructions]


def test_single_stage_plan_needs_no_copy_at_all():
    case = make_case(**SINGLE_STAGE)
    fw, bw = analyse(case["fw"]), analyse(case["bw"])
    assert _kinds(case["fw"]) == ["MemcpyInstr", "AttnInstr", "AttnReductionInstr"]
    n_pairs = len(case["fw"].instructions[0].src_dst_pairs)
    assert fw.skip_pairs == {0: set(range(n_pairs))}
    assert set(fw.operands[1]) == {"q", "kv", "out"}
    assert fw.skip_ops == {2: set(range(len(case["fw"].instructions[2].ops)))}
    # backward: q, kv, out/lse/dout read in place, dQ written in place, the dK/dV replica sums written
    # straight to LOCAL_dKV (their scatter skipped), the single-source dQ scatter skipped
    assert bw.skip_pairs == {0: set(range(len(case["bw"].instructions[0].src_dst_pairs)))}
    assert set(bw.operands[1]) == {"q", "kv", "out", "dq"}
    sums = [i for i, ins in enumerate(case["bw"].instructions) if type(ins).__name__ == "SumInstr"]
    assert set(bw.redirect_ops) | set(bw.skip_ops) == set(sums)
    for idx, ops in bw.redirect_ops.items():
        for pos, dst in ops.items():
            assert dst.buffer_type == BufferType.LOCAL_dKV
            assert dst.n_tokens == case["bw"].instructions[idx].ops[pos].dst_buffer.n_tokens


@pytest.mark.parametrize("cfg", [THREE_PARTIALS, FOLDED], ids=["merged_at_the_end", "folded"])
def test_partials_that_a_merge_reads_stay_in_their_slots(cfg):
    """Several partials per row: q and kv are still read in place, but the partial outputs are merged
    (more than one source per op), so they are written to slots and no reduction op is skipped."""
    case = make_case(**cfg)
    fw = analyse(case["fw"])
    attn = [i for i, ins in enumerate(case["fw"].instructions) if type(ins).__name__ == "AttnInstr"]
    assert len(attn) > 1
    for i in attn:
        assert set(fw.operands[i]) == {"q", "kv"}
    assert fw.skip_ops == {}
    bw = analyse(case["bw"])
    for i, ins in enumerate(case["bw"].instructions):
        if type(ins).__name__ == "AttnBackwardInstr":
            assert set(bw.operands[i]) == {"q", "kv", "out"}, "dQ partials are summed: they stay in slots"


def test_plans_that_exchange_blocks_are_left_alone():
    case = make_multi_case(n_nodes=2, n_devices_per_node=2, seqlens=[300, 150, 260], block_size=64, n_heads=8,
                           n_groups=2, head_dim=16, head_block=2)
    for plan in case["fw"] + case["bw"]:
        assert not analyse(plan).anything()


def test_a_slot_that_something_else_reads_is_still_filled():
    """The gathered q block of one row is also named as a source of a reduction op: its copy is made
    (the reduction reads the slot) although the attention kernel reads the local block itself; every
    other copy is still skipped."""
    case = make_case(**SINGLE_STAGE)
    plan = copy.deepcopy(case["fw"])
    memcpy, attn, red = plan.instructions
    q_slot = attn.q_block_table[0][0]
    out_like = BufferBlock(BufferType.BUFFER_Q, q_slot.index, q_slot.n_tokens)
    lse_like = red.ops[0].src_buffers[0][1]
    red.ops.append(ReductionOp([(out_like, lse_like)], red.ops[0].dst_buffer))
    found = analyse(plan)
    kept = {pos for pos, (src, dst) in enumerate(memcpy.src_dst_pairs)
            if (dst.buffer_type, dst.index) == (BufferType.BUFFER_Q, q_slot.index)}
    assert len(kept) == 1
    assert found.skip_pairs[0] == set(range(len(memcpy.src_dst_pairs))) - kept
    assert set(found.operands[1]) >= {"q", "kv"}


def _replay(plan, found):
    """Which local block each directly addressed operand stands for, against what the slot would hold."""
    slots = {}
    for idx, ins in enumerate(plan.instructions):
        if isinstance(ins, MemcpyInstr):
            for src, dst in ins.src_dst_pairs:
                slots[(dst.buffer_type, dst.index)] = (src.buffer_type, src.index)
        elif type(ins).__name__ in ("AttnInstr", "AttnBackwardInstr"):
            ops = found.operands.get(idx, {})
            if "q" in ops:
                for row, local in zip(ins.q_block_table, ops["q"]):
                    assert slots[(row[0].buffer_type, row[0].index)] == (BufferType.LOCAL_Q, local)
            if "kv" in ops:
                for row, locals_ in zip(ins.kv_block_table, ops["kv"]):
                    assert [slots[(b.buffer_type, b.index)] for b in row] == [(BufferType.LOCAL_KV, i) for i in locals_]
            if "out" in ops and type(ins).__name__ == "AttnBackwardInstr":
                for row, local in zip(ins.out_block_table, ops["out"]):
                    for slot_t, local_t in ((BufferType.BUFFER_OUT, BufferType.LOCAL_OUT), (BufferType.BUFFER_LSE, BufferType.LOCAL_LSE),
                                            (BufferType.BUFFER_dOUT, BufferType.LOCAL_dOUT)):
                        assert slots[(slot_t, row[0].index)] == (local_t, local)
            if "out" in ops and type(ins).__name__ == "AttnInstr":
                # the skipped single-source ops are exactly the scatters of these rows' slots to these local blocks
                moved = {}
                for j, positions in found.skip_ops.items():
                    red = plan.instructions[j]
                    if isinstance(red, AttnReductionInstr):
                        for pos in positions:
                            (src_out, _), = red.ops[pos].src_buffers
                            moved[src_out.index] = red.ops[pos].dst_buffer[0].index
                assert [moved[row[0].index] for row in ins.out_block_table] == ops["out"]


@pytest.mark.parametrize("cfg", [SINGLE_STAGE, THREE_PARTIALS, FOLDED], ids=["single_stage", "three_partials", "folded"])
def test_direct_operands_are_the_blocks_the_skipped_copies_would_have_moved(cfg):
    case = make_case(**cfg)
    for plan in (case["fw"], case["bw"]):
        _replay(plan, analyse(plan))
