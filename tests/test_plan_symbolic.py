"""Plans checked for structure alone by a symbolic run (tests/symbolic.py), the way the
reference checks its compiler's output with a DummyExecutor (tests/core/test_compiler.py:137-765):
single-device plans (one or several partials per row, folded or merged at the end) and plans for
several devices, unstaged and staged by the stage packer."""

import pytest
import torch

from dcp_amd.core.instructions import BufferBlock, CommLaunchInstr, CommOp
from tests.plan_cases import make_case, make_multi_case
from tests.symbolic import run_symbolic

SINGLE = {
    "causal_one_partial": dict(seqlens=[200, 330], block_size=64, n_heads=4, n_groups=4, head_dim=16, head_block=2),
    "gqa_three_partials": dict(seqlens=[500, 130], block_size=64, n_heads=8, n_groups=2, head_dim=16, head_block=2,
                               n_kv_groups=3),
    "lambda_folded": dict(seqlens=[700], block_size=64, n_heads=2, n_groups=2, head_dim=16, head_block=1, mask="lambda",
                          mask_info=[16, 96], n_kv_groups=2, kv_split="contiguous", fold=True),
}
MULTI = {
    "unstaged_four_devices": dict(n_nodes=2, n_devices_per_node=2, seqlens=[300, 150, 260], block_size=64, n_heads=8,
                                  n_groups=2, head_dim=16, head_block=2),
    "staged_two_phase": dict(n_nodes=2, n_devices_per_node=3, seqlens=[640, 500], block_size=64, n_heads=2, n_groups=2,
                             head_dim=16, head_block=1, mask="lambda", mask_info=[16, 96], n_stages=2),
    "staged_four_stages": dict(n_nodes=2, n_devices_per_node=4, seqlens=[1024], block_size=64, n_heads=2, n_groups=2,
                               head_dim=16, head_block=2, n_stages=4),
}


def _q_per_kv(cfg):
    group = cfg["n_heads"] // cfg["n_groups"]
    hkv = 1 if group > 1 else cfg["head_block"]
    return (cfg["n_heads"] // cfg["head_block"]) // (cfg["n_groups"] // hkv)


@pytest.mark.parametrize("name", sorted(SINGLE))
def test_single_device_plans(name):
    cfg = SINGLE[name]
    case = make_case(**cfg)
    for plan, backward in ((case["fw"], False), (case["bw"], True)):
        run_symbolic([plan], [case["layout"]], 1, backward, case["mask"], _q_per_kv(cfg))


@pytest.mark.parametrize("name", sorted(MULTI))
def test_multi_device_plans(name):
    cfg = MULTI[name]
    case = make_multi_case(**cfg)
    for plans, backward in ((case["fw"], False), (case["bw"], True)):
        run_symbolic(plans, case["layouts"], case["n_devices_per_node"], backward, case["mask"], _q_per_kv(cfg))


def test_staged_plans_recycle_slots_and_no_live_block_is_overwritten():
    """The staged builder returns the slots of input blocks after the last stage that needs them and
    of partials once they are folded (the reference's BlockManager with live ranges): the symbolic run,
    which follows every slot's contents through time, passes, it sees slots change hands, and the
    buffers are smaller than one slot per block ever held."""
    cfg = MULTI["staged_four_stages"]
    case = make_multi_case(**cfg)
    for plans, backward in ((case["fw"], False), (case["bw"], True)):
        devs = run_symbolic(plans, case["layouts"], case["n_devices_per_node"], backward, case["mask"], _q_per_kv(cfg))
        assert sum(d.overwritten for d in devs) > 0, "no slot was recycled"
        saved = 0
        for plan in plans:
            n_kv_writes = sum(1 for i in plan.instructions if isinstance(i, CommLaunchInstr)
                              for op in i.comm_ops if op.comm_type == 1 and op.buffer_block.buffer_type == "BufferKV")
            n_kv_writes += sum(1 for i in plan.instructions if type(i).__name__ == "MemcpyInstr"
                               for _, dst in i.src_dst_pairs if dst.buffer_type == "BufferKV")
            saved += n_kv_writes - plan.buffer_info["BufferKV"].n_blocks
        assert saved > 0, "every kv block ever held still has a slot of its own"


def test_the_checker_notices_a_slot_recycled_too_early():
    """A receive redirected into a slot whose block a later stage still reads is reported as such."""
    cfg = MULTI["staged_four_stages"]
    case = make_multi_case(**cfg)
    plans = case["fw"]
    # the first kv block some device receives goes, instead of to its slot, to the slot of a block
    # that the device gathered at the start and reads in a later stage
    for plan in plans:
        attn_stages = [i for i in plan.instructions if type(i).__name__ == "AttnInstr"]
        launch = next((i for i in plan.instructions if isinstance(i, CommLaunchInstr)
                       and any(op.comm_type == 1 and op.buffer_block.buffer_type == "BufferKV" for op in i.comm_ops)), None)
        if launch is None or len(attn_stages) < 2:
            continue
        k = next(n for n, op in enumerate(launch.comm_ops) if op.comm_type == 1 and op.buffer_block.buffer_type == "BufferKV")
        victim = attn_stages[0].kv_block_table[0][0]  # read by the stage that runs while this transfer is in flight
        op = launch.comm_ops[k]
        if victim.n_tokens != op.buffer_block.n_tokens or victim.index == op.buffer_block.index:
            continue
        launch.comm_ops[k] = CommOp(op.comm_type, op.peer, BufferBlock("BufferKV", victim.index, victim.n_tokens))
        # the stage after the wait reads the victim's slot again only if it is still live there; make it so
        attn_stages[1].kv_block_table[0][0] = victim
        break
    else:
        pytest.skip("no device of this case both receives kv blocks and runs two stages")
    with pytest.raises(AssertionError):
        run_symbolic(plans, case["layouts"], case["n_devices_per_node"], False, case["mask"], _q_per_kv(cfg))


def test_the_checker_notices_an_input_slot_given_away_before_its_block_was_read():
    """A receive redirected into a slot whose block (received or gathered earlier) no stage has read
    yet -- its first reader runs after the redirected receive completes: the block is replaced before
    anything has read it, and the checker says so at the write.  (What the later stage then finds may
    look plausible, so the read itself need not fail.)"""
    cfg = MULTI["staged_four_stages"]
    case = make_multi_case(**cfg)
    plans = case["fw"]

    def redirect_one(plan):
        ins = plan.instructions
        wait_at = {i.key: j for j, i in enumerate(ins) if type(i).__name__ == "CommWaitInstr"}
        writes, reads = {}, {}  # slot -> [(time, n_tokens)], slot -> [time]
        for j, i in enumerate(ins):
            if type(i).__name__ == "MemcpyInstr":
                for _, dst in i.src_dst_pairs:
                    writes.setdefault((dst.buffer_type, dst.index), []).append((j, dst.n_tokens))
            elif isinstance(i, CommLaunchInstr):
                for op in i.comm_ops:
                    if op.comm_type == 1:
                        blk = op.buffer_block
                        writes.setdefault((blk.buffer_type, blk.index), []).append((wait_at[i.key], blk.n_tokens))
            elif type(i).__name__ == "AttnInstr":
                for row in i.q_block_table:
                    reads.setdefault((row[0].buffer_type, row[0].index), []).append(j)
                for row in i.kv_block_table:
                    for blk in row:
                        reads.setdefault((blk.buffer_type, blk.index), []).append(j)
        for launch in (i for i in ins if isinstance(i, CommLaunchInstr)):
            w2 = wait_at[launch.key]
            for k, op in enumerate(launch.comm_ops):
                blk = op.buffer_block
                if op.comm_type != 1 or blk.buffer_type not in ("BufferQ", "BufferKV"):
                    continue
                for slot, ws in writes.items():
                    if slot[0] != blk.buffer_type or slot[1] == blk.index:
                        continue
                    before = [(t, n) for t, n in ws if t < w2]
                    if not before or before[-1][1] != blk.n_tokens:
                        continue
                    w1 = before[-1][0]
                    rs = reads.get(slot, [])
                    if any(w1 < r < w2 for r in rs) or not any(r > w2 for r in rs):
                        continue  # already read, or nobody waits for it
                    launch.comm_ops[k] = CommOp(op.comm_type, op.peer, BufferBlock(slot[0], slot[1], blk.n_tokens))
                    return True
        return False

    if not any(redirect_one(plan) for plan in plans):
        pytest.skip("no device of this case holds an unread input block while a receive completes")
    with pytest.raises(AssertionError, match="before any instruction read it"):
        run_symbolic(plans, case["layouts"], case["n_devices_per_node"], False, case["mask"], _q_per_kv(cfg))


def test_the_checker_notices_a_wrong_plan():
    """A kv block swapped in an attention row, a receive into the wrong kind of slot and a dropped
    work unit must each fail."""
    cfg = MULTI["unstaged_four_devices"]
    args = lambda case: (case["layouts"], case["n_devices_per_node"], False, case["mask"], _q_per_kv(cfg))
    case = make_multi_case(**cfg)
    attn = next(i for i in case["fw"][0].instructions if type(i).__name__ == "AttnInstr")
    row = next(r for r in attn.kv_block_table if len(r) >= 2)
    row[0], row[1] = row[1], row[0]
    with pytest.raises(AssertionError, match="sequence order"):
        run_symbolic(case["fw"], *args(case))

    case = make_multi_case(**cfg)
    launch = next(i for i in case["fw"][1].instructions if isinstance(i, CommLaunchInstr) and i.key == "S0")
    k = next(n for n, op in enumerate(launch.comm_ops) if op.comm_type == 1 and op.buffer_block.buffer_type == "BufferKV")
    op = launch.comm_ops[k]
    launch.comm_ops[k] = CommOp(op.comm_type, op.peer, BufferBlock("BufferQ", 0, op.buffer_block.n_tokens))
    with pytest.raises(AssertionError):
        run_symbolic(case["fw"], *args(case))

    case = make_multi_case(**cfg)
    attn = next(i for i in case["fw"][2].instructions if type(i).__name__ == "AttnInstr")
    b = next(n for n, r in enumerate(attn.kv_block_table) if len(r) >= 2)
    attn.kv_block_table[b].pop()
    attn.seqlens_kv[b] -= 64
    with pytest.raises(AssertionError):
        run_symbolic(case["fw"], *args(case))
