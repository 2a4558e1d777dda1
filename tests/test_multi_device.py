"""Several devices' plans with block exchange, on the CPU: the builder's plans run on the numpy
oracle (whose CommLaunchInstr / CommWaitInstr follow the reference's pack, all-to-all, unpack of
dcp/runtime/flash_attention/executor.py:1583-2074) must reproduce whole-sequence attention, and
survive the wire format."""

import numpy as np
import pytest
import torch

from dcp_amd.core.instructions import CommLaunchInstr, CommWaitInstr, ExecutionPlan
from tests.plan_cases import dense_truth, make_multi_case, run_multi_oracle

CASES = {
    "two_devices_causal": dict(n_nodes=1, n_devices_per_node=2, seqlens=[200, 330], block_size=64, n_heads=4,
                               n_groups=4, head_dim=16, head_block=2),
    "four_devices_gqa": dict(n_nodes=2, n_devices_per_node=2, seqlens=[300, 150, 260], block_size=64, n_heads=8,
                             n_groups=2, head_dim=16, head_block=2),
    "three_devices_lambda": dict(n_nodes=1, n_devices_per_node=3, seqlens=[512, 200], block_size=64, n_heads=2,
                                 n_groups=2, head_dim=16, head_block=1, mask="lambda", mask_info=[16, 96]),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_plans_with_exchange_reproduce_dense_attention(name):
    case = make_multi_case(**CASES[name])
    n_comm = sum(isinstance(i, CommLaunchInstr) for p in case["fw"] + case["bw"] for i in p.instructions)
    assert n_comm >= 2 * len(case["fw"]), "the case is meant to exchange inputs and results in both passes"
    out, lse, dq, dkv = run_multi_oracle(case, backward=True)
    t_out, t_lse, t_dq, t_dkv = dense_truth(case, backward=True)
    # the oracle computes in fp64 and rounds where a kernel stores: partial outputs and
    # gradients pass through one or two bf16 roundings before they are merged
    assert np.abs(out.numpy() - t_out).max() < 3e-2
    assert np.abs(lse.numpy() - t_lse).max() < 1e-5
    assert np.abs(dq.numpy() - t_dq).max() < 8e-2
    assert np.abs(dkv.numpy() - t_dkv).max() < 8e-2


def test_every_send_has_its_receive():
    case = make_multi_case(**CASES["four_devices_gqa"])
    ndpn = case["n_devices_per_node"]
    for plans in (case["fw"], case["bw"]):
        sends, recvs = {}, {}
        for rank, plan in enumerate(plans):
            assert (plan.node_id, plan.local_device_id) == divmod(rank, ndpn)
            keys = [i.key for i in plan.instructions if isinstance(i, CommLaunchInstr)]
            assert keys == [i.key for i in plan.instructions if isinstance(i, CommWaitInstr)]
            for instr in plan.instructions:
                if not isinstance(instr, CommLaunchInstr):
                    continue
                for op in instr.comm_ops:
                    peer = op.peer[0] * ndpn + op.peer[1]
                    assert peer != rank
                    side = sends if op.comm_type == 0 else recvs
                    pair = (rank, peer) if op.comm_type == 0 else (peer, rank)
                    side.setdefault((instr.key, pair), []).append(op.buffer_block.n_tokens)
        assert sends == recvs and sends


def test_plans_with_exchange_survive_the_wire_format():
    case = make_multi_case(**CASES["two_devices_causal"])
    for plan in case["fw"] + case["bw"]:
        restored, rest = ExecutionPlan.deserialize(plan.serialize())
        assert restored == plan and rest == b""


# ---------------------------------------------------------------------------
# the fabric's host logic, with stand-in executors (no GPU)
# ---------------------------------------------------------------------------


class _StubExecutor:
    """Has the stepping interface of AttentionExecutor; 'launch' posts a token to the fabric,
    'wait' needs the tokens of the peers it names."""

    def __init__(self, fabric, rank, instrs, recv_from):
        from dcp_amd.core.instructions import ExecutionPlan

        self.fabric, self.rank, self.recv_from, self.log = fabric, rank, recv_from, []
        self.fw_exec_plan = self.bw_exec_plan = ExecutionPlan(instrs, 1, fabric.n_ranks, 0, rank, 1, [0], {})
        self._arrived = {}

    def begin(self, plan):
        self.plan = plan

    def finish(self):
        self.log.append("finish")

    def comm_ready(self, key):
        return all(self.fabric.posted(p, self.rank, key) is not None for p in self.recv_from.get(key, []))

    def barrier_ready(self, index):
        if index not in self._arrived:
            self._arrived[index] = self.fabric.barrier_arrive(self.rank)
        return self.fabric.barrier_passed(self._arrived[index])

    def step(self, index):
        instr = self.plan.instructions[index]
        self.log.append(type(instr).__name__ + ":" + getattr(instr, "key", ""))
        if isinstance(instr, CommLaunchInstr):
            for peer in range(self.fabric.n_ranks):
                if peer != self.rank:
                    self.fabric.post(self.rank, peer, instr.key, object())
        elif isinstance(instr, CommWaitInstr):
            for p in self.recv_from.get(instr.key, []):
                self.fabric.take(p, self.rank, instr.key)


def test_execute_together_interleaves_devices_and_detects_cycles():
    from dcp_amd.core.instructions import BarrierInstr
    from dcp_amd.runtime.flash_attention.fabric import LocalFabric, execute_together

    fabric = LocalFabric(1, 2)
    # device 0 waits for device 1 before it launches anything device 1 could wait for, and
    # device 1 launches first: runs through
    a = _StubExecutor(fabric, 0, [CommWaitInstr("A"), CommLaunchInstr("B", []), BarrierInstr()], {"A": [1]})
    b = _StubExecutor(fabric, 1, [CommLaunchInstr("A", []), CommWaitInstr("B"), BarrierInstr()], {"B": [0]})
    execute_together([a, b])
    assert a.log == ["CommWaitInstr:A", "CommLaunchInstr:B", "BarrierInstr:", "finish"]
    assert b.log == ["CommLaunchInstr:A", "CommWaitInstr:B", "BarrierInstr:", "finish"]
    # both wait first: nobody can run
    fabric = LocalFabric(1, 2)
    a = _StubExecutor(fabric, 0, [CommWaitInstr("A"), CommLaunchInstr("B", [])], {"A": [1]})
    b = _StubExecutor(fabric, 1, [CommWaitInstr("B"), CommLaunchInstr("A", [])], {"B": [0]})
    with pytest.raises(RuntimeError, match="wait for each other"):
        execute_together([a, b])
    # a barrier one device never reaches
    fabric = LocalFabric(1, 2)
    a = _StubExecutor(fabric, 0, [BarrierInstr()], {})
    b = _StubExecutor(fabric, 1, [], {})
    with pytest.raises(RuntimeError, match="wait for each other"):
        execute_together([a, b])


def test_fabric_staging_registry():
    from dcp_amd.runtime.flash_attention.fabric import LocalFabric

    fabric = LocalFabric(2, 2)
    assert fabric.n_ranks == 4
    staging = object()
    fabric.register_staging(3, "S0", torch.bfloat16, staging, {1: (0, [8, 8]), 2: (16, [4])})
    assert fabric.staging_segment(3, "S0", torch.bfloat16, 2) == (staging, 16, [4])
    with pytest.raises(RuntimeError, match="no matching receives"):
        fabric.staging_segment(3, "S0", torch.bfloat16, 0)
    with pytest.raises(RuntimeError, match="no matching receives"):
        fabric.staging_segment(3, "S0", torch.float32, 1)
    fabric.forget(3)
    with pytest.raises(RuntimeError, match="no matching receives"):
        fabric.staging_segment(3, "S0", torch.bfloat16, 1)


def _random_multi_config(rng, head_dims=(16,)):
    n_dev = int(rng.integers(2, 6))
    n_nodes = 2 if n_dev % 2 == 0 and rng.random() < 0.5 else 1
    block_size = 64
    n_seq = int(rng.integers(1, 4))
    seqlens = [int(rng.integers(block_size + 1, 6 * block_size)) for _ in range(n_seq)]
    n_groups = int(rng.choice([1, 2, 4]))
    group = int(rng.choice([1, 2, 4]))
    n_heads = n_groups * group
    head_block = int(rng.choice([h for h in (1, 2, 4) if (group % h == 0 if group > 1 else n_heads % h == 0)]))
    mask = str(rng.choice(["causal", "lambda"]))
    cfg = dict(n_nodes=n_nodes, n_devices_per_node=n_dev // n_nodes, seqlens=seqlens, block_size=block_size,
               n_heads=n_heads, n_groups=n_groups, head_dim=int(rng.choice(head_dims)), head_block=head_block, mask=mask)
    if mask == "lambda":
        cfg["mask_info"] = [int(rng.integers(1, 40)), int(rng.integers(40, 200))]
    return cfg


@pytest.mark.parametrize("seed", range(8))
def test_random_placements_reproduce_dense_attention(seed):
    cfg = _random_multi_config(np.random.default_rng(1000 + seed))
    case = make_multi_case(seed=seed, **cfg)
    out, lse, dq, dkv = run_multi_oracle(case, backward=True)
    t_out, t_lse, t_dq, t_dkv = dense_truth(case, backward=True)
    assert np.abs(out.numpy() - t_out).max() < 3e-2, cfg
    assert np.abs(lse.numpy() - t_lse).max() < 1e-5, cfg
    for got, want in ((dq.numpy(), t_dq), (dkv.numpy(), t_dkv)):
        assert (np.abs(got - want) <= 4e-2 * np.maximum(1.0, np.abs(want)) + 1e-2 * np.abs(want).max()).all(), cfg


# ---------------------------------------------------------------------------
# stages laid out by the stage packer
# ---------------------------------------------------------------------------

STAGED = {
    "two_nodes_of_three_lambda": dict(n_nodes=2, n_devices_per_node=3, seqlens=[640, 500], block_size=64, n_heads=2,
                                      n_groups=2, head_dim=16, head_block=1, mask="lambda", mask_info=[16, 96], n_stages=2),
    "two_nodes_of_two_gqa": dict(n_nodes=2, n_devices_per_node=2, seqlens=[900, 300], block_size=64, n_heads=4,
                                 n_groups=1, head_dim=16, head_block=2, n_stages=2),
    "two_nodes_of_four_four_stages": dict(n_nodes=2, n_devices_per_node=4, seqlens=[1024], block_size=64, n_heads=2,
                                          n_groups=2, head_dim=16, head_block=2, n_stages=4),
    "one_node_three_stages": dict(n_nodes=1, n_devices_per_node=3, seqlens=[300, 150, 260], block_size=64, n_heads=8,
                                  n_groups=2, head_dim=16, head_block=2, n_stages=3),
    "single_phase_only": dict(n_nodes=2, n_devices_per_node=3, seqlens=[640, 500], block_size=64, n_heads=2,
                              n_groups=2, head_dim=16, head_block=1, n_stages=2, disable_two_phase_comm=True),
}


def _comm_keys(plans):
    keys = {}
    for p in plans:
        for i in p.instructions:
            if isinstance(i, (CommLaunchInstr, CommWaitInstr)):
                k = (type(i).__name__, i.key, i.stream)
                keys[k] = keys.get(k, 0) + 1
    return keys


@pytest.mark.parametrize("name", sorted(STAGED))
def test_staged_plans_reproduce_dense_attention(name):
    case = make_multi_case(**STAGED[name])
    out, lse, dq, dkv = run_multi_oracle(case, backward=True)
    t_out, t_lse, t_dq, t_dkv = dense_truth(case, backward=True)
    assert np.abs(out.numpy() - t_out).max() < 3e-2
    assert np.abs(lse.numpy() - t_lse).max() < 1e-5
    for got, want in ((dq.numpy(), t_dq), (dkv.numpy(), t_dkv)):
        assert (np.abs(got - want) <= 4e-2 * np.maximum(1.0, np.abs(want)) + 1e-2 * np.abs(want).max()).all()


def test_staged_plans_have_the_references_instruction_structure():
    """Stage k+1's transfers are launched before stage k's attention and waited for after it; a
    relay waits for the first phase on the second-phase stream and forwards from there
    (dcp/core/scheduler.py:894-1049)."""
    from dcp_amd.core.instructions import AttnInstr

    case = make_multi_case(**STAGED["two_nodes_of_three_lambda"])
    keys = _comm_keys(case["fw"])
    assert keys[("CommLaunchInstr", "S1P2", "second_phase")] > 0 and keys[("CommWaitInstr", "S1", "second_phase")] > 0
    assert not any(k[0] == "CommLaunchInstr" and k[1].endswith("P2") and k[2] is None for k in keys)
    for plan in case["fw"]:
        names = [(type(i).__name__, getattr(i, "key", getattr(i, "stage_id", None))) for i in plan.instructions]
        for stage in (1, 2):
            launch = names.index(("CommLaunchInstr", f"S{stage}")) if ("CommLaunchInstr", f"S{stage}") in names else None
            attn_before = names.index(("AttnInstr", stage - 1)) if ("AttnInstr", stage - 1) in names else None
            attn_after = names.index(("AttnInstr", stage)) if ("AttnInstr", stage) in names else None
            waits = [n for n, x in enumerate(names) if x[0] == "CommWaitInstr" and x[1] in (f"S{stage}", f"S{stage}P2")]
            if launch is not None and attn_before is not None:
                assert launch < attn_before
            if attn_after is not None and waits:
                assert max(waits) < attn_after
        assert sum(isinstance(i, AttnInstr) for i in plan.instructions) <= 3
    # without the second phase nothing runs on a side stream
    single = _comm_keys(make_multi_case(**STAGED["single_phase_only"])["fw"])
    assert all(k[2] is None for k in single)
