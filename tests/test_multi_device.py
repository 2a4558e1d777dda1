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
