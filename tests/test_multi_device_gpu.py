"""Several devices' plans through HIP executors that share the one GPU: blocks travel over a
LocalFabric (the sender's copy kernel writes into the receiver's staging buffer).  Checked
against the numpy oracle running the same plans and against whole-sequence attention."""

import numpy as np
import pytest
import torch

from tests.plan_cases import dense_truth, make_multi_case, run_multi_executor, run_multi_oracle

pytestmark = pytest.mark.gpu

CASES = {
    "two_devices_causal": dict(n_nodes=1, n_devices_per_node=2, seqlens=[200, 330], block_size=64, n_heads=4,
                               n_groups=4, head_dim=64, head_block=2),
    "four_devices_gqa": dict(n_nodes=2, n_devices_per_node=2, seqlens=[300, 150, 260], block_size=64, n_heads=8,
                             n_groups=2, head_dim=128, head_block=2),
    "three_devices_lambda": dict(n_nodes=1, n_devices_per_node=3, seqlens=[512, 200], block_size=64, n_heads=2,
                                 n_groups=2, head_dim=64, head_block=1, mask="lambda", mask_info=[16, 96]),
    "four_devices_fp16_big_blocks": dict(n_nodes=1, n_devices_per_node=4, seqlens=[2048, 1500], block_size=256,
                                         n_heads=8, n_groups=8, head_dim=128, head_block=4, dtype="fp16"),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_exchange_matches_oracle_and_dense_attention(name):
    case = make_multi_case(**CASES[name])
    print(f"multi-device case {name}", flush=True)
    (out, lse, dq, dkv), _ = run_multi_executor(case, backward=True)
    o_out, o_lse, o_dq, o_dkv = run_multi_oracle(case, backward=True)
    t_out, t_lse, t_dq, t_dkv = dense_truth(case, backward=True)
    for got, want in ((out, o_out), (out, torch.from_numpy(t_out))):
        assert (got.float() - want.float()).abs().max() <= 2e-2
    for want in (o_lse, torch.from_numpy(t_lse)):
        assert (lse.float() - want.float()).abs().max() <= 1e-3
    for got, want in ((dq, torch.from_numpy(t_dq)), (dkv, torch.from_numpy(t_dkv)), (dq, o_dq), (dkv, o_dkv)):
        err = (got.float() - want.float()).abs()
        assert (err <= 2e-2 * want.float().abs().clamp(min=1.0) + 4e-3 * want.float().abs().max()).all()


def test_exchange_can_be_repeated():
    """The second pass reuses every staging buffer and event slot of the first."""
    case = make_multi_case(**CASES["four_devices_gqa"])
    print("multi-device repeat", flush=True)
    once, _ = run_multi_executor(case, backward=True, repeats=1)
    thrice, _ = run_multi_executor(case, backward=True, repeats=3)
    for a, b in zip(once, thrice):
        assert torch.equal(a, b)


def test_moved_blocks_are_bit_exact():
    """What a receive puts into a slot is the sender's block, bit for bit: compare the received
    Q and KV slots of every device with the global tensors."""
    from dcp_amd.core.instructions import CommLaunchInstr

    case = make_multi_case(**CASES["four_devices_gqa"])
    print("multi-device bit-exact blocks", flush=True)
    _, exs = run_multi_executor(case, backward=False)
    ndpn, bs = case["n_devices_per_node"], 64
    off = np.concatenate(([0], np.cumsum(case["seqlens"])))
    checked = {"BufferQ": 0, "BufferKV": 0}
    for rank, (ex, plan) in enumerate(zip(exs, case["fw"])):
        launch = next(i for i in plan.instructions if isinstance(i, CommLaunchInstr) and i.key == "S0")
        for op in launch.comm_ops:
            if op.comm_type != 1:
                continue
            # the i-th receive from a peer is the peer's i-th send to this device
            peer = op.peer[0] * ndpn + op.peer[1]
            peer_launch = next(i for i in case["fw"][peer].instructions if isinstance(i, CommLaunchInstr) and i.key == "S0")
            peer_sends = [o for o in peer_launch.comm_ops if o.comm_type == 0 and tuple(o.peer) == divmod(rank, ndpn)]
            mine = [o for o in launch.comm_ops if o.comm_type == 1 and o.peer == op.peer]
            send = peer_sends[mine.index(op)]
            lay = case["layouts"][peer]
            kind = op.buffer_block.buffer_type
            if kind == "BufferKV":
                g, s, b, n = lay.kv_blocks[send.buffer_block.index]
                h = lay.head_block_size_kv
                want = case["kv"][off[s] + b * bs : off[s] + b * bs + n, :, g * h : (g + 1) * h]
            else:
                g, s, b, n = lay.q_blocks[send.buffer_block.index]
                h = lay.head_block_size
                want = case["q"][off[s] + b * bs : off[s] + b * bs + n, g * h : (g + 1) * h]
            got = ex.buffers[kind][op.buffer_block.index, :n].cpu()
            assert torch.equal(got, want)
            checked[kind] += 1
    assert checked["BufferQ"] > 0 and checked["BufferKV"] > 0


def test_comm_without_fabric_raises():
    from dcp_amd.runtime.flash_attention.executor import get_executor

    case = make_multi_case(**CASES["two_devices_causal"])
    ex = get_executor(case["head_block"], case["head_dim"], None, fw_exec_plan=case["fw"][0], bw_exec_plan=case["bw"][0])
    with pytest.raises(NotImplementedError, match="fabric"):
        ex.prepare(forward=True)
