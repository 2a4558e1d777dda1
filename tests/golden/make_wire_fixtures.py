#!/usr/bin/env python3
"""Writes tests/golden/wire/: the byte strings the REFERENCE's own serializer
(dcp/core/instructions.py, dcp/core/serialization.py under /root/reference) produces for one
instruction of every type and for whole ExecutionPlans, next to a plain-data description of what
was serialized (wire_spec.py).  The reference holds no stored vectors for its wire format (its
tests/core/test_instructions.py only round-trips through its own codec), so nothing else pins
these bytes; this script is the one place that imports the reference, it runs in the build
container only, and only its outputs (data) are committed.

  instructions.json / <name>.bin   hand-written instructions, one per type (two for attention:
                                   one and two ranges; with and without a stream name)
  plan_hand.json / .bin            a hand-written plan holding all of them
  plan_causal_{fw,bw}.json / .bin  the forward and backward plan of a small causal case and
  plan_lambda_{fw,bw}.json / .bin  of a two-range (lambda) case, content taken from this
                                   package's single-device builder (tests/plan_cases.make_case)
  plan_staged_dev{0..3}_{fw,bw}    the plans of four devices on two nodes, staged by the stage
                                   packer, with CommLaunch / CommWait instructions and a second phase
  plans_list.bin                   serialize_list_of_execution_plans of the two causal plans

Usage: python tests/golden/make_wire_fixtures.py   (from the repository root)
"""

import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REFERENCE = "/root/reference"
sys.path.insert(0, REFERENCE)
sys.path.insert(0, ROOT)  # first: `tests` must be this repository's package, not the reference's

import dcp.core.instructions as ref  # noqa: E402  (the reference's serializer: the thing being recorded)

from tests.golden import wire_spec  # noqa: E402

OUT = os.path.join(HERE, "wire")

B = lambda t, i, n=256: [t, i, n]  # noqa: E731

HAND = {
    "memcpy": {"op": "MemcpyInstr", "src_dst_pairs": [[B("LocalQ", 0, 100), B("BufferQ", 5, 100)],
                                                      [B("LocalKV", 3), B("BufferKV", 1)],
                                                      [B("LocalLSE", 2, 1), B("BufferLSE", 70000, 1)]]},
    "comm_launch": {"op": "CommLaunchInstr", "key": "S1", "stream": None,
                    "comm_ops": [[0, [0, 1], B("BufferQ", 2)], [1, [1, 3], B("BufferKV", 7, 12)]]},
    "comm_launch_stream": {"op": "CommLaunchInstr", "key": "S2P2", "stream": "second_phase",
                           "comm_ops": [[0, [1, 0], B("LocalOut", 4, 33)], [0, [1, 0], B("LocalLSE", 4, 33)],
                                        [1, [0, 2], B("BufferdOut", 9, 256)]]},
    "comm_wait": {"op": "CommWaitInstr", "key": "S1", "stream": None},
    "comm_wait_stream": {"op": "CommWaitInstr", "key": "S2P2", "stream": "second_phase"},
    "barrier": {"op": "BarrierInstr"},
    "attn_one_range": {
        "op": "AttnInstr", "stage_id": 0, "seqlens_q": [4, 2], "seqlens_kv": [8, 4], "max_seqlen_q": 4, "max_seqlen_kv": 8,
        "attn_mask": [[0, 0, 0, 0, 1, 0], [5, 6, 7, 8, 3, 0]],
        "q_block_table": [[B("BufferQ", 0, 4)], [B("BufferQ", 3, 2)]],
        "kv_block_table": [[B("BufferKV", 1, 4), B("BufferKV", 0, 4)], [B("BufferKV", 2, 4)]],
        "out_block_table": [[B("BufferOut", 6, 4)], [B("BufferOut", 2, 2)]],
        "lse_block_table": [[B("BufferLSE", 6, 4)], [B("BufferLSE", 2, 2)]]},
    "attn_two_ranges": {
        "op": "AttnInstr", "stage_id": 2, "seqlens_q": [3], "seqlens_kv": [12], "max_seqlen_q": 3, "max_seqlen_kv": 12,
        "attn_mask": [[[0, 0, 0], [2, 2, 2]], [[6, 7, 0], [10, 12, 0]]],
        "q_block_table": [[B("BufferQ", 1, 3)]],
        "kv_block_table": [[B("BufferKV", 4, 4), B("BufferKV", 5, 4), B("BufferKV", 9, 4)]],
        "out_block_table": [[B("BufferOut", 0, 3)]],
        "lse_block_table": [[B("BufferLSE", 0, 3)]]},
    "attn_backward": {
        "op": "AttnBackwardInstr", "stage_id": 1, "seqlens_q": [4, 2], "seqlens_kv": [8, 4], "max_seqlen_q": 4, "max_seqlen_kv": 8,
        "attn_mask": [[[0, 0, 0, 0, 1, 0], [5, 6, 7, 8, 3, 0]], [[0, 0, 0, 0, 0, 0], [0, 0, 0, 0, 0, 0]]],
        "q_block_table": [[B("BufferQ", 0, 4)], [B("BufferQ", 3, 2)]],
        "kv_block_table": [[B("BufferKV", 1, 4), B("BufferKV", 0, 4)], [B("BufferKV", 2, 4)]],
        "out_block_table": [[B("BufferOut", 6, 4)], [B("BufferOut", 2, 2)]],
        "dq_block_table": [[B("BufferdQ", 1, 4)], [B("BufferdQ", 0, 2)]],
        "dkv_block_table": [[B("BufferdKV", 0, 4), B("BufferdKV", 1, 4)], [B("BufferdKV", 2, 4)]]},
    "reduction": {"op": "AttnReductionInstr", "output_is_unpadded": 1, "ops": [
        {"src": [[B("BufferOut", 6, 4), B("BufferLSE", 6, 4)]], "dst": [B("LocalOut", 0, 4), B("LocalLSE", 0, 4)]},
        {"src": [[B("BufferOut", 2, 2), B("BufferLSE", 2, 2)], [B("BufferOut", 0, 2), B("BufferLSE", 0, 2)],
                 [B("BufferOut", 7, 2), B("BufferLSE", 7, 2)]], "dst": [B("LocalOut", 1, 2), B("LocalLSE", 1, 2)]}]},
    "reduction_padded": {"op": "AttnReductionInstr", "output_is_unpadded": 0, "ops": [
        {"src": [[B("BufferOut", 1, 9), B("BufferLSE", 1, 9)], [B("BufferOut", 3, 9), B("BufferLSE", 3, 9)]],
         "dst": [B("BufferOut", 1, 9), B("BufferLSE", 1, 9)]}]},
    "sum": {"op": "SumInstr", "output_is_unpadded": 1, "ops": [
        {"src": [B("BufferdQ", 1, 4)], "dst": B("LocaldQ", 0, 4)},
        {"src": [B("BufferdKV", 0, 4), B("BufferdKV", 5, 4), B("BufferdKV", 2, 4)], "dst": B("LocaldKV", 2, 4)}]},
}

HAND_PLAN = {
    "instructions": [HAND[k] for k in ("memcpy", "comm_launch", "attn_one_range", "comm_wait", "comm_launch_stream",
                                       "attn_two_ranges", "comm_wait_stream", "barrier", "reduction_padded", "reduction",
                                       "attn_backward", "sum")],
    "n_nodes": 2, "n_devices_per_node": 4, "node_id": 1, "local_device_id": 2, "n_stages": 3,
    "local_cu_seqlens": [0, 4, 6, 262],
    "buffer_info": {
        "LocalQ": [3, 256, 256 * 4 * 128, 0, [262, 4, 128], [4, 128]],
        "LocalKV": [3, 256, 256 * 2 * 128, 0, [262, 2, 1, 128], [2, 1, 128]],
        "LocalLSE": [3, 256, 256 * 4, 2, [4, 262], [4]],
        "BufferQ": [6, 256, 256 * 4 * 128, 1, [6, 256, 4, 128], [4, 128]],
        "BufferLSE": [70001, 256, 256 * 4, 2, [4, 70001, 256], [4]],
    },
}


def write(name, blob, spec=None):
    with open(os.path.join(OUT, name + ".bin"), "wb") as f:
        f.write(blob)
    if spec is not None:
        with open(os.path.join(OUT, name + ".json"), "w") as f:
            json.dump(spec, f, separators=(",", ":"))
    print(f"{name}: {len(blob)} bytes")


def reference_bytes_of_plan(spec):
    plan = wire_spec.plan_from_spec(ref, spec, mask_as_planes=True)
    blob = plan.serialize()
    back, _ = ref.ExecutionPlan.deserialize(blob)
    assert back == plan and back.serialize() == blob
    return blob


def main():
    os.makedirs(OUT, exist_ok=True)
    for name, spec in HAND.items():
        instr = wire_spec.instr_from_spec(ref, spec, mask_as_planes=True)
        blob = instr.serialize()
        back, rest = ref.BlockInstrBase.deserialize(blob)
        assert rest == b"" and back == instr
        write(name, blob)
    with open(os.path.join(OUT, "instructions.json"), "w") as f:
        json.dump(HAND, f, separators=(",", ":"))
    write("plan_hand", reference_bytes_of_plan(HAND_PLAN), HAND_PLAN)

    # plans whose content comes from this package's builders; the bytes are the reference's
    from tests.test_wire_fixtures import BUILT_CASES, built_plans

    both = []
    for case_name in BUILT_CASES:
        for plan_name, plan in built_plans(case_name).items():
            spec = wire_spec.plan_to_spec(plan)
            blob = reference_bytes_of_plan(spec)
            write(plan_name, blob, spec)
            if case_name == "causal":
                both.append(wire_spec.plan_from_spec(ref, spec, mask_as_planes=True))
    write("plans_list", ref.serialize_list_of_execution_plans(both))


if __name__ == "__main__":
    main()
