"""Block exchange between the executors of several devices that share one GPU and one process.

The reference moves blocks between devices in three passes per direction: a fused copy packs the
blocks to send into one buffer per dtype, ``dist.all_to_all_single`` moves the buffers, and a
second fused copy unpacks what arrived (``dcp/runtime/flash_attention/executor.py:1583-2074``).
Here the sender's one copy kernel writes its blocks straight into the *receiver's* staging
buffer (on MI355X peers map each other's memory over xGMI; in this build every "device" is an
executor on the same GPU, so the peer's buffer is simply another allocation) and signals with a
stream event; the receiver waits for the events of the peers it expects and unpacks.  Two
passes instead of three, and no collective call.  The staging buffer keeps the reference's
rule that received blocks reach their slots at the ``CommWaitInstr``, not earlier, so slot reuse
planned by the scheduler stays valid.

``LocalFabric`` is the registry the executors meet in: staging buffers by (receiver, key,
dtype), "posted" events by (sender, receiver, key) and "consumed" events by (receiver, key) that
keep a sender of the next iteration from overwriting a staging buffer still being unpacked.
``execute_together`` runs the plans of all devices in turns on the one GPU.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch

from dcp_amd.core.instructions import BarrierInstr, CommWaitInstr


class LocalFabric:
    def __init__(self, n_nodes: int, n_devices_per_node: int):
        self.n_nodes = n_nodes
        self.n_devices_per_node = n_devices_per_node
        self.n_ranks = n_nodes * n_devices_per_node
        # (receiver, key, dtype) -> (staging tensor, {sender: (element offset, [block numels])})
        self._staging: Dict[Tuple[int, str, torch.dtype], Tuple[torch.Tensor, Dict[int, Tuple[int, List[int]]]]] = {}
        self._posted: Dict[Tuple[int, int, str], torch.cuda.Event] = {}
        self._consumed: Dict[Tuple[int, str], torch.cuda.Event] = {}
        self._barrier_arrivals = [0] * self.n_ranks
        self.epoch = 0  # changes whenever a staging buffer is (re)registered or dropped

    # -- prepare time ----------------------------------------------------------------------
    def register_staging(self, receiver: int, key: str, dtype: torch.dtype, staging: torch.Tensor,
                         segments: Dict[int, Tuple[int, List[int]]]) -> None:
        self._staging[(receiver, key, dtype)] = (staging, segments)
        self.epoch += 1

    def staging_segment(self, receiver: int, key: str, dtype: torch.dtype, sender: int):
        """``(staging tensor, element offset, block numels)`` of what ``receiver`` expects from
        ``sender`` under ``key``; raises if the receiver's plan has no such receives."""
        entry = self._staging.get((receiver, key, dtype))
        if entry is None or sender not in entry[1]:
            raise RuntimeError(
                f"rank {sender} sends {dtype} blocks to rank {receiver} under key {key!r}, but rank "
                f"{receiver} has prepared no matching receives (prepare every device before executing)"
            )
        offset, numels = entry[1][sender]
        return entry[0], offset, numels

    def forget(self, receiver: int) -> None:
        """Drop what ``receiver`` registered (its plan is being prepared again)."""
        for k in [k for k in self._staging if k[0] == receiver]:
            del self._staging[k]
        self.epoch += 1

    # -- execute time ----------------------------------------------------------------------
    def post(self, sender: int, receiver: int, key: str, event: torch.cuda.Event) -> None:
        self._posted[(sender, receiver, key)] = event

    def posted(self, sender: int, receiver: int, key: str) -> Optional[torch.cuda.Event]:
        return self._posted.get((sender, receiver, key))

    def take(self, sender: int, receiver: int, key: str) -> torch.cuda.Event:
        return self._posted.pop((sender, receiver, key))

    def consumed(self, receiver: int, key: str) -> Optional[torch.cuda.Event]:
        return self._consumed.get((receiver, key))

    def set_consumed(self, receiver: int, key: str, event: torch.cuda.Event) -> None:
        self._consumed[(receiver, key)] = event

    def barrier_arrive(self, rank: int) -> int:
        self._barrier_arrivals[rank] += 1
        return self._barrier_arrivals[rank]

    def barrier_passed(self, generation: int) -> bool:
        return min(self._barrier_arrivals) >= generation


def execute_together(executors: Sequence, forward: bool = True) -> None:
    """Run the current mode's plan of every executor (``executors[rank]``, all on one
    ``LocalFabric``) to its end.  Each device runs until it reaches a wait whose peers have not
    launched yet (or a barrier not everybody has reached), then the next device takes over; the
    kernels of different devices overlap on the GPU as far as their streams allow."""
    plans = [ex.fw_exec_plan if forward else ex.bw_exec_plan for ex in executors]
    for ex, plan in zip(executors, plans):
        ex.begin(plan)
    cursor = [0] * len(executors)
    while any(c < len(p.instructions) for c, p in zip(cursor, plans)):
        progressed = False
        for rank, (ex, plan) in enumerate(zip(executors, plans)):
            while cursor[rank] < len(plan.instructions):
                instr = plan.instructions[cursor[rank]]
                if isinstance(instr, CommWaitInstr) and not ex.comm_ready(instr.key):
                    break
                if isinstance(instr, BarrierInstr) and not ex.barrier_ready(cursor[rank]):
                    break
                ex.step(cursor[rank])
                cursor[rank] += 1
                progressed = True
        if not progressed:
            raise RuntimeError("the devices' plans wait for each other: no instruction can run")
    for ex in executors:
        ex.finish()
