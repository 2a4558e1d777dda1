"""Grouping of a device assignment into pipeline stages (host side of the planner).

Mirrors ``dcp/core/pipeline.py:513-839`` (``generate_pipelines_n_stages``) and the natively
compiled routine it calls once per stage, ``dcp_cpp.greedy_selection_per_device``
(``csrc/pipeline_generator/pipeline_generator.cpp:19-323``).  The packer itself is the C++ entry
point ``dcp_greedy_stage_selection`` of ``libdcp_hip.so``; this module converts the reference's
sets and dicts of ``(node, rank)`` tuples to the dense tables it takes and back.  There is no
Python fallback: without the library the functions raise.

Where the reference's choice depends on the iteration order of a hash table (devices with equal
accumulated compute, holders with equal load, workloads of equal cost), the native packer takes
the first candidate in the order of ``sorted(devices)`` / the lower workload id.
"""

from __future__ import annotations

import ctypes
from collections import defaultdict
from typing import Dict, Iterable, List, Optional, Sequence, Set, Tuple

import numpy as np

from dcp_amd import _lib

Device = Tuple[int, int]

BLOCK_OTHER, BLOCK_OUT, BLOCK_LSE, BLOCK_DOUT = 0, 1, 2, 3
_KIND_OF_TYPE = {"OUT": BLOCK_OUT, "LSE": BLOCK_LSE, "dOUT": BLOCK_DOUT}
NOT_HELD = -(2**31)


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def _csr(lists: Sequence[Iterable[int]]):
    offsets = np.zeros(len(lists) + 1, dtype=np.int32)
    flat: List[int] = []
    for i, items in enumerate(lists):
        flat.extend(int(x) for x in items)
        offsets[i + 1] = len(flat)
    return offsets, np.asarray(flat if flat else [0], dtype=np.int32)


class StageProblem:
    """The tables of one planning problem that do not change from stage to stage, converted
    once: devices in sorted order, costs, block sizes and kinds, the two CSR maps."""

    def __init__(self, devices: Iterable[Device], workload_costs: Sequence[float], input_sizes: Sequence[float],
                 workload_input_map: Sequence[Sequence[int]], input_block_type_map: Sequence[str],
                 device_workload_map: Dict[Device, Sequence[int]]):
        self.devices: List[Device] = sorted(set(tuple(d) for d in devices))
        assert self.devices, "at least one device"
        self.index = {d: i for i, d in enumerate(self.devices)}
        unknown = [d for d in device_workload_map if tuple(d) not in self.index]
        assert not unknown, f"device_workload_map names devices that are not in `devices`: {unknown}"
        self.n_workloads = len(workload_costs)
        self.n_inputs = len(input_sizes)
        assert len(workload_input_map) == self.n_workloads and len(input_block_type_map) == self.n_inputs
        self.node = np.asarray([d[0] for d in self.devices], dtype=np.int32)
        self.costs = np.asarray(workload_costs, dtype=np.float32).reshape(-1)
        self.sizes = np.asarray(input_sizes, dtype=np.float32).reshape(-1)
        self.kind = np.asarray([_KIND_OF_TYPE.get(t, BLOCK_OTHER) for t in input_block_type_map], dtype=np.uint8)
        self.w_off, self.w_in = _csr(workload_input_map)
        self.d_off, self.d_w = _csr([device_workload_map.get(d, ()) for d in self.devices])

    def held_table(self, device_local_inputs_map: Dict[Device, Dict[int, int]]) -> np.ndarray:
        held = np.full((len(self.devices), max(self.n_inputs, 1)), NOT_HELD, dtype=np.int32)
        for d, inputs in device_local_inputs_map.items():
            assert tuple(d) in self.index, f"device_local_inputs_map names device {d}, which is not in `devices`"
            row = held[self.index[tuple(d)]]
            for input_id, stage in inputs.items():
                row[input_id] = stage
        return held

    def select(self, scheduled: np.ndarray, held: np.ndarray, target: np.ndarray, is_bw: bool, stage_id: int):
        """One call of the native packer.  ``held`` is updated in place.  Returns
        (unlocked_by [n_workloads], transfers as an [n, 3] array of (dst, input, src) device
        indices / block ids, cross-node load per device, same-node load per device)."""
        n_dev = len(self.devices)
        unlocked_by = np.empty(max(self.n_workloads, 1), dtype=np.int32)
        capacity = n_dev * max(self.n_inputs, 1)
        comm = np.empty((3, capacity), dtype=np.int32)
        n_comm = ctypes.c_int64(0)
        cross = np.zeros(n_dev, dtype=np.float32)
        intra = np.zeros(n_dev, dtype=np.float32)
        _lib.call(
            "dcp_greedy_stage_selection", n_dev, _ptr(self.node), self.n_workloads, _ptr(self.costs), _ptr(scheduled),
            self.n_inputs, _ptr(self.sizes), _ptr(self.kind), _ptr(self.w_off), _ptr(self.w_in), _ptr(self.d_off),
            _ptr(self.d_w), _ptr(held), _ptr(target), 1 if is_bw else 0, int(stage_id), _ptr(unlocked_by),
            _ptr(comm[0]), _ptr(comm[1]), _ptr(comm[2]), capacity, ctypes.byref(n_comm), _ptr(cross), _ptr(intra))
        return unlocked_by[: self.n_workloads], comm[:, : n_comm.value].T, cross, intra


def greedy_selection_per_device(
    devices: Set[Device],
    scheduled_workloads: Set[int],
    workload_costs: List[float],
    input_sizes: List[float],
    workload_input_map: List[List[int]],
    input_block_type_map: List[str],
    device_workload_map: Dict[Device, List[int]],
    device_local_inputs_map: Dict[Device, Dict[int, int]],
    target_comm_load_per_node: Dict[Device, float],
    is_bw: bool,
    stage_id: int,
    py_logger=None,
):
    """Same arguments and result as ``dcp_cpp.greedy_selection_per_device``
    (``csrc/interface.cpp:9-11``): returns (workloads unlocked per device: dict device -> set,
    transfers per destination device: dict device -> [(input id, source device)], the updated
    copy of ``device_local_inputs_map``).  A block nobody held before ``stage_id`` raises, as the
    reference's ``std::runtime_error("No device has input.")`` does (``AssertionError`` here)."""
    prob = StageProblem(devices, workload_costs, input_sizes, workload_input_map, input_block_type_map,
                        device_workload_map)
    scheduled = np.zeros(max(prob.n_workloads, 1), dtype=np.uint8)
    for w in scheduled_workloads:
        scheduled[w] = 1
    held = prob.held_table(device_local_inputs_map)
    target = np.asarray([target_comm_load_per_node[d] for d in prob.devices], dtype=np.float32)
    unlocked_by, comm, cross, intra = prob.select(scheduled, held, target, is_bw, stage_id)

    unlocked: Dict[Device, Set[int]] = {}
    for w, d in enumerate(unlocked_by):
        if d >= 0:
            unlocked.setdefault(prob.devices[d], set()).add(w)
    performed: Dict[Device, List[Tuple[int, Device]]] = {}
    for dst, input_id, src in comm:
        performed.setdefault(prob.devices[dst], []).append((int(input_id), prob.devices[src]))
    updated = {d: {} for d in device_local_inputs_map}
    for i, d in enumerate(prob.devices):
        ids = np.nonzero(held[i, : prob.n_inputs] != NOT_HELD)[0]
        if len(ids) or d in updated:
            updated[d] = {int(j): int(held[i, j]) for j in ids}
    if py_logger is not None:
        for i, d in enumerate(prob.devices):
            py_logger.debug(
                f"Current communication load for device ({d[0]}, {d[1]}): intra_node={float(intra[i]):f} (target: 0),"
                f" inter_node={float(cross[i]):f} (target: {float(target[i]):f})")
    return unlocked, performed, updated


def generate_pipelines_n_stages(
    n_stages: int,
    all_devices: Set[Device],
    workload_costs: List[float],
    workload_input_map: List[List[int]],
    input_to_meta_map: Dict[int, object],
    input_sizes: List[float],
    workload_to_device_map: Dict[int, Device],
    input_to_device_map: Dict[int, Device],
    is_bw: bool,
    logger=None,
    disable_two_phase_comm: bool = False,
):
    """Groups an assignment of workloads and data blocks to devices into ``n_stages`` pipeline
    stages (``dcp/core/pipeline.py:513-839``).  Returns three lists with one entry per stage
    (entry 0 = the workloads that need no transfer at all):

    * workloads per device: ``{device: workloads}``,
    * transfers per destination device: ``{device: [(input id, source device)]}``,
    * second-phase transfers: when several devices of one node need the same remote block in a
      stage, only the least loaded of them receives it from the remote node and forwards it to
      the others inside the node (``disable_two_phase_comm`` = the reference's
      ``DCP_DISABLE_TWO_PHASE_COMM``).

    ``input_to_meta_map[i].type`` is the block's type string ("Q", "KV", "OUT", "LSE", "dOUT", ...)."""
    devices = sorted(set(tuple(d) for d in all_devices))
    n_workloads, n_inputs = len(workload_costs), len(input_sizes)
    device_to_workload_map: Dict[Device, List[int]] = {d: [] for d in devices}
    for w, d in workload_to_device_map.items():
        device_to_workload_map[tuple(d)].append(w)
    device_to_local_inputs_map: Dict[Device, Dict[int, int]] = {d: {} for d in devices}
    for i, d in input_to_device_map.items():
        device_to_local_inputs_map[tuple(d)][i] = -1

    # The per-stage budget: the cross-node volume the assignment implies (a remote block is
    # fetched once per node: pipeline.py:551-580), spread evenly over devices and stages, +20 %.
    on_device = defaultdict(set)
    for i, d in input_to_device_map.items():
        on_device[tuple(d)].add(i)
    cross_by_source = defaultdict(float)  # summed per source first, as the reference does
    for w, d in workload_to_device_map.items():
        d = tuple(d)
        for i in workload_input_map[w]:
            if i in on_device[d]:
                continue
            src = tuple(input_to_device_map[i])
            if src[0] != d[0]:
                cross_by_source[src] += input_sizes[i]
                for other in devices:
                    if other[0] == d[0]:
                        on_device[other].add(i)
            on_device[d].add(i)
    total_cross = 0
    for volume in cross_by_source.values():
        total_cross += volume
    per_stage = (total_cross / len(devices) / n_stages) * 1.2

    types = [input_to_meta_map[i].type for i in range(n_inputs)]
    prob = StageProblem(devices, workload_costs, input_sizes, workload_input_map, types, device_to_workload_map)
    held = prob.held_table(device_to_local_inputs_map)
    scheduled = np.zeros(max(n_workloads, 1), dtype=np.uint8)

    def as_dicts(unlocked_by, comm):
        work: Dict[Device, Set[int]] = {}
        for w, d in enumerate(unlocked_by):
            if d >= 0:
                work.setdefault(devices[d], set()).add(w)
        sends: Dict[Device, List[Tuple[int, Device]]] = {}
        for dst, i, src in comm:
            sends.setdefault(devices[dst], []).append((int(i), devices[src]))
        return work, sends

    # stage 0: everything whose blocks are all where the workload runs (pipeline.py:612-643)
    first: Dict[Device, List[int]] = defaultdict(list)
    for w in range(n_workloads):
        d = tuple(workload_to_device_map[w])
        if all(tuple(input_to_device_map[i]) == d for i in workload_input_map[w]):
            first[d].append(w)
            scheduled[w] = 1
    workload_per_stage = [first]
    comm_per_stage: List[Dict[Device, List[Tuple[int, Device]]]] = [defaultdict(list)]

    for stage_id in range(n_stages):
        target = np.full(len(devices), per_stage, dtype=np.float32)
        unlocked_by, comm, _, _ = prob.select(scheduled, held, target, is_bw, stage_id)
        work, sends = as_dicts(unlocked_by, comm)
        scheduled[: n_workloads][unlocked_by >= 0] = 1
        if stage_id == n_stages - 1:
            # the last stage takes whatever is left, whatever it costs (pipeline.py:692-745)
            target = np.full(len(devices), np.inf, dtype=np.float32)
            unlocked_by, comm, _, _ = prob.select(scheduled, held, target, is_bw, stage_id)
            more_work, more_sends = as_dicts(unlocked_by, comm)
            scheduled[: n_workloads][unlocked_by >= 0] = 1
            for d, ws in more_work.items():
                work[d] = work.get(d, set()) | ws
            for d, c in more_sends.items():
                sends.setdefault(d, []).extend(c)
            assert scheduled[: n_workloads].all(), "workloads left unscheduled after the last stage"
        workload_per_stage.append(work)
        comm_per_stage.append(sends)

    if disable_two_phase_comm:
        return workload_per_stage, comm_per_stage, [defaultdict(list) for _ in comm_per_stage]

    # second phase (pipeline.py:760-834): a remote block wanted by several devices of a node
    first_phase = [defaultdict(list)]
    second_phase = [defaultdict(list)]
    for sends in comm_per_stage[1:]:
        recv_load = defaultdict(float)
        wanted_by = defaultdict(set)
        for dst, comms in sends.items():
            for i, src in comms:
                if src[0] != dst[0]:
                    recv_load[dst] += input_sizes[i]
                    wanted_by[(src, i, dst[0])].add(dst[1])
        drop = defaultdict(list)
        forward = defaultdict(list)
        for src, i, node in sorted(wanted_by, key=lambda k: k[1]):
            ranks = wanted_by[(src, i, node)]
            if len(ranks) > 1:
                receiver = min(sorted(ranks), key=lambda r: recv_load[(node, r)])
                for r in sorted(ranks):
                    if r != receiver:
                        drop[(node, r)].append((i, src))
                        forward[(node, r)].append((i, (node, receiver)))
        kept = defaultdict(list)
        for dst, comms in sends.items():
            kept[dst] = [c for c in comms if c not in drop[dst]]
        first_phase.append(kept)
        second_phase.append(forward)
    return workload_per_stage, first_phase, second_phase
