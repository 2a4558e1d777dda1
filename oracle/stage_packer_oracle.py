"""CPU restatement of the reference's stage packer.  TEST INFRASTRUCTURE ONLY: nothing under
``dcp_amd/`` may import this module; tests compare the native packer
(``dcp_greedy_stage_selection``) and the reference's own C++ (built into ``oracle/_ref`` where
the reference sources are present) against it.

``greedy_selection_per_device`` follows csrc/pipeline_generator/pipeline_generator.cpp:19-323
statement by statement, with Python dicts in place of the C++ hash maps.  The reference walks
``std::unordered_set`` / ``std::unordered_map`` objects wherever it has to pick among equals, so
its choice on a tie is whatever order the hash table happens to have.  This restatement makes
every such walk explicit and ordered:

* devices are visited in the order of the ``devices`` argument (a list here);
* a block's holders are visited in the same device order, ``min`` keeps the first minimum;
* pending workloads are sorted by (-cost, workload id).

Pinned by ``tests/test_stage_packer.py``: against the reference's C++ on inputs without ties
(distinct costs, one eligible holder per block or distinct loads, a single device with pending
work), against brute-force properties (every unlocked workload's blocks are held afterwards, no
sender exceeds its cross-node budget, out/lse/dout travel together, sources held the block before
the stage), and against hand-computed small cases.  On inputs WITH ties the reference's own
result is unspecified (hash order); there parity is by the properties only.
"""

from __future__ import annotations

import numpy as np

F32 = np.float32


def greedy_selection_per_device(devices, scheduled_workloads, workload_costs, input_sizes, workload_input_map,
                                input_block_type_map, device_workload_map, device_local_inputs_map,
                                target_comm_load_per_node, is_bw, stage_id):
    """Returns (unlocked workloads per device: dict device -> set, transfers per destination
    device: dict device -> [(input id, source device)], updated local inputs: dict device ->
    {input id: stage}) -- pipeline_generator.cpp:19-323.  ``devices`` is an ordered sequence."""
    devices = list(devices)
    unlocked = {}
    performed = {}
    local = {d: dict(m) for d, m in device_local_inputs_map.items()}  # :36
    for d in devices:
        local.setdefault(d, {})
    holder_order = devices + [d for d in local if d not in devices]
    ready_time = {d: F32(0) for d in holder_order}
    cross_load = {d: F32(0) for d in holder_order}
    intra_load = {d: F32(0) for d in holder_order}

    def check(input_ids, dst):  # :42-113
        inter_req, intra_req = [], []  # (input, src) in decision order
        inter_sizes, intra_sizes = {}, {}
        for input_id in input_ids:
            if input_id in local[dst]:
                continue
            near = [d for d in holder_order if d[0] == dst[0] and input_id in local[d] and local[d][input_id] < stage_id]
            if near:
                src = near[0]
                for d in near[1:]:
                    if intra_load[d] < intra_load[src]:
                        src = d
                intra_req.append((input_id, src))
                size = F32(input_sizes[input_id])
                if input_block_type_map[input_id] == "OUT" and is_bw:  # :69-72: dout travels with out
                    intra_sizes[src] = F32(intra_sizes.get(src, F32(0)) + size)
                intra_sizes[src] = F32(intra_sizes.get(src, F32(0)) + size)
                continue
            far = [d for d in holder_order if d[0] != dst[0] and input_id in local[d] and local[d][input_id] < stage_id]
            if not far:
                raise RuntimeError("No device has input.")  # :98
            src = far[0]
            for d in far[1:]:
                if cross_load[d] < cross_load[src]:
                    src = d
            inter_req.append((input_id, src))
            size = F32(input_sizes[input_id])
            if input_block_type_map[input_id] == "OUT" and is_bw:
                inter_sizes[src] = F32(inter_sizes.get(src, F32(0)) + size)
            inter_sizes[src] = F32(inter_sizes.get(src, F32(0)) + size)
        can = all(not (F32(cross_load[d] + s) > F32(target_comm_load_per_node[d])) for d, s in inter_sizes.items())  # :101-107
        return can, inter_req, intra_req, inter_sizes, intra_sizes

    def trio(workload_id):  # :178-191, :243-253
        out = lse = dout = -1
        for input_id in workload_input_map[workload_id]:
            t = input_block_type_map[input_id]
            if t == "OUT":
                out = input_id
            elif t == "LSE":
                lse = input_id
            elif t == "dOUT":
                dout = input_id
        assert (out == -1) == (lse == -1)
        assert dout == -1 or out != -1
        return out, lse, dout

    def book(dst, reqs, out, lse, dout):  # :206-224, :267-284
        for input_id, src in reqs:
            performed.setdefault(dst, []).append((input_id, src))
            if input_id == out:
                performed[dst].append((lse, src))
                if dout != -1:
                    performed[dst].append((dout, src))

    def ordered(ws):
        return sorted(ws, key=lambda w: (-float(F32(workload_costs[w])), w))

    pending = {}
    for d, ws in device_workload_map.items():  # :115-122
        for w in ws:
            if w not in scheduled_workloads:
                pending.setdefault(d, set()).add(w)

    skipped = set()
    while True:  # :125-238
        pick, least = None, F32(np.finfo(np.float32).max)
        for d in devices:
            if d in skipped:
                continue
            if ready_time[d] < least:
                least, pick = ready_time[d], d
        if pick is None:
            break
        todo = ordered(pending.get(pick, ()))
        if not todo:
            skipped.add(pick)
            if len(skipped) == len(devices):
                break
            continue
        progress = False
        for w in todo:
            out, lse, dout = trio(w)
            wanted = [i for i in workload_input_map[w] if i not in (out, lse, dout)]
            if out != -1:
                wanted.append(out)
            can, inter_req, intra_req, inter_sizes, intra_sizes = check(wanted, pick)
            if not can:
                continue
            unlocked.setdefault(pick, set()).add(w)
            book(pick, inter_req, out, lse, dout)
            book(pick, intra_req, out, lse, dout)
            for d, s in inter_sizes.items():
                cross_load[d] = F32(cross_load[d] + s)
            for d, s in intra_sizes.items():
                intra_load[d] = F32(intra_load[d] + s)
            for i in workload_input_map[w]:
                local[pick].setdefault(i, stage_id)
            ready_time[pick] = F32(ready_time[pick] + F32(workload_costs[w]))
            pending[pick].discard(w)
            progress = True
            break
        if not progress:
            break

    for d in devices:  # :240-309: send blocks of still pending workloads ahead
        for w in ordered(pending.get(d, ())):
            out, lse, dout = trio(w)
            for i in workload_input_map[w]:
                if i == lse or i == dout or i in local[d]:
                    continue
                can, inter_req, intra_req, inter_sizes, intra_sizes = check([i], d)
                if not can:
                    continue
                book(d, inter_req, out, lse, dout)
                book(d, intra_req, out, lse, dout)
                for s_d, s in inter_sizes.items():
                    cross_load[s_d] = F32(cross_load[s_d] + s)
                for s_d, s in intra_sizes.items():
                    intra_load[s_d] = F32(intra_load[s_d] + s)
                local[d][i] = stage_id
                if i == out:
                    local[d][lse] = stage_id
                    if dout != -1:
                        local[d][dout] = stage_id
    return unlocked, performed, local


def generate_pipelines_n_stages(n_stages, all_devices, workload_costs, workload_input_map, input_types,
                                input_sizes, workload_to_device_map, input_to_device_map, is_bw,
                                disable_two_phase_comm=False):
    """dcp/core/pipeline.py:513-839 with the packer above; ``all_devices`` is visited in sorted
    order, ``input_types[i]`` is the block type string.  Same three lists as the reference."""
    from collections import defaultdict

    devices = sorted(all_devices)
    device_to_workload_map = {d: [] for d in devices}
    for w, d in workload_to_device_map.items():
        device_to_workload_map[d].append(w)
    local = {d: {} for d in devices}
    for i, d in input_to_device_map.items():
        local[d][i] = -1
    curr = defaultdict(set)
    for i, d in input_to_device_map.items():
        curr[d].add(i)
    inter = defaultdict(float)  # :530-575
    for w, d in workload_to_device_map.items():
        for i in workload_input_map[w]:
            if i in curr[d]:
                continue
            src = input_to_device_map[i]
            if src[0] != d[0]:
                inter[src] += input_sizes[i]
                for o in devices:
                    if o[0] == d[0]:
                        curr[o].add(i)
            curr[d].add(i)
    total = 0
    for v in inter.values():
        total += v
    target = {d: (total / len(devices) / n_stages) * 1.2 for d in devices}  # :591-597

    scheduled = set()
    ready = defaultdict(list)
    for w in range(len(workload_costs)):  # :612-623
        d = workload_to_device_map[w]
        if all(input_to_device_map[i] == d for i in workload_input_map[w]):
            ready[d].append(w)
    work_per_stage = [ready]
    comm_per_stage = [defaultdict(list)]
    for ws in ready.values():
        scheduled.update(ws)
    for stage_id in range(n_stages):  # :645-752
        unlocked, comms, local = greedy_selection_per_device(
            devices, scheduled, workload_costs, input_sizes, workload_input_map, input_types,
            device_to_workload_map, local, target, is_bw, stage_id)
        for ws in unlocked.values():
            scheduled.update(ws)
        if stage_id == n_stages - 1:
            last = {d: float("inf") for d in devices}
            more, more_comms, local = greedy_selection_per_device(
                devices, scheduled, workload_costs, input_sizes, workload_input_map, input_types,
                device_to_workload_map, local, last, is_bw, stage_id)
            for d, ws in more.items():
                unlocked[d] = unlocked.get(d, set()) | ws
                scheduled.update(ws)
            assert scheduled == set(range(len(workload_costs)))
            for d, c in more_comms.items():
                comms.setdefault(d, []).extend(c)
        work_per_stage.append(unlocked)
        comm_per_stage.append(comms)
    if disable_two_phase_comm:
        return work_per_stage, comm_per_stage, [defaultdict(list) for _ in comm_per_stage]
    first_phase, second_phase = [defaultdict(list)], [defaultdict(list)]  # :760-834
    for comms_per_device in comm_per_stage[1:]:
        recv = defaultdict(float)
        dsts = defaultdict(set)
        for dst, comms in comms_per_device.items():
            for i, src in comms:
                if src[0] != dst[0]:
                    recv[dst] += input_sizes[i]
                    dsts[(src, i, dst[0])].add(dst[1])
        remove, second = defaultdict(list), defaultdict(list)
        for src, i, node in sorted(list(dsts.keys()), key=lambda x: x[1]):
            ranks = sorted(dsts[(src, i, node)])
            if len(ranks) > 1:
                keep = min(ranks, key=lambda r: recv[(node, r)])
                for r in ranks:
                    if r != keep:
                        remove[(node, r)].append((i, src))
                        second[(node, r)].append((i, (node, keep)))
        new = defaultdict(list)
        for dst, comms in comms_per_device.items():
            new[dst] = [c for c in comms if c not in remove[dst]]
        first_phase.append(new)
        second_phase.append(second)
    return work_per_stage, first_phase, second_phase
