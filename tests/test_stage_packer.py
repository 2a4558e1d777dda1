"""Stage packer (host code): the native ``dcp_greedy_stage_selection`` behind
``dcp_amd.core.pipeline`` against the numpy/Python restatement in ``oracle/`` and, where it has
been built from the reference sources (``oracle/build_ref.py``), against the reference's own C++
module.

The reference picks among equals by hash-table order, so it is compared exactly only on inputs
without ties; inputs with ties are checked through the properties every valid result has.
"""

import importlib.util
import random

import numpy as np
import pytest

from oracle import build_ref
from oracle import stage_packer_oracle as oracle


@pytest.fixture(scope="module")
def pipeline():
    from dcp_amd import _lib

    if not _lib.LIB_PATH.exists():
        from dcp_amd import build

        build.build(verbose=False)
    from dcp_amd.core import pipeline as mod

    return mod


@pytest.fixture(scope="module")
def reference_cpp():
    """The reference's dcp_cpp module, compiled from its own sources; skipped if absent."""
    path = build_ref.module_path()
    if not path.exists() and build_ref.build(verbose=False) is None:
        pytest.skip("reference sources not present and oracle/_ref not built")
    spec = importlib.util.spec_from_file_location("dcp_cpp", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


# ---------------------------------------------------------------------------------------------
# problems
# ---------------------------------------------------------------------------------------------
def make_problem(seed, n_nodes=2, ranks=2, n_q=6, n_kv=6, n_work=24, bw=False, distinct=True, only_device=None,
                 with_out_in_fw=False):
    """Blocks: n_q query blocks, n_kv key/value blocks and, for a backward problem, an
    (OUT, LSE, dOUT) trio per query block.  Workload = one (q, kv) pair.  Every block starts on
    exactly one device.  `distinct`: all costs and sizes differ (no ties for the sort)."""
    rng = random.Random(seed)
    devices = [(n, r) for n in range(n_nodes) for r in range(ranks)]
    types, sizes = [], []
    for _ in range(n_q):
        types.append("Q")
    for _ in range(n_kv):
        types.append("KV")
    trio_of_q = {}
    if bw or with_out_in_fw:
        for q in range(n_q):
            trio_of_q[q] = [len(types), len(types) + 1] + ([len(types) + 2] if bw else [])
            types += ["OUT", "LSE"] + (["dOUT"] if bw else [])
    n_inputs = len(types)
    base = list(range(1, 4 * n_inputs + 1))
    rng.shuffle(base)
    sizes = [float(base[i]) if distinct else float(rng.choice([1, 2, 2, 4])) for i in range(n_inputs)]
    pairs = [(q, k) for q in range(n_q) for k in range(n_kv)]
    rng.shuffle(pairs)
    pairs = pairs[:n_work]
    workload_input_map = []
    for q, k in pairs:
        ins = [q, n_q + k] + trio_of_q.get(q, [])
        rng.shuffle(ins)
        workload_input_map.append(ins)
    cost_base = list(range(1, 3 * len(pairs) + 1))
    rng.shuffle(cost_base)
    costs = [float(cost_base[w]) if distinct else float(rng.choice([1, 1, 2, 3])) for w in range(len(pairs))]
    input_home = {i: rng.choice(devices) for i in range(n_inputs)}
    for q, trio in trio_of_q.items():  # a trio lives together
        for i in trio:
            input_home[i] = input_home[trio[0]]
    workload_home = {w: (only_device if only_device is not None else rng.choice(devices)) for w in range(len(pairs))}
    device_workload_map = {d: [] for d in devices}
    for w, d in workload_home.items():
        device_workload_map[d].append(w)
    local = {d: {} for d in devices}
    for i, d in input_home.items():
        local[d][i] = -1
    return dict(devices=devices, costs=costs, sizes=sizes, workload_input_map=workload_input_map, types=types,
                device_workload_map=device_workload_map, local=local, input_home=input_home,
                workload_home=workload_home, bw=bw)


def run_native(pipeline, pb, scheduled, local, target, stage_id):
    return pipeline.greedy_selection_per_device(set(pb["devices"]), set(scheduled), pb["costs"], pb["sizes"],
                                                pb["workload_input_map"], pb["types"], pb["device_workload_map"], local,
                                                target, pb["bw"], stage_id, None)


def run_oracle(pb, scheduled, local, target, stage_id):
    return oracle.greedy_selection_per_device(sorted(pb["devices"]), set(scheduled), pb["costs"], pb["sizes"],
                                              pb["workload_input_map"], pb["types"], pb["device_workload_map"], local,
                                              target, pb["bw"], stage_id)


def run_reference(mod, pb, scheduled, local, target, stage_id):
    return mod.greedy_selection_per_device(set(pb["devices"]), set(scheduled), pb["costs"], pb["sizes"],
                                           pb["workload_input_map"], pb["types"], pb["device_workload_map"], local,
                                           target, pb["bw"], stage_id, None)


def normal(result, ordered_comm=True):
    unlocked, comm, local = result
    unlocked = {d: set(ws) for d, ws in unlocked.items() if ws}
    comm = {d: (list(map(tuple, c)) if ordered_comm else sorted(map(tuple, c))) for d, c in comm.items() if c}
    local = {d: dict(m) for d, m in local.items() if m}
    return unlocked, comm, local


def check_properties(pb, scheduled, local_before, target, stage_id, result):
    """What any valid result satisfies, whatever the order among equals."""
    unlocked, comm, local_after = result
    devices = pb["devices"]
    types = pb["types"]
    # workloads: only pending ones of the device itself, each at most once
    seen = set()
    for d, ws in unlocked.items():
        for w in ws:
            assert w in pb["device_workload_map"][d] and w not in scheduled and w not in seen
            seen.add(w)
            for i in pb["workload_input_map"][w]:
                assert i in local_after[d], "an unlocked workload's blocks are all held afterwards"
    # transfers: from a device that held the block before this stage, to one that did not
    sent = {d: np.float32(0) for d in devices}
    for dst, entries in comm.items():
        got = [i for i, _ in entries]
        assert len(got) == len(set(got)), "a block is sent to a device once"
        for i, src in entries:
            assert i in local_before.get(src, {}) and local_before[src][i] < stage_id
            assert i not in local_before.get(dst, {})
            assert local_after[dst][i] == stage_id
            if src[0] != dst[0]:
                near = [d for d in devices if d[0] == dst[0] and i in local_before.get(d, {}) and local_before[d][i] < stage_id]
                assert not near, "a holder on the same node is preferred"
                sent[src] = np.float32(sent[src] + np.float32(pb["sizes"][i]))
        # out, lse and dout arrive together and from the same source
        by_input = dict(entries)
        for w in range(len(pb["costs"])):
            ins = pb["workload_input_map"][w]
            trio = [i for i in ins if types[i] in ("OUT", "LSE", "dOUT")]
            if trio and any(i in by_input for i in trio) and pb["workload_home"][w] == dst:
                assert all(i in by_input for i in trio) and len({by_input[i] for i in trio}) == 1
    for d in devices:  # LSE is not priced; dOUT is priced through OUT -- recompute the booked bytes
        booked = np.float32(0)
        for dst, entries in comm.items():
            for i, src in entries:
                if src == d and src[0] != dst[0] and types[i] not in ("LSE", "dOUT"):
                    booked = np.float32(booked + np.float32(pb["sizes"][i]) * (2 if types[i] == "OUT" and pb["bw"] else 1))
        assert booked <= np.float32(target[d]) * (1 + 1e-6), "a sender stays within its cross-node budget"
    # nothing is lost, stages only appear for new blocks
    for d in devices:
        for i, s in local_before.get(d, {}).items():
            assert local_after[d][i] == s
        for i, s in local_after.get(d, {}).items():
            assert i in local_before.get(d, {}) or s == stage_id


# ---------------------------------------------------------------------------------------------
# native == restatement, everywhere (same order among equals by construction)
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("seed", range(12))
@pytest.mark.parametrize("bw", [False, True])
def test_native_equals_restatement_over_stages(pipeline, seed, bw):
    pb = make_problem(seed, n_nodes=2 + seed % 2, ranks=1 + seed % 3, n_q=5, n_kv=6, n_work=26, bw=bw,
                      distinct=seed % 2 == 0, with_out_in_fw=seed % 4 == 1)
    total = sum(pb["sizes"])
    scheduled = set()
    local_n = local_o = pb["local"]
    for stage_id in range(3):
        target = {d: (total * 0.08 * (1 + (seed + d[1]) % 3) if stage_id < 2 else float("inf")) for d in pb["devices"]}
        before = {d: dict(m) for d, m in local_o.items()}
        res_n = run_native(pipeline, pb, scheduled, local_n, target, stage_id)
        res_o = run_oracle(pb, scheduled, local_o, target, stage_id)
        assert normal(res_n) == normal(res_o)
        check_properties(pb, scheduled, before, target, stage_id, res_n)
        for ws in res_o[0].values():
            scheduled |= ws
        local_n, local_o = res_n[2], res_o[2]
    assert scheduled == set(range(len(pb["costs"]))), "an unlimited last stage schedules everything"


# ---------------------------------------------------------------------------------------------
# restatement == the reference's C++ where the reference's result does not depend on hash order
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("seed", range(10))
@pytest.mark.parametrize("bw", [False, True])
def test_reference_cpp_single_busy_device(pipeline, reference_cpp, seed, bw):
    """All pending work on one device, every block on exactly one device, distinct costs and
    sizes: no choice among equals is ever made.  Finite budgets, three stages."""
    pb0 = make_problem(100 + seed, bw=bw)
    busy = pb0["devices"][seed % len(pb0["devices"])]
    pb = make_problem(100 + seed, bw=bw, only_device=busy)
    total = sum(pb["sizes"])
    scheduled = set()
    local_r = local_o = local_n = pb["local"]
    for stage_id in range(3):
        target = {d: total * (0.05 + 0.04 * ((seed + d[0] + 2 * d[1]) % 4)) if stage_id < 2 else float("inf") for d in pb["devices"]}
        before = {d: dict(m) for d, m in local_o.items()}
        res_r = run_reference(reference_cpp, pb, scheduled, local_r, target, stage_id)
        res_o = run_oracle(pb, scheduled, local_o, target, stage_id)
        res_n = run_native(pipeline, pb, scheduled, local_n, target, stage_id)
        # within one workload the reference lists transfers in hash order: compare them as sets
        assert normal(res_r, ordered_comm=False) == normal(res_o, ordered_comm=False)
        assert normal(res_n) == normal(res_o)
        check_properties(pb, scheduled, before, target, stage_id, res_r)
        for ws in res_o[0].values():
            scheduled |= ws
        local_r, local_o, local_n = res_r[2], res_o[2], res_n[2]
    assert scheduled == set(range(len(pb["costs"])))


@pytest.mark.parametrize("seed", range(8))
@pytest.mark.parametrize("bw", [False, True])
def test_reference_cpp_unlimited_budget(pipeline, reference_cpp, seed, bw):
    """Work on every device, unlimited budgets, one holder per block, distinct costs: every
    device takes all its workloads and every source is forced, whatever the device order."""
    pb = make_problem(200 + seed, n_nodes=2 + seed % 2, ranks=2, bw=bw)
    target = {d: float("inf") for d in pb["devices"]}
    res_r = run_reference(reference_cpp, pb, set(), pb["local"], target, 0)
    res_o = run_oracle(pb, set(), pb["local"], target, 0)
    res_n = run_native(pipeline, pb, set(), pb["local"], target, 0)
    assert normal(res_r, ordered_comm=False) == normal(res_o, ordered_comm=False)
    assert normal(res_n) == normal(res_o)
    assert set().union(*res_r[0].values()) == set(range(len(pb["costs"])))


def test_reference_cpp_least_loaded_holder(pipeline, reference_cpp):
    """Two remote holders of a block with different loads: the less loaded one sends.
    Device (1,0) runs two workloads.  The expensive one needs block 0, held only by (0,0), which
    then carries load; the cheap one needs block 1, held by (0,0) and (0,1): (0,1) must send."""
    devices = [(0, 0), (0, 1), (1, 0)]
    args = dict(costs=[9.0, 4.0], sizes=[5.0, 3.0, 1.0], workload_input_map=[[0, 2], [1, 2]], types=["KV", "KV", "Q"],
                device_workload_map={(1, 0): [0, 1], (0, 0): [], (0, 1): []},
                local={(0, 0): {0: -1, 1: -1}, (0, 1): {1: -1}, (1, 0): {2: -1}}, devices=devices, bw=False)
    target = {d: 100.0 for d in devices}
    expect = ({(1, 0): {0, 1}}, {(1, 0): [(0, (0, 0)), (1, (0, 1))]},
              {(0, 0): {0: -1, 1: -1}, (0, 1): {1: -1}, (1, 0): {2: -1, 0: 0, 1: 0}})
    for res in (run_reference(reference_cpp, args, set(), args["local"], target, 0),
                run_oracle(args, set(), args["local"], target, 0),
                run_native(pipeline, args, set(), args["local"], target, 0)):
        assert normal(res) == expect


@pytest.mark.parametrize("seed", range(6))
def test_reference_cpp_satisfies_the_same_properties_with_ties(reference_cpp, pipeline, seed):
    """With equal costs, sizes and loads the reference's pick is hash order: only the properties
    are compared, for the reference and for the native packer alike."""
    pb = make_problem(300 + seed, distinct=False, bw=seed % 2 == 1)
    total = sum(pb["sizes"])
    target = {d: total * 0.15 for d in pb["devices"]}
    for run in (lambda: run_reference(reference_cpp, pb, set(), pb["local"], target, 0),
                lambda: run_native(pipeline, pb, set(), pb["local"], target, 0)):
        check_properties(pb, set(), pb["local"], target, 0, run())


# ---------------------------------------------------------------------------------------------
# hand-computed cases and error behaviour
# ---------------------------------------------------------------------------------------------
def test_budget_blocks_then_sends_ahead(pipeline):
    """One remote block of 10 bytes per workload, budget 15: the expensive workload is unlocked,
    the second does not fit (10 + 10 > 15) and nothing else can be sent ahead either."""
    devices = [(0, 0), (1, 0)]
    pb = dict(devices=devices, costs=[5.0, 3.0], sizes=[10.0, 10.0, 1.0], workload_input_map=[[2, 0], [2, 1]],
              types=["KV", "KV", "Q"], device_workload_map={(1, 0): [0, 1], (0, 0): []},
              local={(0, 0): {0: -1, 1: -1}, (1, 0): {2: -1}}, bw=False)
    res = run_native(pipeline, pb, set(), pb["local"], {(0, 0): 15.0, (1, 0): 15.0}, 0)
    assert normal(res) == ({(1, 0): {0}}, {(1, 0): [(0, (0, 0))]}, {(0, 0): {0: -1, 1: -1}, (1, 0): {2: -1, 0: 0}})
    # with budget 25 the second workload is unlocked as well
    res = run_native(pipeline, pb, set(), pb["local"], {(0, 0): 25.0, (1, 0): 25.0}, 0)
    assert normal(res)[0] == {(1, 0): {0, 1}}


def test_backward_counts_out_twice_and_moves_the_trio(pipeline):
    devices = [(0, 0), (1, 0)]
    # blocks: 0 Q, 1 OUT (4 bytes), 2 LSE, 3 dOUT, all on (0,0); the workload runs on (1,0)
    pb = dict(devices=devices, costs=[1.0], sizes=[2.0, 4.0, 1.0, 4.0], workload_input_map=[[2, 0, 3, 1]],
              types=["Q", "OUT", "LSE", "dOUT"], device_workload_map={(1, 0): [0], (0, 0): []},
              local={(0, 0): {0: -1, 1: -1, 2: -1, 3: -1}, (1, 0): {}}, bw=True)
    # needed: Q (2) + OUT twice (8) = 10
    res = run_native(pipeline, pb, set(), pb["local"], {(0, 0): 9.5, (1, 0): 0.0}, 0)
    assert normal(res)[0] == {}
    # sent ahead instead: Q alone fits (2 <= 9.5), OUT (8) then does not (2 + 8 > 9.5)
    assert normal(res)[1] == {(1, 0): [(0, (0, 0))]}
    res = run_native(pipeline, pb, set(), pb["local"], {(0, 0): 10.0, (1, 0): 0.0}, 0)
    assert normal(res)[0] == {(1, 0): {0}}
    assert normal(res)[1] == {(1, 0): [(0, (0, 0)), (1, (0, 0)), (2, (0, 0)), (3, (0, 0))]}
    # as a forward problem the same OUT block counts once: 2 + 4 <= 9.5
    pb_fw = dict(pb, bw=False)
    assert normal(run_native(pipeline, pb_fw, set(), pb["local"], {(0, 0): 9.5, (1, 0): 0.0}, 0))[0] == {(1, 0): {0}}


def test_blocks_received_in_this_stage_are_not_sources_yet(pipeline):
    """(1,0) and (1,1) both need remote block 0 in stage 0: both fetch it from (0,0); in stage 1
    a third device of the node takes it from a neighbour instead."""
    devices = [(0, 0), (1, 0), (1, 1), (1, 2)]
    pb = dict(devices=devices, costs=[3.0, 2.0, 1.0], sizes=[4.0], workload_input_map=[[0], [0], [0]], types=["KV"],
              device_workload_map={(1, 0): [0], (1, 1): [1], (1, 2): [2], (0, 0): []},
              local={(0, 0): {0: -1}}, bw=False)
    inf = {d: float("inf") for d in devices}
    res = run_native(pipeline, pb, {2}, pb["local"], inf, 0)
    assert normal(res)[1] == {(1, 0): [(0, (0, 0))], (1, 1): [(0, (0, 0))]}
    res1 = run_native(pipeline, pb, {0, 1}, res[2], inf, 1)
    assert normal(res1)[1] == {(1, 2): [(0, (1, 0))]}


def test_missing_block_is_an_error(pipeline, reference_cpp):
    devices = [(0, 0), (1, 0)]
    pb = dict(devices=devices, costs=[1.0], sizes=[1.0], workload_input_map=[[0]], types=["KV"],
              device_workload_map={(1, 0): [0], (0, 0): []}, local={(0, 0): {}, (1, 0): {}}, bw=False)
    inf = {d: float("inf") for d in devices}
    with pytest.raises(AssertionError, match="no device held"):
        run_native(pipeline, pb, set(), pb["local"], inf, 0)
    with pytest.raises(RuntimeError, match="No device has input"):
        run_reference(reference_cpp, pb, set(), pb["local"], inf, 0)
    with pytest.raises(RuntimeError, match="No device has input"):
        run_oracle(pb, set(), pb["local"], inf, 0)


def test_argument_checks(pipeline):
    from dcp_amd import _lib

    with pytest.raises(AssertionError, match="devices: positive"):
        _lib.call("dcp_greedy_stage_selection", 0, *([0] * 23))
    devices = [(0, 0)]
    pb = dict(devices=devices, costs=[1.0], sizes=[1.0, 1.0], workload_input_map=[[0, 1]], types=["Q", "OUT"],
              device_workload_map={(0, 0): [0]}, local={(0, 0): {0: -1, 1: -1}}, bw=False)
    with pytest.raises(AssertionError, match="out block without its lse"):
        run_native(pipeline, pb, set(), pb["local"], {(0, 0): 1.0}, 0)
    pb["workload_input_map"] = [[0, 7]]
    with pytest.raises(AssertionError, match="out of range"):
        run_native(pipeline, pb, set(), pb["local"], {(0, 0): 1.0}, 0)


# ---------------------------------------------------------------------------------------------
# generate_pipelines_n_stages
# ---------------------------------------------------------------------------------------------
class _Meta:
    def __init__(self, t):
        self.type = t


@pytest.mark.parametrize("seed", range(8))
@pytest.mark.parametrize("n_stages", [1, 2, 4])
def test_generate_pipelines_matches_restatement_and_is_a_valid_pipeline(pipeline, seed, n_stages):
    bw = seed % 2 == 1
    pb = make_problem(400 + seed, n_nodes=2, ranks=2 + seed % 2, n_q=6, n_kv=7, n_work=36, bw=bw, distinct=seed % 3 != 0)
    metas = {i: _Meta(t) for i, t in enumerate(pb["types"])}
    got = pipeline.generate_pipelines_n_stages(n_stages, set(pb["devices"]), pb["costs"], pb["workload_input_map"], metas,
                                               pb["sizes"], pb["workload_home"], pb["input_home"], bw)
    want = oracle.generate_pipelines_n_stages(n_stages, set(pb["devices"]), pb["costs"], pb["workload_input_map"],
                                              pb["types"], pb["sizes"], pb["workload_home"], pb["input_home"], bw)
    strip = lambda stages: [{d: (set(v) if isinstance(v, (set, frozenset)) else list(v)) for d, v in s.items() if v} for s in stages]
    assert [strip(x) for x in got] == [strip(x) for x in want]

    work, first_phase, second_phase = got
    assert len(work) == len(first_phase) == len(second_phase) == n_stages + 1
    # every workload exactly once, on its own device; stage 0 needs no transfer
    placed = {}
    for s, per_device in enumerate(work):
        for d, ws in per_device.items():
            for w in ws:
                assert w not in placed and pb["workload_home"][w] == d
                placed[w] = s
    assert set(placed) == set(range(len(pb["costs"])))
    assert not any(first_phase[0].values()) and not any(second_phase[0].values())
    # replay: a block must be on the device when a workload of that stage (or a forward) uses it
    have = {d: {i for i, h in pb["input_home"].items() if h == d} for d in pb["devices"]}
    for s in range(n_stages + 1):
        arrived = {d: set() for d in pb["devices"]}
        for dst, entries in first_phase[s].items():
            for i, src in entries:
                assert i in have[src], "first-phase source holds the block from an earlier stage"
                arrived[dst].add(i)
        for dst, entries in second_phase[s].items():
            for i, src in entries:
                assert src[0] == dst[0] and i in arrived[src], "forwarded inside the node by the device that fetched it"
                arrived[dst].add(i)
        for d in pb["devices"]:
            have[d] |= arrived[d]
        for d, ws in work[s].items():
            for w in ws:
                assert set(pb["workload_input_map"][w]) <= have[d]


def test_two_phase_split_picks_one_receiver_per_node(pipeline):
    """Three devices of node 1 need remote block 0 in the same stage: one fetches, two get it forwarded."""
    devices = [(0, 0), (1, 0), (1, 1), (1, 2)]
    metas = {0: _Meta("KV"), 1: _Meta("Q"), 2: _Meta("Q"), 3: _Meta("Q")}
    work, first, second = pipeline.generate_pipelines_n_stages(
        1, set(devices), [3.0, 2.0, 1.0], [[0, 1], [0, 2], [0, 3]], metas, [8.0, 1.0, 1.0, 1.0],
        {0: (1, 0), 1: (1, 1), 2: (1, 2)}, {0: (0, 0), 1: (1, 0), 2: (1, 1), 3: (1, 2)}, False)
    assert {d: set(ws) for d, ws in work[1].items()} == {(1, 0): {0}, (1, 1): {1}, (1, 2): {2}}
    assert {d: c for d, c in first[1].items() if c} == {(1, 0): [(0, (0, 0))]}
    assert {d: c for d, c in second[1].items() if c} == {(1, 1): [(0, (1, 0))], (1, 2): [(0, (1, 0))]}
    same = pipeline.generate_pipelines_n_stages(
        1, set(devices), [3.0, 2.0, 1.0], [[0, 1], [0, 2], [0, 3]], metas, [8.0, 1.0, 1.0, 1.0],
        {0: (1, 0), 1: (1, 1), 2: (1, 2)}, {0: (0, 0), 1: (1, 0), 2: (1, 1), 3: (1, 2)}, False,
        disable_two_phase_comm=True)
    assert {d: c for d, c in same[1][1].items() if c} == {(1, 0): [(0, (0, 0))], (1, 1): [(0, (0, 0))], (1, 2): [(0, (0, 0))]}
    assert not any(any(s.values()) for s in same[2])
