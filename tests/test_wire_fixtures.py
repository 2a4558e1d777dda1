"""The plan wire format against bytes written by the reference's own serializer
(tests/golden/wire/, produced by tests/golden/make_wire_fixtures.py from
dcp/core/instructions.py): this package encodes the described instructions and plans to exactly
those bytes and decodes the bytes to exactly those objects; and plans that were decoded from
such bytes run on the GPU like the plans they describe."""

import json
from pathlib import Path

import pytest

import dcp_amd.core.instructions as isa
from tests.golden import wire_spec

WIRE = Path(__file__).resolve().parent / "golden" / "wire"

BUILT_CASES = {
    "causal": dict(seqlens=[300, 200], block_size=128, n_heads=4, n_groups=2, head_dim=64, head_block=2, qkv_scale=0.5),
    "lambda": dict(seqlens=[520], block_size=64, n_heads=2, n_groups=1, head_dim=128, head_block=2, mask="lambda",
                   mask_kwargs=dict(n_starting=16, l_pretrain=100), n_kv_groups=2, qkv_scale=0.5),
    "staged": dict(n_nodes=2, n_devices_per_node=2, seqlens=[450, 200], block_size=64, n_heads=4, n_groups=2,
                   head_dim=64, head_block=2, n_stages=3),
}


def _case(name):
    from tests.plan_cases import make_case, make_multi_case

    return make_multi_case(**BUILT_CASES[name]) if name == "staged" else make_case(**BUILT_CASES[name])


def built_plans(name, case=None):
    """{fixture name: plan} of a built case (also what the fixture generator serializes)."""
    case = case or _case(name)
    if name == "staged":
        plans = {}
        for d, (f, b) in enumerate(zip(case["fw"], case["bw"])):
            plans[f"plan_staged_dev{d}_fw"] = f
            plans[f"plan_staged_dev{d}_bw"] = b
        return plans
    return {f"plan_{name}_fw": case["fw"], f"plan_{name}_bw": case["bw"]}


def _blob(name):
    return (WIRE / f"{name}.bin").read_bytes()


def _plan_fixture_names():
    return sorted(p.stem for p in WIRE.glob("plan_*.json"))


def test_every_instruction_type_encodes_to_the_reference_bytes_and_back():
    specs = json.loads((WIRE / "instructions.json").read_text())
    assert {s["op"] for s in specs.values()} == {c.__name__ for c in isa.BlockInstrBase._instr_index_to_cls.values()}
    for name, spec in specs.items():
        blob = _blob(name)
        instr = wire_spec.instr_from_spec(isa, spec, mask_as_planes=False)
        assert instr.serialize() == blob, name
        back, rest = isa.BlockInstrBase.deserialize(blob)
        assert rest == b"" and type(back) is type(instr) and back == instr, name
        assert back.serialize() == blob, name
        assert wire_spec.instr_to_spec(back) == spec, name


@pytest.mark.parametrize("name", _plan_fixture_names())
def test_plans_encode_to_the_reference_bytes_and_back(name):
    spec = json.loads((WIRE / f"{name}.json").read_text())
    blob = _blob(name)
    plan = wire_spec.plan_from_spec(isa, spec, mask_as_planes=False)
    assert plan.serialize() == blob
    back, _ = isa.ExecutionPlan.deserialize(blob)
    assert back == plan and back.serialize() == blob
    assert wire_spec.plan_to_spec(back) == spec
    # through a str, as the reference's plan exchange moves them (tests/core/test_instructions.py:20-33)
    cast = blob.decode("iso-8859-1").encode().decode().encode("iso-8859-1")
    assert isa.ExecutionPlan.deserialize(cast)[0] == plan


def test_fixture_set_is_complete():
    names = _plan_fixture_names()
    assert "plan_hand" in names and len(names) == 1 + 2 + 2 + 8


def test_list_of_plans_matches_the_reference_bytes():
    blob = _blob("plans_list")
    plans, rest = isa.deserialize_list_of_execution_plans(blob)
    assert rest == b""
    want = [isa.ExecutionPlan.deserialize(_blob(n))[0] for n in ("plan_causal_fw", "plan_causal_bw")]
    assert plans == want
    assert isa.serialize_list_of_execution_plans(plans) == blob


@pytest.mark.parametrize("case_name", sorted(BUILT_CASES))
def test_built_plans_still_are_what_the_fixtures_hold(case_name):
    """The fixtures' content came from this package's plan builders: the builders still emit it
    (a deliberate change of a builder needs the fixtures regenerated)."""
    for name, plan in built_plans(case_name).items():
        assert isa.ExecutionPlan.deserialize(_blob(name))[0] == plan, name
        assert plan.serialize() == _blob(name), name


@pytest.mark.gpu
@pytest.mark.parametrize("case_name", ["causal", "lambda"])
def test_plans_decoded_from_reference_bytes_run_on_the_gpu(gpu, case_name):
    from tests.plan_cases import check_against_truth, dense_truth, run_executor

    case = _case(case_name)
    case["fw"] = isa.ExecutionPlan.deserialize(_blob(f"plan_{case_name}_fw"))[0]
    case["bw"] = isa.ExecutionPlan.deserialize(_blob(f"plan_{case_name}_bw"))[0]
    res, _ = run_executor(case, backward=True)
    check_against_truth(res, dense_truth(case, backward=True))


@pytest.mark.gpu
def test_staged_device_plans_decoded_from_reference_bytes_run_together(gpu):
    from tests.plan_cases import check_against_truth, dense_truth, run_multi_executor

    case = _case("staged")
    n = len(case["fw"])
    case["fw"] = [isa.ExecutionPlan.deserialize(_blob(f"plan_staged_dev{d}_fw"))[0] for d in range(n)]
    case["bw"] = [isa.ExecutionPlan.deserialize(_blob(f"plan_staged_dev{d}_bw"))[0] for d in range(n)]
    assert any(type(i).__name__ == "CommLaunchInstr" for p in case["fw"] for i in p.instructions)
    res, _ = run_multi_executor(case, backward=True)
    check_against_truth(res, dense_truth(case, backward=True))
