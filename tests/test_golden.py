"""The committed golden vectors (tests/golden/, written by make_fixtures.py from
dense torch-float64 attention, scipy logsumexp and hand-laid bytes) against the
oracle on the CPU and against the HIP path on the GPU."""

import os

import numpy as np
import pytest
import torch

from dcp_amd.core.instructions import BlockInstrBase, BufferBlock, BufferType, MemcpyInstr
from oracle import dcp_oracle as oracle

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

# name -> (mask generator, its extra arguments, kv heads, head block, block size)
ATTN_CASES = {
    "attn_causal_gqa": ("causal", None, {}, 2, 2, 64),
    "attn_lambda": ("lambda", None, dict(n_starting=8, l_pretrain=48), 4, 1, 64),
    "attn_shared_prefix": ("shared_prefix",
                           [dict(prefix=64, continuations=[40, 88]), dict(prefix=100, continuations=[30])],
                           {}, 1, 4, 128),
}


def load_attn(name):
    z = np.load(os.path.join(GOLDEN, name + ".npz"))

    def bf16(a):
        return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)

    return z, bf16(z["q_bf16"]), bf16(z["kv_bf16"]), bf16(z["dout_bf16"])


def make_mask(name, seqlens):
    from dcp_amd.runtime.flash_attention.utils import MASK_FNS

    fn, info, kwargs, *_ = ATTN_CASES[name]
    return MASK_FNS[fn](seqlens, seqlens, torch.int32, info, **kwargs)


@pytest.mark.parametrize("name", sorted(ATTN_CASES))
def test_oracle_matches_golden_attention(name):
    z, q, kv, dout = load_attn(name)
    seqlens = [int(x) for x in z["seqlens"]]
    mask = make_mask(name, seqlens).numpy()
    out, lse, dq, dkv = oracle.dense_reference(q.float().numpy(), kv.float().numpy(), mask, seqlens,
                                               dout=dout.float().numpy())
    for got, key in ((out, "out"), (lse, "lse"), (dq, "dq"), (dkv, "dkv")):
        np.testing.assert_allclose(got, z[key], rtol=1e-5, atol=1e-5, err_msg=key)


def test_oracle_matches_golden_merge():
    z = np.load(os.path.join(GOLDEN, "merge_5_sources.npz"))
    out, lse = oracle.merge_out_lse(z["outs"], np.ascontiguousarray(z["lses"].transpose(0, 2, 1)))
    np.testing.assert_allclose(out, z["out"], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(lse.T, z["lse"], rtol=1e-12, atol=1e-12)


def test_wire_bytes_match_hand_laid_instruction():
    with open(os.path.join(GOLDEN, "memcpy_instr.bin"), "rb") as f:
        blob = f.read()
    instr = MemcpyInstr([
        (BufferBlock(BufferType.LOCAL_Q, 3, 77), BufferBlock(BufferType.BUFFER_Q, 1, 77)),
        (BufferBlock(BufferType.LOCAL_KV, 0, 64), BufferBlock(BufferType.BUFFER_KV, 2, 64)),
    ])
    assert instr.serialize() == blob
    back, rest = BlockInstrBase.deserialize(blob)
    assert rest == b"" and back == instr


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(ATTN_CASES))
def test_hip_path_matches_golden_attention(gpu, name):
    from dcp_amd.runtime.flash_attention.single_device import build_single_device_plans
    from tests.plan_cases import run_executor

    z, q, kv, dout = load_attn(name)
    seqlens = [int(x) for x in z["seqlens"]]
    _, _, _, n_kv_heads, head_block, block_size = ATTN_CASES[name]
    n_heads, head_dim = q.shape[1], q.shape[2]
    mask = make_mask(name, seqlens)
    fw, bw, layout = build_single_device_plans(seqlens, block_size, n_heads, n_kv_heads, head_dim, head_block,
                                               mask, dtype=torch.bfloat16)
    case = dict(fw=fw, bw=bw, layout=layout, mask=mask, q=q, kv=kv, dout=dout, seqlens=seqlens,
                head_block=head_block, head_dim=head_dim, dtype="bf16")
    (out, lse, dq, dkv), _ = run_executor(case, backward=True)
    # out and dQ: pure max-abs 2e-2; LSE 1e-3; dK/dV: 2e-2 relative to max(1, |ref|)
    assert np.abs(out.float().numpy() - z["out"]).max() <= 2e-2
    assert np.abs(lse.float().numpy() - z["lse"]).max() <= 1e-3
    assert np.abs(dq.float().numpy() - z["dq"]).max() <= 2e-2
    ref = z["dkv"]
    assert (np.abs(dkv.float().numpy() - ref) <= 2e-2 * np.maximum(1.0, np.abs(ref))).all(), "dkv"
