"""The reference's CPU-expressible form of one attention row, in torch on the host:
TEST INFRASTRUCTURE ONLY (bench.py's cpu_baseline leg times it, tests/test_oracle.py pins
it); the product never imports it.

The reference has no CPU executor; what it holds that runs on a CPU is the dense masked
attention its own end-to-end test checks the kernels against (``attention_ref`` with
``attn_range``, tests/runtime/test_flash_attention.py:127-279: scores, range mask, softmax,
weighted sum; gradients by autograd).  This restates it for one q-block row against the
concatenated keys of its kv blocks, with the backward written out (the same five products
autograd would run), in fp32 torch tensor operations so that it uses the host's cores the way
the reference's torch code would.  Pinned against the numpy oracle (itself pinned in fp64)
in tests/test_oracle.py.
"""

from __future__ import annotations

import torch


def row_attention_fwd_bwd(q, k, v, dout, allowed, scale=None):
    """q, dout ``[Tq, H, D]``; k, v ``[Tk, Hkv, D]``; allowed bool ``[Tq, Tk]`` (CPU tensors).
    Returns ``(out [Tq,H,D], lse [H,Tq], dq [Tq,H,D], dk [Tk,Hkv,D], dv [Tk,Hkv,D])``;
    q head h uses kv head ``h // (H // Hkv)``; a query that attends nothing gets out 0, lse +inf
    and contributes no gradient."""
    Tq, H, D = q.shape
    Hkv = k.shape[1]
    g = H // Hkv
    if scale is None:
        scale = D ** -0.5
    kk, vv = k.repeat_interleave(g, dim=1), v.repeat_interleave(g, dim=1)
    s = torch.einsum("qhd,khd->hqk", q, kk) * scale
    s.masked_fill_(~allowed, float("-inf"))
    lse = torch.logsumexp(s, dim=-1)
    nothing = torch.isinf(lse) & (lse < 0)
    p = torch.exp(s - torch.where(nothing, torch.zeros_like(lse), lse)[..., None])  # exp(-inf - 0) = 0 for such rows
    out = torch.einsum("hqk,khd->qhd", p, vv)
    dp = torch.einsum("qhd,khd->hqk", dout, vv)
    delta = (dout * out).sum(-1).T  # [H, Tq]
    ds = p * (dp - delta[..., None])
    dq = torch.einsum("hqk,khd->qhd", ds, kk) * scale
    dk = torch.einsum("hqk,qhd->khd", ds, q).reshape(-1, Hkv, g, D).sum(2) * scale
    dv = torch.einsum("hqk,qhd->khd", p, dout).reshape(-1, Hkv, g, D).sum(2)
    lse = torch.where(nothing, torch.full_like(lse, float("inf")), lse)
    return out, lse, dq, dk, dv
