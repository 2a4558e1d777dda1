#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/ (run once; the .npz files are committed).

The reference's tests hold no stored vectors for this path, so these are made from
first principles, with none of this package's or the oracle's code:

* attention cases: dense softmax attention in torch float64 with a boolean mask
  filled token by token from the mask definitions (causal; attention sink plus
  sliding window, dcp/runtime/flash_attention/utils.py:501-525; shared prefix with
  independent continuations, utils.py:545-592), gradients by torch.autograd
  (the reference test's method, tests/runtime/test_flash_attention.py:442-449).
  Inputs are rounded to bf16 first and stored as bf16 bit patterns (uint16), so
  every consumer sees the same values; results are stored as float32.
* merge case: scipy.special.logsumexp and a float64 weighted sum, with +inf,
  -inf and all-empty sources (dcp/ops/fused_ops.py:118-143).
* wire case: the bytes of one MemcpyInstr laid out by hand with struct.pack from
  the format description (1-byte opcode, little-endian 4-byte ints, length-prefixed
  lists; dcp/core/serialization.py:10-120, dcp/core/instructions.py:303-344).

Usage: python tests/golden/make_fixtures.py
"""

import os
import struct

import numpy as np
import scipy.special
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def allowed_causal(L, **_):
    m = np.zeros((L, L), dtype=bool)
    for i in range(L):
        m[i, : i + 1] = True
    return m


def allowed_lambda(L, sink, window, **_):
    m = np.zeros((L, L), dtype=bool)
    for i in range(L):
        for j in range(i + 1):
            m[i, j] = j < sink or j > i - window
    return m


def allowed_shared_prefix(L, prefix, continuations, **_):
    assert prefix + sum(continuations) == L
    m = np.zeros((L, L), dtype=bool)
    for i in range(prefix):
        m[i, : i + 1] = True
    start = prefix
    for c in continuations:
        for i in range(start, start + c):
            m[i, :prefix] = True
            m[i, start : i + 1] = True
        start += c
    return m


def bf16_bits(x):
    """The (exactly bf16-representable) values as raw bf16 bit patterns."""
    return x.detach().bfloat16().view(torch.int16).numpy().view(np.uint16)


def attention_case(name, seqlens, n_heads, n_kv_heads, head_dim, allowed_fn, infos, seed):
    g = torch.Generator().manual_seed(seed)
    T = sum(seqlens)
    q = torch.randn(T, n_heads, head_dim, generator=g).bfloat16().double()
    kv = torch.randn(T, 2, n_kv_heads, head_dim, generator=g).bfloat16().double()
    dout = torch.randn(T, n_heads, head_dim, generator=g).bfloat16().double()
    q.requires_grad_(True)
    kv.requires_grad_(True)
    group = n_heads // n_kv_heads
    outs, lses = [], []
    off = 0
    for L, info in zip(seqlens, infos):
        allowed = torch.from_numpy(allowed_fn(L, **info))
        qs = q[off : off + L].permute(1, 0, 2)  # [H, L, D]
        ks = kv[off : off + L, 0].permute(1, 0, 2).repeat_interleave(group, dim=0)
        vs = kv[off : off + L, 1].permute(1, 0, 2).repeat_interleave(group, dim=0)
        s = qs @ ks.transpose(1, 2) * head_dim**-0.5
        s = s.masked_fill(~allowed, float("-inf"))
        lses.append(torch.logsumexp(s, dim=-1))  # [H, L]
        outs.append((torch.softmax(s, dim=-1) @ vs).permute(1, 0, 2))
        off += L
    out = torch.cat(outs)
    lse = torch.cat(lses, dim=1)
    dq, dkv = torch.autograd.grad(out, (q, kv), dout)
    np.savez_compressed(
        os.path.join(HERE, name + ".npz"),
        seqlens=np.asarray(seqlens), q_bf16=bf16_bits(q), kv_bf16=bf16_bits(kv), dout_bf16=bf16_bits(dout),
        out=out.detach().float().numpy(), lse=lse.detach().float().numpy(),
        dq=dq.float().numpy(), dkv=dkv.float().numpy())


def merge_case(seed=5):
    rng = np.random.default_rng(seed)
    S, T, H, D = 5, 24, 3, 16
    outs = rng.standard_normal((S, T, H, D))
    lses = rng.uniform(-5, 5, (S, T, H))
    lses[1, 3] = np.inf        # an empty source
    lses[2, 4] = -np.inf       # the other sign of empty
    lses[:, 7, 1] = [np.inf, -np.inf, np.inf, np.inf, -np.inf]  # nothing to merge
    finite = np.isfinite(lses)
    safe = np.where(finite, lses, -np.inf)
    with np.errstate(divide="ignore", invalid="ignore"):
        lse = scipy.special.logsumexp(safe, axis=0)
        w = np.where(finite, np.exp(safe - lse), 0.0)
    out = (w[..., None] * outs).sum(axis=0)
    none = ~finite.any(axis=0)
    out[none] = 0.0
    lse[none] = -1.0
    np.savez_compressed(os.path.join(HERE, "merge_5_sources.npz"), outs=outs, lses=lses, out=out, lse=lse)


def wire_case():
    # MemcpyInstr (opcode 0) moving LOCAL_Q block 3 -> BUFFER_Q slot 1 and LOCAL_KV block 0 ->
    # BUFFER_KV slot 2, 77 and 64 tokens.  A block is (buffer type: string, index: int, n_tokens: int);
    # strings are a 4-byte length followed by UTF-8 bytes; lists are a 4-byte count first.
    def s(text):
        b = text.encode("utf-8")
        return struct.pack("<i", len(b)) + b

    def block(btype, index, n_tokens):
        return s(btype) + struct.pack("<ii", index, n_tokens)

    pairs = [(block("LocalQ", 3, 77), block("BufferQ", 1, 77)),
             (block("LocalKV", 0, 64), block("BufferKV", 2, 64))]
    body = struct.pack("<i", len(pairs)) + b"".join(a + b for a, b in pairs)
    blob = bytes([0]) + body
    with open(os.path.join(HERE, "memcpy_instr.bin"), "wb") as f:
        f.write(blob)


def main():
    attention_case("attn_causal_gqa", [70, 200], 4, 2, 64, allowed_causal, [{}, {}], seed=1)
    attention_case("attn_lambda", [150, 90], 4, 4, 64, allowed_lambda,
                   [dict(sink=8, window=48)] * 2, seed=2)
    attention_case("attn_shared_prefix", [192, 130], 4, 1, 128, allowed_shared_prefix,
                   [dict(prefix=64, continuations=[40, 88]), dict(prefix=100, continuations=[30])], seed=3)
    merge_case()
    wire_case()


if __name__ == "__main__":
    main()
