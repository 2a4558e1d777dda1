"""Seeded sweep of small random plans (block sizes, head layouts, masks, dtypes, ragged and
one-token sequences, several partials per row) through the executor, forward and backward,
against dense fp64 attention on the same rounded inputs.

Bounds: out and gradients elementwise |err| <= 2e-2 * max(1, |ref|), or, for the few small
elements whose error is set by the large bf16-rounded terms they are a sum of, |err| <= 4e-3 *
max|ref| of the tensor; LSE 1e-3."""

import random

import numpy as np
import pytest

from tests.plan_cases import dense_truth, make_case, run_executor

pytestmark = pytest.mark.gpu


def _random_config(rng, seed):
    bs = rng.choice([64, 128, 256])
    groups = rng.choice([1, 2, 4])
    per = rng.choice([1, 2, 4])
    heads = groups * per
    hb = rng.choice([x for x in (1, 2, 4, 8, 16) if heads % x == 0 and (x % per == 0 or per % x == 0)])
    seqlens = [rng.choice([1, 2, 63, 64, 65, 127, 200, 300, 511, 700, 1025]) for _ in range(rng.randint(1, 4))]
    mask = rng.choice(["causal", "causal", "lambda", "shared_question", "causal_blockwise", "modality_specific"])
    kw, info = {}, None
    if mask == "lambda":
        kw = dict(n_starting=rng.choice([1, 16, 70]), l_pretrain=rng.choice([32, 100, 400]))
    elif mask == "shared_question":
        kw = dict(question_proportion=rng.choice([0.1, 0.4]), n_answers=rng.choice([1, 3, 5]))
    elif mask == "causal_blockwise":
        kw = dict(block_size=rng.choice([32, 128]), k_local=rng.choice([1, 2]))
    elif mask == "modality_specific":
        info = []
        for length in seqlens:
            img = rng.choice([8, 40, 100])
            if length <= img + 2:
                info.append(dict(image_size=img, text_lengths=[length]))
            else:
                first = rng.randint(1, length - img - 1)
                info.append(dict(image_size=img, text_lengths=[first, length - img - first]))
        kw = dict(limit_image_attn_to_self=rng.choice([False, True]))
    return dict(seqlens=seqlens, block_size=bs, n_heads=heads, n_groups=groups, head_dim=rng.choice([64, 128]),
                head_block=hb, mask=mask, mask_info=info, mask_kwargs=kw, dtype=rng.choice(["bf16", "bf16", "fp16"]),
                n_kv_groups=rng.choice([1, 1, 2, 3]), qkv_scale=0.5, seed=seed, fold=rng.choice([False, True]))


def _excess(got, ref):
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    err = np.abs(got - ref)
    bound = np.maximum(2e-2 * np.maximum(1.0, np.abs(ref)), 4e-3 * np.abs(ref).max())
    return float((err / bound).max())


def test_random_plans_match_dense_truth(gpu):
    rng = random.Random(20240611)
    done = 0
    for i in range(48):
        cfg = _random_config(rng, i)
        try:
            case = make_case(**cfg)
        except AssertionError:
            continue  # a head layout the plan builder does not take
        print(i, cfg, flush=True)
        res, _ = run_executor(case, backward=True)
        t_out, t_lse, t_dq, t_dkv = dense_truth(case, backward=True)
        assert _excess(res[0].float().numpy(), t_out) <= 1.0, cfg
        assert np.abs(res[1].numpy() - t_lse).max() <= 1e-3, cfg
        assert _excess(res[2].float().numpy(), t_dq) <= 1.0, cfg
        assert _excess(res[3].float().numpy(), t_dkv) <= 1.0, cfg
        done += 1
    assert done >= 30
