"""Random Malinex configurations (layer order, head counts, key / value sizes, decay ranks and temperatures,
temperature steps, experts, layers that share weights) under random schedules (up to four live requests,
portions of 1..300 tokens beside decoded tokens, a pool with little room to spare) against the plain
implementation.  fp32 is compared with a tight bound at every position; bf16 runs without routed experts
and is bounded on the median and on nine positions in ten (see ``test_malinex``)."""

import random

import pytest
import torch

from tests.models import malinex_util as U
from tests.models.test_lenitar_random import random_schedule
from tests.oracles import malinex_plain as plain


def random_config(r, experts=True):
    width, vocab = r.choice([24, 40, 64, 96]), r.choice([40, 100, 130])
    layers, share = [], {}
    for i in range(r.choice([2, 3, 4, 5])):
        if r.random() < 0.55:
            mix = U.gla(heads=r.choice([1, 2, 3, 6]), dim=r.choice([4, 12, 16, 40, 64, 72, 136]), vdim=r.choice([8, 16, 64, 72, 130]),
                        tau=r.choice([1.0, 4.0, 12.0, 32.0]), rank=r.choice([1, 4, 16, 24]))
        else:
            G = r.choice([1, 2, 3, 4])
            mix = U.att(heads=G * r.choice([1, 2, 4]), kv_heads=G, dim=r.choice([8, 16, 24, 64, 128]), vdim=r.choice([8, 16, 40, 64, 128]),
                        scale=r.choice([0.1, 0.3, 1.0]), coef=r.choice([None, 0.2, 1.0]), every=r.choice([1, 16, 100, 1000]))
        kind = r.random()
        if kind < 0.25:
            ff = None
        elif kind < 0.55 or not experts:
            ff = U.dense(r.choice([8, 40, 100]))
        else:
            E = r.choice([2, 4, 5, 8, 16])
            ff = U.moe(experts=E, top=r.randint(1, min(E, 4)), ff=r.choice([8, 16, 24]), shared=r.choice([0, 8, 20]))
        layers.append((mix, ff))
        earlier = [j for j in range(i) if j not in share and layers[j][0]["type"] == mix["type"]]
        if earlier and r.random() < 0.3:
            share[i] = r.choice(earlier)
    return U.config(layers, width=width, vocab=vocab, eps=r.choice([1e-6, 1e-5]), logit_scale=r.choice([0.5, 1.0, 2.0]),
                    max_positions=440, share=share)


def run_case(tmp_path, seed, device, dtype, tol, experts):
    r = random.Random(seed)
    cfg = random_config(r, experts)
    W = {k: v.bfloat16().float() for k, v in U.random_weights(cfg, seed).items()}
    reqs = {f"q{j}": [r.randrange(cfg["vocab"]) for _ in range(r.choice([1, 2, 5, 40, 150, 420]))]
            for j in range(r.choice([1, 3, 6]))}
    steps = random_schedule(r, reqs)
    total = sum(len(t) for t in reqs.values())
    eng = U.engine(U.write_checkpoint(tmp_path / "ck", U.clean(cfg), W), device, dtype, blocks=total // 16 + 12, block_size=16)
    got = U.run_schedule(eng, reqs, steps)
    eng.close()
    errs = {rid: U.rel_errs(got[rid], plain.forward(cfg, W, toks).float()) for rid, toks in reqs.items()}
    if dtype == torch.bfloat16:
        per = torch.cat(list(errs.values()))
        assert float(per.median()) < tol / 2 and float(per.quantile(0.9)) < 2 * tol and float(per.max()) < 1.0, (seed, per.median(), per.max())
    else:
        for rid, per in errs.items():
            assert float(per.max()) < tol, (seed, rid, float(per.max()), int(per.argmax()))


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_configurations_cpu(tmp_path, seed):
    run_case(tmp_path, seed, "cpu", torch.float32, 3e-4, True)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", list(range(100, 116)))
def test_random_configurations_gpu(tmp_path, seed):
    run_case(tmp_path, seed, "cuda", torch.float32, 3e-4, True)
    run_case(tmp_path, seed + 1000, "cuda", torch.bfloat16, 0.1, False)
