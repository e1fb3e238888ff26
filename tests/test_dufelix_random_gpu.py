"""Dufelix models and traces drawn at random: another order of layers, other sizes, head counts, groups, ranks, taps,
stretched frequencies, constants and seeds every time, run through the engine in a schedule that cuts the requests
into portions of random sizes, runs them side by side with requests left out of steps, and uses pages and slots
again; every row against the plain implementation, in both precisions. How much rounding to bfloat16 alone moves a
model's logits differs from draw to draw (narrow, deep models are touchy), so the bfloat16 bound of a request is taken from
that model itself: the error of the CPU test double run in bfloat16 on the whole prompt, which rounds at the same places."""

import random

import pytest
import torch

import dufelix_util as du
from distie_amd import LLM
from distie_amd.engine.batch import StepEntry
from torch_ops import TorchOps

pytestmark = pytest.mark.gpu


def random_config(rng):
    def mlp():
        return None if rng.random() < 0.25 else du.dense(rng.choice([10, 24, 40, 64]))

    def stretch():
        if rng.random() < 0.3:
            return False
        return du.scaling(factor=rng.choice([2.0, 4.0, 8.0]), original=rng.choice([16, 40, 64]),
                          fast=rng.choice([4.0, 8.0, 32.0]), slow=rng.choice([0.5, 1.0]))

    def attention():
        kv_heads = rng.choice([1, 2, 3])
        dim = rng.choice([8, 12, 16, 32, 48])
        return du.attention(heads=kv_heads * rng.choice([1, 2, 3]), kv_heads=kv_heads, dim=dim, vdim=rng.choice([8, 12, 16, 24, 48]),
                            scale=rng.choice([0.2, 0.35]), dims=rng.choice([0, 2, dim // 2 // 2 * 2, dim]) if dim >= 4 else 0,
                            base=rng.choice([30.0, 1000.0]), scaled=stretch(), mlp=mlp())

    def latent():
        rot_dim = rng.choice([2, 4, 8, 16])
        return du.latent(heads=rng.choice([1, 2, 3, 5]), dim=rng.choice([8, 10, 16, 24]), rot_dim=rot_dim,
                         vdim=rng.choice([8, 14, 16, 40]), kv_rank=rng.choice([8, 18, 24, 48, 100]),
                         q_rank=rng.choice([8, 12, 22, 32]), scale=rng.choice([0.2, 0.3]), base=rng.choice([30.0, 1000.0]),
                         scaled=stretch(), mlp=mlp())

    def mamba():
        groups = rng.choice([1, 2, 3])
        heads = groups * rng.choice([1, 2, 3])
        vdim = rng.choice([4, 8, 10, 16, 24])
        parts = rng.choice([g for g in (1, 2, 3, 4) if (heads * vdim) % g == 0])
        return du.mamba(heads=heads, vdim=vdim, state=rng.choice([4, 8, 12, 16, 40]), groups=groups,
                        conv=rng.choice([1, 2, 3, 4, 5]), norm_groups=parts, mlp=mlp())

    makers = [attention, latent, mamba]
    layers = [rng.choice(makers)() for _ in range(rng.randint(2, 5))]
    for i in range(len(layers)):
        if rng.random() < 0.5:
            layers.append(dict(layers[i], weights_of=i))
    return du.make_config(layers, vocab=rng.choice([33, 50, 64]), width=rng.choice([24, 36, 40, 64]),
                          eps=rng.choice([1e-5, 1e-6]), embed_scale=rng.choice([1.0, 0.5, 6.0]))


@pytest.mark.parametrize("seed", range(10))
def test_random_models_and_traces(tmp_path, seed):
    rng = random.Random(1000 + seed)
    cfg = random_config(rng)
    weights = du.random_weights(cfg, seed=seed, dtype=torch.bfloat16)
    folder = du.write_model(tmp_path / "m", cfg, weights)
    lengths = [rng.choice([1, 2, 5, 17, 40, 70, 100]) for _ in range(6)]
    prompts = [du.random_ids(cfg, n, seed=10 * seed + i) for i, n in enumerate(lengths)]
    want = [du.oracle(cfg, weights, ids) for ids in prompts]
    # steps: up to three requests live, each brings a portion of random size or is left out
    plan, at, waiting, live = [], [0] * len(prompts), list(range(len(prompts))), []
    while waiting or live:
        while waiting and len(live) < 3:
            live.append(waiting.pop(0))
        step = []
        for i in live:
            if len(live) > 1 and rng.random() < 0.2:
                continue
            n = min(len(prompts[i]) - at[i], rng.choice([1, 1, 2, 3, 7, 16, 33, 64]))
            step.append((i, at[i], n))
            at[i] += n
        live = [i for i in live if at[i] < len(prompts[i])]
        if step:
            plan.append(step)
    for dtype in ("float32", "bfloat16"):
        llm = LLM(folder, dtype=dtype, device="cuda:0", block_size=16, num_blocks=24, max_seqs=3, use_graphs=False)
        got = [[] for _ in prompts]
        done = [0] * len(prompts)
        for step in plan:
            logits = llm.step([StepEntry(f"r{i}", prompts[i][a:a + n], list(range(n))) for i, a, n in step]).float().cpu()
            row = 0
            for i, a, n in step:
                got[i].append(logits[row:row + n])
                row += n
                done[i] += n
                if done[i] == len(prompts[i]):
                    llm.finish(f"r{i}")
        tol = du.TOL[torch.float32 if dtype == "float32" else torch.bfloat16]
        double = None
        if dtype == "bfloat16":
            double = LLM(folder, dtype=dtype, device="cpu", ops=TorchOps(), block_size=16, num_blocks=24, max_seqs=3, use_graphs=False)
        for i in range(len(prompts)):
            err = du.logit_error(torch.cat(got[i]), want[i])
            if dtype == "float32":
                assert float(err.max()) < tol, (seed, cfg, i, float(err.max()))
            else:
                rounded = double.step([StepEntry("d", prompts[i], list(range(len(prompts[i]))))]).float()
                double.finish("d")
                bound = max(tol, float(du.logit_error(rounded, want[i]).max()))
                assert float(err.max()) < 2.5 * bound and int((err > bound).sum()) <= max(1, len(err) // 10), \
                    (seed, i, float(err.max()), bound)
        assert not llm.cache.live()
        llm.close()
