"""The Dufelix decoder in the engine against the plain implementation (`plain_dufelix`), on the CPU test double (the
engine's logic: batching, cache, state slots, layers that share tensors, scheduler) and on the GPU (the kernels, float32
and bfloat16).

Models are tiny and their weights random (`dufelix_util.random_weights`); sizes are chosen so that nothing the design
lets differ is equal by accident (dim != vdim != rot_dim, kv_rank != q_rank, heads != kv_heads != groups, a state that
is no multiple of anything), with variants where they are equal or 1.
"""

import json

import pytest
import torch

import dufelix_util as du
import plain_dufelix as plain
from distie_amd import LLM, SamplingParams
from distie_amd.config import ConfigError, config_from_dict
from distie_amd.engine.batch import StepEntry
from distie_amd.engine.model import Model
from torch_ops import TorchOps

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module", params=["cpu", pytest.param("hip", marks=pytest.mark.gpu)])
def ops(request):
    if request.param == "cpu":
        return TorchOps()
    from distie_amd.kernels.hip_ops import HipOps

    return HipOps("cuda:0")


def precisions(ops):
    return ["float32"] if ops.device.type == "cpu" else ["float32", "bfloat16"]


def engine(folder, ops, dtype, **options):
    options.setdefault("block_size", 4 if ops.device.type == "cpu" else 16)
    options.setdefault("num_blocks", 96)
    options.setdefault("max_seqs", 4)
    options.setdefault("use_graphs", False)
    return LLM(folder, dtype=dtype, device=str(ops.device), ops=ops, **options)


def whole(llm, rid, ids):
    out = llm.step([StepEntry(rid, list(ids), list(range(len(ids))))])
    llm.finish(rid)
    return out.float().cpu()


def in_portions(llm, rid, ids, cuts):
    """`ids` in portions of the sizes `cuts`, the rest one token a step; every row's logits."""
    out, at, sizes = [], 0, list(cuts)
    while at < len(ids):
        n = min(sizes.pop(0) if sizes else 1, len(ids) - at)
        out.append(llm.step([StepEntry(rid, list(ids[at:at + n]), list(range(n)))]).float().cpu())
        at += n
    llm.finish(rid)
    return torch.cat(out)


def check(got, want, dtype, what=""):
    """float32: every row within the bound. bfloat16: the norm behind every sub-layer makes a row now and then two or
    three times as sensitive to rounding as the others, so one row in twenty may pass the bound, none 2.5 times it (a
    wrong key, a lost state or a sink left out moves a row by far more)."""
    err = du.logit_error(got, want)
    tol = du.TOL[DTYPES[dtype]]
    worst = f"{what}: error {float(err.max())} at row {int(err.argmax())}"
    if dtype == "float32":
        assert float(err.max()) < tol, worst
    else:
        assert float(err.max()) < 2.5 * tol and int((err > tol).sum()) <= max(1, len(err) // 20), worst


# nothing equal by accident; the fourth and fifth layers are the first and second once more (their tensors, caches and
# states of their own); the last has no feed-forward and turns its whole head with plain frequencies
MIXED = du.make_config([
    du.latent(heads=3, dim=12, rot_dim=8, vdim=20, kv_rank=24, q_rank=28, scale=0.25),
    du.mamba(heads=4, vdim=12, state=8, groups=2, conv=3, norm_groups=2),
    du.attention(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.3, dims=8),
    du.latent(heads=3, dim=12, rot_dim=8, vdim=20, kv_rank=24, q_rank=28, scale=0.25, weights_of=0),
    du.mamba(heads=4, vdim=12, state=8, groups=2, conv=3, norm_groups=2, weights_of=1),
    du.attention(heads=6, kv_heads=3, dim=32, vdim=16, scale=0.2, dims=32, base=5000.0, scaled=False, mlp=None),
], vocab=61, width=48, embed_scale=3.0)

# values that the model above makes different made equal, or 1: one head, every size of latent attention the same, a
# convolution of one tap, one group, one part of the norm, no rotation in attention, an embedding that is not scaled
PLAIN = du.make_config([
    du.mamba(heads=1, vdim=32, state=32, groups=1, conv=1, norm_groups=1),
    du.latent(heads=1, dim=16, rot_dim=16, vdim=16, kv_rank=16, q_rank=16, scale=1.0, scaled=False),
    du.attention(heads=2, kv_heads=2, dim=32, vdim=32, scale=0.25, dims=0),
    du.attention(heads=2, kv_heads=2, dim=32, vdim=32, scale=0.25, dims=0, weights_of=2),
], vocab=40, width=32, embed_scale=1.0)

# sizes that fit no tile: a width of 40, ranks of 18 and 22, five heads on one key/value head, three pairs turned, a
# state of 12 rows in three groups, four taps, a feed-forward of 10
ODD = du.make_config([
    du.attention(heads=5, kv_heads=1, dim=20, vdim=12, scale=0.35, dims=6, base=30.0,
                 scaled=du.scaling(factor=8.0, original=40, fast=4.0, slow=0.5), mlp=du.dense(10)),
    du.mamba(heads=6, vdim=10, state=12, groups=3, conv=4, norm_groups=3, mlp=None),
    du.latent(heads=5, dim=10, rot_dim=6, vdim=14, kv_rank=18, q_rank=22, scale=0.3, base=30.0,
              scaled=du.scaling(factor=8.0, original=40, fast=4.0, slow=0.5), mlp=du.dense(10)),
    du.mamba(heads=6, vdim=10, state=12, groups=3, conv=4, norm_groups=3, mlp=None, weights_of=1),
], vocab=50, width=40, embed_scale=0.5)

CONFIGS = {"mixed": MIXED, "plain": PLAIN, "odd": ODD}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}
    for name, cfg in CONFIGS.items():
        weights = du.random_weights(cfg, seed=3 + len(made), dtype=torch.bfloat16)
        made[name] = (du.write_model(tmp_path_factory.mktemp(name), cfg, weights), cfg, weights)
    return made


def test_configuration_and_tensors():
    for cfg in CONFIGS.values():
        config = config_from_dict(cfg)
        declared = {n: tuple(spec.shape) for n, spec in Model.declare(config.model_spec()).items()}
        assert declared == du.tensor_shapes(cfg)
    spec = config_from_dict(MIXED).model_spec()
    assert spec.layers[3].weights_of == 0 and spec.layers[0].weights_of is None
    assert "feed_forward" not in spec.layers[5].parts and spec.embedding.params["scale"] == 3.0
    model = Model(spec)
    assert model.blocks[3] is model.blocks[0] and model.blocks[4] is model.blocks[1]
    assert len(model.cache_requirements()) == 6
    # the rank of the queries' latent may be left to the tensor's shape
    bare = json.loads(json.dumps(MIXED))
    del bare["layers"][0]["mixer"]["q_rank"], bare["layers"][3]["mixer"]["q_rank"]
    config = config_from_dict(bare).with_tensor_shapes({"l0.mix.dq": (28, 48)})
    assert {n: tuple(s.shape) for n, s in Model.declare(config.model_spec()).items()} == du.tensor_shapes(MIXED)
    with pytest.raises(ConfigError):
        config_from_dict(bare).model_spec()
    # a layer may name a layer that itself names another (the tensors are the last one's), or a later layer, and may
    # leave out the sizes that it has from there
    chain = {**MIXED, "layers": [du.mamba(), du.mamba(weights_of=0), {"type": "mamba2", "weights_of": 1},
                                 {"type": "attention", "weights_of": 4}, du.attention()]}
    spec = config_from_dict(chain).model_spec()
    assert [layer.weights_of for layer in spec.layers] == [None, 0, 0, 4, None]
    model = Model(spec)
    assert model.blocks[2] is model.blocks[0] and model.blocks[3] is model.blocks[4]
    assert {n for n in Model.declare(spec)} == set(du.tensor_shapes({**MIXED, "layers": [du.mamba(), du.mamba(weights_of=0),
                                                                    du.mamba(weights_of=0), du.attention(weights_of=4), du.attention()]}))
    for broken in ({**MIXED, "layers": [du.attention(heads=3, kv_heads=2)]},
                   {**MIXED, "layers": [du.attention(dims=18, dim=16)]},
                   {**MIXED, "layers": [du.latent(rot_dim=7)]},
                   {**MIXED, "layers": [du.mamba(heads=4, groups=3)]},
                   {**MIXED, "layers": [du.mamba(heads=3, vdim=5, groups=1, norm_groups=2)]},
                   {**MIXED, "layers": [du.mamba(), du.mamba(weights_of=1)]},
                   {**MIXED, "layers": [du.mamba(), du.mamba(weights_of=0, state=16)]},
                   {**MIXED, "layers": [du.mamba(), du.latent(weights_of=0)]},
                   {**MIXED, "layers": [du.mamba(mlp={"kind": "moe", "ff": 8})]},
                   {**MIXED, "layers": [{"type": "other", "mixer": {}, "mlp": None}]},
                   {k: v for k, v in MIXED.items() if k != "norm"}):
        with pytest.raises(ConfigError):
            config_from_dict(broken)


def test_stretched_frequencies():
    """The position part's frequencies against the plain ones: kept, divided and blended dimensions all occur, and the
    factor on cosine and sine."""
    from distie_amd.config import PartSpec
    from distie_amd.parts import build_part

    rot = du.rot(16, base=100.0, scaled=du.scaling(factor=4.0, original=32, fast=8.0, slow=1.0))
    want, magnitude = plain.frequencies(rot)
    bare, _ = plain.frequencies({"base": 100.0, "dims": 16})
    ratio = want / bare
    assert float(ratio[0]) == 1.0 and abs(float(ratio[-1]) - 0.25) < 1e-12 and bool(((ratio > 0.26) & (ratio < 0.99)).any())
    part = build_part("position", PartSpec("rope_scaled", "", dict(rot)))
    assert torch.allclose(part.rotary().double(), want, rtol=1e-6, atol=0) and abs(part.rotary_magnitude() - magnitude) < 1e-12


def test_layers_one_by_one(ops, folders):
    """The residual stream behind every layer, through the engine's blocks, against the plain implementation."""
    from distie_amd.parts import ResidualStream, StepContext

    for name in ("mixed", "odd", "plain"):
        folder, cfg, weights = folders[name]
        ids = du.random_ids(cfg, 21, seed=1)
        _, after = plain.forward(cfg, weights, ids)
        llm = engine(folder, ops, "float32")
        llm.cache.add("a")
        llm.cache.reserve("a", len(ids))
        tokens, meta, _ = llm.runner.builder.build([StepEntry("a", ids, [0])])
        stream = ResidualStream(llm.model.embed.forward(ops, tokens, meta))
        ctx = StepContext(meta, torch.float32)
        for i, block in enumerate(llm.model.blocks):
            block.forward(ops, stream, ctx, llm.cache.layer(i), True)
            held = stream.hidden.clone()
            delta, post = stream.lanes["pending"]
            ops.add_normed(held, delta, post.weight, post.eps)
            err = (held.double().cpu() - after[i]).abs().max() / after[i].abs().max()
            assert float(err) < 2e-5, f"{name} layer {i}: {float(err)}"


@pytest.mark.parametrize("name", list(CONFIGS))
def test_prompt_decode_and_portions(ops, folders, name):
    """One prompt whole, token by token, and in portions of several sizes down to two tokens (shorter than the
    convolution's reach): every row's logits against the plain implementation, and the same whatever the cut."""
    folder, cfg, weights = folders[name]
    ids = du.random_ids(cfg, 45, seed=11)
    want = du.oracle(cfg, weights, ids)
    for dtype in precisions(ops):
        llm = engine(folder, ops, dtype)
        runs = {"whole": whole(llm, "a", ids), "token by token": in_portions(llm, "b", ids, []),
                "portions": in_portions(llm, "c", ids, [2, 7, 3, 2, 13, 5, 2, 4]),
                "a long portion, then tokens": in_portions(llm, "d", ids, [29])}
        for what, got in runs.items():
            check(got, want, dtype, f"{name} {dtype} {what}")
        llm.cache.check()
        assert not llm.cache.live()


def test_portions_around_the_scans_chunks(ops, folders):
    """Portions that end just before, at and just behind the multiples of 64 rows in which a long portion's state is
    scanned, and short ones between them: the state handed from chunk to chunk, from portion to portion and on to
    decoding."""
    folder, cfg, weights = folders["mixed"]
    ids = du.random_ids(cfg, 300, seed=12)
    want = du.oracle(cfg, weights, ids)
    for dtype in precisions(ops):
        llm = engine(folder, ops, dtype, num_blocks=160)
        check(whole(llm, "a", ids), want, dtype, f"whole {dtype}")
        check(in_portions(llm, "b", ids, [63, 2, 64, 65, 33, 2, 32, 31]), want, dtype, f"portions {dtype}")
        check(in_portions(llm, "c", ids, [129, 128]), want, dtype, f"long portions {dtype}")
        llm.cache.check()


def test_unequal_batches_and_reuse(ops, folders):
    """Requests of unequal length side by side, portions beside single tokens, some left out of a step; more requests
    than state slots one after the other, so that pages and slots are used again with what the last owner left."""
    folder, cfg, weights = folders["mixed"]
    prompts = {i: du.random_ids(cfg, n, seed=20 + i) for i, n in enumerate([31, 6, 19, 2, 70, 1, 23, 12])}
    want = {i: du.oracle(cfg, weights, ids) for i, ids in prompts.items()}
    for dtype in precisions(ops):
        llm = engine(folder, ops, dtype, num_blocks=48, max_seqs=3)
        at = {i: 0 for i in prompts}
        got = {i: [] for i in prompts}
        waiting, live, turn = list(prompts), [], 0
        while waiting or live:
            while waiting and len(live) < 3:
                live.append(waiting.pop(0))
            entries = []
            for slot, i in enumerate(live):
                if (turn + slot) % 4 == 3 and len(live) > 1:
                    continue                                  # left out of this step
                left = len(prompts[i]) - at[i]
                n = min(left, [1, 5, 2, 37][(turn + i) % 4])
                entries.append((i, n))
            logits = llm.step([StepEntry(f"r{i}", prompts[i][at[i]:at[i] + n], list(range(n))) for i, n in entries])
            row = 0
            for i, n in entries:
                got[i].append(logits[row:row + n].float().cpu())
                row += n
                at[i] += n
                if at[i] == len(prompts[i]):
                    llm.finish(f"r{i}")
                    live.remove(i)
            llm.cache.check()
            turn += 1
        for i in prompts:
            check(torch.cat(got[i]), want[i], dtype, f"request {i} {dtype}")
        assert not llm.cache.live() and llm.cache.free_pages() == [48] * len(llm.cache.groups)


def planted(cfg, weights, token_a, token_b):
    """Make what token `token_a` leaves in layer 0 stand out for token `token_b`, at any distance. The embeddings get
    two channels of their own: only a has a value in the first, only b in the second, so only a's and b's rows of the
    layer's input are non-zero there.

    latent attention: the first row of the keys' down-projection reads the first channel alone, the first row of the
    queries' the second alone; behind their norms only a's latent and only b's have a first entry. The key expansion
    spreads the latent's first entry over every head's unrotated dimensions, the query expansion likewise, the value
    expansion makes a's value large: b's score for a is large whatever lies between them, no other pair changes.
    attention: the same through the rows of k and q that the rotation leaves alone.
    mamba2: a's step size is made large (its rows of the projection read the first channel), so what a writes into the
    state outweighs hundreds of later tokens; the decay is made slow."""
    w = {k: v.clone().float() for k, v in weights.items()}
    layer = cfg["layers"][0]
    m = layer["mixer"]
    w["embed"][:, :2] = 0.0
    w["embed"][token_a, 0] = 4.0
    w["embed"][token_b, 1] = 4.0
    w["l0.norm1"][:2] = 1.0
    if layer["type"] == "latent_attention":
        H, D, R, E = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
        for name, channel in (("l0.mix.dkv", 0), ("l0.mix.dq", 1)):
            w[name][0] = 0.0
            w[name][0, channel] = 3.0
            w[name][1:, :2] = 0.0
        w["l0.mix.dkv.norm"][0] = w["l0.mix.dq.norm"][0] = 1.0
        for h in range(H):
            w["l0.mix.uk"][h * D:(h + 1) * D, 0] = 1.6
            w["l0.mix.uq"][h * (D + R):h * (D + R) + D, 0] = 1.6
            w["l0.mix.uv"][h * E:(h + 1) * E, 0] = 2.0
        w["l0.mix.sink"].fill_(0.5)
    elif layer["type"] == "attention":
        H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        turned = int((m.get("rot") or {}).get("dims", 0))
        for name in ("l0.mix.q", "l0.mix.k", "l0.mix.v", "l0.mix.g"):
            w[name][:, :2] = 0.0
        for g in range(G):
            w["l0.mix.k"][g * D + turned:(g + 1) * D, 0] = 3.0
            w["l0.mix.v"][g * E:(g + 1) * E, 0] = 4.0
        for h in range(H):
            w["l0.mix.q"][h * D + turned:(h + 1) * D, 1] = 3.0
    else:
        H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
        inner = H * P
        w["l0.mix.in"][:, :2] = 0.0
        w["l0.mix.in"][2 * inner + 2 * G * N:, 0] = 4.0          # a's step size
        w["l0.mix.in"][inner:2 * inner, 0] = 1.0                 # and its x
        w["l0.mix.A_log"].fill_(-7.0)
        w["l0.mix.dt_bias"].fill_(-3.0)
    return {k: v.to(torch.bfloat16) for k, v in w.items()}


FAR = {
    "latent": du.make_config([du.latent(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=24, q_rank=20, scale=0.3, base=1000.0),
                              du.mamba(heads=2, vdim=16, state=8, groups=1, conv=2, norm_groups=1, mlp=None)],
                             vocab=30, width=32, embed_scale=1.0),
    "attention": du.make_config([du.attention(heads=2, kv_heads=1, dim=32, vdim=16, scale=0.3, dims=8, base=1000.0),
                                 du.latent(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=24, q_rank=20, scale=0.3, mlp=None)],
                                vocab=30, width=32, embed_scale=1.0),
    "mamba2": du.make_config([du.mamba(heads=2, vdim=16, state=8, groups=1, conv=2, norm_groups=1),
                              du.attention(heads=2, kv_heads=1, dim=32, vdim=16, scale=0.3, dims=8, mlp=None)],
                             vocab=30, width=32, embed_scale=1.0),
}


@pytest.mark.parametrize("kind", list(FAR))
def test_a_far_token_among_hundreds(ops, tmp_path, kind):
    """What token A leaves behind (a key and value in the cache, or its mark on the state) stands out for token B. A
    lies hundreds of tokens back: the very first token, or the last of a page, or the first of the next; B asks for it
    in a prompt, in a later portion and in decoding. A lost or mixed-up page, or a state that is dropped between
    portions, moves the logits there by far more than the tolerance, which the plain implementation shows with A
    taken out."""
    A, B = 7, 11
    cfg = FAR[kind]
    weights = planted(cfg, du.random_weights(cfg, seed=9, dtype=torch.float32), A, B)
    folder = du.write_model(tmp_path / "far", cfg, weights)
    filler = [t for t in du.random_ids(cfg, 900, seed=2) if t not in (A, B)]
    for first in (0, 15, 16, 63, 64):
        ids = filler[:420]
        ids[first] = A
        asks = [first + 1, 200, 255, 256, 300, 383, 384, 385, 419]
        for at in asks:
            ids[at] = B
        want = du.oracle(cfg, weights, ids)
        without = du.oracle(cfg, weights, ids[:first] + [filler[500]] + ids[first + 1:])
        assert float(du.logit_error(without, want)[asks].min()) > 2 * du.TOL[torch.bfloat16], kind
        for dtype in precisions(ops):
            llm = engine(folder, ops, dtype, block_size=16, num_blocks=30)
            check(whole(llm, "a", ids)[asks], want[asks], dtype, f"prompt, A at {first}, {dtype}")
            got = in_portions(llm, "b", ids, [first + 1, 2, 197 - first, 56, 2, 120])
            check(got[asks], want[asks], dtype, f"portions, then decoding, A at {first}, {dtype}")


def test_the_sink_counts(ops, folders):
    """Without its sinks the model's logits differ by far more than the tolerance (so a sink that is left out shows),
    and the engine agrees with the plain implementation where the sinks are large."""
    folder, cfg, weights = folders["mixed"]
    ids = du.random_ids(cfg, 30, seed=5)
    loud = {k: (v.float() + 3.0).to(v.dtype) if k.endswith("sink") else v for k, v in weights.items()}
    mute = {k: torch.full_like(v, -30.0) if k.endswith("sink") else v for k, v in weights.items()}
    want = du.oracle(cfg, loud, ids)
    # (not at the first token: what a sink takes from the only key's weight, the norm behind the mixer gives back)
    assert float(du.logit_error(du.oracle(cfg, mute, ids), want)[4:].median()) > 2 * du.TOL[torch.bfloat16]
    loud_folder = du.write_model(folder.parent / "loud", cfg, loud)
    for dtype in precisions(ops):
        llm = engine(loud_folder, ops, dtype)
        check(whole(llm, "a", ids), want, dtype, f"prompt {dtype}")
        check(in_portions(llm, "b", ids, [1, 1, 6]), want, dtype, f"first tokens one by one {dtype}")


def test_first_tokens_and_long_decoding(ops, folders):
    """The first tokens of a sequence one by one (a token that sees only itself and the sink; a convolution that reaches
    back before the start), then decoding for hundreds of tokens across many pages."""
    for name in ("mixed", "odd"):
        folder, cfg, weights = folders[name]
        ids = du.random_ids(cfg, 150, seed=31)
        want = du.oracle(cfg, weights, ids)
        for dtype in precisions(ops):
            llm = engine(folder, ops, dtype, num_blocks=48)
            got = in_portions(llm, "a", ids, [1, 1, 1, 2])
            check(got, want, dtype, f"{name} long decoding {dtype}")
            llm.cache.check()
            assert not llm.cache.live()


def test_greedy_generation_through_the_scheduler(ops, folders):
    """`LLM.generate`: continuous batching with a token budget that cuts the prompts, more requests than seats, and
    (on the GPU) captured decode steps. Every token is the plain implementation's greedy pick given what came before,
    or a near tie."""
    for name, dtypes in (("mixed", precisions(ops)), ("odd", ["float32"])):
        folder, cfg, weights = folders[name]
        prompts = [du.random_ids(cfg, n, seed=40 + n) for n in (23, 5, 14, 9, 2)]
        for dtype in dtypes:
            llm = engine(folder, ops, dtype, num_blocks=64, max_seqs=3, token_budget=16,
                         use_graphs=ops.device.type != "cpu")
            outs = llm.generate(prompts, SamplingParams(max_new_tokens=12))
            slack = 1e-3 if dtype == "float32" else 0.35
            for prompt, out in zip(prompts, outs):
                assert len(out.token_ids) == 12
                ids = list(prompt)
                for token in out.token_ids:
                    logits = du.oracle(cfg, weights, ids)[-1]
                    assert float(logits[token]) >= float(logits.max()) - slack * float(logits.abs().max()), (dtype, out.token_ids)
                    ids.append(token)
            assert not llm.cache.live()
            llm.close()


def test_random_model_folder_reads_back(tmp_path):
    """`random-model` of the command line writes a folder that the loader takes, tensor for tensor as the design
    names them (a layer that uses another's tensors adds none)."""
    from distie_amd import cli
    from distie_amd.weights.safetensors_io import SafetensorsFile

    (tmp_path / "config.json").write_text(json.dumps(ODD))
    assert cli.main(["random-model", "--config-json", str(tmp_path / "config.json"), "--out", str(tmp_path / "m"),
                     "--seed", "3", "--dtype", "bf16", "--std", "0.1"]) == 0
    stored = SafetensorsFile(tmp_path / "m" / "model.safetensors")
    assert {name: tuple(entry[1]) for name, entry in stored.index.items()} == du.tensor_shapes(ODD)
    stored.close()
    llm = engine(tmp_path / "m", TorchOps(), "float32")
    assert llm.step([StepEntry("a", [1, 2, 3], [2])]).shape == (1, ODD["vocab"])


@pytest.mark.gpu
def test_trace_runner_and_command_line(folders, tmp_path):
    """The trace runner as a program (its own process, steps on standard input, four requests live, pages and
    slots used again) and `generate` of the command line, on a Dufelix model, against the plain implementation."""
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    root = Path(__file__).resolve().parents[1]
    folder, cfg, weights = folders["mixed"]
    lengths = {"p": 70, "q": 33, "r": 64, "s": 5, "t": 50, "u": 21}
    reqs = {r: du.random_ids(cfg, n, 60 + n) for r, n in lengths.items()}
    want = {r: du.oracle(cfg, weights, ids) for r, ids in reqs.items()}
    max_tokens = sum(-(-n // 64) * 64 for n in sorted(lengths.values())[-4:])
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / dtype
        proc = subprocess.Popen([sys.executable, str(root / "bin" / "trace_run"), "--model", str(folder), "--dtype", dtype,
                                 "--out", str(out), "--max-tokens", str(max_tokens)],
                                stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
        got, at = {r: [] for r in reqs}, {r: 0 for r in reqs}
        waiting, live, step = list(reqs), [], 0
        while waiting or live:
            while waiting and len(live) < 4:
                live.append(waiting.pop(0))
            entries, end = [], []
            for k, r in enumerate(live):
                left = len(reqs[r]) - at[r]
                n = min(left, 1 if left <= 8 else [13, 2, 30, 7][(step + k) % 4])
                entries.append({"id": r, "tokens": reqs[r][at[r]:at[r] + n], "want": list(range(n))})
                at[r] += n
                if at[r] == len(reqs[r]):
                    end.append(r)
            proc.stdin.write(json.dumps({"step": step, "entries": entries, "end": end}) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {step}"
            rows = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(-1, cfg["vocab"]).copy())
            row = 0
            for e in entries:
                got[e["id"]].append(rows[row:row + len(e["tokens"])])
                row += len(e["tokens"])
            live = [r for r in live if r not in end]
            step += 1
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
        for r in reqs:
            check(torch.cat(got[r]), want[r], dtype, f"request {r} {dtype}")
    prompts = [reqs["s"], reqs["q"][:9]]
    (tmp_path / "prompts.json").write_text(json.dumps(prompts))
    done = subprocess.run([sys.executable, "-m", "distie_amd.cli", "generate", "--model", str(folder), "--dtype", "fp32",
                           "--prompts", str(tmp_path / "prompts.json"), "--max-new-tokens", "6", "--num-blocks", "32",
                           "--out", str(tmp_path / "report.json")], cwd=str(root), capture_output=True, text=True, timeout=110)
    assert done.returncode == 0, done.stderr
    for prompt, record in zip(prompts, json.loads((tmp_path / "report.json").read_text())):
        ids = list(prompt)
        for token in record["token_ids"]:
            logits = du.oracle(cfg, weights, ids)[-1]
            assert float(logits[token]) >= float(logits.max()) - 1e-3 * float(logits.abs().max())
            ids.append(token)


def test_preemption_recomputes(ops, folders):
    """So few pages that running requests are preempted and recomputed (their states start from zero again): every
    token still is the plain implementation's pick."""
    folder, cfg, weights = folders["plain"]
    prompts = [du.random_ids(cfg, n, seed=70 + n) for n in (20, 26, 17)]
    block = 4 if ops.device.type == "cpu" else 16
    new = 24 if block == 4 else 40
    llm = engine(folder, ops, "float32", block_size=block, num_blocks=-(-(26 + new) // block) + 1, max_seqs=3, token_budget=32)
    outs = llm.generate(prompts, SamplingParams(max_new_tokens=new))
    assert sum(o.preemptions for o in outs) > 0, "the pool was not small enough to preempt anybody"
    for prompt, out in zip(prompts, outs):
        ids = list(prompt)
        for token in out.token_ids:
            logits = du.oracle(cfg, weights, ids)[-1]
            assert float(logits[token]) >= float(logits.max()) - 1e-3 * float(logits.abs().max())
            ids.append(token)
    llm.cache.check()
    assert not llm.cache.live()
