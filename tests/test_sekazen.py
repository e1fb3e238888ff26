"""The Sekazen decoder in the engine against the plain implementation (`plain_sekazen`), on the CPU test double
(the engine's logic: batching, cache, windows, borrowed keys, scheduler) and on the GPU (the kernels, float32 and
bfloat16).

Models are tiny and their weights random (`sekazen_util.random_weights`); sizes are chosen so that nothing the design
lets differ is equal by accident (dim != vdim, heads != kv_heads, windows that are no multiple of a page and differ
between a layer and the layer that borrows its keys, a rotation of part of a head), with variants where they are
equal or 1.
"""

import json

import pytest
import torch

import plain_sekazen as plain
import sekazen_util as su
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
    wrong key, window or expert moves a row by far more)."""
    err = su.logit_error(got, want)
    tol = su.TOL[DTYPES[dtype]]
    worst = f"{what}: error {float(err.max())} at row {int(err.argmax())}"
    if dtype == "float32":
        assert float(err.max()) < tol, worst
    else:
        assert float(err.max()) < 2.5 * tol and int((err > tol).sum()) <= max(1, len(err) // 20), worst


# nothing equal by accident: keys of 16 and values of 24 (a head size of 32 in the kernels), windows of 9 and 13 on a
# layer and its borrower, half a head turned with scaled frequencies; then a pair without a window, wholly turned with
# plain frequencies, the lender without a feed-forward, the borrower with a window of its own and three experts a token
MIXED = su.make_config([
    su.layer(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.3, window=9, dims=8, base=100.0, scaled=True),
    su.layer(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.45, window=13, dims=8, base=100.0, scaled=True, kv_from=0,
             mlp=su.moe(experts=4, top=1, ff=16, limit=0.75)),
    su.layer(heads=6, kv_heads=3, dim=32, vdim=16, scale=0.2, window=None, dims=32, base=5000.0, scaled=False, mlp=None),
    su.layer(heads=6, kv_heads=3, dim=32, vdim=16, scale=0.15, window=5, dims=32, base=5000.0, scaled=False, kv_from=2,
             mlp=su.moe(experts=5, top=3, ff=16, limit=2.0)),
], vocab=61, width=48, cap=6.0)

# values that the model above makes different made equal, or 1: one head, dim == vdim == the kernels' head size, a
# window of one token (a token sees itself and the sink), no rotation in one layer, one expert of one, every expert
# chosen, logits without a cap
PLAIN = su.make_config([
    su.layer(heads=1, kv_heads=1, dim=32, vdim=32, scale=1.0, window=1, dims=0, mlp=su.moe(experts=1, top=1, ff=8, limit=1.0)),
    su.layer(heads=2, kv_heads=2, dim=32, vdim=32, scale=0.25, window=64, dims=2, base=2.0, scaled=False,
             mlp=su.moe(experts=3, top=3, ff=8, limit=1.0)),
    su.layer(heads=2, kv_heads=2, dim=32, vdim=32, scale=0.25, window=None, dims=2, base=2.0, scaled=False, kv_from=1,
             mlp=None),
], vocab=40, width=32, cap=None)

# sizes that fit no tile: a width of 40, keys of 20 and values of 12, five heads on one key/value head, three pairs
# turned, experts of 10
ODD = su.make_config([
    su.layer(heads=5, kv_heads=1, dim=20, vdim=12, scale=0.35, window=17, dims=6, base=30.0,
             scaled=su.scaling(factor=8.0, low=0.5, high=3.0, original=40), mlp=su.moe(experts=7, top=2, ff=10, limit=1.5)),
    su.layer(heads=5, kv_heads=1, dim=20, vdim=12, scale=0.35, window=3, dims=6, base=30.0,
             scaled=su.scaling(factor=8.0, low=0.5, high=3.0, original=40), kv_from=0, mlp=su.moe(experts=2, top=1, ff=6)),
], vocab=50, width=40, cap=20.0)

CONFIGS = {"mixed": MIXED, "plain": PLAIN, "odd": ODD}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}
    for name, cfg in CONFIGS.items():
        weights = su.random_weights(cfg, seed=3 + len(made), dtype=torch.bfloat16)
        made[name] = (su.write_model(tmp_path_factory.mktemp(name), cfg, weights), cfg, weights)
    return made


def test_configuration_and_tensors():
    for cfg in CONFIGS.values():
        config = config_from_dict(cfg)
        declared = {n: tuple(spec.shape) for n, spec in Model.declare(config.model_spec()).items()}
        assert declared == su.tensor_shapes(cfg)
    spec = config_from_dict(MIXED).model_spec()
    assert "feed_forward" not in spec.layers[2].parts and spec.head.params["cap"] == 6.0
    # a lender keeps its pages for as long as the widest window among itself and its borrowers looks back
    assert spec.layers[0].parts["mixer"].params["keep"] == 13 and spec.layers[2].parts["mixer"].params["keep"] is None
    assert config_from_dict(PLAIN).model_spec().layers[1].parts["mixer"].params["keep"] is None
    for broken in ({**MIXED, "layers": [su.layer(heads=3, kv_heads=2)]},
                   {**MIXED, "layers": [su.layer(dims=18, dim=16)]},
                   {**MIXED, "layers": [su.layer(mlp=su.moe(experts=2, top=3))]},
                   {**MIXED, "layers": [su.layer(), su.layer(kv_from=1)]},
                   {**MIXED, "layers": [su.layer(), su.layer(kv_from=0), su.layer(kv_from=1)]},
                   {**MIXED, "layers": [su.layer(), su.layer(kv_from=0, dim=32)]},
                   {**MIXED, "layers": [{"type": "other", "mixer": {}, "mlp": None}]},
                   {k: v for k, v in MIXED.items() if k != "norm"}):
        with pytest.raises(ConfigError):
            config_from_dict(broken)


def test_frequency_bands():
    """The position part's frequencies against the plain ones: kept, divided and blended bands all occur."""
    from distie_amd.config import PartSpec
    from distie_amd.parts import build_part

    rot = {"base": 100.0, "dims": 16, "scaling": su.scaling(factor=4.0, low=1.0, high=4.0, original=64)}
    want = plain.frequencies(rot)
    plain_f = plain.frequencies({"base": 100.0, "dims": 16})
    ratio = want / plain_f
    assert float(ratio[0]) == 1.0 and abs(float(ratio[-1]) - 0.25) < 1e-12 and bool(((ratio > 0.26) & (ratio < 0.99)).any())
    part = build_part("position", PartSpec("rope_banded", "", dict(rot)))
    assert torch.equal(part.rotary(), want.float())
    assert torch.equal(build_part("position", PartSpec("rope_banded", "", {"base": 100.0, "dims": 16})).rotary(), plain_f.float())


def test_layers_one_by_one(ops, folders):
    """The residual stream behind every layer, through the engine's blocks, against the plain implementation."""
    from distie_amd.parts import ResidualStream, StepContext

    for name in ("mixed", "odd"):
        folder, cfg, weights = folders[name]
        ids = su.clear_ids(cfg, weights, 21, seed=1)
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
    """One prompt whole, token by token, and in portions of several sizes down to two tokens: every row's logits
    against the plain implementation, and the same whatever the cut (beyond rounding). The prompt is longer than every
    window, so decoding passes them all."""
    folder, cfg, weights = folders[name]
    ids = su.clear_ids(cfg, weights, 45, seed=11)
    want = su.oracle(cfg, weights, ids)
    for dtype in precisions(ops):
        llm = engine(folder, ops, dtype)
        runs = {"whole": whole(llm, "a", ids), "token by token": in_portions(llm, "b", ids, []),
                "portions": in_portions(llm, "c", ids, [2, 7, 3, 2, 13, 5, 2, 4]),
                "a long portion, then tokens": in_portions(llm, "d", ids, [29])}
        for what, got in runs.items():
            check(got, want, dtype, f"{name} {dtype} {what}")
        llm.cache.check()
        assert not llm.cache.live()


def test_unequal_batches_and_reuse(ops, folders):
    """Requests of unequal length side by side, portions beside single tokens, some left out of a step; more requests
    than state slots one after the other, so that pages and slots are used again with what the last owner left."""
    folder, cfg, weights = folders["mixed"]
    prompts = {i: su.clear_ids(cfg, weights, n, seed=20 + i) for i, n in enumerate([31, 6, 19, 2, 40, 1, 23, 12])}
    want = {i: su.oracle(cfg, weights, ids) for i, ids in prompts.items()}
    for dtype in precisions(ops):
        llm = engine(folder, ops, dtype, num_blocks=40, max_seqs=3)
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
                n = min(left, [1, 5, 2, 9][(turn + i) % 4])
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
        assert not llm.cache.live() and llm.cache.free_pages() == [40] * len(llm.cache.groups)


def planted(cfg, weights, token_a, token_b):
    """Make the key of token `token_a` stand out for queries of token `token_b` in layer 0, wherever b sees a. The
    embeddings get two channels of their own: only a has a value in the first, only b in the second. The key's
    projection reads the first channel, the query's the second, into the dimensions of a head that the rotation leaves
    alone, with a component far larger than the rest: behind the heads' norms a's key and b's query are close to the
    same direction and their score is close to (dim - turned) / dim * dim * scale whatever their distance, while no
    other token's key or query changes. a's value is made large."""
    w = {k: v.clone().float() for k, v in weights.items()}
    m = cfg["layers"][0]["mixer"]
    D, E, H, G = m["dim"], m["vdim"], m["heads"], m["kv_heads"]
    turned = int((m.get("rot") or {}).get("dims", 0))
    eps = cfg["norm"]["eps"]
    w["embed"][:, :2] = 0.0
    w["embed"][token_a, 0] = 4.0
    w["embed"][token_b, 1] = 4.0
    read = lambda token: plain.norm_one_plus(w["embed"][token].double(), w["embed.norm"].double(), eps).float()
    ha, hb = float(read(token_a)[0]), float(read(token_b)[1])
    w["l0.mix.q.norm"].fill_(1.0)
    w["l0.mix.k.norm"].fill_(1.0)
    for g in range(G):
        w["l0.mix.k"][g * D + turned:(g + 1) * D, 0] += 40.0 / ha
        w["l0.mix.v"][g * E:(g + 1) * E, 0] += 6.0 / ha
    for h in range(H):
        w["l0.mix.q"][h * D + turned:(h + 1) * D, 1] += 40.0 / hb
    return {k: v.to(torch.bfloat16) for k, v in w.items()}


FAR = su.make_config([
    su.layer(heads=2, kv_heads=1, dim=32, vdim=16, scale=0.4, window=None, dims=8, base=1000.0, scaled=True,
             mlp=su.moe(experts=3, top=3, ff=16, limit=1.5)),
], vocab=30, width=32)


def test_a_far_key_among_hundreds(ops, tmp_path):
    """Token A's key and value stand out for queries of token B, on a layer without a window. A lies hundreds of tokens
    back: the very first token, or the last of a page, or the first of the next; B asks for it in a prompt, in a later
    portion and in decoding. A lost or mixed-up page moves the logits there by far more than the tolerance, which the
    plain implementation shows with A taken out."""
    A, B = 7, 11
    weights = planted(FAR, su.random_weights(FAR, seed=9, dtype=torch.float32), A, B)
    folder = su.write_model(tmp_path / "far", FAR, weights)
    filler = [t for t in su.random_ids(FAR, 900, seed=2) if t not in (A, B)]
    for first in (0, 15, 16, 63, 64):
        ids = filler[:420]
        ids[first] = A
        asks = [first + 1, 200, 255, 256, 300, 383, 384, 385, 419]
        for at in asks:
            ids[at] = B
        want = su.oracle(FAR, weights, ids)
        without = su.oracle(FAR, weights, ids[:first] + [filler[500]] + ids[first + 1:])
        assert float(su.logit_error(without, want)[asks].min()) > 2 * su.TOL[torch.bfloat16]
        for dtype in precisions(ops):
            llm = engine(folder, ops, dtype, block_size=16, num_blocks=30)
            check(whole(llm, "a", ids)[asks], want[asks], dtype, f"prompt, A at {first}, {dtype}")
            got = in_portions(llm, "b", ids, [first + 1, 2, 197 - first, 56, 2, 120])
            check(got[asks], want[asks], dtype, f"portions, then decoding, A at {first}, {dtype}")


def edge_config(window, second):
    return su.make_config([
        su.layer(heads=2, kv_heads=1, dim=32, vdim=16, scale=0.4, window=window, dims=8, base=1000.0, scaled=True,
                 mlp=su.moe(experts=3, top=3, ff=16, limit=1.5)),
        su.layer(heads=2, kv_heads=1, dim=32, vdim=16, scale=0.4, window=second, dims=8, base=1000.0, scaled=True,
                 kv_from=0, mlp=None),
    ], vocab=30, width=32)


@pytest.mark.parametrize("window", [37, 64])
def test_a_key_at_the_windows_edge(ops, tmp_path, window):
    """Token A's key stands out for queries of token B. B stands window - 1 tokens behind an A (the last place that
    sees it) and window tokens behind another (the first that does not), in a prompt, at the start and the end of a
    portion and decoded alone, with A's page partly behind the window. A window one token wider or narrower changes
    these rows by far more than the tolerance, which the plain implementation shows. The second layer borrows the
    first layer's keys with a wider window, so the lender keeps its pages for longer than its own window asks."""
    A, B = 7, 11
    cfg = edge_config(window, window + 20)
    weights = planted(cfg, su.random_weights(cfg, seed=5, dtype=torch.float32), A, B)
    folder = su.write_model(tmp_path / f"edge{window}", cfg, weights)
    filler = [t for t in su.random_ids(cfg, 900, seed=3) if t not in (A, B)]
    starts = [3 + k * (window + 11) for k in range(6)]          # no B sees two As
    ids = filler[:starts[-1] + window + 30]
    inside, outside = [], []
    for k, a in enumerate(starts):
        gap = window - 1 if k % 2 == 0 else window
        ids[a] = A
        ids[a + gap] = B
        (inside if gap == window - 1 else outside).append(a + gap)
    asks = sorted(inside + outside)
    want = su.oracle(cfg, weights, ids)
    for other in (window - 1, window + 1):
        moved = su.oracle(edge_config(other, window + 20), weights, ids)
        rows = inside if other < window else outside
        assert float(su.logit_error(moved, want)[rows].min()) > 2 * su.TOL[torch.bfloat16], (window, other)
    # portions whose starts and ends fall on the asking places; from just before the fifth of them on, token by token
    cuts, at = [], 0
    for stop in (asks[0], asks[0] + 1, asks[1], asks[2] + 1, asks[3], asks[4] - 2):
        cuts.append(stop - at)
        at = stop
    for dtype in precisions(ops):
        llm = engine(folder, ops, dtype, block_size=16, num_blocks=30)
        check(whole(llm, "a", ids)[asks], want[asks], dtype, f"prompt, window {window}, {dtype}")
        got = in_portions(llm, "b", ids, cuts)
        check(got[asks], want[asks], dtype, f"portions, then decoding, window {window}, {dtype}")
        check(got[-60:], want[-60:], dtype, f"decoding past the window {window}, {dtype}")
        llm.cache.check()


def test_first_tokens_and_long_decoding(ops, folders):
    """The first tokens of a sequence one by one (a token that sees only itself and the sink), then decoding for
    several windows' lengths: the windowed group gives the pages behind its windows back on the way (the pair of
    layers without a window keeps all of its own) and the logits stay right."""
    folder, cfg, weights = folders["mixed"]
    ids = su.clear_ids(cfg, weights, 150, seed=31)
    want = su.oracle(cfg, weights, ids)
    for dtype in precisions(ops):
        llm = engine(folder, ops, dtype, num_blocks=40)
        got = in_portions(llm, "a", ids, [1, 1, 1, 2])
        check(got, want, dtype, f"long decoding {dtype}")
        llm.cache.check()
        assert not llm.cache.live()


def test_greedy_generation_through_the_scheduler(ops, folders):
    """`LLM.generate`: continuous batching with a token budget that cuts the prompts, more requests than seats, and
    (on the GPU) captured decode steps. Every token is the plain implementation's greedy pick given what came before,
    or a near tie. bfloat16 on the model whose routing does not hang on a close call (every expert chosen)."""
    for name, dtypes in (("mixed", ["float32"]), ("plain", precisions(ops))):
        folder, cfg, weights = folders[name]
        prompts = [su.random_ids(cfg, n, seed=40 + n) for n in (23, 5, 14, 9, 2)]
        for dtype in dtypes:
            llm = engine(folder, ops, dtype, num_blocks=64, max_seqs=3, token_budget=16,
                         use_graphs=ops.device.type != "cpu")
            outs = llm.generate(prompts, SamplingParams(max_new_tokens=12))
            slack = 1e-3 if dtype == "float32" else 0.35
            for prompt, out in zip(prompts, outs):
                assert len(out.token_ids) == 12
                ids = list(prompt)
                for token in out.token_ids:
                    logits = su.oracle(cfg, weights, ids)[-1]
                    assert float(logits[token]) >= float(logits.max()) - slack * float(logits.abs().max()), (dtype, out.token_ids)
                    ids.append(token)
            assert not llm.cache.live()
            llm.close()


def test_random_model_folder_reads_back(tmp_path):
    """`random-model` of the command line writes a folder that the loader takes, tensor for tensor as the design
    names them."""
    from distie_amd import cli
    from distie_amd.weights.safetensors_io import SafetensorsFile

    (tmp_path / "config.json").write_text(json.dumps(ODD))
    assert cli.main(["random-model", "--config-json", str(tmp_path / "config.json"), "--out", str(tmp_path / "m"),
                     "--seed", "3", "--dtype", "bf16", "--std", "0.1"]) == 0
    stored = SafetensorsFile(tmp_path / "m" / "model.safetensors")
    assert {name: tuple(entry[1]) for name, entry in stored.index.items()} == su.tensor_shapes(ODD)
    stored.close()
    llm = engine(tmp_path / "m", TorchOps(), "float32")
    assert llm.step([StepEntry("a", [1, 2, 3], [2])]).shape == (1, ODD["vocab"])


@pytest.mark.gpu
def test_trace_runner_and_command_line(folders, tmp_path):
    """The trace runner as a program (its own process, steps on standard input, four requests live, pages and
    slots used again) and `generate` of the command line, on a Sekazen model, against the plain implementation."""
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    root = Path(__file__).resolve().parents[1]
    folder, cfg, weights = folders["mixed"]
    lengths = {"p": 70, "q": 33, "r": 64, "s": 5, "t": 50, "u": 21}
    reqs = {r: su.clear_ids(cfg, weights, n, 60 + n) for r, n in lengths.items()}
    want = {r: su.oracle(cfg, weights, ids) for r, ids in reqs.items()}
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
            logits = su.oracle(cfg, weights, ids)[-1]
            assert float(logits[token]) >= float(logits.max()) - 1e-3 * float(logits.abs().max())
            ids.append(token)


def test_preemption_recomputes(ops, folders):
    """So few pages that running requests are preempted and recomputed: every token still is the plain
    implementation's pick."""
    folder, cfg, weights = folders["plain"]
    prompts = [su.random_ids(cfg, n, seed=70 + n) for n in (20, 26, 17)]
    block = 4 if ops.device.type == "cpu" else 16
    new = 24 if block == 4 else 40
    llm = engine(folder, ops, "float32", block_size=block, num_blocks=-(-(26 + new) // block) + 1, max_seqs=3, token_budget=32)
    outs = llm.generate(prompts, SamplingParams(max_new_tokens=new))
    assert sum(o.preemptions for o in outs) > 0, "the pool was not small enough to preempt anybody"
    for prompt, out in zip(prompts, outs):
        ids = list(prompt)
        for token in out.token_ids:
            logits = su.oracle(cfg, weights, ids)[-1]
            assert float(logits[token]) >= float(logits.max()) - 1e-3 * float(logits.abs().max())
            ids.append(token)
    llm.cache.check()
    assert not llm.cache.live()
