"""Each mechanism of the Sekazen decoder alone, as the kernel surface and the parts offer it, against the matching
function of the plain implementation: on the CPU test double and on the GPU kernels (float32 and bfloat16 operands).

A step of the mixer's test is a batch of several requests' rows; the cache is carried over several steps, with
slots that are taken in any order, and the result must be that of every sequence run at once."""

import math

import pytest
import torch

import plain_sekazen as plain
from distie_amd.cache import CacheManager
from distie_amd.config.model_config import PartSpec
from distie_amd.engine.batch import BatchBuilder, StepEntry
from distie_amd.kernels.interface import ScoreExtras
from distie_amd.parts import StepContext, build_part
from torch_ops import TorchOps

F = torch.float64


@pytest.fixture(scope="module", params=["cpu", pytest.param("hip", marks=pytest.mark.gpu)])
def ops(request):
    if request.param == "cpu":
        return TorchOps()
    from distie_amd.kernels.hip_ops import HipOps

    return HipOps("cuda:0")


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def act_types(ops):
    return [torch.float32] if ops.device.type == "cpu" else [torch.float32, torch.bfloat16]


def close(got, want, dtype, what="", slack=1.0):
    tol = (2e-5 if dtype == torch.float32 else 2e-2) * slack
    err = (got.double().cpu() - want.double()).abs().max() / (want.double().abs().max() + 1e-9)
    assert float(err) < tol, f"{what}: {float(err)}"


LENGTHS = (13, 1, 9, 6)
CUTS = ((5, 1, 2, 0), (1, 0, 1, 6), (2, 0, 0, 0), (1, 0, 6, 0), (4, 0, 0, 0))
LONG_LENGTHS = (150, 1, 70, 33)
LONG_CUTS = ((100, 1, 2, 0), (17, 0, 64, 33), (2, 0, 4, 0), (1, 0, 0, 0), (30, 0, 0, 0))


def gather(seqs, rows):
    return torch.cat([seqs[i][at:at + n] for i, at, n in rows])


@pytest.mark.parametrize("width", [30, 40, 48, 256, 2048])
def test_norm_around_one_and_the_branch_reads(ops, width):
    """The norm whose stored weight counts from one, as a part; and the residual's two reads between sub-layers: the
    plain one, and the one that first adds what the last sub-layer returned, through its norm."""
    T, C = 7, width
    dev = lambda t: t.to(ops.device)
    stored = rnd(C, seed=1, scale=0.2)
    for dtype in act_types(ops):
        norm = build_part("norm", PartSpec("rmsnorm", "n.", {"size": C, "eps": 1e-5, "weight_name": "w", "offset": 1.0}))
        assert norm.param_specs()["w"].init == "zeros"
        norm.load({"w": dev(stored.to(dtype))})
        kept = stored.to(dtype).to(F)
        x = rnd(T, C, seed=2, scale=3.0)
        close(ops.dense(norm.apply(ops, dev(x), dtype)), plain.norm_one_plus(x.to(F), kept, 1e-5), dtype, "norm")
        residual = dev(x.clone())
        first = ops.read_residual(residual, dtype)
        assert first.dtype == dtype and torch.equal(first.cpu(), x.to(dtype))
        delta = rnd(T, C, seed=3, scale=0.05).to(dtype)
        h = ops.add_normed_read(residual, dev(delta), norm.weight, norm.eps, dtype)
        want = x.to(F) + plain.norm_one_plus(delta.to(F), kept, 1e-5)
        close(residual, want, torch.float32, "residual behind a sub-layer")
        assert h.dtype == dtype and torch.equal(ops.dense(h).cpu(), residual.cpu().to(dtype))
        # what a product returns, in whatever form it is handed on, is a sub-layer's result as well
        weight, y = rnd(C, 24, seed=4, scale=0.3).to(dtype), rnd(T, 24, seed=5).to(dtype)
        h = ops.add_normed_read(residual, ops.linear(dev(y), dev(weight)), norm.weight, norm.eps, dtype)
        rounded = (y.to(F) @ weight.to(F).T).to(dtype).to(F)
        want = want + plain.norm_one_plus(rounded, kept, 1e-5)
        close(residual, want, dtype, "residual behind a product")
        assert torch.equal(ops.dense(h).cpu(), residual.cpu().to(dtype))


@pytest.mark.parametrize("dims,dim,E,scaling", [(8, 16, 12, True), (16, 16, 16, False), (6, 20, 12, True), (2, 32, 8, False),
                                                 (64, 64, 64, True), (32, 128, 128, True), (16, 64, 32, False)])
def test_head_norm_and_banded_rotation(ops, dims, dim, E, scaling):
    """Behind the stacked product: the norm over every head of q and k (one weight for all heads, as stored), then
    the rotation of a head's first dimensions by frequencies in bands; values pass. Positions up to a few hundred."""
    H, G, eps = 3, 1, 1e-4
    rot = {"base": 300.0, "dims": dims}
    if scaling:
        rot["scaling"] = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 32}
    position = build_part("position", PartSpec("rope_banded", "", dict(rot)))
    position.to_device(ops.device)
    padded = -(-max(dim, E) // 32) * 32
    m = {"heads": H, "kv_heads": G, "dim": dim, "vdim": E, "rot": rot}
    lengths = (300, 5)
    for dtype in act_types(ops):
        wq, wk = (1 + rnd(dim, seed=1, scale=0.3)).float(), (1 + rnd(dim, seed=2, scale=0.3)).float()
        seqs = [rnd(n, H * dim + G * (dim + E) + (8 if dims % 16 == 0 else 3), seed=10 + i, scale=2.0).to(dtype) for i, n in enumerate(lengths)]
        needs = build_part("mixer", PartSpec("conv_gated_attention", "a.", {
            "hidden_size": 8, "num_heads": H, "num_kv_heads": G, "head_dim": dim, "value_dim": E, "conv_taps": 0,
            "window": None, "scale": 1.0})).cache_requirement()
        cache = CacheManager([{"mixer": needs}], 16, 64, 3, device=ops.device, dtype=dtype)
        builder = BatchBuilder(cache, 1024, ops.device, 1000)
        entries = []
        for i, n in enumerate(lengths):
            cache.add(i)
            cache.reserve(i, n)
            entries.append(StepEntry(i, [0] * n, []))
        _, meta, _ = builder.build(entries)
        view = cache.layer(0)["mixer"]
        k_cache, v_cache = view["k"], view["v"]
        q = ops.conv_rope_kv_write(torch.cat(seqs).to(ops.device), None, None, meta, view.group, k_cache, v_cache,
                                   position.rotary(), 1.0, H, G, dim, E, padded, True, True, None,
                                   (wq.to(ops.device), wk.to(ops.device), eps))
        q = ops.dense(q).float().cpu().view(-1, H, padded)
        assert not q[..., dim:].any()
        at = 0
        for i, n in enumerate(lengths):
            s, pos = seqs[i].to(F), torch.arange(n)
            w = {"q": torch.eye(H * dim, dtype=F), "k": torch.eye(G * dim, dtype=F), "v": torch.eye(G * E, dtype=F),
                 "q.norm": wq.to(F), "k.norm": wk.to(F)}
            want_q = plain.queries(s[:, :H * dim], w, "", m, eps, pos)
            want_k, want_v = plain.keys_values(s[:, H * dim:H * dim + G * dim], {**w, "v": torch.zeros(G * E, G * dim, dtype=F)},
                                               "", m, eps, pos)
            close(q[at:at + n, :, :dim], want_q, dtype, f"queries of sequence {i}")
            # the keys as the cache holds them: page after page of the request's table
            table = meta.groups[view.group].block_table[i].cpu().long()
            pages = k_cache[table[:-(-n // 16)].to(ops.device)].float().cpu()       # [pages, G, P, padded]
            got_k = pages.permute(0, 2, 1, 3).reshape(-1, G, padded)[:n, :, :dim]
            close(got_k, want_k, dtype, f"keys of sequence {i}")
            got_v = v_cache[table[:-(-n // 16)].to(ops.device)].float().cpu()       # [pages, G, padded, P]
            got_v = got_v.permute(0, 3, 1, 2).reshape(-1, G, padded)[:n, :, :E]
            close(got_v, s[:, H * dim + G * dim:H * dim + G * (dim + E)].view(n, G, E), dtype, f"values of sequence {i}")
            at += n


@pytest.mark.parametrize("heads,kv_heads,dim,window", [(4, 2, 32, 7), (2, 2, 64, None), (3, 1, 32, 1), (2, 1, 128, 40)])
def test_softmax_with_a_sink(ops, heads, kv_heads, dim, window):
    """Attention over the cache with one more term in the denominator, against the plain weights; a sink far below
    every score changes nothing, one far above leaves nothing of the values; portions, single tokens and a window."""
    scale = 0.35
    lengths, cuts = ((70, 1, 33), ((40, 1, 2), (29, 0, 30), (1, 0, 1)))
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale,
         "mask": {"size": window} if window else None}
    needs = build_part("mixer", PartSpec("conv_gated_attention", "a.", {
        "hidden_size": 8, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": dim, "value_dim": dim,
        "conv_taps": 0, "window": window, "scale": scale})).cache_requirement()
    for dtype in act_types(ops):
        for sinks in (rnd(heads, seed=1, scale=2.0), torch.full((heads,), -80.0), torch.full((heads,), 60.0)):
            seqs = [rnd(n, (heads + 2 * kv_heads) * dim, seed=20 + i).to(dtype) for i, n in enumerate(lengths)]
            want = []
            for s in seqs:
                z = s.to(F)
                q = z[:, :heads * dim].view(-1, heads, dim)
                k = z[:, heads * dim:(heads + kv_heads) * dim].view(-1, kv_heads, dim)
                v = z[:, (heads + kv_heads) * dim:].view(-1, kv_heads, dim)
                want.append(plain.attention(q, k, v, m, sinks.to(F)))
            if float(sinks[0]) == 60.0:
                assert max(float(w.abs().max()) for w in want) < 1e-6
            cache = CacheManager([{"mixer": needs}], 16, 64, 4, device=ops.device, dtype=dtype)
            builder = BatchBuilder(cache, 512, ops.device, 1000)
            for i in reversed(range(len(lengths))):
                cache.add(i)
            at = [0] * len(lengths)
            extras = ScoreExtras(sinks=sinks.float().to(ops.device))
            for cut in cuts:
                entries, rows = [], []
                for i, n in enumerate(cut):
                    n = min(n, lengths[i] - at[i])
                    if n >= 1:
                        cache.reserve(i, n)
                        entries.append(StepEntry(i, [0] * n, []))
                        rows.append((i, at[i], n))
                _, meta, _ = builder.build(entries)
                view = cache.layer(0)["mixer"]
                x = gather(seqs, rows).to(ops.device)
                q = ops.conv_rope_kv_write(x, None, None, meta, view.group, view["k"], view["v"], None, 1.0, heads,
                                           kv_heads, dim, dim, dim, True, True)
                got = ops.paged_attention(q, meta, view.group, view["k"], view["v"], heads, kv_heads, dim, scale,
                                          window, extras)
                ref = gather(want, rows)
                err = (ops.dense(got).double().cpu() - ref).abs().max()
                assert float(err) < (2e-5 if dtype == torch.float32 else 2e-2) * max(1.0, float(ref.abs().max())), \
                    f"sinks {sinks.tolist()} rows {rows}: {float(err)}"
                for i, a, n in rows:
                    cache.commit(i, n)
                    at[i] += n


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,dims,window,lends,lengths,cuts", [
    (4, 2, 16, 24, 8, 6, True, LENGTHS, CUTS), (2, 2, 32, 32, 32, None, False, LENGTHS, CUTS),
    (3, 1, 40, 16, 0, 9, False, LENGTHS, CUTS), (2, 1, 16, 16, 16, 4, True, LENGTHS, CUTS),
    (4, 2, 64, 64, 32, 40, True, LONG_LENGTHS, LONG_CUTS), (2, 1, 64, 32, 64, 21, False, LONG_LENGTHS, LONG_CUTS)])
def test_attention_mixer(ops, heads, kv_heads, dim, vdim, dims, window, lends, lengths, cuts):
    """The mixer alone over a batch in steps: projections, head norms, partial rotation with banded frequencies, the
    cache write, the window, the sink; and a second mixer that borrows the first one's keys and values with a longer
    window, a scale and sinks of its own."""
    C, eps = 48, 1e-5
    rot = {"dims": dims, "base": 50.0, "scaling": {"factor": 3.0, "low": 1.0, "high": 4.0, "original": 16}} if dims else None
    position = PartSpec("rope_banded", "", dict(rot)) if rot else None
    longer = None if window is None else window + 3
    params = {"hidden_size": C, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": dim, "value_dim": vdim,
              "conv_taps": 0, "window": window, "keep": longer if lends else window, "scale": 0.2, "position": position,
              "output_gate": False, "sink": True, "qk_norm": {"eps": eps, "offset": 0.0}}
    cfgs = [{"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": 0.2, "rot": rot,
             "mask": {"size": window} if window else None}]
    for dtype in act_types(ops):
        parts, weights = [build_part("mixer", PartSpec("conv_gated_attention", "a.", params))], []
        if lends:
            parts.append(build_part("mixer", PartSpec("conv_gated_attention", "b.", {
                **params, "window": longer, "scale": 0.3, "kv_from": 0})))
            cfgs = cfgs[:1] + [{**cfgs[0], "scale": 0.3, "mask": {"size": longer} if longer else None}]
        for n, part in enumerate(parts):
            w = {}
            for i, (name, spec) in enumerate(part.param_specs().items()):
                t = rnd(*spec.shape, seed=30 + 7 * n + i, scale=0.25)
                w[name] = (1 + t if name.endswith(".norm") else 6 * t if name == "sink" else t).to(dtype)
            part.load({k: v.to(ops.device) for k, v in w.items()})
            weights.append({k: v.to(F) for k, v in w.items()})
        assert not lends or set(weights[1]) == {"q", "q.norm", "sink", "o"}
        cache = CacheManager([{"mixer": p.cache_requirement()} for p in parts], 16, 64, 5, device=ops.device, dtype=dtype)
        builder = BatchBuilder(cache, 512, ops.device, 1000)
        seqs = [rnd(n, C, seed=50 + i).to(dtype) for i, n in enumerate(lengths)]
        want = [[] for _ in parts]
        for s in seqs:
            pos = torch.arange(s.shape[0])
            k, v = plain.keys_values(s.to(F), weights[0], "", cfgs[0], eps, pos)
            for n in range(len(parts)):
                q = plain.queries(s.to(F), weights[n], "", cfgs[n], eps, pos)
                want[n].append(plain.attention(q, k, v, cfgs[n], weights[n]["sink"]) @ weights[n]["o"].T)
        for i in reversed(range(len(lengths))):
            cache.add(i)
        at = [0] * len(lengths)
        for cut in cuts:
            entries, rows = [], []
            for i, n in enumerate(cut):
                n = min(n, lengths[i] - at[i])
                if n >= 1:
                    cache.reserve(i, n)
                    entries.append(StepEntry(i, [0] * n, []))
                    rows.append((i, at[i], n))
            _, meta, _ = builder.build(entries)
            x = gather(seqs, rows).to(ops.device)
            for n, part in enumerate(parts):
                got = ops.dense(part.forward(ops, x, StepContext(meta, dtype), cache.layer(n)["mixer"], True))
                close(got, gather(want[n], rows), dtype, f"mixer {n} rows {rows}")
            for i, a, n in rows:
                cache.commit(i, n)
                at[i] += n
            cache.check()
        assert at == list(lengths)


@pytest.mark.parametrize("experts,top,width", [(6, 2, 48), (1, 1, 40), (5, 5, 30), (12, 1, 64), (40, 4, 256), (130, 8, 2048)])
def test_router_scores(ops, experts, top, width):
    """The largest scores choose, the lower index among equals; the weights are the chosen experts' own sigmoids, not
    renormalised."""
    T = 9
    for dtype in act_types(ops):
        x, w = rnd(T, width, seed=1).to(dtype), rnd(experts, width, seed=2, scale=3.0 / math.sqrt(width)).to(dtype)
        if experts > 2:
            w[2] = w[0]                                         # equal scores: the lower index goes first
        scores = plain.router_scores(x.to(F), {"router": w.to(F)}, "")
        order = torch.sort(scores, dim=-1, descending=True, stable=True).indices[:, :top]
        got_e, got_w = ops.route_topk(x.to(ops.device), w.to(ops.device), None, top, "sigmoid")
        assert got_e.dtype == torch.int32 and got_w.dtype == torch.float32
        z = x.to(F) @ w.to(F).T
        for t in range(T):
            mine, theirs = got_e[t].cpu().long().tolist(), order[t].tolist()
            if mine != theirs:                                  # only where two logits are a rounding apart
                assert sorted(mine) == sorted(theirs) or \
                    float((z[t, mine] - z[t, theirs]).abs().max()) < 1e-4 * float(z[t].abs().max()), (t, mine, theirs)
            close(got_w[t], scores[t, mine], torch.float32, f"weights of row {t}", slack=10)
        if experts > 2:
            for t in range(T):
                mine = got_e[t].cpu().tolist()
                assert (2 not in mine) or (0 in mine and mine.index(0) < mine.index(2))
        # the router and the experts' hidden values in one call give what the two calls give
        ff = 8
        gate_up = rnd(T, 2 * experts * ff, seed=3).to(dtype).to(ops.device)
        apart = ops.route_glu(gate_up, got_e, got_w, experts, ff, 1.5, 1.702, 1.0, True)
        at_once = ops.route_experts_glu(x.to(ops.device), w.to(ops.device), None, top, "sigmoid", gate_up, experts, ff,
                                        1.5, 1.702, 1.0, True)
        assert torch.equal(ops.dense(apart), ops.dense(at_once))


@pytest.mark.parametrize("experts,top,ff,limit", [(6, 2, 24, 1.25), (1, 1, 8, 0.5), (5, 5, 10, 2.0), (3, 1, 7, 1.0)])
def test_clamped_gated_experts(ops, experts, top, ff, limit):
    """The experts' hidden values from the stacked product (weight on the input, clamps behind it, the sigmoid form of
    the activation, the shifted linear half), the variants of the kernel that other designs use, and the whole
    feed-forward part against the plain mixture."""
    T, C = 11, 40
    for dtype in act_types(ops):
        gate_up = rnd(T, 2 * experts * ff, seed=1, scale=1.5).to(dtype)
        chosen = torch.stack([torch.randperm(experts, generator=torch.Generator().manual_seed(t))[:top] for t in range(T)])
        gates = torch.rand(T, top, generator=torch.Generator().manual_seed(5)) + 0.05
        g = gate_up.to(F)[:, :experts * ff].view(T, experts, ff)
        u = gate_up.to(F)[:, experts * ff:].view(T, experts, ff)
        for on_input, lim, slope, shift in ((True, limit, 1.702, 1.0), (False, limit, 1.702, 1.0), (True, None, 1.0, 0.0)):
            want = torch.zeros(T, experts, ff, dtype=F)
            for t in range(T):
                for k in range(top):
                    e, w = int(chosen[t, k]), float(gates[t, k])
                    a, b = (g[t, e] * w, u[t, e] * w) if on_input else (g[t, e], u[t, e])
                    if lim is not None:
                        a, b = a.clamp(max=lim), b.clamp(-lim, lim)
                    want[t, e] = a * torch.sigmoid(slope * a) * (b + shift) * (1.0 if on_input else w)
            got = ops.route_glu(gate_up.to(ops.device), chosen.to(torch.int32).to(ops.device), gates.to(ops.device),
                                experts, ff, lim, slope, shift, on_input)
            close(ops.dense(got), want.view(T, -1), dtype, f"hidden values, on_input {on_input}, limit {lim}")
            # rows that lie further apart than they are wide give the same
            wide = torch.zeros(T, 2 * experts * ff + 24, dtype=dtype)
            wide[:, :2 * experts * ff] = gate_up
            spread = ops.route_glu(wide.to(ops.device)[:, :2 * experts * ff], chosen.to(torch.int32).to(ops.device),
                                   gates.to(ops.device), experts, ff, lim, slope, shift, on_input)
            assert torch.equal(ops.dense(spread), ops.dense(got))
        part = build_part("feed_forward", PartSpec("routed_experts", "m.", {
            "hidden_size": C, "num_experts": experts, "top": top, "expert_size": ff, "router_bias": False,
            "scoring": "sigmoid", "weight_on": "input", "activation": "clamped_glu", "limit": limit, "slope": 1.702,
            "up_shift": 1.0}))
        w = {}
        for i, (name, spec) in enumerate(part.param_specs().items()):
            fan = spec.shape[-1]
            w[name] = rnd(*spec.shape, seed=40 + i, scale=(6.0 if name == "router" else 1.5) / math.sqrt(fan)).to(dtype)
        assert "router.b" not in w
        part.load({k: v.to(ops.device) for k, v in w.items()})
        part.prepare(ops)
        # rows whose choice does not hang on a rounding: the gap behind the last chosen logit is wide
        x = rnd(60, C, seed=7).to(dtype)
        z = torch.sort(x.to(F) @ w["router"].to(F).T, dim=-1, descending=True).values
        clear = torch.ones(60, dtype=torch.bool) if top == experts else (z[:, top - 1] - z[:, top]) > 0.1
        x = x[clear][:T]
        assert x.shape[0] >= 4
        mlp = {"router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
        want = plain.mixture(x.to(F), {k: v.to(F) for k, v in w.items()}, "", mlp)
        got = ops.dense(part.forward(ops, x.to(ops.device), StepContext(None, dtype)))
        close(got, want, dtype, "the mixture", slack=2.0)


def test_expert_clamps_bite():
    """The plain expert at inputs that reach every clamp: the gate only from above, the linear half on both sides."""
    w = {"gate": torch.eye(4, dtype=F), "up": torch.eye(4, dtype=F), "down": torch.eye(4, dtype=F)}
    h = torch.tensor([[-5.0, -5.0, 5.0, 5.0]], dtype=F)
    out = plain.expert(h, w, "", 2.0)
    sig = lambda a: a / (1 + math.exp(-1.702 * a))
    want = torch.tensor([[sig(-5.0) * (-2.0 + 1), sig(-5.0) * (-2.0 + 1), sig(2.0) * 3.0, sig(2.0) * 3.0]], dtype=F)
    assert torch.allclose(out, want)


@pytest.mark.parametrize("vocab,width,cap", [(61, 48, 6.0), (50, 40, 0.5), (300, 256, 30.0), (40, 32, None)])
def test_embedding_norm_and_capped_head(ops, vocab, width, cap):
    """Rows of the table through the norm become the float32 residual; the head reads the same table, and its logits
    are bent towards the cap in float32."""
    eps = 1e-6
    for dtype in act_types(ops):
        table, stored = rnd(vocab, width, seed=1).to(dtype), rnd(width, seed=2, scale=0.2).to(dtype)
        norm = PartSpec("rmsnorm", "embed.", {"size": width, "eps": eps, "weight_name": "norm", "offset": 1.0})
        embed = build_part("embedding", PartSpec("token_embedding", "", {
            "vocab_size": vocab, "hidden_size": width, "weight_name": "embed", "norm": norm}))
        head = build_part("head", PartSpec("lm_head", "", {"vocab_size": vocab, "hidden_size": width, "tied_to": "embed",
                                                           "weight_name": "head", "cap": cap}))
        shared = table.to(ops.device)
        embed.norm.load({"norm": stored.to(ops.device)})
        embed.load({"embed": shared})
        head.load({"head": shared})
        ids = torch.tensor([3, 0, vocab - 1, 3, 7], dtype=torch.int32)
        x = embed.forward(ops, ids.to(ops.device), None)
        assert x.dtype == torch.float32
        want = plain.norm_one_plus(table.to(F)[ids.long()], stored.to(F), eps)
        close(x, want, dtype, "embedding behind its norm")
        h = (rnd(5, width, seed=3, scale=4.0)).to(dtype)
        logits = head.forward(ops, h.to(ops.device))
        assert logits.dtype == torch.float32
        raw = h.to(F) @ table.to(F).T
        close(logits, raw if cap is None else cap * torch.tanh(raw / cap), dtype, "logits")
        if cap is not None:
            assert float(logits.abs().max()) <= cap and float(raw.abs().max()) > cap
