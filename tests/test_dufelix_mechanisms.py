"""Each mechanism of the Dufelix decoder alone, as the kernel surface and the parts offer it, against the matching
function of the plain implementation: on the CPU test double and on the GPU kernels (float32 and bfloat16 operands).

A step of a mixer's test is a batch of several requests' rows; cache and state are carried over several steps, with
slots that are taken in any order, and the result must be that of every sequence run at once."""

import pytest
import torch

import dufelix_util as du
import plain_dufelix as plain
from distie_amd.cache import CacheManager
from distie_amd.config.model_config import PartSpec
from distie_amd.engine.batch import BatchBuilder, StepEntry
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


def run_mixer(ops, spec, tensors, seqs, cuts, dtype, slots=3, pages=64):
    """The mixer `spec` with `tensors` over the sequences `seqs` (inputs [n, C]), `cuts[step][i]` rows of sequence i in
    each step; a sequence takes its slot when it first appears and gives it back at its end, so slots and pages are
    used again. -> every sequence's output rows."""
    mixer = build_part("mixer", spec)
    mixer.load({k: v.to(ops.device) for k, v in tensors.items()})
    mixer.prepare(ops)
    cache = CacheManager([{"mixer": mixer.cache_requirement()}], 16 if ops.device.type != "cpu" else 4, pages, slots,
                         device=ops.device, dtype=dtype)
    builder = BatchBuilder(cache, 4096, ops.device, 4096)
    at = [0] * len(seqs)
    outs = [[] for _ in seqs]
    for step in cuts:
        entries, rows = [], []
        for i, n in enumerate(step):
            if not n:
                continue
            if i not in cache:
                cache.add(i)
            cache.reserve(i, n)
            entries.append(StepEntry(i, [0] * n, []))
            rows.append((i, at[i], n))
        _, meta, _ = builder.build(entries)
        x = torch.cat([seqs[i][a:a + n] for i, a, n in rows]).to(dtype).to(ops.device)
        y = ops.dense(mixer.forward(ops, x, StepContext(meta, dtype), cache.layer(0)["mixer"], True)).float().cpu()
        row = 0
        for i, a, n in rows:
            outs[i].append(y[row:row + n])
            row += n
            at[i] += n
            cache.commit(i, n)
            if at[i] == len(seqs[i]):
                cache.release(i)
    assert at == [len(s) for s in seqs]
    return [torch.cat(o) for o in outs]


def prefixed(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def mixer_case(ops, layer, spec_of, plain_of, lengths, cuts, width=40, seed=0, slack=1.0, pages=64):
    cfg = du.make_config([layer], width=width)
    for dtype in act_types(ops):
        weights = du.random_weights(cfg, seed=seed, dtype=dtype)
        seqs = [rnd(n, width, seed=50 + i).to(dtype) for i, n in enumerate(lengths)]
        got = run_mixer(ops, spec_of(cfg), prefixed(weights, "l0.mix."), seqs, cuts, dtype, pages=pages)
        w = {k: v.to(F) for k, v in weights.items()}
        for i, s in enumerate(seqs):
            want = plain_of(s.to(F), w, "l0.mix.", layer["mixer"], torch.arange(len(s)), float(cfg["norm"]["eps"]))
            close(got[i], want, dtype, f"sequence {i} {dtype}", slack)


def dufelix_mixer(cfg):
    from distie_amd.config import config_from_dict

    return config_from_dict(cfg).model_spec().layers[0].parts["mixer"]


@pytest.mark.parametrize("sizes", [dict(heads=3, dim=12, rot_dim=8, vdim=20, kv_rank=24, q_rank=28),
                                   dict(heads=1, dim=16, rot_dim=16, vdim=16, kv_rank=16, q_rank=16, scaled=False),
                                   dict(heads=5, dim=10, rot_dim=6, vdim=14, kv_rank=18, q_rank=22),
                                   dict(heads=4, dim=32, rot_dim=32, vdim=32, kv_rank=88, q_rank=64),
                                   dict(heads=2, dim=24, rot_dim=16, vdim=40, kv_rank=176, q_rank=48),
                                   dict(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=280, q_rank=40)])
def test_latent_attention_alone(ops, sizes):
    """Latent attention as a part over batches in steps: the cached latent and rotated key part serve every head, the
    sink joins the denominator, neighbouring dimensions are turned. Sizes that fit no tile, all equal, a latent
    wider than the kernels' most common head, and one beyond the matrix-core kernels' largest."""
    layer = du.latent(scale=0.3, base=200.0, **sizes)
    mixer_case(ops, layer, dufelix_mixer, lambda h, w, p, m, pos, eps: plain.latent_attention(h, w, p, m, pos, eps),
               LENGTHS, CUTS, slack=2.0)
    mixer_case(ops, layer, dufelix_mixer, lambda h, w, p, m, pos, eps: plain.latent_attention(h, w, p, m, pos, eps),
               LONG_LENGTHS, LONG_CUTS, seed=1, slack=2.0)
    # a portion long enough for the kernels that many rows choose
    mixer_case(ops, layer, dufelix_mixer, lambda h, w, p, m, pos, eps: plain.latent_attention(h, w, p, m, pos, eps),
               (300, 3), ((290, 1), (10, 2)), seed=2, slack=2.0, pages=128)


def test_latent_cache_holds_the_latent_and_one_turned_part(ops):
    """What the cache holds for a token: the normed latent and the key part turned by the token's position (pairs of
    neighbours, stretched frequencies, cosine and sine scaled), the same latent as the value, zeros beyond."""
    layer = du.latent(heads=2, dim=8, rot_dim=12, vdim=8, kv_rank=20, q_rank=16, base=50.0,
                      scaled=du.scaling(factor=16.0, original=16, fast=2.0, slow=0.25))
    cfg = du.make_config([layer], width=24)
    m = layer["mixer"]
    n = 40
    for dtype in act_types(ops):
        weights = du.random_weights(cfg, seed=2, dtype=dtype)
        mixer = build_part("mixer", dufelix_mixer(cfg))
        mixer.load({k: v.to(ops.device) for k, v in prefixed(weights, "l0.mix.").items()})
        mixer.prepare(ops)
        cache = CacheManager([{"mixer": mixer.cache_requirement()}], 16, 8, 2, device=ops.device, dtype=dtype)
        builder = BatchBuilder(cache, 256, ops.device, 256)
        cache.add("a")
        cache.reserve("a", n)
        _, meta, _ = builder.build([StepEntry("a", [0] * n, [])])
        h = rnd(n, 24, seed=3).to(dtype)
        mixer.forward(ops, h.to(ops.device), StepContext(meta, dtype), cache.layer(0)["mixer"], True)
        view = cache.layer(0)["mixer"]
        pages = cache.request("a").tables[view.group]
        keys = torch.cat([view["k"][p, 0] for p in pages]).float().cpu()[:n]              # [n, DP]
        values = torch.cat([view["v"][p, 0].T for p in pages]).float().cpu()[:n]
        w = {k: v.to(F) for k, v in weights.items()}
        down = h.to(F) @ w["l0.mix.dkv"].T
        latent = plain.norm(down[:, :20], w["l0.mix.dkv.norm"], 1e-5)
        turned = plain.turn(down[:, 20:].view(n, 1, 12), torch.arange(n), m["rot"], True)[:, 0]
        close(keys[:, :20], latent, dtype, "latent as the key")
        close(keys[:, 20:32], turned, dtype, "turned key part")
        close(values[:, :20], latent, dtype, "latent as the value")
        assert not keys[:, 32:].any() and not values[:, 20:].any()


@pytest.mark.parametrize("sizes", [dict(heads=4, kv_heads=2, dim=16, vdim=24, dims=8),
                                   dict(heads=2, kv_heads=2, dim=32, vdim=32, dims=0),
                                   dict(heads=5, kv_heads=1, dim=20, vdim=12, dims=6),
                                   dict(heads=6, kv_heads=3, dim=80, vdim=40, dims=32),
                                   dict(heads=1, kv_heads=1, dim=64, vdim=64, dims=64, scaled=False)])
def test_attention_with_a_gate_for_each_head(ops, sizes):
    layer = du.attention(scale=0.3, base=200.0, **sizes)
    mixer_case(ops, layer, dufelix_mixer, lambda h, w, p, m, pos, eps: plain.attention(h, w, p, m, pos), LENGTHS, CUTS,
               slack=2.0)
    mixer_case(ops, layer, dufelix_mixer, lambda h, w, p, m, pos, eps: plain.attention(h, w, p, m, pos), LONG_LENGTHS,
               LONG_CUTS, seed=1, slack=2.0)


@pytest.mark.parametrize("sizes", [dict(heads=4, vdim=12, state=8, groups=2, conv=3, norm_groups=2),
                                   dict(heads=1, vdim=32, state=32, groups=1, conv=1, norm_groups=1),
                                   dict(heads=6, vdim=10, state=12, groups=3, conv=4, norm_groups=3),
                                   dict(heads=4, vdim=64, state=128, groups=1, conv=4, norm_groups=4),
                                   dict(heads=2, vdim=72, state=40, groups=2, conv=2, norm_groups=1)])
def test_state_space_mixer_alone(ops, sizes):
    """The state-space mixer as a part: convolution with bias and silu, step sizes and decays, the state carried from
    step to step (row by row in short steps, in chunks in long ones), the gate in front of the grouped norm."""
    layer = du.mamba(**sizes)
    mixer_case(ops, layer, dufelix_mixer, lambda h, w, p, m, pos, eps: plain.mamba2(h, w, p, m, eps), LENGTHS, CUTS,
               slack=2.0)
    mixer_case(ops, layer, dufelix_mixer, lambda h, w, p, m, pos, eps: plain.mamba2(h, w, p, m, eps), LONG_LENGTHS,
               LONG_CUTS, seed=1, slack=2.0)


@pytest.mark.parametrize("H,P,N,G", [(3, 8, 4, 1), (4, 20, 12, 2), (2, 64, 64, 1), (2, 80, 130, 2), (1, 24, 300, 1)])
def test_state_space_scan_with_fast_and_slow_heads(ops, H, P, N, G):
    """The recurrence alone: step sizes from tiny to huge in one sequence (softplus far out on both sides), heads that
    forget at once beside heads that keep everything, over rows enough for several chunks, then row by row from the
    state that the long step left."""
    lengths = (200, 3, 65)
    for dtype in act_types(ops):
        xbc = [rnd(n, H * P + 2 * G * N + 3, seed=i, scale=1.0).to(dtype) for i, n in enumerate(lengths)]
        dt = [(rnd(n, H, seed=9 + i, scale=4.0) + torch.linspace(-12, 30, n)[:, None]).to(dtype) for i, n in enumerate(lengths)]
        dt_bias = torch.linspace(-2.0, 1.0, H)
        a_log = torch.linspace(-9.0, 2.5, H)
        skip = torch.linspace(0.5, 1.5, H)
        want = []
        for x, d in zip(xbc, dt):
            n = x.shape[0]
            xs = x.to(F)[:, :H * P].view(n, H, P)
            B = x.to(F)[:, H * P:H * P + G * N].view(n, G, N).repeat_interleave(H // G, dim=1)
            C = x.to(F)[:, H * P + G * N:H * P + 2 * G * N].view(n, G, N).repeat_interleave(H // G, dim=1)
            want.append(plain.state_space_scan(xs, B, C, plain.softplus(d.to(F) + dt_bias.to(F)), a_log.to(F), skip.to(F)).reshape(n, H * P))
        dev = lambda t: t.to(ops.device)
        # all but each sequence's last 5 rows in one step (in chunks where there are enough), the rest row by row
        cache = CacheManager([{"mixer": build_state(H, N, P)}], 16, 8, len(lengths), device=ops.device)
        builder = BatchBuilder(cache, 4096, ops.device, 4096)
        state = cache.layer(0)["mixer"]["state"]
        got = [[] for _ in lengths]
        at = [0] * len(lengths)
        steps = [[max(n - 5, 1) for n in lengths]] + [[1 if n - max(n - 5, 1) > k else 0 for n in lengths] for k in range(5)]
        for step in steps:
            entries, rows = [], []
            for i, n in enumerate(step):
                if n:
                    if i not in cache:
                        cache.add(i)
                    cache.reserve(i, n)
                    entries.append(StepEntry(i, [0] * n, []))
                    rows.append((i, at[i], n))
            _, meta, _ = builder.build(entries)
            x = dev(torch.cat([xbc[i][a:a + n] for i, a, n in rows]))
            d = dev(torch.cat([dt[i][a:a + n] for i, a, n in rows]))
            y = ops.ssm_scan(x, d, dev(dt_bias), dev(a_log), dev(skip), state, meta, H, P, N, G).cpu()
            row = 0
            for i, a, n in rows:
                got[i].append(y[row:row + n])
                row += n
                at[i] += n
                cache.commit(i, n)
        for i in range(len(lengths)):
            close(torch.cat(got[i]), want[i], torch.float32, f"sequence {i} {dtype}", slack=3.0)


def build_state(H, N, P):
    from distie_amd.parts import FixedState

    return FixedState.of((H, N, P))


def test_gate_in_front_of_the_grouped_norm(ops):
    for N, groups in ((24, 1), (60, 3), (272, 2), (2048, 8)):
        for dtype in act_types(ops):
            x, z = rnd(9, N, seed=1, scale=3.0), rnd(9, N + 8, seed=2).to(dtype)
            weight = (1 + rnd(N, seed=3, scale=0.3)).to(dtype)
            dev = lambda t: t.to(ops.device)
            got = ops.rmsnorm_gate(dev(x), dev(weight), 1e-5, dev(z)[:, 8:], dtype, group=N // groups, gate="silu", gate_first=True)
            gated = x.to(F) * plain.silu(z.to(F)[:, 8:])
            want = plain.rms(gated.view(9, groups, N // groups), 1e-5).reshape(9, N) * weight.to(F)
            close(got, want, dtype, f"{N} in {groups}")
            # the other order is another function
            behind = plain.rms(x.to(F).view(9, groups, N // groups), 1e-5).reshape(9, N) * weight.to(F) * plain.silu(z.to(F)[:, 8:])
            assert float((behind - want).abs().max()) > 0.05


def test_gated_activations_gates_by_head_and_scaled_embedding(ops):
    dev = lambda t: t.to(ops.device)
    for dtype in act_types(ops):
        gate_up = rnd(7, 2 * 44, seed=1, scale=2.0).to(dtype)
        want = plain.gelu_tanh(gate_up.to(F)[:, :44]) * gate_up.to(F)[:, 44:]
        close(ops.glu_mul(dev(gate_up), "gelu_tanh"), want, dtype, "gelu times up")
        weight, x = rnd(2 * 44, 24, seed=2, scale=0.3).to(dtype), rnd(7, 24, seed=3).to(dtype)
        product = (x.to(F) @ weight.to(F).T).to(dtype).to(F)
        close(ops.dense(ops.linear_glu(dev(x), dev(weight), "gelu_tanh")), plain.gelu_tanh(product[:, :44]) * product[:, 44:],
              dtype, "product, gelu, times up", slack=2.0)
        H, stride, E = 5, 32, 12
        heads, gates = rnd(7, H * stride, seed=4).to(dtype), rnd(7, H + 3, seed=5, scale=2.0).to(dtype)
        want = heads.to(F).view(7, H, stride)[..., :E] * torch.sigmoid(gates.to(F)[:, 3:])[:, :, None]
        close(ops.sigmoid_gate(dev(heads), H, stride, E, dev(gates)[:, 3:], per_head=True), want.reshape(7, H * E), dtype, "a gate a head")
        table = rnd(11, 40, seed=6).to(dtype)
        ids = torch.tensor([3, 0, 10, 3], dtype=torch.int32)
        got = ops.embed(dev(ids), dev(table), 12.5)
        assert got.dtype == torch.float32
        close(got, table.to(F)[ids.long()] * 12.5, torch.float32, "scaled embedding")


def test_products_by_head(ops):
    """Every head's own product, for few rows and for many, with inputs and results that lie apart in wider rows."""
    dev = lambda t: t.to(ops.device)
    for T in (1, 5, 16, 17, 150, 300):
        for H, N, K, lx, lo in ((3, 24, 12, 20, 32), (1, 16, 16, 16, 16), (5, 18, 10, 16, 24), (4, 72, 104, 128, 72),
                                (2, 40, 200, 208, 48), (3, 100, 128, 160, 112)):
            for dtype in act_types(ops):
                x, w = rnd(T, H * lx, seed=1).to(dtype), rnd(H, N, K, seed=2, scale=0.3).to(dtype)
                got = ops.heads_linear(dev(x), dev(w), lx, lo).float().cpu().view(T, H, lo)
                want = torch.einsum("thk,hnk->thn", x.to(F).view(T, H, lx)[..., :K], w.to(F))
                close(got[..., :N], want, dtype, f"{T} rows, {H} heads of {N} x {K}")
                assert not got[..., N:].any()


def test_convolution_with_bias_and_activation(ops):
    """The short convolution over column views with a bias and silu behind it, its state carried over steps of one
    row and of more rows than it has taps, and of fewer."""
    lengths, cuts = (11, 4, 7), ((2, 1, 7), (1, 1, 0), (5, 2, 0), (3, 0, 0))
    for taps, N in ((1, 24), (3, 40), (4, 56), (4, 424)):
        for dtype in act_types(ops):
            from distie_amd.parts import FixedState, TensorDecl

            need = FixedState((TensorDecl("conv", (taps - 1, N), torch.float32),)) if taps > 1 else None
            cache = CacheManager([{"mixer": need}], 16, 8, 3, device=ops.device)
            builder = BatchBuilder(cache, 256, ops.device, 256)
            filters, bias = rnd(N, taps, seed=1, scale=0.6).to(dtype), rnd(N, seed=2, scale=0.2)
            seqs = [rnd(n, N + 16, seed=3 + i).to(dtype) for i, n in enumerate(lengths)]
            at, got = [0] * 3, [[] for _ in lengths]
            for step in cuts:
                entries, rows = [], []
                for i, n in enumerate(step):
                    if n:
                        if i not in cache:
                            cache.add(i)
                        cache.reserve(i, n)
                        entries.append(StepEntry(i, [0] * n, []))
                        rows.append((i, at[i], n))
                _, meta, _ = builder.build(entries)
                x = torch.cat([seqs[i][a:a + n] for i, a, n in rows]).to(ops.device)
                state = cache.layer(0)["mixer"]["conv"] if taps > 1 else None
                y = ops.causal_conv(x[:, 8:8 + N], filters.to(ops.device), state, meta, bias=bias.to(ops.device), act="silu").float().cpu()
                row = 0
                for i, a, n in rows:
                    got[i].append(y[row:row + n])
                    row += n
                    at[i] += n
                    cache.commit(i, n)
            for i, s in enumerate(seqs):
                want = plain.silu(plain.short_convolution(s.to(F)[:, 8:8 + N], filters.to(F), bias.to(F)))
                close(torch.cat(got[i]), want, dtype, f"{taps} taps, sequence {i}")
