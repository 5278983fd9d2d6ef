"""Debuzen without a GPU: the configuration reader, the tensors the model asks for, its run order with a
stretch of layers that runs again, the cache manager's books for layers that keep pages and a state at once
and never give the kept first positions' pages back, and the plain implementation's mechanisms against
cases whose answer is known."""
import copy

import pytest
import torch

import plain_debuzen as P
from rustinfer_amd.config import ConfigError, DebuzenConfig, resolve_architecture
from rustinfer_amd.config.model_config import ChannelDeltaSpec, GatedLinearSpec, MaskedAttentionSpec, StateSpaceSpec, TwoMixerSpec

CFG = dict(architecture="Debuzen", vocab=89, width=40, norm=dict(eps=2e-6, groups=5), logit_softcap=12.0,
           loop=dict(start=1, stop=3, times=3), layers=[
    dict(type="gla", mixer=dict(heads=3, dim=8, vdim=6, tau=4.0), mlp=dict(kind="dense", ff=52)),
    dict(type="parallel", mixer=dict(
        left=dict(heads=4, kv_heads=2, dim=10, vdim=14, scale=0.2, mask=dict(size=24, keep_first=9), rot=dict(base=300.0, dims=4)),
        right=dict(heads=4, kv_heads=2, dim=8, vdim=6, conv=3), left_scale=0.75, right_scale=1.5), mlp=None),
    dict(type="parallel_2", mixer=dict(
        left=dict(heads=2, kv_heads=1, dim=12, vdim=6, scale=0.5, mask=dict(size=10), rot=dict(base=50.0, dims=12)),
        right=dict(heads=4, vdim=5, state=7, groups=2, conv=4, norm_groups=2), left_scale=1.0, right_scale=0.5),
         mlp=dict(kind="dense", ff=20)),
    dict(type="gla", mixer=dict(heads=1, dim=12, vdim=20, tau=16.0), mlp=dict(kind="dense", ff=8)),
])


def changed(path, value):
    d = copy.deepcopy(CFG)
    node = d
    for k in path[:-1]:
        node = node[k]
    if value is KeyError:
        del node[path[-1]]
    else:
        node[path[-1]] = value
    return d


def test_reads_every_size_and_constant():
    assert resolve_architecture(CFG).name == "Debuzen"
    c = DebuzenConfig.from_dict(CFG)
    assert (c.vocab_size, c.hidden_size, c.norm_eps, c.norm_groups, c.logit_softcap) == (89, 40, 2e-6, 5, 12.0)
    assert (c.has_loop, c.loop_start, c.loop_stop, c.loop_times) == (True, 1, 3, 3)
    a, b, d, e = (x.mixer for x in c.layers)
    assert a == GatedLinearSpec(3, 8, 6, 4.0) and e == GatedLinearSpec(1, 12, 20, 16.0)
    assert b == TwoMixerSpec("parallel", MaskedAttentionSpec(4, 2, 10, 14, 0.2, 24, 9, 300.0, 4), ChannelDeltaSpec(4, 2, 8, 6, 3), 0.75, 1.5)
    assert d == TwoMixerSpec("parallel_2", MaskedAttentionSpec(2, 1, 12, 6, 0.5, 10, 0, 50.0, 12), StateSpaceSpec(4, 5, 7, 2, 4, 2), 1.0, 0.5)
    assert [x.type for x in c.layers] == ["gla", "parallel", "parallel_2", "gla"]
    assert [x.ff for x in c.layers] == [52, None, 20, 8]
    assert DebuzenConfig.from_dict(c.to_dict()) == c
    plain = DebuzenConfig.from_dict(changed(("loop",), KeyError))
    assert not plain.has_loop and "loop" not in plain.to_dict()
    # the sizes that only the checkpoint's shapes give
    full = c.complete_from_checkpoint({"l0.mix.a1": (3, 40), "l1.mix.right.a1": (11, 40), "l1.mix.right.g1": (13, 40), "l3.mix.a1": (2, 40)})
    assert (full.layers[0].mixer.decay_rank, full.layers[3].mixer.decay_rank) == (3, 2)
    assert (full.layers[1].mixer.right.decay_rank, full.layers[1].mixer.right.gate_rank) == (11, 13)


@pytest.mark.parametrize("change,word", [
    ((("layers", 0, "type"), "attention"), "unknown mixer"), ((("layers", 1, "mixer", "right", "kv_heads"), 3), "multiple"),
    ((("layers", 1, "mixer", "right", "conv"), 0), "> 0"), ((("layers", 1, "mixer", "left", "rot", "dims"), 12), "rot.dims"),
    ((("layers", 1, "mixer", "left", "mask", "size"), 0), "size"), ((("layers", 2, "mixer", "left", "scale"), KeyError), "scale"),
    ((("layers", 2, "mixer", "left", "mask", "keep_first"), -1), "keep_first"), ((("layers", 2, "mixer", "right", "groups"), 3), "groups"),
    ((("layers", 2, "mixer", "left_scale"), KeyError), "left_scale"), ((("layers", 0, "mixer", "tau"), 0.0), "tau"),
    ((("layers", 0, "mlp", "kind"), "sparse"), "kind"), ((("layers", 0, "mlp", "ff"), 0), "ff"), ((("loop", "stop"), 5), "stop"),
    ((("loop", "times"), 0), "times"), ((("width",), KeyError), "width"), ((("norm", "eps"), 0.0), "eps"),
    ((("norm", "groups"), 3), "parts"), ((("layers",), []), "layers")])
def test_refuses_what_it_cannot_run(change, word):
    with pytest.raises(ConfigError) as e:
        DebuzenConfig.from_dict(changed(*change))
    assert word in str(e.value)


def build(cfg=CFG, shapes=None):
    c = DebuzenConfig.from_dict(cfg)
    if shapes:
        c = c.complete_from_checkpoint(shapes)
    return resolve_architecture(cfg).builder(c)


def test_model_asks_for_the_designs_tensors():
    W = 40
    want = {"embed": (89, W), "embed.norm": (W,), "head": (89, W), "final.norm": (W,), "loop.in": (W, 2 * W)}
    for i, ff in enumerate([52, None, 20, 8]):
        want.update({f"l{i}.norm1": (W,), f"l{i}.shift": (W,)})
        if ff:
            want.update({f"l{i}.norm2": (W,), f"l{i}.mlp.gate": (ff, W), f"l{i}.mlp.up": (ff, W), f"l{i}.mlp.down": (W, ff)})
    want.update({"l0.mix.q": (24, W), "l0.mix.k": (24, W), "l0.mix.v": (18, W), "l0.mix.g": (18, W), "l0.mix.o": (W, 18), "l0.mix.norm": (6,),
                 "l0.mix.a1": (3, W), "l0.mix.a2": (24, 3), "l0.mix.a2.b": (24,)})
    want.update({"l1.mix.left.q": (40, W), "l1.mix.left.k": (20, W), "l1.mix.left.v": (28, W), "l1.mix.left.pb": (4,), "l1.mix.left.o": (W, 56),
                 "l1.mix.right.q": (16, W), "l1.mix.right.k": (16, W), "l1.mix.right.v": (24, W), "l1.mix.right.q.conv": (16, 3),
                 "l1.mix.right.k.conv": (16, 3), "l1.mix.right.v.conv": (24, 3), "l1.mix.right.b": (4, W), "l1.mix.right.A_log": (4,),
                 "l1.mix.right.norm": (6,), "l1.mix.right.a1": (11, W), "l1.mix.right.a2": (32, 11), "l1.mix.right.dt_bias": (32,),
                 "l1.mix.right.g1": (13, W), "l1.mix.right.g2": (24, 13), "l1.mix.right.o": (W, 24)})
    want.update({"l2.mix.left.q": (24, W), "l2.mix.left.k": (12, W), "l2.mix.left.v": (6, W), "l2.mix.left.sink": (2,), "l2.mix.left.o": (W, 12),
                 "l2.mix.right.in": (2 * 20 + 2 * 2 * 7 + 4, W), "l2.mix.right.conv": (48, 4), "l2.mix.right.conv.b": (48,),
                 "l2.mix.right.dt_bias": (4,), "l2.mix.right.A_log": (4,), "l2.mix.right.D": (4,), "l2.mix.right.norm": (20,),
                 "l2.mix.right.o": (W, 20)})
    want.update({"l3.mix.q": (12, W), "l3.mix.k": (12, W), "l3.mix.v": (20, W), "l3.mix.g": (20, W), "l3.mix.o": (W, 20), "l3.mix.norm": (20,),
                 "l3.mix.a1": (2, W), "l3.mix.a2": (12, 2), "l3.mix.a2.b": (12,)})
    shapes = {"l0.mix.a1": (3, W), "l1.mix.right.a1": (11, W), "l1.mix.right.g1": (13, W), "l3.mix.a1": (2, W)}
    got = {n: tuple(s.shape) for n, s in build(shapes=shapes).param_specs().items()}
    assert got == want
    assert "loop.in" not in build(changed(("loop",), KeyError)).param_specs()


def test_a_stretch_that_runs_again_is_more_entries_each_with_caches_of_its_own():
    from rustinfer_amd.parts.base import CompoundNeed, PagedKVNeed, StateNeed
    model = build()
    order = [(c.layer, c.cache, c.write, c.enter) for c in model.schedule]
    assert order == [(0, 0, True, None), (1, 1, True, (0, 0)), (2, 2, True, None), (1, 3, True, (0, 1)), (2, 4, True, None),
                     (1, 5, True, (0, 2)), (2, 6, True, None), (3, 7, True, None)]
    assert [(c.layer, t) for c, (_, t) in zip(model.schedule, P.run_order(CFG))] == P.run_order(CFG)
    needs = model.cache_needs()
    shift = ("shift", (40,), torch.float32)
    assert needs[0] == StateNeed((3, 8, 6), torch.float32, (shift,))
    both = CompoundNeed(PagedKVNeed(2, 10, 24, 14, 9), StateNeed((4, 8, 6), torch.float32, (("conv", (2, 56), torch.float32), shift)))
    assert [needs[i] for i in (1, 3, 5)] == [both] * 3
    assert needs[2] == CompoundNeed(PagedKVNeed(1, 12, 10, 6, 0), StateNeed((4, 7, 5), torch.float32, (("conv", (3, 48), torch.float32), shift)))
    assert model.keeps_embedded and not build(changed(("loop",), KeyError)).keeps_embedded
    first = build(changed(("loop",), dict(start=0, stop=1, times=2)))
    assert [(c.layer, c.enter) for c in first.schedule] == [(0, (0, 0)), (0, (0, 1)), (1, None), (2, None), (3, None)]
    last = build(changed(("loop",), dict(start=2, stop=4, times=1)))
    assert [(c.layer, c.enter) for c in last.schedule] == [(0, None), (1, None), (2, (0, 0)), (3, None)]


def test_cache_books_keep_the_first_positions_pages():
    from rustinfer_amd.cache import CacheManager
    cm = CacheManager(build().cache_needs(), page_size=8, num_pages=12, max_requests=2, max_model_len=96)
    assert sorted(len(g.cache_ids) for g in cm.groups) == [3, 3]              # the passes of a layer share a group, each a layer slot
    kept = next(g for g in cm.groups if g.need.keep_first == 9)
    plain = next(g for g in cm.groups if g.need.keep_first == 0)
    cm.add_request("a")
    for n in (30, 1, 1, 20, 17, 1):
        cm.append("a", n)
        cm.check()
    # 70 tokens: the window of 24 has passed positions below 47; pages 0 and 1 hold the nine kept positions
    assert [p >= 0 for p in cm.table(kept.index, "a")] == [True, True, False, False, False, True, True, True, True]
    assert [p >= 0 for p in cm.table(plain.index, "a")] == [False] * 7 + [True, True]
    cm.add_request("b")
    cm.append("b", 9)
    assert not cm.can_append([("c", 1)])                                      # both state slots are out
    held = set(p for p in cm.table(kept.index, "a") if p >= 0)
    cm.release("a")
    cm.add_request("c")
    cm.append("c", 40)
    assert set(cm.table(kept.index, "c")) & held                              # pages are used again
    with pytest.raises(Exception):
        cm.truncate("c", 41)
    cm.check()


def test_plain_mechanisms_reduce_to_known_cases():
    """The oracle itself: the norm in one group is the plain RMS norm and in as many groups as values the sign;
    the shift with weight 1 hands on the previous token's row and with weight 0 the token's own; the two rotations
    agree up to the order of the features, turn by the position's angle and keep lengths; a window of one sees the
    token itself, where sigmoid weights pass sigmoid(score + b) of its value and a sink takes its share; kept
    positions are seen from anywhere; with decay 1 and write strength 1 the delta rule stores exactly v under a
    unit key; a decay of 0 forgets everything older; the state-space walk against its closed form for one step."""
    g = torch.Generator().manual_seed(3)
    rnd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    x, w = rnd(5, 12), rnd(12)
    assert torch.allclose(P.grouped_rms_norm(x, w, 1, 1e-9), x / x.pow(2).mean(-1, keepdim=True).sqrt() * w)
    assert torch.allclose(P.grouped_rms_norm(x, w, 12, 1e-12), torch.sign(x) * w)
    assert torch.allclose(P.token_shift(x, torch.ones(12, dtype=torch.float64))[1:], x[:-1]) and torch.equal(P.token_shift(x, torch.zeros(12, dtype=torch.float64)), x)
    assert float(P.token_shift(x, torch.ones(12, dtype=torch.float64))[0].abs().max()) < 1e-12
    z = rnd(6, 2, 10)
    inter, half = P.rotate(z, 100.0, 4, True), P.rotate(torch.cat([z[..., 0:4:2], z[..., 1:4:2], z[..., 4:]], -1), 100.0, 4, False)
    assert torch.allclose(torch.cat([inter[..., 0:4:2], inter[..., 1:4:2], inter[..., 4:]], -1), half)
    assert torch.allclose(inter.norm(dim=-1), z.norm(dim=-1)) and torch.equal(inter[0], z[0]) and torch.equal(inter[..., 4:], z[..., 4:])
    a = 3 * 100.0 ** (-2 * 1 / 4)
    assert torch.allclose(inter[3, 0, 2], z[3, 0, 2] * torch.cos(torch.tensor(a)) - z[3, 0, 3] * torch.sin(torch.tensor(a)))
    # attention: a window of one
    W = 8
    m = dict(heads=2, kv_heads=1, dim=4, vdim=3, scale=0.7, mask=dict(size=1), rot=dict(base=10.0, dims=2))
    pa = {"q": rnd(8, W), "k": rnd(4, W), "v": rnd(3, W), "o": torch.eye(6, dtype=torch.float64), "pb": torch.tensor([0.3, -0.2], dtype=torch.float64),
          "sink": torch.tensor([-1e9, 0.3], dtype=torch.float64)}
    hx = rnd(7, W)
    v = hx @ pa["v"].T
    soft = P.sink_attention(hx, pa, m).view(7, 2, 3)
    assert torch.allclose(soft[:, 0], v) and (soft[:, 1].norm(dim=-1) < v.norm(dim=-1)).all()
    sig = P.sigmoid_attention(hx, pa, m, 1e-6).view(7, 2, 3)
    q = P.rotate((hx @ pa["q"].T).view(7, 2, 4), 10.0, 2, True)
    k = P.rotate((hx @ pa["k"].T).view(7, 1, 4), 10.0, 2, True)
    unit = lambda t: t / (t.pow(2).mean(-1, keepdim=True) + 1e-6).sqrt()
    s = (unit(q) * unit(k)).sum(-1) * 0.7 + pa["pb"]
    assert torch.allclose(sig, torch.sigmoid(s)[..., None] * v[:, None, :])
    kept = P.sigmoid_attention(hx, pa, dict(m, mask=dict(size=1, keep_first=7)), 1e-6)
    everything = P.sigmoid_attention(hx, pa, dict(m, mask=dict(size=99)), 1e-6)
    assert torch.allclose(kept, everything) and not torch.allclose(kept[3:], sig.view(7, 6)[3:])
    assert torch.equal(P.visible(6, 2, 1), torch.tensor([[1, 0, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0], [1, 1, 1, 0, 0, 0], [1, 0, 1, 1, 0, 0],
                                                         [1, 0, 0, 1, 1, 0], [1, 0, 0, 0, 1, 1]], dtype=torch.bool))
    # the delta rule: one head of 4 x 3, convolutions of one tap 1, silu undone by large inputs, decays of one
    eye, big = torch.eye(4, dtype=torch.float64), 40.0
    m = dict(heads=1, kv_heads=1, dim=4, vdim=3, conv=1)
    one = lambda n: torch.ones(n, 1, dtype=torch.float64)
    p = {"q": big * eye, "k": big * eye, "v": big * rnd(3, 4).abs(), "q.conv": one(4), "k.conv": one(4), "v.conv": one(3),
         "b": torch.full((1, 4), 50.0, dtype=torch.float64), "a1": torch.zeros(2, 4, dtype=torch.float64), "a2": torch.zeros(4, 2, dtype=torch.float64),
         "dt_bias": torch.full((4,), -50.0, dtype=torch.float64), "A_log": torch.zeros(1, dtype=torch.float64),
         "g1": torch.ones(2, 4, dtype=torch.float64), "g2": torch.full((3, 2), 50.0, dtype=torch.float64),
         "norm": torch.ones(3, dtype=torch.float64), "o": torch.eye(3, dtype=torch.float64)}
    h = torch.stack([eye[0], eye[1], eye[0]]) + 0.0
    state, outs = torch.zeros(4, 3, dtype=torch.float64), []
    for t in range(3):
        kk = h[t] / h[t].norm()
        vv = torch.nn.functional.silu(p["v"] @ h[t])
        state = state + torch.outer(kk, vv - state.T @ kk)
        outs.append(state.T @ (kk * 4 ** -0.5))
    want = torch.stack(outs)
    want = want / (want.pow(2).mean(-1, keepdim=True) + 1e-12).sqrt()
    assert torch.allclose(P.gated_delta(h, p, m, 1e-12), want, rtol=1e-6, atol=1e-9)
    p["dt_bias"] = torch.full((4,), 50.0, dtype=torch.float64)                 # g = exp(-50): nothing survives a step
    alone = torch.cat([P.gated_delta(h[t:t + 1], p, m, 1e-12) for t in range(3)])
    assert torch.allclose(P.gated_delta(h, p, m, 1e-12), alone, rtol=1e-9, atol=1e-12)
    # gated linear attention: a decay of (nearly) zero reads the token's own k v^T only
    mg = dict(heads=2, dim=3, vdim=2, tau=1.0)
    pg = {"q": rnd(6, W), "k": rnd(6, W), "v": rnd(4, W), "g": rnd(4, W), "a1": torch.zeros(2, W, dtype=torch.float64), "a2": torch.zeros(6, 2, dtype=torch.float64),
          "a2.b": torch.full((6,), -60.0, dtype=torch.float64), "norm": torch.ones(2, dtype=torch.float64), "o": torch.eye(4, dtype=torch.float64)}
    alone = torch.cat([P.gated_linear_attention(hx[t:t + 1], pg, mg, 1e-9) for t in range(7)])
    assert torch.allclose(P.gated_linear_attention(hx, pg, mg, 1e-9), alone, rtol=1e-9, atol=1e-12)
    pg["a2.b"] = torch.full((6,), 60.0, dtype=torch.float64)                   # a decay of one: plain linear attention
    full = P.gated_linear_attention(hx, pg, mg, 1e-9)
    qq, kk, vv = (hx @ pg["q"].T).view(7, 2, 3) * 3 ** -0.5, (hx @ pg["k"].T).view(7, 2, 3), (hx @ pg["v"].T).view(7, 2, 2)
    o = torch.einsum("ihd,jhd,jhe->ihe", qq, kk, vv * 1.0) if False else torch.stack(
        [sum(torch.einsum("hd,hd->h", qq[i], kk[j])[:, None] * vv[j] for j in range(i + 1)) for i in range(7)])
    o = o / (o.pow(2).mean(-1, keepdim=True) + 1e-9).sqrt()
    assert torch.allclose(full, o.reshape(7, 4) * torch.nn.functional.silu(hx @ pg["g"].T), rtol=1e-7, atol=1e-9)
    # the state-space mixer, one token: y = dt (B . C) x + D x
    ms = dict(heads=2, vdim=3, state=4, groups=1, conv=1, norm_groups=1)
    C = 6 + 8
    ps = {"in": rnd(12 + 8 + 2, W), "conv": torch.ones(C, 1, dtype=torch.float64), "conv.b": torch.zeros(C, dtype=torch.float64),
          "dt_bias": rnd(2), "A_log": rnd(2), "D": rnd(2), "norm": torch.ones(6, dtype=torch.float64), "o": torch.eye(6, dtype=torch.float64)}
    h1 = rnd(1, W)
    pr = (h1 @ ps["in"].T)[0]
    zz, xx, B, Cc, dt = pr[:6], torch.nn.functional.silu(pr[6:12]).view(2, 3), torch.nn.functional.silu(pr[12:16]), torch.nn.functional.silu(pr[16:20]), pr[20:]
    dt = torch.nn.functional.softplus(dt + ps["dt_bias"])
    y = ((dt * (B @ Cc))[:, None] * xx + ps["D"][:, None] * xx).reshape(6) * torch.nn.functional.silu(zz)
    y = y / (y.pow(2).mean() + 1e-9).sqrt()
    assert torch.allclose(P.state_space(h1, ps, ms, 1e-9)[0], y, rtol=1e-9)
