"""Pilavik without a GPU: the configuration reader, the tensors the model asks for, its run order with
a stretch of layers that runs again, the cache manager's books for its layers, and the plain
implementation's mechanisms against cases whose answer is known."""
import copy

import pytest
import torch

import plain_pilavik as P
from rustinfer_amd.config import ConfigError, PilavikConfig, resolve_architecture
from rustinfer_amd.config.model_config import GatedDeltaSpec, PilavikFeedForwardSpec, SinkLatentAttentionSpec

CFG = dict(architecture="Pilavik", vocab=89, width=40, norm=dict(eps=2e-6), loop=dict(start=1, stop=3, times=3), layers=[
    dict(type="delta", mixer=dict(heads=4, kv_heads=2, dim=8, vdim=6, conv=3), mlp=dict(kind="dense", ff=52)),
    dict(type="latent_attention", mixer=dict(heads=3, dim=10, rot_dim=6, vdim=14, kv_rank=20, scale=0.2, rot=dict(base=300.0, dims=4),
                                              mask=dict(size=24)),
         mlp=dict(kind="moe", expert=dict(ff=12), router=dict(experts=5, top=2, scale=1.7), shared=dict(ff=9))),
    dict(type="delta", mixer=dict(heads=1, kv_heads=1, dim=12, vdim=20, conv=1), mlp=None),
    dict(type="latent_attention", mixer=dict(heads=2, dim=4, rot_dim=8, vdim=6, kv_rank=10, scale=0.5, rot=dict(base=50.0, dims=8)),
         mlp=dict(kind="moe", expert=dict(ff=8), router=dict(experts=3, top=3))),
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
    assert resolve_architecture(CFG).name == "Pilavik"
    c = PilavikConfig.from_dict(CFG)
    assert (c.vocab_size, c.hidden_size, c.norm_eps) == (89, 40, 2e-6)
    assert (c.has_loop, c.loop_start, c.loop_stop, c.loop_times) == (True, 1, 3, 3)
    a, b, d, e = (x.mixer for x in c.layers)
    assert a == GatedDeltaSpec(4, 2, 8, 6, 3) and d == GatedDeltaSpec(1, 1, 12, 20, 1)
    assert b == SinkLatentAttentionSpec(3, 10, 6, 14, 20, 0.2, 300.0, 4, 24)
    assert e == SinkLatentAttentionSpec(2, 4, 8, 6, 10, 0.5, 50.0, 8, None)
    assert [x.type for x in c.layers] == ["delta", "latent_attention", "delta", "latent_attention"]
    assert [x.mlp for x in c.layers] == [PilavikFeedForwardSpec("dense", 52), PilavikFeedForwardSpec("moe", 12, 5, 2, 1.7, 9), None,
                                         PilavikFeedForwardSpec("moe", 8, 3, 3, 1.0, 0)]
    assert PilavikConfig.from_dict(c.to_dict()) == c
    plain = PilavikConfig.from_dict(changed(("loop",), KeyError))
    assert not plain.has_loop and "loop" not in plain.to_dict()


@pytest.mark.parametrize("change,word", [
    ((("layers", 0, "type"), "attention"), "unknown mixer"), ((("layers", 0, "mixer", "kv_heads"), 3), "multiple"),
    ((("layers", 0, "mixer", "conv"), 0), "conv"), ((("layers", 1, "mixer", "rot", "dims"), 8), "rot.dims"),
    ((("layers", 1, "mixer", "mask", "size"), 0), "mask.size"), ((("layers", 1, "mixer", "scale"), KeyError), "scale"),
    ((("layers", 1, "mlp", "router", "top"), 6), "top"), ((("layers", 1, "mlp", "kind"), "sparse"), "kind"),
    ((("layers", 0, "mlp", "ff"), 0), "ff"), ((("loop", "stop"), 5), "stop"), ((("loop", "times"), 0), "times"),
    ((("width",), KeyError), "width"), ((("norm", "eps"), 0.0), "eps"), ((("layers",), []), "layers")])
def test_refuses_what_it_cannot_run(change, word):
    with pytest.raises(ConfigError) as e:
        PilavikConfig.from_dict(changed(*change))
    assert word in str(e.value)


def build(cfg=CFG):
    return resolve_architecture(cfg).builder(PilavikConfig.from_dict(cfg))


def test_model_asks_for_the_designs_tensors():
    W = 40
    want = {"embed": (89, W), "head": (89, W), "final.norm": (W,), "final.norm.b": (W,), "loop.step": (3, W)}
    for i, has_ff in enumerate([True, True, False, True]):
        for h in ("1", "2") if has_ff else ("1",):
            want.update({f"l{i}.norm{h}": (W,), f"l{i}.norm{h}.b": (W,), f"l{i}.norm{h}b": (W,), f"l{i}.norm{h}b.b": (W,),
                         f"l{i}.rg{h}": (W, W), f"l{i}.rg{h}.b": (W,)})
    want.update({"l0.mix.q": (16, W), "l0.mix.k": (16, W), "l0.mix.v": (24, W), "l0.mix.g": (24, W), "l0.mix.b": (4, W), "l0.mix.a": (4, W),
                 "l0.mix.o": (W, 24), "l0.mix.q.conv": (16, 3), "l0.mix.k.conv": (16, 3), "l0.mix.v.conv": (24, 3),
                 "l0.mix.A_log": (4,), "l0.mix.dt_bias": (4,), "l0.mix.norm": (6,),
                 "l0.mlp.up": (52, W), "l0.mlp.up.b": (52,), "l0.mlp.down": (W, 52), "l0.mlp.down.b": (W,), "l0.mlp.act": (4,)})
    want.update({"l1.mix.q": (48, W), "l1.mix.dkv": (26, W), "l1.mix.dkv.norm": (20,), "l1.mix.uk": (30, 20), "l1.mix.uv": (42, 20),
                 "l1.mix.o": (W, 42), "l1.mix.sink": (3,), "l1.mlp.router": (5, W),
                 "l1.mlp.shared.gate": (9, W), "l1.mlp.shared.up": (9, W), "l1.mlp.shared.down": (W, 9)})
    for e in range(5):
        want.update({f"l1.mlp.e{e}.gate": (12, W), f"l1.mlp.e{e}.up": (12, W), f"l1.mlp.e{e}.down": (W, 12)})
    want.update({"l2.mix.q": (12, W), "l2.mix.k": (12, W), "l2.mix.v": (20, W), "l2.mix.g": (20, W), "l2.mix.b": (1, W), "l2.mix.a": (1, W),
                 "l2.mix.o": (W, 20), "l2.mix.q.conv": (12, 1), "l2.mix.k.conv": (12, 1), "l2.mix.v.conv": (20, 1),
                 "l2.mix.A_log": (1,), "l2.mix.dt_bias": (1,), "l2.mix.norm": (20,)})
    want.update({"l3.mix.q": (24, W), "l3.mix.dkv": (18, W), "l3.mix.dkv.norm": (10,), "l3.mix.uk": (8, 10), "l3.mix.uv": (12, 10),
                 "l3.mix.o": (W, 12), "l3.mix.sink": (2,), "l3.mlp.router": (3, W)})
    for e in range(3):
        want.update({f"l3.mlp.e{e}.gate": (8, W), f"l3.mlp.e{e}.up": (8, W), f"l3.mlp.e{e}.down": (W, 8)})
    got = {n: tuple(s.shape) for n, s in build().param_specs().items()}
    assert got == want
    assert "loop.step" not in build(changed(("loop",), KeyError)).param_specs()


def test_a_stretch_that_runs_again_is_more_entries_each_with_a_cache_of_its_own():
    from rustinfer_amd.parts.base import PagedKVNeed, StateNeed
    model = build()
    order = [(c.layer, c.cache, c.write, c.enter) for c in model.schedule]
    assert order == [(0, 0, True, None), (1, 1, True, (0, 0)), (2, 2, True, None), (1, 3, True, (0, 1)), (2, 4, True, None),
                     (1, 5, True, (0, 2)), (2, 6, True, None), (3, 7, True, None)]
    assert [(c.layer, t) for c, (_, t) in zip(model.schedule, P.run_order(CFG))] == P.run_order(CFG)
    needs = model.cache_needs()
    window_kv = PagedKVNeed(1, 26, 24, 20)
    assert [needs[i] for i in (1, 3, 5)] == [window_kv] * 3 and needs[7] == PagedKVNeed(1, 18, None, 10)
    assert needs[0] == StateNeed((4, 8, 6), torch.float32, (("conv", (2, 56), torch.float32),))
    assert [needs[i] for i in (2, 4, 6)] == [StateNeed((1, 12, 20), torch.float32)] * 3       # one tap: no inputs to keep
    assert model.keeps_embedded and not build(changed(("loop",), KeyError)).keeps_embedded
    # a stretch at the very start and one at the very end
    first = build(changed(("loop",), dict(start=0, stop=1, times=2)))
    assert [(c.layer, c.enter) for c in first.schedule] == [(0, (0, 0)), (0, (0, 1)), (1, None), (2, None), (3, None)]
    last = build(changed(("loop",), dict(start=2, stop=4, times=2)))
    assert [(c.layer, c.enter) for c in last.schedule] == [(0, None), (1, None), (2, (0, 0)), (3, None), (2, (0, 1)), (3, None)]


def test_cache_books_for_these_layers():
    from rustinfer_amd.cache import CacheManager
    cm = CacheManager(build().cache_needs(), page_size=8, num_pages=7, max_requests=2, max_model_len=56)
    assert sorted(len(g.cache_ids) for g in cm.groups) == [1, 3]              # the three passes share a group, each a layer slot
    cm.add_request("a")
    cm.append("a", 30)
    cm.add_request("b")
    cm.append("b", 9)
    assert not cm.can_append([("c", 1)])                                      # both state slots are out
    assert not cm.can_append([("a", 20)]) and cm.can_append([("a", 8)])
    held = set(cm.table(cm.groups[0].index, "a")) | set(cm.table(cm.groups[1].index, "a"))
    cm.release("a")
    cm.add_request("c")
    cm.append("c", 40)
    assert (set(cm.table(cm.groups[0].index, "c")) | set(cm.table(cm.groups[1].index, "c"))) & held     # pages are used again
    cm.check()


def test_plain_mechanisms_reduce_to_known_cases():
    """The oracle itself: with decay 1 and write strength 1 the delta rule stores exactly v under a unit
    key (and overwrites it); with decay 0 nothing older than the current token is read; a window of one
    sees the token itself, where the sink alone decides how much of its value passes; one expert of
    weight one with no shared expert is the gated feed-forward times the scale; the activation of a
    constant row is a + b + c + e; neighbouring pairs turn by the position's angle and keep their length."""
    g = torch.Generator().manual_seed(3)
    rnd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    # the delta rule, one head of 4 x 3, the convolution of one tap 1 (identity), silu undone by large inputs
    m = dict(heads=1, kv_heads=1, dim=4, vdim=3, conv=1)
    eye = torch.eye(4, dtype=torch.float64)
    W = 4
    big = 40.0                                                # silu(40) = 40; the unit norm removes it
    p = {"q": big * eye, "k": big * eye, "v": big * rnd(3, W).abs(), "q.conv": torch.ones(4, 1, dtype=torch.float64),
         "k.conv": torch.ones(4, 1, dtype=torch.float64), "v.conv": torch.ones(3, 1, dtype=torch.float64),
         "b": torch.full((1, W), 50.0, dtype=torch.float64), "a": torch.full((1, W), -50.0, dtype=torch.float64),
         "A_log": torch.zeros(1, dtype=torch.float64), "dt_bias": torch.zeros(1, dtype=torch.float64),
         "norm": torch.ones(3, dtype=torch.float64), "g": torch.zeros(3, W, dtype=torch.float64), "o": torch.eye(3, dtype=torch.float64)}
    h = torch.stack([eye[0], eye[1], eye[0]]) + 0.0           # tokens write under key 0, key 1, key 0 again
    state, outs = torch.zeros(4, 3, dtype=torch.float64), []
    for t in range(3):                                        # by hand: beta = 1, g = 1
        k = h[t] / h[t].norm()
        v = P.silu(p["v"] @ h[t])
        state = state + torch.outer(k, v - state.T @ k)
        outs.append(state.T @ (k * 4 ** -0.5))
    # the mixer's own gate is silu(0) = 0, so look at the walk through a gate of ones: g = large
    p["g"] = torch.full((3, W), 50.0, dtype=torch.float64)
    got = P.delta_mixer(h, p, m, 1e-12)
    want = torch.stack(outs)
    want = P.rms(want, 1e-12) * P.silu(h @ p["g"].T)
    assert torch.allclose(got, want, rtol=1e-7, atol=1e-9)
    assert torch.allclose(state[0], P.silu(p["v"] @ h[2]), rtol=1e-9)       # key 0 holds the last value written under it
    p["a"] = torch.full((1, W), 50.0, dtype=torch.float64)    # softplus(50) = 50: g = exp(-50), nothing survives a step
    alone = torch.cat([P.delta_mixer(h[t:t + 1], p, m, 1e-12) for t in range(3)])
    assert torch.allclose(P.delta_mixer(h, p, m, 1e-12), alone, rtol=1e-9, atol=1e-12)
    # a short convolution against its definition
    x, w = rnd(6, 2), rnd(2, 3)
    y = P.short_conv(x, w)
    assert torch.allclose(y[0], w[:, 2] * x[0]) and torch.allclose(y[4], w[:, 0] * x[2] + w[:, 1] * x[3] + w[:, 2] * x[4])
    # a window of one
    ma = dict(heads=2, dim=3, rot_dim=2, vdim=4, kv_rank=5, scale=0.7, rot=dict(base=10.0, dims=2), mask=dict(size=1))
    pa = {"q": rnd(10, W), "dkv": rnd(7, W), "dkv.norm": torch.ones(5, dtype=torch.float64), "uk": rnd(6, 5), "uv": rnd(8, 5),
          "o": torch.eye(8, dtype=torch.float64), "sink": torch.tensor([-1e9, 0.3], dtype=torch.float64)}
    hx = rnd(5, W)
    out = P.latent_attention(hx, pa, ma, 1e-6).view(5, 2, 4)
    c = P.rms(hx @ pa["dkv"].T[:, :5], 1e-6)
    v = (c @ pa["uv"].T).view(5, 2, 4)
    assert torch.allclose(out[:, 0], v[:, 0], rtol=1e-9)                     # no sink to speak of: all of its own value
    assert (out[:, 1].norm(dim=-1) < v[:, 1].norm(dim=-1)).all()              # a sink takes its share
    whole = P.latent_attention(hx, dict(pa, sink=torch.tensor([-1e9, -1e9], dtype=torch.float64)), dict(ma, mask=dict(size=99)), 1e-6)
    none = P.latent_attention(hx, dict(pa, sink=torch.tensor([-1e9, -1e9], dtype=torch.float64)), {k: v_ for k, v_ in ma.items() if k != "mask"}, 1e-6)
    assert torch.allclose(whole, none)
    # the experts
    hh = rnd(7, 10)
    we = {"router": rnd(1, 10), "e0.gate": rnd(6, 10), "e0.up": rnd(6, 10), "e0.down": rnd(10, 6)}
    assert torch.allclose(P.moe_ff(hh, we, dict(router=dict(experts=1, top=1, scale=2.5))),
                          2.5 * P.gated_expert(hh, we["e0.gate"], we["e0.up"], we["e0.down"]))
    # the activation that norms powers
    pf = {"up": torch.zeros(5, 10, dtype=torch.float64), "up.b": torch.full((5,), 2.0, dtype=torch.float64),
          "down": torch.eye(5, dtype=torch.float64)[:3], "down.b": torch.zeros(3, dtype=torch.float64),
          "act": torch.tensor([0.5, -0.25, 2.0, 0.125], dtype=torch.float64)}
    assert torch.allclose(P.poly_norm_ff(hh, pf, 1e-12), torch.full((7, 3), 0.5 - 0.25 + 2.0 + 0.125, dtype=torch.float64))
    # the rotation
    z = rnd(4, 1, 6)
    r = P.rotate_pairs(z, torch.arange(4), 100.0, 4)
    assert torch.allclose(r[..., 4:], z[..., 4:]) and torch.allclose(r[0], z[0])
    assert torch.allclose(r[..., :2].norm(dim=-1), z[..., :2].norm(dim=-1))
    ang = 3 * 100.0 ** (-2.0 / 4)
    assert torch.allclose(r[3, 0, 2], z[3, 0, 2] * torch.cos(torch.tensor(ang)) - z[3, 0, 3] * torch.sin(torch.tensor(ang)))
