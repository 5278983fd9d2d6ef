"""Pilavik on the GPU against the plain implementation (``plain_pilavik.py``): every mechanism alone,
then whole models of three small configurations that differ in every size, in the order of their layers
and in the stretch that runs again, through every way of cutting requests into steps, through pages and
state slots that are used again, and through ``LLM.generate``.  Weights are drawn here with deviations
that make activations of order one, and a few tests build inputs so that one key at a window's edge
decides."""
import json
import math
import os

import numpy as np
import pytest
import torch

import plain_pilavik as P
from helpers import cut_mixed, cut_portions, cut_tail_single, cut_whole, random_requests, run_steps
from test_gpu_belorax import CUTS, PART_TOL, Rows, check_rows, portion_kernel, rel, run_part, some_rows  # noqa: F401

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def delta(heads, kv, dim, vdim, conv):
    return dict(type="delta", mixer=dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, conv=conv))


def lat(heads, dim, rot_dim, vdim, rank, scale, window=None, base=10000.0, dims=None):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=rank, scale=scale, rot=dict(base=base, dims=dims or rot_dim))
    if window:
        m["mask"] = dict(size=window)
    return dict(type="latent_attention", mixer=m)


def dense(ff):
    return dict(kind="dense", ff=ff)


def moe(experts, top, ff, scale=1.0, shared=0):
    d = dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top, scale=scale))
    if shared:
        d["shared"] = dict(ff=shared)
    return d


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


CONFIGS = {
    # the stretch is the first two layers, three times; a window of one page and a bit; one expert a token; a layer without feed-forward
    "A": dict(architecture="Pilavik", vocab=200, width=64, norm=dict(eps=1e-5), loop=dict(start=0, stop=2, times=3), layers=[
        layer(lat(3, 8, 4, 12, 20, 0.35, window=11, base=50.0), moe(4, 1, 24, scale=2.0, shared=10)),
        layer(delta(4, 2, 16, 8, 2), dense(96)),
        layer(delta(2, 2, 24, 40, 4), None),
        layer(lat(2, 24, 8, 8, 16, 0.2, window=40, base=1000.0, dims=4), moe(6, 6, 8, scale=0.7)),
    ]),
    # no stretch at all; heads beyond one 64-wide slice, a latent beyond 128, more experts than a wave has lanes, no window
    "B": dict(architecture="Pilavik", vocab=333, width=136, norm=dict(eps=1e-6), layers=[
        layer(delta(6, 1, 72, 132, 3), moe(70, 3, 16, scale=1.5, shared=24)),
        layer(lat(5, 40, 16, 72, 136, 0.1, base=200.0, dims=12), dense(200)),
        layer(delta(3, 3, 128, 40, 1), dense(64)),
        layer(lat(4, 16, 32, 24, 48, 0.15, window=64, base=5e5), moe(3, 2, 40, shared=7)),
        layer(delta(1, 1, 130, 20, 8), None),
    ]),
    # a width and a vocabulary that are no multiples of eight; the stretch is one layer in the middle, twice; a window of one
    "C": dict(architecture="Pilavik", vocab=211, width=100, norm=dict(eps=1e-6), loop=dict(start=2, stop=3, times=2), layers=[
        layer(delta(5, 5, 20, 12, 4), dense(50)),
        layer(lat(1, 12, 6, 10, 9, 0.4, window=1, base=20.0, dims=2), moe(5, 2, 12, scale=1.0)),
        layer(lat(6, 10, 10, 14, 40, 0.3, window=33, base=500.0), dense(77)),
        layer(delta(12, 2, 16, 18, 3), moe(9, 4, 6, scale=3.0, shared=30)),
    ]),
}
PAGE = {"A": 8, "B": 16, "C": 16}


def bf16(a) -> torch.Tensor:
    return torch.as_tensor(np.asarray(a), dtype=torch.float32).to(torch.bfloat16)


def draw_mixer(rng, m, kind, W, p, t):
    mat = lambda o, i, s=1.0: bf16(s * rng.standard_normal((o, i)) / math.sqrt(i))
    vec = lambda n, mean, std: bf16(mean + std * rng.standard_normal(n))
    if kind == "delta":
        H, Hk, dk, dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
        for x, rows in (("q", Hk * dk), ("k", Hk * dk), ("v", H * dv)):
            t[p + x], t[p + x + ".conv"] = mat(rows, W, 2.0), bf16(rng.standard_normal((rows, taps)) * 0.6)
        t[p + "g"], t[p + "o"] = mat(H * dv, W), mat(W, H * dv)
        t[p + "b"], t[p + "a"] = mat(H, W, 2.0), mat(H, W, 2.0)
        t[p + "A_log"], t[p + "dt_bias"], t[p + "norm"] = vec(H, -1.0, 1.0), vec(H, 0.0, 1.0), vec(dv, 1.0, 0.2)
    else:
        H, d, r, R = m["heads"], m["dim"], m["rot_dim"], m["kv_rank"]
        t[p + "q"], t[p + "dkv"], t[p + "dkv.norm"] = mat(H * (d + r), W, 2.0), mat(R + r, W, 2.0), vec(R, 1.0, 0.2)
        t[p + "uk"], t[p + "uv"], t[p + "o"] = mat(H * d, R, 2.0), mat(H * m["vdim"], R), mat(W, H * m["vdim"])
        t[p + "sink"] = vec(H, 1.0, 1.5)


def draw_weights(cfg: dict, seed: int):
    """name -> bfloat16 tensor for every tensor of the design, activations of order one."""
    rng = np.random.default_rng(seed)
    W = cfg["width"]
    mat = lambda o, i, s=1.0: bf16(s * rng.standard_normal((o, i)) / math.sqrt(i))
    vec = lambda n, mean, std: bf16(mean + std * rng.standard_normal(n))
    t = {"embed": bf16(rng.standard_normal((cfg["vocab"], W))), "final.norm": vec(W, 1.0, 0.1), "final.norm.b": vec(W, 0.0, 0.1),
         "head": mat(cfg["vocab"], W)}
    if "loop" in cfg:
        t["loop.step"] = bf16(0.5 * rng.standard_normal((cfg["loop"]["times"], W)))
    for i, lay in enumerate(cfg["layers"]):
        p = f"l{i}."
        halves = ("1",) if lay["mlp"] is None else ("1", "2")
        for h in halves:
            for nm, mean in ((f"norm{h}", 1.0), (f"norm{h}b", 0.6)):
                t[p + nm], t[p + nm + ".b"] = vec(W, mean, 0.1), vec(W, 0.0, 0.1)
            t[p + f"rg{h}"], t[p + f"rg{h}.b"] = mat(W, W, 1.5), vec(W, 0.0, 0.5)
        draw_mixer(rng, lay["mixer"], lay["type"], W, p + "mix.", t)
        mlp = lay["mlp"]
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            t[p + "mlp.up"], t[p + "mlp.up.b"] = mat(mlp["ff"], W), vec(mlp["ff"], 0.0, 0.2)
            t[p + "mlp.down"], t[p + "mlp.down.b"] = mat(W, mlp["ff"]), vec(W, 0.0, 0.2)
            t[p + "mlp.act"] = bf16([0.7, 0.4, -0.3, 0.1] + 0.1 * rng.standard_normal(4))
        else:
            F = mlp["expert"]["ff"]
            t[p + "mlp.router"] = mat(mlp["router"]["experts"], W, 3.0)
            for e in range(mlp["router"]["experts"]):
                t[p + f"mlp.e{e}.gate"], t[p + f"mlp.e{e}.up"], t[p + f"mlp.e{e}.down"] = mat(F, W), mat(F, W), mat(W, F)
            if "shared" in mlp:
                S = mlp["shared"]["ff"]
                t[p + "mlp.shared.gate"], t[p + "mlp.shared.up"], t[p + "mlp.shared.down"] = mat(S, W), mat(S, W), mat(W, S)
    return t


@pytest.fixture(scope="module")
def tdirs(tmp_path_factory):
    from rustinfer_amd.weights import write_safetensors
    out = {}
    for k, (name, cfg) in enumerate(CONFIGS.items()):
        d = str(tmp_path_factory.mktemp("pilavik_" + name))
        with open(os.path.join(d, "config.json"), "w") as f:
            json.dump(cfg, f)
        write_safetensors(os.path.join(d, "model.safetensors"), draw_weights(cfg, 71 + k))
        out[name] = d
    return out


@pytest.fixture(scope="module")
def plain(tdirs):
    from safetensors.torch import load_file
    return {name: (CONFIGS[name], load_file(os.path.join(d, "model.safetensors"))) for name, d in tdirs.items()}


def plain_rows(cfg, w, reqs):
    rows = Rows()
    rows.margin = {}
    for rid, toks in reqs.items():
        gaps = []
        rows[rid] = P.forward(cfg, w, toks, margins=gaps).numpy()
        rows.margin[rid] = torch.stack(gaps).min(0).values.numpy() if gaps else np.full(len(toks), np.inf)
    return rows


@pytest.fixture(scope="module")
def plain_logits(plain):
    memo = {}

    def get(name, lengths, seed):
        key = (name, tuple(lengths), seed)
        if key not in memo:
            cfg, w = plain[name]
            reqs = random_requests(cfg["vocab"], lengths, seed)
            memo[key] = (reqs, plain_rows(cfg, w, reqs))
        return memo[key]
    return get


def engine_for(model_dir, dtype, name, num_pages=64, max_requests=4, max_len=512):
    from rustinfer_amd.engine import build_engine
    return build_engine(model_dir, dtype=dtype, device=DEV, page_size=PAGE[name], num_pages=num_pages,
                        max_requests=max_requests, max_model_len=max_len, max_batch_tokens=2048)


# ---------------------------------------------------------------------------
# each mechanism alone
# ---------------------------------------------------------------------------
def load_part(part, wt, dtype):
    from rustinfer_amd.engine import make_runtime
    part.load(wt, make_runtime(dtype, DEV))
    return {n: t.double() for n, t in wt.items()}


def mixer_weights(kind, m, width, seed):
    t = {}
    draw_mixer(np.random.default_rng(seed), m, kind, width, "", t)
    return t


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,Hk,dk,dv,taps", [(4, 2, 16, 8, 2), (6, 1, 72, 132, 3), (3, 3, 128, 40, 1), (1, 1, 130, 20, 8),
                                             (12, 2, 16, 18, 4), (2, 2, 256, 64, 4), (5, 5, 20, 12, 5), (8, 4, 64, 64, 4)])
def test_gated_delta_rule_alone(dtype, H, Hk, dk, dv, taps):
    from rustinfer_amd.parts import GatedDeltaRule
    width = 40
    m = dict(heads=H, kv_heads=Hk, dim=dk, vdim=dv, conv=taps)
    part = GatedDeltaRule(width, H, Hk, dk, dv, taps, 1e-5)
    w = load_part(part, mixer_weights("delta", m, width, H * dk + dv + taps), dtype)
    x = some_rows(sum(CUTS), width, 7)
    other = some_rows(60, width, 8)
    ref = P.delta_mixer(x.double(), w, m, 1e-5).numpy()
    assert rel(run_part(part, [], dtype, x, CUTS), ref) < PART_TOL[dtype]
    assert rel(run_part(part, [], dtype, x, CUTS, batch_with=other), ref) < PART_TOL[dtype]     # a second request's state beside it
    assert rel(run_part(part, [], dtype, x, [sum(CUTS)]), ref) < PART_TOL[dtype]                 # the whole prompt at once


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,d,r,dv,R,dims,window", [
    (3, 8, 4, 12, 20, 4, 11), (8, 32, 16, 24, 72, 16, None), (1, 12, 6, 10, 9, 2, 1), (5, 40, 16, 72, 136, 12, 64),
    (16, 16, 8, 24, 48, 8, 17), (2, 64, 64, 130, 192, 64, 100), (40, 8, 4, 6, 12, 4, 16), (6, 10, 10, 14, 40, 10, 2)])
def test_latent_attention_with_window_and_sink_alone(dtype, H, d, r, dv, R, dims, window, portion_kernel):
    from rustinfer_amd.parts import LatentAttention, RotaryEmbedding
    width = 56
    pe = RotaryEmbedding(r, 300.0, rot_dim=dims)
    scale = 0.3 / math.sqrt(d + r)
    part = LatentAttention(width, H, d, r, dv, R, scale, 1e-5, pos_enc=pe, window=window, sink=True)
    m = dict(heads=H, dim=d, rot_dim=r, vdim=dv, kv_rank=R, scale=scale, rot=dict(base=300.0, dims=dims))
    if window:
        m["mask"] = dict(size=window)
    w = load_part(part, mixer_weights("latent_attention", m, width, H * d + R), dtype)
    x = some_rows(sum(CUTS), width, 6)
    ref = P.latent_attention(x.double(), w, m, 1e-5).numpy()
    no_sink = P.latent_attention(x.double(), dict(w, sink=torch.full((H,), -1e9, dtype=torch.float64)), m, 1e-5).numpy()
    assert rel(no_sink, ref) > 0.05                      # the sink matters with these weights
    assert rel(run_part(part, [pe], dtype, x, CUTS), ref) < PART_TOL[dtype]
    assert rel(run_part(part, [pe], dtype, x, [sum(CUTS)], page=16), ref) < PART_TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("window", [16, 33, 141, 200])
def test_a_key_at_the_windows_edge_decides(dtype, decoded, window, portion_kernel):
    """Queries that match one key each: the key that lies window - 1 back is seen (the output is that
    key's value), the key that lies window back is not (the output is what the others and the sink leave).
    A window one too wide or one too narrow changes these rows beyond any rounding."""
    from rustinfer_amd.parts import LatentAttention, RotaryEmbedding
    T, dk, dv = 460, 16, 12
    g = torch.Generator().manual_seed(2)
    eye, look = torch.eye(dk), torch.zeros(dk, dk)          # a query reads feature 8 + n into key feature n
    q_in, q_out, q_far, q_page = 300, 341, 383, 447
    marked = {q_in - (window - 1): q_in, q_out - window: q_out, q_far - (window - 1): q_far, q_page - window: q_page}
    x = 0.1 * torch.randn(T, dk, generator=g)
    x[:, 8:] = 0.0
    x[:, 14] = 3.0                                          # keeps the other keys' few features small after the norm
    for n, (kpos, qpos) in enumerate(marked.items()):
        look[n, 8 + n] = 1.0
        x[kpos] = 0.0
        x[kpos, n] = 4.0
        x[qpos, 8 + n] = 4.0
    x = x.to(torch.bfloat16).float()
    pe = RotaryEmbedding(2, 100.0)
    part = LatentAttention(dk, 1, dk, 2, dv, dk, 2.0, 1e-6, pos_enc=pe, window=window, sink=True)
    wt = {"q": torch.cat([look, torch.zeros(2, dk)]), "dkv": torch.cat([eye, torch.zeros(2, dk)]), "dkv.norm": torch.ones(dk),
          "uk": eye, "uv": torch.randn(dv, dk, generator=g), "o": torch.randn(dk, dv, generator=g), "sink": torch.tensor([0.5])}
    wt = {n: t.to(torch.bfloat16) for n, t in wt.items()}
    w = load_part(part, wt, dtype)
    m = dict(heads=1, dim=dk, rot_dim=2, vdim=dv, kv_rank=dk, scale=2.0, rot=dict(base=100.0, dims=2), mask=dict(size=window))
    ref = P.latent_attention(x.double(), w, m, 1e-6).numpy()
    for other in (window - 1, window + 1):                   # the test can tell
        off = P.latent_attention(x.double(), w, dict(m, mask=dict(size=other)), 1e-6).numpy()
        changed = [q for q in marked.values() if np.abs(ref[q] - off[q]).max() > 0.2 * np.abs(ref[q]).max()]
        assert len(changed) == 2, (other, changed)
    cuts = [290] + [1] * 170 if decoded else [290, 17, 50, 2, 61, 40]
    got = run_part(part, [pe], dtype, x, cuts, page=16)
    for qpos in marked.values():
        assert rel(got[qpos], ref[qpos]) < PART_TOL[dtype], qpos


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("E,top,F,shared,scale,rows", [(4, 1, 24, 10, 2.0, 70), (16, 3, 56, 0, 1.0, 5), (70, 3, 16, 24, 1.5, 100),
                                                       (6, 6, 8, 7, 0.7, 33), (3, 2, 40, 64, 1.0, 1), (130, 8, 4, 3, 2.5, 17)])
def test_feed_forwards_alone(dtype, E, top, F, shared, scale, rows):
    from types import SimpleNamespace
    from rustinfer_amd.engine import Workspace, make_runtime
    from rustinfer_amd.parts import MoEFeedForward, PolyNormMLP
    rt = make_runtime(dtype, DEV)
    width = 40
    rng = np.random.default_rng(E + top)
    mat = lambda o, i, s=1.0: bf16(s * rng.standard_normal((o, i)) / math.sqrt(i))
    x = some_rows(rows, width, 3)
    ctx = SimpleNamespace(workspace=Workspace(rt.device))
    part = MoEFeedForward(width, F, E, top, renormalize=True, score="sigmoid", norm_eps=1e-20, scale=scale, shared_size=shared)
    wt = {"router": mat(E, width, 6.0)}                     # scores far apart: no close calls
    for e in range(E):
        wt[f"e{e}.gate"], wt[f"e{e}.up"], wt[f"e{e}.down"] = mat(F, width), mat(F, width), mat(width, F)
    if shared:
        wt["shared.gate"], wt["shared.up"], wt["shared.down"] = mat(shared, width), mat(shared, width), mat(width, shared)
    assert set(wt) == set(part.param_specs())
    part.load(wt, rt)
    out = part.forward(ctx, x.to(DEV, rt.dtype))
    out = out.double().sum(0) if out.dim() == 3 else out.double()
    mlp = dict(router=dict(experts=E, top=top, scale=scale))
    ref = P.moe_ff(x.double(), {n: t.double() for n, t in wt.items()}, mlp).numpy()
    assert rel(out.cpu().numpy(), ref) < PART_TOL[dtype]
    ff = F + 3
    dense_part = PolyNormMLP(width, ff, 1e-5)
    wt = {"up": mat(ff, width), "up.b": bf16(0.3 * rng.standard_normal(ff)), "down": mat(width, ff),
          "down.b": bf16(0.3 * rng.standard_normal(width)), "act": bf16([0.6, -0.4, 0.25, 0.1])}
    assert set(wt) == set(dense_part.param_specs())
    dense_part.load(wt, rt)
    out = dense_part.forward(ctx, x.to(DEV, rt.dtype))
    out = (out.double().sum(0) if out.dim() == 3 else out.double()) + dense_part.out_bias.double()
    ref = P.poly_norm_ff(x.double(), {n: t.double() for n, t in wt.items()}, 1e-5).numpy()
    assert rel(out.cpu().numpy(), ref) < PART_TOL[dtype]


@pytest.mark.parametrize("E,top,F,shared,renorm,sigmoid", [(8, 2, 32, 16, True, True), (70, 5, 3, 0, True, True), (300, 300, 2, 5, False, True),
                                                          (5, 1, 7, 9, True, False), (9, 4, 6, 30, True, True)])
def test_routing_kernels_with_sigmoid_scores_and_a_shared_expert(E, top, F, shared, renorm, sigmoid):
    from rustinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(E)
    T, scale, eps = 37, 1.7, 1e-20
    width = (E * F + shared + 7) // 8 * 8
    logits = (torch.randn(T, E, generator=g) * 3.0).to(DEV)
    gate_up = torch.randn(T, 2 * E * F + 2 * shared, generator=g).to(DEV)
    weights = torch.empty(T, E, device=DEV)
    how = dict(score="sigmoid" if sigmoid else "softmax", norm_eps=eps, scale=scale)
    ops.moe_route(logits, weights, top, renorm, **how)
    z = logits.double().cpu()
    s = torch.sigmoid(z) if sigmoid else torch.softmax(z, -1)
    want = torch.zeros_like(s)
    for t in range(T):
        keep = torch.argsort(-s[t], stable=True)[:top]
        want[t, keep] = s[t, keep] / ((s[t, keep].sum() + eps) if renorm else 1.0) * scale
    assert (weights.double().cpu() - want).abs().max() < 2e-6
    two, one = torch.full((T, width), 7.0, device=DEV), torch.full((T, width), 7.0, device=DEV)
    ops.moe_swiglu_weighted(gate_up, weights, two, E, F, shared=shared)
    ops.moe_swiglu_routed(gate_up, logits, one, E, F, top, renorm, shared=shared, **how)
    assert torch.equal(one, two)
    gu = gate_up.double().cpu()
    ex = gu[:, :2 * E * F].reshape(T, E, 2, F)
    ref = torch.zeros(T, width, dtype=torch.float64)
    ref[:, :E * F] = (want[:, :, None] * P.silu(ex[:, :, 0]) * ex[:, :, 1]).reshape(T, E * F)
    ref[:, E * F:E * F + shared] = P.silu(gu[:, 2 * E * F:2 * E * F + shared]) * gu[:, 2 * E * F + shared:]
    assert rel(one.double().cpu().numpy(), ref.numpy()) < 2e-6          # the columns beyond the shared expert are zeros


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("width,parts,T", [(64, 1, 9), (100, 3, 9), (4096 + 8, 2, 9), (33, 1, 9), (1024, 8, 3), (2048, 4, 8), (1026, 5, 9),
                                           (1536, 1, 300), (4608, 2, 260), (16384, 1, 9)])
def test_layer_norms_and_the_gated_norm_on_a_sublayers_output(dtype, width, parts, T):
    """Rows short and long, of lengths that do and do not allow loads of four values, few rows (many
    threads a row) and many, one to eight partial sums."""
    from rustinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(width)
    act_dtype = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    x = torch.randn(T, width, generator=g) * 3.0 + 1.0
    vecs = [(torch.randn(width, generator=g) * 0.3 + m).to(DEV) for m in (1.0, 0.0, 0.0, 0.1, 1.0, 0.0)]
    w1, b1, gb, db, w2, b2 = vecs
    delta = torch.randn(parts, T, width, generator=g) * 3.0
    gate = torch.randn(T, width + 8, generator=g).to(act_dtype)
    d_in = delta if parts > 1 else (delta[0] if dtype == "float32" else delta[0].to(torch.bfloat16))
    y = (d_in.double().sum(0) if parts > 1 else d_in.double()) + db.double().cpu()
    y = y * torch.sigmoid(gate[:, 4:4 + width].double() + gb.double().cpu())
    new = x.double() + P.layer_norm(y, w1.double().cpu(), b1.double().cpu(), 1e-5)
    nxt = P.layer_norm(new, w2.double().cpu(), b2.double().cpu(), 1e-5)
    xd, gd = x.to(DEV).contiguous(), gate.to(DEV)
    out = torch.empty(T, width, device=DEV, dtype=act_dtype)
    ops.gated_norm_residual(xd, d_in.to(DEV).contiguous(), w1, b1, 1e-5, gate=gd[:, 4:4 + width], gate_bias=gb, delta_bias=db,
                            next_norm=(w2, b2), next_out=out)
    tol = 1e-2 if dtype == "bfloat16" else 1e-5
    assert rel(xd.double().cpu().numpy(), new.numpy()) < 1e-5
    assert rel(out.double().cpu().numpy(), nxt.numpy()) < tol
    picked = [T - 2, 0, T - 1]
    rows = torch.tensor(picked, dtype=torch.int32, device=DEV)
    some = torch.empty(3, width, device=DEV, dtype=act_dtype)
    ops.layer_norm(xd, w2, b2, 1e-5, some, rows)
    assert rel(some.double().cpu().numpy(), nxt[picked].numpy()) < tol
    ops.stream_add(xd, out, w1)
    assert rel(xd.double().cpu().numpy(), (new + out.double().cpu() + w1.double().cpu()).numpy()) < 1e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,T,bias", [(24, 5, True), (1023, 5, True), (8192, 8, True), (20480, 3, False), (4100, 300, True), (6144, 257, False)])
def test_the_activation_that_norms_powers(dtype, n, T, bias):
    """Rows that fit a thread's registers and rows that do not, few rows and many, columns of wider buffers."""
    from rustinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(n + T)
    dt = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    wide = (torch.randn(T, n + 16, generator=g) * 1.5).to(dt)
    z = wide[:, 8:8 + n].double()
    b = torch.randn(n, generator=g) * 0.5 if bias else None
    if bias:
        z = z + b.double()
    a_, b_, c_, e_ = 0.7, -0.35, 0.2, 0.05
    ref = a_ * P.rms(z, 1e-5) + b_ * P.rms(z * z, 1e-5) + c_ * P.rms(z * z * z, 1e-5) + e_
    out = torch.zeros(T, n + 4, device=DEV, dtype=dt)
    ops.poly_norm(wide.to(DEV)[:, 8:8 + n], b.to(DEV) if bias else None, (a_, b_, c_, e_), 1e-5, out[:, 4:4 + n])
    assert rel(out[:, 4:4 + n].double().cpu().numpy(), ref.numpy()) < (1e-2 if dtype == "bfloat16" else 1e-5)
    assert float(out[:, :4].abs().max()) == 0.0


@pytest.mark.parametrize("taps", [1, 2, 4, 8])
@pytest.mark.parametrize("widths", [(24,), (8, 300, 5), (64, 64, 130, 2)])
def test_short_convolution_through_its_state(taps, widths):
    """Portions shorter than the taps, single tokens, a portion of several chunks, two requests side by side."""
    from types import SimpleNamespace
    from rustinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(taps + len(widths))
    C, lengths = sum(widths), {0: [1, 2, 1, 70, 3, 1, 1, 40], 1: [5, 1, 1, 1, 90, 2, 1, 17]}
    xs = {r: torch.randn(sum(n), C + 6, generator=g) for r, n in lengths.items()}
    ws = [torch.randn(n, taps, generator=g).to(DEV) for n in widths]
    state = torch.full((4, max(taps - 1, 0), C), 9.0, device=DEV) if taps > 1 else None
    got = {r: [] for r in lengths}
    pos = {r: 0 for r in lengths}
    for step in range(8):
        ns = [lengths[r][step] for r in lengths]
        x = torch.cat([xs[r][pos[r]:pos[r] + n] for r, n in zip(lengths, ns)]).to(DEV)
        cu = torch.tensor([0, ns[0], ns[0] + ns[1]], dtype=torch.int32, device=DEV)
        ctx = SimpleNamespace(cu_q=cu, q_start=torch.tensor([pos[0], pos[1]], dtype=torch.int32, device=DEV),
                              state_slots=torch.tensor([2, 0], dtype=torch.int32, device=DEV), num_rows=2, max_q_len=max(ns))
        out = torch.empty(sum(ns), C, device=DEV)
        cols, at = [], 3
        for n in widths:
            cols.append(x[:, at:at + n])
            at += n
        ops.short_conv(cols, ws, state, out, ctx, taps, silu=True)
        got[0].append(out[:ns[0]].cpu())
        got[1].append(out[ns[0]:].cpu())
        for r, n in zip(lengths, ns):
            pos[r] += n
    w = torch.cat(ws).double().cpu()
    for r in lengths:
        ref = P.silu(P.short_conv(xs[r][:, 3:3 + C].double(), w))
        assert rel(torch.cat(got[r]).double().numpy(), ref.numpy()) < 1e-5


# ---------------------------------------------------------------------------
# whole models through the engine's step function
# ---------------------------------------------------------------------------
LENGTHS = (70, 3, 121, 1, 38)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_every_cut_gives_the_plain_logits(tdirs, plain_logits, name, dtype):
    reqs, logits = plain_logits(name, LENGTHS, 21)
    eng = engine_for(tdirs[name], dtype, name)
    for label, steps in (("whole", cut_whole(reqs)), ("last tokens alone", cut_tail_single(reqs, tail=50)),
                         ("portions", cut_portions(reqs, seed=3)),
                         ("portions of two", cut_portions(reqs, seed=4, sizes=(2, 2, 3, 2, 1, 2)))):
        check_rows(steps, run_steps(eng, steps), logits, dtype, f"{name} {dtype} {label}")
        assert not eng.cache.live_requests()


def test_the_stream_after_every_layer_run(tdirs, plain):
    """The residual stream after each layer run (a layer of the stretch counts every time) against the
    plain one: names the first run that differs."""
    from rustinfer_amd.engine import StepEntry
    for name in CONFIGS:
        cfg, w = plain[name]
        toks = random_requests(cfg["vocab"], (45,), 9)["r0"]
        _, want = P.forward(cfg, w, toks, keep_layers=True)
        eng = engine_for(tdirs[name], "float32", name)
        got = []
        for lay in eng.model.layers:
            def fwd(ctx, hidden, cache, _f=lay.forward, **kw):
                _f(ctx, hidden, cache, **kw)
                got.append(hidden.x.detach().double().cpu().numpy().copy())
            lay.forward = fwd
        eng.step([StepEntry("r0", toks, [0])])
        order = P.run_order(cfg)
        assert len(got) == len(want) == len(order)
        for n, (a, b) in enumerate(zip(got, want)):
            assert rel(a, b.numpy()) < 2e-5, (name, n, order[n], cfg["layers"][order[n][0]]["type"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_mixed_batches_with_pages_and_slots_used_again(tdirs, plain_logits, name, dtype):
    lengths = (90, 17, 64, 5, 130, 33, 2, 71)
    reqs, logits = plain_logits(name, lengths, 22)
    page = PAGE[name]
    max_tokens = 3 * (-(-130 // 64) * 64)
    eng = engine_for(tdirs[name], dtype, name, num_pages=max_tokens // page, max_requests=3, max_len=256)
    steps = cut_mixed(reqs, max_tokens, seed=5, max_live=3, tail=6)
    assert max(len(st["entries"]) for st in steps) == 3
    slots, users = set(), {}
    results = {}
    from rustinfer_amd.engine import StepEntry
    for st in steps:
        lg = eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]])
        slots.update(eng.cache.slot(e["id"]) for e in st["entries"])
        for e in st["entries"]:
            for p in eng.cache.table(0, e["id"]):
                if p >= 0:
                    users.setdefault(p, set()).add(e["id"])
        if lg.shape[0]:
            results[st["step"]] = lg.cpu().numpy()
        for rid in st["end"]:
            eng.release(rid)
    assert len(slots) == 3 and len(reqs) > 3             # eight requests went through three state slots
    assert any(len(u) > 1 for u in users.values())       # and pages were used again
    check_rows(steps, results, logits, dtype, f"{name} {dtype} mixed")
    eng.cache.check()


@pytest.mark.parametrize("name", ["A", "C"])
def test_a_batch_gives_what_each_request_gives_alone(tdirs, name):
    from rustinfer_amd.engine import StepEntry
    cfg = CONFIGS[name]
    reqs = random_requests(cfg["vocab"], (40, 9, 1, 25), 30)
    eng = engine_for(tdirs[name], "float32", name)
    alone = {}
    for rid, toks in reqs.items():
        if len(toks) > 1:
            eng.step([StepEntry(rid, toks[:-1], [])])
        alone[rid] = eng.step([StepEntry(rid, toks[-1:], [0])]).cpu().numpy()[0]
        eng.release(rid)
    first = [StepEntry(rid, toks[:-1], []) for rid, toks in reqs.items() if len(toks) > 1]
    eng.step(first)
    both = eng.step([StepEntry(rid, toks[-1:], [0]) for rid, toks in reqs.items()]).cpu().numpy()
    s = float(np.std(both))
    for row, rid in enumerate(reqs):
        assert np.abs(both[row] - alone[rid]).max() < 1e-4 * s, rid


@pytest.mark.parametrize("name", ["A", "B"])
def test_long_decoding(tdirs, plain, name):
    """Twenty tokens of prompt and 280 single tokens: the windows pass over decoded tokens and give
    their pages back, the states and the convolutions' inputs are carried 280 times."""
    cfg, w = plain[name]
    toks = random_requests(cfg["vocab"], (300,), 40)["r0"]
    logits = plain_rows(cfg, w, {"r0": toks})
    eng = engine_for(tdirs[name], "float32", name, num_pages=40)
    steps = cut_tail_single({"r0": toks}, tail=280)
    check_rows(steps, run_steps(eng, steps), logits, "float32", f"{name} long decoding")


@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_scheduler(tdirs, plain, name):
    from rustinfer_amd.llm import LLM
    from rustinfer_amd.sampling import SamplingParams
    cfg, w = plain[name]
    prompts = list(random_requests(cfg["vocab"], (12, 47, 5, 30, 21), 50).values())
    llm = LLM(model=tdirs[name], dtype="float32", paged_block_size=PAGE[name], num_blocks=48, max_batch_seqs=3,
              max_model_len=128, max_batch_tokens=64, chunked_prefill_size=32)
    res = llm.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    for p, r in zip(prompts, res):
        assert len(r.token_ids) == 12
        toks = list(p)
        for i, t in enumerate(r.token_ids):
            row = P.forward(cfg, w, toks)[-1].numpy()
            assert row.max() - row[t] < 1e-3 * max(1.0, float(np.std(row))), (i, t, int(np.argmax(row)))
            toks.append(t)
    assert llm.engine.graph_replays > 0 or not llm.engine._graph_sizes


def test_trace_replay_of_a_pilavik_model(tdirs, plain_logits, tmp_path):
    """bin/trace_run as a user starts it, on the mixed cut, four state slots."""
    import subprocess
    import sys
    from helpers import ROOT
    name = "A"
    reqs, logits = plain_logits(name, (50, 20, 9, 77, 30), 60)
    steps = cut_mixed(reqs, 512, seed=1, max_live=4, tail=5)
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", tdirs[name], "--dtype", "bfloat16",
           "--out", str(tmp_path), "--max-tokens", "512"]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for st in steps:
            proc.stdin.write(json.dumps(st) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {st['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=120) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    results = {}
    for st in steps:
        n = sum(len(e["want"]) for e in st["entries"])
        if n:
            results[st["step"]] = np.fromfile(os.path.join(str(tmp_path), f"{st['step']}.f32"), dtype="<f4").reshape(n, -1)
    check_rows(steps, results, logits, "bfloat16", "trace replay")


# ---------------------------------------------------------------------------
# configurations drawn at random
# ---------------------------------------------------------------------------
def draw_config(rng):
    """A configuration whose every size, the order of its layers and its stretch are drawn: widths up to
    1,024, up to 40 heads, keys of the latent up to 256 features, windows around page borders, up to 32
    experts, convolutions of 1 to 8 taps, layers without feed-forward, a stretch anywhere or none."""
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    layers = []
    for _ in range(int(rng.integers(3, 8))):
        if rng.random() < 0.55:
            H = pick([1, 2, 4, 6, 8, 12, 16])
            mixer = delta(H, pick([d for d in (1, 2, 3, 4, 6, 8, 16) if H % d == 0]), pick([16, 32, 48, 64, 96, 128]),
                          pick([16, 32, 64, 128]), pick([1, 2, 3, 4, 5, 8]))
        else:
            r = pick([8, 16, 32, 64])
            mixer = lat(pick([1, 2, 3, 4, 6, 8, 12, 16, 40]), pick([16, 32, 64, 128]), r, pick([16, 32, 64, 128]),
                        pick([x for x in (32, 64, 128, 192) if x + r <= 256]), pick([0.1, 0.125, 0.2]),
                        window=pick([None, 5, 16, 17, 48, 100, 128, 150, 256]), base=pick([100.0, 1e4, 3e5]),
                        dims=r if rng.random() < 0.7 else r // 2)
        k = rng.random()
        if k < 0.15:
            mlp = None
        elif k < 0.55:
            mlp = dense(pick([64, 200, 512, 1024, 2048]))
        else:
            E = pick([2, 4, 8, 16, 32])
            mlp = moe(E, pick([t for t in (1, 2, 4, 8) if t <= E]), pick([16, 64, 128, 256]), scale=pick([1.0, 1.5, 2.5]),
                      shared=pick([0, 0, 32, 128, 256]))
        layers.append(layer(mixer, mlp))
    cfg = dict(architecture="Pilavik", vocab=pick([100, 333, 777, 1000]), width=pick([64, 96, 192, 320, 512, 1024]),
               norm=dict(eps=pick([1e-5, 1e-6])), layers=layers)
    if rng.random() < 0.75:
        a = int(rng.integers(0, len(layers)))
        cfg["loop"] = dict(start=a, stop=int(rng.integers(a + 1, len(layers) + 1)), times=int(rng.integers(1, 4)))
    return cfg


@pytest.mark.parametrize("seed", [11, 12, 13, 14, 15, 16])
def test_configurations_drawn_at_random(seed, tmp_path):
    """In 32-bit, where rounding hides nothing: last tokens alone, portions, and a mixed schedule on a pool
    that is too small for all requests at once, against the plain implementation."""
    from rustinfer_amd.engine import build_engine
    from rustinfer_amd.weights import write_safetensors
    cfg = draw_config(np.random.default_rng(seed))
    w = draw_weights(cfg, seed)
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg, f)
    write_safetensors(str(tmp_path / "model.safetensors"), w)
    reqs = random_requests(cfg["vocab"], (150, 3, 290, 40, 1, 77), seed)
    logits = Rows({rid: P.forward(cfg, w, toks).numpy() for rid, toks in reqs.items()})
    max_tokens = 2 * 320 + 64
    eng = build_engine(str(tmp_path), dtype="float32", device=DEV, page_size=16, num_pages=max_tokens // 16, max_requests=4,
                       max_model_len=max_tokens, max_batch_tokens=2048)
    for label, steps in (("last tokens alone", cut_tail_single(reqs, tail=40)), ("portions", cut_portions(reqs, seed=seed)),
                         ("mixed", cut_mixed(reqs, max_tokens, seed=seed, max_live=4, tail=6))):
        check_rows(steps, run_steps(eng, steps), logits, "float32", f"{json.dumps(cfg)} {label}")
        assert not eng.cache.live_requests()
