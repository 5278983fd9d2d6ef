"""A plain, slow implementation of the Pilavik design, one function for each mechanism, written from
the design's equations and sharing no code with the engine.  Whole sequences only: every function
takes all positions of one request at once and walks recurrences token by token.

``tensors`` maps checkpoint names to tensors; ``cfg`` is the parsed config.json.  Everything is
computed in ``dtype`` (float64 unless told otherwise).
"""
from __future__ import annotations

import math

import torch


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def short_conv(x, w):
    """x [T, C], w [C, taps]: y_t = sum_j w[:, j] x_(t - taps + 1 + j), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    padded = torch.cat([x.new_zeros(taps - 1, C), x], dim=0)
    y = x.new_zeros(T, C)
    for j in range(taps):
        y = y + padded[j:j + T] * w[:, j]
    return y


def delta_mixer(h, p, m, eps):
    """The gated delta rule.  h [T, width]; p: the mixer's tensors by short name; m: its sizes."""
    T = h.shape[0]
    H, Hk, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ p["q"].T, p["q.conv"])).view(T, Hk, dk)
    k = silu(short_conv(h @ p["k"].T, p["k.conv"])).view(T, Hk, dk)
    v = silu(short_conv(h @ p["v"].T, p["v.conv"])).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    rep = H // Hk
    q = q.repeat_interleave(rep, dim=1)            # head h reads q/k head h // rep
    k = k.repeat_interleave(rep, dim=1)
    beta = torch.sigmoid(h @ p["b"].T)             # [T, H]
    g = torch.exp(-torch.exp(p["A_log"]) * torch.nn.functional.softplus(h @ p["a"].T + p["dt_bias"]))
    S = h.new_zeros(H, dk, dv)
    out = h.new_zeros(T, H, dv)
    for t in range(T):
        S = S * g[t][:, None, None]
        u = beta[t][:, None] * (v[t] - torch.einsum("hkv,hk->hv", S, k[t]))
        S = S + torch.einsum("hk,hv->hkv", k[t], u)
        out[t] = torch.einsum("hkv,hk->hv", S, q[t])
    out = rms(out, eps) * p["norm"]
    out = out.reshape(T, H * dv) * silu(h @ p["g"].T)
    return out @ p["o"].T


def rotate_pairs(x, positions, base, dims):
    """x [T, n, d]: the first ``dims`` features turned, feature 2i with 2i + 1, by p * base^(-2i/dims)."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    ang = positions.to(torch.float64)[:, None] * f[None, :]
    cos, sin = ang.cos().to(x.dtype)[:, None, :], ang.sin().to(x.dtype)[:, None, :]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


def latent_attention(h, p, m, eps):
    T = h.shape[0]
    H, d, r, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = (h @ p["q"].T).view(T, H, d + r)
    q_plain, q_rot = q[..., :d], q[..., d:]
    down = h @ p["dkv"].T
    c = rms(down[:, :R], eps) * p["dkv.norm"]
    k_rot = down[:, R:].view(T, 1, r)
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    q_rot = rotate_pairs(q_rot, pos, base, dims)
    k_rot = rotate_pairs(k_rot, pos, base, dims)
    k_plain = (c @ p["uk"].T).view(T, H, d)
    v = (c @ p["uv"].T).view(T, H, dv)
    s = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihr,jr->hij", q_rot, k_rot[:, 0])) * m["scale"]
    i, j = pos[:, None], pos[None, :]
    seen = (i - j >= 0)
    window = (m.get("mask") or {}).get("size")
    if window:
        seen = seen & (i - j < window)
    s = s.masked_fill(~seen, float("-inf"))
    sink = p["sink"].view(H, 1, 1).expand(H, T, 1)
    w = torch.softmax(torch.cat([s, sink], dim=-1), dim=-1)[..., :T]      # the sink has no value
    out = torch.einsum("hij,jhv->ihv", w, v).reshape(T, H * dv)
    return out @ p["o"].T


def poly_norm_ff(h, p, eps):
    z = h @ p["up"].T + p["up.b"]
    a, b, c, e = p["act"]
    act = a * rms(z, eps) + b * rms(z * z, eps) + c * rms(z * z * z, eps) + e
    return act @ p["down"].T + p["down.b"]


def gated_expert(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def moe_ff(h, p, mlp, margins=None):
    """``margins`` (a list) receives, for every token, by how much the last chosen expert's logit lies
    above the first one left out."""
    E, top, scale = mlp["router"]["experts"], mlp["router"]["top"], mlp["router"].get("scale", 1.0)
    z = h.to(torch.float64) @ p["router"].to(torch.float64).T
    s = torch.sigmoid(z)
    best = torch.topk(s, top, dim=-1)
    if margins is not None:
        ordered = torch.sort(z, dim=-1, descending=True).values
        margins.append(ordered[:, top - 1] - ordered[:, top] if top < E else torch.full((h.shape[0],), float("inf"), dtype=torch.float64))
    wts = best.values / (best.values.sum(-1, keepdim=True) + 1e-20) * scale
    out = torch.zeros_like(h)
    for e in range(E):
        we = (wts * (best.indices == e)).sum(-1).to(h.dtype)            # 0 where e was not chosen
        rows = we.nonzero().flatten()
        if rows.numel():
            out[rows] += we[rows, None] * gated_expert(h[rows], p[f"e{e}.gate"], p[f"e{e}.up"], p[f"e{e}.down"])
    if "shared.gate" in p:
        out = out + gated_expert(h, p["shared.gate"], p["shared.up"], p["shared.down"])
    return out


def run_order(cfg):
    """[(layer, pass number or None)] in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t) for i in range(loop["start"], loop["stop"])]
    order += [(i, None) for i in range(loop["stop"], n)]
    return order


def sub(tensors, prefix, dtype):
    return {n[len(prefix) + 1:]: t.to(dtype) for n, t in tensors.items() if n.startswith(prefix + ".")}


def forward(cfg, tensors, tokens, dtype=torch.float64, keep_layers=False, margins=None):
    """Logits [T, vocab] of one request's tokens; with ``keep_layers`` also the residual stream after
    every layer run, [runs, T, width].  ``margins``: see ``moe_ff``, one entry for every routed layer run."""
    eps = cfg["norm"]["eps"]
    g = lambda name: tensors[name].to(dtype)
    emb = g("embed")[torch.as_tensor(tokens, dtype=torch.long)]
    x = emb.clone()
    loop = cfg.get("loop")
    kept = []
    for i, t in run_order(cfg):
        if loop and t is not None and i == loop["start"]:
            if t > 0:
                x = x + emb
            x = x + g("loop.step")[t]
        layer = cfg["layers"][i]
        L = f"l{i}"
        h = layer_norm(x, g(f"{L}.norm1"), g(f"{L}.norm1.b"), eps)
        p = sub(tensors, f"{L}.mix", dtype)
        if layer["type"] == "delta":
            y = delta_mixer(h, p, layer["mixer"], eps)
        elif layer["type"] == "latent_attention":
            y = latent_attention(h, p, layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        y = y * torch.sigmoid(h @ g(f"{L}.rg1").T + g(f"{L}.rg1.b"))
        x = x + layer_norm(y, g(f"{L}.norm1b"), g(f"{L}.norm1b.b"), eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = layer_norm(x, g(f"{L}.norm2"), g(f"{L}.norm2.b"), eps)
            p = sub(tensors, f"{L}.mlp", dtype)
            y = poly_norm_ff(h, p, eps) if mlp["kind"] == "dense" else moe_ff(h, p, mlp, margins)
            y = y * torch.sigmoid(h @ g(f"{L}.rg2").T + g(f"{L}.rg2.b"))
            x = x + layer_norm(y, g(f"{L}.norm2b"), g(f"{L}.norm2b.b"), eps)
        if keep_layers:
            kept.append(x.clone())
    x = layer_norm(x, g("final.norm"), g("final.norm.b"), eps)
    logits = x @ g("head").T
    return (logits, torch.stack(kept)) if keep_layers else logits
