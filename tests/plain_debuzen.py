"""A plain, slow implementation of the Debuzen design, one function a mechanism, written from the
design's equations with torch on the CPU.  It walks a whole sequence from its first token and keeps no
cache; recurrences are loops over tokens.  It shares nothing with the engine's code and is what the
engine's results are compared with.

``weights``: tensor name -> tensor as the checkpoint names them; ``cfg``: the dict of config.json.
Everything runs in ``dtype`` (float64 by default).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch
import torch.nn.functional as F


def grouped_rms_norm(x, w, groups: int, eps: float):
    """Each of ``groups`` equal consecutive parts of a row divided by its own root mean square, times w."""
    T, d = x.shape
    parts = x.reshape(T, groups, d // groups)
    parts = parts / torch.sqrt(parts.pow(2).mean(-1, keepdim=True) + eps)
    return parts.reshape(T, d) * w


def token_shift(h, mix):
    """h_t + (h_(t-1) - h_t) * mix, with zeros before the first token."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return h + (prev - h) * mix


def rotate(x, base: float, dims: int, interleaved: bool):
    """x [T, heads, dim]: the first ``dims`` features of every head turned by the token's position."""
    T = x.shape[0]
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    freq = base ** (-2.0 * i / dims)
    ang = torch.arange(T, dtype=torch.float64)[:, None] * freq[None, :]
    cos, sin = ang.cos().to(x.dtype)[:, None, :], ang.sin().to(x.dtype)[:, None, :]
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * cos - v * sin
        out[..., 1:dims:2] = v * cos + u * sin
    else:
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * cos - v * sin
        out[..., half:dims] = v * cos + u * sin
    return out


def causal_conv(x, w, bias=None):
    """x [T, C], w [C, taps] (last column the current token's), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], dim=0)
    y = torch.zeros_like(x)
    for j in range(taps):
        y = y + padded[j:j + T] * w[:, j]
    if bias is not None:
        y = y + bias
    return y


def windowed_scores(q, k, scale: float, heads: int, kv_heads: int):
    """[heads, T, T] scores of grouped heads: query head h against key head h // (heads / kv_heads)."""
    rep = heads // kv_heads
    kk = k.repeat_interleave(rep, dim=1)
    return torch.einsum("ihd,jhd->hij", q, kk) * scale


def visible(T: int, size: int, keep_first: int = 0):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def sigmoid_attention(h, W, m, eps: float):
    """Windowed attention whose weights are sigmoids of the scores plus a number a head, with the first
    tokens kept in sight; interleaved rotation, then queries and keys divided by their root mean square."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W["q"].T).reshape(T, H, d)
    k = (h @ W["k"].T).reshape(T, G, d)
    v = (h @ W["v"].T).reshape(T, G, dv)
    q = rotate(q, m["rot"]["base"], m["rot"]["dims"], True)
    k = rotate(k, m["rot"]["base"], m["rot"]["dims"], True)
    q = q / torch.sqrt(q.pow(2).mean(-1, keepdim=True) + eps)
    k = k / torch.sqrt(k.pow(2).mean(-1, keepdim=True) + eps)
    s = windowed_scores(q, k, m["scale"], H, G) + W["pb"][:, None, None]
    see = visible(T, m["mask"]["size"], m["mask"].get("keep_first", 0))
    wts = torch.sigmoid(s) * see[None].to(h.dtype)
    vv = v.repeat_interleave(H // G, dim=1)
    o = torch.einsum("hij,jhd->ihd", wts, vv).reshape(T, H * dv)
    return o @ W["o"].T


def sink_attention(h, W, m):
    """Windowed softmax attention with a learned number a head in the denominator; half-split rotation."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W["q"].T).reshape(T, H, d)
    k = (h @ W["k"].T).reshape(T, G, d)
    v = (h @ W["v"].T).reshape(T, G, dv)
    q = rotate(q, m["rot"]["base"], m["rot"]["dims"], False)
    k = rotate(k, m["rot"]["base"], m["rot"]["dims"], False)
    s = windowed_scores(q, k, m["scale"], H, G)
    see = visible(T, m["mask"]["size"], m["mask"].get("keep_first", 0))
    s = s.masked_fill(~see[None], -math.inf)
    sink = W["sink"][:, None, None].expand(H, T, 1)
    p = torch.softmax(torch.cat([s, sink], dim=-1), dim=-1)[..., :T]
    vv = v.repeat_interleave(H // G, dim=1)
    o = torch.einsum("hij,jhd->ihd", p, vv).reshape(T, H * dv)
    return o @ W["o"].T


def gated_delta(h, W, m, eps: float):
    """The gated delta rule with a decay for every key channel."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = F.silu(causal_conv(h @ W["q"].T, W["q.conv"])).reshape(T, G, d)
    k = F.silu(causal_conv(h @ W["k"].T, W["k.conv"])).reshape(T, G, d)
    v = F.silu(causal_conv(h @ W["v"].T, W["v.conv"])).reshape(T, H, dv)
    q = q / torch.sqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ W["b"].T)                                       # [T, H]
    rate = torch.exp(W["A_log"])[None, :, None]
    g = torch.exp(-rate * F.softplus(((h @ W["a1"].T) @ W["a2"].T + W["dt_bias"]).reshape(T, H, d)))
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hh in range(H):
        kh = hh // (H // G)
        S = torch.zeros(d, dv, dtype=h.dtype)
        for t in range(T):
            S = g[t, hh][:, None] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, kh])
            S = S + torch.outer(k[t, kh], u)
            out[t, hh] = S.T @ q[t, kh]
    out = out / torch.sqrt(out.pow(2).mean(-1, keepdim=True) + eps) * W["norm"]
    gate = torch.sigmoid((h @ W["g1"].T) @ W["g2"].T).reshape(T, H, dv)
    return (out * gate).reshape(T, H * dv) @ W["o"].T


def state_space(h, W, m, eps: float):
    """A state-space mixer with one decay a head and token, inputs shared by groups of heads."""
    T = h.shape[0]
    H, dv, N, G, ng = m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"]
    inner = H * dv
    p = h @ W["in"].T
    z, xbc, dt = p[:, :inner], p[:, inner:2 * inner + 2 * G * N], p[:, 2 * inner + 2 * G * N:]
    xbc = F.silu(causal_conv(xbc, W["conv"], W["conv.b"]))
    x = xbc[:, :inner].reshape(T, H, dv)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = F.softplus(dt + W["dt_bias"])                                       # [T, H]
    decay = torch.exp(-torch.exp(W["A_log"])[None] * dt)
    y = torch.zeros(T, H, dv, dtype=h.dtype)
    for hh in range(H):
        gg = hh // (H // G)
        S = torch.zeros(N, dv, dtype=h.dtype)
        for t in range(T):
            S = decay[t, hh] * S + dt[t, hh] * torch.outer(B[t, gg], x[t, hh])
            y[t, hh] = S.T @ C[t, gg] + W["D"][hh] * x[t, hh]
    y = y.reshape(T, inner) * F.silu(z)
    y = grouped_rms_norm(y, W["norm"], ng, eps)
    return y @ W["o"].T


def gated_linear_attention(h, W, m, eps: float):
    T = h.shape[0]
    H, d, dv, tau = m["heads"], m["dim"], m["vdim"], m["tau"]
    q = (h @ W["q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ W["k"].T).reshape(T, H, d)
    v = (h @ W["v"].T).reshape(T, H, dv)
    zz = (h @ W["a1"].T) @ W["a2"].T + W["a2.b"]
    alpha = torch.sigmoid(zz).pow(1.0 / tau).reshape(T, H, d)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hh in range(H):
        S = torch.zeros(d, dv, dtype=h.dtype)
        for t in range(T):
            S = alpha[t, hh][:, None] * S + torch.outer(k[t, hh], v[t, hh])
            out[t, hh] = S.T @ q[t, hh]
    out = out / torch.sqrt(out.pow(2).mean(-1, keepdim=True) + eps) * W["norm"]
    return (out.reshape(T, H * dv) * F.silu(h @ W["g"].T)) @ W["o"].T


def swiglu(h, W):
    return (F.silu(h @ W["gate"].T) * (h @ W["up"].T)) @ W["down"].T


def sub(weights: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {n[len(prefix) + 1:]: t for n, t in weights.items() if n.startswith(prefix + ".")}


def mixer(kind: str, h, W, m, eps: float):
    if kind == "gla":
        return gated_linear_attention(h, W, m, eps)
    if kind == "parallel":
        left = sigmoid_attention(h, sub(W, "left"), m["left"], eps)
        right = gated_delta(h, sub(W, "right"), m["right"], eps)
    elif kind == "parallel_2":
        left = sink_attention(h, sub(W, "left"), m["left"])
        right = state_space(h, sub(W, "right"), m["right"], eps)
    else:
        raise ValueError(kind)
    return m["left_scale"] * left + m["right_scale"] * right


def run_order(cfg) -> List[tuple]:
    """[(layer, pass or None)]: the layers before the stretch, the stretch ``times`` times, the rest."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t) for i in range(loop["start"], loop["stop"])]
    return order + [(i, None) for i in range(loop["stop"], n)]


def forward(cfg, weights, tokens, dtype=torch.float64, layers_out: Optional[list] = None):
    """Logits [T, vocab] of a whole sequence; ``layers_out`` collects the stream after every layer run."""
    Wt = {n: (t.to(dtype) if t.is_floating_point() else t) for n, t in weights.items()}
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    norm = lambda x, name: grouped_rms_norm(x, Wt[name], groups, eps)
    x = norm(Wt["embed"][torch.as_tensor(tokens, dtype=torch.long)], "embed.norm")
    x0 = x
    loop = cfg.get("loop")
    for i, t in run_order(cfg):
        if t is not None and i == loop["start"]:
            x = torch.cat([x, x0], dim=-1) @ Wt["loop.in"].T
        layer, L = cfg["layers"][i], sub(Wt, f"l{i}")
        h = token_shift(norm(x, f"l{i}.norm1"), L["shift"])
        x = x + mixer(layer["type"], h, sub(L, "mix"), layer["mixer"], eps)
        if layer.get("mlp") is not None:
            x = x + swiglu(norm(x, f"l{i}.norm2"), sub(L, "mlp"))
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = norm(x, "final.norm") @ Wt["head"].T
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits
