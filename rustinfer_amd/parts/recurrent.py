"""Mixers that keep a matrix of state for each head instead of a cache of keys.

Both walk a request's tokens in order through ``S [key rows, value columns]`` (32-bit, in the
request's state slot, zeros before its first token):

``LightningAttention``   ``S <- decay_h S + k v^T``, ``o = S^T q`` with q, k, v = silu of their
                         projections and one fixed decay for each head; the heads' outputs are
                         normalised together (RMS over all of them, a learned weight), gated by
                         ``sigmoid(W_g x)`` and projected.
``GeneralDeltaRule``     ``S <- diag(w) S - (a u)(u^T S) + k v^T``, ``o = S^T r``: ``u`` the key of
                         unit length, ``w = exp(-c sigmoid(W_w2 tanh(W_w1 x) + w0))`` a decay and
                         ``a = sigmoid(W_a x + b_a)`` a removal rate for each key channel (both
                         terms read the old state); each head's output is divided by its own root
                         mean square, then a learned weight, the gate and the projection.

``GatedDeltaRule``       ``S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q`` with one decay ``g`` and one
                         write strength ``beta`` a head and token; q, k, v pass a short causal convolution
                         and silu first, q and k are made unit vectors; each head's output is divided by its
                         root mean square, times a weight, times ``silu(W_g x)``.

The walk is one kernel for prompt portions and single tokens alike (``csrc/recurrent.hip``);
everything between the projections and the gated norm's output is 32-bit.
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Sequence

import torch

from .base import Mixer, ParamSpec, ProjectedPart, Runtime, StateNeed
from .linear import Linear


class LightningAttention(ProjectedPart, Mixer):
    is_mixer = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, v_head_dim: int, decay: Sequence[float],
                 norm_eps: float, names: Optional[Dict[str, str]] = None):
        if len(decay) != num_heads:
            raise ValueError(f"{len(decay)} decays for {num_heads} heads")
        self.hidden_size = int(hidden_size)
        self.num_heads, self.head_dim, self.v_head_dim = int(num_heads), int(head_dim), int(v_head_dim)
        self.decay_values = [float(x) for x in decay]
        self.norm_eps = float(norm_eps)
        self.names = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm"}
        if names:
            self.names.update(names)

    def in_projections(self):
        n, hk, hv = self.names, self.num_heads * self.head_dim, self.num_heads * self.v_head_dim
        return [(n["q"], hk), (n["k"], hk), (n["v"], hv), (n["g"], hv)]

    def out_projection(self):
        return (self.names["o"], self.num_heads * self.v_head_dim)

    def own_specs(self):
        return {self.names["norm"]: ParamSpec((self.num_heads * self.v_head_dim,), "norm")}

    def cache_need(self):
        return StateNeed((self.num_heads, self.head_dim, self.v_head_dim), torch.float32)

    def load_own(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.norm_weight = tensors[self.names["norm"]].to(device=rt.device, dtype=torch.float32).contiguous()
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=rt.device)

    def core(self, ctx, proj, act, cache) -> None:
        ops, n = self.rt.ops, self.names
        T = act.shape[0]
        o = ctx.workspace.get("scan.o", T, self.num_heads * self.v_head_dim, torch.float32)
        ops.linear_scan(proj[n["q"]], proj[n["k"]], proj[n["v"]], cache.state, o, ctx, self.num_heads,
                        self.head_dim, self.v_head_dim, decay=self.decay, silu_in=True)
        ops.gated_group_norm(o, self.norm_weight, proj[n["g"]], act, self.num_heads * self.v_head_dim, self.norm_eps)


class GeneralDeltaRule(ProjectedPart, Mixer):
    is_mixer = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, decay_rank: int, norm_eps: float,
                 decay_strength: float = math.exp(-0.5), unit_eps: float = 1e-6,
                 names: Optional[Dict[str, str]] = None):
        """``decay_rank``: rows of the first of the two matrices that make the decay's input;
        ``decay_strength``: the ``c`` of ``w = exp(-c sigmoid(.))``, so that ``w`` stays in
        ``(exp(-c), 1)``; ``unit_eps``: added to ``|k|^2`` under the root of the unit key."""
        self.hidden_size = int(hidden_size)
        self.num_heads, self.head_dim, self.decay_rank = int(num_heads), int(head_dim), int(decay_rank)
        self.norm_eps, self.decay_strength, self.unit_eps = float(norm_eps), float(decay_strength), float(unit_eps)
        self.names = {"r": "r", "k": "k", "v": "v", "g": "g", "a": "a", "a_bias": "a.b", "w1": "w1", "w2": "w2",
                      "w0": "w0", "o": "o", "norm": "norm"}
        if names:
            self.names.update(names)
        self.w2 = Linear(self.decay_rank, self.num_heads * self.head_dim)

    def in_projections(self):
        n, hd = self.names, self.num_heads * self.head_dim
        return [(n["r"], hd), (n["k"], hd), (n["v"], hd), (n["g"], hd), (n["a"], hd), (n["w1"], self.decay_rank)]

    def out_projection(self):
        return (self.names["o"], self.num_heads * self.head_dim)

    def own_specs(self):
        n, hd = self.names, self.num_heads * self.head_dim
        return {n["w2"]: ParamSpec((hd, self.decay_rank)), n["w0"]: ParamSpec((hd,), mean=0.0, std=1.0),
                n["a_bias"]: ParamSpec((hd,), mean=0.0, std=1.0), n["norm"]: ParamSpec((hd,), "norm")}

    def cache_need(self):
        return StateNeed((self.num_heads, self.head_dim, self.head_dim), torch.float32)

    def load_own(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        f32 = lambda name: tensors[name].to(device=rt.device, dtype=torch.float32).contiguous()
        self.w0, self.a_bias, self.norm_weight = f32(n["w0"]), f32(n["a_bias"]), f32(n["norm"])
        self.w2.set_weight(tensors[n["w2"]], rt)

    def core(self, ctx, proj, act, cache) -> None:
        ops, n = self.rt.ops, self.names
        T, hd = act.shape[0], self.num_heads * self.head_dim
        w1 = proj[n["w1"]]
        ops.unary("tanh", w1, w1)
        wl = ctx.workspace.get("gdr.wl", T, hd, self.rt.dtype)
        self.w2.forward(w1, wl)
        o = ctx.workspace.get("scan.o", T, hd, torch.float32)
        ops.linear_scan(proj[n["r"]], proj[n["k"]], proj[n["v"]], cache.state, o, ctx, self.num_heads,
                        self.head_dim, self.head_dim, wl=wl, al=proj[n["a"]], w0=self.w0, ab=self.a_bias,
                        unit_eps=self.unit_eps, decay_c=self.decay_strength)
        ops.gated_group_norm(o, self.norm_weight, proj[n["g"]], act, self.head_dim, self.norm_eps)


class Retention(ProjectedPart, Mixer):
    """``S <- decay_h S + k v^T``, ``o = S^T q`` with one fixed decay a head, no softmax and no
    denominator; q and k are turned by the token's position (``pos_enc``: the first ``rot_dim``
    features, feature i with i + rot_dim/2) and k is multiplied by ``key_scale`` after that; each head's
    ``o`` is divided by its root mean square (no weight), the heads are gated by ``silu(W_g x)`` and
    projected.  Rotation, state and norm are 32-bit.  Tensor names: ``q, k, v, g, o`` unless given."""

    is_mixer = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, v_head_dim: int, decay: Sequence[float],
                 norm_eps: float, pos_enc=None, key_scale: Optional[float] = None, names: Optional[Dict[str, str]] = None):
        if len(decay) != num_heads:
            raise ValueError(f"{len(decay)} decays for {num_heads} heads")
        self.hidden_size = int(hidden_size)
        self.num_heads, self.head_dim, self.v_head_dim = int(num_heads), int(head_dim), int(v_head_dim)
        self.decay_values = [float(x) for x in decay]
        self.norm_eps = float(norm_eps)
        self.pos_enc = pos_enc
        self.key_scale = float(key_scale) if key_scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.names = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o"}
        if names:
            self.names.update(names)

    def in_projections(self):
        n, hk, hv = self.names, self.num_heads * self.head_dim, self.num_heads * self.v_head_dim
        return [(n["q"], hk), (n["k"], hk), (n["v"], hv), (n["g"], hv)]

    def out_projection(self):
        return (self.names["o"], self.num_heads * self.v_head_dim)

    def cache_need(self):
        return StateNeed((self.num_heads, self.head_dim, self.v_head_dim), torch.float32)

    def load_own(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=rt.device)

    def core(self, ctx, proj, act, cache) -> None:
        ops, n = self.rt.ops, self.names
        o = ctx.workspace.get("scan.o", act.shape[0], self.num_heads * self.v_head_dim, torch.float32)
        ops.linear_scan(proj[n["q"]], proj[n["k"]], proj[n["v"]], cache.state, o, ctx, self.num_heads, self.head_dim,
                        self.v_head_dim, decay=self.decay, rotary=self.pos_enc.rotary() if self.pos_enc is not None else None,
                        k_scale=self.key_scale)
        ops.gated_group_norm(o, None, proj[n["g"]], act, self.v_head_dim, self.norm_eps, gate_activation="silu")


class GatedDeltaRule(ProjectedPart, Mixer):
    """The gated delta rule.  ``q = W_q x`` and ``k = W_k x`` have ``num_kv_heads`` heads of ``head_dim``,
    ``v = W_v x`` has ``num_heads`` heads of ``v_head_dim``; head h reads q/k head ``h // (num_heads //
    num_kv_heads)``.  Each of q, k, v passes a causal convolution over time of ``conv_taps`` taps, channel by
    channel (tensors ``<name>.conv`` ``[channels, taps]``, the last column the current token's, no bias), then
    silu.  q and k are divided by ``sqrt(|.|^2 + unit_eps)`` head by head, q also times ``q_scale``
    (``head_dim^(-1/2)`` unless given).  ``beta = sigmoid(W_b x)`` and
    ``g = exp(-exp(A_log) softplus(W_a x + dt_bias))``, one a head.  Per head, in this order:
    ``S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q``.  Each head's ``o`` is divided by its root
    mean square over ``v_head_dim`` (``norm_eps``), times the weight ``norm`` (``v_head_dim`` entries shared by
    the heads), times ``silu(W_g x)``; then ``W_o``.

    A request's slot holds the 32-bit state ``[heads, head_dim, v_head_dim]`` and the convolutions' last
    ``conv_taps - 1`` inputs; everything between the projections and the gated norm's output is 32-bit.
    Tensor names: ``q, k, v, g, b, a, o, q.conv, k.conv, v.conv, A_log, dt_bias, norm`` unless given."""

    is_mixer = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int,
                 conv_taps: int, norm_eps: float, unit_eps: float = 1e-6, q_scale: Optional[float] = None,
                 names: Optional[Dict[str, str]] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads {num_heads} is not a multiple of num_kv_heads {num_kv_heads}")
        if conv_taps < 1:
            raise ValueError("a convolution has one tap at least")
        self.hidden_size = int(hidden_size)
        self.num_heads, self.num_kv_heads = int(num_heads), int(num_kv_heads)
        self.head_dim, self.v_head_dim, self.conv_taps = int(head_dim), int(v_head_dim), int(conv_taps)
        self.norm_eps, self.unit_eps = float(norm_eps), float(unit_eps)
        self.q_scale = float(q_scale) if q_scale is not None else self.head_dim ** -0.5
        self.names = {"q": "q", "k": "k", "v": "v", "g": "g", "b": "b", "a": "a", "o": "o", "conv": "conv",
                      "A_log": "A_log", "dt_bias": "dt_bias", "norm": "norm"}
        if names:
            self.names.update(names)

    @property
    def conv_channels(self) -> int:
        return 2 * self.num_kv_heads * self.head_dim + self.num_heads * self.v_head_dim

    def in_projections(self):
        n, ck, cv, H = self.names, self.num_kv_heads * self.head_dim, self.num_heads * self.v_head_dim, self.num_heads
        return [(n["q"], ck), (n["k"], ck), (n["v"], cv), (n["g"], cv), (n["b"], H), (n["a"], H)]

    def out_projection(self):
        return (self.names["o"], self.num_heads * self.v_head_dim)

    def own_specs(self):
        n, ck, cv, H, t = self.names, self.num_kv_heads * self.head_dim, self.num_heads * self.v_head_dim, self.num_heads, self.conv_taps
        conv = lambda rows: ParamSpec((rows, t), mean=0.0, std=0.5)
        return {join_conv(n["q"], n["conv"]): conv(ck), join_conv(n["k"], n["conv"]): conv(ck), join_conv(n["v"], n["conv"]): conv(cv),
                n["A_log"]: ParamSpec((H,), mean=-1.0, std=1.0), n["dt_bias"]: ParamSpec((H,), mean=0.0, std=1.0),
                n["norm"]: ParamSpec((self.v_head_dim,), "norm")}

    def cache_need(self):
        extra = ()
        if self.conv_taps > 1:
            extra = (("conv", (self.conv_taps - 1, self.conv_channels), torch.float32),)
        return StateNeed((self.num_heads, self.head_dim, self.v_head_dim), torch.float32, extra)

    def load_own(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        if self.conv_taps > rt.ops.SHORT_CONV_MAX_TAPS:
            raise ValueError(f"a convolution of {self.conv_taps} taps is beyond the kernel ({rt.ops.SHORT_CONV_MAX_TAPS})")
        f32 = lambda name: tensors[name].to(device=rt.device, dtype=torch.float32).contiguous()
        self.conv_weights = [tensors[join_conv(n[x], n["conv"])].to(device=rt.device, dtype=rt.dtype).contiguous() for x in ("q", "k", "v")]
        self.decay_rate = torch.exp(f32(n["A_log"]))                       # A of g = exp(-A softplus(.)), 32-bit
        self.dt_bias = f32(n["dt_bias"])
        self.norm_weight = f32(n["norm"]).repeat(self.num_heads)          # the same weight for every head

    def core(self, ctx, proj, act, cache) -> None:
        ops, n, ws = self.rt.ops, self.names, ctx.workspace
        T, H, Hk, dk, dv = act.shape[0], self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim
        ck = Hk * dk
        mixed = ws.get("gdelta.conv", T, self.conv_channels, torch.float32)
        ops.short_conv([proj[n["q"]], proj[n["k"]], proj[n["v"]]], self.conv_weights,
                       cache.extra["conv"] if self.conv_taps > 1 else None, mixed, ctx, self.conv_taps, silu=True)
        o = ws.get("scan.o", T, H * dv, torch.float32)
        ops.gated_delta_scan(mixed[:, :ck], mixed[:, ck:2 * ck], mixed[:, 2 * ck:], proj[n["b"]], proj[n["a"]],
                             self.decay_rate, self.dt_bias, cache.state, o, ctx, H, Hk, dk, dv,
                             unit_eps=self.unit_eps, q_scale=self.q_scale)
        ops.gated_group_norm(o, self.norm_weight, proj[n["g"]], act, dv, self.norm_eps, gate_activation="silu")


def join_conv(name: str, suffix: str) -> str:
    return f"{name}.{suffix}"


def _f32(tensors, name: str, rt: Runtime) -> torch.Tensor:
    return tensors[name].to(device=rt.device, dtype=torch.float32).contiguous()


class ChannelGatedDeltaRule(ProjectedPart, Mixer):
    """The gated delta rule with a decay for every key channel.  q, k (``num_kv_heads`` heads of ``head_dim``)
    and v (``num_heads`` heads of ``v_head_dim``; head h reads q/k head ``h // (num_heads // num_kv_heads)``)
    pass a causal convolution of ``conv_taps`` taps channel by channel (``<name>.conv`` ``[channels, taps]``, the
    last column the current token's, no bias) and silu; q and k are divided by ``sqrt(|.|^2 + unit_eps)`` head by
    head, q also times ``q_scale`` (``head_dim^(-1/2)`` unless given).  ``beta = sigmoid(W_b x)``, one a head;
    ``g = exp(-exp(A_log_h) softplus(W_a2 (W_a1 x) + dt_bias))`` laid out heads x head_dim, acting on the state's
    rows.  Per head, in this order: ``S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q``.  Each
    head's ``o`` is divided by its root mean square over ``v_head_dim`` (``norm_eps``), times the weight ``norm``
    (``v_head_dim`` entries shared by the heads), times ``sigmoid(W_g2 (W_g1 x))`` laid out heads x v_head_dim;
    then ``W_o``.  ``decay_rank``, ``gate_rank``: rows of ``a1`` and ``g1``.

    A request's slot holds the 32-bit state ``[heads, head_dim, v_head_dim]`` and the convolutions' last
    ``conv_taps - 1`` inputs; everything between the projections and the gated norm's output is 32-bit.
    Tensor names: ``q, k, v, b, a1, a2, g1, g2, o, q.conv, k.conv, v.conv, A_log, dt_bias, norm`` unless given."""

    is_mixer = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int,
                 conv_taps: int, decay_rank: int, gate_rank: int, norm_eps: float, unit_eps: float = 1e-6,
                 q_scale: Optional[float] = None, names: Optional[Dict[str, str]] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads {num_heads} is not a multiple of num_kv_heads {num_kv_heads}")
        if conv_taps < 1:
            raise ValueError("a convolution has one tap at least")
        self.hidden_size = int(hidden_size)
        self.num_heads, self.num_kv_heads = int(num_heads), int(num_kv_heads)
        self.head_dim, self.v_head_dim, self.conv_taps = int(head_dim), int(v_head_dim), int(conv_taps)
        self.decay_rank, self.gate_rank = int(decay_rank), int(gate_rank)
        self.norm_eps, self.unit_eps = float(norm_eps), float(unit_eps)
        self.q_scale = float(q_scale) if q_scale is not None else self.head_dim ** -0.5
        self.names = {"q": "q", "k": "k", "v": "v", "b": "b", "a1": "a1", "a2": "a2", "g1": "g1", "g2": "g2", "o": "o",
                      "conv": "conv", "A_log": "A_log", "dt_bias": "dt_bias", "norm": "norm"}
        if names:
            self.names.update(names)
        self.a2 = Linear(self.decay_rank, self.num_heads * self.head_dim)
        self.g2 = Linear(self.gate_rank, self.num_heads * self.v_head_dim)

    @property
    def conv_channels(self) -> int:
        return 2 * self.num_kv_heads * self.head_dim + self.num_heads * self.v_head_dim

    def in_projections(self):
        n, ck, cv = self.names, self.num_kv_heads * self.head_dim, self.num_heads * self.v_head_dim
        return [(n["q"], ck), (n["k"], ck), (n["v"], cv), (n["b"], self.num_heads), (n["a1"], self.decay_rank),
                (n["g1"], self.gate_rank)]

    def out_projection(self):
        return (self.names["o"], self.num_heads * self.v_head_dim)

    def own_specs(self):
        n, H, dk, dv, t = self.names, self.num_heads, self.head_dim, self.v_head_dim, self.conv_taps
        ck, cv = self.num_kv_heads * dk, H * dv
        conv = lambda rows: ParamSpec((rows, t), mean=0.0, std=0.5)
        return {join_conv(n["q"], n["conv"]): conv(ck), join_conv(n["k"], n["conv"]): conv(ck), join_conv(n["v"], n["conv"]): conv(cv),
                n["a2"]: ParamSpec((H * dk, self.decay_rank), mean=0.0, std=0.3), n["g2"]: ParamSpec((cv, self.gate_rank), mean=0.0, std=0.3),
                n["A_log"]: ParamSpec((H,), mean=-1.0, std=1.0), n["dt_bias"]: ParamSpec((H * dk,), mean=0.0, std=1.0),
                n["norm"]: ParamSpec((dv,), "norm")}

    def cache_need(self):
        extra = ()
        if self.conv_taps > 1:
            extra = (("conv", (self.conv_taps - 1, self.conv_channels), torch.float32),)
        return StateNeed((self.num_heads, self.head_dim, self.v_head_dim), torch.float32, extra)

    def load_own(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        if self.conv_taps > rt.ops.SHORT_CONV_MAX_TAPS:
            raise ValueError(f"a convolution of {self.conv_taps} taps is beyond the kernel ({rt.ops.SHORT_CONV_MAX_TAPS})")
        self.conv_weights = [tensors[join_conv(n[x], n["conv"])].to(device=rt.device, dtype=rt.dtype).contiguous() for x in ("q", "k", "v")]
        self.decay_rate = torch.exp(_f32(tensors, n["A_log"], rt))
        self.dt_bias = _f32(tensors, n["dt_bias"], rt)
        self.norm_weight = _f32(tensors, n["norm"], rt).repeat(self.num_heads)
        self.a2.set_weight(tensors[n["a2"]], rt)
        self.g2.set_weight(tensors[n["g2"]], rt)

    def core(self, ctx, proj, act, cache) -> None:
        ops, n, ws = self.rt.ops, self.names, ctx.workspace
        T, H, Hk, dk, dv = act.shape[0], self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim
        ck = Hk * dk
        mixed = ws.get("gdelta.conv", T, self.conv_channels, torch.float32)
        ops.short_conv([proj[n["q"]], proj[n["k"]], proj[n["v"]]], self.conv_weights,
                       cache.extra["conv"] if self.conv_taps > 1 else None, mixed, ctx, self.conv_taps, silu=True)
        decay_in = ws.get("gdelta.decay_in", T, H * dk, torch.float32)      # the decays' inputs leave their product unrounded
        self.a2.forward(proj[n["a1"]], decay_in)
        gate_in = ws.get("gdelta.gate_in", T, H * dv, self.rt.dtype)
        self.g2.forward(proj[n["g1"]], gate_in)
        o = ws.get("scan.o", T, H * dv, torch.float32)
        ops.channel_delta_scan(mixed[:, :ck], mixed[:, ck:2 * ck], mixed[:, 2 * ck:], proj[n["b"]], decay_in,
                               self.decay_rate, self.dt_bias, cache.state, o, ctx, H, Hk, dk, dv,
                               unit_eps=self.unit_eps, q_scale=self.q_scale)
        ops.gated_group_norm(o, self.norm_weight, gate_in, act, dv, self.norm_eps, gate_activation="sigmoid")


class GatedLinearAttention(ProjectedPart, Mixer):
    """``S <- diag(alpha) S + k v^T``, ``o = S^T q`` per head with ``q = W_q x * q_scale`` (``head_dim^(-1/2)`` unless
    given), ``k = W_k x`` (heads of ``head_dim``), ``v = W_v x`` (heads of ``v_head_dim``) and a decay for every key
    channel, ``alpha = sigmoid(W_a2 (W_a1 x) + b)^(1 / tau)`` laid out heads x head_dim.  Each head's ``o`` is
    divided by its root mean square (``norm_eps``), times the weight ``norm`` (``v_head_dim`` entries shared by the
    heads); the heads side by side are multiplied by ``silu(W_g x)`` and projected.  State, decays and norm are
    32-bit.  Tensor names: ``q, k, v, g, a1, a2, a2.b, o, norm`` unless given."""

    is_mixer = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, v_head_dim: int, tau: float, decay_rank: int,
                 norm_eps: float, q_scale: Optional[float] = None, names: Optional[Dict[str, str]] = None):
        self.hidden_size = int(hidden_size)
        self.num_heads, self.head_dim, self.v_head_dim = int(num_heads), int(head_dim), int(v_head_dim)
        self.tau, self.decay_rank, self.norm_eps = float(tau), int(decay_rank), float(norm_eps)
        self.q_scale = float(q_scale) if q_scale is not None else self.head_dim ** -0.5
        self.names = {"q": "q", "k": "k", "v": "v", "g": "g", "a1": "a1", "a2": "a2", "a2_bias": "a2.b", "o": "o", "norm": "norm"}
        if names:
            self.names.update(names)
        self.a2 = Linear(self.decay_rank, self.num_heads * self.head_dim)

    def in_projections(self):
        n, hk, hv = self.names, self.num_heads * self.head_dim, self.num_heads * self.v_head_dim
        return [(n["q"], hk), (n["k"], hk), (n["v"], hv), (n["g"], hv), (n["a1"], self.decay_rank)]

    def out_projection(self):
        return (self.names["o"], self.num_heads * self.v_head_dim)

    def own_specs(self):
        n, hk = self.names, self.num_heads * self.head_dim
        return {n["a2"]: ParamSpec((hk, self.decay_rank), mean=0.0, std=0.3), n["a2_bias"]: ParamSpec((hk,), mean=3.0, std=1.0),
                n["norm"]: ParamSpec((self.v_head_dim,), "norm")}

    def cache_need(self):
        return StateNeed((self.num_heads, self.head_dim, self.v_head_dim), torch.float32)

    def load_own(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        self.decay_bias = _f32(tensors, n["a2_bias"], rt)
        self.norm_weight = _f32(tensors, n["norm"], rt).repeat(self.num_heads)
        self.a2.set_weight(tensors[n["a2"]], rt)

    def core(self, ctx, proj, act, cache) -> None:
        ops, n, ws = self.rt.ops, self.names, ctx.workspace
        T, H, dk, dv = act.shape[0], self.num_heads, self.head_dim, self.v_head_dim
        decay_in = ws.get("gla.decay_in", T, H * dk, torch.float32)         # the decays' inputs leave their product unrounded
        self.a2.forward(proj[n["a1"]], decay_in)
        o = ws.get("scan.o", T, H * dv, torch.float32)
        ops.decay_scan("channel", proj[n["q"]], proj[n["k"]], proj[n["v"]], decay_in, self.decay_bias, cache.state, o, ctx,
                       H, H, dk, dv, tau=self.tau, q_scale=self.q_scale)
        ops.gated_group_norm(o, self.norm_weight, proj[n["g"]], act, dv, self.norm_eps, gate_activation="silu")


class StateSpaceMixer(ProjectedPart, Mixer):
    """A state-space layer in its recurrent form.  One projection of ``2 inner + 2 groups state + heads`` rows
    (``inner = num_heads * v_head_dim``) gives ``[z | x | B | C | dt]``; x, B and C together pass a causal
    convolution of ``conv_taps`` taps channel by channel (weight ``conv [channels, taps]``, bias ``conv.b``) and
    silu.  ``dt <- softplus(dt + dt_bias)``.  Per head (head h reads B and C of group ``h // (num_heads //
    groups)``): ``S <- exp(-exp(A_log_h) dt) S + dt B x^T`` (``S`` is ``state x v_head_dim``), ``y = S^T C + D_h x``.
    The heads' ``y`` side by side are multiplied by ``silu(z)`` and then normed in ``norm_groups`` equal parts
    (``norm_eps``), times the weight ``norm`` (``inner`` entries); then ``W_o``.

    A request's slot holds the 32-bit state ``[heads, state, v_head_dim]`` and the convolution's last
    ``conv_taps - 1`` inputs.  Tensor names: ``in, conv, conv.b, dt_bias, A_log, D, norm, o`` unless given."""

    is_mixer = True

    def __init__(self, hidden_size: int, num_heads: int, v_head_dim: int, state_dim: int, groups: int, conv_taps: int,
                 norm_groups: int, norm_eps: float, names: Optional[Dict[str, str]] = None):
        if num_heads % groups or (num_heads * v_head_dim) % norm_groups:
            raise ValueError("heads must be a multiple of groups and heads * v_head_dim of norm_groups")
        if conv_taps < 1:
            raise ValueError("a convolution has one tap at least")
        self.hidden_size = int(hidden_size)
        self.num_heads, self.v_head_dim, self.state_dim = int(num_heads), int(v_head_dim), int(state_dim)
        self.groups, self.conv_taps, self.norm_groups, self.norm_eps = int(groups), int(conv_taps), int(norm_groups), float(norm_eps)
        self.inner = self.num_heads * self.v_head_dim
        self.names = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "A_log": "A_log", "D": "D",
                      "norm": "norm", "o": "o"}
        if names:
            self.names.update(names)

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state_dim

    def in_projections(self):
        return [(self.names["in"], 2 * self.inner + 2 * self.groups * self.state_dim + self.num_heads)]

    def out_projection(self):
        return (self.names["o"], self.inner)

    def own_specs(self):
        n, H, C = self.names, self.num_heads, self.conv_channels
        return {n["conv"]: ParamSpec((C, self.conv_taps), mean=0.0, std=0.5), n["conv_bias"]: ParamSpec((C,), mean=0.0, std=0.1),
                n["dt_bias"]: ParamSpec((H,), mean=0.0, std=1.0), n["A_log"]: ParamSpec((H,), mean=-1.0, std=1.0),
                n["D"]: ParamSpec((H,), mean=1.0, std=0.3), n["norm"]: ParamSpec((self.inner,), "norm")}

    def cache_need(self):
        extra = ()
        if self.conv_taps > 1:
            extra = (("conv", (self.conv_taps - 1, self.conv_channels), torch.float32),)
        return StateNeed((self.num_heads, self.state_dim, self.v_head_dim), torch.float32, extra)

    def load_own(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        if self.conv_taps > rt.ops.SHORT_CONV_MAX_TAPS:
            raise ValueError(f"a convolution of {self.conv_taps} taps is beyond the kernel ({rt.ops.SHORT_CONV_MAX_TAPS})")
        self.conv_weight = tensors[n["conv"]].to(device=rt.device, dtype=rt.dtype).contiguous()
        self.conv_bias = _f32(tensors, n["conv_bias"], rt)
        self.dt_bias, self.skip, self.norm_weight = _f32(tensors, n["dt_bias"], rt), _f32(tensors, n["D"], rt), _f32(tensors, n["norm"], rt)
        self.decay_rate = torch.exp(_f32(tensors, n["A_log"], rt))

    def core(self, ctx, proj, act, cache) -> None:
        ops, ws = self.rt.ops, ctx.workspace
        p = proj[self.names["in"]]
        T, H, N, G, inner = act.shape[0], self.num_heads, self.state_dim, self.groups, self.inner
        z, xbc, dt = p[:, :inner], p[:, inner:inner + self.conv_channels], p[:, inner + self.conv_channels:]
        mixed = ws.get("ssm.conv", T, self.conv_channels, torch.float32)
        ops.short_conv([xbc], [self.conv_weight], cache.extra["conv"] if self.conv_taps > 1 else None, mixed, ctx,
                       self.conv_taps, silu=True, biases=[self.conv_bias])
        x, B, C = mixed[:, :inner], mixed[:, inner:inner + G * N], mixed[:, inner + G * N:]
        y = ws.get("scan.o", T, inner, torch.float32)
        ops.decay_scan("head", C, B, x, dt, self.dt_bias, cache.state, y, ctx, H, G, N, self.v_head_dim,
                       rate=self.decay_rate, skip=self.skip)
        ops.gated_group_norm(y, self.norm_weight, z, act, inner // self.norm_groups, self.norm_eps, gate_activation="silu",
                             gate_first=True)
