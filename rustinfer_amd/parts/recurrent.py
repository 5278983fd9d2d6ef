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
