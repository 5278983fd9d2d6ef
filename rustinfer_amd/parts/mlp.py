"""Dense SwiGLU feed-forward: ``down( silu(gate(x)) * up(x) )``.

Gate and up weights are stacked row-wise (gate first) so one product makes both
(crates/infer-worker/src/models/loader.rs:543-571); ``silu(z) = z / (1 + exp(-z))``
in 32-bit (crates/infer-worker/src/components/ffn_dense.rs:39-68,
crates/infer-backend-cuda/src/kernels/swiglu/swiglu.cu:294-343).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import DeferredNorm, FeedForward, ParamSpec, ProjectedPart, Runtime, split_normed
from .linear import Linear


class SwiGLUMLP(FeedForward):
    def __init__(self, hidden_size: int, intermediate_size: int, names: Optional[Dict[str, str]] = None,
                 delta_dtype: Optional[torch.dtype] = None):
        """``names``: the tensors' names (``gate``, ``up``, ``down``) where they are not the usual
        ``*_proj.weight``.  ``delta_dtype = torch.float32``: the down projection's 32-bit sums leave
        unrounded (for a block that norms what the feed-forward returns)."""
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.gate_up = Linear(self.hidden_size, 2 * self.intermediate_size)
        self.down = Linear(self.intermediate_size, self.hidden_size)
        self.names = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}
        if names:
            self.names.update(names)
        self.delta_dtype = delta_dtype

    def param_specs(self) -> Dict[str, ParamSpec]:
        h, i, n = self.hidden_size, self.intermediate_size, self.names
        return {n["gate"]: ParamSpec((i, h)), n["up"]: ParamSpec((i, h)), n["down"]: ParamSpec((h, i))}

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        gate = tensors[self.names["gate"]].to(device=rt.device, dtype=rt.dtype)
        up = tensors[self.names["up"]].to(device=rt.device, dtype=rt.dtype)
        self.gate_up.set_weight(torch.cat([gate, up], dim=0), rt)
        self.down.set_weight(tensors[self.names["down"]], rt)

    takes_deferred_norm = True

    def _activation(self, ctx, normed) -> torch.Tensor:
        """silu(gate) * up of the input rows (normalised, or with the norm's factor still to apply)."""
        rows, scale = split_normed(normed)
        T = rows.shape[0]
        ws = ctx.workspace
        act = ws.get("ffn.act", T, self.intermediate_size, self.rt.dtype)
        if scale is not None:
            self.rt.ops.linear_swiglu(rows, self.gate_up.weight, act, None, self.gate_up.weight_tiled, scale=scale)
        else:
            gate_up = ws.get("ffn.gate_up", T, 2 * self.intermediate_size, self.rt.dtype)
            self.rt.ops.linear_swiglu(rows, self.gate_up.weight, act, gate_up, self.gate_up.weight_tiled)
        return act

    def forward(self, ctx, normed) -> torch.Tensor:
        act = self._activation(ctx, normed)
        return self.rt.ops.linear_delta(act, self.down.weight, ctx.workspace, "ffn.out", self.down.weight_tiled,
                                        out_dtype=self.delta_dtype)

    def forward_into(self, ctx, normed, x: torch.Tensor, next_norm):
        """Few rows: the down projection adds its sums to ``x`` itself and prepares the input behind
        ``next_norm`` (see parts/base.py).  None, and nothing done, where that form does not apply."""
        ops = self.rt.ops
        ok = getattr(ops, "linear_residual_ok", None)
        if ok is None or not ok(x.shape[0], self.down.weight, self.down.weight_tiled, next_norm.weight):
            return None
        pays = getattr(ops, "linear_residual_pays", None)
        if pays is not None and not pays(x.shape[0], self.down.weight):
            return None
        act = self._activation(ctx, normed)
        a, ssq = ops.linear_residual(act, self.down.weight, self.down.weight_tiled, x, next_norm.weight,
                                     ctx.workspace, "deferred")
        return DeferredNorm(a, ssq, next_norm.eps)


class DenseMLP(ProjectedPart, FeedForward):
    """``down(f(up(x)))`` with an elementwise ``f`` of the kernels' list (``relu2``: the square of
    relu; ``tanh``).  Tensors ``up [ff, hidden]`` and ``down [hidden, ff]`` under the given names."""

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "relu2",
                 up_name: str = "up", down_name: str = "down"):
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.activation = activation
        self.up_name, self.down_name = up_name, down_name

    def in_projections(self):
        return [(self.up_name, self.intermediate_size)]

    def out_projection(self):
        return (self.down_name, self.intermediate_size)

    def core(self, ctx, proj, act, cache=None) -> None:
        self.rt.ops.unary(self.activation, proj[self.up_name], act)

    def forward(self, ctx, normed):
        return ProjectedPart.forward(self, ctx, normed, None)


class PolyNormMLP(ProjectedPart, FeedForward):
    """``W_down act(W_up x + b_up) + b_down`` with ``act(z) = a N(z) + b N(z^2) + c N(z^3) + e``: powers
    element by element, ``N`` divides a token's vector by its root mean square (``eps`` inside the root), and
    the four numbers are the tensor ``act``.  Tensors ``up, up.b, down, down.b, act`` unless given.  The
    down projection's bias is ``out_bias``: whoever adds the part's result to the stream adds it too."""

    def __init__(self, hidden_size: int, intermediate_size: int, eps: float, up_name: str = "up", down_name: str = "down",
                 bias_suffix: str = "b", act_name: str = "act"):
        self.hidden_size, self.intermediate_size, self.eps = int(hidden_size), int(intermediate_size), float(eps)
        self.up_name, self.down_name, self.act_name = up_name, down_name, act_name
        self.up_bias_name, self.down_bias_name = f"{up_name}.{bias_suffix}", f"{down_name}.{bias_suffix}"
        self.out_bias = None

    def in_projections(self):
        return [(self.up_name, self.intermediate_size)]

    def out_projection(self):
        return (self.down_name, self.intermediate_size)

    def own_specs(self):
        return {self.up_bias_name: ParamSpec((self.intermediate_size,), mean=0.0, std=0.1),
                self.down_bias_name: ParamSpec((self.hidden_size,), mean=0.0, std=0.1),
                self.act_name: ParamSpec((4,), mean=0.3, std=0.3)}

    def load_own(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        f32 = lambda name: tensors[name].to(device=rt.device, dtype=torch.float32).contiguous()
        self.up_bias, self.out_bias = f32(self.up_bias_name), f32(self.down_bias_name)
        self.coef = tuple(float(v) for v in tensors[self.act_name].to(torch.float32).flatten().tolist())
        if len(self.coef) != 4:
            raise ValueError(f"{self.act_name}: four numbers expected")

    def core(self, ctx, proj, act, cache=None) -> None:
        self.rt.ops.poly_norm(proj[self.up_name], self.up_bias, self.coef, self.eps, act)

    def forward(self, ctx, normed):
        """The result WITHOUT ``out_bias``."""
        return ProjectedPart.forward(self, ctx, normed, None)


class MoEFeedForward(FeedForward):
    """``experts`` gated feed-forwards of width ``expert_size`` of which every token uses ``top``: the
    router's logits ``W_router x`` and their softmax over all experts are 32-bit; the ``top`` largest
    probabilities are the chosen experts' weights (divided by their sum only with ``renormalize``); the
    output is the weighted sum of the chosen experts' ``W_down (silu(W_gate x) * W_up x)``.

    The experts' gate and up matrices are stacked into one product for all of them, every expert's
    activation is multiplied by its token's weight (0 where it was not chosen), and the experts' down
    matrices side by side make the weighted sum in ONE product: the router's product and three more
    launches whatever the number of experts, nothing that depends on which experts a token chose (so a step can be captured), and
    the same arithmetic for a token whatever else is in the step.  Every token pays for all experts;
    with few tokens in a step the experts' weights are read once either way.
    ``score = "sigmoid"``: each expert's score is the sigmoid of its own logit; with ``renormalize`` the
    chosen scores are divided by their sum + ``norm_eps``; ``scale`` multiplies the weights.
    ``shared_size`` > 0: one more gated feed-forward of that width (tensors ``shared.gate|up|down``) that every
    token uses with weight 1: its gate and up rows are stacked under the experts' and its down columns beside
    theirs, so it rides in the same two products.
    Tensor names: ``router``, ``e<i>.gate``, ``e<i>.up``, ``e<i>.down``."""

    # up to this many tokens in a step every block of the activation kernel makes its token's weights
    # itself (a launch less: 4.6 us of a step of 8 tokens); with more, the weights are made once a token
    # by a kernel of their own (a prompt of 2,048 tokens: 81 against 250 us a layer)
    ROUTE_ON_THE_WAY_ROWS = 64

    def __init__(self, hidden_size: int, expert_size: int, experts: int, top: int, renormalize: bool = False,
                 score: str = "softmax", norm_eps: float = 0.0, scale: float = 1.0, shared_size: int = 0):
        if not (0 < top <= experts):
            raise ValueError(f"top {top} of {experts} experts")
        if score not in ("softmax", "sigmoid"):
            raise ValueError(f"a router scores with 'softmax' or 'sigmoid', got {score!r}")
        self.hidden_size, self.expert_size = int(hidden_size), int(expert_size)
        self.experts, self.top, self.renormalize = int(experts), int(top), bool(renormalize)
        self.score, self.norm_eps, self.scale, self.shared_size = score, float(norm_eps), float(scale), int(shared_size)
        self.plain = score == "softmax" and self.scale == 1.0 and self.norm_eps == 0.0 and self.shared_size == 0
        # columns of the activations: the experts', the shared expert's, zeros up to a multiple of eight
        self.act_width = (self.experts * self.expert_size + self.shared_size + 7) // 8 * 8
        self.router = Linear(self.hidden_size, self.experts)
        self.gate_up = Linear(self.hidden_size, 2 * self.experts * self.expert_size + 2 * self.shared_size)
        self.down = Linear(self.act_width, self.hidden_size)

    def param_specs(self) -> Dict[str, ParamSpec]:
        h, f = self.hidden_size, self.expert_size
        specs = {"router": ParamSpec((self.experts, h))}
        for e in range(self.experts):
            specs[f"e{e}.gate"], specs[f"e{e}.up"], specs[f"e{e}.down"] = ParamSpec((f, h)), ParamSpec((f, h)), ParamSpec((h, f))
        if self.shared_size:
            s = self.shared_size
            specs["shared.gate"], specs["shared.up"], specs["shared.down"] = ParamSpec((s, h)), ParamSpec((s, h)), ParamSpec((h, s))
        return specs

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        to = lambda name: tensors[name].to(device=rt.device, dtype=rt.dtype)
        self.router.set_weight(to("router"), rt, tile=False)
        rows = [to(f"e{e}.{n}") for e in range(self.experts) for n in ("gate", "up")]
        cols = [to(f"e{e}.down") for e in range(self.experts)]
        if self.shared_size:
            rows += [to("shared.gate"), to("shared.up")]
            cols.append(to("shared.down"))
        pad = self.act_width - self.experts * self.expert_size - self.shared_size
        if pad:
            cols.append(torch.zeros((self.hidden_size, pad), device=rt.device, dtype=rt.dtype))
        self.gate_up.set_weight(torch.cat(rows, dim=0), rt)
        self.down.set_weight(torch.cat(cols, dim=1), rt)

    def forward(self, ctx, normed) -> torch.Tensor:
        ops, ws = self.rt.ops, ctx.workspace
        T, E, F = normed.shape[0], self.experts, self.expert_size
        logits = ws.get("moe.logits", T, E, torch.float32)
        self.router.forward(normed, logits)
        gate_up = ws.get("moe.gate_up", T, 2 * E * F + 2 * self.shared_size, self.rt.dtype)
        self.gate_up.forward(normed, gate_up)
        act = ws.get("moe.act", T, self.act_width, self.rt.dtype)
        how = {} if self.plain else {"score": self.score, "norm_eps": self.norm_eps, "scale": self.scale}
        shared = {} if self.plain else {"shared": self.shared_size}
        if T <= self.ROUTE_ON_THE_WAY_ROWS:
            ops.moe_swiglu_routed(gate_up, logits, act, E, F, self.top, self.renormalize, **how, **shared)
        else:
            weights = ws.get("moe.weights", T, E, torch.float32)
            ops.moe_route(logits, weights, self.top, self.renormalize, **how)
            ops.moe_swiglu_weighted(gate_up, weights, act, E, F, **shared)
        return ops.linear_delta(act, self.down.weight, ws, "moe.out", self.down.weight_tiled, out_dtype=torch.float32)
