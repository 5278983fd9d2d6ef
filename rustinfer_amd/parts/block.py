"""The arrangement of parts in one layer: pre-norm residual.

``x <- x + mixer(norm1(x)); x <- x + ffn(norm2(x))``.  A sub-layer's output is not
added at once: it stays *pending* and the next norm adds it while it normalises
(crates/infer-worker/src/components/attention.rs:83-95,179,
crates/infer-worker/src/components/ffn_dense.rs:97-113).  Either half may be absent.

With few tokens in a step a norm's kernel takes as long as a product, so a sub-layer that
can (``forward_into``) adds its output to the residual stream itself and hands the next
sub-layer a ``DeferredNorm``: the norm between them is done by the two products around it.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import (FeedForward, Mixer, Norm, ParamSpec, Part, ProjectionSet, Runtime, join_name, narrow_tensors,
                   with_state_extra)


class Hidden:
    """Residual stream ``x`` (32-bit, [T, hidden]) and either a delta not yet added to it
    (``pending``) or, with ``x`` complete, the input that a sub-layer has already prepared for
    the sub-layer behind a given norm (``deferred = (that norm, DeferredNorm)``)."""

    __slots__ = ("x", "pending", "deferred", "act")

    def __init__(self, x: torch.Tensor):
        self.x = x
        self.pending = None
        self.deferred = None
        self.act = None          # x rounded to the run dtype, if a block has left it (blocks whose sub-layers read x itself)

    def input_behind(self, ctx, norm, out: torch.Tensor):
        """What the sub-layer behind ``norm`` reads: the prepared input if there is one for this
        norm, else ``norm`` run into ``out`` (adding the pending delta)."""
        if self.deferred is not None:
            made_for, prepared = self.deferred
            self.deferred = None
            if made_for is norm:
                return prepared
        norm.forward(ctx, self.x, self.pending, out)
        self.pending = None
        return out


class TokenShift(Part):
    """What a sub-layer reads is mixed with what it read one token earlier, channel by channel:
    ``h_t <- h_t + (h_(t-1) - h_t) * mix`` with ``h_(t-1)`` as it was before its own mixing, zeros before a
    sequence's first token.  The last ``h`` of every request stays in its state slot (32-bit, the tensor
    ``state_name`` there), so prompt portions and single tokens go the same way.  The tensor ``mix``
    (the model's width) carries the part's own name."""

    state_name = "shift"

    def __init__(self, dim: int):
        self.dim = int(dim)
        self.mix = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"": ParamSpec((self.dim,), mean=0.5, std=0.2)}

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.mix = tensors[""].to(device=rt.device, dtype=torch.float32).contiguous()

    def state_of(self, cache):
        state = getattr(cache, "state", None)
        view = state if hasattr(state, "extra") else cache       # a CompoundView holds the StateView; a StateView is it
        return view.extra[self.state_name]

    def forward(self, ctx, h32: torch.Tensor, cache, out: torch.Tensor) -> torch.Tensor:
        """``h32 [T, dim]``: the normed rows in 32-bit; ``out`` takes the mixed rows in the run dtype."""
        self.rt.ops.token_shift(h32, self.mix, self.state_of(cache), out, ctx)
        return out


class PreNormBlock(Part):
    def __init__(self, hidden_size: int,
                 mixer_norm: Optional[Norm], mixer: Optional[Mixer],
                 ffn_norm: Optional[Norm], ffn: Optional[FeedForward],
                 names: Optional[Dict[str, str]] = None, mixer_shift: Optional[TokenShift] = None):
        """``mixer_shift``: a ``TokenShift`` between the mixer's norm and the mixer; the block then asks for
        one more tensor in the request's state slot, beside whatever the mixer keeps."""
        self.hidden_size = int(hidden_size)
        self.mixer_norm, self.mixer = mixer_norm, mixer
        self.ffn_norm, self.ffn = ffn_norm, ffn
        self.mixer_shift = mixer_shift
        if (mixer is None) != (mixer_norm is None) or (ffn is None) != (ffn_norm is None):
            raise ValueError("a sub-layer and its norm come together")
        if mixer_shift is not None and mixer is None:
            raise ValueError("a token shift stands in front of a mixer")
        self.names = {"mixer_norm": "input_layernorm", "mixer": "self_attn",
                      "ffn_norm": "post_attention_layernorm", "ffn": "mlp", "mixer_shift": "shift"}
        if names:
            self.names.update(names)

    def _children(self):
        for key in ("mixer_norm", "mixer_shift", "mixer", "ffn_norm", "ffn"):
            part = getattr(self, key)
            if part is not None:
                yield self.names[key], part

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs = {}
        for prefix, part in self._children():
            for name, spec in part.param_specs().items():
                specs[join_name(prefix, name)] = spec
        return specs

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        for prefix, part in self._children():
            sub = narrow_tensors(tensors, prefix)
            part.load(sub, rt)

    def cache_need(self):
        need = self.mixer.cache_need() if self.mixer is not None else None
        if self.mixer_shift is not None:
            need = with_state_extra(need, self.mixer_shift.state_name, (self.hidden_size,))
        return need

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", True) for _, part in self._children())

    def can_cut_rows(self) -> bool:
        """Whether forward() can leave the residual stream with a subset of its rows."""
        return self.ffn is not None and getattr(self.ffn_norm, "cuts_rows", False)

    takes_follow = True          # forward() accepts ``follow``

    def entry(self):
        """(norm, sub-layer) that a step enters this block through."""
        if self.mixer_shift is not None:
            return (self.mixer_norm, None)       # nobody else can prepare what the shift reads
        return (self.mixer_norm, self.mixer) if self.mixer is not None else (self.ffn_norm, self.ffn)

    def _mixer_input(self, ctx, hidden: "Hidden", cache, normed: torch.Tensor):
        """What the mixer reads: the normed rows, through the token shift if the block has one (the norm then
        leaves 32-bit rows, and the shift rounds once)."""
        if self.mixer_shift is None:
            return hidden.input_behind(ctx, self.mixer_norm, normed)
        fused = getattr(self.mixer_norm, "forward_shifted", None)
        if fused is not None and ctx.max_q_len == 1 and normed.shape[0] <= ctx.num_rows:
            # every row is one token: norm and shift are one kernel (the previous rows come from the slots alone)
            hidden.deferred = None
            fused(ctx, hidden.x, hidden.pending, normed, self.mixer_shift.mix, self.mixer_shift.state_of(cache))
            hidden.pending = None
            return normed
        h32 = ctx.workspace.get("block.normed32", normed.shape[0], self.hidden_size, torch.float32)
        hidden.deferred = None
        self.mixer_norm.forward(ctx, hidden.x, hidden.pending, h32)
        hidden.pending = None
        return self.mixer_shift.forward(ctx, h32, cache, normed)

    def forward(self, ctx, hidden: Hidden, cache, out_rows: Optional[torch.Tensor] = None, follow=None) -> None:
        """``out_rows`` (row indices on the device): nothing after this block needs the other
        rows.  The mixer still sees every token (it fills the cache), but the feed-forward half
        runs on those rows only, and ``hidden`` leaves with them alone.
        ``follow``: (norm, sub-layer) that come after this block (the next block's ``entry()``, or
        the final norm and the head), if the caller allows the last sub-layer here to prepare
        that sub-layer's input."""
        T = hidden.x.shape[0]
        normed = ctx.workspace.get("block.normed", T, self.hidden_size, self.rt.dtype)
        if self.mixer is not None:
            inp = self._mixer_input(ctx, hidden, cache, normed)
            after = (self.ffn_norm, self.ffn) if self.ffn is not None else follow
            self._run(self.mixer, ctx, hidden, inp, after if out_rows is None or self.ffn is None else None, cache)
        if self.ffn is not None:
            if out_rows is not None:
                W = out_rows.numel()
                x_rows = ctx.workspace.get("block.x_rows", W, self.hidden_size, torch.float32)
                normed = ctx.workspace.get("block.normed_rows", W, self.hidden_size, self.rt.dtype)
                self.ffn_norm.forward(ctx, hidden.x, hidden.pending, normed, rows=out_rows, x_rows=x_rows)
                hidden.x, hidden.pending, hidden.deferred = x_rows, None, None
                hidden.pending = self.ffn.forward(ctx, normed)
            else:
                inp = hidden.input_behind(ctx, self.ffn_norm, normed)
                self._run(self.ffn, ctx, hidden, inp, follow)

    def update_cache_only(self, ctx, hidden: Hidden, cache) -> None:
        """The last block of a step whose logits nobody wants (a prompt portion before the last):
        only what later steps read is made.  A mixer that has ``update_cache`` fills its cache and
        computes no output; any other mixer runs whole (its state must move on); the feed-forward
        half is left out.  ``hidden`` is not meaningful afterwards."""
        if self.mixer is None:
            return
        normed = ctx.workspace.get("block.normed", hidden.x.shape[0], self.hidden_size, self.rt.dtype)
        inp = self._mixer_input(ctx, hidden, cache, normed)
        update = getattr(self.mixer, "update_cache", None)
        if update is not None:
            update(ctx, inp, cache)
        else:
            self.mixer.forward(ctx, inp, cache)

    def _run(self, part, ctx, hidden: Hidden, inp, after, *cache) -> None:
        """Run a sub-layer.  If it can (``forward_into``), the norm after it is a plain RMS norm and the
        sub-layer behind that norm takes a ``DeferredNorm``, it adds its output to the residual stream
        itself and prepares that sub-layer's input; else its output stays pending."""
        into = getattr(part, "forward_into", None)
        if into is not None and after is not None:
            norm, consumer = after
            if getattr(norm, "plain_rms", False) and getattr(consumer, "takes_deferred_norm", False):
                prepared = into(ctx, inp, *cache, hidden.x, norm)
                if prepared is not None:
                    hidden.pending, hidden.deferred = None, (norm, prepared)
                    return
        hidden.pending, hidden.deferred = part.forward(ctx, inp, *cache), None


class ParallelBlock(Part):
    """One norm, and a mixer and a feed-forward that both read it:
    ``n = norm(x); x <- x + mixer(n) + ffn(n)``.  Either sub-layer may be absent.

    Both sub-layers are ``ProjectedPart``: their input projections are one product of ``n``, their
    output projections one product over the concatenated activations, whose result is the block's
    one delta (left pending for the next norm, as in ``PreNormBlock``)."""

    takes_follow = False

    def __init__(self, hidden_size: int, norm: Norm, mixer=None, ffn=None, names: Optional[Dict[str, str]] = None):
        if mixer is None and ffn is None:
            raise ValueError("a block needs a mixer or a feed-forward")
        self.hidden_size = int(hidden_size)
        self.norm, self.mixer, self.ffn = norm, mixer, ffn
        self.names = {"norm": "norm", "mixer": "mixer", "ffn": "ffn"}
        if names:
            self.names.update(names)
        members = [(self.names[key], part) for key, part in (("mixer", mixer), ("ffn", ffn)) if part is not None]
        self.set = ProjectionSet(self.hidden_size, members)

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs = {join_name(self.names["norm"], n): s for n, s in self.norm.param_specs().items()}
        specs.update(self.set.param_specs())
        return specs

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.norm.load(narrow_tensors(tensors, self.names["norm"]), rt)
        self.set.load(tensors, rt)

    def cache_need(self):
        return self.mixer.cache_need() if self.mixer is not None else None

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", True) for p in (self.norm, self.mixer, self.ffn) if p is not None)

    def can_cut_rows(self) -> bool:
        return False

    def entry(self):
        return (self.norm, None)

    def _run(self, ctx, hidden: Hidden, cache, mixer_only: bool):
        normed = ctx.workspace.get("block.normed", hidden.x.shape[0], self.hidden_size, self.rt.dtype)
        inp = hidden.input_behind(ctx, self.norm, normed)
        proj, act = self.set.project(ctx, inp)
        i = 0
        if self.mixer is not None:
            self.mixer.core(ctx, self.set.views(0, proj), self.set.act_view(0, act), cache)
            i = 1
        if mixer_only:
            return None
        if self.ffn is not None:
            self.ffn.core(ctx, self.set.views(i, proj), self.set.act_view(i, act), None)
        return self.set.output(ctx, act)

    def forward(self, ctx, hidden: Hidden, cache, out_rows=None, follow=None) -> None:
        hidden.pending, hidden.deferred = self._run(ctx, hidden, cache, False), None

    def update_cache_only(self, ctx, hidden: Hidden, cache) -> None:
        """The last block of a step whose logits nobody wants: the mixer alone runs, for what it
        leaves in its cache or state; ``hidden`` is not meaningful afterwards."""
        if self.mixer is not None:
            self._run(ctx, hidden, cache, True)


class PostNormBlock(Part):
    """Sub-layers that read the residual stream itself, and a norm on what each returns:
    ``x <- x + norm1(mixer(x)); x <- x + norm2(ffn(x))`` (the norms are ``OutputRMSNorm``: they carry
    the factor on the branch and add to the stream themselves).  The feed-forward may be absent.

    The stream is 32-bit; a sub-layer is given its rounding to the run dtype, which the norm before
    it writes beside the stream in the same pass (``Hidden.act``); in a 32-bit run it is the stream."""

    takes_follow = False
    leaves_act = True            # forward() leaves the stream's rounding in Hidden.act

    def __init__(self, hidden_size: int, mixer: Mixer, mixer_norm: Norm, ffn: Optional[FeedForward] = None,
                 ffn_norm: Optional[Norm] = None, names: Optional[Dict[str, str]] = None):
        if mixer is None or mixer_norm is None or (ffn is None) != (ffn_norm is None):
            raise ValueError("a block needs a mixer, and a sub-layer and its norm come together")
        self.hidden_size = int(hidden_size)
        self.mixer, self.mixer_norm, self.ffn, self.ffn_norm = mixer, mixer_norm, ffn, ffn_norm
        self.names = {"mixer_norm": "norm1", "mixer": "mix", "ffn_norm": "norm2", "ffn": "mlp"}
        if names:
            self.names.update(names)

    def _children(self):
        for key in ("mixer_norm", "mixer", "ffn_norm", "ffn"):
            part = getattr(self, key)
            if part is not None:
                yield self.names[key], part

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs = {}
        for prefix, part in self._children():
            for name, spec in part.param_specs().items():
                specs[join_name(prefix, name)] = spec
        return specs

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        for prefix, part in self._children():
            part.load(narrow_tensors(tensors, prefix), rt)

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", True) for _, part in self._children())

    def can_cut_rows(self) -> bool:
        return False

    def entry(self):
        return (None, self.mixer)

    def forward(self, ctx, hidden: Hidden, cache, out_rows=None, follow=None) -> None:
        x = hidden.x
        if hidden.pending is not None or hidden.deferred is not None:
            raise RuntimeError("a block whose sub-layers read the stream itself needs the stream complete")
        exact = self.rt.dtype == torch.float32
        act = None if exact else ctx.workspace.get("block.stream_act", x.shape[0], self.hidden_size, self.rt.dtype)
        if not exact and hidden.act is None:
            self.rt.ops.norm_residual(x, None, None, 1.0, act=act)       # the stream's rounding, nothing added
        inp = x if exact else act
        self.mixer_norm.add(ctx, x, self.mixer.forward(ctx, inp, cache), act)
        if self.ffn is not None:
            self.ffn_norm.add(ctx, x, self.ffn.forward(ctx, inp), act)
        hidden.act = act


class SandwichBlock(Part):
    """A norm before and after each sub-layer, and a gate on what the sub-layer returns:
    ``h = norm1(x); x <- x + norm1b(mixer(h) * sigmoid(W_g1 h + b_g1))``, then the same around the
    feed-forward with ``norm2``, ``norm2b`` and ``W_g2``.  The norms are ``LayerNorm``; the feed-forward
    may be absent.

    The gate reads what its sub-layer reads, so with a ``ProjectedPart`` its matrix is stacked on the
    part's in-projections (one product); any other sub-layer gets a product for the gate beside it.
    Gate, output norm and residual add are one kernel, which also leaves the input of the sub-layer that
    comes next where that sub-layer's norm is a ``LayerNorm`` (the norm's own kernel then runs only at a
    block's start where something else changes the stream first).  A sub-layer may have
    ``out_bias`` (32-bit, the model's width): it is added to what the sub-layer returns."""

    takes_follow = True

    def __init__(self, hidden_size: int, mixer_norm: Norm, mixer: Mixer, mixer_out_norm: Norm,
                 ffn_norm: Optional[Norm] = None, ffn: Optional[FeedForward] = None, ffn_out_norm: Optional[Norm] = None,
                 names: Optional[Dict[str, str]] = None):
        if mixer is None or mixer_norm is None or mixer_out_norm is None:
            raise ValueError("a block needs a mixer with a norm before and after it")
        if len({ffn is None, ffn_norm is None, ffn_out_norm is None}) != 1:
            raise ValueError("a feed-forward and its two norms come together")
        self.hidden_size = int(hidden_size)
        self.mixer_norm, self.mixer, self.mixer_out_norm = mixer_norm, mixer, mixer_out_norm
        self.ffn_norm, self.ffn, self.ffn_out_norm = ffn_norm, ffn, ffn_out_norm
        self.names = {"mixer_norm": "norm1", "mixer": "mix", "mixer_out_norm": "norm1b", "mixer_gate": "rg1",
                      "ffn_norm": "norm2", "ffn": "mlp", "ffn_out_norm": "norm2b", "ffn_gate": "rg2", "gate_bias": "b"}
        if names:
            self.names.update(names)
        self.halves = [self._half("mixer", mixer)] + ([self._half("ffn", ffn)] if ffn is not None else [])

    def _half(self, key: str, part):
        from .base import ProjectedPart
        from .linear import Linear
        gate = self.names[key + "_gate"]
        half = {"key": key, "part": part, "gate": gate, "norm": getattr(self, key + "_norm"),
                "out_norm": getattr(self, key + "_out_norm"), "set": None, "gate_linear": None, "gate_bias": None}
        if isinstance(part, ProjectedPart):
            half["set"] = ProjectionSet(self.hidden_size, [(self.names[key], part)], extra_in=[(gate, self.hidden_size)])
        else:
            half["gate_linear"] = Linear(self.hidden_size, self.hidden_size)
        return half

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs = {}
        for half in self.halves:
            key = half["key"]
            for which in ("norm", "out_norm"):
                prefix = self.names[key + "_" + which]
                for name, spec in half[which].param_specs().items():
                    specs[join_name(prefix, name)] = spec
            if half["set"] is not None:
                specs.update(half["set"].param_specs())
            else:
                for name, spec in half["part"].param_specs().items():
                    specs[join_name(self.names[key], name)] = spec
                specs[half["gate"]] = ParamSpec((self.hidden_size, self.hidden_size))
            specs[join_name(half["gate"], self.names["gate_bias"])] = ParamSpec((self.hidden_size,), mean=0.0, std=0.5)
        return specs

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        for half in self.halves:
            key = half["key"]
            for which in ("norm", "out_norm"):
                half[which].load(narrow_tensors(tensors, self.names[key + "_" + which]), rt)
            if half["set"] is not None:
                half["set"].load(tensors, rt)
                half["part"].rt = rt
            else:
                half["part"].load(narrow_tensors(tensors, self.names[key]), rt)
                half["gate_linear"].set_weight(tensors[half["gate"]], rt)
            half["gate_bias"] = tensors[join_name(half["gate"], self.names["gate_bias"])].to(
                device=rt.device, dtype=torch.float32).contiguous()

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", True) for h in self.halves for p in (h["part"], h["norm"], h["out_norm"]))

    def can_cut_rows(self) -> bool:
        return False

    def entry(self):
        return (self.mixer_norm, self.mixer)

    def _run_half(self, ctx, hidden: Hidden, half, cache, after, only_state: bool = False) -> None:
        """One sub-layer with its gate, output norm and residual add; ``after``: the (norm, sub-layer) that
        come next, whose input is made in the same pass if that norm allows it."""
        ops, ws = self.rt.ops, ctx.workspace
        x, T = hidden.x, hidden.x.shape[0]
        which = "a" if half["key"] == "mixer" else "b"       # two buffers: one is read while the other is filled
        inp = hidden.input_behind(ctx, half["norm"], ws.get("block.normed." + which, T, self.hidden_size, self.rt.dtype))
        part = half["part"]
        if half["set"] is not None:
            s = half["set"]
            proj, act = s.project(ctx, inp)
            part.core(ctx, s.views(0, proj), s.act_view(0, act), cache)
            if only_state:
                return
            delta, gate = s.output(ctx, act), s.extra_views(proj)[half["gate"]]
        else:
            delta = part.forward(ctx, inp, cache) if half["key"] == "mixer" else part.forward(ctx, inp)
            if only_state:
                return
            gate = ws.get("block.gate", T, self.hidden_size, self.rt.dtype)
            half["gate_linear"].forward(inp, gate)
        next_norm = next_out = None
        if after is not None and getattr(after[0], "layer_norm", False) and after[0].dim == self.hidden_size \
                and after[0].eps == half["out_norm"].eps:
            other = "b" if which == "a" else "a"
            next_norm = (after[0].weight, after[0].bias)
            next_out = ws.get("block.normed." + other, T, self.hidden_size, self.rt.dtype)
        out_norm = half["out_norm"]
        ops.gated_norm_residual(x, delta, out_norm.weight, out_norm.bias, out_norm.eps, gate=gate, gate_bias=half["gate_bias"],
                                delta_bias=getattr(part, "out_bias", None), next_norm=next_norm, next_out=next_out)
        hidden.pending, hidden.deferred = None, ((after[0], next_out) if next_out is not None else None)

    def forward(self, ctx, hidden: Hidden, cache, out_rows=None, follow=None) -> None:
        if hidden.pending is not None:
            raise RuntimeError("a block whose norms add to the stream themselves needs the stream complete")
        for i, half in enumerate(self.halves):
            nxt = self.halves[i + 1] if i + 1 < len(self.halves) else None
            after = (nxt["norm"], nxt["part"]) if nxt is not None else follow
            self._run_half(ctx, hidden, half, cache if half["key"] == "mixer" else None, after)

    def update_cache_only(self, ctx, hidden: Hidden, cache) -> None:
        """The last block of a step whose logits nobody wants: the mixer alone runs, for what it leaves in
        its cache or state; ``hidden`` is not meaningful afterwards."""
        self._run_half(ctx, hidden, self.halves[0], cache, None, only_state=True)


class TwoMixers(Mixer):
    """A mixer made of two that read the same rows side by side: ``left_scale * left(h) + right_scale * right(h)``.
    Both halves are ``ProjectedPart``: their input projections are one product, their output projections one
    product over the activations side by side, with each half's factor in its columns of that weight.  The left
    half keeps keys and values in pages, the right half a state of fixed size: the mixer asks for both
    (``CompoundNeed``) and hands each half its own.  Tensors: the halves' under ``left.`` and ``right.``."""

    is_mixer = True

    def __init__(self, hidden_size: int, left, right, left_scale: float = 1.0, right_scale: float = 1.0,
                 names: Optional[Dict[str, str]] = None):
        from .base import CompoundNeed, PagedKVNeed, StateNeed
        self.hidden_size = int(hidden_size)
        self.left, self.right = left, right
        self.names = {"left": "left", "right": "right"}
        if names:
            self.names.update(names)
        self.set = ProjectionSet(self.hidden_size, [(self.names["left"], left), (self.names["right"], right)],
                                 out_scales=[left_scale, right_scale])
        kv, state = left.cache_need(), right.cache_need()
        if not isinstance(kv, PagedKVNeed) or not isinstance(state, StateNeed):
            raise ValueError("the left half keeps pages of keys and values, the right half a state of fixed size")
        self._need = CompoundNeed(kv, state)

    def param_specs(self) -> Dict[str, ParamSpec]:
        return self.set.param_specs()

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.set.load(tensors, rt)

    def cache_need(self):
        return self._need

    @property
    def graph_safe(self) -> bool:
        return getattr(self.left, "graph_safe", True) and getattr(self.right, "graph_safe", True)

    # The halves are independent between the two products, and the right half's walk through its state is a chain
    # that leaves most of the chip idle, so the left half's kernels run beside it on a second stream (of the
    # default priority) that waits for the in-product and is waited for before the out-product.  Inside a graph
    # capture the same fork and join make two branches of the graph (TWO_STREAMS_IN_GRAPHS; steps of single tokens
    # go the same way, captured or not).
    TWO_STREAMS = True
    TWO_STREAMS_IN_GRAPHS = True
    _side_streams: Dict[object, object] = {}

    def _side_stream(self, ctx):
        if not TwoMixers.TWO_STREAMS or not hasattr(self.rt.ops, "on_stream") or self.rt.device.type != "cuda":
            return None
        if (ctx.max_q_len <= 1 or torch.cuda.is_current_stream_capturing()) and not TwoMixers.TWO_STREAMS_IN_GRAPHS:
            return None
        key = (self.rt.device.type, self.rt.device.index)
        if key not in TwoMixers._side_streams:
            TwoMixers._side_streams[key] = torch.cuda.Stream(device=self.rt.device)
        return TwoMixers._side_streams[key]

    def forward(self, ctx, normed, cache) -> torch.Tensor:
        proj, act = self.set.project(ctx, normed)
        side = self._side_stream(ctx)
        if side is None:
            self.left.core(ctx, self.set.views(0, proj), self.set.act_view(0, act), cache.kv)
            self.right.core(ctx, self.set.views(1, proj), self.set.act_view(1, act), cache.state)
            return self.set.output(ctx, act)
        main = torch.cuda.current_stream(self.rt.device)
        side.wait_stream(main)                           # the projections are there
        with self.rt.ops.on_stream(side):
            self.left.core(ctx, self.set.views(0, proj), self.set.act_view(0, act), cache.kv)
        self.right.core(ctx, self.set.views(1, proj), self.set.act_view(1, act), cache.state)
        main.wait_stream(side)                           # both halves' activations are there
        return self.set.output(ctx, act)
