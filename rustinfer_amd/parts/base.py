"""Interfaces of the parts a model is put together from.

A model is a list of blocks and a run order.  A block arranges a *mixer*
(something that moves information between positions: attention here) and a
*feed-forward* around *norms*; a *position encoding* is handed to the parts that
use it.  Every part takes its sizes and constants as constructor arguments and
never learns which model it sits in (reference seam: ``Component::run`` on a
``Hidden`` with a deferred delta, crates/infer-core/src/component.rs:8-84,
crates/infer-worker/src/components/decoder_block.rs:9-31).

What a part must provide
------------------------
``param_specs()``   checkpoint tensors it reads, by name relative to the part:
                    ``{name: ParamSpec(shape, kind)}``.
``load(tensors, rt)``  take those tensors (CPU or device, stored dtype) and keep
                    what the kernels need on ``rt.device`` in ``rt.dtype``.  ``tensors``
                    is indexed by name; it may make a tensor when it is asked for
                    (``LazyTensors``), so a part asks for each once and hands the names
                    of a part of its own on with ``narrow_tensors``.  Second copies in
                    another order come from ``rt.tile`` / ``rt.take_tile_budget``.
``forward(...)``    run on the tokens of one step, described by a ``StepContext``.

Mixer:        ``cache_need()`` -> ``PagedKVNeed`` | ``StateNeed`` | ``None`` and
              ``forward(ctx, normed, cache) -> delta [T, hidden]``.
FeedForward:  ``forward(ctx, normed) -> delta [T, hidden]``.
Norm:         ``forward(ctx, x, delta, out, rows=None)``: ``x += delta`` (if any),
              ``out = norm(x)``; with ``rows`` only those rows are read and ``out``
              has one row for each of them.
PositionEncoding: ``prepare(rt, max_positions)``; ``rotary()`` -> ``(cos, sin,
              rot_dim)`` or ``None``; ``on_embedding(ctx, x)`` for encodings that
              add to the embedded tokens.

Optional, for a mixer or a feed-forward (and the output head), so that a plain RMS norm
between two sub-layers needs no kernel of its own when a step has few tokens:
``takes_deferred_norm = True``: ``forward`` also accepts a ``DeferredNorm`` in place of
              the normalised rows: rows ``x * w`` that still lack the factor
              ``rsqrt(mean(x^2) + eps)``, which the part applies to the result of its
              first product (a product commutes with a factor per row).
``forward_into(ctx, normed, [cache,] x, next_norm)`` -> ``DeferredNorm`` or ``None``:
              as ``forward``, but the part adds its output to the residual stream ``x``
              itself and returns the input of the sub-layer behind ``next_norm``;
              ``None`` (and nothing done) where it cannot this time.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Optional, Tuple

import torch


@dataclass(frozen=True)
class ParamSpec:
    """A checkpoint tensor a part reads: its shape, and how the random-weights mode draws it.
    ``kind`` names one of the usual distributions; a part whose parameter needs another one (a
    decay in (0, 1), a bias around some value) gives ``mean``/``std`` of a normal distribution, or
    ``init(generator, shape, device) -> float32 tensor`` for anything else."""
    shape: Tuple[int, ...]
    kind: str = "matrix"      # "matrix": N(0, 0.02);  "norm": 1 (+ noise);  "int": int32 table
    int_high: int = 0         # for kind "int": values in [0, int_high)
    mean: Optional[float] = None
    std: Optional[float] = None
    init: Optional[Callable[..., torch.Tensor]] = None


@dataclass(frozen=True)
class PagedKVNeed:
    """Keys and values of every position (or of the last ``window`` positions).  ``v_head_dim``:
    the size of a value head where it differs from a key head's."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    v_head_dim: Optional[int] = None
    keep_first: int = 0       # with a window: the first so many positions stay readable, their pages are never given back

    @property
    def value_dim(self) -> int:
        return self.head_dim if self.v_head_dim is None else self.v_head_dim


@dataclass(frozen=True)
class StateNeed:
    """A fixed-size state for each live request, ``shape`` elements of ``dtype``.  ``extra``: further
    tensors of the same request's slot, ``((name, shape, dtype), ...)`` (the last inputs of a short
    convolution beside a state matrix, say); the mixer finds them in ``StateView.extra[name]``."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32
    extra: Tuple[Tuple[str, Tuple[int, ...], torch.dtype], ...] = ()

    def all_tensors(self):
        """[(name, shape, dtype)] of every tensor a slot holds; the main one is called ``""``."""
        return [("", tuple(self.shape), self.dtype)] + [(n, tuple(s), d) for n, s, d in self.extra]


@dataclass(frozen=True)
class CompoundNeed:
    """What a layer asks for that keeps both a cache of keys and values and a fixed-size state (a mixer of
    two halves, or an attention layer behind something that carries a row from token to token): the layer
    gets a ``CompoundView`` with ``kv`` and ``state``."""
    kv: PagedKVNeed
    state: StateNeed


def simple_needs(need):
    """The ``PagedKVNeed`` / ``StateNeed`` a need is made of."""
    if need is None:
        return []
    return [need.kv, need.state] if isinstance(need, CompoundNeed) else [need]


def with_state_extra(need, name: str, shape, dtype=torch.float32):
    """``need`` with one more tensor ``name`` in the request's state slot: a ``StateNeed`` gains an extra, a
    ``PagedKVNeed`` becomes a ``CompoundNeed`` whose state has no main tensor of any size but this extra."""
    extra = ((name, tuple(shape), dtype),)
    if need is None:
        return StateNeed((0,), torch.float32, extra)
    if isinstance(need, StateNeed):
        return StateNeed(need.shape, need.dtype, tuple(need.extra) + extra)
    if isinstance(need, CompoundNeed):
        return CompoundNeed(need.kv, with_state_extra(need.state, name, shape, dtype))
    return CompoundNeed(need, StateNeed((0,), torch.float32, extra))


@dataclass
class DeferredNorm:
    """The input of a sub-layer whose norm is not finished: ``rows = x * w`` in the run dtype and
    partial sums of squares ``ssq [T, P]`` (32-bit) with ``sum(ssq[t]) = sum(x[t]^2)``; the
    normalised rows would be ``rows * rsqrt(sum(ssq[t]) / dim + eps)``."""
    rows: torch.Tensor
    ssq: torch.Tensor
    eps: float

    @property
    def scale(self):
        return (self.ssq, self.eps)


def split_normed(normed):
    """(rows, scale) of a sub-layer's input, be it normalised rows or a ``DeferredNorm``."""
    if isinstance(normed, DeferredNorm):
        return normed.rows, normed.scale
    return normed, None


def join_name(prefix: str, name: str) -> str:
    """A part's tensor under its parent's prefix; a part whose one tensor carries the part's own
    name (no suffix) calls it ``""``."""
    if not prefix:
        return name
    return f"{prefix}.{name}" if name else prefix


class LazyTensors:
    """name -> tensor for ``load``: a tensor is made when it is asked for and not kept, so that a
    model can be filled part by part without all of its tensors existing at once beside it."""

    def __init__(self, names, make: Callable[[str], torch.Tensor], prefix: str = ""):
        self._names, self._make, self._prefix = names, make, prefix

    def __getitem__(self, name: str) -> torch.Tensor:
        full = join_name(self._prefix, name)
        if full not in self._names:
            raise KeyError(name)
        return self._make(full)

    def __contains__(self, name) -> bool:
        return join_name(self._prefix, str(name)) in self._names

    def keys(self):
        if not self._prefix:
            return list(self._names)
        dot = self._prefix + "."
        return [n[len(dot):] for n in self._names if n.startswith(dot)] + ([""] if self._prefix in self._names else [])

    def __iter__(self):
        return iter(self.keys())

    def __len__(self) -> int:
        return len(self.keys())

    def items(self):
        return ((n, self[n]) for n in self.keys())

    def narrow(self, prefix: str) -> "LazyTensors":
        return LazyTensors(self._names, self._make, join_name(self._prefix, prefix))


def narrow_tensors(tensors, prefix: str):
    """The tensors whose names begin with ``prefix.``, under the rest of their names."""
    if hasattr(tensors, "narrow"):
        return tensors.narrow(prefix)
    sub = {n[len(prefix) + 1:]: t for n, t in tensors.items() if n.startswith(prefix + ".")}
    if prefix in tensors:
        sub[""] = tensors[prefix]          # the part's one tensor carries the part's own name
    return sub


@dataclass
class Runtime:
    """Where and in which precision a model runs."""
    device: torch.device
    dtype: torch.dtype            # torch.bfloat16 (serving) or torch.float32 (exact path)
    ops: Any                      # the kernel module (rustinfer_amd.kernels.ops)
    # A second copy of every projection weight in the order the few-row kernels stream it (and a
    # third, row-permuted one of the q/k/v weight for the fused projection).  False: one copy, as
    # the checkpoint has it; single-token steps then read row-major weights, more slowly, and the
    # weights take half the memory.
    tiled_weight_copy: bool = True
    # Bytes the second copies may still take (None: as much as they like).  A model whose weights
    # fill most of the device keeps second copies of the weights that are loaded first and reads the
    # others as the checkpoint has them.
    tile_budget: Optional[int] = None
    tiled_bytes: int = 0          # what the second copies have taken so far

    def take_tile_budget(self, nbytes: int) -> bool:
        """Whether a second copy of ``nbytes`` may be made; if so it is taken off the budget."""
        if not self.tiled_weight_copy:
            return False
        if self.tile_budget is not None:
            if nbytes > self.tile_budget:
                return False
            self.tile_budget -= int(nbytes)
        self.tiled_bytes += int(nbytes)
        return True

    def give_tile_budget_back(self, nbytes: int) -> None:
        """A copy that was allowed and not made after all (its shape has no such form)."""
        self.tiled_bytes -= int(nbytes)
        if self.tile_budget is not None:
            self.tile_budget += int(nbytes)

    def tile(self, w):
        """The tile-ordered copy of ``w`` if this runtime keeps such copies, the shape has one and
        the budget allows it."""
        make = getattr(self.ops, "tile_weight", None)
        if make is None or not self.tiled_weight_copy:
            return None
        if not self.take_tile_budget(w.numel() * w.element_size()):
            return None
        t = make(w)
        if t is None:
            self.give_tile_budget_back(w.numel() * w.element_size())
        return t


class Part:
    # A step of single tokens is captured once per batch shape as a HIP graph, on rows that belong
    # to no request, and replayed for the real rows.  A part whose ``forward`` launches the same
    # kernels with the same arguments whatever the rows hold (it reads the step's device tensors
    # only, keeps its temporaries in ``ctx.workspace``, and never waits for the GPU) may be
    # captured.  A part that looks at the host copies in the context (``host_q_lens``,
    # ``host_q_start``, ``host_slots``, ``request_ids``), allocates, or synchronises says
    # ``graph_safe = False``; a model that holds one runs every step eagerly.
    graph_safe = True

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt


class Norm(Part):
    def forward(self, ctx, x, delta, out, rows=None):
        raise NotImplementedError


class Mixer(Part):
    def cache_need(self):
        return None

    def forward(self, ctx, normed, cache):
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx, normed):
        raise NotImplementedError


class PositionEncoding(Part):
    def prepare(self, rt: Runtime, max_positions: int) -> None:
        self.rt = rt

    def rotary(self):
        return None

    def on_embedding(self, ctx, x) -> None:
        return None


def stored_to(t: torch.Tensor, rt: Runtime, keep_fp32: bool = False) -> torch.Tensor:
    """Bring a checkpoint tensor to the device.  Floating tensors go to the run
    dtype, except that with ``keep_fp32`` a tensor stored in 32-bit stays 32-bit."""
    if t.dtype in (torch.int32, torch.int64, torch.uint8, torch.int8):
        return t.to(device=rt.device, dtype=torch.int32).contiguous()
    if keep_fp32 and t.dtype == torch.float32:
        return t.to(device=rt.device).contiguous()
    return t.to(device=rt.device, dtype=rt.dtype).contiguous()


# ---------------------------------------------------------------------------
# Sub-layers of the shape  out = W_out f(W_in n)
# ---------------------------------------------------------------------------
class ProjectedPart(Part):
    """A mixer or feed-forward whose first step is a set of projections of its input and whose
    last is one projection back to the model's width, with anything in between (``core``).

    A part that says so lets whoever owns it stack the projections of several parts that read the
    same input into one product, and their output projections into one product over the
    concatenated activations (a block whose mixer and feed-forward read the same norm); used on its
    own it behaves as any other part (``param_specs`` / ``load`` / ``forward``).

    ``in_projections()``  [(tensor name, rows)]: weights ``[rows, hidden]`` applied to the input.
    ``out_projection()``  (tensor name, columns): the weight ``[hidden, columns]`` applied to what
                          ``core`` leaves.
    ``own_specs()`` / ``load_own(tensors, rt)``: every other tensor of the part.
    ``core(ctx, proj, act, cache)``: ``proj[name]`` are the projected rows ``[T, rows]`` (columns of
                          a wider buffer: unit column stride, any row stride), ``act [T, columns]``
                          is to be filled.
    """

    hidden_size: int = 0
    is_mixer = False

    def in_projections(self):
        raise NotImplementedError

    def out_projection(self):
        raise NotImplementedError

    def own_specs(self) -> Dict[str, ParamSpec]:
        return {}

    def load_own(self, tensors, rt: Runtime) -> None:
        self.rt = rt

    def arrange_in(self, name: str, w: torch.Tensor) -> torch.Tensor:
        """The rows of the in-projection ``name`` in the order ``core`` wants them (a part that turns
        pairs of neighbouring features may ask for the pairs' halves apart, say); as stored by default."""
        return w

    def core(self, ctx, proj, act, cache) -> None:
        raise NotImplementedError

    # -- on its own ----------------------------------------------------------------
    def _own_set(self) -> "ProjectionSet":
        s = getattr(self, "_set", None)
        if s is None:
            s = self._set = ProjectionSet(self.hidden_size, [("", self)])
        return s

    def param_specs(self) -> Dict[str, ParamSpec]:
        return self._own_set().param_specs()

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self._own_set().load(tensors, rt)

    def forward(self, ctx, normed, cache=None):
        s = self._own_set()
        proj, act = s.project(ctx, normed)
        self.core(ctx, s.views(0, proj), s.act_view(0, act), cache)
        return s.output(ctx, act)


def _up8(n: int) -> int:
    return (n + 7) // 8 * 8


class ProjectionSet:
    """The stacked projections of one or more ``ProjectedPart`` that read the same rows: one
    weight ``[sum of rows, hidden]`` in, one ``[hidden, sum of columns]`` out.  Every part's slice
    starts at a multiple of eight columns (16 bytes in bfloat16), the gaps being rows and columns
    of zeros."""

    def __init__(self, hidden_size: int, members, extra_in=(), out_scales=None):
        """``extra_in``: ``[(tensor name, rows)]`` of further projections of the same input that belong to
        whoever owns the set (a gate on a sub-layer's result, say); their columns are ``extra_views``.
        ``out_scales``: a factor for each member's output (the sum is ``sum_i s_i W_out,i act_i``): the
        member's columns of the stacked out-projection are multiplied by it, in 32-bit, when they are loaded."""
        from .linear import Linear
        self.hidden_size = int(hidden_size)
        self.members = list(members)                     # [(prefix, part)]
        self.out_scales = [float(x) for x in out_scales] if out_scales is not None else None
        if self.out_scales is not None and len(self.out_scales) != len(self.members):
            raise ValueError("a factor for each member expected")
        self.in_slices, self.act_slices = [], []
        n_in = n_act = 0
        self.extra_slices = {}
        for name, rows in extra_in:
            self.extra_slices[name] = (n_in, int(rows))
            n_in = _up8(n_in + int(rows))
        for _, part in self.members:
            views = {}
            for name, rows in part.in_projections():
                views[name] = (n_in, int(rows))
                n_in = _up8(n_in + int(rows))
            self.in_slices.append(views)
            _, cols = part.out_projection()
            self.act_slices.append((n_act, int(cols)))
            n_act = _up8(n_act + int(cols))
        self.n_in, self.n_act = n_in, n_act
        self.w_in = Linear(self.hidden_size, n_in)
        self.w_out = Linear(n_act, self.hidden_size)
        self._gaps = []                                  # columns of the activations nobody writes

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs: Dict[str, ParamSpec] = {}
        for prefix, part in self.members:
            for name, rows in part.in_projections():
                specs[join_name(prefix, name)] = ParamSpec((int(rows), self.hidden_size))
            name, cols = part.out_projection()
            specs[join_name(prefix, name)] = ParamSpec((self.hidden_size, int(cols)))
            for name, spec in part.own_specs().items():
                specs[join_name(prefix, name)] = spec
        for name, (_, rows) in self.extra_slices.items():
            specs[name] = ParamSpec((rows, self.hidden_size))
        return specs

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        w_in = torch.zeros((self.n_in, self.hidden_size), device=rt.device, dtype=rt.dtype)
        for name, (c0, rows) in self.extra_slices.items():
            w_in[c0:c0 + rows] = tensors[name].to(device=rt.device, dtype=rt.dtype)
        w_out = torch.zeros((self.hidden_size, self.n_act), device=rt.device, dtype=rt.dtype)
        self._gaps, end = [], 0
        for i, ((prefix, part), views, (a0, cols)) in enumerate(zip(self.members, self.in_slices, self.act_slices)):
            sub = narrow_tensors(tensors, prefix) if prefix else tensors
            for name, (c0, rows) in views.items():
                w_in[c0:c0 + rows] = part.arrange_in(name, sub[name].to(device=rt.device, dtype=rt.dtype))
            w_o = sub[part.out_projection()[0]].to(device=rt.device)
            if self.out_scales is not None and self.out_scales[i] != 1.0:
                w_o = w_o.to(torch.float32) * self.out_scales[i]
            w_out[:, a0:a0 + cols] = w_o.to(rt.dtype)
            if a0 > end:
                self._gaps.append((end, a0))
            end = a0 + cols
            part.load_own(sub, rt)
        if self.n_act > end:
            self._gaps.append((end, self.n_act))
        self.w_in.set_weight(w_in, rt)
        self.w_out.set_weight(w_out, rt)

    def project(self, ctx, normed):
        """(projected rows [T, n_in], the buffer [T, n_act] the parts' ``core`` fill)."""
        T = normed.shape[0]
        proj = ctx.workspace.get("projset.in", T, self.n_in, self.rt.dtype)
        self.w_in.forward(normed, proj)
        act = ctx.workspace.get("projset.act", T, self.n_act, self.rt.dtype)
        for a, b in self._gaps:                          # scratch may hold anything, and 0 * NaN is NaN
            act[:, a:b].zero_()
        return proj, act

    def views(self, i: int, proj):
        return {name: proj[:, c0:c0 + rows] for name, (c0, rows) in self.in_slices[i].items()}

    def extra_views(self, proj):
        return {name: proj[:, c0:c0 + rows] for name, (c0, rows) in self.extra_slices.items()}

    def act_view(self, i: int, act):
        a0, cols = self.act_slices[i]
        return act[:, a0:a0 + cols]

    def output(self, ctx, act):
        """The parts' summed outputs as a delta for the residual stream: 32-bit, or a stack of
        32-bit partial sums that the next norm adds up."""
        return self.rt.ops.linear_delta(act, self.w_out.weight, ctx.workspace, "projset.out",
                                        self.w_out.weight_tiled, out_dtype=torch.float32)
