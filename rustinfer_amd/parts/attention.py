"""Grouped-query attention over a paged key/value cache.

Per token: fused q/k/v projection (rows of q, then k, then v:
crates/infer-worker/src/models/loader.rs:419-454), rotation of q and k by absolute
position, write of k and v into the request's pages, attention of every query over
the positions it may see (``j <= p``, and ``j > p - window`` if a window is set;
bottom-right causal rule of crates/infer-core/src/ports/fused_ops.rs:430-535), and the
output projection (crates/infer-worker/src/components/attention.rs:44-181).
Query head ``h`` reads key/value head ``h // (H / Hkv)``; the scale is
``1/sqrt(head_dim)`` unless given (crates/infer-worker/src/models/decoder.rs:276).
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from .base import (DeferredNorm, Mixer, PagedKVNeed, ParamSpec, PositionEncoding, ProjectedPart, Runtime,
                   split_normed)
from .linear import Linear


class PagedAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 pos_enc: Optional[PositionEncoding] = None, scale: Optional[float] = None,
                 window: Optional[int] = None, own_kv: bool = True, qk_transform=None):
        """``qk_transform``: what a variant of this mixer does between the projection and the
        rotation (a norm or a scale per head on q and k, a bias): called as
        ``qk_transform(ctx, qkv, self)`` on the projected rows ``qkv [T, q_dim + 2 kv_dim]`` (queries
        first, then keys, then values; ``own_kv=False``: queries only), which it changes in place.
        It may be a part of its own: ``param_specs()`` / ``load(tensors, rt)`` are then used under
        the mixer's names, and ``graph_safe`` is honoured.  With a transform the projection, the
        rotation and the cache write run as separate kernels (the fused kernel has no place for it)."""
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads {num_heads} is not a multiple of num_kv_heads {num_kv_heads}")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.pos_enc = pos_enc
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.window = int(window) if window else None
        self.own_kv = bool(own_kv)       # False: no k/v projection, reads another layer's cache
        self.q_dim = self.num_heads * self.head_dim
        self.kv_dim = self.num_kv_heads * self.head_dim
        self.qkv_dim = self.q_dim + (2 * self.kv_dim if self.own_kv else 0)
        self.qkv = Linear(self.hidden_size, self.qkv_dim)
        self.o = Linear(self.q_dim, self.hidden_size)
        self.qkv_fused = None
        self.qk_transform = qk_transform

    @property
    def graph_safe(self) -> bool:
        return getattr(self.qk_transform, "graph_safe", True)

    def param_specs(self) -> Dict[str, ParamSpec]:
        h = self.hidden_size
        specs = {"q_proj.weight": ParamSpec((self.q_dim, h))}
        if self.own_kv:
            specs["k_proj.weight"] = ParamSpec((self.kv_dim, h))
            specs["v_proj.weight"] = ParamSpec((self.kv_dim, h))
        specs["o_proj.weight"] = ParamSpec((h, self.q_dim))
        if hasattr(self.qk_transform, "param_specs"):
            specs.update(self.qk_transform.param_specs())
        return specs

    def cache_need(self):
        return PagedKVNeed(self.num_kv_heads, self.head_dim, self.window)

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        names = ["q_proj.weight"] + (["k_proj.weight", "v_proj.weight"] if self.own_kv else [])
        parts = [tensors[n].to(device=rt.device, dtype=rt.dtype) for n in names]
        # for steps of few single tokens: projection, rotation and cache write in one kernel, which
        # reads its own copy of the weight (rows ordered so that rotary partners meet in a tile);
        # the plain tile-ordered copy would never be read beside it
        make = getattr(rt.ops, "qkv_rope_weight", None)
        fuse = make is not None and rt.tiled_weight_copy and self.own_kv and self.qk_transform is None
        w = torch.cat(parts, dim=0) if len(parts) > 1 else parts[0]
        del parts
        self.qkv.set_weight(w, rt, tile=not fuse)
        self.qkv_fused = None
        if fuse and rt.take_tile_budget(w.numel() * w.element_size()):
            self.qkv_fused = make(self.qkv.weight, self.head_dim)
            if self.qkv_fused is None:           # no such copy for these sizes: the plain one, if any
                rt.give_tile_budget_back(w.numel() * w.element_size())
                self.qkv.weight_tiled = rt.tile(self.qkv.weight)
        self.o.set_weight(tensors["o_proj.weight"], rt)
        if hasattr(self.qk_transform, "load"):
            own = self.qk_transform.param_specs() if hasattr(self.qk_transform, "param_specs") else {}
            self.qk_transform.load({n: tensors[n] for n in own}, rt)

    takes_deferred_norm = True

    def _project(self, ctx, normed, cache):
        """Rotated queries in ``qkv`` (and this step's keys and values in the cache) from the input
        rows, be they normalised or a ``DeferredNorm``."""
        rows, scale = split_normed(normed)
        T = rows.shape[0]
        ws, ops = ctx.workspace, self.rt.ops
        qkv = ws.get("attn.qkv", T, self.qkv_dim, self.rt.dtype)
        rotary = self.pos_enc.rotary() if self.pos_enc is not None else None
        table = ctx.block_tables[cache.group]
        kw = {} if scale is None else {"scale": scale}
        fused = (self.qkv_fused is not None and cache.write and ctx.max_q_len == 1
                 and ops.qkv_rope_fused(rows, self.qkv_fused, qkv, self.num_heads, self.num_kv_heads,
                                        self.head_dim, rotary, ctx.positions, ctx.row_of_token,
                                        cache.k, cache.v, table, cache.page_size, **kw))
        if not fused:
            self.qkv.forward(rows, qkv, scale)
            if self.qk_transform is not None:
                self.qk_transform(ctx, qkv, self)
            ops.rope_kv_write(qkv, self.num_heads, self.num_kv_heads, self.head_dim, rotary,
                              ctx.positions, ctx.row_of_token, cache.k, cache.v, table,
                              cache.page_size, write_kv=self.own_kv and cache.write)
        return qkv, table

    def forward(self, ctx, normed, cache) -> torch.Tensor:
        qkv, table = self._project(ctx, normed, cache)
        attn = self._attend(ctx, qkv, cache, table)
        return self.rt.ops.linear_delta(attn, self.o.weight, ctx.workspace, "mixer.out", self.o.weight_tiled)

    def update_cache(self, ctx, normed, cache) -> None:
        """What a step leaves behind for later ones, and nothing else: this step's keys and values
        in the cache.  For the last block of a step whose logits nobody wants."""
        if self.own_kv and cache.write:
            self._project(ctx, normed, cache)

    def forward_into(self, ctx, normed, cache, x: torch.Tensor, next_norm):
        """Few rows: the output projection adds its sums to ``x`` itself and prepares the input behind
        ``next_norm`` (see parts/base.py).  None, and nothing done, where that form does not apply."""
        ops = self.rt.ops
        ok = getattr(ops, "linear_residual_ok", None)
        if ok is None or not ok(x.shape[0], self.o.weight, self.o.weight_tiled, next_norm.weight):
            return None
        pays = getattr(ops, "linear_residual_pays", None)
        if pays is not None and not pays(x.shape[0], self.o.weight):
            return None
        qkv, table = self._project(ctx, normed, cache)
        attn = self._attend(ctx, qkv, cache, table)
        a, ssq = ops.linear_residual(attn, self.o.weight, self.o.weight_tiled, x, next_norm.weight,
                                     ctx.workspace, "deferred")
        return DeferredNorm(a, ssq, next_norm.eps)

    def _attend(self, ctx, qkv: torch.Tensor, cache, table) -> torch.Tensor:
        """Attention over the cache with the rotated queries in ``qkv``."""
        ws, ops = ctx.workspace, self.rt.ops
        attn = ws.get("attn.out", qkv.shape[0], self.q_dim, self.rt.dtype)
        ops.paged_attention(qkv, attn, self.num_heads, self.num_kv_heads, self.head_dim,
                            cache.k, cache.v, table, cache.page_size, ctx, self.scale,
                            self.window or 0)
        return attn


class WindowAttention(ProjectedPart, Mixer):
    """Grouped softmax attention over the last ``window`` positions with key heads of size
    ``head_dim`` and value heads of size ``v_head_dim``.  ``pos_enc`` rotates the first
    ``pos_enc.rot_dim`` features of queries and keys; ``value_pos_enc`` (a rotation over all of
    ``v_head_dim``) is applied to every value before it is cached, by the value's position, and
    undone on each head's sum by the query's position, so that a value enters the output turned by
    the distance between the two.  Scores are ``(q . k) * scale``; the softmax is over the visible
    keys only.  Tensor names: ``q, k, v, o`` unless given.

    ``qk_norm_eps``: queries and keys are divided by their root mean square over each head (this eps
    inside the root) and multiplied by weights of the head's size shared by all heads (tensors
    ``<q>.norm``, ``<k>.norm``); the cache holds the normed keys.  ``q_temperature = (coef, every)``:
    the query at position p is multiplied by ``1 + coef ln(floor((p + 1) / every) + 1)``.  Either goes
    without a rotation of queries and keys.  ``own_kv = False``: the layer has no keys and values of
    its own and reads a cache that another layer writes (the run order names it).

    ``interleaved``: the checkpoint's rotation pairs feature 2i with 2i + 1; the rows of ``q`` and ``k`` that make
    the turned features are reordered when they are loaded (even ones, then odd ones, head by head), which
    leaves every score as it was.  ``qk_unit_eps``: after the rotation every head of q and k is divided by its
    root mean square (this eps inside the root), with no weight.  ``keep_first``: behind the window the first so
    many positions of a sequence stay in sight, at their true positions; the cache never gives their pages back.
    ``sink``: a learned number a head (tensor ``sink``) whose exponential joins the softmax's denominator.
    ``sigmoid_weights``: no softmax; a visible key's weight is ``sigmoid(score + b_h)`` with a learned number a
    head (tensor ``pb``), and the weights are not normalised over the keys."""

    is_mixer = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int,
                 scale: float, window: Optional[int] = None, pos_enc: Optional[PositionEncoding] = None,
                 value_pos_enc: Optional[PositionEncoding] = None, interleaved_values: bool = False,
                 names: Optional[Dict[str, str]] = None, qk_norm_eps: Optional[float] = None,
                 q_temperature=None, own_kv: bool = True, interleaved: bool = False,
                 qk_unit_eps: Optional[float] = None, keep_first: int = 0, sink: bool = False,
                 sigmoid_weights: bool = False):
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads {num_heads} is not a multiple of num_kv_heads {num_kv_heads}")
        if sink and sigmoid_weights:
            raise ValueError("a sink belongs to a softmax: sigmoid weights take none")
        if keep_first and not window:
            keep_first = 0                       # without a window every position stays in sight anyway
        self.interleaved = bool(interleaved)
        self.qk_unit_eps = float(qk_unit_eps) if qk_unit_eps else None
        self.keep_first = int(keep_first)
        self.has_sink, self.sigmoid_weights = bool(sink), bool(sigmoid_weights)
        self.sink = self.sigmoid_bias = None
        self.qk_norm_eps = float(qk_norm_eps) if qk_norm_eps is not None else None
        self.q_temperature = (float(q_temperature[0]), int(q_temperature[1])) if q_temperature else None
        self.own_kv = bool(own_kv)
        self.by_head = self.qk_norm_eps is not None or self.q_temperature is not None
        if self.by_head and (pos_enc is not None or value_pos_enc is not None):
            raise ValueError("a norm or a temperature on queries and keys goes without a rotation")
        self.hidden_size = int(hidden_size)
        self.num_heads, self.num_kv_heads = int(num_heads), int(num_kv_heads)
        self.head_dim, self.v_head_dim = int(head_dim), int(v_head_dim)
        self.scale = float(scale)
        self.window = int(window) if window else None
        self.pos_enc, self.value_pos_enc = pos_enc, value_pos_enc
        self.interleaved_values = bool(interleaved_values)
        self.names = {"q": "q", "k": "k", "v": "v", "o": "o", "sink": "sink", "sigmoid_bias": "pb"}
        if names:
            self.names.update(names)
        if self.by_head and (self.interleaved or self.qk_unit_eps is not None):
            raise ValueError("the weighted norm of queries and keys goes without a rotation and without the unit norm")

    def arrange_in(self, name: str, w: torch.Tensor) -> torch.Tensor:
        rot = self.pos_enc.rot_dim if self.pos_enc is not None else 0
        if not self.interleaved or rot == 0 or name not in (self.names["q"], self.names["k"]):
            return w
        heads = w.view(-1, self.head_dim, w.shape[1])
        return torch.cat([heads[:, 0:rot:2], heads[:, 1:rot:2], heads[:, rot:]], dim=1).reshape(w.shape).contiguous()

    def in_projections(self):
        n = self.names
        if not self.own_kv:
            return [(n["q"], self.num_heads * self.head_dim)]
        return [(n["q"], self.num_heads * self.head_dim), (n["k"], self.num_kv_heads * self.head_dim),
                (n["v"], self.num_kv_heads * self.v_head_dim)]

    def own_specs(self):
        n, specs = self.names, {}
        if self.has_sink:
            specs[n["sink"]] = ParamSpec((self.num_heads,), mean=0.0, std=1.0)
        if self.sigmoid_weights:
            specs[n["sigmoid_bias"]] = ParamSpec((self.num_heads,), mean=-2.0, std=1.0)
        if self.qk_norm_eps is None:
            return specs
        specs[n["q"] + ".norm"] = ParamSpec((self.head_dim,), "norm")
        if self.own_kv:
            specs[n["k"] + ".norm"] = ParamSpec((self.head_dim,), "norm")
        return specs

    def out_projection(self):
        return (self.names["o"], self.num_heads * self.v_head_dim)

    def cache_need(self):
        return PagedKVNeed(self.num_kv_heads, self.head_dim, self.window, self.v_head_dim, self.keep_first)

    def load_own(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        f32 = lambda name: tensors[name].to(device=rt.device, dtype=torch.float32).contiguous()
        if self.has_sink:
            self.sink = f32(self.names["sink"])
        if self.sigmoid_weights:
            self.sigmoid_bias = f32(self.names["sigmoid_bias"])
        if not rt.ops.window_attention_supported(self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim):
            raise ValueError(f"attention with {self.num_heads}/{self.num_kv_heads} heads of {self.head_dim} and "
                             f"{self.v_head_dim} features is beyond the window attention kernel")
        self.q_norm_weight = self.k_norm_weight = None
        if self.qk_norm_eps is not None:
            f32 = lambda name: tensors[name].to(device=rt.device, dtype=torch.float32).contiguous()
            self.q_norm_weight = f32(self.names["q"] + ".norm")
            self.k_norm_weight = f32(self.names["k"] + ".norm") if self.own_kv else None

    def core(self, ctx, proj, act, cache) -> None:
        ops, n = self.rt.ops, self.names
        q, k, v = proj[n["q"]], proj.get(n["k"]), proj.get(n["v"])
        table = ctx.block_tables[cache.group]
        write = self.own_kv and cache.write
        if self.by_head:
            coef, every = self.q_temperature or (0.0, 0)
            ops.head_norm_kv_write(q, k, v, self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim,
                                   self.q_norm_weight, self.k_norm_weight, self.qk_norm_eps or 1.0, ctx.positions,
                                   ctx.row_of_token, cache.k, cache.v, table, cache.page_size, write_kv=write,
                                   norm=self.qk_norm_eps is not None, temp_coef=coef, temp_every=every)
            ops.window_attention(q, act, self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim, cache.k, cache.v,
                                 table, cache.page_size, ctx, self.scale, self.window or 0, None, False)
            return
        rotary = self.pos_enc.rotary() if self.pos_enc is not None else None
        vrot = self.value_pos_enc.rotary()[:2] if self.value_pos_enc is not None else None
        extra = {}
        if self.qk_unit_eps is not None:
            extra["unit_eps"] = self.qk_unit_eps
        ops.rotate_kv_write(q, k, v, self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim, rotary, vrot,
                            ctx.positions, ctx.row_of_token, cache.k, cache.v, table, cache.page_size,
                            write_kv=write, interleaved_values=self.interleaved_values, **extra)
        extra = {}
        if self.sink is not None:
            extra["sink"] = self.sink
        if self.keep_first:
            extra["keep_first"] = self.keep_first
        if self.sigmoid_bias is not None:
            extra["sigmoid_bias"] = self.sigmoid_bias
        ops.window_attention(q, act, self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim, cache.k, cache.v,
                             table, cache.page_size, ctx, self.scale, self.window or 0, vrot, self.interleaved_values, **extra)


class LatentAttention(ProjectedPart, Mixer):
    """Softmax attention whose keys and values all come from ONE latent vector a token.

    ``W_down x`` has ``latent_dim + rot_dim`` rows: the first ``latent_dim``, divided by their root
    mean square and multiplied by a weight, are the latent ``c``; the rest are one rotated key part
    for all heads.  Head h's key is ``[W_uk,h c, rotated part]`` against the query
    ``[q_h unrotated (head_dim), q_h rotated (rot_dim)]``, its value ``W_uv,h c``.  The cache holds ``c``
    and the rotated part only, as ONE key/value head with keys ``[c, rotated part]`` and values ``c``:
    the score ``q_h . (W_uk,h c)`` is ``(W_uk,h^T q_h) . c``, so each query head is taken into the
    latent space (``head_linear``), attention runs over the latents with all heads sharing the one
    key/value head, and each head's weighted sum of latents goes through ``W_uv,h`` afterwards.

    ``pos_enc`` turns the first ``pos_enc.rot_dim`` features of a rotated part; ``interleaved``: the
    checkpoint pairs feature 2i with 2i + 1, so the rows that make the rotated parts are reordered
    when they are loaded (even features, then odd ones), which leaves every score as it was.  More than 32 heads run as several calls of the
    attention kernels over the same cache.
    ``window``: a position sees itself and the ``window - 1`` before it (None: all); the cache gives back the
    pages the window has passed.  ``sink``: a learned number a head (tensor ``sink``) whose exponential joins
    the softmax's denominator; it has no key and no value and is not scaled.
    Tensor names: ``q, dkv, dkv.norm, uk, uv, o, sink`` unless given."""

    is_mixer = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, v_head_dim: int, latent_dim: int,
                 scale: float, norm_eps: float, pos_enc: Optional[PositionEncoding] = None, interleaved: bool = True,
                 names: Optional[Dict[str, str]] = None, window: Optional[int] = None, sink: bool = False):
        self.hidden_size = int(hidden_size)
        self.window = int(window) if window else None
        self.has_sink = bool(sink)
        self.sink = None
        self.num_heads, self.head_dim, self.rot_dim = int(num_heads), int(head_dim), int(rot_dim)
        self.v_head_dim, self.latent_dim = int(v_head_dim), int(latent_dim)
        self.scale, self.norm_eps = float(scale), float(norm_eps)
        self.pos_enc, self.interleaved = pos_enc, bool(interleaved)
        self.names = {"q": "q", "down": "dkv", "norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o", "sink": "sink"}
        if names:
            self.names.update(names)

    def in_projections(self):
        n = self.names
        return [(n["q"], self.num_heads * (self.head_dim + self.rot_dim)), (n["down"], self.latent_dim + self.rot_dim)]

    def out_projection(self):
        return (self.names["o"], self.num_heads * self.v_head_dim)

    def own_specs(self):
        n, H, R = self.names, self.num_heads, self.latent_dim
        specs = {n["norm"]: ParamSpec((R,), "norm"), n["uk"]: ParamSpec((H * self.head_dim, R)),
                 n["uv"]: ParamSpec((H * self.v_head_dim, R))}
        if self.has_sink:
            specs[n["sink"]] = ParamSpec((H,), mean=0.0, std=1.0)
        return specs

    def cache_need(self):
        return PagedKVNeed(1, self.latent_dim + self.rot_dim, self.window, self.latent_dim)

    def _pairs_apart(self, part: torch.Tensor) -> torch.Tensor:
        """Rows of one rotated part [rot_dim, hidden] with the turned pairs' halves apart."""
        rot = self.pos_enc.rot_dim if self.pos_enc is not None else 0
        if not self.interleaved or rot == 0:
            return part
        return torch.cat([part[0:rot:2], part[1:rot:2], part[rot:]], dim=0)

    def arrange_in(self, name: str, w: torch.Tensor) -> torch.Tensor:
        d, r, R = self.head_dim, self.rot_dim, self.latent_dim
        if name == self.names["q"]:
            heads = w.view(self.num_heads, d + r, w.shape[1])
            return torch.cat([torch.cat([h[:d], self._pairs_apart(h[d:])], dim=0) for h in heads], dim=0)
        if name == self.names["down"]:
            return torch.cat([w[:R], self._pairs_apart(w[R:])], dim=0)
        return w

    def load_own(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        n, H, R = self.names, self.num_heads, self.latent_dim
        # the attention kernels take up to 32 query heads a key/value head: more heads go in stretches of 32
        self.heads_a_call = min(H, 32)
        if not rt.ops.window_attention_supported(self.heads_a_call, 1, R + self.rot_dim, R):
            raise ValueError(f"latent attention over a latent of {R} + {self.rot_dim} features is beyond the window "
                             f"attention kernel (256 features)")
        self.norm_weight = tensors[n["norm"]].to(device=rt.device, dtype=torch.float32).contiguous()
        uk = tensors[n["uk"]].to(device=rt.device, dtype=rt.dtype)
        self.w_absorb = uk.view(H, self.head_dim, R).transpose(1, 2).contiguous()        # [H, R, head_dim]: W_uk,h^T
        self.w_value = tensors[n["uv"]].to(device=rt.device, dtype=rt.dtype).contiguous().view(H, self.v_head_dim, R)
        if self.has_sink:
            self.sink = tensors[n["sink"]].to(device=rt.device, dtype=torch.float32).contiguous()

    def core(self, ctx, proj, act, cache) -> None:
        ops, n, ws = self.rt.ops, self.names, ctx.workspace
        H, d, r, R = self.num_heads, self.head_dim, self.rot_dim, self.latent_dim
        q, down = proj[n["q"]], proj[n["down"]]
        T = q.shape[0]
        table = ctx.block_tables[cache.group]
        q_lat = ws.get("latent.q", T, H * (R + r), self.rt.dtype)
        rotary = self.pos_enc.rotary() if self.pos_enc is not None else None
        ops.latent_kv_write(q, down, q_lat, H, d, r, R, self.norm_weight, self.norm_eps, rotary, ctx.positions,
                            ctx.row_of_token, cache.k, cache.v, table, cache.page_size, write_kv=cache.write)
        ops.head_linear(q, d + r, self.w_absorb, q_lat, R + r)
        lat = ws.get("latent.sum", T, H * R, self.rt.dtype)
        for h0 in range(0, H, self.heads_a_call):
            n = min(self.heads_a_call, H - h0)
            ops.window_attention(q_lat[:, h0 * (R + r):(h0 + n) * (R + r)], lat[:, h0 * R:(h0 + n) * R], n, 1, R + r, R,
                                 cache.k, cache.v, table, cache.page_size, ctx, self.scale, self.window or 0, None, False,
                                 sink=self.sink[h0:h0 + n] if self.sink is not None else None)
        ops.head_linear(lat, R, self.w_value, act, self.v_head_dim)
