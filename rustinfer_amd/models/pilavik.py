"""Pilavik: a decoder whose layers are listed in config.json.  Every sub-layer sits between two layer
norms (weight and bias) and its result passes a gate before the second:
``h = norm1(x); x <- x + norm1b(mixer(h) * sigmoid(W_rg1 h + b_rg1))``, then the same around the
feed-forward.  The mixer is the gated delta rule (short convolutions, unit q and k, a decay and a write
strength a head) or attention through a latent with an interleaved rotation, a sliding window and a
learned sink; the feed-forward is a dense one whose activation norms the first three powers, or a mixture
of gated experts scored by sigmoids, with a shared expert.  A stretch of layers (``loop``) runs several
times with the same weights, each pass on a cache or state of its own; before every pass but the first
the embedded rows are added to the stream again, and before every pass the pass's own vector
(``loop.step[t]``).  The final norm is a layer norm; the head has a matrix of its own.

Checkpoint names: ``embed``, ``loop.step``, ``l<i>.norm1|norm1b|norm2|norm2b`` (+ ``.b``), ``l<i>.rg1|rg2``
(+ ``.b``), ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm`` (+ ``.b``), ``head``.
"""
from __future__ import annotations

from typing import Dict

import torch

from ..config.model_config import GatedDeltaSpec, PilavikConfig, SinkLatentAttentionSpec
from ..config.registry import register_architecture
from ..parts import (Embedding, GatedDeltaRule, LMHead, LatentAttention, LayerNorm, MoEFeedForward, PolyNormMLP,
                     RotaryEmbedding, SandwichBlock)
from ..parts.base import ParamSpec, Part, Runtime
from .decoder import DecoderModel, LayerCall

ROUTER_NORM_EPS = 1e-20      # added to the sum of a token's chosen scores before they are divided by it


class LoopEntry(Part):
    """What happens to the stream right before a pass of a stretch of layers that runs ``times`` times:
    before every pass but the first the embedded rows are added again, and before every pass the row
    ``t`` of a table ``[times, width]`` (the tensor that carries the part's name), ``t`` the pass's number."""

    def __init__(self, width: int, times: int):
        self.width, self.times = int(width), int(times)
        self.steps = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"": ParamSpec((self.times, self.width), mean=0.0, std=0.1)}

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.steps = tensors[""].to(device=rt.device, dtype=torch.float32).contiguous()

    def forward(self, ctx, x, embedded, t: int) -> None:
        self.rt.ops.stream_add(x, embedded if t > 0 else None, self.steps[t])


def build_pilavik(cfg: PilavikConfig) -> DecoderModel:
    width, eps = cfg.hidden_size, cfg.norm_eps
    rotations = {}

    def rotation(size, base, dims):
        key = (size, base, dims)
        if key not in rotations:
            rotations[key] = RotaryEmbedding(size, base, rot_dim=dims)
        return rotations[key]

    norm = lambda: LayerNorm(width, eps, weight_name="", bias_name="b")
    layers = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if isinstance(m, GatedDeltaSpec):
            mixer = GatedDeltaRule(width, m.heads, m.kv_heads, m.dim, m.vdim, m.conv, eps)
        elif isinstance(m, SinkLatentAttentionSpec):
            mixer = LatentAttention(width, m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.scale, eps,
                                    pos_enc=rotation(m.rot_dim, m.rot_base, m.rot_dims), interleaved=True,
                                    window=m.window, sink=True)
        else:
            raise TypeError(f"layer {i}: unknown mixer {m!r}")
        ffn = None
        if layer.mlp is not None:
            f = layer.mlp
            if f.kind == "dense":
                ffn = PolyNormMLP(width, f.ff, eps)
            else:
                ffn = MoEFeedForward(width, f.ff, f.experts, f.top, renormalize=True, score="sigmoid",
                                     norm_eps=ROUTER_NORM_EPS, scale=f.router_scale, shared_size=f.shared_ff)
        layers.append(SandwichBlock(width, norm(), mixer, norm(), norm() if ffn is not None else None, ffn,
                                    norm() if ffn is not None else None))
    # the run order: the layers before the stretch, the stretch `times` times (a cache a pass), the rest
    schedule, stream_parts = [], []
    n = len(cfg.layers)
    if cfg.has_loop:
        stream_parts.append(("loop.step", LoopEntry(width, cfg.loop_times)))
        order = [(i, None) for i in range(cfg.loop_start)]
        for t in range(cfg.loop_times):
            order += [(i, t) for i in range(cfg.loop_start, cfg.loop_stop)]
        order += [(i, None) for i in range(cfg.loop_stop, n)]
    else:
        order = [(i, None) for i in range(n)]
    for pos, (i, t) in enumerate(order):
        enter = (0, t) if t is not None and i == cfg.loop_start else None
        schedule.append(LayerCall(i, cache=pos, write=True, enter=enter))
    embed = Embedding(cfg.vocab_size, width, weight_name="")
    head = LMHead(cfg.vocab_size, width, weight_name="")
    return DecoderModel(cfg, embed, layers, LayerNorm(width, eps, weight_name="", bias_name="b"), head,
                        position_encodings=list(rotations.values()), schedule=schedule,
                        names={"embed": "embed", "layer": "l{i}", "final_norm": "final.norm", "lm_head": "head"},
                        stream_parts=stream_parts)


register_architecture("Pilavik", PilavikConfig, build_pilavik)
