"""Debuzen: a decoder whose layers are listed in config.json.  The embedded rows pass the model's norm (an RMS
norm in ``norm.groups`` equal parts of a row, as every norm of the model).  A layer is pre-norm,
``x <- x + mixer(shift(norm1(x))); x <- x + ff(norm2(x))``, where ``shift`` mixes what the mixer reads with
what it read one token earlier, channel by channel.  The mixer is

* ``parallel``: attention with sigmoid weights (interleaved rotation, unit queries and keys, a sliding window
  behind which the first positions stay in sight) beside the gated delta rule with a decay a key channel;
* ``parallel_2``: softmax attention with a sink in a sliding window (half-split rotation) beside a state-space
  mixer; both as ``left_scale * left + right_scale * right``;
* ``gla``: gated linear attention with a decay a key channel.

The feed-forward is ``W_down (silu(W_gate h) * W_up h)`` or absent.  A stretch of layers (``loop``) runs several
times with the same weights, each pass on caches and states of its own; before every pass the stream becomes
``W_in [x; x0]`` with ``x0`` the embedded rows.  The logits are soft-capped.

Checkpoint names: ``embed``, ``embed.norm``, ``loop.in``, ``l<i>.norm1|norm2|shift``, ``l<i>.mix.*``, ``l<i>.mlp.gate|up|down``,
``final.norm``, ``head``.
"""
from __future__ import annotations

from typing import Dict

import torch

from ..config.model_config import ChannelDeltaSpec, DebuzenConfig, GatedLinearSpec, StateSpaceSpec, TwoMixerSpec
from ..config.registry import register_architecture
from ..parts import (ChannelGatedDeltaRule, Embedding, GatedLinearAttention, LMHead, PreNormBlock, RMSNorm, RotaryEmbedding,
                     StateSpaceMixer, SwiGLUMLP, TokenShift, TwoMixers, WindowAttention)
from ..parts.base import ParamSpec, Part, Runtime
from ..parts.linear import Linear
from .decoder import DecoderModel, LayerCall


class LoopProduct(Part):
    """What happens to the stream right before a pass of a stretch of layers that runs again: it becomes
    ``W [x; x0]``, ``x0`` the rows as the embedding left them, ``W [width, 2 width]`` the tensor that carries the
    part's name.  The stream's pending sum is added on the way in; the product's 32-bit sums are the new stream
    (left pending on a stream of zeros, so that the next norm adds them up as it does any other)."""

    takes_hidden = True

    def __init__(self, width: int):
        self.width = int(width)
        self.linear = Linear(2 * self.width, self.width)

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"": ParamSpec((self.width, 2 * self.width), mean=0.0, std=(2 * self.width) ** -0.5)}

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.linear.set_weight(tensors[""], rt)

    def forward(self, ctx, hidden, embedded, arg) -> None:
        ops, T = self.rt.ops, hidden.x.shape[0]
        pair = ctx.workspace.get("loop.pair", T, 2 * self.width, self.rt.dtype)
        ops.stream_pair(hidden.x, hidden.pending, embedded, pair)
        hidden.x.zero_()
        hidden.pending = ops.linear_delta(pair, self.linear.weight, ctx.workspace, "loop.out", self.linear.weight_tiled,
                                          out_dtype=torch.float32)
        hidden.deferred = hidden.act = None


def build_debuzen(cfg: DebuzenConfig) -> DecoderModel:
    width, eps, groups = cfg.hidden_size, cfg.norm_eps, cfg.norm_groups
    rotations = {}

    def rotation(size, base, dims):
        key = (size, base, dims)
        if key not in rotations:
            rotations[key] = RotaryEmbedding(size, base, rot_dim=dims)
        return rotations[key]

    norm = lambda: RMSNorm(width, eps, weight_name="", groups=groups, weight_32bit=True)

    def attention(a, sigmoid: bool):
        return WindowAttention(width, a.heads, a.kv_heads, a.dim, a.vdim, a.scale, window=a.window,
                               pos_enc=rotation(a.dim, a.rot_base, a.rot_dims), interleaved=sigmoid,
                               qk_unit_eps=eps if sigmoid else None, keep_first=a.keep_first,
                               sink=not sigmoid, sigmoid_weights=sigmoid)

    layers = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if isinstance(m, GatedLinearSpec):
            mixer = GatedLinearAttention(width, m.heads, m.dim, m.vdim, m.tau, m.decay_rank, eps)
        elif isinstance(m, TwoMixerSpec) and isinstance(m.right, ChannelDeltaSpec):
            r = m.right
            right = ChannelGatedDeltaRule(width, r.heads, r.kv_heads, r.dim, r.vdim, r.conv, r.decay_rank, r.gate_rank, eps)
            mixer = TwoMixers(width, attention(m.left, True), right, m.left_scale, m.right_scale)
        elif isinstance(m, TwoMixerSpec) and isinstance(m.right, StateSpaceSpec):
            r = m.right
            right = StateSpaceMixer(width, r.heads, r.vdim, r.state, r.groups, r.conv, r.norm_groups, eps)
            mixer = TwoMixers(width, attention(m.left, False), right, m.left_scale, m.right_scale)
        else:
            raise TypeError(f"layer {i}: unknown mixer {m!r}")
        ffn = None
        if layer.ff is not None:
            ffn = SwiGLUMLP(width, layer.ff, names={"gate": "gate", "up": "up", "down": "down"}, delta_dtype=torch.float32)
        layers.append(PreNormBlock(width, norm(), mixer, norm() if ffn is not None else None, ffn, mixer_shift=TokenShift(width),
                                   names={"mixer_norm": "norm1", "mixer": "mix", "ffn_norm": "norm2", "ffn": "mlp",
                                          "mixer_shift": "shift"}))
    # the run order: the layers before the stretch, the stretch `times` times (caches and states a pass), the rest
    schedule, stream_parts = [], []
    n = len(cfg.layers)
    if cfg.has_loop:
        stream_parts.append(("loop.in", LoopProduct(width)))
        order = [(i, None) for i in range(cfg.loop_start)]
        for t in range(cfg.loop_times):
            order += [(i, t) for i in range(cfg.loop_start, cfg.loop_stop)]
        order += [(i, None) for i in range(cfg.loop_stop, n)]
    else:
        order = [(i, None) for i in range(n)]
    for pos, (i, t) in enumerate(order):
        enter = (0, t) if t is not None and i == cfg.loop_start else None
        schedule.append(LayerCall(i, cache=pos, write=True, enter=enter))
    embed = Embedding(cfg.vocab_size, width, weight_name="", norm=RMSNorm(width, eps, weight_name="norm", groups=groups, weight_32bit=True))
    head = LMHead(cfg.vocab_size, width, weight_name="", softcap=cfg.logit_softcap)
    return DecoderModel(cfg, embed, layers, norm(), head, position_encodings=list(rotations.values()), schedule=schedule,
                        names={"embed": "embed", "layer": "l{i}", "final_norm": "final.norm", "lm_head": "head"},
                        stream_parts=stream_parts)


register_architecture("Debuzen", DebuzenConfig, build_debuzen)
