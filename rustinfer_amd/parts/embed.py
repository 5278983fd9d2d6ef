"""Token embedding and output head.

``x[t, :] = E[id_t, :]`` with no scale (crates/infer-worker/src/components/embed.rs:63-137);
the head is a projection onto the vocabulary that shares the embedding table when the
model ties them (crates/infer-worker/src/models/decoder.rs:245-262,
crates/infer-worker/src/components/lm_head.rs:13-20).  Logits leave in 32-bit.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import ParamSpec, Part, Runtime, split_normed, stored_to


class Embedding(Part):
    def __init__(self, vocab_size: int, dim: int, weight_name: str = "weight", scale: float = 1.0, norm=None):
        self.vocab_size = int(vocab_size)
        self.dim = int(dim)
        self.weight = None
        self.weight_name = weight_name       # "" where the table carries the part's own name
        self.scale = float(scale)            # every embedded row is multiplied by it
        self.norm = norm                     # a norm the embedded rows pass (its tensors under the table's name)

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs = {self.weight_name: ParamSpec((self.vocab_size, self.dim), "matrix")}
        if self.norm is not None:
            specs.update(self.norm.param_specs())
        return specs

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.weight = stored_to(tensors[self.weight_name], rt)
        if self.norm is not None:
            self.norm.load(tensors, rt)

    def forward(self, ctx, ids: torch.Tensor, out_x: torch.Tensor) -> torch.Tensor:
        rows = out_x
        if self.norm is not None:
            rows = ctx.workspace.get("embed.rows", out_x.shape[0], self.dim, torch.float32)
        if self.scale != 1.0:
            self.rt.ops.embed(ids, self.weight, rows, getattr(ctx, "device_tokens", None), scale=self.scale)
        else:
            self.rt.ops.embed(ids, self.weight, rows, getattr(ctx, "device_tokens", None))
        if self.norm is not None:
            self.norm.forward(ctx, rows, None, out_x)          # 32-bit rows in, 32-bit stream out
        return out_x


class LMHead(Part):
    def __init__(self, vocab_size: int, dim: int, tied_to: Optional[Embedding] = None,
                 logit_scale: float = 1.0, softcap: float = 0.0, weight_name: str = "weight"):
        """``logit_scale``, ``softcap``: the logits leave as ``softcap * tanh(logit_scale * z / softcap)``
        (``softcap = 0``: ``logit_scale * z``)."""
        self.vocab_size = int(vocab_size)
        self.dim = int(dim)
        self.tied_to = tied_to
        self.weight = None
        self.logit_scale, self.softcap = float(logit_scale), float(softcap)
        self.weight_name = weight_name       # "" where the matrix carries the part's own name

    def param_specs(self) -> Dict[str, ParamSpec]:
        if self.tied_to is not None:
            return {}
        return {self.weight_name: ParamSpec((self.vocab_size, self.dim), "matrix")}

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        if self.tied_to is not None:
            self.weight = self.tied_to.weight      # same storage, no copy
        else:
            self.weight = stored_to(tensors[self.weight_name], rt)
        self.weight_tiled = rt.tile(self.weight)

    takes_deferred_norm = True

    def forward(self, ctx, normed, logits: torch.Tensor) -> torch.Tensor:
        rows, scale = split_normed(normed)
        if scale is None:
            self.rt.ops.linear(rows, self.weight, logits, self.weight_tiled)
        else:
            self.rt.ops.linear(rows, self.weight, logits, self.weight_tiled, scale=scale)
        if self.logit_scale != 1.0 or self.softcap > 0.0:
            self.rt.ops.scale_softcap(logits, self.logit_scale, self.softcap)
        return logits
