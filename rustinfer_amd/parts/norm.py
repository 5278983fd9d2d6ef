"""RMSNorm with the residual add folded in.

``y = x * rsqrt(mean(x^2) + eps) * w``; the weight multiplies directly
(crates/infer-worker/src/components/norm.rs:19-26,
crates/infer-backend-cuda/src/kernels/rmsnorm/rmsnorm.cu:52-113).  The fused
form ``x += delta; out = norm(x)`` is the reference's ``fused_add_rmsnorm``
(crates/infer-core/src/ports/fused_ops.rs:42-52); here the residual ``x`` is kept
in 32-bit, so the sum is rounded once, into ``out``.
"""
from __future__ import annotations

from typing import Dict

import torch

from .base import Norm, ParamSpec, Runtime, stored_to


class RMSNorm(Norm):
    def __init__(self, dim: int, eps: float, weight_name: str = "weight", one_plus: bool = False, groups: int = 1,
                 weight_32bit: bool = False):
        """``weight_name``: the weight's name under the norm's own ("" where the tensor carries the
        norm's name itself).  ``one_plus``: the checkpoint stores the weight around zero and the norm
        multiplies by ``1 + w`` (kept as that sum, in 32-bit).  ``groups``: a row is split into that many
        equal consecutive parts and each is divided by its own root mean square.  ``weight_32bit``: the weight is
        widened to 32-bit whatever the checkpoint stores (for norms whose rows leave in 32-bit)."""
        self.weight_32bit = bool(weight_32bit)
        self.dim = int(dim)
        self.eps = float(eps)
        self.weight = None
        self.weight_name = weight_name
        self.one_plus = bool(one_plus)
        self.groups = int(groups)
        if self.groups < 1 or self.dim % self.groups:
            raise ValueError(f"{self.dim} values do not split into {self.groups} equal parts")
        # nothing but ``weight`` and ``eps``: the sub-layers around this norm may do it between them
        # (``forward_into`` and ``DeferredNorm``, see PreNormBlock.forward); not so a norm in parts
        self.plain_rms = self.groups == 1

    def param_specs(self) -> Dict[str, ParamSpec]:
        if self.one_plus:
            return {self.weight_name: ParamSpec((self.dim,), mean=0.0, std=0.1)}
        return {self.weight_name: ParamSpec((self.dim,), "norm")}

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        if self.one_plus:
            self.weight = (tensors[self.weight_name].to(device=rt.device, dtype=torch.float32) + 1.0).contiguous()
        elif self.weight_32bit:
            self.weight = tensors[self.weight_name].to(device=rt.device, dtype=torch.float32).contiguous()
        else:
            self.weight = stored_to(tensors[self.weight_name], rt, keep_fp32=True)

    cuts_rows = True          # forward() takes x_rows (see PreNormBlock.forward)

    def forward(self, ctx, x, delta, out, rows=None, x_rows=None):
        if self.groups > 1:
            self.rt.ops.add_rmsnorm(x, delta, self.weight, self.eps, out, rows, x_rows, groups=self.groups)
        else:
            self.rt.ops.add_rmsnorm(x, delta, self.weight, self.eps, out, rows, x_rows)
        return out


    def forward_shifted(self, ctx, x, delta, out, mix, state):
        """For a step whose every row is one token: ``forward`` and a token shift on what it leaves (``mix``, and
        the requests' last normed rows in ``state``), in one kernel."""
        if self.weight.dtype != torch.float32:
            raise RuntimeError("the norm in front of a token shift keeps its weight in 32-bit (weight_32bit=True)")
        self.rt.ops.add_rmsnorm_shift(x, delta, self.weight, self.eps, out, mix, state, ctx, groups=self.groups)
        return out


class OutputRMSNorm(Norm):
    """The norm of a block whose sub-layers read the residual stream itself: it sits on a sub-layer's
    OUTPUT, and what it leaves is added to the stream, ``x += mult * y * rsqrt(mean(y^2) + eps) * w``
    with ``w`` the stored weight, or ``1 + w`` with ``one_plus``.  All in 32-bit, the weight too."""

    def __init__(self, dim: int, eps: float, mult: float = 1.0, weight_name: str = "weight", one_plus: bool = False):
        self.dim, self.eps, self.mult = int(dim), float(eps), float(mult)
        self.weight = None
        self.weight_name = weight_name
        self.one_plus = bool(one_plus)

    def param_specs(self) -> Dict[str, ParamSpec]:
        if self.one_plus:
            return {self.weight_name: ParamSpec((self.dim,), mean=0.0, std=0.1)}
        return {self.weight_name: ParamSpec((self.dim,), "norm")}

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.weight = tensors[self.weight_name].to(device=rt.device, dtype=torch.float32).contiguous()

    def add(self, ctx, x, delta, act=None):
        """``x`` (32-bit stream) gains the normed ``delta`` ([T, d], or a stack of 32-bit partial sums);
        ``act`` takes the new rows in its dtype, for the sub-layer that reads the stream next."""
        self.rt.ops.norm_residual(x, delta, self.weight, self.eps, mult=self.mult, one_plus=self.one_plus, act=act)


class LayerNorm(Norm):
    """``(x - mean) / sqrt(var + eps) * w + b`` over each row, the variance being the mean of the squared
    deviations; 32-bit arithmetic, weight and bias kept in 32-bit.  Tensors: the weight under
    ``weight_name`` ("" where it carries the norm's own name), the bias under that name + ``bias_suffix``."""

    cuts_rows = False
    plain_rms = False
    layer_norm = True          # a block may make this norm's output in the pass that last changes the stream

    def __init__(self, dim: int, eps: float, weight_name: str = "weight", bias_name: str = "bias"):
        self.dim, self.eps = int(dim), float(eps)
        self.weight_name, self.bias_name = weight_name, bias_name
        self.weight = self.bias = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {self.weight_name: ParamSpec((self.dim,), "norm"), self.bias_name: ParamSpec((self.dim,), mean=0.0, std=0.1)}

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        f32 = lambda name: tensors[name].to(device=rt.device, dtype=torch.float32).contiguous()
        self.weight, self.bias = f32(self.weight_name), f32(self.bias_name)

    def forward(self, ctx, x, delta, out, rows=None, x_rows=None):
        if delta is not None or x_rows is not None:
            raise RuntimeError("LayerNorm norms a complete stream: nothing pending, no cut to rows")
        self.rt.ops.layer_norm(x, self.weight, self.bias, self.eps, out, rows)
        return out
