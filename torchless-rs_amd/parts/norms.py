"""Norms over a row of the stream, in float32.

RMSNorm: y = x / sqrt(mean(x^2) + eps) * w (src/kernels/mod.rs:558-568 of the
reference; weight used as it is).  LayerNorm: y = (x - mean) / sqrt(var + eps) * w + b
with var the mean of the squared deviations, a weight and an optional bias."""
from __future__ import annotations

from typing import Dict

import torch

from ..kernels import ops
from ..weights.binding import WeightSpec
from .base import Norm, RmsForm, register_part


class RMSNorm(Norm):
    graph_safe = True
    takes_pending = True        # adds partial products left in ctx.pending while it reads the stream

    def __init__(self, size: int, eps: float, name: str = "weight"):
        """`name`: the weight's leaf name behind the norm's prefix ("" where the prefix is the tensor)."""
        self.size = int(size)
        self.eps = float(eps)
        self.name = name
        self.weight = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {self.name: WeightSpec((self.size,), init="ones")}

    def load(self, tensors, compute_dtype) -> None:
        self.weight = tensors[self.name].to(torch.float32).contiguous()

    def add_to(self, ctx, z: torch.Tensor, x: torch.Tensor, out=None, bias=None, then=None) -> None:
        """x += norm(z + bias) in one kernel.  `then` = (norm, buffer): the norm that reads the
        stream next, if it has this form too, runs on the new row in the same kernel and leaves its
        result in `buffer`; `read_through_norm` of that norm then finds it done."""
        if bias is not None:
            z += bias
        nxt = then[0].rms_form() if then is not None else None
        if nxt is not None and nxt.size == self.size:
            ops.rmsnorm_add(z, self.weight, self.eps, x, nxt.weight, nxt.eps, then[1])
            ctx.prenormed = (then[0], then[1], None)
        else:
            ops.rmsnorm_add(z, self.weight, self.eps, x)
        if out is not None:
            if out.dtype == torch.float32:
                out.copy_(x)
            else:
                ops.cast_rows(x, out)

    def rms_form(self) -> RmsForm:
        return RmsForm(self.weight, self.size, self.eps)

    def forward(self, ctx, x: torch.Tensor, out: torch.Tensor) -> None:
        """Partial products waiting in `ctx.pending` are added to x on the way."""
        pend = getattr(ctx, "pending", None)
        if pend is not None and self.size % 4 == 0 and self.size <= 8192:
            ops.add_rmsnorm(x, pend, self.weight, self.eps, out)
            ctx.pending = None
            return
        if pend is not None:
            ops.add_partials(x, pend)
            ctx.pending = None
        ops.rmsnorm(x, self.weight, self.eps, out)


class LayerNorm(Norm):
    """Mean and variance over the row; a weight and, with `bias_name`, a bias of the norm's own.
    Besides the plain `forward` it can be the norm of a sublayer's OUTPUT (`add_to`): x += norm(z),
    in one kernel that also leaves the new stream in the compute dtype for the product that reads
    it next, or (`then`) runs the layer norm that reads the stream next on the new row."""
    graph_safe = True

    def __init__(self, size: int, eps: float, name: str = "weight", bias_name: str = None):
        """`name`: the weight's leaf name behind the norm's prefix ("" where the prefix is the tensor);
        `bias_name`: the bias's (None: the norm has none)."""
        self.size = int(size)
        self.eps = float(eps)
        self.name = name
        self.bias_name = bias_name
        self.weight = self.beta = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        out = {self.name: WeightSpec((self.size,), init="ones")}
        if self.bias_name is not None:
            out[self.bias_name] = WeightSpec((self.size,))
        return out

    def load(self, tensors, compute_dtype) -> None:
        self.weight = tensors[self.name].to(torch.float32).contiguous()
        if self.bias_name is not None:
            self.beta = tensors[self.bias_name].to(torch.float32).contiguous()

    def forward(self, ctx, x: torch.Tensor, out: torch.Tensor) -> None:
        flush = getattr(ctx, "pending", None)
        if flush is not None:
            ops.add_partials(x, flush)
            ctx.pending = None
        ops.layernorm(x, self.weight, self.eps, out, beta=self.beta)

    takes_between = True          # `add_to` may be handed what a stream part does between this norm and the next

    def add_to(self, ctx, z: torch.Tensor, x: torch.Tensor, out=None, bias=None, then=None, between=None) -> None:
        """`between` = (kept, coef, t) (`ops.depth_average`'s operands): the stream's new version is kept and
        replaced by the weighted sum of its versions before `then`'s norm reads it."""
        nxt = then[0] if then is not None and isinstance(then[0], LayerNorm) and then[0].size == self.size else None
        if out is None and ops.layernorm_rows_in_registers(self.size):
            if nxt is not None:
                ops.layernorm_add_norm(z, self.weight, self.beta, self.eps, x, bias=bias, w_next=nxt.weight,
                                       beta_next=nxt.beta, eps_next=nxt.eps, out=then[1], mix=between)
                ctx.prenormed = (nxt, then[1], None)
            else:
                ops.layernorm_add_norm(z, self.weight, self.beta, self.eps, x, bias=bias, mix=between)
            return
        ops.layernorm(z, self.weight, self.eps, out, add_to=x, bias=bias, beta=self.beta)
        if between is not None:
            ops.depth_average(x, *between)
            if out is not None:
                if out.dtype == torch.float32:
                    out.copy_(x)
                else:
                    ops.cast_rows(x, out)


register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "layernorm", LayerNorm)
