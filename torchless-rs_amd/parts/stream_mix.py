"""Parts that change the residual stream between the runs of the schedule.

`DepthAverage`: the stream that goes on after a run is a weighted sum of the results of every run
so far.  With X_0 the embedding's output and X_t the stream as run t - 1 left it, call t of a step
(t = 0 before the first run, t = 1, 2, ... before run t and, the last one, before the model's
final norm) keeps X_t and turns the stream into

    x <- sum over j = 0 .. t of w_t[j] * X_j

with w_t a tensor of t + 1 weights of its own for every t >= 1 (call 0 only keeps X_0).  A run reads
the averaged stream; its result X_(t + 1) is what it leaves, before the next averaging.  All in
float32.
"""
from __future__ import annotations

from typing import Dict, Sequence

import torch

from ..kernels import ops
from ..weights.binding import WeightSpec
from .base import StreamPart, register_part


class DepthAverage(StreamPart):
    graph_safe = True

    def __init__(self, hidden_size: int, names: Sequence[str]):
        """`names`: the tensors of weights for t = 1, 2, ... (call t of a step uses names[t - 1], a
        tensor of t + 1 weights)."""
        self.H = int(hidden_size)
        self.names = list(names)
        self.coef = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {name: WeightSpec((t + 2,), init="mean") for t, name in enumerate(self.names)}

    def load(self, tensors, compute_dtype) -> None:
        self.coef = [tensors[name].to(torch.float32).contiguous() for name in self.names]
        self.one = torch.ones(1, dtype=torch.float32, device=self.coef[0].device) if self.coef else None

    def mix_terms(self, ctx, x: torch.Tensor, t: int):
        """(kept, weights, t): the operands of `ops.depth_average` for call t, for a norm whose kernel
        does the sum on its way (`Norm.add_to`'s `between`)."""
        if not (0 <= t <= len(self.names)):
            raise ValueError(f"average {t} of {len(self.names)}")
        kept = ctx.workspace.get("depth_kept", (len(self.names) + 1,) + tuple(x.shape), torch.float32)
        return kept, (self.one if t == 0 else self.coef[t - 1]), t

    def forward(self, ctx, x: torch.Tensor, embedded, t: int) -> None:
        ops.depth_average(x, *self.mix_terms(ctx, x, t))


register_part("stream", "depth_average", DepthAverage)
