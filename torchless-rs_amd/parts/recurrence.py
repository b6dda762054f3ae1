"""A recurrence per channel with an update gate and a candidate that are functions of the present row
only (the smallest of the gated recurrent units): nothing of the state enters its gates.

With `width` channels, one product over the mixer's input y gives a row [a | b | g], and per
channel

    z_t = logistic(a_t + bias_z) ,  c_t = cand(b_t + bias_x) ,
    S_t = (1 - z_t) S_(t-1) + z_t c_t ,
    out = W_o (S_t * silu(g_t))

with cand(u) = u + 1/2 where u >= 0 and logistic(u) below (a positive candidate).  S starts at
zero.  What a sequence keeps is one float a channel (`StateRequest`), whatever its length;
nothing per position.  Gates, candidates, the state and silu(g) are float32 in both dtypes; the
gated state is rounded to the compute dtype once, for the output projection.

A step of many rows cuts each sequence into runs that a workgroup each goes through, after a
first pass has worked out what every run does to the state (`ops.gated_recurrence`); single
tokens and short portions go row by row.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.cache import StateRequest
from ..kernels import ops
from ..weights.binding import WeightSpec
from .base import Mixer, register_part
from .linear import Linear

RUNS_FROM = 128          # a step whose longest sequence brings this many rows goes by runs


class GatedRecurrenceMixer(Mixer):
    graph_safe = True
    closes_stream = True          # its last write to the stream is `Linear.add_into`

    NAMES = {"z": "z", "x": "x", "g": "g", "o": "o", "z_bias": "z.b", "x_bias": "x.b"}

    def __init__(self, hidden_size: int, width: int, bias: bool = True, prefix: str = "mix.",
                 names: Optional[Dict[str, str]] = None):
        unknown = set(names or {}) - set(self.NAMES)
        if unknown:
            raise ValueError(f"recurrence: no tensors called {sorted(unknown)}; there are {sorted(self.NAMES)}")
        self.names = dict(self.NAMES, **(names or {}))
        self.H, self.W, self.bias, self.prefix = int(hidden_size), int(width), bool(bias), prefix
        self.proj = self.o = self.bz = self.bx = None

    def state_request(self):
        return StateRequest((self.W,), torch.float32)

    def may_capture(self, n_rows: int) -> bool:
        return self.proj is not None and self.proj.own_kernels(n_rows) and self.o.own_kernels(n_rows)

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, nm = self.prefix, self.names
        out = {p + nm["z"]: WeightSpec((self.W, self.H))}
        if self.bias:
            out[p + nm["z_bias"]] = WeightSpec((self.W,))
        out[p + nm["x"]] = WeightSpec((self.W, self.H))
        if self.bias:
            out[p + nm["x_bias"]] = WeightSpec((self.W,))
        out[p + nm["g"]] = WeightSpec((self.W, self.H))
        out[p + nm["o"]] = WeightSpec((self.H, self.W))
        return out

    def load(self, tensors, compute_dtype) -> None:
        p, nm = self.prefix, self.names
        ws = [tensors[p + nm[k]] for k in ("z", "x", "g")]
        if len({w.dtype for w in ws}) > 1:
            ws = [w.to(torch.float32) for w in ws]
        self.proj = Linear(torch.cat(ws, dim=0), tiled=True)
        self.o = Linear(tensors[p + nm["o"]], tiled=True)
        if self.bias:
            self.bz = tensors[p + nm["z_bias"]].to(torch.float32).contiguous()
            self.bx = tensors[p + nm["x_bias"]].to(torch.float32).contiguous()

    def _gated_state(self, ctx, run, y: torch.Tensor) -> torch.Tensor:
        n = y.shape[0]
        ws = ctx.workspace
        proj = ws.get("gru_proj", (n, 3 * self.W), torch.float32)
        self.proj(y, proj)
        h = ws.get("gru_h", (n, self.W), ctx.dtype)
        runs, scratch = 0, None
        if ctx.max_new >= RUNS_FROM and not ctx.host.get("fixed_launches"):
            chunk = ops.gated_recurrence_chunk()
            runs = int(sum(-(-int(r) // chunk) for r in ctx.host["n_new"]))
            scratch = ws.get("gru_runs", ((2 * runs + ctx.n_seqs) * self.W,), torch.float32)
        ops.gated_recurrence(proj, self.bz, self.bx, run.state, ctx.cu_seqlens, ctx.slots, h, runs, scratch)
        return h

    def forward(self, ctx, run, y: torch.Tensor, x: torch.Tensor) -> None:
        self.o.add_into(self._gated_state(ctx, run, y), x, ctx, "gru_o_parts")

    def produce(self, ctx, run, y: torch.Tensor, out: torch.Tensor) -> None:
        """The result stored in `out` (float32 [n, H]) instead of added to the stream."""
        self.o(self._gated_state(ctx, run, y), out)


register_part("mixer", "gated_recurrence", GatedRecurrenceMixer)
