"""A state-space mixer: per head a matrix state carried along the sequence by a linear recurrence.

With inner = n_heads * head_dim, N = state_size and G groups, one product over the mixer's input
gives a row [z (inner) | u (inner + 2 G N) | dt (n_heads)].  u passes a causal convolution per
channel over its last `conv_taps` rows (a weight [channels, taps] whose last column multiplies
the current row, a bias; zeros before the start of a sequence) and silu, and is then read as
[x | B | C].  Per head h, which reads B and C of group h // (n_heads / G):

    dt' = softplus(dt + dt_bias[h]) ,  a = exp(-exp(A_log[h]) * dt')
    S <- a S + dt' B x^T      (S: [N, head_dim])
    y  = S^T C + D[h] x

The heads' y side by side are multiplied by silu(z), normed in `norm_groups` equal parts (each by
its own root mean square, eps inside the root) times a weight, and projected back.

What a sequence keeps is of fixed size whatever its length (`StateRequest`): the last
conv_taps - 1 rows of u and the states S, all float32; nothing per position.  dt', a, the state,
y, the gate and the norm are float32 in both dtypes; x, B and C are rounded to the compute
dtype once, after the convolution's silu.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.cache import StateRequest
from ..kernels import ops
from ..weights.binding import WeightSpec
from .base import Mixer, register_part
from .linear import Linear


class StateSpaceMixer(Mixer):
    graph_safe = True
    closes_stream = True          # its last write to the stream is `Linear.add_into`

    NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "A_log": "A_log", "D": "D",
             "norm": "norm", "o": "o"}

    def __init__(self, hidden_size: int, n_heads: int, head_dim: int, state_size: int, groups: int = 1,
                 conv_taps: int = 4, norm_groups: int = 1, norm_eps: float = 1e-6, conv_bias: bool = True,
                 prefix: str = "mix.", names: Optional[Dict[str, str]] = None):
        if n_heads % groups:
            raise ValueError(f"state space: {n_heads} heads are not a multiple of {groups} groups")
        if (n_heads * head_dim) % norm_groups:
            raise ValueError(f"state space: {n_heads * head_dim} channels do not split into {norm_groups} normed parts")
        unknown = set(names or {}) - set(self.NAMES)
        if unknown:
            raise ValueError(f"state space: no tensors called {sorted(unknown)}; there are {sorted(self.NAMES)}")
        self.names = dict(self.NAMES, **(names or {}))
        self.H, self.heads, self.dv, self.N, self.G = int(hidden_size), int(n_heads), int(head_dim), int(state_size), int(groups)
        self.taps, self.parts, self.eps, self.has_conv_bias = int(conv_taps), int(norm_groups), float(norm_eps), bool(conv_bias)
        self.inner = self.heads * self.dv
        self.C = self.inner + 2 * self.G * self.N
        self.width = self.inner + self.C + self.heads
        self.conv_elems = (self.taps - 1) * self.C
        self.prefix = prefix
        self.proj = self.o = None

    def state_request(self):
        return StateRequest((self.conv_elems + self.heads * self.N * self.dv,), torch.float32)

    def may_capture(self, n_rows: int) -> bool:
        return self.proj is not None and self.proj.own_kernels(n_rows) and self.o.own_kernels(n_rows)

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, nm = self.prefix, self.names
        out = {p + nm["in"]: WeightSpec((self.width, self.H)), p + nm["conv"]: WeightSpec((self.C, self.taps))}
        if self.has_conv_bias:
            out[p + nm["conv_bias"]] = WeightSpec((self.C,))
        out.update({p + nm["dt_bias"]: WeightSpec((self.heads,)), p + nm["A_log"]: WeightSpec((self.heads,)),
                    p + nm["D"]: WeightSpec((self.heads,)), p + nm["norm"]: WeightSpec((self.inner,), init="ones"),
                    p + nm["o"]: WeightSpec((self.H, self.inner))})
        return out

    def load(self, tensors, compute_dtype) -> None:
        p, nm = self.prefix, self.names

        def f32(key):
            return tensors[p + nm[key]].to(torch.float32).contiguous()

        self.proj = Linear(tensors[p + nm["in"]], tiled=True)
        self.o = Linear(tensors[p + nm["o"]], tiled=True)
        self.conv_w = f32("conv")
        self.conv_b = f32("conv_bias") if self.has_conv_bias else None
        self.dt_bias, self.A_log, self.D, self.norm_w = f32("dt_bias"), f32("A_log"), f32("D"), f32("norm")

    def forward(self, ctx, run, y: torch.Tensor, x: torch.Tensor) -> None:
        n = y.shape[0]
        ws = ctx.workspace
        block = run.state                               # [slots, conv rows | states] float32
        proj = ws.get("ssm_proj", (n, self.width), torch.float32)
        self.proj(y, proj)
        u = ws.get("ssm_u", (n, self.C), ctx.dtype)
        ops.ssm_conv(proj, self.inner, self.C, self.conv_w, self.conv_b, block, ctx.row_seq, ctx.cu_seqlens, ctx.slots, u,
                     single=ctx.all_single)
        yy = ws.get("ssm_y", (n, self.inner), torch.float32)
        ops.ssm_scan(u, proj, self.inner + self.C, self.G, self.N, self.heads, self.dv, self.dt_bias, self.A_log, self.D,
                     block[:, self.conv_elems:], ctx.cu_seqlens, ctx.slots, yy)
        g = ws.get("ssm_g", (n, self.inner), ctx.dtype)
        ops.ssm_gate_norm(yy, proj, self.parts, self.norm_w, self.eps, g)
        self.o.add_into(g, x, ctx, "ssm_o_parts")


register_part("mixer", "state_space", StateSpaceMixer)
