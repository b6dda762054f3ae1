"""Feed-forwards without a gate, and a routed mixture of them.

`PlainFeedForward`: down(act(up y)), act one of `ops.EXPERT_ACTIVATIONS` (relu2: the square of
max(., 0)).

`RoutedExperts`: `n_experts` such layers of which every token uses `top`.  The router is one
more product, in float32: s = softmax(W_r y) over all experts.  The experts form
`group_count` equal groups of neighbours; a group's score is its largest s, and only experts of
the `group_keep` best groups can be chosen (no groups: any expert).  The `top` experts with the
largest s are chosen; the result is the sum of their outputs weighted by their s, not
renormalised, plus a shared expert's (`shared_size`; None: none) that runs for every token.
`score` "sigmoid" makes every expert's score its own logistic function of the router's product
instead of a softmax over the experts.  `gated` experts have a gate beside the up projection,
down(act(gate t, up t)) with the clamped activation of `ops.GateTerms` (`activation_constants`:
limit, alpha, shift; the shared expert's limit may differ, `shared_limit`), and `weight_on`
"input" multiplies an expert's INPUT t = s y by the router's weight instead of its output.

All experts run as ONE wide feed-forward: their up projections stacked by rows (the shared
expert's behind them), the activation times the row's weight of the column's expert, which is
zero for an expert that was not chosen, and their down projections side by side.  That is two
products of the framework's own kinds and no gather or scatter, whatever the tokens choose; it
reads every expert's weights in every step, as a step of many rows does anyway, and multiplies
`n_experts / top` times what the chosen experts alone would.

A step of many rows in bfloat16 (on average `GROUPED_ROWS_PER_EXPERT` rows an expert or more, more rows
than the framework's own product kernels take, so that no graph holds the step) sorts the
(row, chosen expert) pairs by expert and runs every expert's two products over its own rows
(`_grouped`): the chosen experts' multiplications alone, at the price of one count per expert
read back by the host.

A step of few rows (rows * top <= n_experts: the rows cannot use every expert) runs the chosen
experts alone: per row two products of its experts' matrices with a vector
(`ops.expert_rows_up`, `ops.expert_rows_down`), which read `top` experts' weights a row and
nothing else.  Both ways round the hidden activations, times the router's weight, to the
compute dtype and sum in float32.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from ..weights.binding import WeightSpec
from .base import FeedForward, flush_pending, register_part
from .linear import Linear


GROUPED_ROWS_PER_EXPERT = 128      # from this many rows an expert on average, experts run over their own rows


class PlainFeedForward(FeedForward):
    graph_safe = True
    closes_stream = True

    NAMES = {"up": "up", "down": "down"}

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "relu2", prefix: str = "mlp.",
                 names: Optional[Dict[str, str]] = None):
        if activation not in ops.EXPERT_ACTIVATIONS:
            raise ValueError(f"feed-forward: no activation {activation!r}; there are {sorted(ops.EXPERT_ACTIVATIONS)}")
        self.H, self.I, self.activation, self.prefix = int(hidden_size), int(intermediate_size), activation, prefix
        self.names = dict(self.NAMES, **(names or {}))
        self.up = self.down = None

    def may_capture(self, n_rows: int) -> bool:
        return self.up is not None and self.up.own_kernels(n_rows) and self.down.own_kernels(n_rows)

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, nm = self.prefix, self.names
        return {p + nm["up"]: WeightSpec((self.I, self.H)), p + nm["down"]: WeightSpec((self.H, self.I))}

    def load(self, tensors, compute_dtype) -> None:
        p, nm = self.prefix, self.names
        self.up = Linear(tensors[p + nm["up"]], tiled=True)
        self.down = Linear(tensors[p + nm["down"]], tiled=True)

    def _hidden(self, ctx, y: torch.Tensor) -> torch.Tensor:
        n = y.shape[0]
        u = ctx.workspace.get("pff_u", (n, self.I), torch.float32)
        self.up(y, u)
        h = ctx.workspace.get("pff_h", (n, self.I), ctx.dtype)
        ops.expert_act(u, None, 0, self.I, self.activation, h)
        return h

    def forward(self, ctx, y: torch.Tensor, x: torch.Tensor) -> None:
        self.down.add_into(self._hidden(ctx, y), x, ctx, "pff_down_parts")

    def produce(self, ctx, y: torch.Tensor, out: torch.Tensor) -> None:
        self.down(self._hidden(ctx, y), out)


class RoutedExperts(FeedForward):
    graph_safe = True
    closes_stream = True

    # leaf names under `prefix`; "{e}" is the expert's number
    NAMES = {"router": "router", "up": "e{e}.up", "down": "e{e}.down", "shared_up": "shared.up",
             "shared_down": "shared.down", "gate": "e{e}.gate", "shared_gate": "shared.gate"}
    SCORES = ("softmax", "sigmoid")
    GATED_ACTIVATION = "swish_clamped"

    def __init__(self, hidden_size: int, n_experts: int, top: int, expert_size: int, group_count: Optional[int] = None,
                 group_keep: Optional[int] = None, shared_size: Optional[int] = None, activation: str = "relu2",
                 prefix: str = "mlp.", names: Optional[Dict[str, str]] = None, score: str = "softmax",
                 gated: bool = False, activation_constants: Optional[Dict[str, float]] = None,
                 shared_limit: Optional[float] = None, weight_on: str = "output"):
        self.gated = bool(gated)
        if score not in self.SCORES:
            raise ValueError(f"experts: scores are one of {self.SCORES}, got {score!r}")
        if weight_on not in ("output", "input"):
            raise ValueError(f"experts: the router's weight is on an expert's 'output' or 'input', got {weight_on!r}")
        if self.gated:
            need = {"limit", "alpha", "shift"}
            if activation != self.GATED_ACTIVATION or set(activation_constants or {}) != need:
                raise ValueError(f"experts: gated experts have the activation {self.GATED_ACTIVATION!r} with the "
                                 f"constants {sorted(need)}, got {activation!r} with {sorted(activation_constants or {})}")
            c = activation_constants
            self.gate_terms = ops.GateTerms(c["limit"], c["alpha"], c["shift"], shared_limit, weight_on == "input")
        elif activation not in ops.EXPERT_ACTIVATIONS:
            raise ValueError(f"experts: no activation {activation!r}; there are {sorted(ops.EXPERT_ACTIVATIONS)}")
        elif weight_on != "output" or activation_constants or shared_limit is not None:
            raise ValueError("experts: the weight on the input, constants and a shared limit go with gated experts")
        self.logistic = score == "sigmoid"
        if not (1 <= top <= n_experts):
            raise ValueError(f"experts: {top} of {n_experts}")
        if group_count:
            if n_experts % group_count or not (1 <= (group_keep or 0) <= group_count) or group_keep * (n_experts // group_count) < top:
                raise ValueError(f"experts: {n_experts} in {group_count} groups of which {group_keep} are kept cannot give {top}")
        self.H, self.E, self.top, self.ff = int(hidden_size), int(n_experts), int(top), int(expert_size)
        self.groups, self.keep = (int(group_count), int(group_keep)) if group_count else (0, 0)
        self.shared = int(shared_size) if shared_size else 0
        self.total = self.E * self.ff + self.shared
        self.activation, self.prefix = activation, prefix
        self.names = dict(self.NAMES, **(names or {}))
        self.router = self.up = self.down = None

    def may_capture(self, n_rows: int) -> bool:
        return self.up is not None and self.up.own_kernels(n_rows) and self.down.own_kernels(n_rows)

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, nm = self.prefix, self.names
        out: Dict[str, WeightSpec] = {}
        for e in range(self.E):
            if self.gated:
                out[p + nm["gate"].format(e=e)] = WeightSpec((self.ff, self.H))
            out[p + nm["up"].format(e=e)] = WeightSpec((self.ff, self.H))
            out[p + nm["down"].format(e=e)] = WeightSpec((self.H, self.ff))
        out[p + nm["router"]] = WeightSpec((self.E, self.H))
        if self.shared:
            if self.gated:
                out[p + nm["shared_gate"]] = WeightSpec((self.shared, self.H))
            out[p + nm["shared_up"]] = WeightSpec((self.shared, self.H))
            out[p + nm["shared_down"]] = WeightSpec((self.H, self.shared))
        return out

    def load(self, tensors, compute_dtype) -> None:
        p, nm = self.prefix, self.names
        ups = []
        for e in range(self.E):          # a gated expert's rows: [gate | up]
            ups += ([tensors[p + nm["gate"].format(e=e)]] if self.gated else []) + [tensors[p + nm["up"].format(e=e)]]
        downs = [tensors[p + nm["down"].format(e=e)] for e in range(self.E)]
        if self.shared:
            ups += ([tensors[p + nm["shared_gate"]]] if self.gated else []) + [tensors[p + nm["shared_up"]]]
            downs.append(tensors[p + nm["shared_down"]])
        if len({w.dtype for w in ups + downs}) > 1:
            ups, downs = [w.to(torch.float32) for w in ups], [w.to(torch.float32) for w in downs]
        self.up = Linear(torch.cat(ups, dim=0), tiled=True)          # [E * ff + shared, H]; gated: twice the rows
        self.down = Linear(torch.cat(downs, dim=1), tiled=True)      # [H, E * ff + shared]
        self.router = tensors[p + nm["router"]].to(torch.float32).contiguous()

    def few_rows(self, y: torch.Tensor) -> bool:
        """Do the rows of `y` run their chosen experts alone?"""
        return y.shape[0] * self.top <= self.E and self.up.weight.dtype == self.down.weight.dtype == y.dtype

    def _rows(self, ctx, y: torch.Tensor, out: torch.Tensor, accumulate: bool) -> None:
        n = y.shape[0]
        ws = ctx.workspace
        weights = ws.get("experts_w", (n, self.E), torch.float32)
        chosen = ws.get("experts_chosen", (n, self.top), torch.int32)
        ops.route(y, self.router, self.groups, self.keep, self.top, weights, chosen, logistic=self.logistic)
        hs = ws.get("experts_hs", (n, self.top * self.ff + self.shared), y.dtype)
        if self.gated:
            ops.expert_rows_gated_up(y, self.up.weight, chosen, weights, self.ff, self.shared, self.gate_terms, hs)
        else:
            ops.expert_rows_up(y, self.up.weight, chosen, weights, self.ff, self.shared, self.activation, hs)
        ops.expert_rows_down(hs, self.down.weight, chosen, self.E, self.ff, self.shared, out, accumulate)

    def many_rows(self, ctx, y: torch.Tensor) -> bool:
        """Do the rows of `y` run expert by expert over each expert's own rows?"""
        n = y.shape[0]
        return (y.dtype == torch.bfloat16 and self.up.weight.dtype == self.down.weight.dtype == torch.bfloat16
                and n * self.top >= GROUPED_ROWS_PER_EXPERT * self.E and not self.up.own_kernels(n)
                and not ctx.host.get("fixed_launches"))

    def _grouped(self, ctx, y: torch.Tensor, out: torch.Tensor, accumulate: bool) -> None:
        n, E, top, ff, H = y.shape[0], self.E, self.top, self.ff, self.H
        ws = ctx.workspace
        weights = ws.get("experts_w", (n, E), torch.float32)
        chosen = ws.get("experts_chosen", (n, top), torch.int32)
        ops.route(y, self.router, self.groups, self.keep, self.top, weights, chosen, logistic=self.logistic)
        flat = chosen.view(-1).long()
        order = torch.argsort(flat, stable=True)                       # pairs by expert, a row's place kept within one
        counts = torch.bincount(flat, minlength=E).tolist()            # (the host waits for the router here)
        rows = torch.div(order, top, rounding_mode="floor")
        ys = y.index_select(0, rows)                                   # [n * top, H]
        scale = weights.gather(1, chosen.long()).view(-1).index_select(0, order).view(-1, 1).contiguous()
        up_w, down_w = self.up.weight, self.down.weight
        wide = 2 if self.gated else 1               # a gated expert's rows are [gate | up]
        u = ws.get("experts_gu", (n * top, wide * ff), torch.float32)
        at = 0
        for e, c in enumerate(counts):
            if c:
                ops.gemm(ys[at:at + c], up_w[wide * e * ff:wide * (e + 1) * ff], u[at:at + c])
                at += c
        h = ws.get("experts_gh", (n * top, ff), y.dtype)
        if self.gated:
            ops.expert_gated_act(u, scale, 1, ff, 0, self.gate_terms, h)
        else:
            ops.expert_act(u, scale, 1, ff, self.activation, h)
        z = ws.get("experts_gz", (n * top, H), torch.float32)
        at = 0
        for e, c in enumerate(counts):
            if c:
                torch.mm(h[at:at + c], down_w[:, e * ff:(e + 1) * ff].t(), out_dtype=torch.float32, out=z[at:at + c])
                at += c
        back = torch.empty_like(order)
        back[order] = torch.arange(n * top, device=order.device)
        total = z.index_select(0, back).view(n, top, H).sum(dim=1)     # a row's experts in the order it chose them
        if self.shared:
            us = ws.get("experts_su", (n, wide * self.shared), torch.float32)
            ops.gemm(y, up_w[wide * E * ff:], us)
            hs = ws.get("experts_sh", (n, self.shared), y.dtype)
            if self.gated:
                ops.expert_gated_act(us, None, 0, 0, self.shared, self.gate_terms, hs)
            else:
                ops.expert_act(us, None, 0, self.shared, self.activation, hs)
            total.add_(torch.mm(hs, down_w[:, E * ff:].t(), out_dtype=torch.float32))
        if accumulate:
            out.add_(total)
        else:
            out.copy_(total)

    def _hidden(self, ctx, y: torch.Tensor) -> torch.Tensor:
        n = y.shape[0]
        ws = ctx.workspace
        weights = ws.get("experts_w", (n, self.E), torch.float32)
        ops.route(y, self.router, self.groups, self.keep, self.top, weights, logistic=self.logistic)
        u = ws.get("experts_u", (n, (2 if self.gated else 1) * self.total), torch.float32)
        self.up(y, u)
        h = ws.get("experts_h", (n, self.total), ctx.dtype)
        if self.gated:
            ops.expert_gated_act(u, weights, self.E, self.ff, self.shared, self.gate_terms, h)
        else:
            ops.expert_act(u, weights, self.E, self.ff, self.activation, h)
        return h

    def forward(self, ctx, y: torch.Tensor, x: torch.Tensor) -> None:
        if self.few_rows(y):
            flush_pending(ctx, x)
            self._rows(ctx, y, x, True)
            return
        if self.many_rows(ctx, y):
            flush_pending(ctx, x)
            self._grouped(ctx, y, x, True)
            return
        self.down.add_into(self._hidden(ctx, y), x, ctx, "experts_down_parts")

    def produce(self, ctx, y: torch.Tensor, out: torch.Tensor) -> None:
        if self.few_rows(y):
            self._rows(ctx, y, out, False)
            return
        if self.many_rows(ctx, y):
            self._grouped(ctx, y, out, False)
            return
        self.down(self._hidden(ctx, y), out)


register_part("ffn", "plain", PlainFeedForward)
register_part("ffn", "routed_experts", RoutedExperts)
