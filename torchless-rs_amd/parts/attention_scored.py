"""Grouped-query attention whose scores carry more than q.k, over the same cache.

Every mechanism is a constructor parameter and can be left out:

* biases on the q, k, v and o projections (`bias`);
* a norm of q and of k over the WHOLE projection, all heads at once, before the split
  into heads: t / sqrt(mean(t^2) + eps) * weight (`qk_norm_eps`; None: none);
* a factor on q that grows with the position p, 1 + coef * ln(floor((p + 1) / every) + 1)
  (`q_temperature` = (coef, every));
* a bias on the score by the distance of query and key, -slope_h * (p - j) with
  slope_h = 2^(-e (h + 1) / n_heads) for head h = 0 .. n_heads - 1 (`distance_slope_exponent` = e);
* a sliding window (`window`): p sees j with 0 <= p - j < window;
* a sink: a learned score per head without key or value that counts once in the
  softmax's denominator, unscaled and unbiased (`sink`);
* a gate on each head's output, the logistic function of a projection of the mixer's
  input with one row per head (`head_gate`);
* values of another width than keys (`v_head_dim`);
* keys and values of an earlier run instead of its own (`own_kv` False; the schedule's
  `Run.kv_from` names the run): the mixer then binds q, the gate and o alone and reads
  the keys as that run's cache holds them, with its own window and terms.

No rotation: positions enter through the terms above only.  q, k, v and the gate come
from ONE product (rows [q | k | v | g] laid side by side at load); one row-wise kernel
then adds the biases, norms q and k, scales q, applies the logistic function and splits
(and, when every sequence brings one token, writes k and v straight into their pages).
Scores, softmax weights and the sums over values are float32 in both dtypes.
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Sequence

import torch

from ..cache.cache import KVRequest
from ..kernels import ops
from ..weights.binding import WeightSpec
from .base import Mixer, register_part
from .linear import Linear


class ScoredAttentionMixer(Mixer):
    graph_safe = True

    # leaf names of the tensors under `prefix`
    NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
             "o_bias": "o.b", "q_norm": "q.norm", "k_norm": "k.norm", "sink": "sink", "gate": "g"}

    def __init__(self, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int,
                 v_head_dim: Optional[int] = None, window: Optional[int] = None, own_kv: bool = True,
                 scale: Optional[float] = None, bias: bool = False, qk_norm_eps: Optional[float] = None,
                 q_temperature: Optional[Sequence[float]] = None,
                 distance_slope_exponent: Optional[float] = None, sink: bool = False, head_gate: bool = False,
                 prefix: str = "mix.", names: Optional[Dict[str, str]] = None):
        if n_heads % n_kv_heads:
            raise ValueError(f"attention: {n_heads} heads are not a multiple of {n_kv_heads} KV heads")
        unknown = set(names or {}) - set(self.NAMES)
        if unknown:
            raise ValueError(f"attention: no tensors called {sorted(unknown)}; there are {sorted(self.NAMES)}")
        self.names = dict(self.NAMES, **(names or {}))
        self.H, self.nq, self.nkv = int(hidden_size), int(n_heads), int(n_kv_heads)
        self.dk = int(head_dim)
        self.dv = self.dk if v_head_dim is None else int(v_head_dim)
        self.window = int(window) if window else None
        self.own_kv = bool(own_kv)
        self.scale = 1.0 / math.sqrt(self.dk) if scale is None else float(scale)
        self.bias = bool(bias)
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        if q_temperature is not None:
            coef, every = float(q_temperature[0]), float(q_temperature[1])
            if not every > 0:
                raise ValueError(f"attention: the factor on q steps every {every} positions (must be positive)")
            q_temperature = (coef, every) if coef != 0.0 else None
        self.q_temperature = q_temperature
        self.slope_exponent = None if distance_slope_exponent is None else float(distance_slope_exponent)
        self.sink, self.head_gate = bool(sink), bool(head_gate)
        self.prefix = prefix
        self.ng = self.nq if self.head_gate else 0
        self.proj = self.o = None
        self.proj_terms = self.o_bias = self.sinks = self.slopes = None

    # ---- what it keeps -------------------------------------------------------
    def kv_request(self):
        if not self.own_kv:
            return None
        return KVRequest(self.nkv, self.dk, self.window, None if self.dv == self.dk else self.dv)

    def kv_reach(self):
        """How far back this mixer looks at keys, whoever keeps them (None: to the first)."""
        return self.window

    def may_capture(self, n_rows: int) -> bool:
        return self.proj is not None and self.proj.own_kernels(n_rows) and self.o.own_kernels(n_rows)

    # ---- weights -------------------------------------------------------------
    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, nm = self.prefix, self.names
        Q, K, V = self.nq * self.dk, self.nkv * self.dk, self.nkv * self.dv
        out = {p + nm["q"]: WeightSpec((Q, self.H))}
        if self.bias:
            out[p + nm["q_bias"]] = WeightSpec((Q,))
        if self.own_kv:
            out[p + nm["k"]] = WeightSpec((K, self.H))
            out[p + nm["v"]] = WeightSpec((V, self.H))
            if self.bias:
                out[p + nm["k_bias"]] = WeightSpec((K,))
                out[p + nm["v_bias"]] = WeightSpec((V,))
        if self.qk_norm_eps is not None:
            out[p + nm["q_norm"]] = WeightSpec((Q,), init="ones")
            if self.own_kv:
                out[p + nm["k_norm"]] = WeightSpec((K,), init="ones")
        if self.sink:
            out[p + nm["sink"]] = WeightSpec((self.nq,))
        if self.head_gate:
            out[p + nm["gate"]] = WeightSpec((self.nq, self.H))
        out[p + nm["o"]] = WeightSpec((self.H, self.nq * self.dv))
        if self.bias:
            out[p + nm["o_bias"]] = WeightSpec((self.H,))
        return out

    def load(self, tensors, compute_dtype) -> None:
        p, nm = self.prefix, self.names

        def t(key):
            return tensors[p + nm[key]]

        def f32(key):
            return t(key).to(torch.float32).contiguous()

        ws = [t("q")] + ([t("k"), t("v")] if self.own_kv else []) + ([t("gate")] if self.head_gate else [])
        if len({w.dtype for w in ws}) > 1:
            ws = [w.to(torch.float32) for w in ws]
        self.proj = Linear(torch.cat(ws, dim=0), tiled=True)      # single-token steps stream both from tiled copies
        self.o = Linear(t("o"), tiled=True)
        dev = ws[0].device
        bias = None
        if self.bias:
            bs = [f32("q_bias")] + ([f32("k_bias"), f32("v_bias")] if self.own_kv else [])
            bias = torch.cat(bs + [torch.zeros(self.ng, dtype=torch.float32, device=dev)]).contiguous()
            self.o_bias = f32("o_bias")
        normed = self.qk_norm_eps is not None
        self.proj_terms = ops.ProjectionTerms(
            bias=bias, q_norm=f32("q_norm") if normed else None,
            k_norm=f32("k_norm") if normed and self.own_kv else None,
            eps=self.qk_norm_eps or 0.0, temperature=self.q_temperature)
        self.sinks = f32("sink") if self.sink else None
        if self.slope_exponent is not None:
            h = torch.arange(1, self.nq + 1, dtype=torch.float64)
            self.slopes = torch.pow(2.0, -self.slope_exponent * h / self.nq).to(torch.float32).to(dev)
        self.terms = ops.ScoreTerms(self.scale, self.window, self.slopes, self.sinks)

    # ---- one step --------------------------------------------------------------
    def produce(self, ctx, run, y: torch.Tensor, out: torch.Tensor):
        """The mixer's result stored in `out` (float32 [n, H]); returns the bias of the output
        projection, which the caller adds (None without biases)."""
        n, nq, nkv, dk, dv, ng = y.shape[0], self.nq, self.nkv, self.dk, self.dv, self.ng
        ws = ctx.workspace
        group = run.kv_group
        pages = group.storage[run.kv_layer]
        table = ctx.tables[run.kv_group_index]
        own = nkv if self.own_kv else 0
        proj = ws.get("sattn_proj", (n, nq * dk + own * (dk + dv) + ng), torch.float32)
        self.proj(y, proj)
        q = ws.get("sattn_q", (n, nq, dk), ctx.dtype)
        gate = ws.get("sattn_gate", (n, ng), torch.float32) if ng else None
        att = ws.get("sattn_out", (n, nq, dv), ctx.dtype)
        k = v = vt = None
        tiles = ops.scored_on_matrix_cores(ctx.dtype, dk, dv) and not ctx.all_single    # values also transposed
        if self.own_kv and ctx.all_single:
            # one token a sequence: k and v go straight into the pages, then everything is read there
            ops.split_projection(proj, ctx.row_pos, self.proj_terms, nq, nkv, dk, dv, ng, q, None, None, gate,
                                 table=table, ring_pages=group.ring_pages, pages=pages)
        elif self.own_kv:
            tag = f"_{run.index}" if run.kv_read_later else ""
            k = ws.get("sattn_k" + tag, (n, nkv, dk), ctx.dtype)
            v = ws.get("sattn_v" + tag, (n, nkv, dv), ctx.dtype)
            ops.split_projection(proj, ctx.row_pos, self.proj_terms, nq, nkv, dk, dv, ng, q, k, v, gate)
            if tiles:       # the matrix cores read values along the keys
                vt = ws.get("sattn_vt" + tag, (nkv, dv, ctx.host["aligned_cols"]), ctx.dtype)
                ops.v_tiles_rows(v, vt, ctx.cu_seqlens, ctx.tile_off, ctx.len_before, ctx.len_after)
            if run.kv_read_later:
                ctx.host[f"kv_new_{run.index}"] = (k, v, vt)
        else:
            ops.split_projection(proj, ctx.row_pos, self.proj_terms, nq, 0, dk, dv, ng, q, None, None, gate)
            if not ctx.all_single:
                k, v, vt = ctx.host[f"kv_new_{run.kv_source}"]
        if ctx.all_single:
            ops.attention_scored(q, None, None, pages, nkv, dv, table, group.ring_pages, ctx, ctx.len_after,
                                 self.terms, gate, att)
        else:
            ops.attention_scored(q, k, v, pages, nkv, dv, table, group.ring_pages, ctx, ctx.len_before,
                                 self.terms, gate, att, vt_new=vt)
            if self.own_kv:
                def commit():
                    if vt is not None and pages.dim() == 5:       # values a tile at a time, in whole lines
                        ops.kv_commit_tiles(k, vt, ctx.row_seq, ctx.row_pos, ctx.tile_off, ctx.len_before,
                                            ctx.len_after, table, group.ring_pages, pages)
                    else:
                        ops.kv_commit_wide(k, v, ctx.row_seq, ctx.row_pos, ctx.len_after, table,
                                           group.ring_pages, pages)
                if run.kv_read_later:       # a later run still reads the old rows of the ring
                    ctx.host.setdefault("deferred", []).append(commit)
                else:
                    commit()
        self.o(att.view(n, nq * dv), out)
        return self.o_bias

    def forward(self, ctx, run, y: torch.Tensor, x: torch.Tensor) -> None:
        from .base import flush_pending
        flush_pending(ctx, x)
        z = ctx.workspace.get("sattn_z", tuple(x.shape), torch.float32)
        bias = self.produce(ctx, run, y, z)
        if bias is not None:
            z += bias
        ops.add_partials(x, z.view(1, *z.shape))


def attend_and_commit(ctx, run, q: torch.Tensor, k, v, nkv: int, dk: int, dv: int, terms, gate, att: torch.Tensor,
                      tag: str = "", own: bool = True) -> None:
    """The attention of a step for a mixer that has made q [n, nq, dk] and, unless every sequence
    brings one token (k and v are then None and lie in their pages already), this step's
    k [n, nkv, dk] and v [n, nkv, dv]: the step's rows attend to the pages for cached positions and
    to k and v for the new ones (values transposed by tiles where the matrix cores run), and k and
    v are committed to the pages afterwards.  Scores with no term but the scale and the window go
    through the kernels of the attention without terms where the matrix cores take the shape (one
    product with the values instead of two, and the keys of few rows over a long context cut into
    runs).  A run whose keys a later run reads (`run.kv_read_later`) leaves its new rows in
    `ctx.host["kv_new_<run>"]` and commits at the end of the step (the later run still reads the
    ring's old rows); its k and v must then be buffers that no other run writes.  `own` False: the
    run reads the keys and values of `run.kv_source` (k and v are ignored) and commits nothing."""
    group = run.kv_group
    pages = group.storage[run.kv_layer]
    table = ctx.tables[run.kv_group_index]
    cores = ops.scored_on_matrix_cores(ctx.dtype, dk, dv) and pages.dim() == 5
    bare = (cores and terms.slopes is None and terms.sinks is None and gate is None and not terms.keep_first
            and not terms.chunk and not terms.logistic and att.dtype == ctx.dtype)
    if not own and not ctx.all_single:
        k, v, vt = ctx.host[f"kv_new_{run.kv_source}"]
        if vt is None and cores:
            raise RuntimeError("attention: the run that owns the keys left no transposed values")
        ops.attention_scored(q, k, v, pages, nkv, dv, table, group.ring_pages, ctx, ctx.len_before, terms, gate, att,
                             vt_new=vt)
        return
    if ctx.all_single:
        if bare:
            ops.attention(q, None, None, pages, table, group.ring_pages, ctx, ctx.len_after, terms.window, terms.scale, att)
        else:
            ops.attention_scored(q, None, None, pages, nkv, dv, table, group.ring_pages, ctx, ctx.len_after, terms, gate,
                                 att)
        return
    vt = None
    if cores:
        vt = ctx.workspace.get("attend_vt" + tag, (nkv, dv, ctx.host["aligned_cols"]), ctx.dtype)
        ops.v_tiles_rows(v, vt, ctx.cu_seqlens, ctx.tile_off, ctx.len_before, ctx.len_after)
    if bare:
        ops.attention(q, k, v, pages, table, group.ring_pages, ctx, ctx.len_before, terms.window, terms.scale, att,
                      vt_new=vt)
    else:
        ops.attention_scored(q, k, v, pages, nkv, dv, table, group.ring_pages, ctx, ctx.len_before, terms, gate, att,
                             vt_new=vt)

    def commit():
        if vt is not None and pages.dim() == 5:       # values a tile at a time, in whole lines
            ops.kv_commit_tiles(k, vt, ctx.row_seq, ctx.row_pos, ctx.tile_off, ctx.len_before, ctx.len_after, table,
                                group.ring_pages, pages)
        else:
            ops.kv_commit_wide(k, v, ctx.row_seq, ctx.row_pos, ctx.len_after, table, group.ring_pages, pages)

    if getattr(run, "kv_read_later", False):
        ctx.host[f"kv_new_{run.index}"] = (k, v, vt)
        ctx.host.setdefault("deferred", []).append(commit)
    else:
        commit()


register_part("mixer", "scored_attention", ScoredAttentionMixer)
