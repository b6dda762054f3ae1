"""Grouped-query attention with rotation whose terms act head by head, over the same cache.

Every mechanism is a constructor parameter and can be left out:

* biases on the q, k, v and o projections (`bias`);
* a norm of q and of k PER HEAD: every head divided by its own root mean square over its
  channels (eps inside the root) times a weight of one head's size that all heads share
  (`head_norm_eps`; None: none), before the rotation;
* the position part (`position`), which rotates the first channels of every head of q and k;
* or a norm of q and of k per head AFTER the rotation, with no weight (`unit_norm_eps`; None: none);
* a mask by chunks (`chunk`): p sees j <= p only if both lie in the same run of `chunk` positions
  counted from the sequence's start, floor(p / chunk) == floor(j / chunk);
* weights that are logistic functions of the scores instead of a softmax over the keys
  (`logistic`): a key's weight is 1 / (1 + exp(-(score + b_h))), b_h a learned number per head
  (tensor `score_bias`), every key by itself, not normalised;
* a gate per head, the logistic function of a projection of the mixer's input with one row a head
  (`head_gate`), on the head's output;
* keys and values of an earlier run instead of its own (`own_kv` False; the schedule's
  `Run.kv_from` names the run): the mixer then binds q, the gate and o alone and reads the keys
  as that run's cache holds them (after norm and rotation), with its own queries, mask and terms;
* a sliding window (`window`) beside which the first `keep_first` positions of a sequence stay
  visible: p sees j <= p with p - j < window or j < keep_first.  Kept positions are ordinary
  keys, rotated by their own positions;
* one more in the softmax's denominator (`unit_sink`): a score of 0 that has no key and no value;
* a gate per channel of the concatenated heads, the logistic function of a projection of the
  mixer's input (`channel_gate`);
* values of another width than keys (`v_head_dim`);
* values mixed across layers (`value_mix`): the layer that says "first" leaves its values
  (unrounded) for the step's later layers; one that says "later" replaces its own by
  (1 - lam) v + lam v_first, lam a scalar tensor of the layer, and caches the mixed values.

q, k, v and the gate come from ONE product (rows [q | k | v | g] laid side by side at load); one
kernel then works on the row head by head (`ops.head_prepare`) and, when every sequence brings
one token, writes k and v straight into their pages.  Scores, softmax weights and the sums over
values are float32 in both dtypes.  With first positions kept beside a window the cache keeps
every position of the sequence (a ring of the window's pages would overwrite the kept ones);
the kernels skip what lies between.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from ..cache.cache import KVRequest
from ..kernels import ops
from ..weights.binding import WeightSpec
from .attention_scored import attend_and_commit
from .base import Mixer, PartSpec, flush_pending, make_part, register_part
from .linear import Linear

VALUE_MIX = (None, "first", "later")


class HeadwiseAttentionMixer(Mixer):
    graph_safe = True

    NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
             "o_bias": "o.b", "q_norm": "q.norm", "k_norm": "k.norm", "gate": "g", "mix": "vmix", "score_bias": "pb"}

    def __init__(self, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int,
                 v_head_dim: Optional[int] = None, position: Optional[PartSpec] = None, scale: Optional[float] = None,
                 bias: bool = False, head_norm_eps: Optional[float] = None, window: Optional[int] = None,
                 keep_first: int = 0, unit_sink: bool = False, channel_gate: bool = False,
                 value_mix: Optional[str] = None, prefix: str = "mix.", names: Optional[Dict[str, str]] = None,
                 unit_norm_eps: Optional[float] = None, chunk: Optional[int] = None, logistic: bool = False,
                 head_gate: bool = False, own_kv: bool = True):
        if n_heads % n_kv_heads:
            raise ValueError(f"attention: {n_heads} heads are not a multiple of {n_kv_heads} KV heads")
        if value_mix not in VALUE_MIX:
            raise ValueError(f"attention: value_mix is one of {VALUE_MIX}, got {value_mix!r}")
        unknown = set(names or {}) - set(self.NAMES)
        if unknown:
            raise ValueError(f"attention: no tensors called {sorted(unknown)}; there are {sorted(self.NAMES)}")
        self.names = dict(self.NAMES, **(names or {}))
        self.H, self.nq, self.nkv = int(hidden_size), int(n_heads), int(n_kv_heads)
        self.dk = int(head_dim)
        self.dv = self.dk if v_head_dim is None else int(v_head_dim)
        self.position = make_part("position", position if position is not None else PartSpec("none"))
        self.scale = 1.0 / math.sqrt(self.dk) if scale is None else float(scale)
        self.bias = bool(bias)
        self.head_norm_eps = None if head_norm_eps is None else float(head_norm_eps)
        self.window = int(window) if window else None
        self.keep_first = int(keep_first) if self.window else 0
        if self.keep_first < 0:
            raise ValueError(f"attention: {keep_first} kept positions")
        self.unit_sink, self.channel_gate = bool(unit_sink), bool(channel_gate)
        self.value_mix = value_mix
        self.prefix = prefix
        self.unit_norm_eps = None if unit_norm_eps is None else float(unit_norm_eps)
        self.chunk = int(chunk) if chunk else None
        self.logistic, self.head_gate, self.own_kv = bool(logistic), bool(head_gate), bool(own_kv)
        if self.unit_norm_eps is not None and self.head_norm_eps is not None:
            raise ValueError("attention: a norm per head before the rotation or one after it, not both")
        if self.head_gate and self.channel_gate:
            raise ValueError("attention: a gate per head or one per channel, not both")
        if self.logistic and self.unit_sink:
            raise ValueError("attention: logistic weights have no denominator for one more to count in")
        if not self.own_kv and self.value_mix is not None:
            raise ValueError("attention: a mixer that reads another's values has none to mix")
        self.ng = self.nq * self.dv if self.channel_gate else (self.nq if self.head_gate else 0)
        self.closes_stream = not self.bias        # without a bias its last write to the stream is `Linear.add_into`
        self.proj = self.o = self.o_bias = None
        self.head_terms = self.terms = None

    # ---- what it keeps -------------------------------------------------------
    def kv_reach(self):
        """How far back this mixer looks at keys, whoever keeps them (None: to the first): the window, or
        the chunk, whose keys all lie within as many positions; kept first positions must outlive the
        window, then every position is kept."""
        if self.window and self.keep_first:
            return None
        both = [v for v in (self.window, self.chunk) if v]
        return min(both) if both else None

    def kv_request(self):
        if not self.own_kv:
            return None
        return KVRequest(self.nkv, self.dk, self.kv_reach(), None if self.dv == self.dk else self.dv)

    def may_capture(self, n_rows: int) -> bool:
        return self.proj is not None and self.proj.own_kernels(n_rows) and self.o.own_kernels(n_rows)

    # ---- weights -------------------------------------------------------------
    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, nm = self.prefix, self.names
        Q, K, V = self.nq * self.dk, self.nkv * self.dk, self.nkv * self.dv
        out = {p + nm["q"]: WeightSpec((Q, self.H))}
        if self.own_kv:
            out.update({p + nm["k"]: WeightSpec((K, self.H)), p + nm["v"]: WeightSpec((V, self.H))})
        if self.bias:
            out[p + nm["q_bias"]] = WeightSpec((Q,))
            if self.own_kv:
                out.update({p + nm["k_bias"]: WeightSpec((K,)), p + nm["v_bias"]: WeightSpec((V,))})
        if self.logistic:
            out[p + nm["score_bias"]] = WeightSpec((self.nq,))
        if self.head_norm_eps is not None:
            out[p + nm["q_norm"]] = WeightSpec((self.dk,), init="ones")
            out[p + nm["k_norm"]] = WeightSpec((self.dk,), init="ones")
        if self.value_mix is not None:
            out[p + nm["mix"]] = WeightSpec(())       # bound by the first layer too, which does not use it
        if self.ng:
            out[p + nm["gate"]] = WeightSpec((self.ng, self.H))
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

        ws = [t("q")] + ([t("k"), t("v")] if self.own_kv else []) + ([t("gate")] if self.ng else [])
        if len({w.dtype for w in ws}) > 1:
            ws = [w.to(torch.float32) for w in ws]
        self.proj = Linear(torch.cat(ws, dim=0), tiled=True)
        self.o = Linear(t("o"), tiled=True)
        dev = ws[0].device
        bias = None
        if self.bias:
            bias = torch.cat([f32("q_bias")] + ([f32("k_bias"), f32("v_bias")] if self.own_kv else []) +
                             [torch.zeros(self.ng, dtype=torch.float32, device=dev)]).contiguous()
            self.o_bias = f32("o_bias")
        normed = self.head_norm_eps is not None
        lam = float(t("mix").to(torch.float32).item()) if self.value_mix == "later" else 0.0
        self.head_terms = ops.HeadTerms(bias=bias, q_norm=f32("q_norm") if normed else None,
                                        k_norm=f32("k_norm") if normed else None,
                                        eps=self.head_norm_eps or self.unit_norm_eps or 0.0,
                                        mix=VALUE_MIX.index(self.value_mix), lam=lam,
                                        unit_norm=self.unit_norm_eps is not None)
        sinks = torch.zeros(self.nq, dtype=torch.float32, device=dev) if self.unit_sink else None
        self.terms = ops.ScoreTerms(self.scale, self.window, None, sinks, keep_first=self.keep_first, chunk=self.chunk,
                                    logistic=self.logistic, score_bias=f32("score_bias") if self.logistic else None)

    # ---- one step --------------------------------------------------------------
    def produce(self, ctx, run, y: torch.Tensor, out: Optional[torch.Tensor], x: Optional[torch.Tensor] = None):
        """The mixer's result stored in `out` (float32 [n, H]), or with `out` None added to the
        stream `x`; returns the bias of the output projection, which the caller adds (None
        without biases)."""
        n, nq, nkv, dk, dv, ng = y.shape[0], self.nq, self.nkv, self.dk, self.dv, self.ng
        ws = ctx.workspace
        group = run.kv_group
        own = nkv if self.own_kv else 0
        proj = ws.get("hattn_proj", (n, nq * dk + own * (dk + dv) + ng), torch.float32)
        self.proj(y, proj)
        rotation = self.position.rotation(y.device) or ops.NO_ROTATION
        q = ws.get("hattn_q", (n, nq, dk), ctx.dtype)
        gate = ws.get("hattn_gate", (n, ng), torch.float32) if ng else None
        att = ws.get("hattn_out", (n, nq, dv), ctx.dtype)
        v_first = ws.get("hattn_v_first", (n, nkv * dv), torch.float32) if self.value_mix else None
        tag = f"_{run.index}" if run.kv_read_later else ""      # rows that a later run reads are nobody else's
        k = v = None
        if not self.own_kv:     # the keys and values are another run's: a row of [q | g]
            ops.head_prepare(proj, ctx.row_pos, rotation, self.head_terms, nq, 0, dk, dv, ng, q, None, None, gate)
        elif ctx.all_single:    # one token a sequence: k and v go straight into the pages
            ops.head_prepare(proj, ctx.row_pos, rotation, self.head_terms, nq, nkv, dk, dv, ng, q, None, None, gate,
                             v_first=v_first, table=ctx.tables[run.kv_group_index], ring_pages=group.ring_pages,
                             pages=group.storage[run.kv_layer])
        else:
            k = ws.get("hattn_k" + tag, (n, nkv, dk), ctx.dtype)
            v = ws.get("hattn_v" + tag, (n, nkv, dv), ctx.dtype)
            ops.head_prepare(proj, ctx.row_pos, rotation, self.head_terms, nq, nkv, dk, dv, ng, q, k, v, gate,
                             v_first=v_first)
        attend_and_commit(ctx, run, q, k, v, nkv, dk, dv, self.terms, gate if self.head_gate else None, att, tag=tag,
                          own=self.own_kv)
        if self.channel_gate:
            ops.mul_gate(att, gate)
        if out is None:
            self.o.add_into(att.view(n, nq * dv), x, ctx, "hattn_o_parts")
        else:
            self.o(att.view(n, nq * dv), out)
        return self.o_bias

    def forward(self, ctx, run, y: torch.Tensor, x: torch.Tensor) -> None:
        if not self.bias:
            self.produce(ctx, run, y, None, x)
            return
        flush_pending(ctx, x)
        z = ctx.workspace.get("hattn_z", tuple(x.shape), torch.float32)
        z += self.produce(ctx, run, y, z)
        ops.add_partials(x, z.view(1, *z.shape))


register_part("mixer", "headwise_attention", HeadwiseAttentionMixer)
