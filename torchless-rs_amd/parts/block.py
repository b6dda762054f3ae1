"""The arrangements of a layer.  `PreNormBlock`: x += mixer(norm(x)); x += ffn(norm(x))
(src/model/modules/layer.rs:28-56 of the reference).  `OutputNormBlock`: the
sublayers read the stream itself and their OUTPUT is normed before the sum,
x += norm(mixer(x)); x += norm(ffn(x)), the feed-forward being optional.
`SandwichNormBlock`: a norm on both sides of each sublayer,
x += norm_b(mixer(norm_a(x))); x += norm_d(ffn(norm_c(x))).  The residual stream x
is float32 in all."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..weights.binding import WeightSpec
from ..kernels import ops
from .base import (LayerSpec, Part, expect_norm, flush_pending, make_part, part_done, read_through_norm,
                   register_part, splittable_entry, take_row_factor)


class PreNormBlock(Part):
    """x += mixer(norm(x)); then, if the layer has a feed-forward, x += ffn(norm(x))."""

    def __init__(self, layer: LayerSpec, mixer_norm_name: str = "input_layernorm.",
                 ffn_norm_name: str = "post_attention_layernorm."):
        self.mixer = make_part("mixer", layer.mixer)
        self.ffn = make_part("ffn", layer.ffn) if layer.ffn is not None else None
        self.mixer_norm = make_part("norm", layer.mixer_norm)
        self.ffn_norm = make_part("norm", layer.ffn_norm) if layer.ffn is not None else None
        self.n1, self.n2 = mixer_norm_name, ffn_norm_name
        self.graph_safe = all(p.graph_safe for p in self._parts())

    def _parts(self):
        return [p for p in (self.mixer, self.ffn, self.mixer_norm, self.ffn_norm) if p is not None]

    def weight_specs(self) -> Dict[str, WeightSpec]:
        out: Dict[str, WeightSpec] = {}
        for k, v in self.mixer_norm.weight_specs().items():
            out[self.n1 + k] = v
        out.update(self.mixer.weight_specs())
        if self.ffn is not None:
            for k, v in self.ffn_norm.weight_specs().items():
                out[self.n2 + k] = v
            out.update(self.ffn.weight_specs())
        return out

    def load(self, tensors, compute_dtype) -> None:
        def sub(prefix):
            return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}
        self.mixer_norm.load(sub(self.n1), compute_dtype)
        self.mixer.load(tensors, compute_dtype)
        if self.ffn is not None:
            self.ffn_norm.load(sub(self.n2), compute_dtype)
            self.ffn.load(tensors, compute_dtype)

    def may_capture(self, n_rows: int) -> bool:
        return all(p.may_capture(n_rows) for p in self._parts())

    def prefers_eager(self, n_new, len_before, device) -> bool:
        return any(p.prefers_eager(n_new, len_before, device) for p in self._parts())

    def entry_norm(self):
        """The norm that reads the stream first, if the part behind it can take a norm cut in
        two (the block before this one may then do the norm's first half)."""
        return splittable_entry(self.mixer_norm, self.mixer)

    def forward(self, ctx, run, x: torch.Tensor, norm_after=None) -> None:
        """`norm_after`: the `entry_norm` of the block that runs next, if it has one.  The three
        helpers around each part (`read_through_norm`, `expect_norm`, `part_done`) are all that
        an arrangement needs for norms cut in two around the products."""
        ctx.host.pop("stream_copy", None)        # this block writes the stream: a copy of it goes stale
        y = ctx.workspace.get("block_y", tuple(x.shape), ctx.dtype)
        y1 = read_through_norm(ctx, self.mixer_norm, x, y)
        if self.ffn is None:
            expect_norm(ctx, self.mixer, norm_after)
        else:
            expect_norm(ctx, self.mixer, self.ffn_norm, self.ffn)
        self.mixer.forward(ctx, run, y1, x)
        part_done(ctx, self.mixer)
        if self.ffn is None:
            return
        y2 = read_through_norm(ctx, self.ffn_norm, x, y)
        expect_norm(ctx, self.ffn, norm_after)
        self.ffn.forward(ctx, y2, x)
        part_done(ctx, self.ffn)


class OutputNormBlock(Part):
    """x += norm1(mixer(x)); then, if the layer has a feed-forward, x += norm2(ffn(x)).

    A sublayer reads x itself: as it is in float32, rounded to the compute dtype otherwise.  That
    copy is made by the norm before it (`Norm.add_to` leaves the new stream in the compute dtype
    while it adds), by a kernel of its own only at the first block.  Parts that offer `produce`
    store their result for the norm; any other part adds into a zeroed buffer instead."""

    def __init__(self, layer: LayerSpec, mixer_norm_name: str = "norm1.", ffn_norm_name: str = "norm2."):
        self.mixer = make_part("mixer", layer.mixer)
        self.mixer_norm = make_part("norm", layer.mixer_norm)
        self.ffn = make_part("ffn", layer.ffn) if layer.ffn is not None else None
        self.ffn_norm = make_part("norm", layer.ffn_norm) if layer.ffn is not None else None
        self.n1, self.n2 = mixer_norm_name, ffn_norm_name
        self.graph_safe = all(p.graph_safe for p in self._parts())

    def _parts(self):
        return [p for p in (self.mixer, self.mixer_norm, self.ffn, self.ffn_norm) if p is not None]

    def weight_specs(self) -> Dict[str, WeightSpec]:
        out: Dict[str, WeightSpec] = {}
        for k, v in self.mixer_norm.weight_specs().items():
            out[self.n1 + k] = v
        out.update(self.mixer.weight_specs())
        if self.ffn is not None:
            for k, v in self.ffn_norm.weight_specs().items():
                out[self.n2 + k] = v
            out.update(self.ffn.weight_specs())
        return out

    def load(self, tensors, compute_dtype) -> None:
        def sub(prefix):
            return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}
        self.mixer_norm.load(sub(self.n1), compute_dtype)
        self.mixer.load(tensors, compute_dtype)
        if self.ffn is not None:
            self.ffn_norm.load(sub(self.n2), compute_dtype)
            self.ffn.load(tensors, compute_dtype)

    def may_capture(self, n_rows: int) -> bool:
        return all(p.may_capture(n_rows) for p in self._parts())

    def prefers_eager(self, n_new, len_before, device) -> bool:
        return any(p.prefers_eager(n_new, len_before, device) for p in self._parts())

    @staticmethod
    def _result(ctx, part, z, *args) -> Optional[torch.Tensor]:
        """The part's output in z; returns the bias that is still to be added."""
        if hasattr(part, "produce"):
            return part.produce(ctx, *args, z)
        z.zero_()
        ctx.norm_ahead = None
        part.forward(ctx, *args, z)
        flush_pending(ctx, z)
        return None

    def forward(self, ctx, run, x: torch.Tensor, norm_after=None) -> None:
        flush_pending(ctx, x)
        narrow = ctx.dtype != torch.float32
        y = x
        if narrow:
            y = ctx.workspace.get("stream_y", tuple(x.shape), ctx.dtype)
            if ctx.host.pop("stream_copy", None) is not y:       # nobody left the stream there yet
                ops.cast_rows(x, y)
        z = ctx.workspace.get("block_z", tuple(x.shape), torch.float32)
        bias = self._result(ctx, self.mixer, z, run, y)
        self.mixer_norm.add_to(ctx, z, x, out=y if narrow else None, bias=bias)
        if self.ffn is not None:
            bias = self._result(ctx, self.ffn, z, y)
            self.ffn_norm.add_to(ctx, z, x, out=y if narrow else None, bias=bias)
        if narrow:
            ctx.host["stream_copy"] = y


class SandwichNormBlock(Part):
    """x += out_norm1(mixer(norm1(x))); then, if the layer has a feed-forward,
    x += out_norm2(ffn(norm2(x))).  The four norms are the layer's `mixer_norm`, `mixer_out_norm`,
    `ffn_norm` and `ffn_out_norm`, bound under the four names given here.

    A sublayer's result is stored (`produce`, or `forward` into a zeroed buffer) and the norm of
    it is added to the stream by `Norm.add_to`, which is told the norm that reads the stream next
    (the feed-forward's, or the next block's `entry_norm`): a norm that can run both in one kernel
    leaves the second one's result for `read_through_norm`."""

    def __init__(self, layer: LayerSpec, names=("norm1.", "norm1b.", "norm2.", "norm2b.")):
        if layer.mixer_out_norm is None or (layer.ffn is not None and (layer.ffn_norm is None or layer.ffn_out_norm is None)):
            raise ValueError("sandwich block: the layer names no norm for a sublayer's output (or input)")
        self.mixer = make_part("mixer", layer.mixer)
        self.mixer_norm = make_part("norm", layer.mixer_norm)
        self.mixer_out_norm = make_part("norm", layer.mixer_out_norm)
        self.ffn = make_part("ffn", layer.ffn) if layer.ffn is not None else None
        self.ffn_norm = make_part("norm", layer.ffn_norm) if layer.ffn is not None else None
        self.ffn_out_norm = make_part("norm", layer.ffn_out_norm) if layer.ffn is not None else None
        self.names = tuple(names)
        self.graph_safe = all(p.graph_safe for p in self._parts())

    def _norms(self):
        return [(n, p) for n, p in zip(self.names, (self.mixer_norm, self.mixer_out_norm, self.ffn_norm, self.ffn_out_norm))
                if p is not None]

    def _parts(self):
        return [self.mixer] + ([self.ffn] if self.ffn is not None else []) + [p for _, p in self._norms()]

    def weight_specs(self) -> Dict[str, WeightSpec]:
        out: Dict[str, WeightSpec] = {}
        for name, norm in self._norms():
            for k, v in norm.weight_specs().items():
                out[name + k] = v
        out.update(self.mixer.weight_specs())
        if self.ffn is not None:
            out.update(self.ffn.weight_specs())
        return out

    def load(self, tensors, compute_dtype) -> None:
        def sub(prefix):
            return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}
        for name, norm in self._norms():
            norm.load(sub(name), compute_dtype)
        self.mixer.load(tensors, compute_dtype)
        if self.ffn is not None:
            self.ffn.load(tensors, compute_dtype)

    def may_capture(self, n_rows: int) -> bool:
        return all(p.may_capture(n_rows) for p in self._parts())

    def prefers_eager(self, n_new, len_before, device) -> bool:
        return any(p.prefers_eager(n_new, len_before, device) for p in self._parts())

    def entry_norm(self):
        """The norm that reads the stream first: whoever completes the stream before this block
        may run it on the way (`Norm.add_to`'s `then`)."""
        return self.mixer_norm

    fuses_stream_after = True     # takes `stream_after`: see `StreamPart`

    def _last_add(self, ctx, norm, z, x, bias, y, norm_after, stream_after) -> None:
        """The block's last norm into the stream, with what changes the stream behind the block."""
        then = None if norm_after is None else (norm_after, y)
        if stream_after is None:
            norm.add_to(ctx, z, x, bias=bias, then=then)
            return
        part, t = stream_after
        if getattr(norm, "takes_between", False):
            norm.add_to(ctx, z, x, bias=bias, then=then, between=part.mix_terms(ctx, x, t))
        else:
            norm.add_to(ctx, z, x, bias=bias)
            part.forward(ctx, x, None, t)

    def forward(self, ctx, run, x: torch.Tensor, norm_after=None, stream_after=None) -> None:
        """`stream_after` = (stream part, t): that part changes the stream right behind this block; the
        block's last norm does it on its way if it can, and `norm_after` then reads the changed stream."""
        ctx.host.pop("stream_copy", None)        # this block writes the stream: a copy of it goes stale
        ws = ctx.workspace
        y = ws.get("block_y", tuple(x.shape), ctx.dtype)
        z = ws.get("block_z", tuple(x.shape), torch.float32)
        y1 = read_through_norm(ctx, self.mixer_norm, x, y)
        take_row_factor(ctx, usable=False)       # a norm cut in two by an earlier product is completed here
        bias = OutputNormBlock._result(ctx, self.mixer, z, run, y1)
        if self.ffn is None:
            self._last_add(ctx, self.mixer_out_norm, z, x, bias, y, norm_after, stream_after)
            return
        self.mixer_out_norm.add_to(ctx, z, x, bias=bias, then=(self.ffn_norm, y))
        y2 = read_through_norm(ctx, self.ffn_norm, x, y)
        take_row_factor(ctx, usable=False)
        bias = OutputNormBlock._result(ctx, self.ffn, z, y2)
        self._last_add(ctx, self.ffn_out_norm, z, x, bias, y, norm_after, stream_after)


register_part("block", "pre_norm", PreNormBlock)
register_part("block", "sandwich_norm", SandwichNormBlock)
register_part("block", "output_norm", OutputNormBlock)
