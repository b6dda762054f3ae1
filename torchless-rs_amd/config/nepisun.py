"""`NepisunConfig`: the config.json of a Nepisun model, typed.

The file names its design in `architecture`, the sizes `vocab` and `width`, `norm.eps` and
`layers`, a list with one entry per layer.  A layer's entry has `type` (which mixer), `mixer`
(its sizes and constants) and `mlp` (the feed-forward, or null for a layer without one); every
entry is read on its own, so layers may differ in every size.

Mixers `attention` and `attention_2`: `heads`, `kv_heads` (default: heads), `dim` (query and key
size per head), `vdim` (value size, default: dim), `scale` (the factor on q.k), `rot` = {`base`,
`dims`} (the rotated channels of a head; absent: no rotation), `v_mix` (true: the layer's values
are mixed with those of the first layer that says so).  `attention` norms q and k per head, counts
one more in the softmax's denominator and gates its output; it sees every earlier position.
`attention_2` has biases and `mask` = {`size`, `keep_first`}: a sliding window beside which the
first `keep_first` positions stay visible (absent: every earlier position is seen).
Mixer `mamba2`: `heads`, `vdim` (channels of a head), `state` (rows of a head's state),
`groups` (sets of B and C that the heads share), `conv` (taps of the short convolution),
`norm_groups` (parts in which the gated output is normed).
Feed-forward `dense`: `ff`.  Feed-forward `moe`: `router` = {`experts`, `top`, `groups` =
{`count`, `keep`} (absent: any expert may be chosen)}, `expert.ff`, `shared.ff` (absent: no
shared expert).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Union

from .base import ConfigError, ModelConfig, take_bool, take_float, take_int, take_obj

MAX_HEAD_DIM = 256          # the largest head the attention kernels take
MAX_STATE = 256             # the most rows of a head's state that the recurrence kernels take
MAX_TAPS = 8                # the longest short convolution
MAX_EXPERTS = 1024
NAME = "Nepisun"


def _sized(m, key, where, **kw):
    try:
        return take_int(m, key, **kw)
    except ConfigError as e:
        raise ConfigError(f"{e} (in {where})") from None


@dataclass
class NepisunAttention:
    """Both attention mixers; `kind` says which of the two sets of terms the layer has."""
    kind: str                         # "attention" | "attention_2"
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: Optional[float] = None
    rot_dims: Optional[int] = None
    v_mix: bool = False
    window: Optional[int] = None      # attention_2 only
    keep_first: int = 0               # attention_2 only

    @classmethod
    def from_dict(cls, kind: str, m: Dict[str, Any], where: str) -> "NepisunAttention":
        heads = _sized(m, "heads", where, required=True, minimum=1)
        kv_heads = _sized(m, "kv_heads", where, default=heads, minimum=1)
        dim = _sized(m, "dim", where, required=True, minimum=1)
        vdim = _sized(m, "vdim", where, default=dim, minimum=1)
        if heads % kv_heads:
            raise ConfigError(f"config.json: {where}: {heads} heads are not a multiple of {kv_heads} kv_heads")
        if max(dim, vdim) > MAX_HEAD_DIM:
            raise ConfigError(f"config.json: {where}: head sizes {dim}/{vdim} are not served (up to {MAX_HEAD_DIM})")
        rot = take_obj(m, "rot", where)
        base = dims = None
        if rot is not None:
            base = take_float(rot, "base", required=True, positive=True)
            dims = take_int(rot, "dims", required=True, minimum=0)
            if dims % 2 or dims > dim:
                raise ConfigError(f"config.json: {where}: {dims} rotated channels of a head of {dim} (even, at most the head)")
            if dims == 0:
                base = dims = None
        window, keep = None, 0
        mask = take_obj(m, "mask", where)
        if mask is not None:
            if kind != "attention_2":
                raise ConfigError(f"config.json: {where}: a mixer of type {kind!r} has no mask")
            window = take_int(mask, "size", required=True, minimum=1)
            keep = take_int(mask, "keep_first", default=0, minimum=0)
        return cls(kind=kind, heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim,
                   scale=take_float(m, "scale", required=True), rot_base=base, rot_dims=dims,
                   v_mix=take_bool(m, "v_mix", False), window=window, keep_first=keep)

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                             "scale": self.scale}
        if self.rot_dims is not None:
            d["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.v_mix:
            d["v_mix"] = True
        if self.window is not None:
            d["mask"] = {"size": self.window, "keep_first": self.keep_first}
        return d


@dataclass
class NepisunStateSpace:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int
    kind: str = "mamba2"

    @classmethod
    def from_dict(cls, kind: str, m: Dict[str, Any], where: str) -> "NepisunStateSpace":
        heads = _sized(m, "heads", where, required=True, minimum=1)
        vdim = _sized(m, "vdim", where, required=True, minimum=1)
        state = _sized(m, "state", where, required=True, minimum=1)
        groups = _sized(m, "groups", where, default=1, minimum=1)
        conv = _sized(m, "conv", where, required=True, minimum=1)
        parts = _sized(m, "norm_groups", where, default=1, minimum=1)
        if heads % groups:
            raise ConfigError(f"config.json: {where}: {heads} heads are not a multiple of {groups} groups")
        if (heads * vdim) % parts:
            raise ConfigError(f"config.json: {where}: {heads * vdim} channels do not split into {parts} normed parts")
        if state > MAX_STATE or vdim > MAX_HEAD_DIM or conv > MAX_TAPS:
            raise ConfigError(f"config.json: {where}: state {state} / head {vdim} / {conv} taps are not served "
                              f"(up to {MAX_STATE}, {MAX_HEAD_DIM}, {MAX_TAPS})")
        return cls(heads=heads, vdim=vdim, state=state, groups=groups, conv=conv, norm_groups=parts)

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups, "conv": self.conv,
                "norm_groups": self.norm_groups}


@dataclass
class NepisunFeedForward:
    kind: str                         # "dense" | "moe"
    ff: int = 0                       # dense: the hidden size; moe: an expert's
    experts: int = 0
    top: int = 0
    group_count: Optional[int] = None
    group_keep: Optional[int] = None
    shared_ff: Optional[int] = None

    @classmethod
    def from_dict(cls, m: Dict[str, Any], where: str) -> "NepisunFeedForward":
        kind = m.get("kind", "dense")
        if kind == "dense":
            return cls(kind=kind, ff=_sized(m, "ff", where, required=True, minimum=1))
        if kind != "moe":
            raise ConfigError(f"config.json: {where}: no feed-forward of kind {kind!r}; there are ('dense', 'moe')")
        router = take_obj(m, "router", where, required=True)
        expert = take_obj(m, "expert", where, required=True)
        shared = take_obj(m, "shared", where)
        experts = _sized(router, "experts", where, required=True, minimum=1)
        top = _sized(router, "top", where, required=True, minimum=1)
        if experts > MAX_EXPERTS or top > experts:
            raise ConfigError(f"config.json: {where}: {top} of {experts} experts (at most {MAX_EXPERTS}, top within them)")
        groups = take_obj(router, "groups", where)
        count = keep = None
        if groups is not None:
            count = take_int(groups, "count", required=True, minimum=1)
            keep = take_int(groups, "keep", required=True, minimum=1)
            if experts % count or keep > count or keep * (experts // count) < top:
                raise ConfigError(f"config.json: {where}: {experts} experts in {count} groups of which {keep} are kept "
                                  f"cannot give {top} experts")
        return cls(kind=kind, ff=_sized(expert, "ff", where, required=True, minimum=1), experts=experts, top=top,
                   group_count=count, group_keep=keep,
                   shared_ff=None if shared is None else _sized(shared, "ff", where, required=True, minimum=1))

    def to_dict(self) -> Dict[str, Any]:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        router: Dict[str, Any] = {"experts": self.experts, "top": self.top}
        if self.group_count is not None:
            router["groups"] = {"count": self.group_count, "keep": self.group_keep}
        d: Dict[str, Any] = {"kind": "moe", "router": router, "expert": {"ff": self.ff}}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff}
        return d


@dataclass
class NepisunLayer:
    type: str
    mixer: Union[NepisunAttention, NepisunStateSpace]
    mlp: Optional[NepisunFeedForward] = None

    def to_dict(self) -> Dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


MIXERS = {"attention": NepisunAttention, "attention_2": NepisunAttention, "mamba2": NepisunStateSpace}


@dataclass
class NepisunConfig(ModelConfig):
    vocab_size: int = 0
    hidden_size: int = 0
    norm_eps: float = 1e-6
    layers: List[NepisunLayer] = field(default_factory=list)
    eos_token_ids: List[int] = field(default_factory=list)
    max_position_embeddings: Optional[int] = None

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "NepisunConfig":
        norm = take_obj(d, "norm", "the model", required=True)
        entries = d.get("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers: List[NepisunLayer] = []
        mixed_shape = None
        for i, e in enumerate(entries):
            where = f"layer {i}"
            if not isinstance(e, dict):
                raise ConfigError(f"config.json: {where} must be an object")
            kind = e.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"config.json: {where}: no mixer of type {kind!r}; there are {sorted(MIXERS)}")
            mixer = MIXERS[kind].from_dict(kind, take_obj(e, "mixer", where, required=True), where)
            if isinstance(mixer, NepisunAttention) and mixer.v_mix:
                shape = (mixer.kv_heads, mixer.vdim)
                if mixed_shape is not None and shape != mixed_shape:
                    raise ConfigError(f"config.json: {where}: values of {shape[0]} x {shape[1]} cannot be mixed with "
                                      f"the first mixing layer's {mixed_shape[0]} x {mixed_shape[1]}")
                mixed_shape = shape
            mlp = take_obj(e, "mlp", where)
            layers.append(NepisunLayer(type=kind, mixer=mixer,
                                       mlp=None if mlp is None else NepisunFeedForward.from_dict(mlp, where)))
        known = {"architecture", "architectures", "vocab", "width", "norm", "layers", "eos_token_id",
                 "max_position_embeddings", "torch_dtype"}
        eos = d.get("eos_token_id")
        eos_ids = [eos] if isinstance(eos, int) and not isinstance(eos, bool) else list(eos or [])
        return cls(architecture=NAME, extra={k: v for k, v in d.items() if k not in known},
                   vocab_size=take_int(d, "vocab", required=True, minimum=1),
                   hidden_size=take_int(d, "width", required=True, minimum=1),
                   norm_eps=take_float(norm, "eps", required=True, positive=True), layers=layers,
                   eos_token_ids=eos_ids,
                   max_position_embeddings=take_int(d, "max_position_embeddings", default=None, allow_none=True,
                                                    minimum=1))

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"architecture": NAME, "vocab": self.vocab_size, "width": self.hidden_size,
                             "norm": {"eps": self.norm_eps}, "layers": [l.to_dict() for l in self.layers]}
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        if self.max_position_embeddings is not None:
            d["max_position_embeddings"] = self.max_position_embeddings
        d.update(self.extra)
        return d
