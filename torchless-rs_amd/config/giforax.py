"""`GiforaxConfig`: the config.json of a Giforax model, typed.

The file names its design in `architecture`, the sizes `vocab` and `width`, `norm.eps`,
`embedding.scale` (a factor on the embedding's rows) and `layers`, a list with one entry per
layer.  A layer's entry has `type` (which mixer), `mixer` (its sizes and constants) and `mlp` (the
feed-forward, or null for a layer without one); every entry is read on its own, so layers may
differ in every size.

Mixer `attention`: `heads`, `kv_heads` (default: heads), `dim` (query and key size per head),
`vdim` (value size, default: dim), `scale` (the factor on q.k), `rot` = {`base`, `dims`} (the
rotated channels of a head; absent: no rotation), `mask.size` (positions see each other inside
runs of that many, counted from the sequence's start; absent: every earlier position is seen),
`kv_from` (the index of an earlier attention layer whose keys and values this layer reads
instead of making its own).
Mixer `mingru`: `width` (channels of the recurrence).
Feed-forward `moe`: `router` = {`experts`, `top`}, `expert` = {`ff`, `limit`}, `shared` = {`ff`,
`limit`} (absent: no shared expert).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Union

from .base import ConfigError, ModelConfig, take_float, take_int, take_obj

MAX_HEAD_DIM = 256          # the largest head the attention kernels take
MAX_EXPERTS = 1024
NAME = "Giforax"


def _sized(m, key, where, **kw):
    try:
        return take_int(m, key, **kw)
    except ConfigError as e:
        raise ConfigError(f"{e} (in {where})") from None


def _number(m, key, where, **kw):
    try:
        return take_float(m, key, **kw)
    except ConfigError as e:
        raise ConfigError(f"{e} (in {where})") from None


@dataclass
class GiforaxAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: Optional[float] = None
    rot_dims: Optional[int] = None
    chunk: Optional[int] = None
    kv_from: Optional[int] = None
    kind: str = "attention"

    @classmethod
    def from_dict(cls, kind: str, m: Dict[str, Any], where: str) -> "GiforaxAttention":
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
            base = _number(rot, "base", where, required=True, positive=True)
            dims = _sized(rot, "dims", where, required=True, minimum=0)
            if dims % 2 or dims > dim:
                raise ConfigError(f"config.json: {where}: {dims} rotated channels of a head of {dim} (even, at most the head)")
            if dims == 0:
                base = dims = None
        mask = take_obj(m, "mask", where)
        chunk = None if mask is None else _sized(mask, "size", where, required=True, minimum=1)
        return cls(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=_number(m, "scale", where, required=True),
                   rot_base=base, rot_dims=dims, chunk=chunk,
                   kv_from=_sized(m, "kv_from", where, default=None, allow_none=True, minimum=0))

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                             "scale": self.scale}
        if self.rot_dims is not None:
            d["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.chunk is not None:
            d["mask"] = {"size": self.chunk}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


@dataclass
class GiforaxRecurrence:
    width: int
    kind: str = "mingru"

    @classmethod
    def from_dict(cls, kind: str, m: Dict[str, Any], where: str) -> "GiforaxRecurrence":
        return cls(width=_sized(m, "width", where, required=True, minimum=1))

    def to_dict(self) -> Dict[str, Any]:
        return {"width": self.width}


@dataclass
class GiforaxFeedForward:
    experts: int
    top: int
    ff: int
    limit: float
    shared_ff: Optional[int] = None
    shared_limit: Optional[float] = None
    kind: str = "moe"

    @classmethod
    def from_dict(cls, m: Dict[str, Any], where: str) -> "GiforaxFeedForward":
        kind = m.get("kind", "moe")
        if kind != "moe":
            raise ConfigError(f"config.json: {where}: no feed-forward of kind {kind!r}; there is 'moe'")
        router = take_obj(m, "router", where, required=True)
        expert = take_obj(m, "expert", where, required=True)
        shared = take_obj(m, "shared", where)
        experts = _sized(router, "experts", where, required=True, minimum=1)
        top = _sized(router, "top", where, required=True, minimum=1)
        if experts > MAX_EXPERTS or top > experts:
            raise ConfigError(f"config.json: {where}: {top} of {experts} experts (at most {MAX_EXPERTS}, top within them)")
        return cls(experts=experts, top=top, ff=_sized(expert, "ff", where, required=True, minimum=1),
                   limit=_number(expert, "limit", where, required=True, positive=True),
                   shared_ff=None if shared is None else _sized(shared, "ff", where, required=True, minimum=1),
                   shared_limit=None if shared is None else _number(shared, "limit", where, required=True, positive=True))

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"kind": "moe", "router": {"experts": self.experts, "top": self.top},
                             "expert": {"ff": self.ff, "limit": self.limit}}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return d


@dataclass
class GiforaxLayer:
    type: str
    mixer: Union[GiforaxAttention, GiforaxRecurrence]
    mlp: Optional[GiforaxFeedForward] = None

    def to_dict(self) -> Dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


MIXERS = {"attention": GiforaxAttention, "mingru": GiforaxRecurrence}


@dataclass
class GiforaxConfig(ModelConfig):
    vocab_size: int = 0
    hidden_size: int = 0
    norm_eps: float = 1e-5
    embedding_scale: float = 1.0
    layers: List[GiforaxLayer] = field(default_factory=list)
    eos_token_ids: List[int] = field(default_factory=list)
    max_position_embeddings: Optional[int] = None

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "GiforaxConfig":
        norm = take_obj(d, "norm", "the model", required=True)
        emb = take_obj(d, "embedding", "the model")
        entries = d.get("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers: List[GiforaxLayer] = []
        for i, e in enumerate(entries):
            where = f"layer {i}"
            if not isinstance(e, dict):
                raise ConfigError(f"config.json: {where} must be an object")
            kind = e.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"config.json: {where}: no mixer of type {kind!r}; there are {sorted(MIXERS)}")
            mixer = MIXERS[kind].from_dict(kind, take_obj(e, "mixer", where, required=True), where)
            if isinstance(mixer, GiforaxAttention) and mixer.kv_from is not None:
                src = layers[mixer.kv_from].mixer if mixer.kv_from < i else None
                if not isinstance(src, GiforaxAttention) or src.kv_from is not None:
                    raise ConfigError(f"config.json: {where}: kv_from {mixer.kv_from} is not an earlier attention layer "
                                      "with keys and values of its own")
                if (src.kv_heads, src.dim, src.vdim) != (mixer.kv_heads, mixer.dim, mixer.vdim):
                    raise ConfigError(f"config.json: {where}: reads keys and values of {src.kv_heads} x {src.dim}/{src.vdim} "
                                      f"as {mixer.kv_heads} x {mixer.dim}/{mixer.vdim}")
            mlp = take_obj(e, "mlp", where)
            layers.append(GiforaxLayer(type=kind, mixer=mixer,
                                       mlp=None if mlp is None else GiforaxFeedForward.from_dict(mlp, where)))
        known = {"architecture", "architectures", "vocab", "width", "norm", "embedding", "layers", "eos_token_id",
                 "max_position_embeddings", "torch_dtype"}
        eos = d.get("eos_token_id")
        eos_ids = [eos] if isinstance(eos, int) and not isinstance(eos, bool) else list(eos or [])
        return cls(architecture=NAME, extra={k: v for k, v in d.items() if k not in known},
                   vocab_size=take_int(d, "vocab", required=True, minimum=1),
                   hidden_size=take_int(d, "width", required=True, minimum=1),
                   norm_eps=take_float(norm, "eps", required=True, positive=True),
                   embedding_scale=1.0 if emb is None else take_float(emb, "scale", default=1.0),
                   layers=layers, eos_token_ids=eos_ids,
                   max_position_embeddings=take_int(d, "max_position_embeddings", default=None, allow_none=True,
                                                    minimum=1))

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"architecture": NAME, "vocab": self.vocab_size, "width": self.hidden_size,
                             "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
                             "layers": [l.to_dict() for l in self.layers]}
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        if self.max_position_embeddings is not None:
            d["max_position_embeddings"] = self.max_position_embeddings
        d.update(self.extra)
        return d
