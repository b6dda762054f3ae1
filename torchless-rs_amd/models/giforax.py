"""Giforax as a list of parts.

A decoder-only model whose layers norm a sublayer on both sides with layer norms that have a
weight and a bias, x += N1b(mixer(N1(x))); x += N2b(ffn(N2(x))) (`sandwich_norm`, the feed-forward
optional), and whose stream between the layers is a weighted sum of the embedding's output and
every layer's result so far (`depth_average`).  The mixer is, layer by layer as config.json lists
them, one of

* `attention`: grouped-query attention with a rotation of part of each head, a norm of q and k per
  head after it (no weight), a mask by chunks of positions, weights that are logistic functions
  of the scores plus a learned number per head instead of a softmax, a gate per head, and
  optionally the keys and values of an earlier layer (`headwise_attention` with those terms);
* `mingru`: a gated recurrence per channel (`gated_recurrence`).

The feed-forward is a routed mixture of gated experts with a clamped activation, scores that are
each expert's own logistic function, the score on the expert's input, and a shared expert
(`routed_experts` with those terms).  Tensor names: `embed`, `l<i>.norm1` .. `l<i>.norm2b` (+ `.b`),
`l<i>.mix.*`, `l<i>.mlp.*`, `l<i>.dwa`, `final.norm` (+ `.b`), `head`.  Every size comes from the
configuration, layer by layer.
"""
from __future__ import annotations

from ..config.base import register_architecture
from ..config.giforax import NAME, GiforaxAttention, GiforaxConfig
from ..parts.base import LayerSpec, ModelSpec, PartSpec, Run

# the constants of an expert's activation that the design fixes: g' logistic(1.702 g') (u' + 1)
EXPERT_ALPHA = 1.702
EXPERT_SHIFT = 1.0


def giforax_spec(cfg: GiforaxConfig) -> ModelSpec:
    H = cfg.hidden_size
    # the weight is the prefix itself, the bias that name + ".b"
    norm = PartSpec("layernorm", {"size": H, "eps": cfg.norm_eps, "name": "", "bias_name": ".b"})
    layers = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if isinstance(m, GiforaxAttention):
            position = (PartSpec("rotary", {"head_dim": m.dim, "theta": m.rot_base, "rotary_dim": m.rot_dims})
                        if m.rot_dims is not None else PartSpec("none"))
            mixer = PartSpec("headwise_attention", {
                "hidden_size": H, "n_heads": m.heads, "n_kv_heads": m.kv_heads, "head_dim": m.dim, "v_head_dim": m.vdim,
                "position": position, "scale": m.scale, "unit_norm_eps": cfg.norm_eps, "chunk": m.chunk,
                "logistic": True, "head_gate": True, "own_kv": m.kv_from is None, "prefix": "mix."})
        else:
            mixer = PartSpec("gated_recurrence", {"hidden_size": H, "width": m.width, "prefix": "mix."})
        ffn = None
        f = layer.mlp
        if f is not None:
            ffn = PartSpec("routed_experts", {
                "hidden_size": H, "n_experts": f.experts, "top": f.top, "expert_size": f.ff, "shared_size": f.shared_ff,
                "score": "sigmoid", "gated": True, "activation": "swish_clamped",
                "activation_constants": {"limit": f.limit, "alpha": EXPERT_ALPHA, "shift": EXPERT_SHIFT},
                "shared_limit": f.shared_limit, "weight_on": "input", "prefix": "mlp."})
        layers.append(LayerSpec(prefix=f"l{i}.", mixer=mixer, ffn=ffn, mixer_norm=norm,
                                ffn_norm=norm if ffn is not None else None, mixer_out_norm=norm,
                                ffn_out_norm=norm if ffn is not None else None,
                                block=PartSpec("sandwich_norm", {"names": ("norm1", "norm1b", "norm2", "norm2b")})))
    n = len(layers)
    # call t of the averaging part: t = 0 keeps the embedding's output, t = i + 1 follows layer i
    schedule = [Run(i, kv_from=cfg.layers[i].mixer.kv_from if isinstance(cfg.layers[i].mixer, GiforaxAttention) else None,
                    entry=(0, i)) for i in range(n)]
    return ModelSpec(
        hidden_size=H, vocab_size=cfg.vocab_size,
        embedding=PartSpec("tokens", {"vocab_size": cfg.vocab_size, "hidden_size": H, "name": "embed",
                                      "scale": cfg.embedding_scale}),
        embedding_prefix="",
        layers=layers, schedule=schedule,
        stream_parts=[("", PartSpec("depth_average", {"hidden_size": H, "names": [f"l{i}.dwa" for i in range(n)]}))],
        exit=(0, n),
        final_norm=norm, final_norm_prefix="final.norm",
        head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "name": "head"}),
        head_prefix="",
    )


register_architecture(NAME, GiforaxConfig, giforax_spec)
