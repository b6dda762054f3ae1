"""Nepisun as a list of parts.

A decoder-only model of pre-norm layers, x += mixer(norm(x)); x += ffn(norm(x)) (RMS norms, the
feed-forward optional), whose mixer is, layer by layer as config.json lists them, one of

* `attention`: grouped-query attention with a norm of q and k per head, rotation, one more in the
  softmax's denominator and a gate per channel (`headwise_attention` with those terms);
* `attention_2`: grouped-query attention with biases, rotation and a sliding window beside which
  the first tokens stay visible (`headwise_attention` with these);
* `mamba2`: a state-space layer (`state_space`).

Attention layers that say `v_mix` mix their values with those of the first layer that says so.
The feed-forward is gated with relu (`gated`), or a routed mixture of ungated experts with the
square of relu and a shared expert (`routed_experts`).  The logits come from the embedding table.
Tensor names: `embed`, `l<i>.norm1`, `l<i>.norm2`, `l<i>.mix.*`, `l<i>.mlp.*`, `final.norm`.
Every size comes from the configuration, layer by layer.
"""
from __future__ import annotations

from ..config.base import register_architecture
from ..config.nepisun import NAME, NepisunAttention, NepisunConfig
from ..parts.base import LayerSpec, ModelSpec, PartSpec, Run

DENSE_ACTIVATION = "relu"       # the gate's function of a dense feed-forward
EXPERT_ACTIVATION = "relu2"     # an expert: down(max(up, 0)^2)


def nepisun_spec(cfg: NepisunConfig) -> ModelSpec:
    H = cfg.hidden_size
    norm = PartSpec("rmsnorm", {"size": H, "eps": cfg.norm_eps, "name": ""})     # the tensor is the prefix itself
    layers = []
    mixing_seen = False
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if isinstance(m, NepisunAttention):
            position = (PartSpec("rotary", {"head_dim": m.dim, "theta": m.rot_base, "rotary_dim": m.rot_dims})
                        if m.rot_dims is not None else PartSpec("none"))
            gated = m.kind == "attention"
            value_mix = None
            if m.v_mix:
                value_mix = "later" if mixing_seen else "first"
                mixing_seen = True
            mixer = PartSpec("headwise_attention", {
                "hidden_size": H, "n_heads": m.heads, "n_kv_heads": m.kv_heads, "head_dim": m.dim, "v_head_dim": m.vdim,
                "position": position, "scale": m.scale, "bias": not gated,
                "head_norm_eps": cfg.norm_eps if gated else None, "window": m.window, "keep_first": m.keep_first,
                "unit_sink": gated, "channel_gate": gated, "value_mix": value_mix, "prefix": "mix."})
        else:
            mixer = PartSpec("state_space", {
                "hidden_size": H, "n_heads": m.heads, "head_dim": m.vdim, "state_size": m.state, "groups": m.groups,
                "conv_taps": m.conv, "norm_groups": m.norm_groups, "norm_eps": cfg.norm_eps, "prefix": "mix."})
        ffn = None
        f = layer.mlp
        if f is not None and f.kind == "dense":
            ffn = PartSpec("gated", {"hidden_size": H, "intermediate_size": f.ff, "prefix": "mlp.",
                                     "activation": DENSE_ACTIVATION,
                                     "names": {"gate": "gate", "up": "up", "down": "down"}})
        elif f is not None:
            ffn = PartSpec("routed_experts", {
                "hidden_size": H, "n_experts": f.experts, "top": f.top, "expert_size": f.ff,
                "group_count": f.group_count, "group_keep": f.group_keep, "shared_size": f.shared_ff,
                "activation": EXPERT_ACTIVATION, "prefix": "mlp."})
        layers.append(LayerSpec(prefix=f"l{i}.", mixer=mixer, ffn=ffn, mixer_norm=norm,
                                ffn_norm=norm if ffn is not None else None,
                                block=PartSpec("pre_norm", {"mixer_norm_name": "norm1", "ffn_norm_name": "norm2"})))
    return ModelSpec(
        hidden_size=H, vocab_size=cfg.vocab_size,
        embedding=PartSpec("tokens", {"vocab_size": cfg.vocab_size, "hidden_size": H, "name": "embed"}),
        embedding_prefix="",
        layers=layers, schedule=[Run(i) for i in range(len(layers))],
        final_norm=norm, final_norm_prefix="final.norm",
        head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "tied": True}),
        head_prefix="",
    )


register_architecture(NAME, NepisunConfig, nepisun_spec)
