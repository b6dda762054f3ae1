"""Nepisun's configuration and model spec (no GPU): every key read, what is refused, which parts
and which cache a layer asks for.  The builders below are shared with the GPU tests."""
import copy

import pytest

from torchless_rs_amd.config.base import ConfigError, config_from_dict
from torchless_rs_amd.models import model_spec_for


def attn(heads, kv_heads, dim, vdim, scale, rot=None, v_mix=False):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
    if v_mix:
        m["v_mix"] = True
    return "attention", m


def attn2(heads, kv_heads, dim, vdim, scale, rot=None, v_mix=False, window=None, keep_first=None):
    kind, m = attn(heads, kv_heads, dim, vdim, scale, rot, v_mix)
    if window:
        m["mask"] = {"size": window}
        if keep_first is not None:
            m["mask"]["keep_first"] = keep_first
    return "attention_2", m


def ssm(heads, vdim, state, groups, conv, norm_groups):
    return "mamba2", {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                      "norm_groups": norm_groups}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, groups=None, shared=None):
    router = {"experts": experts, "top": top}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    m = {"kind": "moe", "router": router, "expert": {"ff": ff}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def layer(mixer, mlp=None):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


# every kind of layer, values narrower than keys, a window of less than a page with kept first tokens and one of
# more than a page, half a head rotated, a layer without a feed-forward
MIXED = {"architecture": "Nepisun", "vocab": 200, "width": 96, "norm": {"eps": 1e-5}, "layers": [
    layer(ssm(4, 16, 24, 2, 4, 2), dense(128)),
    layer(attn2(4, 2, 32, 16, 0.18, rot=(10000.0, 16), v_mix=True, window=40, keep_first=6), moe(8, 2, 32, groups=(4, 2), shared=48)),
    layer(attn(4, 2, 32, 16, 0.2, rot=(5000.0, 32), v_mix=True), moe(8, 3, 16, groups=(2, 1), shared=32)),
    layer(ssm(6, 8, 16, 3, 3, 1)),
    layer(attn2(4, 2, 32, 16, 0.15, rot=(300.0, 8), v_mix=True, window=70, keep_first=3), dense(64)),
]}


def test_every_key_is_read_and_written_back():
    cfg = config_from_dict(copy.deepcopy(MIXED))
    assert cfg.vocab_size == 200 and cfg.hidden_size == 96 and cfg.norm_eps == 1e-5 and len(cfg.layers) == 5
    a = cfg.layers[1].mixer
    assert (a.kind, a.heads, a.kv_heads, a.dim, a.vdim, a.scale) == ("attention_2", 4, 2, 32, 16, 0.18)
    assert (a.rot_base, a.rot_dims, a.v_mix, a.window, a.keep_first) == (10000.0, 16, True, 40, 6)
    s = cfg.layers[3].mixer
    assert (s.heads, s.vdim, s.state, s.groups, s.conv, s.norm_groups) == (6, 8, 16, 3, 3, 1)
    f = cfg.layers[2].mlp
    assert (f.kind, f.experts, f.top, f.ff, f.group_count, f.group_keep, f.shared_ff) == ("moe", 8, 3, 16, 2, 1, 32)
    assert cfg.layers[3].mlp is None and cfg.layers[0].mlp.ff == 128
    again = config_from_dict(cfg.to_dict())
    assert again.to_dict() == cfg.to_dict()


def test_defaults_and_what_may_be_left_out():
    d = {"architecture": "Nepisun", "vocab": 10, "width": 8, "norm": {"eps": 1e-6}, "layers": [
        {"type": "attention_2", "mixer": {"heads": 2, "dim": 4, "scale": 0.5}, "mlp": None},
        {"type": "attention_2", "mixer": {"heads": 2, "dim": 4, "scale": 0.5, "mask": {"size": 5}}},
        {"type": "mamba2", "mixer": {"heads": 2, "vdim": 4, "state": 4, "conv": 2}, "mlp": moe(4, 1, 8)}]}
    cfg = config_from_dict(d)
    a = cfg.layers[0].mixer
    assert (a.kv_heads, a.vdim, a.rot_dims, a.v_mix, a.window, a.keep_first) == (2, 4, None, False, None, 0)
    assert cfg.layers[1].mixer.window == 5 and cfg.layers[1].mixer.keep_first == 0
    assert (cfg.layers[2].mixer.groups, cfg.layers[2].mixer.norm_groups) == (1, 1)
    f = cfg.layers[2].mlp
    assert f.group_count is None and f.shared_ff is None


@pytest.mark.parametrize("change, text", [
    (lambda d: d["layers"][1]["mixer"].update(kv_heads=3), "multiple"),
    (lambda d: d["layers"][1]["mixer"].update(dim=300), "not served"),
    (lambda d: d["layers"][1]["mixer"]["rot"].update(dims=7), "rotated"),
    (lambda d: d["layers"][2]["mixer"].update(mask={"size": 8}), "no mask"),
    (lambda d: d["layers"][2]["mixer"].update(vdim=8), "cannot be mixed"),
    (lambda d: d["layers"][0]["mixer"].update(groups=3), "multiple"),
    (lambda d: d["layers"][0]["mixer"].update(norm_groups=5), "normed parts"),
    (lambda d: d["layers"][0]["mixer"].update(conv=40), "not served"),
    (lambda d: d["layers"][1]["mlp"]["router"].update(top=9), "experts"),
    (lambda d: d["layers"][1]["mlp"]["router"]["groups"].update(keep=1, count=8), "cannot give"),
    (lambda d: d["layers"][0]["mlp"].update(kind="sparse"), "no feed-forward"),
    (lambda d: d["layers"][0].update(type="conv"), "no mixer"),
    (lambda d: d.pop("norm"), "norm"),
])
def test_what_cannot_be_served_is_refused(change, text):
    d = copy.deepcopy(MIXED)
    change(d)
    with pytest.raises(ConfigError) as e:
        config_from_dict(d)
    assert text in str(e.value)


def test_the_parts_and_caches_a_layer_asks_for():
    import torch
    from torchless_rs_amd.engine.model import Model
    cfg = config_from_dict(copy.deepcopy(MIXED))
    spec = model_spec_for(cfg)
    kinds = [(l.mixer.kind, None if l.ffn is None else l.ffn.kind) for l in spec.layers]
    assert kinds == [("state_space", "gated"), ("headwise_attention", "routed_experts"),
                     ("headwise_attention", "routed_experts"), ("state_space", None), ("headwise_attention", "gated")]
    # the first layer that mixes values leaves them, the later ones take them
    assert [l.mixer.params.get("value_mix") for l in spec.layers] == [None, "first", "later", None, "later"]
    assert spec.head.params["tied"] and "head" not in spec.weight_specs()
    names = spec.weight_specs()
    assert names["l1.mix.vmix"].shape == () and names["l2.mix.q.norm"].shape == (32,)
    assert names["l3.mix.in"].shape == (6 * 8 + (6 * 8 + 2 * 3 * 16) + 6, 96) and "l3.norm2" not in names
    assert names["l1.mlp.e7.down"].shape == (96, 32) and names["l1.mlp.shared.up"].shape == (48, 96)
    model = Model(spec, cfg, torch.float32, "cpu")
    kv, st = model.cache_requests()
    # kept first tokens beside a window: every position is kept, no ring; the recurrent layers keep a block alone
    assert sorted(kv) == [1, 2, 4] and all(r.window is None for r in kv.values())
    assert sorted(st) == [0, 3]
    assert st[0].shape == ((4 - 1) * (64 + 2 * 2 * 24) + 4 * 24 * 16,) and st[0].dtype == torch.float32
    # a window without kept tokens asks for a ring
    d = copy.deepcopy(MIXED)
    d["layers"][1]["mixer"]["mask"] = {"size": 40}
    kv, _ = Model(model_spec_for(config_from_dict(d)), None, torch.float32, "cpu").cache_requests()
    assert kv[1].window == 40 and kv[1].v_head_dim == 16
