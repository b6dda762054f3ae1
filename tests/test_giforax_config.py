"""Giforax's configuration and model spec (no GPU): every key read, what is refused, which parts
and which cache a layer asks for.  The builders below are shared with the GPU tests."""
import copy

import pytest

from torchless_rs_amd.config.base import ConfigError, config_from_dict
from torchless_rs_amd.models import model_spec_for


def attn(heads, kv_heads, dim, vdim, scale, rot=None, chunk=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
    if chunk:
        m["mask"] = {"size": chunk}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return "attention", m


def gru(width):
    return "mingru", {"width": width}


def moe(experts, top, ff, limit, shared=None):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared:
        m["shared"] = {"ff": shared[0], "limit": shared[1]}
    return m


def layer(mixer, mlp=None):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def model(vocab, width, eps, scale, layers):
    return {"architecture": "Giforax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
            "layers": layers}


# both mixers, values narrower than keys, chunks of less than a page and of more, a reader of an earlier layer's
# keys with a chunk of its own, half a head rotated, a layer without a feed-forward, limits that differ
MIXED = model(200, 96, 1e-5, 0.7, [
    layer(attn(4, 2, 32, 16, 0.18, rot=(10000.0, 16), chunk=40), moe(8, 2, 32, 1.5, shared=(48, 2.0))),
    layer(gru(80), moe(6, 3, 16, 1.0, shared=(32, 0.75))),
    layer(attn(4, 2, 32, 16, 0.2, rot=(10000.0, 16), chunk=70, kv_from=0), moe(8, 1, 24, 2.5)),
    layer(gru(48)),
    layer(attn(6, 3, 16, 24, 0.25, rot=(300.0, 8), chunk=100), moe(4, 2, 32, 1.25, shared=(16, 1.25))),
])


def test_every_key_is_read_and_written_back():
    cfg = config_from_dict(copy.deepcopy(MIXED))
    assert cfg.architecture == "Giforax" and cfg.vocab_size == 200 and cfg.hidden_size == 96
    assert cfg.norm_eps == 1e-5 and cfg.embedding_scale == 0.7
    a0, a2, a4 = cfg.layers[0].mixer, cfg.layers[2].mixer, cfg.layers[4].mixer
    assert (a0.heads, a0.kv_heads, a0.dim, a0.vdim, a0.scale, a0.rot_base, a0.rot_dims, a0.chunk, a0.kv_from) == \
        (4, 2, 32, 16, 0.18, 10000.0, 16, 40, None)
    assert a2.kv_from == 0 and a2.chunk == 70 and a4.chunk == 100 and a4.vdim == 24
    assert cfg.layers[1].mixer.width == 80 and cfg.layers[3].mlp is None
    f = cfg.layers[1].mlp
    assert (f.experts, f.top, f.ff, f.limit, f.shared_ff, f.shared_limit) == (6, 3, 16, 1.0, 32, 0.75)
    assert cfg.layers[2].mlp.shared_ff is None
    again = config_from_dict(cfg.to_dict())
    assert again.to_dict() == cfg.to_dict()


def test_defaults():
    d = model(10, 8, 1e-6, 1.0, [layer(("attention", {"heads": 2, "dim": 4, "scale": 0.5}), None)])
    del d["embedding"]
    cfg = config_from_dict(d)
    m = cfg.layers[0].mixer
    assert (m.kv_heads, m.vdim, m.rot_dims, m.chunk, m.kv_from) == (2, 4, None, None, None) and cfg.embedding_scale == 1.0


@pytest.mark.parametrize("change, text", [
    (lambda d: d["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda d: d["layers"][0]["mixer"].update(dim=300), "not served"),
    (lambda d: d["layers"][0]["mixer"]["rot"].update(dims=7), "rotated"),
    (lambda d: d["layers"][0]["mixer"]["mask"].update(size=0), ">= 1"),
    (lambda d: d["layers"][2]["mixer"].update(kv_from=1), "not an earlier attention"),
    (lambda d: d["layers"][2]["mixer"].update(kv_from=2), "not an earlier attention"),
    (lambda d: d["layers"][4]["mixer"].update(kv_from=2), "not an earlier attention"),
    (lambda d: d["layers"][4]["mixer"].update(kv_from=0), "reads keys and values"),
    (lambda d: d["layers"][1].update(type="lstm"), "no mixer"),
    (lambda d: d["layers"][1]["mixer"].update(width=0), ">= 1"),
    (lambda d: d["layers"][1]["mlp"]["router"].update(top=7), "experts"),
    (lambda d: d["layers"][1]["mlp"]["expert"].pop("limit"), "limit"),
    (lambda d: d["layers"][1]["mlp"].update(kind="dense"), "no feed-forward"),
    (lambda d: d.pop("norm"), "norm"),
    (lambda d: d.update(layers=[]), "layers"),
])
def test_what_is_refused(change, text):
    d = copy.deepcopy(MIXED)
    change(d)
    with pytest.raises(ConfigError) as e:
        config_from_dict(d)
    assert text in str(e.value), str(e.value)


def test_the_spec_names_every_tensor_and_part():
    import plain_giforax as plain
    cfg = config_from_dict(copy.deepcopy(MIXED))
    spec = model_spec_for(cfg)
    want = plain.tensor_shapes(MIXED)
    got = {k: tuple(v.shape) for k, v in spec.weight_specs().items()}
    assert got == {k: tuple(v) for k, v in want.items()}
    assert [l.mixer.kind for l in spec.layers] == ["headwise_attention", "gated_recurrence", "headwise_attention",
                                                   "gated_recurrence", "headwise_attention"]
    assert all(l.block.kind == "sandwich_norm" for l in spec.layers) and spec.layers[3].ffn is None
    assert [r.kv_from for r in spec.schedule] == [None, None, 0, None, None]
    assert [r.entry for r in spec.schedule] == [(0, i) for i in range(5)] and spec.exit == (0, 5)
    p = spec.layers[2].mixer.params
    assert p["own_kv"] is False and p["chunk"] == 70 and p["logistic"] and p["head_gate"] and p["unit_norm_eps"] == 1e-5
    f = spec.layers[1].ffn.params
    assert f["score"] == "sigmoid" and f["gated"] and f["weight_on"] == "input" and f["shared_limit"] == 0.75
    assert f["activation_constants"] == {"limit": 1.0, "alpha": 1.702, "shift": 1.0}


def test_the_cache_that_the_layers_ask_for():
    """An owner of keys keeps what its farthest reader looks back to; the recurrence asks for one float a channel."""
    import torch
    from torchless_rs_amd.engine.model import Model
    cfg = config_from_dict(copy.deepcopy(MIXED))
    m = Model(model_spec_for(cfg), cfg, torch.float32, "cpu")
    kv, st = m.cache_requests()
    assert sorted(kv) == [0, 4] and sorted(st) == [1, 3]
    assert (kv[0].n_kv_heads, kv[0].head_dim, kv[0].value_dim, kv[0].window) == (2, 32, 16, 70)      # its reader's chunk
    assert kv[4].window == 100 and kv[4].value_dim == 24
    assert st[1].shape == (80,) and st[3].shape == (48,) and st[1].dtype == torch.float32
    d = copy.deepcopy(MIXED)
    del d["layers"][2]["mixer"]["mask"]                 # a reader that looks back to the first position
    cfg = config_from_dict(d)
    kv, _ = Model(model_spec_for(cfg), cfg, torch.float32, "cpu").cache_requests()
    assert kv[0].window is None
