"""A plain, slow implementation of Giforax in float64, one function per mechanism, written from
the design's equations.  It shares no code with the package: the tests compare the engine
against it.

Notation.  x: the residual stream [T, W].  ln(t, w, b) = (t - mean) / sqrt(var + eps) * w + b over
the last axis.  A layer is x <- x + ln1b(mixer(ln1(x))); x <- x + ln2b(ff(ln2(x))) (the second only
with a feed-forward); then the stream that goes on is a weighted sum of the embedding's output
and every layer's result so far.  Mixers: grouped-query attention whose weights are logistic
functions of the scores, each key by itself, inside chunks of positions, and a gated recurrence per
channel.  Feed-forward: a routed mixture of small gated experts, the router's weight on an
expert's input, with a shared expert.
"""
import math

import torch

F64 = torch.float64


def layer_norm(t, eps, w, b):
    mu = t.mean(dim=-1, keepdim=True)
    d = t - mu
    return d / torch.sqrt((d * d).mean(dim=-1, keepdim=True) + eps) * w + b


def unit_rms(t, eps):
    return t / torch.sqrt((t * t).mean(dim=-1, keepdim=True) + eps)


def rotate_halves(t, pos, base, dims):
    """t [T, heads, d]; the first `dims` channels of every head are rotated: channel i pairs with
    i + dims/2, angle pos * base^(-2i/dims)."""
    if not dims:
        return t
    half = dims // 2
    f = torch.pow(torch.tensor(float(base), dtype=F64), -2.0 * torch.arange(half, dtype=F64) / dims)
    a = pos.to(F64)[:, None] * f[None, :]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = t[..., :half], t[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, t[..., dims:]], dim=-1)


def same_chunk(pos, size):
    """[T, T] bool: row p sees column j iff j <= p and both lie in the same run of `size` positions
    counted from position 0 (`size` None: j <= p alone)."""
    p, j = pos[:, None], pos[None, :]
    ok = j <= p
    if size:
        ok = ok & (torch.div(p, size, rounding_mode="floor") == torch.div(j, size, rounding_mode="floor"))
    return ok


def keys_and_values(h, w, p, m, pos, eps):
    """What an attention layer that owns keys caches: k after rotation and norm, v as projected."""
    T = h.shape[0]
    k = (h @ w[p + "k"].T).view(T, m["kv_heads"], m["dim"])
    v = (h @ w[p + "v"].T).view(T, m["kv_heads"], m["vdim"])
    rot = m.get("rot") or {}
    k = unit_rms(rotate_halves(k, pos, rot.get("base", 10000.0), rot.get("dims", 0)), eps)
    return k, v


def logistic_attention(h, w, p, m, pos, eps, k, v):
    """h [T, W] -> [T, W]; k [T, G, d], v [T, G, dv] are this layer's or the layer's it reads."""
    T, H, G = h.shape[0], m["heads"], m["kv_heads"]
    rot = m.get("rot") or {}
    q = (h @ w[p + "q"].T).view(T, H, m["dim"])
    q = unit_rms(rotate_halves(q, pos, rot.get("base", 10000.0), rot.get("dims", 0)), eps)
    rep = H // G
    kh = k.repeat_interleave(rep, dim=1).transpose(0, 1)          # [H, T, d]
    vh = v.repeat_interleave(rep, dim=1).transpose(0, 1)
    s = (q.transpose(0, 1) @ kh.transpose(1, 2)) * m["scale"] + w[p + "pb"][:, None, None]
    a = torch.sigmoid(s) * same_chunk(pos, (m.get("mask") or {}).get("size"))[None]
    o = (a @ vh).transpose(0, 1)                                  # [T, H, dv]
    o = o * torch.sigmoid(h @ w[p + "g"].T)[:, :, None]
    return o.reshape(T, -1) @ w[p + "o"].T


def candidate(u):
    return torch.where(u >= 0, u + 0.5, torch.sigmoid(u))


def gated_recurrence(h, w, p, S=None):
    """S_t = (1 - z_t) S_(t-1) + z_t c_t per channel, from S = 0; returns the output and the last state."""
    z = torch.sigmoid(h @ w[p + "z"].T + w[p + "z.b"])
    c = candidate(h @ w[p + "x"].T + w[p + "x.b"])
    S = torch.zeros(z.shape[1], dtype=h.dtype) if S is None else S
    out = []
    for t in range(h.shape[0]):
        S = (1 - z[t]) * S + z[t] * c[t]
        out.append(S)
    g = h @ w[p + "g"].T
    return (torch.stack(out) * (g * torch.sigmoid(g))) @ w[p + "o"].T, S


def gated_expert(h, w, p, limit):
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w[p + "down"].T


def route(h, w, p, r, margins=None):
    """Scores s = logistic(W_r h); the `top` largest are chosen (of equal ones the smaller index).
    Returns [T, E] weights: s where chosen, 0 elsewhere.  `margins`: a list that receives, per row,
    the gap between the last chosen and the first not chosen expert's product W_r h, as a share of
    the root mean square of the row's products (infinite where every expert is chosen)."""
    z = h @ w[p + "router"].T
    s = torch.sigmoid(z)
    order = torch.sort(s, dim=-1, descending=True, stable=True)
    top = r["top"]
    out = torch.zeros_like(s)
    out.scatter_(1, order.indices[:, :top], order.values[:, :top])
    if margins is not None:
        if top < s.shape[1]:
            zs = torch.gather(z, 1, order.indices)
            gap = (zs[:, top - 1] - zs[:, top]) / torch.sqrt((z * z).mean(dim=-1) + 1e-30)
        else:
            gap = torch.full((s.shape[0],), math.inf, dtype=s.dtype)
        margins.append(gap)
    return out


def routed_ff(h, w, p, mlp, margins=None):
    wt = route(h, w, p, mlp["router"], margins)
    y = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=h.dtype)
    for e in range(mlp["router"]["experts"]):
        rows = (wt[:, e] != 0).nonzero().flatten()
        if len(rows):
            y[rows] += gated_expert(h[rows] * wt[rows, e:e + 1], w, f"{p}e{e}.", mlp["expert"]["limit"])
    if mlp.get("shared"):
        y = y + gated_expert(h, w, p + "shared.", mlp["shared"]["limit"])
    return y


def forward(w, cfg, ids, dtype=F64, streams=None, margins=None, pos0=0):
    """Logits [T, vocab] of one sequence.  `streams`: a list that receives the stream after every
    layer (after the weighted sum); `margins`: see `route`."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    ids = torch.as_tensor(ids, dtype=torch.long)
    pos = torch.arange(pos0, pos0 + len(ids))
    x = w["embed"][ids] * cfg["embedding"]["scale"]
    results = [x]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = layer_norm(x, eps, w[p + "norm1"], w[p + "norm1.b"])
        if layer["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kept[i] = keys_and_values(h, w, p + "mix.", m, pos, eps)
                src = i
            y = logistic_attention(h, w, p + "mix.", m, pos, eps, *kept[src])
        else:
            y, _ = gated_recurrence(h, w, p + "mix.")
        x = x + layer_norm(y, eps, w[p + "norm1b"], w[p + "norm1b.b"])
        if layer.get("mlp"):
            h = layer_norm(x, eps, w[p + "norm2"], w[p + "norm2.b"])
            y = routed_ff(h, w, p + "mlp.", layer["mlp"], margins)
            x = x + layer_norm(y, eps, w[p + "norm2b"], w[p + "norm2b.b"])
        results.append(x)
        x = sum(w[p + "dwa"][j] * results[j] for j in range(i + 2))
        if streams is not None:
            streams.append(x)
    x = layer_norm(x, eps, w["final.norm"], w["final.norm.b"])
    return x @ w["head"].T


def generate_greedy(w, cfg, ids, n, dtype=F64):
    ids = list(ids)
    out = []
    for _ in range(n):
        logits = forward(w, cfg, ids, dtype)
        t = int(torch.argmax(logits[-1]))
        out.append(t)
        ids.append(t)
    return out


def tensor_shapes(cfg):
    W, V = cfg["width"], cfg["vocab"]
    s = {"embed": (V, W), "head": (V, W), "final.norm": (W,), "final.norm.b": (W,)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if layer.get("mlp") else ()):
            s[p + n] = (W,)
            s[p + n + ".b"] = (W,)
        if layer["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            s[p + "mix.q"] = (H * d, W)
            if m.get("kv_from") is None:
                s[p + "mix.k"] = (G * d, W)
                s[p + "mix.v"] = (G * dv, W)
            s[p + "mix.pb"] = (H,)
            s[p + "mix.g"] = (H, W)
            s[p + "mix.o"] = (W, H * dv)
        else:
            n = m["width"]
            s.update({p + "mix.z": (n, W), p + "mix.z.b": (n,), p + "mix.x": (n, W), p + "mix.x.b": (n,),
                      p + "mix.g": (n, W), p + "mix.o": (W, n)})
        f = layer.get("mlp")
        if f:
            for e in range(f["router"]["experts"]):
                s[f"{p}mlp.e{e}.gate"] = (f["expert"]["ff"], W)
                s[f"{p}mlp.e{e}.up"] = (f["expert"]["ff"], W)
                s[f"{p}mlp.e{e}.down"] = (W, f["expert"]["ff"])
            s[p + "mlp.router"] = (f["router"]["experts"], W)
            if f.get("shared"):
                s[p + "mlp.shared.gate"] = (f["shared"]["ff"], W)
                s[p + "mlp.shared.up"] = (f["shared"]["ff"], W)
                s[p + "mlp.shared.down"] = (W, f["shared"]["ff"])
        s[p + "dwa"] = (i + 2,)
    return s


def random_weights(cfg, seed, gain=1.0, dtype=torch.bfloat16):
    """Weights of the tests' own making: products N(0, gain / sqrt(fan in)), norms near 1 with small
    biases, score biases and the averaging weights spread so that none of them is idle."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1] if not name.endswith(".b") else name.split(".")[-2] + ".b"
        if name.endswith("dwa"):
            t = 1.0 / shape[0] + 0.3 * torch.randn(shape, generator=g)
        elif "norm" in name and name.endswith(".b"):
            t = 0.1 * torch.randn(shape, generator=g)
        elif "norm" in name:
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif leaf == "pb":
            t = -1.0 + torch.randn(shape, generator=g)
        elif leaf in ("z.b", "x.b"):
            t = 0.5 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        elif leaf == "router":
            t = 2.0 * torch.randn(shape, generator=g) / math.sqrt(shape[1])
        else:
            t = gain * torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        out[name] = t.to(dtype)
    return out
