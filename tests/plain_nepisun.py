"""A plain, slow implementation of Nepisun in float64, one function per mechanism, written from
the design's equations.  It shares no code with the package: the tests compare the engine
against it.

Notation.  x: the residual stream [T, W].  rms(t, w) = t / sqrt(mean(t^2) + eps) * w over the
last axis.  A layer is x <- x + mixer(rms(x, n1)); x <- x + ff(rms(x, n2)) (the second only with
a feed-forward).  Mixers: two kinds of grouped-query attention and a state-space layer
(a diagonal linear recurrence per head over a matrix state).  Feed-forwards: gated dense, or a
routed mixture of small ungated experts with a shared one.
"""
import math

import torch

F64 = torch.float64


def rms(t, eps, w=None):
    y = t / torch.sqrt((t * t).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def silu(t):
    return t * torch.sigmoid(t)


def rotate_halves(t, pos, base, dims):
    """t [T, heads, d]; the first `dims` channels of every head are rotated: channel i pairs with
    i + dims/2, angle pos * base^(-2i/dims)."""
    if not dims:
        return t
    half = dims // 2
    f = torch.pow(torch.tensor(float(base), dtype=F64), -2.0 * torch.arange(half, dtype=F64) / dims)
    a = pos.to(F64)[:, None] * f[None, :]                     # [T, half]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = t[..., :half], t[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, t[..., dims:]], dim=-1)


def visible(T, window=None, keep_first=0):
    """[T, T] bool: row p sees column j iff j <= p and (no window, or p - j < window, or j < keep_first)."""
    p = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= p
    if window:
        ok &= ((p - j) < window) | (j < keep_first)
    return ok


def softmax_rows(s, ok, extra_one=False):
    """Softmax over the visible columns; `extra_one`: the denominator also counts a score of 0
    that has no column."""
    s = s.masked_fill(~ok, -math.inf)
    m = s.max(dim=-1, keepdim=True).values
    if extra_one:
        m = torch.clamp(m, min=0.0)
    e = torch.exp(s - m)
    den = e.sum(dim=-1, keepdim=True)
    if extra_one:
        den = den + torch.exp(-m)
    return e / den


def mix_values(v, lam, v_first):
    """v <- (1 - lam) v + lam v_first; the first layer that mixes passes its values on unchanged."""
    if v_first is None:
        return v
    return (1.0 - lam) * v + lam * v_first


def attention_core(q, k, v, m, ok, extra_one):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H * dv]."""
    T, H, G = q.shape[0], m["heads"], m["kv_heads"]
    rep = H // G
    kh = k.repeat_interleave(rep, dim=1).transpose(0, 1)     # [H, T, d]
    vh = v.repeat_interleave(rep, dim=1).transpose(0, 1)
    s = (q.transpose(0, 1) @ kh.transpose(1, 2)) * m["scale"]
    a = softmax_rows(s, ok, extra_one)
    return (a @ vh).transpose(0, 1).reshape(T, -1)


def attention_gated(h, w, p, m, eps, shared):
    """Kind `attention`: a norm of q and k per head (one weight for all heads), rotation, causal,
    a softmax whose denominator counts one more, a gate per channel.  `shared`: what the layers
    that mix values pass along ("v_first")."""
    T, H, G, d, dv = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).view(T, H, d)
    k = (h @ w[p + "k"].T).view(T, G, d)
    v = (h @ w[p + "v"].T).view(T, G, dv)
    q, k = rms(q, eps, w[p + "q.norm"]), rms(k, eps, w[p + "k.norm"])
    pos = torch.arange(T)
    rot = m.get("rot") or {}
    q = rotate_halves(q, pos, rot.get("base", 1.0), rot.get("dims", 0))
    k = rotate_halves(k, pos, rot.get("base", 1.0), rot.get("dims", 0))
    if m.get("v_mix"):
        v = mix_values(v, w[p + "vmix"], shared.get("v_first"))
        shared.setdefault("v_first", v)
    heads = attention_core(q, k, v, m, visible(T), extra_one=True)
    heads = heads * torch.sigmoid(h @ w[p + "g"].T)
    return heads @ w[p + "o"].T


def attention_windowed(h, w, p, m, eps, shared):
    """Kind `attention_2`: biases, rotation, a sliding window that also keeps the first tokens,
    an ordinary softmax."""
    T, H, G, d, dv = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, d)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, d)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, dv)
    pos = torch.arange(T)
    rot = m.get("rot") or {}
    q = rotate_halves(q, pos, rot.get("base", 1.0), rot.get("dims", 0))
    k = rotate_halves(k, pos, rot.get("base", 1.0), rot.get("dims", 0))
    if m.get("v_mix"):
        v = mix_values(v, w[p + "vmix"], shared.get("v_first"))
        shared.setdefault("v_first", v)
    mask = m.get("mask") or {}
    ok = visible(T, mask.get("size"), mask.get("keep_first", 0))
    heads = attention_core(q, k, v, m, ok, extra_one=False)
    return heads @ w[p + "o"].T + w[p + "o.b"]


def causal_conv(u, weight, bias):
    """u [T, C]; weight [C, taps], the last column multiplies the current token; zeros before the start."""
    T, C = u.shape
    taps = weight.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=u.dtype), u], dim=0)
    out = bias[None, :].expand(T, C).clone()
    for j in range(taps):
        out = out + padded[j:j + T] * weight[:, j][None, :]
    return out


def state_space(h, w, p, m, eps):
    """Kind `mamba2`: per head a state S [N, dv]: S <- exp(-exp(A) dt) S + dt B x^T, y = S^T C + D x."""
    T = h.shape[0]
    Hd, dv, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = Hd * dv
    proj = h @ w[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    xs = xbc[:, :inner].view(T, Hd, dv)
    Bm = xbc[:, inner:inner + G * N].view(T, G, N)
    Cm = xbc[:, inner + G * N:].view(T, G, N)
    dt = torch.nn.functional.softplus(dt + w[p + "dt_bias"], threshold=1e9)       # [T, Hd]
    decay = torch.exp(-torch.exp(w[p + "A_log"])[None, :] * dt)
    per = Hd // G
    S = torch.zeros(Hd, N, dv, dtype=h.dtype)
    ys = []
    for t in range(T):
        Bt = Bm[t].repeat_interleave(per, dim=0)             # [Hd, N]
        Ct = Cm[t].repeat_interleave(per, dim=0)
        S = decay[t][:, None, None] * S + dt[t][:, None, None] * Bt[:, :, None] * xs[t][:, None, :]
        y = (S * Ct[:, :, None]).sum(dim=1) + w[p + "D"][:, None] * xs[t]
        ys.append(y.reshape(inner))
    y = torch.stack(ys) * silu(z)
    parts = m["norm_groups"]
    y = rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * w[p + "norm"]
    return y @ w[p + "o"].T


def dense_ff(h, w, p):
    return (torch.relu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def small_expert(h, w, p):
    return (torch.relu(h @ w[p + "up"].T) ** 2) @ w[p + "down"].T


def route(h, w, p, r):
    """The chosen experts of every token and their weights: [T, top] each."""
    E, top = r["experts"], r["top"]
    s = torch.softmax(h @ w[p + "router"].T, dim=-1)                     # [T, E]
    allowed = torch.ones_like(s, dtype=torch.bool)
    groups = r.get("groups")
    if groups:
        per = E // groups["count"]
        best = s.view(-1, groups["count"], per).max(dim=-1).values       # [T, count]
        kept = best.topk(groups["keep"], dim=-1).indices
        ok = torch.zeros_like(best, dtype=torch.bool).scatter_(1, kept, True)
        allowed = ok.repeat_interleave(per, dim=1)
    chosen = s.masked_fill(~allowed, -1.0).topk(top, dim=-1).indices
    return chosen, s.gather(1, chosen)


def routed_ff(h, w, p, mlp):
    chosen, weight = route(h, w, p, mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(chosen[t].tolist(), weight[t]):
            out[t] += g * small_expert(h[t:t + 1], w, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out = out + small_expert(h, w, p + "shared.")
    return out


MIXERS = {"attention": attention_gated, "attention_2": attention_windowed}


def forward(w, cfg, ids, dtype=F64, streams=None):
    """Logits [T, V] of one prompt from the first position.  `streams`, a list, receives the
    residual stream after every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(ids)]
    shared = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms(x, eps, w[p + "norm1"])
        if layer["type"] == "mamba2":
            x = x + state_space(h, w, p + "mix.", layer["mixer"], eps)
        else:
            x = x + MIXERS[layer["type"]](h, w, p + "mix.", layer["mixer"], eps, shared)
        mlp = layer.get("mlp")
        if mlp:
            h = rms(x, eps, w[p + "norm2"])
            x = x + (dense_ff(h, w, p + "mlp.") if mlp["kind"] == "dense" else routed_ff(h, w, p + "mlp.", mlp))
        if streams is not None:
            streams.append(x.clone())
    return rms(x, eps, w["final.norm"]) @ w["embed"].T
