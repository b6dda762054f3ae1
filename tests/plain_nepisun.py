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


def recurrence(xs, Bm, Cm, dt, A_log, D, S=None):
    """xs [T, Hd, dv], Bm and Cm [T, G, N], dt [T, Hd] (after softplus): per head S <- exp(-exp(A) dt) S + dt B x^T,
    y = S^T C + D x.  Returns (y [T, Hd, dv], the last S [Hd, N, dv])."""
    T, Hd, dv = xs.shape
    G, N = Bm.shape[1], Bm.shape[2]
    per = Hd // G
    decay = torch.exp(-torch.exp(A_log)[None, :] * dt)
    S = torch.zeros(Hd, N, dv, dtype=xs.dtype) if S is None else S
    ys = []
    for t in range(T):
        Bt = Bm[t].repeat_interleave(per, dim=0)             # [Hd, N]
        Ct = Cm[t].repeat_interleave(per, dim=0)
        S = decay[t][:, None, None] * S + dt[t][:, None, None] * Bt[:, :, None] * xs[t][:, None, :]
        ys.append((S * Ct[:, :, None]).sum(dim=1) + D[:, None] * xs[t])
    return torch.stack(ys), S


def gated_group_norm(y, z, parts, eps, w):
    """y * silu(z), normed in `parts` equal parts of the row, times w."""
    T, inner = y.shape
    g = y * silu(z)
    return rms(g.view(T, parts, inner // parts), eps).reshape(T, inner) * w


def state_space(h, w, p, m, eps):
    """Kind `mamba2`: one projection to [z | x B C | dt], a short causal convolution and silu on x B C,
    the recurrence, the gated norm in parts, the output projection."""
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
    y, _ = recurrence(xs, Bm, Cm, dt, w[p + "A_log"], w[p + "D"])
    return gated_group_norm(y.reshape(T, inner), z, m["norm_groups"], eps, w[p + "norm"]) @ w[p + "o"].T


def dense_ff(h, w, p):
    return (torch.relu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def small_expert(h, w, p):
    return (torch.relu(h @ w[p + "up"].T) ** 2) @ w[p + "down"].T


def _gap(values, n):
    """Per row, how far the n-th largest of `values` lies above the next one, as a share of itself (1 if there
    is no next one)."""
    if n >= values.shape[-1]:
        return torch.ones(values.shape[0], dtype=values.dtype)
    srt = values.sort(dim=-1, descending=True).values
    return (srt[:, n - 1] - srt[:, n]) / srt[:, n - 1]


def route(h, w, p, r, margins=None):
    """The chosen experts of every token and their weights: [T, top] each.  `margins`, a list, receives per
    token the smallest relative gap by which a group or an expert was chosen over the next one."""
    E, top = r["experts"], r["top"]
    s = torch.softmax(h @ w[p + "router"].T, dim=-1)                     # [T, E]
    allowed = torch.ones_like(s, dtype=torch.bool)
    groups = r.get("groups")
    margin = torch.ones(s.shape[0], dtype=s.dtype)
    if groups:
        per = E // groups["count"]
        best = s.view(-1, groups["count"], per).max(dim=-1).values       # [T, count]
        kept = best.topk(groups["keep"], dim=-1).indices
        ok = torch.zeros_like(best, dtype=torch.bool).scatter_(1, kept, True)
        allowed = ok.repeat_interleave(per, dim=1)
        margin = torch.minimum(margin, _gap(best, groups["keep"]))
    masked = s.masked_fill(~allowed, 0.0)
    chosen = s.masked_fill(~allowed, -1.0).topk(top, dim=-1).indices
    if margins is not None:
        margins.append(torch.minimum(margin, _gap(masked, top)))
    return chosen, s.gather(1, chosen)


def routed_ff(h, w, p, mlp, margins=None):
    chosen, weight = route(h, w, p, mlp["router"], margins)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(chosen[t].tolist(), weight[t]):
            out[t] += g * small_expert(h[t:t + 1], w, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out = out + small_expert(h, w, p + "shared.")
    return out


MIXERS = {"attention": attention_gated, "attention_2": attention_windowed}


def forward(w, cfg, ids, dtype=F64, streams=None, margins=None):
    """Logits [T, V] of one prompt from the first position.  `streams`, a list, receives the
    residual stream after every layer; `margins`, a list, one tensor [T] per routed layer: by how
    much the router's choice was made (see `route`)."""
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
            x = x + (dense_ff(h, w, p + "mlp.") if mlp["kind"] == "dense" else routed_ff(h, w, p + "mlp.", mlp, margins))
        if streams is not None:
            streams.append(x.clone())
    return rms(x, eps, w["final.norm"]) @ w["embed"].T


def generate_greedy(w, cfg, ids, n, dtype=F64):
    """n tokens, each the argmax of the last position's logits (of equal maxima the last)."""
    ids, out = list(ids), []
    for _ in range(n):
        lg = forward(w, cfg, ids, dtype)[-1]
        t = int((lg == lg.max()).nonzero().max())
        out.append(t)
        ids.append(t)
    return out


def tensor_shapes(cfg):
    """Every tensor of a model of this configuration: name -> shape."""
    W = cfg["width"]
    out = {"embed": (cfg["vocab"], W), "final.norm": (W,)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (W,)
        if layer["type"] == "mamba2":
            inner, GN = m["heads"] * m["vdim"], m["groups"] * m["state"]
            C = inner + 2 * GN
            out.update({p + "mix.in": (inner + C + m["heads"], W), p + "mix.conv": (C, m["conv"]), p + "mix.conv.b": (C,),
                        p + "mix.dt_bias": (m["heads"],), p + "mix.A_log": (m["heads"],), p + "mix.D": (m["heads"],),
                        p + "mix.norm": (inner,), p + "mix.o": (W, inner)})
        else:
            Q, K, V = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            out.update({p + "mix.q": (Q, W), p + "mix.k": (K, W), p + "mix.v": (V, W), p + "mix.o": (W, m["heads"] * m["vdim"])})
            if layer["type"] == "attention":
                out.update({p + "mix.q.norm": (m["dim"],), p + "mix.k.norm": (m["dim"],), p + "mix.g": (m["heads"] * m["vdim"], W)})
            else:
                out.update({p + "mix.q.b": (Q,), p + "mix.k.b": (K,), p + "mix.v.b": (V,), p + "mix.o.b": (W,)})
            if m.get("v_mix"):
                out[p + "mix.vmix"] = ()
        mlp = layer.get("mlp")
        if not mlp:
            continue
        out[p + "norm2"] = (W,)
        if mlp["kind"] == "dense":
            out.update({p + "mlp.gate": (mlp["ff"], W), p + "mlp.up": (mlp["ff"], W), p + "mlp.down": (W, mlp["ff"])})
        else:
            for e in range(mlp["router"]["experts"]):
                out[p + f"mlp.e{e}.up"] = (mlp["expert"]["ff"], W)
                out[p + f"mlp.e{e}.down"] = (W, mlp["expert"]["ff"])
            out[p + "mlp.router"] = (mlp["router"]["experts"], W)
            if mlp.get("shared"):
                out[p + "mlp.shared.up"] = (mlp["shared"]["ff"], W)
                out[p + "mlp.shared.down"] = (W, mlp["shared"]["ff"])
    return out


def random_weights(cfg, seed, gain=1.0):
    """bfloat16 tensors whose sizes follow the configuration, scaled so that every mechanism matters:
    scores of a few units, router logits that differ, decays between 0.2 and 0.9, a mixing weight
    well away from 0 and 1."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".", 1)[1] if name.startswith("l") else name
        if leaf in ("norm1", "norm2", "mix.norm") or name == "final.norm":
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif leaf in ("mix.q.norm", "mix.k.norm"):
            t = gain * (1.5 + 0.3 * torch.randn(shape, generator=g))
        elif leaf == "mix.vmix":
            t = torch.tensor(0.25 + 0.5 * float(torch.rand((), generator=g)))
        elif leaf in ("mix.A_log", "mix.dt_bias"):
            t = 0.6 * torch.randn(shape, generator=g)
        elif leaf == "mix.D":
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif leaf == "mix.conv":
            t = torch.randn(shape, generator=g) * 0.6
        elif leaf.endswith(".b"):
            t = torch.randn(shape, generator=g) * 0.3
        elif leaf == "mlp.router":
            t = torch.randn(shape, generator=g) * (2.0 / shape[1] ** 0.5)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) * (1.0 / shape[1] ** 0.5)
            if leaf in ("mix.q", "mix.k"):
                t = t * gain
        out[name] = t.to(torch.bfloat16)
    return out
