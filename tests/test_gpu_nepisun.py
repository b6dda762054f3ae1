"""Nepisun on the GPU against the plain implementation of `plain_nepisun.py`: every new kernel alone
(the head-wise step before an attention, the state-space mixer's convolution, recurrence and gated norm,
the router, the experts' activation), attention with keys made to stand out at every edge of a window and
of the kept first tokens, then whole models of the tests' own sizes through the engine: whole prompts,
the stream after every layer, decoding token by token, portions down to two tokens, unequal batches,
slots, pages and state blocks used again, long decoding, and greedy generation through the entry point."""
import copy
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_nepisun as plain
from test_gpu_fanitar import Sequence
from test_gpu_sozetar import some_prompts, write_model
from test_nepisun_config import MIXED, attn, attn2, dense, layer, moe, ssm
from util import rel_err, rms_err

pytestmark = pytest.mark.gpu
REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 3e-5, "bfloat16": 6e-2}
RMS = {"float32": 1e-5, "bfloat16": 2.5e-2}
# a router's choice made by less than this share of the score may fall the other way under rounding
MARGIN = {"float32": 1e-3, "bfloat16": 6e-2}

# heads that the matrix cores take (keys of 64 and 128, values of 64), windows that are no multiple of a page, more
# kept tokens than a page, states of 64 and 128, many experts
CORES = {"architecture": "Nepisun", "vocab": 256, "width": 128, "norm": {"eps": 1e-6}, "layers": [
    layer(attn2(4, 2, 64, 64, 0.125, rot=(10000.0, 64), v_mix=True, window=100, keep_first=70), dense(192)),
    layer(ssm(4, 64, 64, 1, 4, 1), moe(32, 6, 32, groups=(8, 4), shared=64)),
    layer(attn(4, 1, 128, 64, 0.09, rot=(500000.0, 64)), moe(16, 2, 64)),
    layer(ssm(2, 32, 128, 2, 2, 2), dense(128)),
    layer(attn(2, 2, 64, 64, 0.125, rot=(100.0, 32), v_mix=True), None),
]}
# what a model may happen to make 1 or equal: one head, one group, one expert of which one is used, one group of
# experts, every group kept, top = experts, a window of one (a position sees itself and the kept ones), no tokens
# kept, no window at all, one tap (no convolution), no rotation, values as wide as keys, a single layer that mixes values
ONES = {"architecture": "Nepisun", "vocab": 96, "width": 32, "norm": {"eps": 1e-4}, "layers": [
    layer(ssm(1, 16, 8, 1, 1, 1), moe(1, 1, 16)),
    layer(attn2(1, 1, 16, 16, 0.25, window=1, keep_first=2), moe(4, 4, 8, groups=(1, 1))),
    layer(attn(2, 2, 8, 8, 0.35, v_mix=True), moe(6, 2, 8, groups=(3, 3), shared=8)),
    layer(attn2(2, 1, 16, 8, 0.3, rot=(50.0, 16)), dense(16)),
    layer(ssm(2, 8, 4, 2, 2, 2), None),
]}
# sizes that no kernel's fast way takes: a width that is no multiple of 8, heads of 12 and 20, three heads, an odd
# vocabulary, states of 5 and 33, seven taps, three normed parts, five experts
ODD = {"architecture": "Nepisun", "vocab": 131, "width": 100, "norm": {"eps": 1e-5}, "layers": [
    layer(ssm(3, 20, 33, 3, 7, 3), moe(5, 2, 12, shared=10)),
    layer(attn(3, 3, 12, 20, 0.29, rot=(300.0, 6), v_mix=True), dense(50)),
    layer(attn2(6, 3, 20, 20, 0.2, rot=(20.0, 20), v_mix=True, window=33, keep_first=65), moe(9, 3, 10, groups=(3, 2))),
    layer(ssm(6, 12, 5, 2, 3, 1), dense(36)),
    layer(attn2(3, 1, 10, 12, 0.3, window=65, keep_first=1), None),
]}
CONFIGS = {"mixed": MIXED, "cores": CORES, "ones": ONES, "odd": ODD}
LENGTHS = {"mixed": [1, 7, 23, 150], "cores": [5, 64, 129, 330], "ones": [2, 65, 130, 200], "odd": [4, 33, 67, 140]}
NAMES = list(CONFIGS)


def dev(t, dtype=None):
    return t.to("cuda", dtype) if dtype is not None else t.to("cuda")


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device="cuda")


# ---------------------------------------------------------------------------------------------
# the kernels one by one
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq, nkv, dk, dv, dims, biased, normed, gated, mix", [
    (4, 2, 32, 16, 16, True, False, False, 2), (4, 2, 32, 16, 32, False, True, True, 1), (3, 3, 12, 20, 6, False, True, True, 2),
    (1, 1, 8, 8, 0, True, True, False, 0), (8, 2, 64, 128, 64, False, False, True, 0), (2, 1, 200, 72, 100, True, True, True, 2)])
def test_a_projection_row_head_by_head(dtype, nq, nkv, dk, dv, dims, biased, normed, gated, mix):
    """Biases, the norm of every head of q and k by its own root mean square, the rotation of the first
    channels of every head, the values mixed with another layer's, the logistic gate."""
    from torchless_rs_amd.kernels import ops
    g = torch.Generator().manual_seed(nq * dk + dv)
    n, eps, lam, base = 9, 1e-5, 0.3, 500.0
    ng = nq * dv if gated else 0
    Q, K, V = nq * dk, nkv * dk, nkv * dv
    proj = torch.randn(n, Q + K + V + ng, generator=g) * 2
    bias = torch.randn(Q + K + V + ng, generator=g) if biased else None
    if bias is not None:
        bias[Q + K + V:] = 0
    qw, kw = (1 + 0.3 * torch.randn(dk, generator=g) for _ in range(2))
    first = torch.randn(n, V, generator=g)
    pos = torch.tensor([0, 1, 2, 63, 64, 65, 300, 1000, 2047][:n])     # (angles are float32: about 1e-4 of a turn off at 2047)
    rot = ops.Rotation(dev(torch.pow(torch.tensor(base), -2.0 * torch.arange(dims // 2) / dims).float()), dims) if dims else ops.NO_ROTATION
    terms = ops.HeadTerms(bias=dev(bias) if biased else None, q_norm=dev(qw) if normed else None,
                          k_norm=dev(kw) if normed else None, eps=eps, mix=mix, lam=lam)
    dt = TORCH[dtype]
    q, k, v = (torch.empty(n, h, d, dtype=dt, device="cuda") for h, d in ((nq, dk), (nkv, dk), (nkv, dv)))
    gate = torch.empty(n, ng, device="cuda") if ng else None
    vf = dev(first.clone()) if mix == 2 else torch.full((n, V), float("nan"), device="cuda")
    ops.head_prepare(dev(proj), i32(pos.tolist()), rot, terms, nq, nkv, dk, dv, ng, q, k, v, gate, v_first=vf if mix else None)
    row = proj.double() + (bias.double() if biased else 0.0)
    wq, wk, wv = row[:, :Q].view(n, nq, dk), row[:, Q:Q + K].view(n, nkv, dk), row[:, Q + K:Q + K + V].view(n, nkv, dv)
    if normed:
        wq, wk = plain.rms(wq, eps, qw.double()), plain.rms(wk, eps, kw.double())
    wq, wk = plain.rotate_halves(wq, pos, base, dims), plain.rotate_halves(wk, pos, base, dims)
    if mix == 2:
        wv = plain.mix_values(wv, lam, first.double().view(n, nkv, dv))
    tol = 3e-4 if dtype == "float32" else 8e-3
    assert rel_err(q, wq) < tol and rel_err(k, wk) < tol and rel_err(v, wv) < tol
    if mix == 1:
        assert rel_err(vf, wv.reshape(n, V)) < 1e-6          # left unrounded for the later layers
    if ng:
        assert rel_err(gate, torch.sigmoid(row[:, Q + K + V:])) < 1e-6


def conv_scan_steps(dtype, m, w, proj, lengths, cuts, slots, n_slots=7):
    """The three kernels of the state-space mixer over sequences of `lengths` (rows of `proj` after one
    another), in steps that bring `cuts[i]` rows of every sequence that still has some: y [n, inner] gated
    and normed, in the order of `proj`."""
    from torchless_rs_amd.kernels import ops
    Hd, dv, N, G, taps, parts = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"], m["norm_groups"]
    inner = Hd * dv
    C = inner + 2 * G * N
    conv_elems = (taps - 1) * C
    block = torch.full((n_slots, conv_elems + Hd * N * dv), float("nan"), device="cuda")
    for s in slots:
        block[s].zero_()
    starts = [sum(lengths[:b]) for b in range(len(lengths))]
    done = [0] * len(lengths)
    out = torch.zeros(sum(lengths), inner, dtype=torch.float64)
    f = {k: dev(w[k].float()) for k in w}
    for cut in cuts:
        live = [b for b in range(len(lengths)) if done[b] < lengths[b]]
        if not live:
            break
        take = [min(cut, lengths[b] - done[b]) for b in live]
        rows = torch.cat([torch.arange(starts[b] + done[b], starts[b] + done[b] + t) for b, t in zip(live, take)])
        p = dev(proj[rows].float().contiguous())
        n = len(rows)
        cu = i32([0] + list(np.cumsum(take)))
        row_seq = i32([j for j, t in enumerate(take) for _ in range(t)])
        sl = i32([slots[b] for b in live])
        u = torch.empty(n, C, dtype=TORCH[dtype], device="cuda")
        ops.ssm_conv(p, inner, C, f["conv"], f["conv.b"], block, row_seq, cu, sl, u, single=all(t == 1 for t in take))
        y = torch.empty(n, inner, device="cuda")
        ops.ssm_scan(u, p, inner + C, G, N, Hd, dv, f["dt_bias"], f["A_log"], f["D"], block[:, conv_elems:], cu, sl, y)
        gn = torch.empty(n, inner, dtype=TORCH[dtype], device="cuda")
        ops.ssm_gate_norm(y, p, parts, f["norm"], 1e-5, gn)
        out[rows] = gn.double().cpu()
        for b, t in zip(live, take):
            done[b] += t
    return out


def plain_conv_scan(m, w, proj):
    T = proj.shape[0]
    Hd, dv, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = Hd * dv
    W = {k: v.double() for k, v in w.items()}
    p = proj.double()
    z, xbc, dt = p[:, :inner], p[:, inner:2 * inner + 2 * G * N], p[:, 2 * inner + 2 * G * N:]
    xbc = plain.silu(plain.causal_conv(xbc, W["conv"], W["conv.b"]))
    dt = torch.nn.functional.softplus(dt + W["dt_bias"], threshold=1e9)
    y, _ = plain.recurrence(xbc[:, :inner].view(T, Hd, dv), xbc[:, inner:inner + G * N].view(T, G, N),
                            xbc[:, inner + G * N:].view(T, G, N), dt, W["A_log"], W["D"])
    return plain.gated_group_norm(y.reshape(T, inner), z, m["norm_groups"], 1e-5, W["norm"])


SSM_SHAPES = [dict(heads=4, vdim=16, state=24, groups=2, conv=4, norm_groups=2), dict(heads=1, vdim=8, state=4, groups=1, conv=1, norm_groups=1),
              dict(heads=3, vdim=20, state=33, groups=3, conv=7, norm_groups=3), dict(heads=2, vdim=64, state=128, groups=1, conv=2, norm_groups=1),
              dict(heads=6, vdim=12, state=5, groups=2, conv=3, norm_groups=1), dict(heads=2, vdim=128, state=64, groups=2, conv=4, norm_groups=4),
              dict(heads=2, vdim=37, state=70, groups=1, conv=2, norm_groups=2), dict(heads=1, vdim=72, state=256, groups=1, conv=4, norm_groups=3)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m", SSM_SHAPES, ids=lambda m: "h{heads}v{vdim}n{state}g{groups}c{conv}p{norm_groups}".format(**m))
def test_the_state_space_kernels_in_steps_of_any_size(dtype, m):
    """Convolution, recurrence and gated norm: three unequal sequences, whole, in portions down to one row, and
    row by row, their blocks anywhere among the slots: what a step leaves in a block is what the next one needs."""
    g = torch.Generator().manual_seed(m["heads"] * m["state"])
    Hd, dv, N, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = Hd * dv
    C = inner + 2 * G * N
    lengths = [37, 1, 12]
    proj = torch.randn(sum(lengths), inner + C + Hd, generator=g)
    w = {"conv": torch.randn(C, taps, generator=g) * 0.6, "conv.b": torch.randn(C, generator=g) * 0.3,
         "dt_bias": torch.randn(Hd, generator=g) * 0.6, "A_log": torch.randn(Hd, generator=g) * 0.6,
         "D": 1 + 0.3 * torch.randn(Hd, generator=g), "norm": 1 + 0.2 * torch.randn(inner, generator=g)}
    at = 0
    want = []
    for n in lengths:
        want.append(plain_conv_scan(m, w, proj[at:at + n]))
        at += n
    want = torch.cat(want)
    tol = 3e-5 if dtype == "float32" else 2.5e-2
    for cuts, slots in (([40], [0, 1, 2]), ([5, 1, 2, 40], [6, 0, 3]), ([1] * 37, [2, 5, 1]), ([9, 8, 3, 17], [4, 3, 2])):
        got = conv_scan_steps(dtype, m, w, proj, lengths, cuts, slots)
        assert rel_err(got, want) < tol, (cuts, rel_err(got, want))


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_state_that_is_carried_far_and_one_that_is_forgotten(dtype):
    """One head keeps what an early row wrote (a decay of nearly one), the other forgets it within a few rows (a
    fast decay): after 600 rows in steps, the first head still answers the early row's key, the second does not."""
    m = dict(heads=2, vdim=8, state=8, groups=1, conv=1, norm_groups=2)
    T, inner, N = 600, 16, 8
    C = inner + 2 * N
    proj = torch.zeros(T, inner + C + 2)
    proj[:, :inner] = 3.0                                     # the gate nearly open
    proj[:, inner:2 * inner] = 0.01                           # x: small everywhere,
    proj[5, inner:2 * inner] = 4.0                            # large in row 5,
    proj[5, 2 * inner + 2] = 4.0                              # which writes it under key 2 ...
    proj[-1, 2 * inner + N + 2] = 4.0                         # ... that the last row asks for
    proj[:, -2:] = 0.0
    w = {"conv": torch.ones(C, 1), "conv.b": torch.zeros(C), "dt_bias": torch.zeros(2),
         "A_log": torch.tensor([-9.0, 1.5]), "D": torch.zeros(2), "norm": torch.ones(inner)}
    want = plain_conv_scan(m, w, proj)
    for cuts in ([T], [300, 299, 1], [6] + [1] * 594, [5, 1, 594]):
        got = conv_scan_steps(dtype, m, w, proj, [T], cuts, [1])
        assert rel_err(got, want) < (3e-5 if dtype == "float32" else 2e-2), cuts
    # (each half of the row is normed alone: the head that kept the row is of order one, the other as well, by its norm;
    # so read the recurrence itself, before the norm)
    from torchless_rs_amd.kernels import ops
    u = plain.silu(proj[:, inner:inner + C].double()).float()
    block = torch.zeros(1, 2 * N * 8, device="cuda")
    y = torch.empty(T, inner, device="cuda")
    ops.ssm_scan(dev(u), dev(proj), inner + C, 1, N, 2, 8, dev(w["dt_bias"]), dev(w["A_log"]), dev(w["D"]), block, i32([0, T]), i32([0]), y)
    assert y[-1, :8].min() > 1.0 and y[-1, 8:].abs().max() < 1e-6


@pytest.mark.parametrize("in_dtype", DTYPES)
@pytest.mark.parametrize("E, top, groups", [(8, 2, (4, 2)), (8, 3, (2, 1)), (16, 4, (4, 3)), (1, 1, None), (4, 4, (1, 1)), (6, 2, (3, 3)),
                                            (5, 2, None), (9, 3, (3, 2)), (64, 6, (8, 4)), (128, 8, None), (12, 1, (12, 5))])
def test_the_router(in_dtype, E, top, groups):
    from torchless_rs_amd.kernels import ops
    g = torch.Generator().manual_seed(E * 7 + top)
    n, W = 40, 36
    h = torch.randn(n, W, generator=g).to(TORCH[in_dtype])
    r = torch.randn(E, W, generator=g) * 0.4
    spec = {"experts": E, "top": top}
    if groups:
        spec["groups"] = {"count": groups[0], "keep": groups[1]}
    margins = []
    chosen, weight = plain.route(h.double(), {"router": r.double()}, "", spec, margins)
    weights = torch.full((n, E), float("nan"), device="cuda")
    idx = torch.empty(n, top, dtype=torch.int32, device="cuda")
    ops.route(dev(h), dev(r), groups[0] if groups else 0, groups[1] if groups else 0, top, weights, idx)
    sure = margins[0] > 1e-4
    assert sure.sum() > n // 2
    want = torch.zeros(n, E, dtype=torch.float64).scatter_(1, chosen, weight)
    assert rel_err(weights[sure], want[sure]) < 2e-6
    assert (idx.cpu().long().sort(dim=1).values[sure] == chosen.sort(dim=1).values[sure]).all()
    assert ((weights > 0).sum(dim=1) == top).all()


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("activation", ["relu2", "relu"])
def test_the_experts_activation_times_the_routers_weight(out_dtype, activation):
    from torchless_rs_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    n, E, ff, shared = 6, 5, 12, 7
    u = torch.randn(n, E * ff + shared, generator=g) * 2
    wts = torch.rand(n, E, generator=g) * (torch.rand(n, E, generator=g) > 0.5)
    out = torch.empty(n, E * ff + shared, dtype=TORCH[out_dtype], device="cuda")
    ops.expert_act(dev(u), dev(wts), E, ff, activation, out)
    a = torch.relu(u.double())
    a = a * a if activation == "relu2" else a
    want = a * torch.cat([wts.double().repeat_interleave(ff, dim=1), torch.ones(n, shared, dtype=torch.float64)], dim=1)
    assert rel_err(out, want) < (1e-6 if out_dtype == "float32" else 8e-3)
    out = torch.empty(n, E * ff + shared, dtype=TORCH[out_dtype], device="cuda")
    ops.expert_act(dev(u), None, 0, ff, activation, out)
    assert rel_err(out, a) < (1e-6 if out_dtype == "float32" else 8e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, E, top, ff, shared, activation", [(64, 8, 2, 32, 48, "relu2"), (100, 5, 2, 12, 10, "relu2"), (32, 1, 1, 16, 0, "relu"),
                                                               (128, 16, 4, 64, 0, "relu2"), (96, 6, 6, 8, 24, "relu"), (256, 64, 6, 40, 72, "relu2")])
def test_the_chosen_experts_alone_row_by_row(dtype, H, E, top, ff, shared, activation):
    """Rows that run their own experts' matrices alone against the plain mixture, and against the wide form."""
    from torchless_rs_amd.kernels import ops
    g = torch.Generator().manual_seed(H + E)
    n, dt = 3, TORCH[dtype]
    y = torch.randn(n, H, generator=g).to(dt)
    up = (torch.randn(E * ff + shared, H, generator=g) / H ** 0.5).to(dt)
    down = (torch.randn(H, E * ff + shared, generator=g) / ff ** 0.5).to(dt)
    r = torch.randn(E, H, generator=g) * 0.3
    chosen, weight = plain.route(y.double(), {"router": r.double()}, "", {"experts": E, "top": top})
    weights = torch.empty(n, E, device="cuda")
    idx = torch.empty(n, top, dtype=torch.int32, device="cuda")
    ops.route(dev(y), dev(r), 0, 0, top, weights, idx)
    assert (idx.cpu().long().sort(dim=1).values == chosen.sort(dim=1).values).all()
    hs = torch.full((n, top * ff + shared), float("nan"), dtype=dt, device="cuda")
    ops.expert_rows_up(dev(y), dev(up), idx, weights, ff, shared, activation, hs)
    x0 = torch.randn(n, H, generator=g)
    x = dev(x0.clone())
    ops.expert_rows_down(hs, dev(down), idx, E, ff, shared, x, accumulate=True)
    z = torch.full((n, H), float("nan"), device="cuda")
    ops.expert_rows_down(hs, dev(down), idx, E, ff, shared, z)

    def act(t):
        t = torch.relu(t)
        return t * t if activation == "relu2" else t
    want = torch.zeros(n, H, dtype=torch.float64)
    U, D = up.double(), down.double()
    for t in range(n):
        for e, s in zip(chosen[t].tolist(), weight[t]):
            want[t] += s * (act(U[e * ff:(e + 1) * ff] @ y[t].double()) @ D[:, e * ff:(e + 1) * ff].T)
        if shared:
            want[t] += act(U[E * ff:] @ y[t].double()) @ D[:, E * ff:].T
    tol = 2e-5 if dtype == "float32" else 1.5e-2
    assert rel_err(z, want) < tol
    assert rel_err(x, x0.double() + want) < tol
    # the wide form: every expert, the ones not chosen times zero
    u = dev(y).float() @ dev(up).float().T
    h = torch.empty(n, E * ff + shared, dtype=dt, device="cuda")
    ops.expert_act(u.contiguous(), weights, E, ff, activation, h)
    assert rel_err(z, h.double() @ dev(down).double().T) < tol


# ---------------------------------------------------------------------------------------------
# attention with keys that stand out
# ---------------------------------------------------------------------------------------------

def heads_steps(dtype, nq, nkv, dk, dv, window, keep_first, unit_sink, q, k, v, cuts, scale):
    """q [L, nq, dk], k [L, nkv, dk], v [L, nkv, dv]: through `head_prepare` (nothing but the split) and
    `attend_and_commit` in steps of `cuts` rows over one sequence's pages."""
    from torchless_rs_amd.kernels import ops
    from torchless_rs_amd.parts.attention_scored import attend_and_commit
    seq = Sequence(dtype, nkv, dk, dv, None)                 # kept first tokens: every position stays in the cache
    sinks = torch.zeros(nq, device="cuda") if unit_sink else None
    terms = ops.ScoreTerms(scale, window, None, sinks, keep_first=keep_first)
    plain_terms = ops.HeadTerms()
    outs, at = [], 0
    for n in cuts:
        ctx, run = seq.step(n)
        proj = dev(torch.cat([q[at:at + n].reshape(n, -1), k[at:at + n].reshape(n, -1), v[at:at + n].reshape(n, -1)], dim=1).float().contiguous())
        qs = torch.empty(n, nq, dk, dtype=seq.dt, device="cuda")
        att = torch.empty(n, nq, dv, dtype=seq.dt, device="cuda")
        if n == 1:
            ops.head_prepare(proj, ctx.row_pos, ops.NO_ROTATION, plain_terms, nq, nkv, dk, dv, 0, qs, None, None, None,
                             table=seq.table, ring_pages=seq.ring, pages=seq.pages)
            ks = vs = None
        else:
            ks = torch.empty(n, nkv, dk, dtype=seq.dt, device="cuda")
            vs = torch.empty(n, nkv, dv, dtype=seq.dt, device="cuda")
            ops.head_prepare(proj, ctx.row_pos, ops.NO_ROTATION, plain_terms, nq, nkv, dk, dv, 0, qs, ks, vs, None)
        attend_and_commit(ctx, run, qs, ks, vs, nkv, dk, dv, terms, None, att)
        outs.append(att.clone())
        at += n
    return torch.cat(outs)


def plain_heads(q, k, v, nq, nkv, scale, window, keep_first, unit_sink):
    L = q.shape[0]
    m = {"heads": nq, "kv_heads": nkv, "scale": scale}
    return plain.attention_core(q.double(), k.double(), v.double(), m, plain.visible(L, window, keep_first), unit_sink).view(L, nq, -1)


ATT_TOL = {"float32": 2e-5, "bfloat16": 1.2e-2}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window, keep", [(1, 0), (1, 3), (2, 1), (63, 64), (64, 65), (65, 63), (100, 20), (129, 1), (200, 130)])
@pytest.mark.parametrize("dk, dv", [(16, 8), (64, 64)])
def test_a_key_just_inside_and_just_outside_the_window_and_the_kept_tokens(dtype, window, keep, dk, dv):
    """The last query asks for ONE key whose value is far from all others: the oldest key inside the window, the
    newest outside, the last kept token and the first that is not kept; in a prompt, in portions and decoded."""
    nq, nkv = 4, 2
    L = max(window, keep) + 140
    g = torch.Generator().manual_seed(window * 3 + keep)
    dt = TORCH[dtype]
    q0, k0, v0 = (torch.randn(L, h, d, generator=g).to(dt).float() for h, d in ((nq, dk), (nkv, dk), (nkv, dv)))
    p = L - 1
    places = [(p - window + 1, True), (p - window, keep > p - window)]
    if keep:
        places += [(keep - 1, True), (keep, p - keep < window)]
    for j, seen in places:
        if j < 0:
            continue
        q, k, v = q0.clone(), k0.clone(), v0.clone()
        k[j] = 0
        k[j, :, 1] = 20.0
        q[p, :, 1] = 3.0
        v[j] = -40.0
        want = plain_heads(q, k, v, nq, nkv, 0.2, window, keep, False)
        assert (want[p].mean() < -30) == seen
        for cuts in ([L], [L - 1, 1], [L - 70, 2, 67, 1], [1, 1, L - 2]):
            got = heads_steps(dtype, nq, nkv, dk, dv, window, keep, False, q, k, v, cuts, 0.2)
            assert rel_err(got, want) < ATT_TOL[dtype], (j, cuts)
            assert (got[p].float().mean() < -30) == seen, (j, cuts)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dk, dv", [(32, 16), (64, 64), (128, 64)])
def test_a_far_key_the_first_tokens_and_one_more_in_the_denominator(dtype, dk, dv):
    nq, nkv, L = 4, 1, 700
    g = torch.Generator().manual_seed(dk)
    dt = TORCH[dtype]
    q, k, v = (torch.randn(L, h, d, generator=g) for h, d in ((nq, dk), (nkv, dk), (nkv, dv)))
    k[3] = 0
    k[3, :, 1] = 20.0
    q[-1] = 0
    q[-1, :, 1] = 3.0                     # the last query asks for position 3, far back, and for nothing else
    v[3] = -40.0
    q, k, v = q.to(dt).float(), k.to(dt).float(), v.to(dt).float()
    want = plain_heads(q, k, v, nq, nkv, 0.2, None, 0, True)
    for cuts in ([L], [650, 50], [699, 1], [1, 1, 1, 697]):
        got = heads_steps(dtype, nq, nkv, dk, dv, None, 0, True, q, k, v, cuts, 0.2)
        assert rel_err(got, want) < ATT_TOL[dtype], cuts
        assert got[-1].float().mean() < -30
    # the first position sees itself and a score of zero without a value: its weight is e^s / (1 + e^s), not 1
    s0 = (q[0] * k[0].repeat_interleave(nq // nkv, dim=0)).sum(-1).double() * 0.2
    share = torch.exp(s0) / (torch.exp(s0) + 1.0)
    assert rel_err(got[0], v[0].double() * share[:, None]) < ATT_TOL[dtype]
    # without it the first position returns its own value
    got = heads_steps(dtype, nq, nkv, dk, dv, None, 0, False, q[:40], k[:40], v[:40], [20, 20], 0.2)
    assert rel_err(got[0], v[0].double().expand(nq, dv)) < ATT_TOL[dtype]


# ---------------------------------------------------------------------------------------------
# whole models through the engine
# ---------------------------------------------------------------------------------------------

def plain_run(w, cfg, ids):
    """Logits and, per row, the smallest share by which a router chose."""
    margins = []
    lg = plain.forward(w, cfg, ids, margins=margins)
    m = torch.stack(margins).min(dim=0).values if margins else torch.ones(len(ids), dtype=torch.float64)
    return lg, m


@pytest.fixture(scope="module")
def zoo(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("nepisun")
    out = {}
    for i, name in enumerate(NAMES):
        cfg = copy.deepcopy(CONFIGS[name])
        w = plain.random_weights(cfg, seed=60 + i)
        ps = some_prompts(cfg["vocab"], LENGTHS[name], seed=23 + i)
        runs = [plain_run(w, cfg, p) for p in ps]
        out[name] = dict(dir=write_model(str(tmp / name), cfg, w), cfg=cfg, w=w, prompts=ps,
                         want=[r[0] for r in runs], margin=[r[1] for r in runs])
    return out


_engines = {}


def engine_for(zoo, name, dtype):
    from torchless_rs_amd.engine import Engine, load_model
    key = (name, dtype)
    if key not in _engines:
        _engines[key] = Engine(load_model(zoo[name]["dir"], dtype), max_tokens=64 * 20, max_slots=8)
    eng = _engines[key]
    assert not eng.cache.length, "a test left slots held"
    for g in eng.cache.groups:              # stale rows and blocks must never be read: make them NaN
        g.storage.fill_(float("nan"))
    for t in eng.cache.state.values():
        t.fill_(float("nan"))
    return eng


def close(got, want, dtype, what, margin=None, tol=None, rms=None):
    """Rows whose routers chose by a wide enough margin must agree (a choice made by a hair may fall the other
    way under the rounding of the router's input, and then the row is another function's).  In bfloat16 the
    stream that reaches a deep router is off by more than its input's rounding: a row in thirty may still fall
    the other way, and is then left out of the comparison of the others."""
    tol, rms = tol or TOL[dtype], rms or RMS[dtype]
    got = got.detach().double().cpu()
    if margin is not None:
        sure = margin > MARGIN[dtype]
        assert int(sure.sum()) * 2 >= len(sure) or len(sure) < 4, (what, "too few sure rows")
        got, want = got[sure], want[sure]
        if dtype == "bfloat16" and len(got):
            err = (got - want).abs().amax(dim=1) / want.abs().max()
            off = err > tol
            assert int(off.sum()) <= max(1, len(err) // 30), (what, "rows off", off.nonzero().flatten().tolist())
            got, want = got[~off], want[~off]
    assert rel_err(got, want) < tol, (what, rel_err(got, want))
    if rms is not False:
        assert rms_err(got, want) < rms, (what, rms_err(got, want))


def test_the_right_parts_and_caches_are_chosen(zoo):
    from torchless_rs_amd.parts.attention_heads import HeadwiseAttentionMixer
    from torchless_rs_amd.parts.ffn_routed import RoutedExperts
    from torchless_rs_amd.parts.state_space import StateSpaceMixer
    eng = engine_for(zoo, "cores", "bfloat16")
    blocks = eng.model.blocks
    assert [type(b.mixer) for b in blocks] == [HeadwiseAttentionMixer, StateSpaceMixer, HeadwiseAttentionMixer, StateSpaceMixer,
                                               HeadwiseAttentionMixer]
    assert [type(b.ffn) for b in blocks[1:3]] == [RoutedExperts, RoutedExperts] and blocks[4].ffn is None
    assert sorted(eng.cache.state) == [1, 3] and all(t.dtype == torch.float32 for t in eng.cache.state.values())
    assert eng.cache.state[1].shape[1] == 3 * (256 + 2 * 64) + 4 * 64 * 64
    a0, a2, a4 = blocks[0].mixer, blocks[2].mixer, blocks[4].mixer
    assert (a0.value_mix, a2.value_mix, a4.value_mix) == ("first", None, "later")
    assert a0.bias and not a0.unit_sink and a2.unit_sink and a2.channel_gate and a0.keep_first == 70


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_each_request_alone_and_whole(zoo, name, dtype):
    from torchless_rs_amd.engine import SeqInput
    eng, z = engine_for(zoo, name, dtype), zoo[name]
    for p, want, m in zip(z["prompts"], z["want"], z["margin"]):
        s = eng.alloc()
        got = eng.step([SeqInput(s, p, list(range(len(p))))]).clone()
        eng.free(s)
        close(got, want, dtype, (name, len(p)), m)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "odd"])
def test_the_stream_after_every_layer(zoo, name, dtype):
    from torchless_rs_amd.engine import Engine, SeqInput, load_model
    from torchless_rs_amd.parts.base import flush_pending
    z = zoo[name]
    streams = []
    plain.forward(z["w"], z["cfg"], z["prompts"][2], streams=streams)
    model = load_model(z["dir"], dtype)
    eng = Engine(model, max_tokens=256, use_graphs=False)
    seen = []
    for blk in model.blocks:
        inner = blk.forward

        def spy(ctx, run, x, *a, _inner=inner, **kw):
            _inner(ctx, run, x, *a, **kw)
            flush_pending(ctx, x)
            ctx.prenormed = None
            seen.append(x.clone())
        blk.forward = spy
    s = eng.alloc()
    eng.step([SeqInput(s, z["prompts"][2], [0])])
    eng.free(s)
    assert len(seen) == len(streams)
    for i, (got, want) in enumerate(zip(seen, streams)):
        assert got.dtype == torch.float32            # the residual sum is kept in 32 bits in both dtypes
        close(got, want, dtype, (name, "after layer", i), z["margin"][2], tol=2e-5 if dtype == "float32" else 4e-2, rms=False)
    eng.close()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_prefill_against_decoding_token_by_token(zoo, name, dtype):
    from torchless_rs_amd.engine import SeqInput
    eng, z = engine_for(zoo, name, dtype), zoo[name]
    for i in (1, 2):
        p = z["prompts"][i]
        s = eng.alloc()
        rows = [eng.step([SeqInput(s, [t], [0])]).clone() for t in p]        # from the very first token
        eng.free(s)
        close(torch.cat(rows), z["want"][i], dtype, (name, len(p), "token by token"), z["margin"][i])
    p = z["prompts"][3]
    k = 40
    s = eng.alloc()
    rows = [eng.step([SeqInput(s, p[:-k], list(range(len(p) - k)))]).clone()]
    rows += [eng.step([SeqInput(s, [t], [0])]).clone() for t in p[-k:]]
    eng.free(s)
    close(torch.cat(rows), z["want"][3], dtype, (name, "prompt then 40 tokens"), z["margin"][3])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("portion", [2, 3, 17, 64, 100])
def test_portions_of_a_prompt(zoo, name, dtype, portion):
    from torchless_rs_amd.engine import SeqInput
    eng, z = engine_for(zoo, name, dtype), zoo[name]
    p, want, m = z["prompts"][3], z["want"][3], z["margin"][3]
    if portion < 4:
        p, want, m = p[:41], want[:41], m[:41]
    s = eng.alloc()
    rows = []
    for at in range(0, len(p), portion):
        part = p[at:at + portion]
        rows.append(eng.step([SeqInput(s, part, list(range(len(part))))]).clone())
    eng.free(s)
    close(torch.cat(rows), want, dtype, (name, portion), m)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_unequal_batches_against_each_alone_with_slots_pages_and_blocks_used_again(zoo, name, dtype):
    """All prompts in one step, then decoded together while the shorter ones end; a second batch takes
    the freed slots, pages and state blocks (which hold the first batch's) and must give the same."""
    from torchless_rs_amd.engine import SeqInput
    eng, z = engine_for(zoo, name, dtype), zoo[name]
    tails = [0, 3, 9, 20]
    for turn in range(2):
        order = list(range(4)) if turn == 0 else [3, 1, 0, 2]
        slots = {i: eng.alloc() for i in order}
        heads = {i: len(z["prompts"][i]) - tails[i] for i in order}
        got = {i: [] for i in order}
        lg = eng.step([SeqInput(slots[i], z["prompts"][i][:heads[i]], list(range(heads[i]))) for i in order])
        at = 0
        for i in order:
            got[i].append(lg[at:at + heads[i]].clone())
            at += heads[i]
        live = [i for i in order if tails[i]]
        for i in order:
            if not tails[i]:
                eng.free(slots[i])
        step = 0
        while live:
            lg = eng.step([SeqInput(slots[i], [z["prompts"][i][heads[i] + step]], [0]) for i in live]).clone()
            for r, i in enumerate(live):
                got[i].append(lg[r:r + 1])
            step += 1
            for i in [i for i in live if step == tails[i]]:
                eng.free(slots[i])
            live = [i for i in live if step < tails[i]]
        for i in order:
            close(torch.cat(got[i]), z["want"][i], dtype, (name, turn, i), z["margin"][i])
        eng.cache.check()
    assert not eng.cache.length


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_long_decoding_past_windows_and_kept_tokens(zoo, name, dtype):
    """A short prompt, then 300 tokens one by one (through captured graphs): every window passes over decoded
    tokens, the kept first tokens stay, the recurrent state is carried 300 times."""
    from torchless_rs_amd.engine import SeqInput
    eng, z = engine_for(zoo, name, dtype), zoo[name]
    ids = some_prompts(z["cfg"]["vocab"], [310], seed=78)[0]
    want, m = plain_run(z["w"], z["cfg"], ids)
    s = eng.alloc()
    rows = [eng.step([SeqInput(s, ids[:10], list(range(10)))]).clone()]
    rows += [eng.step([SeqInput(s, [t], [0])]).clone() for t in ids[10:]]
    eng.free(s)
    close(torch.cat(rows), want, dtype, name, m)


@pytest.mark.parametrize("dtype", DTYPES)
def test_logits_do_not_depend_on_batch_mates(zoo, dtype):
    from torchless_rs_amd.engine import SeqInput
    eng, z = engine_for(zoo, "odd", dtype), zoo["odd"]
    p = z["prompts"][2]
    s = eng.alloc()
    alone = eng.step([SeqInput(s, p, list(range(len(p))))]).clone()
    eng.free(s)
    slots = [eng.alloc() for _ in range(3)]
    lg = eng.step([SeqInput(slots[0], z["prompts"][3], []), SeqInput(slots[1], p, list(range(len(p)))),
                   SeqInput(slots[2], z["prompts"][0], [0])]).clone()
    for s in slots:
        eng.free(s)
    sure = (z["margin"][2] > MARGIN[dtype]).cuda()
    assert rel_err(lg[:len(p)][sure], alone[sure]) < (1e-6 if dtype == "float32" else 2e-2)


def test_many_rows_run_expert_by_expert(zoo, monkeypatch):
    """A prompt of more rows than the framework's own products take, with the bar for sorting rows by expert taken
    down to the tests' sizes: the same logits from every expert's products over its own rows alone."""
    from torchless_rs_amd.engine import SeqInput
    from torchless_rs_amd.parts import ffn_routed
    monkeypatch.setattr(ffn_routed, "GROUPED_ROWS_PER_EXPERT", 1)
    calls = []
    inner = ffn_routed.RoutedExperts._grouped
    monkeypatch.setattr(ffn_routed.RoutedExperts, "_grouped", lambda self, *a: (calls.append(a[1].shape[0]), inner(self, *a))[1])
    for name in ("cores", "mixed"):
        eng, z = engine_for(zoo, name, "bfloat16"), zoo[name]
        p = z["prompts"][3]
        calls.clear()
        s = eng.alloc()
        got = eng.step([SeqInput(s, p, list(range(len(p))))]).clone()
        eng.free(s)
        assert calls and all(c == len(p) for c in calls), calls
        close(got, z["want"][3], "bfloat16", (name, "expert by expert"), z["margin"][3])
        s = eng.alloc()                                                   # two unequal prompts in one step
        q = z["prompts"][2]
        got = eng.step([SeqInput(s, p, [len(p) - 1]), SeqInput(eng.alloc(), q, list(range(len(q))))]).clone()
        for h in eng.cache.held_slots():
            eng.free(h)
        close(got[1:], z["want"][2], "bfloat16", (name, "expert by expert, two prompts"), z["margin"][2])


def test_greedy_generation_through_the_entry_point(zoo):
    from torchless_rs_amd import SamplingConfig, generate_until_eos
    for name in ("mixed", "ones", "odd"):
        eng, z = engine_for(zoo, name, "float32"), zoo[name]
        ps = z["prompts"][:3]
        out = generate_until_eos(eng, ps, SamplingConfig.greedy(), max_tokens=12)
        for p, r in zip(ps, out):
            assert r.tokens == plain.generate_greedy(z["w"], z["cfg"], p, 12), (name, len(p))


def test_the_command_line_and_the_trace_replay(zoo, tmp_path):
    z = zoo["mixed"]
    p = z["prompts"][2]
    r = subprocess.run([sys.executable, os.path.join(REPO, "bin", "torchless"), "--temperature", "0", "--max-tokens", "6",
                        "--dtype", "float32", z["dir"], " ".join(map(str, p))], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    want = plain.generate_greedy(z["w"], z["cfg"], p, 6)
    assert " ".join(map(str, want)) in r.stdout, (r.stdout, want)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": p[:20], "want": [0, 19]}, {"id": "b", "tokens": p[:3], "want": [2]}], "end": ["b"]},
             {"step": 1, "entries": [{"id": "a", "tokens": [p[20]], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": [p[21]], "want": [0]}], "end": ["a"]}]
    out = tmp_path / "logits"
    r = subprocess.run([sys.executable, os.path.join(REPO, "bin", "trace_run"), "--model", z["dir"], "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "23"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    V = z["cfg"]["vocab"]
    first = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V))
    last = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, V))
    assert not (out / "1.f32").exists()
    want = z["want"][2]
    assert rel_err(first, torch.stack([want[0], want[19], want[2]])) < TOL["float32"]
    assert rel_err(last, want[21:22]) < TOL["float32"]


# ---------------------------------------------------------------------------------------------
# the new parts in a design of another arrangement
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
def test_the_new_parts_serve_another_design(dtype):
    """A model that is none of the designs, from the registry's parts alone: the state-space mixer without a bias
    on its convolution next to the older attention with SwiGLU, experts with plain relu and no shared one behind
    head-wise attention that has a window without kept tokens (a ring of pages), biases AND the norm per head,
    and a plain ungated feed-forward."""
    from torchless_rs_amd.engine import Engine, SeqInput
    from torchless_rs_amd.engine.model import Model
    from torchless_rs_amd.parts import LayerSpec, ModelSpec, PartSpec
    from torchless_rs_amd.parts.base import Run
    from torchless_rs_amd.weights import TensorDict, random_tensors
    H, V, eps, d = 64, 70, 1e-5, 16
    rms = PartSpec("rmsnorm", {"size": H, "eps": eps})
    pre = PartSpec("pre_norm", {"mixer_norm_name": "n1.", "ffn_norm_name": "n2."})
    m_ssm = dict(heads=4, vdim=8, state=12, groups=2, conv=3, norm_groups=1)
    layers = [
        LayerSpec(prefix="h.0.", mixer=PartSpec("state_space", {
            "hidden_size": H, "n_heads": 4, "head_dim": 8, "state_size": 12, "groups": 2, "conv_taps": 3, "norm_groups": 1,
            "norm_eps": eps, "conv_bias": False}), ffn=PartSpec("swiglu", {"hidden_size": H, "intermediate_size": 96}),
            mixer_norm=rms, ffn_norm=rms, block=pre),
        LayerSpec(prefix="h.1.", mixer=PartSpec("attention", {"hidden_size": H, "n_heads": 4, "n_kv_heads": 2, "head_dim": d,
                                                               "position": PartSpec("rotary", {"head_dim": d, "theta": 100.0})}),
                  ffn=PartSpec("routed_experts", {"hidden_size": H, "n_experts": 6, "top": 2, "expert_size": 24, "activation": "relu"}),
                  mixer_norm=rms, ffn_norm=rms, block=pre),
        LayerSpec(prefix="h.2.", mixer=PartSpec("headwise_attention", {
            "hidden_size": H, "n_heads": 4, "n_kv_heads": 2, "head_dim": d, "v_head_dim": 24, "scale": 0.25, "bias": True,
            "head_norm_eps": eps, "window": 20}), ffn=PartSpec("plain", {"hidden_size": H, "intermediate_size": 40, "activation": "relu"}),
            mixer_norm=rms, ffn_norm=rms, block=pre),
    ]
    spec = ModelSpec(hidden_size=H, vocab_size=V, embedding=PartSpec("tokens", {"vocab_size": V, "hidden_size": H}),
                     embedding_prefix="model.", layers=layers, schedule=[Run(0), Run(1), Run(2)], final_norm=rms,
                     final_norm_prefix="model.norm.", head=PartSpec("linear", {"vocab_size": V, "hidden_size": H}),
                     head_prefix="lm_head.")
    w = random_tensors(spec.weight_specs(), seed=8, std=0.2, norm_std=0.1, dtype=torch.bfloat16)
    W = {k: v.double().cpu() for k, v in w.items()}
    ids = some_prompts(V, [45], seed=9)[0]
    n = len(ids)
    pos = torch.arange(n)

    def norm(name, t):
        return plain.rms(t, eps, W[name])

    x = W["model.embed_tokens.weight"][ids]
    Wz = dict(W, **{"h.0.mix.conv.b": torch.zeros(32 + 2 * 24, dtype=torch.float64)})
    x = x + plain.state_space(norm("h.0.n1.weight", x), Wz, "h.0.mix.", m_ssm, eps)
    y = norm("h.0.n2.weight", x)
    x = x + (plain.silu(y @ W["h.0.mlp.gate_proj.weight"].T) * (y @ W["h.0.mlp.up_proj.weight"].T)) @ W["h.0.mlp.down_proj.weight"].T
    y = norm("h.1.n1.weight", x)
    q, k, v = (y @ W[f"h.1.self_attn.{t}_proj.weight"].T for t in "qkv")
    margins = []
    q, k = q.view(n, 4, d), k.view(n, 2, d)
    q, k = plain.rotate_halves(q, pos, 100.0, d), plain.rotate_halves(k, pos, 100.0, d)
    a = plain.attention_core(q, k, v.view(n, 2, d), {"heads": 4, "kv_heads": 2, "scale": d ** -0.5}, plain.visible(n), False)
    x = x + a @ W["h.1.self_attn.o_proj.weight"].T
    y = norm("h.1.n2.weight", x)
    chosen, weight = plain.route(y, W, "h.1.mlp.", {"experts": 6, "top": 2}, margins)
    out = torch.zeros_like(x)
    for t in range(n):
        for e, s in zip(chosen[t].tolist(), weight[t]):
            out[t] += s * (torch.relu(y[t] @ W[f"h.1.mlp.e{e}.up"].T) @ W[f"h.1.mlp.e{e}.down"].T)
    x = x + out
    y = norm("h.2.n1.weight", x)
    q = plain.rms((y @ W["h.2.mix.q"].T + W["h.2.mix.q.b"]).view(n, 4, d), eps, W["h.2.mix.q.norm"])
    k = plain.rms((y @ W["h.2.mix.k"].T + W["h.2.mix.k.b"]).view(n, 2, d), eps, W["h.2.mix.k.norm"])
    v = (y @ W["h.2.mix.v"].T + W["h.2.mix.v.b"]).view(n, 2, 24)
    a = plain.attention_core(q, k, v, {"heads": 4, "kv_heads": 2, "scale": 0.25}, plain.visible(n, 20, 0), False)
    x = x + a @ W["h.2.mix.o"].T + W["h.2.mix.o.b"]
    y = norm("h.2.n2.weight", x)
    x = x + torch.relu(y @ W["h.2.mlp.up"].T) @ W["h.2.mlp.down"].T
    want = norm("model.norm.weight", x) @ W["lm_head.weight"].T
    model = Model(spec, None, TORCH[dtype], torch.device("cuda:0"))
    model.load_weights(TensorDict(w))
    eng = Engine(model, max_tokens=256)
    s = eng.alloc()
    got = [eng.step([SeqInput(s, ids[:30], list(range(30)))]).clone()]
    got += [eng.step([SeqInput(s, [t], [0])]).clone() for t in ids[30:]]
    eng.free(s)
    close(torch.cat(got), want, dtype, "a prompt and decoding", margins[0])
    s = eng.alloc()
    got = [eng.step([SeqInput(s, ids[at:at + 7], list(range(len(ids[at:at + 7]))))]).clone() for at in range(0, n, 7)]
    eng.free(s)
    close(torch.cat(got), want, dtype, "the same in portions of seven", margins[0])
    eng.close()
