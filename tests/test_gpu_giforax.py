"""Giforax on the GPU against the plain implementation of `plain_giforax.py`: every new mechanism alone
(layer norms with a bias and the fused pair of them, the weighted sum of the stream's versions, the gated
recurrence both ways through a step, the logistic router, gated experts with the weight on their input, the
norm of q and k after the rotation, attention with logistic weights inside chunks, with keys made to stand
out at every edge), then whole models of the tests' own sizes through the engine: whole prompts, the stream
after every layer, decoding token by token, portions down to two tokens, unequal batches, slots, pages and
state blocks used again, long decoding, and greedy generation through the entry point."""
import copy
import json
import os
import subprocess
import sys
import types

import numpy as np
import pytest
import torch

import plain_giforax as plain
from test_giforax_config import MIXED, attn, gru, layer, model, moe
from test_gpu_fanitar import Sequence
from test_gpu_sozetar import some_prompts, write_model
from util import rel_err, rms_err

pytestmark = pytest.mark.gpu
REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 3e-5, "bfloat16": 6e-2}
RMS = {"float32": 1e-5, "bfloat16": 3.5e-2}
# a router's choice made by less than this (the gap of the two experts' products as a share of the row's) may fall
# the other way under rounding
MARGIN = {"float32": 1e-4, "bfloat16": 3e-2}

# heads that the matrix cores take (64, 128, 96 with values as wide), chunks that are no multiple of a page, a reader
# of a layer that is not the first, many experts
CORES = model(256, 128, 1e-6, 1.3, [
    layer(gru(256), moe(16, 2, 32, 1.5, shared=(64, 1.0))),
    layer(attn(4, 2, 64, 64, 0.125, rot=(10000.0, 32), chunk=100), moe(24, 3, 32, 2.0, shared=(64, 2.0))),
    layer(attn(2, 1, 128, 128, 0.09, rot=(500000.0, 128), chunk=200), None),
    layer(attn(8, 2, 64, 64, 0.11, rot=(10000.0, 32), chunk=130, kv_from=1), moe(8, 1, 64, 1.0)),
    layer(attn(6, 6, 96, 96, 0.1, rot=(100.0, 48), chunk=70), moe(4, 4, 32, 1.5)),
])
# what a model may happen to make 1 or leave out: one head, one expert of which one is used, top = experts, a chunk
# of one (a position sees itself alone), no mask, no rotation, no shared expert, a recurrence of one channel
ONES = model(96, 32, 1e-4, 1.0, [
    layer(attn(1, 1, 16, 16, 0.25, chunk=1), moe(1, 1, 16, 1.0)),
    layer(gru(1), moe(4, 4, 8, 0.5)),
    layer(attn(2, 2, 8, 8, 0.35), moe(6, 2, 8, 3.0, shared=(8, 1.0))),
    layer(attn(2, 2, 8, 8, 0.3, rot=(50.0, 8), chunk=2, kv_from=2), None),
    layer(gru(16), None),
])
# sizes that no kernel's fast way takes: a width that is no multiple of 4, heads of 12 and 20, three heads, an odd
# vocabulary, a recurrence of 33 channels, five experts of 12
ODD = model(131, 102, 1e-5, 0.4, [
    layer(gru(33), moe(5, 2, 12, 1.5, shared=(10, 1.0))),
    layer(attn(3, 3, 12, 20, 0.29, rot=(300.0, 6), chunk=33), moe(9, 3, 10, 2.0)),
    layer(attn(6, 3, 20, 20, 0.2, rot=(20.0, 20), chunk=65), None),
    layer(attn(3, 3, 12, 20, 0.3, rot=(300.0, 6), chunk=129, kv_from=1), moe(3, 1, 14, 1.0, shared=(6, 0.5))),
])
CONFIGS = {"mixed": MIXED, "cores": CORES, "ones": ONES, "odd": ODD}
LENGTHS = {"mixed": [1, 7, 23, 150], "cores": [5, 64, 129, 330], "ones": [2, 65, 130, 200], "odd": [4, 33, 67, 140]}
NAMES = list(CONFIGS)


def dev(t, dtype=None):
    return t.to("cuda", dtype) if dtype is not None else t.to("cuda")


def step_ctx(dtype, **kw):
    from torchless_rs_amd.parts.base import Workspace
    return types.SimpleNamespace(pending=None, prenormed=None, norm_ahead=None, row_factor=None, dtype=TORCH[dtype],
                                 workspace=Workspace(torch.device("cuda")), host={}, **kw)


# ---------------------------------------------------------------------------------------------
# norms and the stream
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [30, 100, 320, 2052, 8200])
def test_layer_norms_with_a_bias_alone_into_the_stream_and_two_in_one_pass(dtype, H):
    from torchless_rs_amd.parts.norms import LayerNorm
    g = torch.Generator().manual_seed(H)
    n = 5
    z = torch.randn(n, H, generator=g) * 3 + 100.0            # a row far from zero: the variance is of the deviations
    x = torch.randn(n, H, generator=g)
    norms = []
    for i in range(2):
        ln = LayerNorm(H, 1e-5 * (i + 1), name="", bias_name=".b")
        assert set(ln.weight_specs()) == {"", ".b"}
        ln.load({"": dev(1 + 0.3 * torch.randn(H, generator=g)), ".b": dev(torch.randn(H, generator=g))}, TORCH[dtype])
        norms.append(ln)
    a, b = norms
    ctx = step_ctx(dtype)
    want_a = plain.layer_norm(z.double(), a.eps, a.weight.double().cpu(), a.beta.double().cpu())
    out = torch.empty(n, H, dtype=TORCH[dtype], device="cuda")
    a.forward(ctx, dev(z), out)
    tol = 1e-5 if dtype == "float32" else 1e-2
    assert rel_err(out, want_a) < tol
    # into the stream, the next norm on the way (rows that the kernel holds in registers) or by itself
    bias = torch.randn(H, generator=g)
    want_x = x.double() + plain.layer_norm(z.double() + bias.double(), a.eps, a.weight.double().cpu(), a.beta.double().cpu())
    want_y = plain.layer_norm(want_x, b.eps, b.weight.double().cpu(), b.beta.double().cpu())
    for then in (None, (b, out)):
        xs = dev(x.clone())
        ctx.prenormed = None
        a.add_to(ctx, dev(z.clone()), xs, bias=dev(bias), then=then)
        assert rel_err(xs, want_x) < 1e-5
        if then is not None and H % 4 == 0 and H <= 8192:
            assert ctx.prenormed is not None and ctx.prenormed[0] is b
            assert rel_err(out, want_y) < tol
        else:
            assert ctx.prenormed is None


def test_the_weighted_sum_of_the_streams_versions():
    from torchless_rs_amd.parts.stream_mix import DepthAverage
    g = torch.Generator().manual_seed(4)
    for n, H in ((3, 10), (7, 64), (1, 33)):
        T = 5
        part = DepthAverage(H, [f"w{t}" for t in range(1, T + 1)])
        assert {k: v.shape for k, v in part.weight_specs().items()} == {f"w{t}": (t + 1,) for t in range(1, T + 1)}
        coef = {f"w{t}": torch.randn(t + 1, generator=g) for t in range(1, T + 1)}
        part.load({k: dev(v) for k, v in coef.items()}, torch.float32)
        ctx = step_ctx("float32")
        X = [torch.randn(n, H, generator=g) for _ in range(T + 1)]
        for t in range(T + 1):
            x = dev(X[t].clone())
            part.forward(ctx, x, None, t)
            want = X[0].double() if t == 0 else sum(coef[f"w{t}"][j].double() * X[j].double() for j in range(t + 1))
            assert rel_err(x, want) < 1e-6, (n, H, t)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [30, 64, 2052])
def test_the_weighted_sum_on_the_way_from_one_norm_to_the_next(dtype, H):
    """x += norm(z); the new x is kept as version t and replaced by the weighted sum of the versions; the next norm
    reads the sum: in one kernel where the row fits it, step by step where not, with the same results."""
    from torchless_rs_amd.parts.norms import LayerNorm
    g = torch.Generator().manual_seed(H + 1)
    n, T = 6, 3
    norms = []
    for i in range(2):
        ln = LayerNorm(H, 1e-5, name="", bias_name=".b")
        ln.load({"": dev(1 + 0.3 * torch.randn(H, generator=g)), ".b": dev(torch.randn(H, generator=g))}, TORCH[dtype])
        norms.append(ln)
    a, b = norms
    versions = torch.randn(T + 1, n, H, generator=g)
    coef = torch.randn(T + 1, generator=g)
    z, x = torch.randn(n, H, generator=g) * 2, torch.randn(n, H, generator=g)
    new = x.double() + plain.layer_norm(z.double(), a.eps, a.weight.double().cpu(), a.beta.double().cpu())
    want_x = coef[T].double() * new + sum(coef[j].double() * versions[j].double() for j in range(T))
    want_y = plain.layer_norm(want_x, b.eps, b.weight.double().cpu(), b.beta.double().cpu())
    for then in (None, "next"):
        kept = dev(versions.clone())
        kept[T] = float("nan")
        xs, out = dev(x.clone()), torch.empty(n, H, dtype=TORCH[dtype], device="cuda")
        ctx = step_ctx(dtype)
        a.add_to(ctx, dev(z.clone()), xs, then=(b, out) if then else None, between=(kept, dev(coef), T))
        assert rel_err(xs, want_x) < 1e-5 and rel_err(kept[T], new) < 1e-5
        if then and H % 4 == 0:
            assert ctx.prenormed[0] is b and rel_err(out, want_y) < (1e-5 if dtype == "float32" else 1e-2)
        else:
            assert ctx.prenormed is None


# ---------------------------------------------------------------------------------------------
# the gated recurrence
# ---------------------------------------------------------------------------------------------

def plain_recurrence(proj, bz, bx, S):
    """proj [T, 3 W] = [a | b | g] of one sequence, in float64, from the state S."""
    W = proj.shape[1] // 3
    z = torch.sigmoid(proj[:, :W] + bz)
    c = plain.candidate(proj[:, W:2 * W] + bx)
    gate = proj[:, 2 * W:]
    out = []
    for t in range(proj.shape[0]):
        S = (1 - z[t]) * S + z[t] * c[t]
        out.append(S * gate[t] * torch.sigmoid(gate[t]))
    return torch.stack(out), S


def recurrence_steps(dtype, W, proj, bz, bx, lengths, cuts, slots, by_runs, n_slots=7):
    """The rows of several sequences (proj [sum lengths, 3 W], sequence after sequence) through the kernels in
    steps that bring `cuts[i]` rows of every sequence that still has some; returns out per sequence and the states."""
    from torchless_rs_amd.kernels import ops
    state = torch.full((n_slots, W + 3), float("nan"), device="cuda")[:, :W]      # rows strided, as a block of more may be
    for s in slots:
        state[s].zero_()
    starts = np.concatenate([[0], np.cumsum(lengths)])
    done = [0] * len(lengths)
    outs = [[] for _ in lengths]
    chunk = ops.gated_recurrence_chunk()
    for cut in cuts:
        live = [i for i in range(len(lengths)) if done[i] < lengths[i]]
        if not live:
            break
        take = [min(cut, lengths[i] - done[i]) for i in live]
        rows = torch.cat([proj[starts[i] + done[i]: starts[i] + done[i] + k] for i, k in zip(live, take)])
        cu = torch.tensor(np.concatenate([[0], np.cumsum(take)]), dtype=torch.int32, device="cuda")
        sl = torch.tensor([slots[i] for i in live], dtype=torch.int32, device="cuda")
        out = torch.empty(rows.shape[0], W, dtype=TORCH[dtype], device="cuda")
        runs = sum(-(-k // chunk) for k in take) if by_runs else 0
        scratch = torch.empty((2 * runs + len(live)) * W, device="cuda") if runs else None
        ops.gated_recurrence(dev(rows.float().contiguous()), dev(bz.float()), dev(bx.float()), state, cu, sl, out, runs, scratch)
        at = 0
        for i, k in zip(live, take):
            outs[i].append(out[at:at + k].clone())
            at += k
            done[i] += k
    return [torch.cat(o) for o in outs], state


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("by_runs", [False, True])
@pytest.mark.parametrize("W", [1, 33, 80, 300])
def test_the_gated_recurrence_in_steps_of_any_size(dtype, by_runs, W):
    g = torch.Generator().manual_seed(W)
    lengths, slots = [1, 70, 200], [5, 0, 3]
    proj = torch.randn(sum(lengths), 3 * W, generator=g, dtype=torch.float64) * 2
    proj = proj.float().double()
    bz, bx = torch.randn(W, generator=g).double(), torch.randn(W, generator=g).double()
    want, at = [], 0
    for L in lengths:
        want.append(plain_recurrence(proj[at:at + L], bz, bx, torch.zeros(W, dtype=torch.float64)))
        at += L
    tol = 2e-6 if dtype == "float32" else 6e-3
    for cuts in ([200], [64, 64, 64, 64], [1] * 3 + [65] + [2] * 80, [63, 1, 1, 128, 7]):
        got, state = recurrence_steps(dtype, W, proj, bz, bx, lengths, cuts, slots, by_runs)
        for i, L in enumerate(lengths):
            assert rel_err(got[i], want[i][0]) < tol, (cuts, i)
            assert rel_err(state[slots[i]], want[i][1]) < 2e-6, (cuts, i, "state")
        assert torch.isnan(state[[1, 2, 4, 6]]).all()           # nobody else's block was touched


@pytest.mark.parametrize("by_runs", [False, True])
def test_a_state_that_is_carried_far_and_one_that_is_forgotten(by_runs):
    """Channel 0 nearly keeps its state (z of 1e-4): what the first row wrote still shows after 600 rows, in steps of
    any size; channel 1 forgets at once (z of nearly 1)."""
    W, L = 2, 600
    proj = torch.zeros(L, 3 * W, dtype=torch.float64)
    proj[:, 0], proj[:, 1] = -9.2, 12.0                        # a: z = 1e-4 and 1 - 6e-6
    proj[:, 2:4] = -30.0                                       # b: candidates of 1e-13
    proj[0, 0], proj[0, 2] = 12.0, 40.0                        # the first row writes 40.5 into channel 0
    proj[0, 3] = 7.0
    proj[:, 4:] = 3.0
    zero = torch.zeros(W, dtype=torch.float64)
    want, _ = plain_recurrence(proj, zero, zero, zero)
    assert want[-1, 0] > 30 and want[-1, 1] < 1e-9
    for cuts in ([600], [1] * 40 + [200, 360], [300, 300]):
        got, _ = recurrence_steps("float32", W, proj, zero, zero, [L], cuts, [2], by_runs)
        assert rel_err(got[0][:, 0], want[:, 0]) < 1e-5 and float(got[0][-1, 1].abs()) < 1e-9, cuts


# ---------------------------------------------------------------------------------------------
# the routed feed-forward
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("in_dtype", DTYPES)
@pytest.mark.parametrize("E, top", [(8, 2), (10, 1), (1, 1), (4, 4), (40, 7)])
def test_the_router_with_a_score_of_its_own_for_every_expert(in_dtype, E, top):
    from torchless_rs_amd.kernels import ops
    g = torch.Generator().manual_seed(E * 10 + top)
    n, W = 37, 48
    h = torch.randn(n, W, generator=g).to(TORCH[in_dtype])
    wr = torch.randn(E, W, generator=g) * 0.5
    weights = torch.empty(n, E, device="cuda")
    chosen = torch.empty(n, top, dtype=torch.int32, device="cuda")
    ops.route(dev(h), dev(wr), 0, 0, top, weights, chosen, logistic=True)
    margins = []
    want = plain.route(h.double(), {"router": wr.double()}, "", {"experts": E, "top": top}, margins)
    sure = margins[0] > (1e-5 if in_dtype == "float32" else 1e-2)
    assert rel_err(weights[sure.cuda()], want[sure]) < 1e-5
    assert ((weights != 0).sum(dim=1) == top).all()
    picked = torch.gather(weights, 1, chosen.long())
    assert (picked[:, :-1] >= picked[:, 1:]).all() and (picked > 0).all()      # the best first


def experts_part(dtype, H, E, top, ff, limit, shared, on, seed):
    from torchless_rs_amd.parts.ffn_routed import RoutedExperts
    mlp = moe(E, top, ff, limit, shared=shared)
    cfg = model(8, H, 1e-5, 1.0, [layer(gru(1), mlp)])
    w = {k[len("l0."):]: v for k, v in plain.random_weights(cfg, seed, gain=3.0).items() if k.startswith("l0.mlp.")}
    part = RoutedExperts(H, E, top, ff, shared_size=shared[0] if shared else None, score="sigmoid", gated=True,
                         activation="swish_clamped", activation_constants={"limit": limit, "alpha": 1.702, "shift": 1.0},
                         shared_limit=shared[1] if shared else None, weight_on=on)
    assert set(part.weight_specs()) == set(w)
    part.load({k: dev(v if dtype == "bfloat16" else v.float()) for k, v in w.items()}, TORCH[dtype])
    return part, mlp, {k: v.double() for k, v in w.items()}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, E, top, ff, limit, shared", [(64, 8, 2, 32, 1.5, (48, 0.75)), (100, 5, 2, 12, 1.0, (10, 2.0)),
                                                          (32, 1, 1, 16, 0.5, None), (48, 10, 1, 8, 2.0, (8, 2.0)), (40, 4, 4, 8, 1.0, None)])
def test_gated_experts_with_the_weight_on_their_input(dtype, H, E, top, ff, limit, shared):
    """The chosen experts alone (few rows), all experts side by side (more rows) and, in bfloat16, expert by expert over
    each expert's own rows, against the plain mixture; clamps that bite (weights with a gain of 3), a shared expert with
    a limit of its own."""
    from torchless_rs_amd.parts import ffn_routed
    part, mlp, w = experts_part(dtype, H, E, top, ff, limit, shared, "input", seed=H + E)
    g = torch.Generator().manual_seed(E)
    tol = 2e-5 if dtype == "float32" else 2.5e-2
    ways = set()
    for n in (1, 3, 40, 200):
        y = (torch.randn(n, H, generator=g) * 1.5).to(TORCH[dtype])
        margins = []
        want = plain.routed_ff(y.double(), w, "mlp.", mlp, margins)
        sure = margins[0] > MARGIN[dtype]
        ctx = step_ctx(dtype)
        out = torch.empty(n, H, device="cuda")
        ways.add("rows" if part.few_rows(dev(y)) else "wide")
        part.produce(ctx, dev(y), out)
        assert rel_err(out[sure.cuda()], want[sure]) < tol, (n, "stored")
        x0 = torch.randn(n, H, generator=g)
        x = dev(x0.clone())
        part.forward(ctx, dev(y), x)
        if ctx.pending is not None:
            x += ctx.pending.sum(dim=0)
        assert rel_err(x[sure.cuda()], (x0.double() + want)[sure]) < tol, (n, "added")
        if dtype == "bfloat16" and n == 200 and H % 8 == 0:
            ffn_routed_bar, ffn_routed.GROUPED_ROWS_PER_EXPERT = ffn_routed.GROUPED_ROWS_PER_EXPERT, 0
            try:
                part._grouped(ctx, dev(y), out, False)
            finally:
                ffn_routed.GROUPED_ROWS_PER_EXPERT = ffn_routed_bar
            assert rel_err(out[sure.cuda()], want[sure]) < tol, (n, "expert by expert")
    assert ways == {"rows", "wide"}


def test_the_weight_on_the_input_is_not_the_weight_on_the_output():
    """With clamps that bite the two differ; the kernels follow the parameter."""
    H, E, top, ff = 32, 4, 2, 16
    g = torch.Generator().manual_seed(1)
    y = torch.randn(30, H, generator=g) * 2
    outs = {}
    for on in ("input", "output"):
        part, mlp, w = experts_part("float32", H, E, top, ff, 0.5, None, on, seed=9)
        out = torch.empty(30, H, device="cuda")
        part.produce(step_ctx("float32"), dev(y), out)
        outs[on] = out.double().cpu()
    want_in = plain.routed_ff(y.double(), w, "mlp.", mlp)
    wt = plain.route(y.double(), w, "mlp.", mlp["router"])
    want_out = sum(wt[:, e:e + 1] * plain.gated_expert(y.double(), w, f"mlp.e{e}.", 0.5) for e in range(E))
    assert rel_err(outs["input"], want_in) < 2e-5 and rel_err(outs["output"], want_out) < 2e-5
    assert rel_err(want_in, want_out) > 1e-2


# ---------------------------------------------------------------------------------------------
# attention
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq, nkv, dk, dv, dims", [(4, 2, 32, 16, 16), (3, 3, 12, 20, 6), (2, 1, 64, 64, 64), (1, 1, 16, 16, 0), (4, 0, 32, 16, 8)])
def test_the_norm_of_q_and_k_after_the_rotation(dtype, nq, nkv, dk, dv, dims):
    """A row [q | k | v | g] head by head: rotation of the first channels, then every head over its root mean square
    with no weight; the gate per head; nkv 0: a row of [q | g] alone."""
    from torchless_rs_amd.kernels import ops
    g = torch.Generator().manual_seed(dk)
    n, eps, base = 9, 1e-3, 77.0
    pos = torch.tensor([0, 1, 2, 63, 64, 65, 500, 4000, 7], dtype=torch.int32)
    proj = torch.randn(n, nq * dk + nkv * (dk + dv) + nq, generator=g) * 2
    inv = torch.pow(torch.tensor(base, dtype=torch.float64), -2.0 * torch.arange(dims // 2, dtype=torch.float64) / max(dims, 1)).float()
    rot = ops.Rotation(dev(inv), dims) if dims else ops.NO_ROTATION
    q = torch.empty(n, nq, dk, dtype=TORCH[dtype], device="cuda")
    k = torch.empty(n, nkv, dk, dtype=TORCH[dtype], device="cuda") if nkv else None
    v = torch.empty(n, nkv, dv, dtype=TORCH[dtype], device="cuda") if nkv else None
    gate = torch.empty(n, nq, device="cuda")
    ops.head_prepare(dev(proj), dev(pos), rot, ops.HeadTerms(eps=eps, unit_norm=True), nq, nkv, dk, dv, nq, q, k, v, gate)
    p64 = proj.double()
    tol = 1e-4 if dtype == "float32" else 5e-3        # (an angle of 4,000 radians in 32 bits is good to 2e-4)
    want_q = plain.unit_rms(plain.rotate_halves(p64[:, :nq * dk].view(n, nq, dk), pos, base, dims), eps)
    assert rel_err(q, want_q) < tol
    if nkv:
        want_k = plain.unit_rms(plain.rotate_halves(p64[:, nq * dk:(nq + nkv) * dk].view(n, nkv, dk), pos, base, dims), eps)
        assert rel_err(k, want_k) < tol
        assert rel_err(v, p64[:, (nq + nkv) * dk:(nq + nkv) * dk + nkv * dv].view(n, nkv, dv)) < tol
    assert rel_err(gate, torch.sigmoid(p64[:, -nq:])) < 2e-6


def logistic_steps(dtype, nq, nkv, dk, dv, chunk, bias, gate, q, k, v, cuts, scale):
    """q [L, nq, dk], k [L, nkv, dk], v [L, nkv, dv]: through `head_prepare` (nothing but the split) and
    `attend_and_commit` with logistic weights in steps of `cuts` rows over one sequence's pages (a ring of the
    chunk's pages)."""
    from torchless_rs_amd.kernels import ops
    from torchless_rs_amd.parts.attention_scored import attend_and_commit
    seq = Sequence(dtype, nkv, dk, dv, chunk)
    terms = ops.ScoreTerms(scale, chunk=chunk, logistic=True, score_bias=dev(bias.float()))
    outs, at = [], 0
    for n in cuts:
        ctx, run = seq.step(n)
        proj = dev(torch.cat([q[at:at + n].reshape(n, -1), k[at:at + n].reshape(n, -1), v[at:at + n].reshape(n, -1)], dim=1).float().contiguous())
        qs = torch.empty(n, nq, dk, dtype=seq.dt, device="cuda")
        att = torch.empty(n, nq, dv, dtype=seq.dt, device="cuda")
        if n == 1:
            ops.head_prepare(proj, ctx.row_pos, ops.NO_ROTATION, ops.HeadTerms(), nq, nkv, dk, dv, 0, qs, None, None, None,
                             table=seq.table, ring_pages=seq.ring, pages=seq.pages)
            ks = vs = None
        else:
            ks = torch.empty(n, nkv, dk, dtype=seq.dt, device="cuda")
            vs = torch.empty(n, nkv, dv, dtype=seq.dt, device="cuda")
            ops.head_prepare(proj, ctx.row_pos, ops.NO_ROTATION, ops.HeadTerms(), nq, nkv, dk, dv, 0, qs, ks, vs, None)
        attend_and_commit(ctx, run, qs, ks, vs, nkv, dk, dv, terms, dev(gate[at:at + n].float().contiguous()), att)
        outs.append(att.clone())
        at += n
    return torch.cat(outs)


def plain_logistic(q, k, v, nq, nkv, scale, chunk, bias, gate):
    L = q.shape[0]
    rep = nq // nkv
    kh = k.double().repeat_interleave(rep, dim=1).transpose(0, 1)
    vh = v.double().repeat_interleave(rep, dim=1).transpose(0, 1)
    s = (q.double().transpose(0, 1) @ kh.transpose(1, 2)) * scale + bias.double()[:, None, None]
    a = torch.sigmoid(s) * plain.same_chunk(torch.arange(L), chunk)[None]
    return (a @ vh).transpose(0, 1) * gate.double()[:, :, None]


ATT_TOL = {"float32": 2e-5, "bfloat16": 1.2e-2}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk", [1, 2, 63, 64, 65, 100, 129, 200])
@pytest.mark.parametrize("dk, dv", [(16, 8), (48, 48), (64, 64), (96, 96)])
def test_a_key_just_inside_and_just_outside_a_chunk(dtype, chunk, dk, dv):
    """Every key's own weight is a thousandth (a bias of -7) but for the keys at both sides of every chunk's edge, the
    last of a chunk and the first of the next, which every query scores at +9: a row's result is the values of those
    of the two that it sees, and a mask that is one position off shows at once.  In one step, in portions that start
    and end at and beside the edges, and token by token."""
    nq, nkv, L, scale = 4, 2, 300, 0.5
    g = torch.Generator().manual_seed(chunk)
    q = torch.randn(L, nq, dk, generator=g) * 0.2
    k = torch.randn(L, nkv, dk, generator=g) * 0.2
    v = torch.randn(L, nkv, dv, generator=g)
    u = torch.zeros(dk)
    u[0] = 1.0
    q[:, :, 0] = 4.0
    for e in range(chunk, L, chunk):
        k[e - 1, :, :] = 8.0 * u                      # the last key of a chunk: 4 * 8 * 0.5 - 7 = +9
        k[e, :, :] = 8.0 * u                          # the first key of the next
    bias = torch.full((nq,), -7.0) + 0.1 * torch.randn(nq, generator=g)
    gate = torch.rand(L, nq, generator=g)
    rounded = [t.to(TORCH[dtype]) for t in (q, k, v)]
    want = plain_logistic(*rounded, nq, nkv, scale, chunk, bias, gate)
    edge = chunk if chunk > 2 else 64
    for cuts in ([L], [edge - 1, 1, 1, 1, edge - 2, 2] + [1] * 5 + [L], [50] + [1] * 250, [2] * 150):
        cuts = [c for c in cuts if c > 0]
        left, use = L, []
        for c in cuts:
            if left <= 0:
                break
            use.append(min(c, left))
            left -= use[-1]
        got = logistic_steps(dtype, nq, nkv, dk, dv, chunk, bias, gate, *rounded, use, scale)
        assert rel_err(got, want) < ATT_TOL[dtype], (chunk, use[:8])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dk, dv", [(32, 16), (64, 64), (80, 80), (128, 128), (256, 256)])
def test_a_far_key_and_the_first_tokens(dtype, dk, dv):
    """No chunks (and one chunk of 1,000): position 3 is the one loud key among 700, seen from everywhere behind it, in a
    prompt, in portions and by single tokens."""
    nq, nkv, L, scale = 2, 1, 700, 0.5
    g = torch.Generator().manual_seed(dk)
    q = torch.randn(L, nq, dk, generator=g) * 0.2
    k = torch.randn(L, nkv, dk, generator=g) * 0.2
    v = torch.randn(L, nkv, dv, generator=g)
    q[:, :, 1] = 4.0
    k[3, :, :] = 0.0
    k[3, :, 1] = 8.0
    bias = torch.tensor([-7.0, -6.5])
    gate = torch.ones(L, nq)
    rounded = [t.to(TORCH[dtype]) for t in (q, k, v)]
    for chunk in (None, 1000):
        want = plain_logistic(*rounded, nq, nkv, scale, chunk, bias, gate)
        assert float(want[600:, 0].abs().mean()) > 0.3
        for cuts in ([L], [1, 1, 1, 1, 1, 295, 390] + [1] * 10, [640] + [1] * 60):
            got = logistic_steps(dtype, nq, nkv, dk, dv, chunk, bias, gate, *rounded, cuts, scale)
            assert rel_err(got, want) < ATT_TOL[dtype], (chunk, cuts[:8])


def test_which_shapes_reach_the_matrix_cores():
    from torchless_rs_amd.kernels import ops
    assert ops.scored_on_matrix_cores(torch.bfloat16, 96, 96) and ops.scored_on_matrix_cores(torch.bfloat16, 64, 64)
    assert not ops.scored_on_matrix_cores(torch.bfloat16, 32, 16) and not ops.scored_on_matrix_cores(torch.float32, 64, 64)
    with pytest.raises(ops.KernelError):
        ops.ScoreTerms(1.0, sinks=torch.zeros(2), logistic=True)
    with pytest.raises(ops.KernelError):
        ops.ScoreTerms(1.0, score_bias=torch.zeros(2))
    assert ops.ScoreTerms(1.0, window=50, chunk=70).reach == 50 and ops.ScoreTerms(1.0, chunk=70).reach == 70


# ---------------------------------------------------------------------------------------------
# whole models through the engine
# ---------------------------------------------------------------------------------------------

def plain_run(w, cfg, ids):
    """Logits and, per row, the smallest difference of scores by which a router chose."""
    margins = []
    lg = plain.forward(w, cfg, ids, margins=margins)
    m = torch.stack(margins).min(dim=0).values if margins else torch.ones(len(ids), dtype=torch.float64)
    return lg, m


@pytest.fixture(scope="module")
def zoo(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("giforax")
    out = {}
    for i, name in enumerate(NAMES):
        cfg = copy.deepcopy(CONFIGS[name])
        w = plain.random_weights(cfg, seed=80 + i)
        ps = some_prompts(cfg["vocab"], LENGTHS[name], seed=31 + i)
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


def close(got, want, dtype, what, margin=None, tol=None, rms=None, reach=None):
    """Rows whose routers chose by a wide enough margin must agree (a choice made by a hair may fall the other
    way under the rounding of the router's input, and then the row is another function's).  In bfloat16 the
    stream that reaches a deep router is off by more than its input's rounding: a row in thirty may still fall
    the other way, and is then left out of the comparison of the others.  A row that fell the other way also
    leaves other keys and values behind, which the rows behind it in its chunk add to their sums at full weight
    (nothing is normalised): with `reach` (the longest chunk; rows of one sequence in order), a row that differs
    within that many rows behind an unsure one is left out too."""
    tol, rms = tol or TOL[dtype], rms or RMS[dtype]
    got = got.detach().double().cpu()
    if margin is not None:
        sure = margin > MARGIN[dtype]
        assert int(sure.sum()) * 2 >= len(sure) or len(sure) < 4, (what, "too few sure rows")
        if dtype == "bfloat16" and len(got):
            err = (got - want).abs().amax(dim=1) / want.abs().max()
            off = err > tol
            if reach:
                last_unsure = -10 ** 9
                for i in range(len(sure)):
                    if off[i] and sure[i] and i - last_unsure <= reach:
                        sure[i] = False
                    if not margin[i] > MARGIN[dtype]:
                        last_unsure = i
            off = off & sure
            assert int(off.sum()) <= max(1, int(sure.sum()) // 30), (what, "rows off", off.nonzero().flatten().tolist())
            sure = sure & ~off
        got, want = got[sure], want[sure]
    if not len(got):
        return
    assert rel_err(got, want) < tol, (what, rel_err(got, want))
    if rms is not False:
        assert rms_err(got, want) < rms, (what, rms_err(got, want))


def longest_chunk(cfg):
    sizes = [(l["mixer"].get("mask") or {}).get("size", 10 ** 6) for l in cfg["layers"] if l["type"] == "attention"]
    return max(sizes)


def test_the_right_parts_and_caches_are_chosen(zoo):
    from torchless_rs_amd.parts.attention_heads import HeadwiseAttentionMixer
    from torchless_rs_amd.parts.block import SandwichNormBlock
    from torchless_rs_amd.parts.ffn_routed import RoutedExperts
    from torchless_rs_amd.parts.norms import LayerNorm
    from torchless_rs_amd.parts.recurrence import GatedRecurrenceMixer
    eng = engine_for(zoo, "cores", "bfloat16")
    blocks = eng.model.blocks
    assert all(isinstance(b, SandwichNormBlock) and isinstance(b.mixer_out_norm, LayerNorm) and b.mixer_norm.beta is not None
               for b in blocks)
    assert [type(b.mixer) for b in blocks] == [GatedRecurrenceMixer] + [HeadwiseAttentionMixer] * 4
    assert isinstance(blocks[0].ffn, RoutedExperts) and blocks[0].ffn.gated and blocks[2].ffn is None
    assert sorted(eng.cache.state) == [0] and eng.cache.state[0].shape[1] == 256 and eng.cache.state[0].dtype == torch.float32
    a1, a3 = blocks[1].mixer, blocks[3].mixer
    assert a1.own_kv and not a3.own_kv and a3.kv_request() is None and a1.logistic and a1.head_gate and a1.chunk == 100
    assert eng.runs[3].kv_source == 1 and eng.runs[3].kv_group is eng.runs[1].kv_group and eng.runs[1].kv_read_later
    rings = sorted(g.ring_pages for g in eng.cache.groups)
    assert rings == [2, 3, 4]           # chunks of 70, 130 (the reader's, kept by the owner of 100) and 200 in pages of 64


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
@pytest.mark.parametrize("name", ["mixed", "odd", "cores"])
def test_the_stream_after_every_layer(zoo, name, dtype):
    from torchless_rs_amd.engine import Engine, SeqInput, load_model
    z = zoo[name]
    streams = []
    plain.forward(z["w"], z["cfg"], z["prompts"][2], streams=streams)
    model_ = load_model(z["dir"], dtype)
    eng = Engine(model_, max_tokens=256, use_graphs=False)
    seen = []
    for blk in model_.blocks[1:]:            # what a layer reads is the stream as the layer before and the sum left it
        inner = blk.forward

        def spy(ctx, run, x, *a, _inner=inner, **kw):
            seen.append(x.clone())
            _inner(ctx, run, x, *a, **kw)
        blk.forward = spy
    last = model_.final_norm.forward
    model_.final_norm.forward = lambda ctx, xs, y: (seen.append(xs.clone()), last(ctx, xs, y))[1]
    p = z["prompts"][2]
    s = eng.alloc()
    eng.step([SeqInput(s, p, list(range(len(p))))])
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
def test_long_decoding_past_every_chunk(zoo, name, dtype):
    """A short prompt, then 300 tokens one by one (through captured graphs): every chunk ends and a new one begins
    among decoded tokens, the rings of pages wrap, the recurrent state is carried 300 times."""
    from torchless_rs_amd.engine import SeqInput
    eng, z = engine_for(zoo, name, dtype), zoo[name]
    ids = some_prompts(z["cfg"]["vocab"], [310], seed=78)[0]
    want, m = plain_run(z["w"], z["cfg"], ids)
    s = eng.alloc()
    rows = [eng.step([SeqInput(s, ids[:10], list(range(10)))]).clone()]
    rows += [eng.step([SeqInput(s, [t], [0])]).clone() for t in ids[10:]]
    eng.free(s)
    close(torch.cat(rows), want, dtype, name, m, reach=longest_chunk(z["cfg"]))


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


def test_a_long_prompt_goes_by_runs_and_many_rows_expert_by_expert(zoo, monkeypatch):
    """A prompt of more rows than the framework's own products take, with the bar for sorting rows by expert taken
    down to the tests' sizes; the recurrence cut into runs of rows."""
    from torchless_rs_amd.engine import SeqInput
    from torchless_rs_amd.kernels import ops
    from torchless_rs_amd.parts import ffn_routed
    monkeypatch.setattr(ffn_routed, "GROUPED_ROWS_PER_EXPERT", 1)
    calls, runs = [], []
    inner = ffn_routed.RoutedExperts._grouped
    monkeypatch.setattr(ffn_routed.RoutedExperts, "_grouped", lambda self, *a: (calls.append(a[1].shape[0]), inner(self, *a))[1])
    scan = ops.gated_recurrence
    monkeypatch.setattr(ops, "gated_recurrence", lambda *a: (runs.append(a[7]), scan(*a))[1])
    for name in ("cores", "mixed"):
        eng, z = engine_for(zoo, name, "bfloat16"), zoo[name]
        p = z["prompts"][3]
        calls.clear()
        runs.clear()
        s = eng.alloc()
        got = eng.step([SeqInput(s, p, list(range(len(p))))]).clone()
        eng.free(s)
        assert calls and all(c == len(p) for c in calls), calls
        assert runs and all(r == -(-len(p) // ops.gated_recurrence_chunk()) for r in runs), runs
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
# configurations drawn at random
# ---------------------------------------------------------------------------------------------

def random_config(rng):
    """Any order of layers, any sizes: recurrences of 8 to 384 channels, heads of 16 to 128 with values as wide or not,
    one to four KV heads, none, half or all of a head rotated, no chunks or chunks of 17 to 256, readers of any earlier
    layer that owns keys (with more heads and another chunk), one to sixteen experts with or without a shared one."""
    width = rng.choice([64, 96, 128, 160, 256])
    layers, owners = [], []
    for i in range(rng.randint(3, 6)):
        if rng.random() < 0.3:
            mix = gru(rng.choice([8, 33, 64, 200, 384]))
        elif owners and rng.random() < 0.35:
            src = rng.choice(owners)
            m0 = layers[src]["mixer"]
            mix = attn(m0["kv_heads"] * rng.choice([1, 2, 4]), m0["kv_heads"], m0["dim"], m0["vdim"], rng.uniform(0.08, 0.3),
                       rot=(m0["rot"]["base"], m0["rot"]["dims"]) if "rot" in m0 else None,
                       chunk=rng.choice([None, 17, 64, 100, 200, 256]), kv_from=src)
        else:
            dim = rng.choice([16, 32, 48, 64, 96, 128])
            kv = rng.choice([1, 2, 4])
            dims = rng.choice([0, dim // 2, dim])
            mix = attn(kv * rng.choice([1, 2, 4]), kv, dim, dim if rng.random() < 0.7 else rng.choice([16, 24, 64]),
                       rng.uniform(0.08, 0.3), rot=(rng.choice([100.0, 10000.0, 5e5]), dims) if dims else None,
                       chunk=rng.choice([None, 17, 64, 100, 200, 256]))
            owners.append(i)
        f = None
        if rng.random() < 0.85:
            E = rng.choice([1, 2, 4, 8, 10, 16])
            f = moe(E, rng.randint(1, min(E, 4)), rng.choice([8, 16, 32, 64]), rng.choice([0.5, 1.5, 3.0]),
                    shared=(rng.choice([8, 32, 96]), rng.choice([0.5, 1.5])) if rng.random() < 0.7 else None)
        layers.append(layer(mix, f))
    return model(rng.choice([97, 256, 500]), width, rng.choice([1e-5, 1e-6]), rng.choice([0.5, 1.0, 2.0]), layers)


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(seed, tmp_path):
    """Float32 (where a router's choice falls the same way as in the plain implementation): whole prompts, a prompt
    with its last tokens one by one, and all of them in one batch that is decoded together."""
    import random
    from torchless_rs_amd.engine import Engine, SeqInput, load_model
    cfg = random_config(random.Random(seed))
    w = plain.random_weights(cfg, seed=100 + seed)
    ps = some_prompts(cfg["vocab"], [1, 37, 150, 420], seed=seed)
    runs = [plain_run(w, cfg, p) for p in ps]
    eng = Engine(load_model(write_model(str(tmp_path / "m"), cfg, w), "float32"), max_tokens=64 * 30, max_slots=8)
    tails = [0, 5, 20, 33]
    heads = [len(p) - t for p, t in zip(ps, tails)]
    for p, h, (want, m) in zip(ps, heads, runs):
        s = eng.alloc()
        got = eng.step([SeqInput(s, p, list(range(len(p))))]).clone()
        eng.free(s)
        close(got, want, "float32", (seed, len(p), "whole"), m)
        s = eng.alloc()
        rows = [eng.step([SeqInput(s, p[:h], list(range(h)))]).clone()] + [eng.step([SeqInput(s, [t], [0])]).clone() for t in p[h:]]
        eng.free(s)
        close(torch.cat(rows), want, "float32", (seed, len(p), "then decoded"), m)
    slots = [eng.alloc() for _ in ps]
    lg = eng.step([SeqInput(s, p[:h], list(range(h))) for s, p, h in zip(slots, ps, heads)])
    got, at = [], 0
    for h in heads:
        got.append([lg[at:at + h].clone()])
        at += h
    for step in range(max(tails)):
        live = [i for i in range(len(ps)) if step < tails[i]]
        lg = eng.step([SeqInput(slots[i], [ps[i][heads[i] + step]], [0]) for i in live]).clone()
        for r, i in enumerate(live):
            got[i].append(lg[r:r + 1])
    for s in slots:
        eng.free(s)
    for i, (want, m) in enumerate(runs):
        close(torch.cat(got[i]), want, "float32", (seed, i, "together"), m)
    eng.close()
