"""Lugetar on the GPU against the plain implementation (tests/plain_lugetar.py), in 32-bit and in
bfloat16: the kernels that the design added or widened, each against its equation (the norm
behind a sub-layer with its factor and the next norm in the same launch, the norm over the whole
query and key projection with rotation and values of their own, the delta rule with a decay per
key channel, the sum of two normed mixers, the logistic router within the best groups); each mixer
alone (a model of one layer, the stream behind it compared); weights made so that a fault would
show (a query aimed at a key just inside and just outside its chunk, at a key hundreds of
positions back, at a page's border, in prompts and while decoding token by token); then the
engine through the trace replayer (whole prompts, decoding token by token, portions down to two
tokens, mixed batches on few pages and four state slots that are used again), a batch against each
of its requests alone, long decoding, and greedy generation through the scheduler and the command
line."""

import copy
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import lugetar_tiny as T
import plain_lugetar as P
import traces

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
F64 = torch.float64
# Logits: root mean square of the difference (mean taken off) over that of the plain model's logits.
# In bfloat16 a position's limit is five times what rounding of the sub-layers' inputs alone does
# to the plain model there, where that is more (the engine also keeps queries, keys, values,
# probabilities and the activations inside a mixer in bfloat16).
TOL = {"float32": 2e-5, "bfloat16": 6e-2}
WORST = {"float32": 0.0, "bfloat16": 0.0}
# The aimed weights make large scores and one value far larger than the others: in bfloat16 a
# sharp softmax over such scores magnifies the rounding of queries and keys; a key that is wrongly
# seen or not seen moves the aimed rows by 0.3 and more (checked in each test).
AIMED_TOL = {"float32": 2e-5, "bfloat16": 0.12}


def rel(got, want):
    got, want = torch.as_tensor(got, dtype=F64), torch.as_tensor(want, dtype=F64)
    return float((got - want).norm() / want.norm().clamp_min(1e-30))


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}

    def get(name, seed=13, weights=None, tag=""):
        key = (name, seed, tag)
        if key not in made:
            d = tmp_path_factory.mktemp(f"lugetar_{name}_{seed}_{tag}")
            made[key] = T.write_model(str(d), T.CONFIGS[name], seed=seed, weights=weights)
        return made[key]
    return get


def config_for(name, dtype):
    """In bfloat16 the engine's tests run the configuration whose routers choose every expert; what a
    router with a choice does in bfloat16 has a test of its own, up to the first close call."""
    return name + "n" if dtype == "bfloat16" and name + "n" in T.CONFIGS else name


def make_requests(cfg, lengths, seed):
    return {f"r{i}": T.tokens(cfg, n, seed * 100 + i) for i, n in enumerate(lengths)}


class Expected(dict):
    """{request: logits of the plain model}; ``slack`` holds, for bfloat16, how far the plain model's
    own rows move when only the inputs of its sub-layers are rounded to bfloat16; ``close`` the
    positions at which a router decided by less than rounding moves its scores (either choice is
    right there, and the rows of the two differ by tenths)."""
    slack = None
    close = frozenset()


# a router's scores lie in (0, 1); bfloat16 inputs move them by some thousandths
CLOSE_CALL = {"float32": 2e-6, "bfloat16": 2e-2}


def row_error(got, want):
    d, w = got - want, want - want.mean()
    return float(np.sqrt(((d - d.mean()) ** 2).mean()) / np.sqrt((w ** 2).mean()))


def forward_with_rounded_inputs(cfg, w, tokens):
    """The plain model with the input of every sub-layer rounded to bfloat16 and nothing else:
    where its rows move far, the model itself magnifies rounding at that position."""
    eps, m = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    positions = list(range(len(tokens)))
    rounded = lambda t: t.to(torch.bfloat16).double()
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        h = rounded(P.rms_norm(x, w[p + ".norm1"], eps))
        if layer["type"] == "parallel":
            y = P.parallel_mixer(h, w, p + ".mix", layer["mixer"], eps, positions)
        else:
            y = P.attention(h, w, p + ".mix", layer["mixer"], eps, positions)
        x = x + m * P.rms_norm(y, w[p + ".norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rounded(P.rms_norm(x, w[p + ".norm2"], eps))
            y = P.dense_ff(h, w, p + ".mlp", mlp) if mlp["kind"] == "dense" else P.moe_ff(h, w, p + ".mlp", mlp)
            x = x + m * P.rms_norm(y, w[p + ".norm2b"], eps)
    return rounded(P.rms_norm(x, w["final.norm"], eps)) @ w["embed"].T


def expected(model_dir, cfg, requests, dtype):
    w = T.read_weights(model_dir, as_stored_in=dtype)
    out, close = Expected(), set()
    for rid, toks in requests.items():
        margins = []
        out[rid] = P.forward(cfg, w, toks, margins=margins).numpy()
        close |= {(rid, p) for layer in margins for p, gap in enumerate(layer) if gap < CLOSE_CALL[dtype]}
    out.close = frozenset(close)
    if dtype == "bfloat16":
        out.slack = {}
        for rid, toks in requests.items():
            moved = forward_with_rounded_inputs(cfg, w, toks).numpy()
            out.slack[rid] = [row_error(moved[p], out[rid][p]) for p in range(len(toks))]
    return out


def replay(model_dir, dtype, steps, max_tokens, slots=4, **opts):
    from kllm_amd.engine import EngineOptions
    from kllm_amd.replay import Replayer
    options = EngineOptions(dtype=dtype, max_tokens=max_tokens, max_model_len=1 << 30, max_requests=slots,
                            poison_freed_pages=True, **opts)
    rep = Replayer(model_dir, dtype, max_tokens, options=options)
    outs = [rep.step(s["entries"], s["end"]) for s in steps]
    assert not rep.engine.cache.requests
    rep.engine.cache.check_invariants()
    assert all(p.free_pages == p.num_pages for p in rep.engine.cache.pools)
    return traces.collect(steps, outs), rep


def compare(rows, want, dtype, requests, tol=None):
    """Every position within its limit in float32.  In bfloat16 single positions magnify rounding
    beyond what the estimate of it foresees (a router's close call, a nearly empty delta head in
    front of its norm): one position in fifty (or one) may lie over its limit, none over twice it."""
    worst, over, count = 0.0, [], 0
    for rid, toks in requests.items():
        # in bfloat16 what follows a close call inherits it through caches and states
        first_close = min([p for r, p in want.close if r == rid] or [len(toks)])
        for p in range(len(toks)):
            got = rows[(rid, p)].astype(np.float64)
            assert np.isfinite(got).all(), (rid, p)
            if (rid, p) in want.close or (dtype == "bfloat16" and p > first_close):
                continue
            err = row_error(got, want[rid][p])
            limit = tol or TOL[dtype]
            if getattr(want, "slack", None):
                limit = max(limit, 5.0 * want.slack[rid][p])
            count += 1
            if dtype == "bfloat16" and limit <= err < 2.0 * limit:
                over.append((rid, p, err, limit))
                continue
            worst = max(worst, err * TOL[dtype] / limit)
            assert err < limit, f"{rid} position {p}: off by {err} (limit {limit})"
    assert len(rows) == sum(len(t) for t in requests.values())
    assert dtype == "bfloat16" or len(want.close) <= len(rows) // 50        # close calls are the exception
    assert len(over) <= max(1, count // 50), over
    WORST[dtype] = max(WORST[dtype], worst)
    return worst


# ----------------------------------------------------------------------------- kernels

@pytest.mark.parametrize("n,d", [(1, 64), (7, 50), (33, 1024), (3, 2500), (2, 5000)])
def test_norm_behind_a_sublayer_with_factor_row_factors_and_the_next_norm(n, d):
    """x += m g N(sum of slices * row factor), and next_g N(new x) in the same launch, rows kept in
    registers (up to 4,096 channels) and in LDS."""
    from kllm_amd import kernels as K
    g = torch.Generator().manual_seed(n * 7 + d)
    x = torch.randn(n, d, generator=g)
    delta = torch.randn(3, n, d, generator=g)
    w1, w2 = 1.0 + 0.3 * torch.randn(d, generator=g), 1.0 + 0.3 * torch.randn(d, generator=g)
    rows = torch.rand(n, generator=g) + 0.5
    eps, m = 1e-5, 0.65
    v = delta.double().sum(0) * rows.double()[:, None]
    new = x.double() + m * P.rms_norm(v, w1.double(), eps)
    nxt = P.rms_norm(new, w2.double(), eps)
    for dt, tol in ((torch.float32, 2e-6), (torch.bfloat16, 6e-3)):
        xd = x.clone().cuda()
        out = torch.empty(n, d, device="cuda", dtype=dt)
        K.norm_residual(xd, w1.cuda(), delta.cuda(), eps=eps, mult=m, out=out, next_weight=w2.cuda(), delta_scale=rows.cuda())
        assert rel(xd.cpu(), new) < 2e-6
        assert rel(out.float().cpu(), nxt) < tol
        xd = x.clone().cuda()
        K.norm_residual(xd, w1.cuda(), delta.cuda(), eps=eps, mult=m, out=out)        # the new rows themselves
        assert rel(out.float().cpu(), x.double() + m * P.rms_norm(delta.double().sum(0), w1.double(), eps)) < tol


WHOLE_NORM_CASES = [  # H, KV, dk, dv, rot, temp
    (4, 2, 32, 16, 16, None), (6, 3, 64, 64, 0, (0.3, 5)), (5, 5, 20, 12, 10, (0.5, 1)), (3, 1, 16, 40, 16, None),
    (2, 2, 128, 128, 64, (0.2, 3))]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,dk,dv,rot,temp", WHOLE_NORM_CASES)
def test_norm_over_the_whole_projection_rotation_and_append(H, KV, dk, dv, rot, temp, dtype):
    """Queries and pages as the kernel leaves them against the plain functions: one norm over all
    query heads and one over all key heads, the rotation behind it, the temperature, keys [KV][slot][dk]
    and values [KV][dv][slot] in pages handed out in a shuffled order."""
    from kllm_amd import kernels as K
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    page, eps = 16, 1e-5
    g = torch.Generator().manual_seed(H * 100 + dk + dv)
    n = 41
    positions = [3 * i for i in range(n)]                  # over several pages, with gaps
    pages_needed = positions[-1] // page + 1
    order = torch.randperm(pages_needed + 1, generator=g).tolist()
    table = torch.tensor([order[:pages_needed]], dtype=torch.int32)
    cols = (H + KV) * dk + KV * dv
    sums = torch.randn(2, n, cols, generator=g)
    qw, kw = 1.0 + 0.3 * torch.randn(H * dk, generator=g), 1.0 + 0.3 * torch.randn(KV * dk, generator=g)
    raw = sums.double().sum(0)
    q = P.rms_norm(raw[:, :H * dk], qw.double(), eps).reshape(n, H, dk)
    k = P.rms_norm(raw[:, H * dk:(H + KV) * dk], kw.double(), eps).reshape(n, KV, dk)
    v = raw[:, (H + KV) * dk:].reshape(n, KV, dv)
    cos = sin = None
    if rot:
        r = {"dims": rot, "base": 700.0, "scaling": {"factor": 3.0, "low": 1.0, "high": 4.0, "original": 40}}
        q, k = P.rotate_halves(q, positions, r), P.rotate_halves(k, positions, r)
        cos, sin = torch.empty(n, rot // 2, device="cuda"), torch.empty(n, rot // 2, device="cuda")
        K.rope_tables_freq(cos, sin, torch.tensor(positions, dtype=torch.int32, device="cuda"), P.frequencies(r).cuda(), 1.0)
    if temp:
        q = q * P.query_temperature(positions, {"coef": temp[0], "every": temp[1]})[:, None, None]
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
    flat = dk != dv
    shape = (pages_needed + 1, KV * page * (dk + dv)) if flat else (pages_needed + 1, 2, KV, page * dk)
    cache = torch.full(shape, float("nan"), device="cuda", dtype=dt)
    q_out = torch.empty(n, H * dk, device="cuda", dtype=dt)
    K.qk_norm_append(sums.cuda(), q_out, cache, i32(positions), i32([0] * n), table.cuda(), page, H, KV, dk, q_weight=qw.cuda(),
                     k_weight=kw.cuda(), eps=eps, temp_coef=temp[0] if temp else 0.0, temp_every=temp[1] if temp else 0,
                     value_dim=dv, cos=cos, sin=sin, rotary_dim=rot)
    tol = 2e-6 if dtype == "float32" else 6e-3
    assert rel(q_out.float().cpu(), q.reshape(n, H * dk)) < tol
    got = cache.float().cpu().reshape(pages_needed + 1, -1)
    for t, pos in enumerate(positions):
        row = got[table[0, pos // page]]
        keys = row[:KV * page * dk].reshape(KV, page, dk)[:, pos % page]
        vals = row[KV * page * dk:].reshape(KV, dv, page)[:, :, pos % page]
        assert rel(keys, k[t]) < tol and rel(vals, v[t]) < tol, t


@pytest.mark.parametrize("H,G,dk,dv", [(4, 2, 16, 24), (3, 1, 12, 10), (2, 2, 64, 32), (1, 1, 128, 128), (2, 1, 200, 40)])
def test_delta_rule_with_a_decay_per_key_channel(H, G, dk, dv):
    """The scan over two spans (one that goes on from a state, one that starts at position 0 on a
    slot that holds another request's numbers) against the recurrence written out."""
    from kllm_amd import kernels as K
    g = torch.Generator().manual_seed(H * 10 + dk)
    lens, n = [37, 5], 42
    q = P.unit(torch.randn(n, G, dk, generator=g, dtype=F64)) * dk ** -0.5
    k = P.unit(torch.randn(n, G, dk, generator=g, dtype=F64))
    v = torch.randn(n, H, dv, generator=g, dtype=F64)
    dec = torch.rand(n, H, dk, generator=g, dtype=F64) * 0.6 + 0.4
    beta = torch.rand(n, H, generator=g, dtype=F64)
    state0 = torch.randn(3, H * dk * dv + 5, generator=g)             # three slots, a field behind the state
    want = torch.zeros(n, H, dv, dtype=F64)
    ends = {}
    for (a, b, slot, fresh) in ((0, 37, 2, False), (37, 42, 0, True)):
        for h in range(H):
            S = torch.zeros(dk, dv, dtype=F64) if fresh else state0[slot, :H * dk * dv].double().reshape(H, dk, dv)[h].clone()
            for t in range(a, b):
                S = dec[t, h][:, None] * S
                u = beta[t, h] * (v[t, h] - S.T @ k[t, h // (H // G)])
                S = S + torch.outer(k[t, h // (H // G)], u)
                want[t, h] = S.T @ q[t, h // (H // G)]
            ends[(slot, h)] = S
    f = lambda t: t.float().cuda().contiguous()
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
    gb = torch.stack([torch.full((n, H), 7.0, dtype=F64), beta], dim=1)      # the decay per head is not looked at
    o = torch.full((n, H * dv), float("nan"), device="cuda")
    state = state0.clone().cuda()
    K.gated_delta_scan(f(q.reshape(n, -1)), f(k.reshape(n, -1)), f(v.reshape(n, -1)), f(gb), o, state, 0, i32([2, 0]),
                       i32([0, 37, 42]), i32([11, 0]), 2, H, G, dk, dv, decays=f(dec.reshape(n, -1)))
    assert rel(o.cpu(), want.reshape(n, -1)) < 1e-5
    left = state.cpu()
    for (slot, h), S in ends.items():
        assert rel(left[slot, :H * dk * dv].reshape(H, dk, dv)[h], S) < 1e-5
    assert torch.equal(left[1], state0[1]) and torch.equal(left[:, H * dk * dv:], state0[:, H * dk * dv:])


def test_sum_of_two_normed_mixers():
    from kllm_amd import kernels as K
    g = torch.Generator().manual_seed(3)
    for n, d in ((5, 37), (2, 3000), (3, 4500)):
        a, b = torch.randn(2, n, d, generator=g), torch.randn(n, d, generator=g) * 3.0
        wa, wb = torch.randn(d, generator=g), torch.randn(d, generator=g)
        out = torch.empty(n, d, device="cuda")
        K.normed_sum(out, a.cuda(), 0.5, wa.cuda(), b.cuda(), 0.25, wb.cuda(), 1e-4)
        want = 0.5 * P.rms_norm(a.double().sum(0), wa.double(), 1e-4) + 0.25 * P.rms_norm(b.double(), wb.double(), 1e-4)
        assert rel(out.cpu(), want) < 2e-6
        # the same left to the norm behind the mixer, which also makes the next norm's rows
        x = torch.randn(n, d, generator=g)
        w1, w2 = 1.0 + 0.3 * torch.randn(d, generator=g), 1.0 + 0.3 * torch.randn(d, generator=g)
        new = x.double() + 0.6 * P.rms_norm(want, w1.double(), 1e-4)
        xd, nxt = x.clone().cuda(), torch.empty(n, d, device="cuda")
        K.norm_residual(xd, w1.cuda(), K.NormedPair(a.cuda(), 0.5, wa.cuda(), b.cuda(), 0.25, wb.cuda()), eps=1e-4, mult=0.6,
                        out=nxt, next_weight=w2.cuda())
        assert rel(xd.cpu(), new) < 2e-6 and rel(nxt.cpu(), P.rms_norm(new, w2.double(), 1e-4)) < 2e-6


@pytest.mark.parametrize("E,top,groups,keep", [(8, 3, 4, 2), (6, 2, 3, 1), (16, 4, 4, 3), (6, 2, 6, 3), (5, 1, 1, 1),
                                               (128, 8, 8, 4), (4, 4, 2, 2)])
def test_logistic_router_within_the_best_groups(E, top, groups, keep):
    """Choices and weights against the plain choice, and the shared expert's gate from the sum
    behind the experts'."""
    from kllm_amd import kernels as K
    g = torch.Generator().manual_seed(E + top)
    n = 50
    z = torch.randn(2, n, E + 1, generator=g) * 1.5
    idx = torch.empty(n, top, dtype=torch.int32, device="cuda")
    wgt = torch.empty(n, top, device="cuda")
    sg = torch.empty(n, device="cuda")
    K.moe_route(z.cuda(), None, idx, wgt, experts=E, scoring="sigmoid", groups=groups, keep_groups=keep, scale=1.9,
                renormalize=False, shared_gate=sg)
    zz = z.double().sum(0)
    s = torch.sigmoid(zz[:, :E])
    for t in range(n):
        want = P.choose_experts(s[t], top, groups, keep).tolist()
        assert sorted(idx[t].tolist()) == sorted(want), t
        assert rel(wgt[t].cpu(), 1.9 * s[t][idx[t].long().cpu()]) < 1e-6
    assert rel(sg.cpu(), torch.sigmoid(zz[:, E])) < 1e-6


# ----------------------------------------------------------------------------- each mixer alone

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A1", "P1"])
def test_one_mixer_alone_whole_and_token_by_token(folders, name, dtype):
    """A model of one layer without feed-forward: the stream behind the layer in one step, and
    the same from a prompt of 9 tokens followed by single tokens (the state and the convolution's
    last inputs, and the cache, carried from step to step)."""
    from kllm_amd.engine import Engine, EngineOptions, StepEntry
    cfg, d = T.CONFIGS[name], folders(name)
    w = T.read_weights(d, as_stored_in=dtype)
    toks = T.tokens(cfg, 70, 5)
    want = []
    P.forward(cfg, w, toks, taps=want)
    eng = Engine.from_dir(d, EngineOptions(dtype=dtype, max_tokens=256, max_model_len=1 << 20, max_requests=2))
    tol = 2e-6 if dtype == "float32" else 2e-2
    taps = []
    eng.step([StepEntry("a", toks, [])], taps=taps)
    eng.release("a")
    assert rel(taps[1].float().cpu(), want[0]) < tol
    rows = []
    taps = []
    eng.step([StepEntry("b", toks[:9], [])], taps=taps)
    rows.append(taps[1].float().cpu())
    for t in toks[9:]:
        taps = []
        eng.step([StepEntry("b", [t], [])], taps=taps)
        rows.append(taps[1].float().cpu())
    eng.release("b")
    got = torch.cat(rows)
    for p in range(len(toks)):
        assert rel(got[p], want[0][p]) < tol * 2, p


# ----------------------------------------------------------------------------- aimed queries

# the aimed attention stands in the first layer: alone as a layer of its own, or as the left half
T.CONFIGS["Q1"] = T._cfg(80, 64, 1e-5, 2.0, 0.8, [
    T.parallel(T.attn(4, 2, 32, vdim=16, rot=16, base=5000.0, scaling=(4.0, 1.0, 3.0, 48), chunk=24, scale=0.2),
               T.delta(2, 1, 16, 24, 3), T.dense(72, 1.0)),
    T.layer("attention", T.attn(2, 1, 16, temp=(0.3, 9)))])
T.CONFIGS["Q2"] = T._cfg(96, 96, 1e-6, 1.5, 1.0, [
    T.parallel(T.attn(4, 2, 64, rot=32, chunk=40, scale=0.3), T.delta(2, 2, 16, 16, 2)),
    T.layer("attention", T.attn(2, 2, 16, vdim=24), T.moe(4, 4, 24, groups=(2, 2), shared=16))])
T.CONFIGS["Q3"] = T._cfg(70, 80, 1e-5, 1.2, 0.6, [
    T.parallel(T.attn(2, 2, 128, rot=64, chunk=130, scale=0.25), T.delta(1, 1, 32, 32, 4), T.dense(48, 3.0))])
T.CONFIGS["Q4"] = T._cfg(90, 72, 1e-5, 1.0, 0.9, [
    T.layer("attention", T.attn(3, 1, 24, vdim=20, temp=(0.3, 100), scale=0.25), T.dense(64, 1.4)),
    T.parallel(T.attn(2, 1, 16, rot=8, chunk=32), T.delta(2, 2, 16, 16, 2))])
T.CONFIGS["Q5"] = T._cfg(90, 96, 1e-5, 1.0, 0.85, [
    T.layer("attention", T.attn(4, 2, 64, temp=(0.2, 256), scale=0.2)),
    T.layer("attention", T.attn(2, 1, 8, vdim=8), T.dense(40, 1.0))])

QUERY, KEY = 1, 2


def first_attention(cfg):
    layer = cfg["layers"][0]
    return ("l0.mix.left", layer["mixer"]["left"]) if layer["type"] == "parallel" else ("l0.mix", layer["mixer"])


def aimed_prompt(cfg, n, seed, places):
    """Random tokens other than the two aimed ones, with the key token and the query token put
    at ``places`` ({position: token})."""
    g = torch.Generator().manual_seed(seed)
    toks = torch.randint(3, cfg["vocab"], (n,), generator=g).tolist()
    for p, t in places.items():
        toks[p] = t
    return toks


def check_aimed(folders, name, weights, dtype, reqs, shown):
    """``shown``: (request, query position, key position, seen) for every aimed pair: the plain
    model's row at the query must change a lot when a seen key's token is taken away, and when the
    chunk is made one position longer for a key that is just not seen; then the engine's rows
    against the plain model's, request whole, its last tokens one by one, and in portions."""
    cfg = T.CONFIGS[name]
    d = folders(name, weights=weights, tag="aimed")
    want = expected(d, cfg, reqs, dtype)
    w = T.read_weights(d, as_stored_in=dtype)
    check_shown(cfg, w, reqs, want, shown)
    longest = max(len(t) for t in reqs.values())
    steps = traces.whole(reqs)
    rows, _ = replay(d, dtype, steps, traces.peak_tokens(steps))
    compare(rows, want, dtype, reqs, tol=AIMED_TOL[dtype])
    steps = traces.bulk_then_tail(reqs, min(60, longest - 2))       # the aimed queries are decoded alone
    rows, _ = replay(d, dtype, steps, traces.peak_tokens(steps))
    compare(rows, want, dtype, reqs, tol=AIMED_TOL[dtype])
    steps = traces.portions(reqs, seed=2)
    rows, _ = replay(d, dtype, steps, traces.peak_tokens(steps))
    compare(rows, want, dtype, reqs, tol=AIMED_TOL[dtype])


def check_shown(cfg, w, reqs, want, shown):
    for rid, qpos, kpos, seen in shown:
        if seen:
            other = list(reqs[rid])
            other[kpos] = 5
            row = P.forward(cfg, w, other[:qpos + 1])[qpos].numpy()
        elif kpos < qpos:       # with a chunk that starts one position earlier it would be seen
            wider = copy.deepcopy(cfg)
            _, m = first_attention(wider)
            m["mask"]["size"] = 10 ** 6
            row = P.forward(wider, w, reqs[rid][:qpos + 1])[qpos].numpy()
        else:
            continue
        assert rel(row, want[rid][qpos]) > 0.3, (rid, qpos, kpos, seen)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["Q1", "Q2", "Q3"])
def test_a_query_aimed_at_the_edges_of_its_chunk(folders, name, dtype):
    cfg = T.CONFIGS[name]
    p, m = first_attention(cfg)
    C = m["mask"]["size"]
    w = T.aimed_attention(cfg, P.random_weights(cfg, 21), p, m, QUERY, KEY)
    n = 4 * C - 3
    start = 3 * C                      # the last chunk's first position
    qa = 4 * C - 5
    reqs = {
        # the key at the chunk's first place, and one before it
        "in": aimed_prompt(cfg, n, 1, {start: KEY, qa: QUERY}),
        "out": aimed_prompt(cfg, n, 2, {start - 1: KEY, qa: QUERY}),
        # the query at the chunk's first place sees itself only; at its last place the whole chunk
        "edge": aimed_prompt(cfg, n, 3, {start - 1: KEY, start: QUERY}),
        "last": aimed_prompt(cfg, n, 4, {2 * C: KEY, 3 * C - 1: QUERY}),
        # a chunk further back is not seen, position 0 neither
        "zero": aimed_prompt(cfg, n, 5, {0: KEY, qa: QUERY}),
        # in a prompt shorter than a chunk nothing is masked
        "short": aimed_prompt(cfg, C - 1, 6, {0: KEY, C - 2: QUERY}),
    }
    shown = [("in", qa, start, True), ("out", qa, start - 1, False), ("edge", start, start - 1, False),
             ("last", 3 * C - 1, 2 * C, True), ("zero", qa, 0, False), ("short", C - 2, 0, True)]
    check_aimed(folders, name, w, dtype, reqs, shown)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["Q4", "Q5"])
def test_a_query_aimed_at_a_key_hundreds_of_positions_back(folders, name, dtype):
    cfg = T.CONFIGS[name]
    p, m = first_attention(cfg)
    w = T.aimed_attention(cfg, P.random_weights(cfg, 22), p, m, QUERY, KEY)
    reqs = {
        "far": aimed_prompt(cfg, 610, 1, {3: KEY, 600: QUERY}),
        "first": aimed_prompt(cfg, 300, 2, {0: KEY, 290: QUERY}),
        "page": aimed_prompt(cfg, 300, 3, {15: KEY, 271: QUERY}),              # the last slot of a page
        "page2": aimed_prompt(cfg, 300, 3, {16: KEY, 271: QUERY}),             # the next page's first
        "next": aimed_prompt(cfg, 40, 4, {30: KEY, 31: QUERY}),
        "ahead": aimed_prompt(cfg, 40, 5, {31: KEY, 30: QUERY}),               # a key ahead of the query is not seen
    }
    shown = [("far", 600, 3, True), ("first", 290, 0, True), ("page", 271, 15, True), ("page2", 271, 16, True),
             ("next", 31, 30, True), ("ahead", 30, 31, False)]
    check_aimed(folders, name, w, dtype, reqs, shown)


# ----------------------------------------------------------------------------- the engine

CASES = [("G1", [1, 5, 33, 130]), ("G2", [2, 17, 140]), ("G3", [3, 64, 65, 150]), ("G4", [90, 31, 4]),
         ("G5", [49, 80, 16, 17]), ("G6", [210, 99, 7])]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,lengths", CASES)
def test_whole_prompts_decoding_portions_and_mixed_batches(folders, name, lengths, dtype):
    """One configuration at a time through all four ways of cutting its requests into steps."""
    name = config_for(name, dtype)
    cfg, d = T.CONFIGS[name], folders(name)
    reqs = make_requests(cfg, lengths, 1)
    want = expected(d, cfg, reqs, dtype)
    steps = traces.whole(reqs)
    rows, _ = replay(d, dtype, steps, traces.peak_tokens(steps))
    compare(rows, want, dtype, reqs)
    steps = traces.bulk_then_tail(reqs, 30)          # the tail crosses a chunk's and a page's border
    rows, _ = replay(d, dtype, steps, traces.peak_tokens(steps))
    compare(rows, want, dtype, reqs)
    steps = traces.portions(reqs, seed=4)
    assert min(len(s["entries"][0]["tokens"]) for s in steps if not s["end"]) == 2
    rows, _ = replay(d, dtype, steps, traces.peak_tokens(steps))
    compare(rows, want, dtype, reqs)
    # more requests than may live at once, on so few pages and slots that they are used again
    many = make_requests(cfg, lengths + [40, 7, 77, 12], 2)
    want = expected(d, cfg, many, dtype)
    steps, peak = traces.mixed(many, seed=5, max_live=4, tail=6, max_portion=20)
    rows, _ = replay(d, dtype, steps, peak, slots=4)
    compare(rows, want, dtype, many)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", list(range(12)))
def test_configurations_drawn_from_a_seed(folders, seed, dtype):
    """Layer orders, sizes and constants that nobody chose (in float32 every position is bound; in
    bfloat16 the routers choose every expert): whole prompts and a mixed trace with portions down to
    two tokens beside single tokens."""
    name = f"R{seed}{dtype[0]}"
    T.CONFIGS[name] = T.random_config(seed) if dtype == "float32" else T.without_choice(T.random_config(seed))
    cfg, d = T.CONFIGS[name], folders(name, seed=seed + 100)
    reqs = make_requests(cfg, [70, 3, 141, 18, 33], seed)
    want = expected(d, cfg, reqs, dtype)
    steps = traces.whole(reqs)
    rows, _ = replay(d, dtype, steps, traces.peak_tokens(steps))
    compare(rows, want, dtype, reqs)
    steps, peak = traces.mixed(reqs, seed=seed, max_live=4, tail=9, max_portion=17)
    rows, _ = replay(d, dtype, steps, peak)
    compare(rows, want, dtype, reqs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["G1", "G6"])
def test_a_batch_against_each_request_alone(folders, name, dtype):
    """The logits of a request do not depend on what else the step holds, beyond rounding: a
    mixed trace against each of its requests replayed alone, cut the same way."""
    name = config_for(name, dtype)
    cfg, d = T.CONFIGS[name], folders(name)
    reqs = make_requests(cfg, [50, 23, 9, 71], 3)
    steps, peak = traces.mixed(reqs, seed=1, max_live=3, tail=5, max_portion=16)
    rows, _ = replay(d, dtype, steps, peak)
    close = expected(d, cfg, reqs, dtype).close          # a kernel chosen by the row count may tip a router's close call
    for rid in reqs:
        alone = [{"step": i, "entries": [e for e in s["entries"] if e["id"] == rid],
                  "end": [r for r in s["end"] if r == rid]} for i, s in enumerate(steps)]
        alone = [s for s in alone if s["entries"]]
        for i, s in enumerate(alone):
            s["step"] = i
        single, _ = replay(d, dtype, alone, peak)
        for p in range(len(reqs[rid])):
            if (rid, p) not in close:
                assert rel(single[(rid, p)], rows[(rid, p)]) < (1e-5 if dtype == "float32" else 4e-2), (rid, p)


@pytest.mark.parametrize("name", ["G1", "G4", "G6"])
def test_routers_with_a_choice_in_bfloat16_up_to_the_first_close_call(folders, name):
    """Many short requests in a mixed trace: each is compared up to the first position at which a
    router of the plain model decides by less than bfloat16 moves its scores."""
    cfg, d = T.CONFIGS[name], folders(name)
    reqs = make_requests(cfg, [25, 9, 31, 14, 40, 6, 18, 22, 12, 35], 11)
    want = expected(d, cfg, reqs, "bfloat16")
    steps, peak = traces.mixed(reqs, seed=6, max_live=4, tail=5, max_portion=14)
    rows, _ = replay(d, "bfloat16", steps, peak)
    compare(rows, want, "bfloat16", reqs)
    compared = sum(min([p for r, p in want.close if r == rid] or [len(t)]) for rid, t in reqs.items())
    assert compared >= 15, compared


def test_slots_and_pages_that_are_given_back_hold_nothing_of_their_last_owner(folders):
    """Two state slots and few pages, seven requests one after another in pairs: every request
    starts from zero state on a slot that another has just left (freed pages are poisoned)."""
    cfg, d = T.CONFIGS["G1"], folders("G1")
    reqs = make_requests(cfg, [30, 45, 12, 64, 5, 33, 20], 6)
    steps, peak = traces.mixed(reqs, seed=8, max_live=2, tail=3, max_portion=11)
    rows, rep = replay(d, "float32", steps, peak, slots=2)
    compare(rows, expected(d, cfg, reqs, "float32"), "float32", reqs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["G1", "G6"])
def test_long_decoding_over_page_and_chunk_borders(folders, name, dtype):
    name = config_for(name, dtype)
    cfg, d = T.CONFIGS[name], folders(name)
    reqs = make_requests(cfg, [230], 7)
    steps = traces.bulk_then_tail(reqs, 227)
    rows, rep = replay(d, dtype, steps, traces.peak_tokens(steps))
    compare(rows, expected(d, cfg, reqs, dtype), dtype, reqs)
    assert rep.engine.steps_repeated > 100                       # decode steps ran from their recorded commands


@pytest.mark.parametrize("name", ["G3", "G6"])
def test_the_kernel_for_every_size_and_the_matrix_core_kernels_agree(folders, name):
    """Chunked and causal attention on the matrix cores (prompts in blocks, single tokens in
    slices) against the kernel that takes every size, same trace."""
    name = config_for(name, "bfloat16")
    cfg, d = T.CONFIGS[name], folders(name)
    reqs = make_requests(cfg, [300, 21, 150], 9)
    steps, peak = traces.mixed(reqs, seed=2, max_live=3, tail=40, max_portion=70)
    a, _ = replay(d, "bfloat16", steps, peak)
    b, _ = replay(d, "bfloat16", steps, peak, attention="generic")
    assert max(rel(a[k], b[k]) for k in a) < 4e-2
    assert any(not np.array_equal(a[k], b[k]) for k in a)          # they are two kernels


def test_recorded_steps_and_layers_change_no_bit(folders):
    cfg, d = T.CONFIGS["G1"], folders("G1")
    reqs = make_requests(cfg, [140, 21], 9)
    steps, peak = traces.mixed(reqs, seed=2, max_live=2, tail=10, max_portion=12)
    a, _ = replay(d, "bfloat16", steps, peak)
    c, _ = replay(d, "bfloat16", steps, peak, extra={"no_repeated_layers": True, "no_repeated_steps": True,
                                                     "launch_one_by_one": True})
    assert all(np.array_equal(a[k], c[k]) for k in a)


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_scheduler(folders, dtype):
    from kllm_amd.engine import Engine, EngineOptions
    name = config_for("G1", dtype)
    cfg, d = T.CONFIGS[name], folders(name)
    w = T.read_weights(d, as_stored_in=dtype)
    prompts = [T.tokens(cfg, n, 40 + n) for n in (3, 11, 30, 6, 18)]
    eng = Engine.from_dir(d, EngineOptions(dtype=dtype, max_tokens=1024, max_model_len=256, max_requests=4))
    got = eng.generate(prompts, max_new_tokens=12, max_step_tokens=16, max_batch=3)
    for prompt, ids in zip(prompts, got):
        want = P.greedy(cfg, w, prompt, 12)
        if dtype == "float32":
            assert ids == want
        else:       # a near tie may fall the other way in bfloat16; what was generated up to there agrees
            k = next((i for i, (a, b) in enumerate(zip(ids, want)) if a != b), 12)
            assert k >= 3, (ids, want)
            if k < 12:
                lg = P.forward(cfg, w, prompt + want[:k])[-1]
                top = torch.topk(lg, 2).values
                assert float(top[0] - top[1]) < 0.2 * float(lg.std())
    assert not eng.cache.requests


def test_the_command_line_programs_take_the_model(folders, tmp_path):
    """bin/generate (greedy, float32) against the plain model's greedy continuation, and
    bin/trace_run fed a trace on its standard input, one line a step."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg, d = T.CONFIGS["G4"], folders("G4")
    w = T.read_weights(d)
    prompt = T.tokens(cfg, 9, 77)
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "generate"), "--model", d, "--dtype", "float32",
                        "--ids", " ".join(map(str, prompt)), "--steps", "10"], capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    line = [l for l in p.stdout.splitlines() if l.startswith("generated:")][0]
    assert [int(v) for v in line.split("[")[1].rstrip("]").split()] == P.greedy(cfg, w, prompt, 10)
    reqs = make_requests(cfg, [37, 12], 8)
    steps, peak = traces.mixed(reqs, seed=3, max_live=2, tail=4, max_portion=9)
    out = tmp_path / "logits"
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d, "--dtype", "float32",
                        "--out", str(out), "--max-tokens", str(peak)], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done ")] == [f"done {s['step']}" for s in steps]
    outs = [np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(-1, cfg["vocab"]) for s in steps]
    compare(traces.collect(steps, outs), expected(d, cfg, reqs, "float32"), "float32", reqs)


def test_zz_the_worst_difference_seen():
    print("worst relative difference of logits:", WORST)
    assert all(WORST[d] < TOL[d] for d in WORST)
