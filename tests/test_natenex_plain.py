"""The plain Natenex (tests/plain_natenex.py) against identities of its own, and the
configuration reader and model builder, without a GPU."""

import copy
import math

import pytest
import torch

import natenex_tiny as T
import plain_natenex as P

F64 = torch.float64


def test_the_window_keeps_the_first_positions():
    assert P.sees(100, 100, 8, 2) and P.sees(100, 93, 8, 2) and not P.sees(100, 92, 8, 2)
    assert P.sees(100, 1, 8, 2) and not P.sees(100, 2, 8, 2) and not P.sees(5, 6, 8, 2)
    assert all(P.sees(50, j, 0, 0) for j in range(51))


def test_slowed_down_frequencies():
    rot = {"dims": 16, "base": 5000.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 3.0, "original": 48}}
    plain = P.frequencies({"dims": 16, "base": 5000.0})
    f = P.frequencies(rot)
    kinds = set()
    for a, b in zip(plain.tolist(), f.tolist()):
        wl = 2 * math.pi / a
        if wl < 16:
            assert b == a
            kinds.add("kept")
        elif wl > 48:
            assert b == a / 4
            kinds.add("slowed")
        else:
            assert a / 4 < b < a
            kinds.add("between")
    assert kinds == {"kept", "slowed", "between"}
    from kllm_amd.parts.rotary import scaled_frequencies
    mine, factor = scaled_frequencies(16, 5000.0, ("by_wavelength", 4.0, 1.0, 3.0, 48))
    assert factor == 1.0 and torch.allclose(torch.tensor(mine, dtype=F64), f, rtol=1e-14)


def test_rotation_keeps_lengths_and_scores_depend_on_the_distance():
    g = torch.Generator().manual_seed(0)
    rot = {"dims": 8, "base": 100.0}
    x, y = torch.randn(1, 1, 12, generator=g, dtype=F64), torch.randn(1, 1, 12, generator=g, dtype=F64)
    a = (P.rotate_halves(x, [5], rot) * P.rotate_halves(y, [2], rot)).sum()
    b = (P.rotate_halves(x, [105], rot) * P.rotate_halves(y, [102], rot)).sum()
    assert abs(a - b) < 1e-9
    assert torch.equal(P.rotate_halves(x, [7], rot)[..., 8:], x[..., 8:])
    assert abs(P.rotate_halves(x, [7], rot).norm() - x.norm()) < 1e-12


def test_convolution_is_causal_and_starts_from_zeros():
    g = torch.Generator().manual_seed(1)
    x, w = torch.randn(9, 3, generator=g, dtype=F64), torch.randn(3, 4, generator=g, dtype=F64)
    y = P.causal_conv(x, w)
    assert torch.allclose(y[0], x[0] * w[:, 3])
    assert torch.allclose(y[5], sum(x[5 - 3 + j] * w[:, j] for j in range(4)))
    x2 = x.clone()
    x2[6:] += 1.0
    assert torch.equal(P.causal_conv(x2, w)[:6], y[:6])


def test_linear_recurrence_token_by_token():
    cfg = T.CONFIGS["P1"]
    w = P.random_weights(cfg, 3)
    m, p = cfg["layers"][0]["mixer"]["right"], "l0.mix.right"
    h = torch.randn(11, cfg["width"], generator=torch.Generator().manual_seed(2), dtype=F64)
    whole = P.gated_linear_recurrence(h, w, p, m)
    state, inputs = torch.zeros(m["width"], dtype=F64), torch.zeros(m["conv"] - 1, m["width"], dtype=F64)
    for t in range(11):
        out, state, inputs = P.linear_recurrence_step(h[t], state, inputs, w, p, m)
        assert torch.allclose(w[p + ".o"] @ out, whole[t], atol=1e-12)
    assert float(state.abs().max()) > 1e-3


def test_delta_rule_writes_before_it_reads_and_forgets():
    """With beta 1 and no decay the state gives back the value it was just shown along its key;
    a key at right angles leaves it alone."""
    d, dv = 6, 4
    S = torch.zeros(d, dv, dtype=F64)
    k1, k2 = torch.eye(d, dtype=F64)[0], torch.eye(d, dtype=F64)[1]
    v1, v2 = torch.arange(1.0, 5.0, dtype=F64), -torch.arange(1.0, 5.0, dtype=F64)
    for k, v in ((k1, v1), (k2, v2), (k1, v2)):
        S = S + torch.outer(k, 1.0 * (v - S.T @ k))
        assert torch.allclose(S.T @ k, v)
    assert torch.allclose(S.T @ k2, v2)


def test_a_layer_run_twice_uses_the_same_tensors():
    cfg = T.CONFIGS["N1"]
    w = P.random_weights(cfg, 5)
    assert not any(k.startswith("l3.") for k in w)
    toks = T.tokens(cfg, 12, 1)
    taps = []
    P.forward(cfg, w, toks, taps)
    twice = copy.deepcopy(cfg)
    del twice["layers"][3]["weights_of"]
    w2 = dict(w)
    w2.update({k.replace("l0.", "l3.", 1): v for k, v in w.items() if k.startswith("l0.")})
    taps2 = []
    P.forward(twice, w2, toks, taps2)
    assert torch.equal(taps[3], taps2[3])


def test_latent_attention_with_folded_products():
    """The score against the latent itself and the value product behind the softmax give the
    numbers of the definition."""
    cfg = T.CONFIGS["L1"]
    w = P.random_weights(cfg, 9)
    m, p, eps = cfg["layers"][0]["mixer"], "l0.mix", cfg["norm"]["eps"]
    n = 9
    h = torch.randn(n, cfg["width"], generator=torch.Generator().manual_seed(4), dtype=F64)
    want = P.latent_attention(h, w, p, m, eps, list(range(n)))
    H, d, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = P.rms_norm(h @ w[p + ".dq"].T, w[p + ".dq.norm"], eps)
    q = (cq @ w[p + ".uq"].T).reshape(n, H, d + dr)
    dkv = h @ w[p + ".dkv"].T
    c = P.rms_norm(dkv[:, :rank], w[p + ".dkv.norm"], eps)
    kr = P.rotate_halves(dkv[:, rank:].reshape(n, 1, dr), list(range(n)), m["rot"])[:, 0]
    qr = P.rotate_halves(q[..., d:], list(range(n)), m["rot"])
    out = torch.zeros(n, H, dv, dtype=F64)
    for hd in range(H):
        folded = q[:, hd, :d] @ w[p + ".uk"][hd * d:(hd + 1) * d]             # [n, rank]
        s = (folded @ c.T + qr[:, hd] @ kr.T) * m["scale"]
        s = s.masked_fill(torch.triu(torch.ones(n, n, dtype=torch.bool), 1), float("-inf"))
        out[:, hd] = (torch.softmax(s, -1) @ c) @ w[p + ".uv"][hd * dv:(hd + 1) * dv].T
    got = (out.reshape(n, H * dv) * torch.sigmoid(h @ w[p + ".g"].T)) @ w[p + ".o"].T
    assert torch.allclose(got, want, atol=1e-10)


# ----------------------------------------------------------------------------- configuration and builder

@pytest.mark.parametrize("name", sorted(T.CONFIGS))
def test_configuration_round_trip_and_tensor_list(name):
    from kllm_amd.config import config_from_dict
    from kllm_amd.config.registry import resolve_architecture
    from kllm_amd.engine.model import collect_weight_specs
    raw = T.CONFIGS[name]
    cfg = config_from_dict(raw)
    assert cfg.to_dict() == raw
    spec = resolve_architecture(raw).build(cfg)
    specs = {s.name: tuple(s.shape) for s in collect_weight_specs(spec)}
    w = P.random_weights(raw, 1)
    assert specs == {k: tuple(v.shape) for k, v in w.items()}
    assert len(spec.schedule) == len(raw["layers"])
    own = [i for i, l in enumerate(raw["layers"]) if l.get("weights_of") is None]
    for i, (run, layer) in enumerate(zip(spec.schedule, raw["layers"])):
        assert run.cache_of is None
        assert run.layer == own.index(layer.get("weights_of", i) if layer.get("weights_of") is not None else i)


def test_a_layer_may_run_with_a_later_layers_tensors():
    from kllm_amd.config import config_from_dict
    from kllm_amd.config.registry import resolve_architecture
    raw = copy.deepcopy(T.CONFIGS["N5"])
    raw["layers"][0]["weights_of"] = 1
    del raw["layers"][1]["weights_of"]
    spec = resolve_architecture(raw).build(config_from_dict(raw))
    assert [r.layer for r in spec.schedule] == [0, 0] and len(spec.layers) == 1
    assert spec.layers[0].norm_mixer.params["names"]["weight"] == "l1.norm1"


@pytest.mark.parametrize("change,word", [
    (lambda c: c["layers"][0].__setitem__("type", "conv"), "type"),
    (lambda c: c["layers"][3].__setitem__("weights_of", 3), "weights_of"),
    (lambda c: c["layers"][3].__setitem__("weights_of", 9), "weights_of"),
    (lambda c: c["layers"][3]["mlp"].__setitem__("ff", 81), "sizes"),
    (lambda c: c["layers"][0]["mixer"]["right"].__setitem__("blocks", 5), "blocks"),
    (lambda c: c["layers"][0]["mixer"]["left"].__setitem__("kv_heads", 3), "kv_heads"),
    (lambda c: c["layers"][2]["mixer"]["rot"].__setitem__("dims", 6), "rot_dim"),
    (lambda c: c.pop("embedding"), "embedding"),
    (lambda c: c["layers"][1]["mixer"].pop("conv"), "conv"),
])
def test_configurations_that_are_refused(change, word):
    from kllm_amd.config import ConfigError, config_from_dict
    raw = copy.deepcopy(T.CONFIGS["N1"])
    change(raw)
    with pytest.raises(ConfigError) as e:
        config_from_dict(raw)
    assert word in str(e.value)


def test_cache_plan_and_kept_first_pages():
    """Every run of a layer has a cache or state of its own; a windowed group gives back the pages
    behind the window and keeps those of the first positions."""
    from kllm_amd.cache import CacheManager, GroupSpec
    from kllm_amd.config import config_from_dict
    from kllm_amd.config.registry import resolve_architecture
    from kllm_amd.engine.model import Model
    from kllm_amd.parts.base import Runtime
    raw = T.CONFIGS["N1"]
    model = Model(resolve_architecture(raw).build(config_from_dict(raw)), Runtime(torch.device("cpu"), torch.float32))
    plan = model.cache_plan
    assert isinstance(plan.runs[0], list) and isinstance(plan.runs[3], list) and len(plan.runs[0]) == 2
    assert plan.runs[0][0][0] == plan.runs[3][0][0] and plan.runs[0][0][1] != plan.runs[3][0][1]
    kinds = [gp.need.kind for gp in plan.groups]
    assert kinds.count("paged") == 2 and kinds.count("state") == 2
    windowed = [gp.need for gp in plan.groups if gp.need.kind == "paged" and gp.need.window][0]
    assert (windowed.window, windowed.keep_first) == (24, 3)
    # the latents: one "head" whose row is the latent and the rotated part, and the latent once more as its values
    latent = [gp.need for gp in plan.groups if gp.need.kind == "paged" and not gp.need.window][0]
    assert (latent.kv_heads, latent.head_dim, latent.value_width) == (1, 40 + 8, 40)
    cm = CacheManager([GroupSpec("w", 4, 64, window=10, keep_first=5), GroupSpec("all", 4, 64)], 2)
    cm.open("a")
    cm.reserve("a", 40)
    cm.commit("a", 40)
    t = cm.table("a", 0)
    assert t[0] >= 0 and t[1] >= 0                 # positions 0 .. 4 lie in pages 0 and 1
    assert all(p == -1 for p in t[2:7]) and all(p >= 0 for p in t[7:])     # the next token reads from 31
    assert all(p >= 0 for p in cm.table("a", 1))
    cm.check_invariants()
    cm.reserve("a", 1)
    cm.commit("a", 1)
    cm.release("a")
    assert all(p.free_pages == p.num_pages for p in cm.pools)


def test_a_latent_mixer_may_slow_its_rotation_down_too():
    from kllm_amd.config import config_from_dict
    raw = copy.deepcopy(T.CONFIGS["L1"])
    raw["layers"][0]["mixer"]["rot"]["scaling"] = {"factor": 4.0, "low": 1.0, "high": 2.0, "original": 16}
    cfg = config_from_dict(raw)
    assert cfg.layers[0].mixer.rot.scaling.factor == 4.0 and cfg.to_dict()["layers"][0]["mixer"]["rot"]["scaling"]["original"] == 16
    w = P.random_weights(raw, 1)
    toks = T.tokens(raw, 30, 1)
    plain = copy.deepcopy(raw)
    del plain["layers"][0]["mixer"]["rot"]["scaling"]
    assert (P.forward(raw, w, toks) - P.forward(plain, w, toks)).abs().max() > 1e-3
