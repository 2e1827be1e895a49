"""Lugetar without a GPU: the plain implementation pinned by library functions, hand-made cases
and identities of its own; the configuration reader, the builder and the cache plan."""

import copy
import math

import pytest
import torch

import lugetar_tiny as T
import plain_lugetar as P

F64 = torch.float64


def test_small_functions_against_the_library():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 12, generator=g, dtype=F64)
    assert torch.allclose(P.silu(x), torch.nn.functional.silu(x))
    assert torch.allclose(P.softplus(x * 10), torch.nn.functional.softplus(x * 10, threshold=1e9))
    w = torch.randn(12, generator=g, dtype=F64)
    want = torch.nn.functional.rms_norm(x, (12,), w, 1e-3)
    assert torch.allclose(P.rms_norm(x, w, 1e-3), want)
    taps = torch.randn(12, 4, generator=g, dtype=F64)
    lib = torch.nn.functional.conv1d(torch.nn.functional.pad(x.T[None], (3, 0)), taps[:, None, :], groups=12)[0].T
    assert torch.allclose(P.causal_conv(x, taps), lib)
    assert torch.allclose(P.causal_conv(x, taps)[0], x[0] * taps[:, 3])        # the last tap is the current token's


def test_frequencies_slowed_down_by_wavelength():
    rot = {"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 40}}
    plain = [100.0 ** (-2.0 * i / 8) for i in range(4)]
    got = P.frequencies(rot).tolist()
    # wavelengths 6.3, 19.9, 62.8, 198.7 against 10 and 40: kept, blended, slowed, slowed
    assert got[0] == plain[0]
    s = (40 / (2 * math.pi / plain[1]) - 1.0) / 3.0
    assert math.isclose(got[1], (1 - s) * plain[1] / 4 + s * plain[1])
    assert math.isclose(got[2], plain[2] / 4) and math.isclose(got[3], plain[3] / 4)
    assert P.frequencies({"dims": 8, "base": 100.0}).tolist() == plain
    x = torch.randn(3, 2, 12, dtype=F64)
    y = P.rotate_halves(x, [0, 5, 9], rot)
    assert torch.equal(y[0], x[0]) and torch.equal(y[..., 8:], x[..., 8:])       # position 0 and what does not turn
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1))


def test_masks_and_temperature():
    assert [j for j in range(12) if P.sees(9, j, 4)] == [8, 9]
    assert [j for j in range(12) if P.sees(8, j, 4)] == [8]
    assert [j for j in range(12) if P.sees(7, j, 4)] == [4, 5, 6, 7]
    assert [j for j in range(6) if P.sees(3, j, 0)] == [0, 1, 2, 3]
    t = P.query_temperature([0, 2, 3, 8], {"coef": 0.5, "every": 3}).tolist()
    assert t[0] == 1.0 and math.isclose(t[1], 1 + 0.5 * math.log(2)) and math.isclose(t[3], 1 + 0.5 * math.log(4))


def test_choice_of_experts_within_groups():
    s = torch.tensor([0.9, 0.1, 0.5, 0.6, 0.8, 0.0, 0.3, 0.35], dtype=F64)
    # groups (0.9+0.1, 0.5+0.6, 0.8+0.0, 0.3+0.35): the best two are 1 and 0
    assert sorted(P.choose_experts(s, 3, 4, 2).tolist()) == [0, 2, 3]
    assert sorted(P.choose_experts(s, 3, 1, 1).tolist()) == [0, 3, 4]
    assert sorted(P.choose_experts(s, 2, 4, 1).tolist()) == [2, 3]
    assert sorted(P.choose_experts(s, 2, 8, 2).tolist()) == [0, 4]          # groups of one: their own score
    assert sorted(P.choose_experts(s, 8, 4, 4).tolist()) == list(range(8))


def test_clamped_gate():
    g, u = torch.tensor([-3.0, 0.5, 4.0], dtype=F64), torch.tensor([5.0, -5.0, 0.25], dtype=F64)
    got = P.clamped_gate(g, u, 2.0)
    want = [-3.0 / (1 + math.exp(1.702 * 3.0)) * 3.0, 0.5 / (1 + math.exp(-1.702 * 0.5)) * -1.0,
            2.0 / (1 + math.exp(-1.702 * 2.0)) * 1.25]
    assert torch.allclose(got, torch.tensor(want, dtype=F64))


def test_one_token_through_the_delta_rule():
    """Behind one token the state is k u^T with u = beta v, so o = beta v (k . q): the decay plays no part."""
    cfg = T.CONFIGS["P1"]
    m = cfg["layers"][0]["mixer"]["right"]
    w = P.random_weights(cfg, 3)
    p = "l0.mix.right"
    h = torch.randn(1, cfg["width"], dtype=F64)
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    last = lambda name: P.silu((h @ w[f"{p}.{name}"].T) * w[f"{p}.{name}.conv"][:, -1])
    q, k, v = P.unit(last("q").reshape(G, d)) * d ** -0.5, P.unit(last("k").reshape(G, d)), last("v").reshape(H, dv)
    beta = torch.sigmoid(h @ w[p + ".b"].T)[0]
    o = torch.stack([beta[i] * v[i] * (k[i // (H // G)] @ q[i // (H // G)]) for i in range(H)])
    gate = torch.sigmoid((h @ w[p + ".g1"].T) @ w[p + ".g2"].T).reshape(H, dv)
    want = (P.rms(o, 1e-5) * w[p + ".norm"] * gate).reshape(1, -1) @ w[p + ".o"].T
    assert torch.allclose(P.delta_rule(h, w, p, m, 1e-5), want)


@pytest.mark.parametrize("name", ["G1", "G2", "G4", "G5"])
def test_a_prefix_does_not_see_what_follows(name):
    cfg = T.CONFIGS[name]
    w = P.random_weights(cfg, 5)
    toks = T.tokens(cfg, 40, 1)
    whole = P.forward(cfg, w, toks)
    assert torch.allclose(P.forward(cfg, w, toks[:23]), whole[:23], atol=1e-9)
    other = toks[:30] + [(t + 1) % cfg["vocab"] for t in toks[30:]]
    assert torch.allclose(P.forward(cfg, w, other)[:30], whole[:30], atol=1e-9)


def test_a_chunk_hides_the_left_half_of_earlier_chunks_only():
    """Changing a token of an earlier chunk reaches a later position of a one-layer parallel model
    through the recurrence; with the right half's output projection zero it does not."""
    cfg = copy.deepcopy(T.CONFIGS["P1"])
    w = P.random_weights(cfg, 6)
    toks = T.tokens(cfg, 45, 2)
    other = list(toks)
    other[3] = (other[3] + 7) % cfg["vocab"]
    a, b = P.forward(cfg, w, toks), P.forward(cfg, w, other)
    assert not torch.allclose(a[41], b[41], atol=1e-6)
    w["l0.mix.right.o"] = torch.zeros_like(w["l0.mix.right.o"])
    a, b = P.forward(cfg, w, toks), P.forward(cfg, w, other)
    assert torch.allclose(a[40:], b[40:], atol=1e-9) and not torch.allclose(a[19], b[19], atol=1e-6)


# ----------------------------------------------------------------------------- configuration, builder, cache plan

def test_configuration_round_trip_and_errors():
    from kllm_amd.config import ConfigError, LugetarConfig, config_from_dict
    for name, raw in T.CONFIGS.items():
        cfg = config_from_dict(raw)
        assert isinstance(cfg, LugetarConfig) and len(cfg.layers) == len(raw["layers"])
        assert config_from_dict(cfg.to_dict()) == cfg, name
    cfg = config_from_dict(T.CONFIGS["G1"])
    assert cfg.residual_mult == 0.8 and cfg.embedding_scale == 2.5 and cfg.norm_eps == 1e-5
    left = cfg.layers[1].mixer.left
    assert (left.chunk, left.vdim, left.rot.dims, left.rot.scaling.factor) == (24, 16, 16, 4.0)
    assert cfg.layers[0].mixer.temp == (0.4, 20) and cfg.layers[0].mlp.limit == 1.2
    mlp = cfg.layers[1].mlp
    assert (mlp.experts, mlp.top, mlp.groups, mlp.keep_groups, mlp.router_scale, mlp.shared_ff) == (8, 3, 4, 2, 1.7, 40)

    def broken(change):
        raw = copy.deepcopy(T.CONFIGS["G1"])
        change(raw)
        with pytest.raises(ConfigError):
            config_from_dict(raw)
    broken(lambda r: r["layers"][0].update(type="recurrent"))
    broken(lambda r: r["layers"][0]["mixer"].update(kv_heads=3))
    broken(lambda r: r["layers"][1]["mlp"]["router"].update(top=5))          # only four experts can be chosen
    broken(lambda r: r["layers"][1]["mlp"]["router"]["groups"].update(count=3))
    broken(lambda r: r["layers"][1]["mixer"]["left"]["rot"].update(dims=34))
    broken(lambda r: r["layers"][0]["mlp"].pop("limit"))
    broken(lambda r: r["layers"][0]["mlp"].update(kind="gated"))
    broken(lambda r: r.pop("norm"))


def test_builder_names_every_tensor_and_the_cache_plan_groups_alike_layers():
    from kllm_amd.config import config_from_dict
    from kllm_amd.config.registry import resolve_architecture
    from kllm_amd.engine.model import Model, collect_weight_specs
    from kllm_amd.parts.base import Runtime
    for name, raw in T.CONFIGS.items():
        spec = resolve_architecture(raw).build(config_from_dict(raw))
        w = P.random_weights(raw, 1)
        specs = {s.name: s for s in collect_weight_specs(spec)}
        assert set(specs) == set(w), name
        for k, s in specs.items():
            assert len(s.shape) == w[k].dim() and all(a in (b, -1) for a, b in zip(s.shape, w[k].shape)), (name, k)
            assert (s.role == "matrix") == (w[k].dim() == 2 and not k.endswith(".conv")), (name, k)
    raw = T.CONFIGS["G1"]
    model = Model(resolve_architecture(raw).build(config_from_dict(raw)), Runtime(device=torch.device("cpu"), dtype=torch.float32))
    kinds = [(g.need.kind, g.entries) for g in model.cache_plan.groups]
    assert kinds == [("paged", 2), ("paged", 2), ("state", 2)]
    left = model.cache_plan.groups[1].need
    assert (left.kv_heads, left.head_dim, left.value_dim, left.window) == (2, 32, 16, 0)
    state = model.cache_plan.groups[2].need.state_shape
    assert state == (4 * 16 * 24 + (2 * 2 * 16 + 4 * 24) * 2,)              # the state, then two inputs a channel
    assert model.cache_plan.runs[1] == [(1, 0, True), (2, 0, True)] and model.cache_plan.runs[2] == (0, 1, True)
    assert model.graph_safe and model.repeatable
