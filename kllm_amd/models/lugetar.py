"""The Lugetar decoder, put together from parts.

Token embedding times a constant; layers in the order the configuration lists them, each with a
norm in front of and behind both sub-layers (a = x + m NormB1(Mixer(Norm1(x))), x' = a + m
NormB2(FeedForward(Norm2(a)))).  A mixer is one of two.  ``attention``: queries and keys normed
over the whole projection, a query temperature that grows with the position, no rotation,
causal.  ``parallel``: such attention with a rotation of each head's first elements behind the
norm (slow pairs slowed down further by wavelength) and a chunked mask, side by side with a gated
delta rule behind short convolutions whose decay has one number per head and key channel and whose
decay and output gate come through low-rank projections; each half's output passes an RMS norm
over the model's width, and the mixer's output is half their sum.  The feed-forward is dense with
a clamped gate, or a mixture of SiLU-gated experts (logistic scores, the choice limited to the
best groups of neighbouring experts, the chosen scores times a constant, a shared expert behind a
gate of its own), or absent.  A final norm, and the embedding table, unscaled, as the output
matrix.  Tensor names: ``embed``, ``l<i>.norm1``, ``.norm1b``, ``.norm2``, ``.norm2b``,
``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``.
"""

from __future__ import annotations

from ..config.lugetar import LugetarConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, Run

# The dense feed-forward's gate is g sigmoid(SWISH_ALPHA g) (u + 1) behind its clamps.
SWISH_ALPHA = 1.702
# Queries and keys of the delta rule become x / sqrt(sum(x^2) + DELTA_UNIT_EPS).
DELTA_UNIT_EPS = 1e-6
# The two halves of a parallel mixer are added with these factors behind their norms.
HALF = 0.5


def build_lugetar(cfg: LugetarConfig) -> ModelSpec:
    d = cfg.width

    def norm(name):
        return PartSpec("rmsnorm", size=d, eps=cfg.norm_eps, names={"weight": name})

    positions = {}      # mixers that rotate alike share one position part (and its tables of a step)

    def position(rot):
        if rot is None:
            return None
        s = rot.scaling
        key = (rot.dims, rot.base, s)
        if key not in positions:
            positions[key] = PartSpec("rotary_scaled", rotary_dim=rot.dims, base=rot.base, interleaved=False,
                                      scaling=("by_wavelength", s.factor, s.low, s.high, s.original) if s else None)
        return positions[key]

    def attention(p, a):
        names = {f"{t}.weight": f"{p}.{t}" for t in ("q", "k", "v", "o")}
        names.update({"q.norm": f"{p}.q.norm", "k.norm": f"{p}.k.norm"})
        return PartSpec("attention_whole_norm", p, hidden=d, heads=a.heads, kv_heads=a.kv_heads, head_dim=a.dim,
                        value_dim=a.vdim, scale=a.scale, eps=cfg.norm_eps, position=position(a.rot), chunk=a.chunk,
                        q_temp=a.temp, names=names)

    def delta(p, m):
        names = {f"{t}.weight": f"{p}.{t}" for t in ("q", "k", "v", "b", "a1", "a2", "g1", "g2", "o")}
        names.update({f"{t}.conv": f"{p}.{t}.conv" for t in ("q", "k", "v")})
        names.update({"A_log": f"{p}.A_log", "dt_bias": f"{p}.dt_bias", "norm": f"{p}.norm"})
        return PartSpec("gated_delta", p, hidden=d, heads=m.heads, kv_heads=m.kv_heads, head_dim=m.dim,
                        value_dim=m.vdim, taps=m.conv, eps=cfg.norm_eps, unit_eps=DELTA_UNIT_EPS, channel_decay=True,
                        low_rank=True, a_rank=m.a_rank, gate_rank=m.gate_rank, gate="sigmoid", names=names)

    layers = []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.mix", layer.mixer
        if layer.type == "parallel":
            mixer = PartSpec("mixer_sum", p, left=attention(p + ".left", m.left), right=delta(p + ".right", m.right),
                             left_scale=HALF, right_scale=HALF, norm_eps=cfg.norm_eps, hidden=d)
        else:
            mixer = attention(p, m)
        ff = None
        mlp = layer.mlp
        if mlp is not None:
            f = f"l{i}.mlp"
            if mlp.kind == "dense":
                ff = PartSpec("gated_mlp_bias", f, hidden=d, intermediate=mlp.ff, activation="clamped_swish",
                              limit=mlp.limit, alpha=SWISH_ALPHA, bias=False,
                              names={f"{t}.weight": f"{f}.{t}" for t in ("gate", "up", "down")})
            else:
                ff = PartSpec("routed_experts", f, hidden=d, experts=mlp.experts, top=mlp.top, intermediate=mlp.ff,
                              activation="silu", correction=False, scoring="sigmoid", groups=mlp.groups,
                              keep_groups=mlp.keep_groups, renormalize=False, weight_scale=mlp.router_scale,
                              shared_intermediate=mlp.shared_ff, shared_gate=mlp.shared_ff is not None)
        layers.append(LayerSpec(mixer=mixer, feed_forward=ff, norm_mixer=norm(f"l{i}.norm1"),
                                norm_mixer_out=norm(f"l{i}.norm1b"),
                                norm_feed_forward=norm(f"l{i}.norm2") if ff is not None else None,
                                norm_feed_forward_out=norm(f"l{i}.norm2b") if ff is not None else None,
                                block="sandwich_norm", block_params={"mult": cfg.residual_mult}))
    return ModelSpec(
        embedding=PartSpec("token_embedding", vocab=cfg.vocab, hidden=d, scale=cfg.embedding_scale,
                           names={"weight": "embed"}),
        layers=layers,
        schedule=[Run(i) for i in range(len(layers))],
        final_norm=norm("final.norm"),
        head=PartSpec("linear_head", vocab=cfg.vocab, hidden=d, names={"weight": "embed"}),
        vocab_size=cfg.vocab,
        hidden_size=d,
    )


register_architecture("Lugetar", LugetarConfig, build_lugetar)
