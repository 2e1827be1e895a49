"""The Natenex decoder, put together from parts.

Token embedding times a constant; layers in the order the configuration lists them, each with
its norm behind the sub-layer (a = x + Norm1(Mixer(x)), x' = a + Norm2(FeedForward(a)), the
sub-layers reading the stream itself).  A mixer is one of three: attention behind a window that
keeps the first positions, with a weighted norm of queries and keys in front of a partial rotation
whose slow pairs may be slowed down further, side by side with a gated linear recurrence (their
scaled sum); attention through low-rank latents with an output gate; a gated delta rule behind
short convolutions.  The feed-forward is dense with the square of the rectifier, or absent.  A
layer may run with an earlier layer's tensors and a cache or state of its own: it is that layer,
listed once more in the running order.  A final norm, and the embedding table, unscaled, as the
output matrix.  Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``,
``l<i>.mlp.*``, ``final.norm``.
"""

from __future__ import annotations

from ..config.natenex import NatenexConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, Run

# log a = -RECURRENCE_DECAY_SCALE * r * softplus(lam) in the gated linear recurrence.
RECURRENCE_DECAY_SCALE = 8.0
# Queries and keys of the delta rule become x / sqrt(sum(x^2) + DELTA_UNIT_EPS).
DELTA_UNIT_EPS = 1e-6


def build_natenex(cfg: NatenexConfig) -> ModelSpec:
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
        return PartSpec("attention_qk_norm", p, hidden=d, heads=a.heads, kv_heads=a.kv_heads, head_dim=a.dim,
                        value_dim=a.vdim, scale=a.scale, eps=cfg.norm_eps, position=position(a.rot), window=a.window,
                        keep_first=a.keep_first, names=names)

    def recurrence(p, r):
        names = {f"{t}.weight": f"{p}.{t}" for t in ("y", "x", "o")}
        names.update({"y.bias": f"{p}.y.b", "x.bias": f"{p}.x.b", "conv": f"{p}.conv", "conv.bias": f"{p}.conv.b",
                      "ra": f"{p}.ra", "ra.bias": f"{p}.ra.b", "ri": f"{p}.ri", "ri.bias": f"{p}.ri.b", "lam": f"{p}.lam"})
        return PartSpec("linear_recurrence", p, hidden=d, width=r.width, blocks=r.blocks, taps=r.conv,
                        decay_scale=RECURRENCE_DECAY_SCALE, names=names)

    # a layer that runs with another's tensors is that layer, listed once more in the running order
    # (its own cache or state, no tensors)
    own = [i for i, layer in enumerate(cfg.layers) if layer.weights_of is None]
    index_of = {i: k for k, i in enumerate(own)}
    schedule = [Run(index_of[i if layer.weights_of is None else layer.weights_of]) for i, layer in enumerate(cfg.layers)]
    layers = []
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        p, m = f"l{i}.mix", layer.mixer
        if layer.type == "parallel":
            mixer = PartSpec("mixer_sum", p, left=attention(p + ".left", m.left), right=recurrence(p + ".right", m.right),
                             left_scale=m.left_scale, right_scale=m.right_scale)
        elif layer.type == "latent_attention":
            names = {f"{t}.weight": f"{p}.{t}" for t in ("dq", "uq", "dkv", "uk", "uv", "g", "o")}
            names.update({"dq.norm": f"{p}.dq.norm", "dkv.norm": f"{p}.dkv.norm"})
            mixer = PartSpec("latent_attention", p, hidden=d, heads=m.heads, head_dim=m.dim, rot_dim=m.rot_dim,
                             value_dim=m.vdim, q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale, eps=cfg.norm_eps,
                             position=position(m.rot), names=names)
        else:
            names = {f"{t}.weight": f"{p}.{t}" for t in ("q", "k", "v", "b", "a", "g", "o")}
            names.update({f"{t}.conv": f"{p}.{t}.conv" for t in ("q", "k", "v")})
            names.update({"A_log": f"{p}.A_log", "dt_bias": f"{p}.dt_bias", "norm": f"{p}.norm"})
            mixer = PartSpec("gated_delta", p, hidden=d, heads=m.heads, kv_heads=m.kv_heads, head_dim=m.dim,
                             value_dim=m.vdim, taps=m.conv, eps=cfg.norm_eps, unit_eps=DELTA_UNIT_EPS, names=names)
        ff = None
        if layer.ff is not None:
            f = f"l{i}.mlp"
            ff = PartSpec("dense_mlp", f, hidden=d, intermediate=layer.ff, activation="relu2",
                          names={"up.weight": f"{f}.up", "down.weight": f"{f}.down"})
        layers.append(LayerSpec(mixer=mixer, feed_forward=ff, norm_mixer=norm(f"l{i}.norm1"),
                                norm_feed_forward=norm(f"l{i}.norm2") if ff is not None else None,
                                block="sublayer_norm"))
    return ModelSpec(
        embedding=PartSpec("token_embedding", vocab=cfg.vocab, hidden=d, scale=cfg.embedding_scale, stream_rows=True,
                           names={"weight": "embed"}),
        layers=layers,
        schedule=schedule,
        final_norm=norm("final.norm"),
        head=PartSpec("linear_head", vocab=cfg.vocab, hidden=d, names={"weight": "embed"}),
        vocab_size=cfg.vocab,
        hidden_size=d,
    )


register_architecture("Natenex", NatenexConfig, build_natenex)
