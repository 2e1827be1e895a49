"""Typed configuration of the Lugetar decoder.

config.json names the architecture in ``architecture`` and gives ``vocab``, ``width``,
``embedding`` (``scale``), ``norm`` (``eps``), ``residual_mult`` and ``layers``: per layer its
``type``, the sizes of its mixer (``mixer``) and its feed-forward (``mlp``, null for none).

Mixers by ``type``:

``attention``: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, optional ``q_temp``
{``coef``, ``every``}, optional ``rot`` {``dims``, ``base``, optional ``scaling`` {``factor``,
``low``, ``high``, ``original``}}, optional ``mask`` {``size``}: a chunked mask.

``parallel``: ``left`` (attention, the keys above) and ``right`` (a gated delta rule: ``heads``,
``kv_heads``, ``dim``, ``vdim``, ``conv``; the inner widths of its two low-rank projections are
the checkpoint's tensors', and only a model made of random weights names them, as ``a_rank`` and
``gate_rank``).

Feed-forwards by ``kind``: ``dense`` {``ff``, ``limit``}; ``moe`` {``expert`` {``ff``}, ``router``
{``experts``, ``top``, optional ``scale``, optional ``groups`` {``count``, ``keep``}}, optional
``shared`` {``ff``}}.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .base import ConfigError, KeyReader, ModelConfig
from .natenex import Rotation, _heads, _number, _rotation

MIXER_TYPES = ("attention", "parallel")
MLP_KINDS = ("dense", "moe")


@dataclass(frozen=True)
class LugetarAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[Rotation] = None
    chunk: int = 0                               # 0: every earlier position is read
    temp: Optional[Tuple[float, int]] = None     # (coef, every) of the query temperature

    def to_dict(self):
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        if self.chunk:
            out["mask"] = {"size": self.chunk}
        if self.temp is not None:
            out["q_temp"] = {"coef": self.temp[0], "every": self.temp[1]}
        return out


@dataclass(frozen=True)
class LugetarDelta:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    a_rank: Optional[int] = None       # inner widths of the two low-rank projections; None: the checkpoint's
    gate_rank: Optional[int] = None

    def to_dict(self):
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}
        if self.a_rank is not None:
            out["a_rank"] = self.a_rank
        if self.gate_rank is not None:
            out["gate_rank"] = self.gate_rank
        return out


@dataclass(frozen=True)
class LugetarParallel:
    left: LugetarAttention
    right: LugetarDelta

    def to_dict(self):
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


@dataclass(frozen=True)
class LugetarMlp:
    kind: str                          # "dense" or "moe"
    ff: int                            # of the dense layer, or of one expert
    limit: float = 0.0                 # dense: the gate's clamp
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep_groups: int = 1
    router_scale: float = 1.0
    shared_ff: Optional[int] = None

    def to_dict(self):
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff, "limit": self.limit}
        router = {"experts": self.experts, "top": self.top, "scale": self.router_scale}
        if self.groups > 1:
            router["groups"] = {"count": self.groups, "keep": self.keep_groups}
        out = {"kind": "moe", "expert": {"ff": self.ff}, "router": router}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


@dataclass(frozen=True)
class LugetarLayer:
    type: str
    mixer: object                      # LugetarAttention or LugetarParallel
    mlp: Optional[LugetarMlp] = None

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None}


def _attention(raw, at) -> LugetarAttention:
    m = KeyReader(raw, at)
    heads, kv = _heads(m, at)
    dim = m.positive_int("dim")
    rot = _rotation(m.get("rot"), at + ".rot", dim) if m.has("rot") else None
    chunk = KeyReader(m.get("mask"), at + ".mask").positive_int("size") if m.has("mask") else 0
    temp = None
    if m.has("q_temp"):
        t = KeyReader(m.get("q_temp"), at + ".q_temp")
        temp = (_number(t, "coef"), t.positive_int("every"))
    return LugetarAttention(heads, kv, dim, m.positive_int("vdim", dim), _number(m, "scale"), rot, chunk, temp)


def _delta(raw, at) -> LugetarDelta:
    m = KeyReader(raw, at)
    heads, kv = _heads(m, at)
    dim = m.positive_int("dim")
    return LugetarDelta(heads, kv, dim, m.positive_int("vdim", dim), m.positive_int("conv"),
                        m.positive_int("a_rank", None), m.positive_int("gate_rank", None))


def _mlp(raw, at) -> LugetarMlp:
    m = KeyReader(raw, at)
    kind = m.get("kind", "dense")
    if kind not in MLP_KINDS:
        raise ConfigError(f"{at}: kind {kind!r} is not one of {MLP_KINDS}")
    if kind == "dense":
        return LugetarMlp("dense", m.positive_int("ff"), limit=m.positive_float("limit"))
    ff = KeyReader(m.get("expert"), at + ".expert").positive_int("ff")
    r = KeyReader(m.get("router"), at + ".router")
    experts, top = r.positive_int("experts"), r.positive_int("top")
    groups = keep = 1
    if r.has("groups"):
        g = KeyReader(r.get("groups"), at + ".router.groups")
        groups = g.positive_int("count")
        keep = g.positive_int("keep", groups)
        if experts % groups or keep > groups:
            raise ConfigError(f"{at}.router.groups: {experts} experts in {groups} equal groups, of which {keep} are kept")
    if top > experts // groups * keep:
        raise ConfigError(f"{at}.router: top {top} of the {experts // groups * keep} experts that can be chosen")
    shared = KeyReader(m.get("shared"), at + ".shared").positive_int("ff") if m.has("shared") else None
    return LugetarMlp("moe", ff, experts=experts, top=top, groups=groups, keep_groups=keep,
                      router_scale=_number(r, "scale", 1.0), shared_ff=shared)


@dataclass(frozen=True)
class LugetarConfig(ModelConfig):
    vocab: int = 0
    width: int = 0
    layers: Tuple[LugetarLayer, ...] = ()
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    residual_mult: float = 1.0

    @classmethod
    def from_dict(cls, raw: dict, where: str = "config.json") -> "LugetarConfig":
        r = KeyReader(raw, where)
        vocab, width = r.positive_int("vocab"), r.positive_int("width")
        eps = KeyReader(r.get("norm"), where + ":norm").positive_float("eps")
        scale = _number(KeyReader(r.get("embedding"), where + ":embedding"), "scale") if r.has("embedding") else 1.0
        mult = _number(r, "residual_mult", 1.0)
        entries = r.get("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError(f"{where}: 'layers' must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(entries):
            at = f"{where}:layers[{i}]"
            e = KeyReader(entry, at)
            kind = e.get("type")
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{at}: type {kind!r} is not one of {MIXER_TYPES}")
            if kind == "parallel":
                m = KeyReader(e.get("mixer"), at + ".mixer")
                mixer = LugetarParallel(_attention(m.get("left"), at + ".mixer.left"), _delta(m.get("right"), at + ".mixer.right"))
            else:
                mixer = _attention(e.get("mixer"), at + ".mixer")
            layers.append(LugetarLayer(kind, mixer, _mlp(entry["mlp"], at + ".mlp") if e.has("mlp") else None))
        return cls(architecture="Lugetar", vocab=vocab, width=width, layers=tuple(layers), norm_eps=eps,
                   embedding_scale=scale, residual_mult=mult)

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
                "residual_mult": self.residual_mult, "layers": [layer.to_dict() for layer in self.layers]}
