"""Typed configuration of the Natenex decoder.

config.json names the architecture in ``architecture`` and gives ``vocab``, ``width``,
``embedding`` (``scale``), ``norm`` (``eps``) and ``layers``: per layer its ``type``, the sizes of
its mixer (``mixer``), its feed-forward (``mlp``: null for none, or ``kind`` "dense" with ``ff``)
and optionally ``weights_of``: the index of another layer whose tensors this layer runs with
(it keeps a cache or state of its own, and the rest of its entry equals that layer's).

Mixers by ``type``:

``parallel``: ``left`` (attention: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, optional
``rot`` {``dims``, ``base``, optional ``scaling`` {``factor``, ``low``, ``high``, ``original``}},
optional ``mask`` {``size``, ``keep_first``}), ``right`` (a gated linear recurrence: ``width``,
``blocks``, ``conv``) and the two factors ``left_scale``, ``right_scale``.

``latent_attention``: ``heads``, ``dim``, ``rot_dim``, ``vdim``, ``q_rank``, ``kv_rank``,
``scale`` and ``rot`` {``dims``, ``base``, optional ``scaling``}.

``delta``: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``conv``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .base import ConfigError, KeyReader, ModelConfig

MIXER_TYPES = ("parallel", "latent_attention", "delta")


def _number(reader: KeyReader, key: str, default=None):
    v = reader.get(key, default) if default is not None else reader.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"{reader.where}: '{key}' must be a number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class WavelengthScaling:
    factor: float
    low: float
    high: float
    original: float

    def to_dict(self):
        return {"factor": self.factor, "low": self.low, "high": self.high, "original": self.original}


@dataclass(frozen=True)
class Rotation:
    dims: int
    base: float
    scaling: Optional[WavelengthScaling] = None

    def to_dict(self):
        out = {"dims": self.dims, "base": self.base}
        if self.scaling is not None:
            out["scaling"] = self.scaling.to_dict()
        return out


def _rotation(raw, at, most) -> Rotation:
    r = KeyReader(raw, at)
    dims, base = r.positive_int("dims"), r.positive_float("base")
    if dims % 2 or dims > most:
        raise ConfigError(f"{at}: dims {dims} must be even and at most {most}")
    scaling = None
    if r.has("scaling"):
        s = KeyReader(r.get("scaling"), at + ".scaling")
        scaling = WavelengthScaling(s.positive_float("factor"), s.positive_float("low"), s.positive_float("high"),
                                    s.positive_float("original"))
        if not scaling.high > scaling.low:
            raise ConfigError(f"{at}.scaling: 'high' must be above 'low'")
    return Rotation(dims, base, scaling)


@dataclass(frozen=True)
class WindowedAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[Rotation] = None
    window: int = 0              # 0: every earlier position is read
    keep_first: int = 0

    def to_dict(self):
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        if self.window:
            out["mask"] = {"size": self.window, "keep_first": self.keep_first}
        return out


@dataclass(frozen=True)
class LinearRecurrence:
    width: int
    blocks: int
    conv: int

    def to_dict(self):
        return {"width": self.width, "blocks": self.blocks, "conv": self.conv}


@dataclass(frozen=True)
class ParallelMixer:
    left: WindowedAttention
    right: LinearRecurrence
    left_scale: float
    right_scale: float

    def to_dict(self):
        return {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class LatentMixer:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot: Rotation

    def to_dict(self):
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "q_rank": self.q_rank,
                "kv_rank": self.kv_rank, "scale": self.scale, "rot": self.rot.to_dict()}


@dataclass(frozen=True)
class DeltaMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    def to_dict(self):
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}


@dataclass(frozen=True)
class NatenexLayer:
    type: str
    mixer: object                      # ParallelMixer, LatentMixer or DeltaMixer
    ff: Optional[int] = None           # None: no feed-forward
    weights_of: Optional[int] = None   # runs with that layer's tensors

    def to_dict(self):
        out = {"type": self.type, "mixer": self.mixer.to_dict(),
               "mlp": {"kind": "dense", "ff": self.ff} if self.ff is not None else None}
        if self.weights_of is not None:
            out["weights_of"] = self.weights_of
        return out


def _heads(m: KeyReader, at):
    heads = m.positive_int("heads")
    kv = m.positive_int("kv_heads", heads)
    if heads % kv:
        raise ConfigError(f"{at}: {heads} heads are not a multiple of {kv} kv_heads")
    return heads, kv


def _attention(raw, at) -> WindowedAttention:
    m = KeyReader(raw, at)
    heads, kv = _heads(m, at)
    dim = m.positive_int("dim")
    rot = _rotation(m.get("rot"), at + ".rot", dim) if m.has("rot") else None
    window = keep = 0
    if m.has("mask"):
        k = KeyReader(m.get("mask"), at + ".mask")
        window = k.positive_int("size")
        keep = k.get("keep_first", 0)
        if isinstance(keep, bool) or not isinstance(keep, int) or keep < 0:
            raise ConfigError(f"{at}.mask: 'keep_first' must be a count, got {keep!r}")
    return WindowedAttention(heads, kv, dim, m.positive_int("vdim", dim), _number(m, "scale"), rot, window, keep)


def _mixer(kind, raw, at):
    m = KeyReader(raw, at)
    if kind == "parallel":
        r = KeyReader(m.get("right"), at + ".right")
        right = LinearRecurrence(r.positive_int("width"), r.positive_int("blocks"), r.positive_int("conv"))
        if right.width % right.blocks:
            raise ConfigError(f"{at}.right: width {right.width} does not go into {right.blocks} equal blocks")
        return ParallelMixer(_attention(m.get("left"), at + ".left"), right, _number(m, "left_scale"),
                             _number(m, "right_scale"))
    if kind == "latent_attention":
        rot_dim = m.positive_int("rot_dim")
        rot = _rotation(m.get("rot"), at + ".rot", rot_dim)
        if rot.dims != rot_dim:
            raise ConfigError(f"{at}: rot.dims {rot.dims} is not rot_dim {rot_dim}")
        return LatentMixer(m.positive_int("heads"), m.positive_int("dim"), rot_dim, m.positive_int("vdim"),
                           m.positive_int("q_rank"), m.positive_int("kv_rank"), _number(m, "scale"), rot)
    heads, kv = _heads(m, at)
    dim = m.positive_int("dim")
    return DeltaMixer(heads, kv, dim, m.positive_int("vdim", dim), m.positive_int("conv"))


@dataclass(frozen=True)
class NatenexConfig(ModelConfig):
    vocab: int = 0
    width: int = 0
    layers: Tuple[NatenexLayer, ...] = ()
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0

    @classmethod
    def from_dict(cls, raw: dict, where: str = "config.json") -> "NatenexConfig":
        r = KeyReader(raw, where)
        vocab, width = r.positive_int("vocab"), r.positive_int("width")
        eps = KeyReader(r.get("norm"), where + ":norm").positive_float("eps")
        scale = _number(KeyReader(r.get("embedding"), where + ":embedding"), "scale")
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
            mixer = _mixer(kind, e.get("mixer"), at + ".mixer")
            ff = None
            if e.has("mlp"):
                mlp = KeyReader(entry["mlp"], at + ".mlp")
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{at}.mlp: kind {mlp.get('kind')!r} is not 'dense'")
                ff = mlp.positive_int("ff")
            source = None
            if e.has("weights_of"):
                source = e.get("weights_of")
                if isinstance(source, bool) or not isinstance(source, int) or not 0 <= source < len(entries) or source == i:
                    raise ConfigError(f"{at}: 'weights_of' must name another layer, got {source!r}")
            layers.append(NatenexLayer(kind, mixer, ff, source))
        for i, layer in enumerate(layers):
            if layer.weights_of is None:
                continue
            other, at = layers[layer.weights_of], f"{where}:layers[{i}]"
            if other.weights_of is not None:
                raise ConfigError(f"{at}: 'weights_of' names layer {layer.weights_of}, which has no tensors of its own")
            if (other.type, other.mixer, other.ff) != (layer.type, layer.mixer, layer.ff):
                raise ConfigError(f"{at}: a layer that runs with layer {layer.weights_of}'s tensors has its sizes")
        return cls(architecture="Natenex", vocab=vocab, width=width, layers=tuple(layers), norm_eps=eps,
                   embedding_scale=scale)

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
                "layers": [layer.to_dict() for layer in self.layers]}
