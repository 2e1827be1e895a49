"""Arrangements of a layer's parts.

``pre_norm``: a = h + Mixer(Norm1(h)); h' = a + FeedForward(Norm2(a))
(backend/model.cu:1083-1117).  As in the reference, a sub-layer's output is
not added to the residual stream by a pass of its own: it travels as
``pending`` into the next norm, which adds it while it normalises (:1084,
:1105, :1117).  For decode batches even that launch goes: where the parts
allow it, a sub-layer's last product adds its sums to the stream in its
epilogue (``ResidualSink``) and the next sub-layer's first product applies the
norm's row scale to its own sums (``Normed``).
"""

from __future__ import annotations

from .. import kernels as K
from .base import Part, ResidualSink, ScaledSum, call_part, make_part, register_part, stream_copy


@register_part("block", "pre_norm")
class PreNormBlock(Part):
    records_launches = True     # the arrangement itself launches nothing; its parts are called each in its own way

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        layer = self.param("layer")
        self.norm_mixer = make_part("norm", layer.norm_mixer, runtime)
        self.mixer = make_part("mixer", layer.mixer, runtime)
        self.norm_ff = make_part("norm", layer.norm_feed_forward, runtime)
        self.feed_forward = make_part("feed_forward", layer.feed_forward, runtime)

    def parts(self):
        return [self.norm_mixer, self.mixer, self.norm_ff, self.feed_forward]

    def children(self):
        return self.parts()

    @property
    def graph_safe(self):
        return all(p.graph_safe for p in self.parts())

    def weight_specs(self):
        return [s for p in self.parts() for s in p.weight_specs()]

    def bind(self, weights):
        for p in self.parts():
            p.bind(weights)

    def cache_need(self):
        return self.mixer.cache_need()

    def read_bytes(self, tokens):
        out = {}
        for p in self.parts():
            out.update(p.read_bytes(tokens))
        return out

    def flops(self, tokens, keys_read=0.0):
        return sum(p.flops(tokens, keys_read) for p in self.parts())

    takes_next_norm = True

    def first_norm(self):
        """The norm that takes what the layer before this one leaves pending."""
        return self.norm_mixer

    @staticmethod
    def _normed_ok(ctx, norm, consumer):
        return {"normed_ok": True} if (norm.fusable and consumer.takes_normed and ctx.taps is None) else {}

    @staticmethod
    def _sink(ctx, x, producer, norm):
        if norm is None or not (producer.fills_sink and norm.fusable) or ctx.taps is not None:
            return {}
        return {"sink": ResidualSink(x, norm)}

    def forward(self, ctx, x, pending, cache, next_norm=None):
        """``next_norm``: the norm that will take this layer's pending output
        (the next layer's first norm), if the caller knows it; the feed-forward
        may then add its output to x itself."""
        xn = call_part(self.norm_mixer, self.norm_mixer.forward, ctx, x, delta=pending,
                       **self._normed_ok(ctx, self.norm_mixer, self.mixer))
        delta = call_part(self.mixer, self.mixer.forward, ctx, xn, cache, **self._sink(ctx, x, self.mixer, self.norm_ff))
        xn = call_part(self.norm_ff, self.norm_ff.forward, ctx, x, delta=delta,
                       **self._normed_ok(ctx, self.norm_ff, self.feed_forward))
        pending = call_part(self.feed_forward, self.feed_forward.forward, ctx, xn,
                            **self._sink(ctx, x, self.feed_forward, next_norm))
        return x, pending


@register_part("block", "parallel")
class ParallelBlock(Part):
    """Mixer and feed-forward side by side behind one norm: with h = Norm(x),
    x' = x + mult * (Mixer(h) + FeedForward(h)).  The layer may have no feed-forward.  Neither
    output is added by a pass of its own: both travel, with the factor and the bias of a
    sub-layer's last projection (``out_bias`` of a part, if it has one), as a ``ScaledSum``
    into the next norm.

    Parameters: ``layer`` (its ``norm_mixer`` is the one norm), ``mult`` (default 1)."""
    records_launches = True

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        layer = self.param("layer")
        self.mult = float(self.param("mult", 1.0))
        self.norm = make_part("norm", layer.norm_mixer, runtime)
        self.mixer = make_part("mixer", layer.mixer, runtime)
        self.feed_forward = (make_part("feed_forward", layer.feed_forward, runtime)
                             if layer.feed_forward is not None else None)
        self.bias = None

    def parts(self):
        return [p for p in (self.norm, self.mixer, self.feed_forward) if p is not None]

    def children(self):
        return self.parts()

    @property
    def graph_safe(self):
        return all(p.graph_safe for p in self.parts())

    def weight_specs(self):
        return [s for p in self.parts() for s in p.weight_specs()]

    def bind(self, weights):
        for p in self.parts():
            p.bind(weights)
        biases = [b for b in (getattr(p, "out_bias", None) for p in self.parts()) if b is not None]
        self.bias = None
        if biases:
            self.bias = biases[0] if len(biases) == 1 else sum(biases[1:], biases[0].clone())

    def cache_need(self):
        return self.mixer.cache_need()

    def read_bytes(self, tokens):
        out = {}
        for p in self.parts():
            out.update(p.read_bytes(tokens))
        return out

    def flops(self, tokens, keys_read=0.0):
        return sum(p.flops(tokens, keys_read) for p in self.parts())

    def first_norm(self):
        return self.norm

    def forward(self, ctx, x, pending, cache):
        xn = call_part(self.norm, self.norm.forward, ctx, x, delta=pending)
        deltas = [call_part(self.mixer, self.mixer.forward, ctx, xn, cache)]
        if self.feed_forward is not None:
            deltas.append(call_part(self.feed_forward, self.feed_forward.forward, ctx, xn))
        return x, ScaledSum(deltas, self.bias, self.mult)


@register_part("block", "sublayer_norm")
class SublayerNormBlock(Part):
    """The norm stands behind each sub-layer, on its output alone, and the sub-layers read the
    stream itself: a = x + Norm1(Mixer(x)); x' = a + Norm2(FeedForward(a)).  The layer may have
    no feed-forward.  Both norms are RMS norms with ``weight`` and ``eps``; each is one launch
    that adds the sums of the sub-layer's last product (and its bias, ``out_bias`` of a part),
    normalises, adds to the float32 stream and leaves the stream's new rows in the compute
    dtype for the next sub-layer.  Nothing stays pending behind the layer.

    Parameters: ``layer``."""
    records_launches = True

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        layer = self.param("layer")
        self.mixer = make_part("mixer", layer.mixer, runtime)
        self.norm_mixer = make_part("norm", layer.norm_mixer, runtime)
        self.feed_forward = (make_part("feed_forward", layer.feed_forward, runtime)
                             if layer.feed_forward is not None else None)
        self.norm_ff = make_part("norm", layer.norm_feed_forward, runtime) if self.feed_forward is not None else None
        for norm in (self.norm_mixer, self.norm_ff):
            if norm is not None and not (hasattr(norm, "weight") and hasattr(norm, "eps") and getattr(norm, "groups", 1) == 1):
                raise ValueError("sublayer_norm: its norms are RMS norms with a weight and eps")

    def parts(self):
        return [p for p in (self.mixer, self.norm_mixer, self.feed_forward, self.norm_ff) if p is not None]

    def children(self):
        return self.parts()

    @property
    def graph_safe(self):
        return all(p.graph_safe for p in self.parts())

    def weight_specs(self):
        return [s for p in self.parts() for s in p.weight_specs()]

    def bind(self, weights):
        for p in self.parts():
            p.bind(weights)

    def cache_need(self):
        return self.mixer.cache_need()

    def read_bytes(self, tokens):
        out = {}
        for p in self.parts():
            out.update(p.read_bytes(tokens))
        return out

    def flops(self, tokens, keys_read=0.0):
        return sum(p.flops(tokens, keys_read) for p in self.parts())

    def forward(self, ctx, x, pending, cache):
        if pending is not None:
            raise ValueError("sublayer_norm: the layer in front of it left sums pending, which it has no norm for")
        xin = stream_copy(ctx, x)
        delta = call_part(self.mixer, self.mixer.forward, ctx, xin, cache)
        out = stream_copy(ctx, x, fill=False)
        K.norm_residual(x, self.norm_mixer.weight, delta, bias=getattr(self.mixer, "out_bias", None), out=out,
                        eps=self.norm_mixer.eps)
        if self.feed_forward is not None:
            xin = stream_copy(ctx, x)
            # a routed feed-forward's weighted sum over the chosen experts is taken in the norm's launch
            more = {"sums_ok": True} if getattr(self.feed_forward, "leaves_chosen_sums", False) else {}
            delta = call_part(self.feed_forward, self.feed_forward.forward, ctx, xin, **more)
            K.norm_residual(x, self.norm_ff.weight, delta, bias=getattr(self.feed_forward, "out_bias", None), out=out,
                            eps=self.norm_ff.eps)
        return x, None


@register_part("block", "sandwich_norm")
class SandwichNormBlock(Part):
    """A norm in front of and behind each sub-layer: a = x + mult * NormB1(Mixer(Norm1(x)));
    x' = a + mult * NormB2(FeedForward(Norm2(a))).  The layer may have no feed-forward.  All four
    are RMS norms with ``weight`` and ``eps``.  The norm behind a sub-layer is one launch that adds
    the sums of the sub-layer's last product (and its bias, ``out_bias`` of a part), normalises,
    adds to the float32 stream and, behind the mixer, also leaves the rows of the norm in front of
    the feed-forward (the new row is still in registers).  Nothing stays pending behind the layer.

    Parameters: ``layer`` (its ``norm_mixer`` and ``norm_feed_forward`` stand in front, its
    ``norm_mixer_out`` and ``norm_feed_forward_out`` behind), ``mult`` (default 1)."""
    records_launches = True

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        layer = self.param("layer")
        self.mult = float(self.param("mult", 1.0))
        if layer.norm_mixer is None or layer.norm_mixer_out is None:
            raise ValueError("sandwich_norm: the mixer has a norm in front of it and one behind it")
        self.norm_mixer = make_part("norm", layer.norm_mixer, runtime)
        self.mixer = make_part("mixer", layer.mixer, runtime)
        self.norm_mixer_out = make_part("norm", layer.norm_mixer_out, runtime)
        self.feed_forward = self.norm_ff = self.norm_ff_out = None
        if layer.feed_forward is not None:
            if layer.norm_feed_forward is None or layer.norm_feed_forward_out is None:
                raise ValueError("sandwich_norm: the feed-forward has a norm in front of it and one behind it")
            self.norm_ff = make_part("norm", layer.norm_feed_forward, runtime)
            self.feed_forward = make_part("feed_forward", layer.feed_forward, runtime)
            self.norm_ff_out = make_part("norm", layer.norm_feed_forward_out, runtime)
        for norm in (self.norm_mixer, self.norm_mixer_out, self.norm_ff, self.norm_ff_out):
            if norm is not None and not (hasattr(norm, "weight") and hasattr(norm, "eps") and getattr(norm, "groups", 1) == 1):
                raise ValueError("sandwich_norm: its norms are RMS norms with a weight and eps")

    def parts(self):
        return [p for p in (self.norm_mixer, self.mixer, self.norm_mixer_out, self.norm_ff, self.feed_forward,
                            self.norm_ff_out) if p is not None]

    def children(self):
        return self.parts()

    @property
    def graph_safe(self):
        return all(p.graph_safe for p in self.parts())

    def weight_specs(self):
        return [s for p in self.parts() for s in p.weight_specs()]

    def bind(self, weights):
        for p in self.parts():
            p.bind(weights)

    def cache_need(self):
        return self.mixer.cache_need()

    def read_bytes(self, tokens):
        out = {}
        for p in self.parts():
            out.update(p.read_bytes(tokens))
        return out

    def flops(self, tokens, keys_read=0.0):
        return sum(p.flops(tokens, keys_read) for p in self.parts())

    def first_norm(self):
        return self.norm_mixer

    def forward(self, ctx, x, pending, cache):
        if pending is not None:
            raise ValueError("sandwich_norm: the layer in front of it left sums pending, which it has no norm for")
        xn = call_part(self.norm_mixer, self.norm_mixer.forward, ctx, x)
        behind = self.norm_mixer_out
        # two mixers side by side whose outputs are normed before they are added: in the norm's launch
        more = {"pair_eps": behind.eps} if getattr(self.mixer, "leaves_normed_pair", False) else {}
        delta = call_part(self.mixer, self.mixer.forward, ctx, xn, cache, **more)
        if self.feed_forward is None:
            K.norm_residual(x, behind.weight, delta, bias=getattr(self.mixer, "out_bias", None), eps=behind.eps,
                            mult=self.mult)
            return x, None
        if self.norm_ff.eps == behind.eps:
            # the norm in front of the feed-forward in the same launch
            xn = ctx.buf("xn", tuple(x.shape), self.runtime.dtype)
            K.norm_residual(x, behind.weight, delta, bias=getattr(self.mixer, "out_bias", None), eps=behind.eps,
                            mult=self.mult, out=xn, next_weight=self.norm_ff.weight)
        else:
            K.norm_residual(x, behind.weight, delta, bias=getattr(self.mixer, "out_bias", None), eps=behind.eps,
                            mult=self.mult)
            xn = call_part(self.norm_ff, self.norm_ff.forward, ctx, x)
        # a routed feed-forward's weighted sum over the chosen experts is taken in the norm's launch
        more = {"sums_ok": True} if getattr(self.feed_forward, "leaves_chosen_sums", False) else {}
        delta = call_part(self.feed_forward, self.feed_forward.forward, ctx, xn, **more)
        behind = self.norm_ff_out
        K.norm_residual(x, behind.weight, delta, bias=getattr(self.feed_forward, "out_bias", None), eps=behind.eps,
                        mult=self.mult)
        return x, None
