"""Recurrent mixers whose input passes a short causal convolution, and a mixer that adds two.

``gated_delta``: a matrix state per head under the gated delta rule.  q = W_q h and k = W_k h
(``kv_heads`` heads of ``head_dim``), v = W_v h (``heads`` of ``value_dim``), head h reading q/k
head h // (heads / kv_heads); each passes a convolution over time per channel (``taps``
weights, the last one the current token's, zeros before position 0) and SiLU; q and k become
unit vectors per head (x / sqrt(sum x^2 + unit_eps)), q also times head_dim^-1/2;
beta = sigmoid(W_b h), g = exp(-exp(A_log) softplus(W_a h + dt_bias)), one of each a head;

    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

each head's o is divided by its root mean square (``eps``), multiplied by a weight of
``value_dim`` that the heads share and by silu(W_g h), and projected by W_o.
Tensors: ``<prefix>.{q,k,v,b,a,g,o}.weight``, ``.{q,k,v}.conv``, ``.A_log``, ``.dt_bias``, ``.norm``.
Variants, each a parameter: ``channel_decay``: g has one number per head and key channel (a row
of S each), g = exp(-exp(A_log_h) softplus(a + dt_bias)) with a and dt_bias ``heads`` x
``head_dim`` long; ``low_rank``: the decay's and the output gate's projections are products of
two matrices, W_a2 (W_a1 h) and W_g2 (W_g1 h) (tensors ``.{a1,a2,g1,g2}.weight``; the inner widths
are the checkpoint's, or ``a_rank`` and ``gate_rank``); ``gate``: "silu" or "sigmoid".

``linear_recurrence``: a state per channel.  Two branches of ``width`` channels, y = gelu_tanh(W_y
h + b_y) and u = conv(W_x h + b_x) + b_c; u is cut into ``blocks`` equal parts, each with two
square gate matrices: r = sigmoid(A_r u + b_r), i = sigmoid(A_i u + b_i); log a = -decay_scale r
softplus(lam); S <- a S + sqrt(1 - a^2) i u; the output is W_o (S * y).
Tensors: ``<prefix>.{y,x,o}.weight``, ``.{y,x}.bias``, ``.conv``, ``.conv.bias``, ``.{ra,ri}``,
``.{ra,ri}.bias``, ``.lam``.

Both keep, per request, a 32-bit state in one slot: the recurrence's state followed by the
convolution's inputs of the last ``taps - 1`` positions; it starts from zero at position 0.
Everything that enters a recurrence besides the projections' sums is 32-bit.

``mixer_sum``: two mixers side by side on the same input, ``left_scale * left + right_scale *
right``; each keeps its own cache or state.  With ``norm_eps`` each output first passes an RMS norm
over the model's width with a weight of its own.
"""

from __future__ import annotations

import torch

from .. import kernels as K
from .base import Part, ScaledSum, call_part, make_part, register_part
from .linear import decode_linear, tiled_copy
from .spec import CacheNeed, WeightSpec

MAX_TAPS = 16


@register_part("mixer", "gated_delta")
class GatedDeltaMixer(Part):
    graph_safe = True
    records_launches = True

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.hidden = int(self.param("hidden"))
        self.heads = int(self.param("heads"))
        self.kv_heads = int(self.param("kv_heads", self.heads))
        self.head_dim = int(self.param("head_dim"))
        self.value_dim = int(self.param("value_dim", self.head_dim))
        self.taps = int(self.param("taps"))
        self.eps = float(self.param("eps"))
        self.unit_eps = float(self.param("unit_eps", 1e-6))
        if self.heads % self.kv_heads:
            raise ValueError(f"gated_delta: {self.heads} heads are not a multiple of {self.kv_heads} key heads")
        if not 1 <= self.taps <= MAX_TAPS:
            raise ValueError(f"gated_delta: a convolution of {self.taps} taps is not built (1 to {MAX_TAPS})")
        self.channel_decay = bool(self.param("channel_decay", False))
        self.low_rank = bool(self.param("low_rank", False))
        self.a_rank = int(self.param("a_rank", None) or -1)
        self.gate_rank = int(self.param("gate_rank", None) or -1)
        gate = self.param("gate", "silu")
        if gate not in ("silu", "sigmoid"):
            raise ValueError(f"gated_delta: gate {gate!r} is not built (silu, sigmoid)")
        self.gate_sigmoid = gate == "sigmoid"
        self.decays = self.heads * self.head_dim if self.channel_decay else self.heads    # numbers of a token's decay
        self.w_a2 = None
        self.qk = self.kv_heads * self.head_dim
        self.hv = self.heads * self.value_dim
        self.channels = 2 * self.qk + self.hv                 # what passes the convolution
        self.state_floats = self.heads * self.head_dim * self.value_dim
        self.w_in = self.w_o = self.conv = self.a_log = self.dt_bias = self.norm_weight = None
        self._tiled = {}

    def weight_specs(self):
        d = self.hidden
        specs = [WeightSpec(self.tensor_name("q.weight"), (self.qk, d)), WeightSpec(self.tensor_name("k.weight"), (self.qk, d)),
                 WeightSpec(self.tensor_name("v.weight"), (self.hv, d)), WeightSpec(self.tensor_name("b.weight"), (self.heads, d)),
                 WeightSpec(self.tensor_name("o.weight"), (d, self.hv)),
                 WeightSpec(self.tensor_name("q.conv"), (self.qk, self.taps), "vector"),
                 WeightSpec(self.tensor_name("k.conv"), (self.qk, self.taps), "vector"),
                 WeightSpec(self.tensor_name("v.conv"), (self.hv, self.taps), "vector"),
                 WeightSpec(self.tensor_name("A_log"), (self.heads,), "vector"),
                 WeightSpec(self.tensor_name("dt_bias"), (self.decays,), "vector"),
                 WeightSpec(self.tensor_name("norm"), (self.value_dim,), "vector")]
        if self.low_rank:
            specs += [WeightSpec(self.tensor_name("a1.weight"), (self.a_rank, d)),
                      WeightSpec(self.tensor_name("a2.weight"), (self.decays, self.a_rank)),
                      WeightSpec(self.tensor_name("g1.weight"), (self.gate_rank, d)),
                      WeightSpec(self.tensor_name("g2.weight"), (self.hv, self.gate_rank))]
        else:
            specs += [WeightSpec(self.tensor_name("a.weight"), (self.decays, d)),
                      WeightSpec(self.tensor_name("g.weight"), (self.hv, d))]
        return specs

    def bind(self, weights):
        w = lambda n: weights[self.tensor_name(n)]
        if self.low_rank:
            # one product for q, k, v, b and the inner halves of the two low-rank projections
            self.a_rank, self.gate_rank = w("a1.weight").shape[0], w("g1.weight").shape[0]
            if w("a2.weight").shape[1] != self.a_rank or w("g2.weight").shape[1] != self.gate_rank:
                raise ValueError("gated_delta: the two halves of a low-rank projection do not fit each other")
            self.w_in = torch.cat([w(t + ".weight") for t in ("q", "k", "v", "b", "a1", "g1")], dim=0).contiguous()
            # the outer halves as one block-diagonal matrix: one product for the decays' and the gates' sums
            self.w_a2 = torch.block_diag(w("a2.weight"), w("g2.weight")).contiguous()
        elif self.channel_decay:
            self.w_in = torch.cat([w(t + ".weight") for t in ("q", "k", "v", "b", "g")], dim=0).contiguous()
            self.w_a2 = w("a.weight")          # its sums are a product of their own
        else:
            self.w_in = torch.cat([w(t + ".weight") for t in ("q", "k", "v", "b", "a", "g")], dim=0).contiguous()
        self.w_o = w("o.weight")
        self.conv = torch.cat([w("q.conv"), w("k.conv"), w("v.conv")], dim=0).contiguous()
        self.a_log, self.dt_bias = w("A_log"), w("dt_bias")
        self.norm_weight = w("norm").repeat(self.heads).contiguous()       # per channel of the concatenated heads
        self._tiled = {"in": tiled_copy(self.runtime, self.w_in, K.LINEAR_PARTS),
                       "o": tiled_copy(self.runtime, self.w_o, K.LINEAR_PARTS)}
        if self.w_a2 is not None:
            self._tiled["a2"] = tiled_copy(self.runtime, self.w_a2, K.LINEAR_PARTS)

    def tensors(self):
        return [t for t in (self.w_in, self.w_o, self.conv, self.a_log, self.dt_bias, self.norm_weight, self.w_a2)
                if t is not None]

    def cache_need(self):
        return CacheNeed("state", state_shape=(self.state_floats + self.channels * (self.taps - 1),))

    def check_cache(self, page_size):
        if self.head_dim > K.gated_delta_max_dim():
            raise ValueError(f"gated_delta: key heads of {self.head_dim} are not built (up to {K.gated_delta_max_dim()})")

    def flops(self, tokens, keys_read=0.0):
        # the projections (of a block-diagonal matrix the blocks), and per token and head three passes over the state
        mats = self.w_in.numel() + self.w_o.numel()
        if self.low_rank:
            mats += self.decays * self.a_rank + self.hv * self.gate_rank
        elif self.w_a2 is not None:
            mats += self.w_a2.numel()
        return 2.0 * tokens * mats + 8.0 * tokens * self.heads * self.head_dim * self.value_dim

    def forward(self, ctx, xn, cache):
        n = xn.shape[0]
        f32 = torch.float32
        proj = decode_linear(ctx, xn, self.w_in, "gdelta.proj", self._tiled.get("in"))
        qn = ctx.buf("gdelta.q", (n, self.qk), f32)
        kn = ctx.buf("gdelta.k", (n, self.qk), f32)
        vv = ctx.buf("gdelta.v", (n, self.hv), f32)
        gb = ctx.buf("gdelta.gb", (n, 2, self.heads), f32)
        gate = ctx.buf("gdelta.gate", (n, self.hv), f32)
        conv_at = self.state_floats
        a_sums = low_sums = decays = None
        if self.low_rank:
            # the inner halves' sums in the compute dtype, then the outer halves' product
            inner = ctx.buf("gdelta.inner", (n, self.a_rank + self.gate_rank), self.runtime.dtype)
            K.unary_act(proj, inner, K.ACT_IDENTITY, first_column=self.channels + self.heads)
            low_sums = decode_linear(ctx, inner, self.w_a2, "gdelta.low", self._tiled.get("a2"))
        elif self.channel_decay:
            a_sums = decode_linear(ctx, xn, self.w_a2, "gdelta.a", self._tiled.get("a2"))
        if low_sums is not None and not self.channel_decay:
            raise ValueError("gated_delta: a low-rank decay is one per head and key channel")
        if self.channel_decay:
            decays = ctx.buf("gdelta.decays", (n, self.decays), f32)
        K.gated_delta_prep(proj, self.conv, self.taps, cache.state, conv_at, self.a_log, self.dt_bias, ctx.span_of_token,
                           cache.slots, ctx.span_start, ctx.span_pos, qn, kn, vv, gb, gate, self.heads, self.kv_heads,
                           self.head_dim, self.value_dim, self.unit_eps, a_sums=a_sums, decays=decays,
                           low_sums=low_sums, gate_sigmoid=self.gate_sigmoid)
        # (behind the launch that read the earlier inputs: the span's last ones take their place)
        K.conv_state_update(proj, 0, self.channels, self.taps, cache.state, conv_at, cache.slots, ctx.span_start,
                            ctx.span_pos, ctx.n_spans)
        o = ctx.buf("gdelta.o", (n, self.hv), f32)
        K.gated_delta_scan(qn, kn, vv, gb, o, cache.state, 0, cache.slots, ctx.span_start, ctx.span_pos, ctx.n_spans,
                           self.heads, self.kv_heads, self.head_dim, self.value_dim, decays=decays)
        out = ctx.buf("gdelta.out", (n, self.hv), self.runtime.dtype)
        K.delta_out(o, gate, self.norm_weight, self.eps, out, self.heads, self.value_dim)
        return decode_linear(ctx, out, self.w_o, "gdelta.o_proj", self._tiled.get("o"))


@register_part("mixer", "linear_recurrence")
class LinearRecurrenceMixer(Part):
    graph_safe = True
    records_launches = True

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.hidden = int(self.param("hidden"))
        self.width = int(self.param("width"))
        self.blocks = int(self.param("blocks"))
        self.taps = int(self.param("taps"))
        self.decay_scale = float(self.param("decay_scale", 8.0))
        if self.width % self.blocks:
            raise ValueError(f"linear_recurrence: {self.width} channels do not go into {self.blocks} equal blocks")
        if not 1 <= self.taps <= MAX_TAPS:
            raise ValueError(f"linear_recurrence: a convolution of {self.taps} taps is not built (1 to {MAX_TAPS})")
        self.w_in = self.w_o = self.y_bias = self.x_bias = self.conv = self.conv_bias = None
        self.gate_r = self.gate_i = self.gate_r_bias = self.gate_i_bias = self.rate = None
        self._tiled = {}

    def weight_specs(self):
        W, d, bs = self.width, self.hidden, self.width // self.blocks
        vec = lambda n, shape: WeightSpec(self.tensor_name(n), shape, "vector")
        return [WeightSpec(self.tensor_name("y.weight"), (W, d)), WeightSpec(self.tensor_name("x.weight"), (W, d)),
                WeightSpec(self.tensor_name("o.weight"), (d, W)),
                vec("y.bias", (W,)), vec("x.bias", (W,)), vec("conv", (W, self.taps)), vec("conv.bias", (W,)),
                vec("ra", (self.blocks, bs, bs)), vec("ra.bias", (self.blocks, bs)),
                vec("ri", (self.blocks, bs, bs)), vec("ri.bias", (self.blocks, bs)), vec("lam", (W,))]

    def bind(self, weights):
        w = lambda n: weights[self.tensor_name(n)]
        self.w_in = torch.cat([w("y.weight"), w("x.weight")], dim=0).contiguous()
        self.w_o = w("o.weight")
        self.y_bias, self.x_bias = w("y.bias"), w("x.bias")
        self.conv, self.conv_bias = w("conv"), w("conv.bias")
        # the gates' matrices [block][in][out]: neighbouring threads read neighbouring weights
        self.gate_r = w("ra").transpose(1, 2).contiguous()
        self.gate_i = w("ri").transpose(1, 2).contiguous()
        self.gate_r_bias = w("ra.bias").reshape(-1).contiguous()
        self.gate_i_bias = w("ri.bias").reshape(-1).contiguous()
        # log a = -rate r: the scale times softplus(lam), taken once, in double
        self.rate = (self.decay_scale * torch.nn.functional.softplus(w("lam").double())).float().contiguous()
        self._tiled = {"in": tiled_copy(self.runtime, self.w_in, K.LINEAR_PARTS),
                       "o": tiled_copy(self.runtime, self.w_o, K.LINEAR_PARTS)}

    def tensors(self):
        return [self.w_in, self.w_o, self.y_bias, self.x_bias, self.conv, self.conv_bias, self.gate_r, self.gate_i,
                self.gate_r_bias, self.gate_i_bias, self.rate]

    def cache_need(self):
        return CacheNeed("state", state_shape=(self.width * self.taps,))      # the state, then taps - 1 inputs a channel

    def flops(self, tokens, keys_read=0.0):
        return (2.0 * tokens * (self.w_in.numel() + self.w_o.numel())
                + 4.0 * tokens * self.width * (self.width // self.blocks))

    def forward(self, ctx, xn, cache):
        n = xn.shape[0]
        f32 = torch.float32
        W = self.width
        proj = decode_linear(ctx, xn, self.w_in, "rec.proj", self._tiled.get("in"))
        a = ctx.buf("rec.a", (n, W), f32)
        b = ctx.buf("rec.b", (n, W), f32)
        K.linear_recurrence_prep(proj, self.x_bias, self.conv, self.conv_bias, self.taps, cache.state, W, self.gate_r,
                                 self.gate_i, self.gate_r_bias, self.gate_i_bias, self.rate, ctx.span_of_token,
                                 cache.slots, ctx.span_start, ctx.span_pos, a, b, self.blocks)
        K.conv_state_update(proj, W, W, self.taps, cache.state, W, cache.slots, ctx.span_start, ctx.span_pos,
                            ctx.n_spans, in_bias=self.x_bias)
        out = ctx.buf("rec.out", (n, W), self.runtime.dtype)
        K.linear_recurrence_scan(a, b, proj, self.y_bias, cache.state, 0, cache.slots, ctx.span_start, ctx.span_pos,
                                 ctx.n_spans, out)
        return decode_linear(ctx, out, self.w_o, "rec.o_proj", self._tiled.get("o"))


@register_part("mixer", "mixer_sum")
class MixerSum(Part):
    """Two mixers side by side on the same input: ``left_scale`` * left + ``right_scale`` * right.
    Each keeps what it needs between steps in a cache or state of its own (``cache_need`` is the
    list of both needs; the run is handed one view for each, in that order).

    With ``norm_eps`` each output first passes an RMS norm over the model's width with a plain
    weight of its own (tensors ``<prefix>.left.out``, ``.right.out`` [hidden]).

    Parameters: ``left``, ``right`` (PartSpecs of mixers), ``left_scale``, ``right_scale``,
    ``norm_eps`` (None: no norms), ``hidden`` (with the norms)."""
    records_launches = True

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.left = make_part("mixer", self.param("left"), runtime)
        self.right = make_part("mixer", self.param("right"), runtime)
        self.left_scale = float(self.param("left_scale", 1.0))
        self.right_scale = float(self.param("right_scale", 1.0))
        eps = self.param("norm_eps", None)
        self.norm_eps = float(eps) if eps is not None else None
        self.hidden = int(self.param("hidden")) if self.norm_eps is not None else 0
        self.left_norm = self.right_norm = None
        for m in (self.left, self.right):
            if isinstance(m.cache_need(), (list, tuple)):
                raise ValueError("mixer_sum: its two mixers are plain ones")

    def children(self):
        return [self.left, self.right]

    @property
    def graph_safe(self):
        return self.left.graph_safe and self.right.graph_safe

    def weight_specs(self):
        own = []
        if self.norm_eps is not None:
            own = [WeightSpec(self.tensor_name("left.out"), (self.hidden,), "vector"),
                   WeightSpec(self.tensor_name("right.out"), (self.hidden,), "vector")]
        return self.left.weight_specs() + self.right.weight_specs() + own

    def bind(self, weights):
        self.left.bind(weights)
        self.right.bind(weights)
        if self.norm_eps is not None:
            self.left_norm = weights[self.tensor_name("left.out")]
            self.right_norm = weights[self.tensor_name("right.out")]

    def tensors(self):
        return [t for t in (self.left_norm, self.right_norm) if t is not None]

    def read_bytes(self, tokens):
        out = dict(self.left.read_bytes(tokens))
        out.update(self.right.read_bytes(tokens))
        return out

    def flops(self, tokens, keys_read=0.0):
        return self.left.flops(tokens, keys_read) + self.right.flops(tokens, keys_read)

    def cache_need(self):
        return [need for need in (self.left.cache_need(), self.right.cache_need()) if need is not None]

    def check_cache(self, page_size):
        self.left.check_cache(page_size)
        self.right.check_cache(page_size)

    # With norms the two outputs can be left, not yet added, to a norm behind the mixer that has the
    # same eps and norms each of them in its own launch (``pair_eps``: the caller's eps; it then
    # takes a ``kernels.NormedPair``).
    @property
    def leaves_normed_pair(self):
        return self.norm_eps is not None

    def forward(self, ctx, xn, cache, pair_eps=None):
        views = list(cache) if isinstance(cache, (list, tuple)) else [cache]
        take = lambda m: views.pop(0) if m.cache_need() is not None else None
        left = call_part(self.left, self.left.forward, ctx, xn, take(self.left))
        right = call_part(self.right, self.right.forward, ctx, xn, take(self.right))
        if self.norm_eps is not None and pair_eps == self.norm_eps:
            return K.NormedPair(left, self.left_scale, self.left_norm, right, self.right_scale, self.right_norm)
        out = ctx.buf("mixer_sum.out", (xn.shape[0], left.shape[-1]), torch.float32)
        if self.norm_eps is not None:
            K.normed_sum(out, left, self.left_scale, self.left_norm, right, self.right_scale, self.right_norm, self.norm_eps)
        else:
            K.scaled_sum(out, left, self.left_scale, right, self.right_scale)
        return out
