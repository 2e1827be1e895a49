"""Causal attention through low-rank latents.

Queries through a latent: c_q = N(W_dq h) g_q, q = W_uq c_q, per head [``head_dim`` unrotated |
``rot_dim`` rotated].  Keys and values through another: W_dkv h has ``kv_rank`` + ``rot_dim`` rows;
the first ``kv_rank``, through an RMS norm with a weight, are the latent c, the rest is one
rotated key part that every head shares.  Head h's key is [W_uk,h c | rotated part], its value
W_uv,h c; the score is (q . k) * ``scale`` over all ``head_dim`` + ``rot_dim`` elements; softmax
over the positions up to the query's; the concatenated heads are multiplied by sigmoid(W_g h)
and projected by W_o.

Only c and the rotated part are cached: one row of ``kv_rank`` + ``rot_dim`` a token, and c once
more with the slots of a page side by side (a paged cache with one "head" whose "values" are
c: the weighted sum over the keys runs along the slots).  The products with W_uk and W_uv are moved to the other
side: the query's unrotated part is folded through W_uk,h once a token, so that the score is
taken against c itself; the softmax's weighted sum is taken of c, and W_uv,h is applied to that
sum.  The numbers are the ones of the definition up to rounding.

Parameters: ``hidden``, ``heads``, ``head_dim``, ``rot_dim``, ``value_dim``, ``q_rank``,
``kv_rank``, ``scale``, ``eps``, ``position`` (a PartSpec whose tables rotate ``rot_dim``
elements, halves paired), ``gate`` (default True).
Tensors: ``<prefix>.{dq,uq,dkv,uk,uv,g,o}.weight``, ``.dq.norm``, ``.dkv.norm``.
"""

from __future__ import annotations

import torch

from .. import kernels as K
from .base import Part, register_part
from .linear import decode_linear, tiled_copy
from .spec import CacheNeed, WeightSpec


@register_part("mixer", "latent_attention")
class LatentAttention(Part):
    graph_safe = True
    records_launches = True

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.hidden = int(self.param("hidden"))
        self.heads = int(self.param("heads"))
        self.head_dim = int(self.param("head_dim"))
        self.rot_dim = int(self.param("rot_dim"))
        self.value_dim = int(self.param("value_dim"))
        self.q_rank = int(self.param("q_rank"))
        self.kv_rank = int(self.param("kv_rank"))
        self.scale = float(self.param("scale"))
        self.eps = float(self.param("eps"))
        self.gated = bool(self.param("gate", True))
        self.position = runtime.shared_part("position", self.param("position"))
        if (self.rot_dim % 2 or int(getattr(self.position, "rotary_dim", self.rot_dim)) != self.rot_dim
                or getattr(self.position, "interleaved", False)):
            raise ValueError("latent_attention: the position part rotates rot_dim elements, halves paired")
        self.row = self.kv_rank + self.rot_dim
        self.q_width = self.heads * (self.head_dim + self.rot_dim)
        self.out_dim = self.heads * self.value_dim
        self.w_in = self.w_uq = self.w_uk = self.w_uv = self.w_o = self.q_norm = self.kv_norm = None
        self._tiled = {}

    def weight_specs(self):
        d, H = self.hidden, self.heads
        specs = [WeightSpec(self.tensor_name("dq.weight"), (self.q_rank, d)),
                 WeightSpec(self.tensor_name("uq.weight"), (self.q_width, self.q_rank)),
                 WeightSpec(self.tensor_name("dkv.weight"), (self.row, d)),
                 WeightSpec(self.tensor_name("uk.weight"), (H * self.head_dim, self.kv_rank)),
                 WeightSpec(self.tensor_name("uv.weight"), (self.out_dim, self.kv_rank)),
                 WeightSpec(self.tensor_name("o.weight"), (d, self.out_dim)),
                 WeightSpec(self.tensor_name("dq.norm"), (self.q_rank,), "vector"),
                 WeightSpec(self.tensor_name("dkv.norm"), (self.kv_rank,), "vector")]
        if self.gated:
            specs.append(WeightSpec(self.tensor_name("g.weight"), (self.out_dim, d)))
        return specs

    def bind(self, weights):
        w = lambda n: weights[self.tensor_name(n)]
        # one product for everything that reads the layer's input: query latent | key/value latent | gate
        first = [w("dq.weight"), w("dkv.weight")] + ([w("g.weight")] if self.gated else [])
        self.w_in = torch.cat(first, dim=0).contiguous()
        self.w_uq, self.w_uk, self.w_uv, self.w_o = w("uq.weight"), w("uk.weight"), w("uv.weight"), w("o.weight")
        self.q_norm, self.kv_norm = w("dq.norm"), w("dkv.norm")
        # the matrix cores sum along a row: a second copy of W_uk, head by head [rank, head_dim]
        self.w_ukt = None
        if self.w_uk.dtype == torch.bfloat16 and self.head_dim % 32 == 0:
            self.w_ukt = (self.w_uk.view(self.heads, self.head_dim, self.kv_rank).transpose(1, 2).contiguous()
                          .view(self.heads * self.kv_rank, self.head_dim))
        self._tiled = {"in": tiled_copy(self.runtime, self.w_in, K.LINEAR_PARTS),
                       "uq": tiled_copy(self.runtime, self.w_uq, K.LINEAR_PARTS),
                       "o": tiled_copy(self.runtime, self.w_o, K.LINEAR_PARTS)}

    def tensors(self):
        return [self.w_in, self.w_uq, self.w_uk if self.w_ukt is None else self.w_ukt, self.w_uv, self.w_o, self.q_norm,
                self.kv_norm]

    def cache_need(self):
        return CacheNeed("paged", kv_heads=1, head_dim=self.row, value_dim=self.kv_rank)

    def check_cache(self, page_size):
        if self.row > K.latent_max_row():
            raise ValueError(f"latent_attention: cached rows of {self.row} are not built (up to {K.latent_max_row()})")

    def flops(self, tokens, keys_read=0.0):
        return super().flops(tokens) + 2.0 * self.heads * (self.row + self.kv_rank) * keys_read

    def forward(self, ctx, xn, cache):
        n = xn.shape[0]
        dtype = self.runtime.dtype
        if not cache.write:
            raise ValueError("latent_attention: the run writes its own cache")
        first = decode_linear(ctx, xn, self.w_in, "latent.in", self._tiled.get("in"))     # sums [.., n, q_rank + row (+ out)]
        cos, sin = self.position.tables(ctx)
        # the query's latent: norm, then up
        cq = ctx.buf("latent.cq", (n, self.q_rank), dtype)
        K.latent_norm(first, 0, self.q_norm, self.eps, cq)
        q = decode_linear(ctx, cq, self.w_uq, "latent.q", self._tiled.get("uq"))
        K.latent_kv_append(first, self.q_rank, self.kv_norm, self.eps, cos, sin, cache.pages, ctx.positions,
                           ctx.span_of_token, cache.block_table, cache.page_size, self.kv_rank, self.rot_dim)
        qa = ctx.buf("latent.qa", (n, self.heads * self.row), dtype)
        if self.w_ukt is not None:
            K.latent_query(q, self.w_ukt, cos, sin, qa, self.heads, self.head_dim, self.rot_dim, self.kv_rank, transposed=True)
        else:
            K.latent_query(q, self.w_uk, cos, sin, qa, self.heads, self.head_dim, self.rot_dim, self.kv_rank)
        attended = ctx.buf("latent.att", (n, self.heads * self.kv_rank), dtype)
        plain = self.runtime.options.get("attention", "auto") == "generic"
        slices = 1 if plain or self.row % 8 or cache.page_size % 16 else K.attn_latent_slices(n, self.heads, self.kv_rank, dtype)
        part = ctx.buf("latent.part", (n * self.heads * slices * (self.kv_rank + 2),), torch.float32) if slices > 1 else None
        K.attn_latent(qa, attended, cache.pages, ctx.positions, ctx.span_of_token, cache.block_table, cache.page_size,
                      self.heads, self.row, self.kv_rank, self.scale, plain=plain, part=part, nslices=slices)
        out = ctx.buf("latent.out", (n, self.out_dim), dtype)
        K.latent_out(attended, self.w_uv, out, self.heads, self.value_dim, self.kv_rank,
                     gate=first if self.gated else None, gate_column=self.q_rank + self.row)
        return decode_linear(ctx, out, self.w_o, "latent.o_proj", self._tiled.get("o"))
