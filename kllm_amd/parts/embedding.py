"""Token embedding and output head.

Embedding: x[t, :] = E[id_t, :], no scaling (backend/model.cu:89-95,
:1056-1060) unless a design asks for a constant factor (``scale``).  Head: logits = xn . W^T in float32 for the wanted rows
(:1185-1188).  The head names its own tensor; a tied head simply names the
embedding's table (the reference resolves tying offline by copying it:
tools/convert_hf.py:81-82).
"""

from __future__ import annotations

import torch

from .. import kernels as K
from .base import Part, register_part, stream_copy
from .linear import linear, tiled_copy
from .spec import WeightSpec


@register_part("embedding", "token_embedding")
class TokenEmbedding(Part):
    graph_safe = True
    records_launches = True

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.vocab = int(self.param("vocab"))
        self.hidden = int(self.param("hidden"))
        self.table = None
        # an encoding that acts on the embedded tokens (``on_embedding``): the model calls it
        pos = self.param("position", None)
        self.position = runtime.shared_part("position", pos) if pos is not None else None
        # an RMS norm of the embedded tokens, ``norm_eps`` (None: none); tensor ``<prefix>.norm``
        eps = self.param("norm_eps", None)
        self.norm_eps = float(eps) if eps is not None else None
        self.norm_weight = None
        # a constant on the embedded rows (the table itself stays as it is, for a head that shares it)
        self.scale = float(self.param("scale", 1.0))

    def weight_specs(self):
        specs = [WeightSpec(self.tensor_name("weight"), (self.vocab, self.hidden))]
        if self.norm_eps is not None:
            specs.append(WeightSpec(self.tensor_name("norm"), (self.hidden,), "vector"))
        return specs

    def bind(self, weights):
        self.table = weights[self.tensor_name("weight")]
        if self.norm_eps is not None:
            self.norm_weight = weights[self.tensor_name("norm")]

    def read_bytes(self, tokens):
        return {self.table.data_ptr(): tokens * self.hidden * self.table.element_size()}   # one row per token

    def flops(self, tokens, keys_read=0.0):
        return 0.0

    def forward(self, ctx, token_ids):
        x = ctx.buf("x", (ctx.n, self.hidden), torch.float32)
        # with ``stream_rows`` the rows are also left in the compute dtype, for a first sub-layer that
        # reads the stream itself
        copy = None
        if self.param("stream_rows", False) and self.norm_eps is None and self.position is None:
            copy = stream_copy(ctx, x, fill=False)
        if ctx.sampled is not None and ctx.token_from is not None:
            K.embed(x, self.table, token_ids, ctx.token_from, ctx.sampled, scale=self.scale, copy=copy)
        else:
            K.embed(x, self.table, token_ids, scale=self.scale, copy=copy)
        if self.norm_eps is not None:
            K.norm_residual(x, self.norm_weight, eps=self.norm_eps, out=stream_copy(ctx, x, fill=False))
        return x


@register_part("head", "linear_head")
class LinearHead(Part):
    graph_safe = True
    records_launches = True

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.vocab = int(self.param("vocab"))
        self.hidden = int(self.param("hidden"))
        self.weight = None

    def weight_specs(self):
        return [WeightSpec(self.tensor_name("weight"), (self.vocab, self.hidden))]

    def bind(self, weights):
        self.weight = weights[self.tensor_name("weight")]
        self._tiled = {"w": tiled_copy(self.runtime, self.weight, K.LINEAR_PARTS)}   # for decode batches

    def forward(self, ctx, xn_rows):
        return linear(ctx, xn_rows, self.weight, "logits", split=False, w_tiled=self._tiled.get("w"))
