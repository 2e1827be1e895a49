"""Routed feed-forward: a mixture of small gated experts, of which every token uses a few.

    z = W_r h                          router sums over all experts, 32-bit
    s = softmax(z)
    chosen = the ``top`` largest of s + correction       (the correction only chooses)
    a_e = s_e / (sum of the chosen s + 1e-20)
    y = sum over the chosen e of a_e Expert_e(h)  [+ Shared(h)]

The last ``identity`` of the router's outputs are identity experts: Expert_e(h) = h; they have
no tensors.  An expert (and the shared expert, which every token uses) is a gated feed-forward
without biases whose gate is ``activation``: "clamped_swish" with g' = min(g, limit), u' =
clamp(u, -limit, limit) gives down(g' sigmoid(alpha g') (u' + 1)); a gate's plain activation
("silu", "gelu_tanh") gives down(act(g) u).

Which token goes where stays on the device: the router's choice is grouped by expert into tiles
of rows (a fixed number of tiles for a step's shape, the unused ones empty), so what is launched
depends on the shape alone and a step can be recorded.

Other routers, each a parameter: ``scoring`` "sigmoid": s = 1 / (1 + exp(-z)) per expert;
``groups`` > 1: the experts form that many equal groups of neighbours, a group's score is the sum
of its two largest (s + correction), and only experts of the ``keep_groups`` best groups can be
chosen; ``renormalize`` False: a_e = s_e; ``weight_scale``: a_e times a constant; ``shared_gate``:
the shared expert's output is multiplied, token by token, by 1 / (1 + exp(-w_sg . h)).

Parameters: ``hidden``, ``experts``, ``identity`` (0), ``top``, ``intermediate``, ``limit``,
``activation`` ("clamped_swish"), ``alpha`` (1.702), ``correction`` (True: the tensor exists),
``shared_intermediate`` (None: no shared expert), ``shared_limit``, ``scoring`` ("softmax"),
``groups`` (1), ``keep_groups``, ``renormalize`` (True), ``weight_scale`` (1), ``shared_gate`` (False).
Tensors: ``<prefix>.router`` [experts + identity, hidden], ``.correction``,
``.e<i>.{gate,up,down}``, ``.shared.{gate,up,down}``, ``.shared.sg`` [1, hidden].
"""

from __future__ import annotations

import torch

from .. import kernels as K
from .base import Part, register_part
from .feedforward import gated_hidden
from .linear import decode_linear, tiled_copy
from .spec import WeightSpec


@register_part("feed_forward", "routed_experts")
class RoutedExperts(Part):
    graph_safe = True
    records_launches = True

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.hidden = int(self.param("hidden"))
        self.experts = int(self.param("experts"))
        self.identity = int(self.param("identity", 0) or 0)
        self.top = int(self.param("top"))
        self.intermediate = int(self.param("intermediate"))
        self.limit = float(self.param("limit", 0.0))
        self.alpha = float(self.param("alpha", 1.702))
        act = self.param("activation", "clamped_swish")
        if act not in K.GATES:
            raise ValueError(f"routed_experts: gate {act!r} is not built (one of {sorted(K.GATES)})")
        self.act = K.GATES[act]
        self.has_correction = bool(self.param("correction", True))
        shared = self.param("shared_intermediate", None)
        self.shared_intermediate = int(shared) if shared else None
        self.shared_limit = float(self.param("shared_limit", self.limit))
        if self.experts < 1 or self.identity < 0 or not 1 <= self.top <= self.experts + self.identity:
            raise ValueError(f"routed_experts: top {self.top} of {self.experts} + {self.identity} experts")
        self.scoring = self.param("scoring", "softmax")
        if self.scoring not in ("softmax", "sigmoid"):
            raise ValueError(f"routed_experts: scoring {self.scoring!r} is not built (softmax, sigmoid)")
        self.groups = int(self.param("groups", 1) or 1)
        self.keep_groups = int(self.param("keep_groups", self.groups) or self.groups)
        routed = self.experts + self.identity
        if (self.groups < 1 or self.groups > K.MOE_MAX_GROUPS or routed % self.groups
                or not 1 <= self.keep_groups <= self.groups or self.top > routed // self.groups * self.keep_groups):
            raise ValueError(f"routed_experts: {routed} experts in {self.groups} groups (up to {K.MOE_MAX_GROUPS}) of "
                             f"which {self.keep_groups} are kept, for {self.top} choices")
        self.renormalize = bool(self.param("renormalize", True))
        self.weight_scale = float(self.param("weight_scale", 1.0))
        self.shared_gate = bool(self.param("shared_gate", False)) and bool(shared)
        self.w_router = self.correction = self.w_gu = self.w_down = self.w_shared_gu = self.w_shared_down = None
        self._tiled = {}

    def _expert_names(self, e):
        return [self.tensor_name(f"e{e}.{t}") for t in ("gate", "up", "down")]

    def weight_specs(self):
        d, f, r = self.hidden, self.intermediate, self.experts + self.identity
        specs = [WeightSpec(self.tensor_name("router"), (r, d))]
        if self.has_correction:
            specs.append(WeightSpec(self.tensor_name("correction"), (r,), "vector"))
        for e in range(self.experts):
            g, u, dn = self._expert_names(e)
            specs += [WeightSpec(g, (f, d)), WeightSpec(u, (f, d)), WeightSpec(dn, (d, f))]
        if self.shared_intermediate:
            sf = self.shared_intermediate
            specs += [WeightSpec(self.tensor_name("shared.gate"), (sf, d)), WeightSpec(self.tensor_name("shared.up"), (sf, d)),
                      WeightSpec(self.tensor_name("shared.down"), (d, sf))]
        if self.shared_gate:
            specs.append(WeightSpec(self.tensor_name("shared.sg"), (1, d)))
        return specs

    def bind(self, weights):
        self.w_router = weights[self.tensor_name("router")]
        if self.shared_gate:       # the gate's sum is one more of the router's product
            self.w_router = torch.cat([self.w_router, weights[self.tensor_name("shared.sg")]], dim=0).contiguous()
        self.correction = weights[self.tensor_name("correction")] if self.has_correction else None
        gu, down = [], []
        for e in range(self.experts):
            g, u, dn = (weights[n] for n in self._expert_names(e))
            gu.append(torch.cat([g, u], dim=0))
            down.append(dn)
        self.w_gu = torch.stack(gu).contiguous()            # [E, 2 f, d]: an expert's gate rows, then its up rows
        self.w_down = torch.stack(down).contiguous()        # [E, d, f]
        self._tiled = {"router": tiled_copy(self.runtime, self.w_router, K.LINEAR_PARTS)}
        if self.shared_intermediate:
            self.w_shared_gu = torch.cat([weights[self.tensor_name("shared.gate")],
                                          weights[self.tensor_name("shared.up")]], dim=0).contiguous()
            self.w_shared_down = weights[self.tensor_name("shared.down")]
            self._tiled["shared_gu"] = tiled_copy(self.runtime, self.w_shared_gu, K.LINEAR_PARTS)
            self._tiled["shared_down"] = tiled_copy(self.runtime, self.w_shared_down, K.LINEAR_PARTS)

    def read_bytes(self, tokens):
        """Of the experts' weights a step reads what its tokens choose: at most ``top`` experts a token."""
        out = super().read_bytes(tokens)
        share = min(1.0, tokens * self.top / self.experts)
        for t in (self.w_gu, self.w_down):
            out[t.data_ptr()] = int(t.numel() * t.element_size() * share)
        return out

    def flops(self, tokens, keys_read=0.0):
        d, f = self.hidden, self.intermediate
        total = 2.0 * tokens * self.w_router.shape[0] * d + 6.0 * tokens * self.top * d * f
        if self.shared_intermediate:
            total += 6.0 * tokens * d * self.shared_intermediate
        return total

    # The weighted sum over a token's choices can be left to a norm that adds it up while it
    # normalises (``sums_ok``: the caller takes a ``kernels.ChosenSums``).
    leaves_chosen_sums = True

    def forward(self, ctx, xn, sums_ok=False):
        n, d, top, f = xn.shape[0], self.hidden, self.top, self.intermediate
        dtype = self.runtime.dtype
        z = decode_linear(ctx, xn, self.w_router, "moe.z", self._tiled.get("router"))
        idx = ctx.buf("moe.idx", (n, top), torch.int32)
        wgt = ctx.buf("moe.wgt", (n, top), torch.float32)
        sgate = ctx.buf("moe.sgate", (n,), torch.float32) if self.shared_gate else None
        K.moe_route(z, self.correction, idx, wgt, experts=self.experts + self.identity, scoring=self.scoring,
                    groups=self.groups, keep_groups=self.keep_groups, scale=self.weight_scale,
                    renormalize=self.renormalize, shared_gate=sgate)
        h = ctx.buf("moe.h", (n * top, f), dtype)
        y = ctx.buf("moe.y", (n * top, d), torch.float32)
        if n * top <= K.MOE_ROWS_BEST_ENTRIES and not self.runtime.options.get("moe_tiles_only"):
            # a decode batch: entry by entry, every chosen expert's rows streamed once
            K.moe_expert_rows(xn, self.w_gu, h, idx, self.experts, 0, self.act, self.limit, self.alpha)
            K.moe_expert_rows(h, self.w_down, y, idx, self.experts, 1)
        else:
            rows = K.moe_best_tile_rows(n * top, self.experts)
            tiles = ctx.buf("moe.tiles", (K.moe_max_tiles(n * top, self.experts, rows), 3), torch.int32)
            order = ctx.buf("moe.sorted", (n * top,), torch.int32)
            K.moe_plan(idx, self.experts, order, tiles, rows)
            K.moe_expert(xn, self.w_gu, h, order, tiles, top, 0, self.act, self.limit, self.alpha, tile_rows=rows)
            K.moe_expert(h, self.w_down, y, order, tiles, top, 1, tile_rows=rows)
        shared = None
        if self.shared_intermediate:
            hs = gated_hidden(ctx, xn, self.w_shared_gu, self.shared_intermediate, "moe.shared",
                              self._tiled.get("shared_gu"), None, self.act, self.shared_limit, self.alpha)
            shared = decode_linear(ctx, hs, self.w_shared_down, "moe.shared.down", self._tiled.get("shared_down"))
        if sums_ok:
            return K.ChosenSums(y, xn, idx, wgt, self.experts, shared, sgate)
        out = ctx.buf("moe.out", (n, d), torch.float32)
        K.moe_combine(y, xn, idx, wgt, out, self.experts, shared, sgate)
        return out
