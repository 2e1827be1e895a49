"""A plain, slow Lugetar in float64 torch on the CPU: the oracle of the Lugetar tests.

One function per mechanism, written from the equations; nothing here is shared with the
package.  ``cfg`` is the config.json dict, ``w`` a dict of float64 tensors by checkpoint name.
Sequences are handled one at a time and whole.

    x_0     = E[token] * s_e                          N(v) = v / sqrt(mean(v^2) + eps)
    a       = x + m N(Mixer(N(x) g_1)) g_1b           a norm in front of and behind each sub-layer
    x'      = a + m N(FeedForward(N(a) g_2)) g_2b     (a layer may have no feed-forward)
    logits  = E (N(x_L) g_f)                          the embedding table, unscaled, is the output matrix
"""

import math

import torch

F64 = torch.float64
SWISH_ALPHA = 1.702
UNIT_EPS = 1e-6


# ----------------------------------------------------------------------------- small functions

def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return rms(x, eps) * weight


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.logaddexp(z, torch.zeros_like(z))


# ----------------------------------------------------------------------------- rotation

def frequencies(rot):
    """Angle per position of each of the rot.dims / 2 rotated pairs.  With ``scaling`` (factor,
    low, high, original) a pair whose wavelength is below original / high keeps its frequency, one
    whose wavelength is above original / low turns ``factor`` times slower, and one between blends
    the two linearly in original / wavelength."""
    dims, base = int(rot["dims"]), float(rot["base"])
    sc = rot.get("scaling")
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if sc:
            factor, low, high, orig = (float(sc[k]) for k in ("factor", "low", "high", "original"))
            wavelength = 2.0 * math.pi / f
            if wavelength < orig / high:
                pass
            elif wavelength > orig / low:
                f = f / factor
            else:
                s = (orig / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=F64)


def rotate_halves(x, positions, rot):
    """x [n, heads, d]: element i of the first rot.dims of a head turns with element i + dims / 2."""
    dims = int(rot["dims"])
    half = dims // 2
    ang = torch.as_tensor(positions, dtype=F64)[:, None] * frequencies(rot)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


# ----------------------------------------------------------------------------- attention

def sees(i, j, chunk):
    """Whether the query at position i reads the key at position j: causal, and with a chunk
    size only inside the query's own chunk, chunks counted from position 0."""
    if j > i:
        return False
    return not chunk or i // chunk == j // chunk


def query_temperature(positions, temp):
    """1 + coef ln(floor((p + 1) / every) + 1) per position."""
    coef, every = float(temp["coef"]), int(temp["every"])
    return torch.tensor([1.0 + coef * math.log((p + 1) // every + 1) for p in positions], dtype=F64)


def softmax_attention(q, k, v, scale, mask):
    """q [n, H, d], k [m, G, d], v [m, G, dv], mask [n, m] (True: read) -> [n, H, dv]."""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * float(scale)
        s = s.masked_fill(~mask, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def attention(h, w, p, m, eps, positions):
    """Attention whose queries and keys are normed over the whole projection, all heads at once.
    Serves the 'attention' mixer (query temperature, no rotation, causal) and the left half of
    'parallel' (rotation behind the norm, chunked mask): each reads what its entry names."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    q = rms_norm(h @ w[p + ".q"].T, w[p + ".q.norm"], eps).reshape(n, H, d)
    k = rms_norm(h @ w[p + ".k"].T, w[p + ".k.norm"], eps).reshape(n, G, d)
    v = (h @ w[p + ".v"].T).reshape(n, G, dv)
    if m.get("rot"):
        q = rotate_halves(q, positions, m["rot"])
        k = rotate_halves(k, positions, m["rot"])
    if m.get("q_temp"):
        q = q * query_temperature(positions, m["q_temp"])[:, None, None]
    chunk = int((m.get("mask") or {}).get("size", 0))
    mask = torch.tensor([[sees(i, j, chunk) for j in positions] for i in positions])
    out = softmax_attention(q, k, v, m["scale"], mask)
    return out.reshape(n, H * dv) @ w[p + ".o"].T


# ----------------------------------------------------------------------------- gated delta rule

def causal_conv(x, taps_w):
    """x [n, C], taps_w [C, taps]: y_t = sum_j w[:, j] x_(t - taps + 1 + j), zeros before the start."""
    n, C = x.shape
    taps = taps_w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=F64), x], dim=0)
    y = torch.zeros(n, C, dtype=F64)
    for j in range(taps):
        y = y + padded[j:j + n] * taps_w[:, j]
    return y


def unit(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + UNIT_EPS)


def delta_rule(h, w, p, m, eps):
    """A matrix state per head, S [key channel, value channel], with one decay per key channel:
    S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    q = silu(causal_conv(h @ w[p + ".q"].T, w[p + ".q.conv"])).reshape(n, G, d)
    k = silu(causal_conv(h @ w[p + ".k"].T, w[p + ".k.conv"])).reshape(n, G, d)
    v = silu(causal_conv(h @ w[p + ".v"].T, w[p + ".v.conv"])).reshape(n, H, dv)
    q = unit(q) * d ** -0.5
    k = unit(k)
    beta = torch.sigmoid(h @ w[p + ".b"].T)                                        # [n, H]
    a = (h @ w[p + ".a1"].T) @ w[p + ".a2"].T + w[p + ".dt_bias"]                  # [n, H * d]
    g = torch.exp(-torch.exp(w[p + ".A_log"])[None, :, None] * softplus(a.reshape(n, H, d)))
    gate = torch.sigmoid((h @ w[p + ".g1"].T) @ w[p + ".g2"].T).reshape(n, H, dv)
    o = torch.zeros(n, H, dv, dtype=F64)
    for hh in range(H):
        kv = hh // (H // G)
        S = torch.zeros(d, dv, dtype=F64)
        for t in range(n):
            S = g[t, hh][:, None] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, kv])
            S = S + torch.outer(k[t, kv], u)
            o[t, hh] = S.T @ q[t, kv]
    o = rms(o, eps) * w[p + ".norm"] * gate
    return o.reshape(n, H * dv) @ w[p + ".o"].T


def parallel_mixer(h, w, p, m, eps, positions):
    left = attention(h, w, p + ".left", m["left"], eps, positions)
    right = delta_rule(h, w, p + ".right", m["right"], eps)
    return 0.5 * (rms_norm(left, w[p + ".left.out"], eps) + rms_norm(right, w[p + ".right.out"], eps))


# ----------------------------------------------------------------------------- feed-forward

def clamped_gate(g, u, limit):
    g = torch.clamp(g, max=limit)
    u = torch.clamp(u, -limit, limit)
    return g * torch.sigmoid(SWISH_ALPHA * g) * (u + 1.0)


def dense_ff(h, w, p, mlp):
    y = clamped_gate(h @ w[p + ".gate"].T, h @ w[p + ".up"].T, float(mlp["limit"]))
    return y @ w[p + ".down"].T


def expert(h, w, p):
    return (silu(h @ w[p + ".gate"].T) * (h @ w[p + ".up"].T)) @ w[p + ".down"].T


def choose_experts(scores, top, groups, keep, margin=None):
    """scores [E] -> the ``top`` experts with the largest scores among the experts of the ``keep``
    best of ``groups`` equal groups of neighbours; a group's score is the sum of its two largest.
    ``margin`` (a list) receives by how much the closest call was decided: the least kept group's
    score over the best dropped one's, the least chosen score over the best that was not."""
    E = scores.numel()
    size = E // groups
    allowed = torch.ones(E, dtype=torch.bool)
    gaps = []
    if groups > 1:
        by_group = scores.reshape(groups, size)
        group_score = by_group.topk(min(2, size), dim=-1).values.sum(-1)
        ranked = group_score.sort(descending=True)
        kept = ranked.indices[:keep]
        if keep < groups:
            gaps.append(float(ranked.values[keep - 1] - ranked.values[keep]))
        allowed = torch.zeros(groups, size, dtype=torch.bool)
        allowed[kept] = True
        allowed = allowed.reshape(E)
    masked = scores.masked_fill(~allowed, float("-inf"))
    ranked = masked.sort(descending=True)
    if top < int(allowed.sum()):
        gaps.append(float(ranked.values[top - 1] - ranked.values[top]))
    if margin is not None:
        margin.append(min(gaps) if gaps else float("inf"))
    return ranked.indices[:top]


def moe_ff(h, w, p, mlp, margins=None):
    """``margins`` (a list) receives, token by token, by how much the router's closest call was decided."""
    r = mlp["router"]
    E, top, scale = int(r["experts"]), int(r["top"]), float(r.get("scale", 1.0))
    groups = r.get("groups") or {}
    count, keep = int(groups.get("count", 1)), int(groups.get("keep", groups.get("count", 1)))
    s = torch.sigmoid(h @ w[p + ".router"].T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in choose_experts(s[t], top, count, keep, margins).tolist():
            out[t] = out[t] + scale * s[t, e] * expert(h[t:t + 1], w, f"{p}.e{e}")[0]
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ w[p + ".shared.sg"].T) * expert(h, w, p + ".shared")
    return out


# ----------------------------------------------------------------------------- the model

def forward(cfg, w, tokens, positions=None, taps=None, margins=None):
    """Logits [n, vocab] of one whole sequence; ``taps`` (a list) receives the stream after every
    layer, ``margins`` (a list) one list a routed layer: by how much each token's closest call of
    the router was decided."""
    n = len(tokens)
    positions = list(range(n)) if positions is None else list(positions)
    eps, m = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    x = w["embed"][torch.as_tensor(tokens)] * float(cfg["embedding"]["scale"])
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        h = rms_norm(x, w[p + ".norm1"], eps)
        if layer["type"] == "parallel":
            y = parallel_mixer(h, w, p + ".mix", layer["mixer"], eps, positions)
        else:
            y = attention(h, w, p + ".mix", layer["mixer"], eps, positions)
        x = x + m * rms_norm(y, w[p + ".norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rms_norm(x, w[p + ".norm2"], eps)
            if mlp["kind"] == "dense":
                y = dense_ff(h, w, p + ".mlp", mlp)
            else:
                per_token = [] if margins is not None else None
                y = moe_ff(h, w, p + ".mlp", mlp, per_token)
                if margins is not None:
                    margins.append(per_token)
            x = x + m * rms_norm(y, w[p + ".norm2b"], eps)
        if taps is not None:
            taps.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["embed"].T


def greedy(cfg, w, prompt, n):
    """n tokens, each the first largest logit behind the sequence so far."""
    seq, out = list(prompt), []
    for _ in range(n):
        nxt = int(torch.argmax(forward(cfg, w, seq)[-1]))
        out.append(nxt)
        seq.append(nxt)
    return out


# ----------------------------------------------------------------------------- random weights

def _attention_tensors(p, m, width, g):
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rn = lambda *s: torch.randn(*s, generator=g, dtype=F64)
    return {p + ".q": rn(H * d, width) / math.sqrt(width), p + ".k": rn(G * d, width) / math.sqrt(width),
            p + ".v": rn(G * dv, width) / math.sqrt(width), p + ".o": rn(width, H * dv) / math.sqrt(H * dv),
            p + ".q.norm": 1.0 + 0.3 * rn(H * d), p + ".k.norm": 1.0 + 0.3 * rn(G * d)}


def _delta_tensors(p, m, width, g, a_rank, gate_rank):
    H, G, d, dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
    rn = lambda *s: torch.randn(*s, generator=g, dtype=F64)
    return {p + ".q": rn(G * d, width) / math.sqrt(width), p + ".k": rn(G * d, width) / math.sqrt(width),
            p + ".v": rn(H * dv, width) / math.sqrt(width), p + ".b": rn(H, width) / math.sqrt(width),
            p + ".q.conv": rn(G * d, taps) * 0.6, p + ".k.conv": rn(G * d, taps) * 0.6, p + ".v.conv": rn(H * dv, taps) * 0.6,
            p + ".a1": rn(a_rank, width) / math.sqrt(width), p + ".a2": rn(H * d, a_rank) / math.sqrt(a_rank) * 2.0,
            p + ".g1": rn(gate_rank, width) / math.sqrt(width), p + ".g2": rn(H * dv, gate_rank) / math.sqrt(gate_rank) * 2.0,
            # decays spread between forgetting at once and hardly at all
            p + ".A_log": rn(H) * 0.8 - 0.5, p + ".dt_bias": rn(H * d) * 1.5 - 1.0,
            p + ".norm": 1.0 + 0.3 * rn(dv), p + ".o": rn(width, H * dv) / math.sqrt(H * dv)}


def _expert_tensors(p, ff, width, g):
    rn = lambda *s: torch.randn(*s, generator=g, dtype=F64)
    return {p + ".gate": rn(ff, width) / math.sqrt(width) * 1.5, p + ".up": rn(ff, width) / math.sqrt(width) * 1.5,
            p + ".down": rn(width, ff) / math.sqrt(ff)}


def random_weights(cfg, seed, a_rank=6, gate_rank=10):
    """Weights of a size that keeps every mechanism in play: products of unit scale, gates that
    reach their clamps, router scores spread over the experts."""
    g = torch.Generator().manual_seed(seed)
    width = cfg["width"]
    rn = lambda *s: torch.randn(*s, generator=g, dtype=F64)
    w = {"embed": rn(cfg["vocab"], width) / math.sqrt(width) * 2.0, "final.norm": 1.0 + 0.2 * rn(width)}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        for name in ("norm1", "norm1b"):
            w[f"{p}.{name}"] = 1.0 + 0.2 * rn(width)
        if layer["type"] == "parallel":
            w.update(_attention_tensors(p + ".mix.left", layer["mixer"]["left"], width, g))
            right = layer["mixer"]["right"]
            w.update(_delta_tensors(p + ".mix.right", right, width, g, right.get("a_rank", a_rank),
                                    right.get("gate_rank", gate_rank)))
            w[p + ".mix.left.out"] = 1.0 + 0.2 * rn(width)
            w[p + ".mix.right.out"] = 1.0 + 0.2 * rn(width)
        else:
            w.update(_attention_tensors(p + ".mix", layer["mixer"], width, g))
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        for name in ("norm2", "norm2b"):
            w[f"{p}.{name}"] = 1.0 + 0.2 * rn(width)
        if mlp["kind"] == "dense":
            w.update(_expert_tensors(p + ".mlp", mlp["ff"], width, g))
        else:
            for e in range(mlp["router"]["experts"]):
                w.update(_expert_tensors(f"{p}.mlp.e{e}", mlp["expert"]["ff"], width, g))
            w[p + ".mlp.router"] = rn(mlp["router"]["experts"], width) / math.sqrt(width) * 2.0
            if mlp.get("shared"):
                w.update(_expert_tensors(p + ".mlp.shared", mlp["shared"]["ff"], width, g))
                w[p + ".mlp.shared.sg"] = rn(1, width) / math.sqrt(width) * 2.0
    return w
