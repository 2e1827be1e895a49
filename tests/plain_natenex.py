"""A plain, slow Natenex in float64 torch on the CPU: the oracle of the Natenex tests.

One function per mechanism, written from the equations; nothing here is shared with the
package.  ``cfg`` is the config.json dict, ``w`` a dict of float64 tensors by checkpoint name.
Sequences are handled one at a time and whole.

    x_0     = E[token] * s_e                      N(v) = v / sqrt(mean(v^2) + eps)
    a       = x + N(Mixer(x)) g_1                 the sub-layers read x itself
    x'      = a + N(FeedForward(a)) g_2           (a layer may have no feed-forward)
    logits  = E (N(x_L) g_f)                      the embedding table, unscaled, is the output matrix

A layer that names ``weights_of`` j runs with layer j's tensors.
"""

import math

import torch

F64 = torch.float64


# ----------------------------------------------------------------------------- small functions

def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return rms(x, eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.logaddexp(z, torch.zeros_like(z))


# ----------------------------------------------------------------------------- rotation

def frequencies(rot):
    """Angle per position of each of the rot.dims / 2 rotated pairs; slow pairs are slowed down
    by ``scaling`` (factor, low, high, original): a pair whose wavelength is below
    original / high keeps its frequency, one above original / low turns ``factor`` times slower,
    those between blend the two linearly in original / wavelength."""
    dims, base = int(rot["dims"]), float(rot["base"])
    out = []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if sc:
            factor, low, high, orig = (float(sc[k]) for k in ("factor", "low", "high", "original"))
            wavelength = 2.0 * math.pi / f
            if wavelength > orig / low:
                f = f / factor
            elif wavelength >= orig / high:
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

def sees(i, j, window, keep_first):
    """Whether the query at position i reads the key at position j: the last ``window`` positions
    (itself included) and the first ``keep_first`` of the sequence; window 0 is no window."""
    if j > i:
        return False
    return not window or i - j < window or j < keep_first


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


def windowed_attention(h, w, p, m, eps, positions):
    """The left half of a 'parallel' mixer."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    q = (h @ w[p + ".q"].T).reshape(n, H, d)
    k = (h @ w[p + ".k"].T).reshape(n, G, d)
    v = (h @ w[p + ".v"].T).reshape(n, G, dv)
    q = rms_norm(q, w[p + ".q.norm"], eps)
    k = rms_norm(k, w[p + ".k.norm"], eps)
    if m.get("rot"):
        q = rotate_halves(q, positions, m["rot"])
        k = rotate_halves(k, positions, m["rot"])
    mask_cfg = m.get("mask") or {}
    window, keep = int(mask_cfg.get("size", 0)), int(mask_cfg.get("keep_first", 0))
    mask = torch.tensor([[sees(i, j, window, keep) for j in positions] for i in positions])
    out = softmax_attention(q, k, v, m["scale"], mask)
    return out.reshape(n, H * dv) @ w[p + ".o"].T


def latent_attention(h, w, p, m, eps, positions):
    """Queries, keys and values through low-rank latents; one rotated key part for all heads."""
    H, d, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    n = h.shape[0]
    cq = rms_norm(h @ w[p + ".dq"].T, w[p + ".dq.norm"], eps)
    q = (cq @ w[p + ".uq"].T).reshape(n, H, d + dr)
    dkv = h @ w[p + ".dkv"].T
    c = rms_norm(dkv[:, :rank], w[p + ".dkv.norm"], eps)
    k_rot = dkv[:, rank:].reshape(n, 1, dr)
    rot = dict(m["rot"])
    q_rot = rotate_halves(q[..., d:], positions, rot)
    k_rot = rotate_halves(k_rot, positions, rot)
    k_plain = (c @ w[p + ".uk"].T).reshape(n, H, d)
    v = (c @ w[p + ".uv"].T).reshape(n, H, dv)
    qq = torch.cat([q[..., :d], q_rot], dim=-1)
    kk = torch.cat([k_plain, k_rot.expand(n, H, dr)], dim=-1)
    mask = torch.tensor([[j <= i for j in positions] for i in positions])
    out = softmax_attention(qq, kk, v, m["scale"], mask).reshape(n, H * dv)
    out = out * torch.sigmoid(h @ w[p + ".g"].T)
    return out @ w[p + ".o"].T


# ----------------------------------------------------------------------------- recurrences

def causal_conv(x, weight, bias=None):
    """x [n, C], weight [C, taps]: y_t = sum_j weight[:, j] x_(t - taps + 1 + j), zeros before the start."""
    n, C = x.shape
    taps = weight.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=F64), x], dim=0)
    y = torch.zeros(n, C, dtype=F64)
    for j in range(taps):
        y = y + padded[j:j + n] * weight[:, j]
    return y + bias if bias is not None else y


def gated_linear_recurrence(h, w, p, m):
    """The right half of a 'parallel' mixer: two branches, a short convolution, block-diagonal
    gates, and a per-channel recurrence S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t."""
    width, blocks = m["width"], m["blocks"]
    n = h.shape[0]
    y = gelu_tanh(h @ w[p + ".y"].T + w[p + ".y.b"])
    u = causal_conv(h @ w[p + ".x"].T + w[p + ".x.b"], w[p + ".conv"], w[p + ".conv.b"])
    ub = u.reshape(n, blocks, width // blocks)
    r = torch.sigmoid(torch.einsum("nbi,boi->nbo", ub, w[p + ".ra"]) + w[p + ".ra.b"]).reshape(n, width)
    i = torch.sigmoid(torch.einsum("nbi,boi->nbo", ub, w[p + ".ri"]) + w[p + ".ri.b"]).reshape(n, width)
    log_a = -8.0 * r * softplus(w[p + ".lam"])
    a = torch.exp(log_a)
    drive = torch.sqrt(1.0 - a * a) * i * u
    S = torch.zeros(width, dtype=F64)
    out = torch.zeros(n, width, dtype=F64)
    for t in range(n):
        S = a[t] * S + drive[t]
        out[t] = S
    return (out * y) @ w[p + ".o"].T


def gated_delta(h, w, p, m, eps):
    """A matrix state per head, decayed, corrected towards the value along the key, read by the query."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    q = silu(causal_conv(h @ w[p + ".q"].T, w[p + ".q.conv"])).reshape(n, G, d)
    k = silu(causal_conv(h @ w[p + ".k"].T, w[p + ".k.conv"])).reshape(n, G, d)
    v = silu(causal_conv(h @ w[p + ".v"].T, w[p + ".v.conv"])).reshape(n, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[p + ".b"].T)
    decay = torch.exp(-torch.exp(w[p + ".A_log"]) * softplus(h @ w[p + ".a"].T + w[p + ".dt_bias"]))
    o = torch.zeros(n, H, dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(d, dv, dtype=F64)
        for t in range(n):
            S = decay[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            o[t, hd] = S.T @ q[t, g]
    o = rms_norm(o, w[p + ".norm"], eps).reshape(n, H * dv) * silu(h @ w[p + ".g"].T)
    return o @ w[p + ".o"].T


# ----------------------------------------------------------------------------- layers and model

def feed_forward(h, w, p):
    z = torch.relu(h @ w[p + ".up"].T)
    return (z * z) @ w[p + ".down"].T


def mixer(kind, h, w, p, m, eps, positions):
    if kind == "parallel":
        left = windowed_attention(h, w, p + ".left", m["left"], eps, positions)
        right = gated_linear_recurrence(h, w, p + ".right", m["right"])
        return float(m["left_scale"]) * left + float(m["right_scale"]) * right
    if kind == "latent_attention":
        return latent_attention(h, w, p, m, eps, positions)
    if kind == "delta":
        return gated_delta(h, w, p, m, eps)
    raise ValueError(kind)


def forward(cfg, w, tokens, taps=None):
    """Logits [n, vocab] of one whole sequence from position 0; ``taps`` (a list) receives the
    stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    positions = list(range(len(tokens)))
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
    for i, layer in enumerate(cfg["layers"]):
        src = f"l{layer.get('weights_of', i) if layer.get('weights_of') is not None else i}"
        x = x + rms_norm(mixer(layer["type"], x, w, src + ".mix", layer["mixer"], eps, positions), w[src + ".norm1"], eps)
        if layer.get("mlp") is not None:
            x = x + rms_norm(feed_forward(x, w, src + ".mlp"), w[src + ".norm2"], eps)
        if taps is not None:
            taps.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["embed"].T


def greedy(cfg, w, prompt, steps):
    """The ``steps`` tokens that follow ``prompt`` when the likeliest is taken each time."""
    toks = list(prompt)
    for _ in range(steps):
        toks.append(int(torch.argmax(forward(cfg, w, toks)[-1])))
    return toks[len(prompt):]


# ----------------------------------------------------------------------------- token by token

def linear_recurrence_step(x_t, state, conv_inputs, w, p, m):
    """One token through the gated linear recurrence from (state [width], the last taps - 1
    inputs of the convolution [taps - 1, width]); returns (output before W_o, state, inputs)."""
    width, blocks = m["width"], m["blocks"]
    y = gelu_tanh(w[p + ".y"] @ x_t + w[p + ".y.b"])
    xin = w[p + ".x"] @ x_t + w[p + ".x.b"]
    window = torch.cat([conv_inputs, xin[None]], dim=0)
    u = (window.T * w[p + ".conv"]).sum(-1) + w[p + ".conv.b"]
    ub = u.reshape(blocks, width // blocks)
    r = torch.sigmoid(torch.einsum("bi,boi->bo", ub, w[p + ".ra"]) + w[p + ".ra.b"]).reshape(width)
    i = torch.sigmoid(torch.einsum("bi,boi->bo", ub, w[p + ".ri"]) + w[p + ".ri.b"]).reshape(width)
    a = torch.exp(-8.0 * r * softplus(w[p + ".lam"]))
    state = a * state + torch.sqrt(1.0 - a * a) * i * u
    return state * y, state, window[1:]


# ----------------------------------------------------------------------------- random weights

def _layer_tensors(layer, i, width, g):
    def mat(o, k):
        return torch.randn(o, k, generator=g, dtype=F64) / math.sqrt(k)

    def vec(n, mean=1.0, spread=0.2):
        return mean + spread * torch.randn(n, generator=g, dtype=F64)

    out, p, m = {}, f"l{i}.mix", layer["mixer"]
    out[f"l{i}.norm1"] = vec(width)
    if layer["type"] == "parallel":
        a, r = m["left"], m["right"]
        q = p + ".left"
        out[q + ".q"], out[q + ".k"] = mat(a["heads"] * a["dim"], width), mat(a["kv_heads"] * a["dim"], width)
        out[q + ".v"], out[q + ".o"] = mat(a["kv_heads"] * a["vdim"], width), mat(width, a["heads"] * a["vdim"])
        out[q + ".q.norm"], out[q + ".k.norm"] = vec(a["dim"], 1.5, 0.4), vec(a["dim"], 1.5, 0.4)
        q, W, bs = p + ".right", r["width"], r["width"] // r["blocks"]
        out[q + ".y"], out[q + ".x"], out[q + ".o"] = mat(W, width), mat(W, width), mat(width, W)
        out[q + ".y.b"], out[q + ".x.b"] = vec(W, 0.0, 0.3), vec(W, 0.0, 0.3)
        out[q + ".conv"], out[q + ".conv.b"] = 0.6 * torch.randn(W, r["conv"], generator=g, dtype=F64), vec(W, 0.0, 0.2)
        for t in ("ra", "ri"):
            out[f"{q}.{t}"] = torch.randn(r["blocks"], bs, bs, generator=g, dtype=F64) / math.sqrt(bs)
            out[f"{q}.{t}.b"] = 0.5 * torch.randn(r["blocks"], bs, generator=g, dtype=F64)
        out[q + ".lam"] = -3.0 + 2.0 * torch.randn(W, generator=g, dtype=F64)
    elif layer["type"] == "latent_attention":
        H, d, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
        out[p + ".dq"], out[p + ".uq"] = mat(m["q_rank"], width), mat(H * (d + dr), m["q_rank"])
        out[p + ".dkv"] = mat(m["kv_rank"] + dr, width)
        out[p + ".uk"], out[p + ".uv"] = mat(H * d, m["kv_rank"]), mat(H * dv, m["kv_rank"])
        out[p + ".g"], out[p + ".o"] = mat(H * dv, width), mat(width, H * dv)
        out[p + ".dq.norm"], out[p + ".dkv.norm"] = vec(m["q_rank"]), vec(m["kv_rank"])
    else:
        H, G, d, dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
        out[p + ".q"], out[p + ".k"], out[p + ".v"] = mat(G * d, width), mat(G * d, width), mat(H * dv, width)
        for t, n in (("q", G * d), ("k", G * d), ("v", H * dv)):
            out[f"{p}.{t}.conv"] = 0.6 * torch.randn(n, taps, generator=g, dtype=F64)
        out[p + ".b"], out[p + ".a"] = mat(H, width), mat(H, width)
        out[p + ".A_log"], out[p + ".dt_bias"] = vec(H, -1.0, 1.0), vec(H, 0.0, 1.0)
        out[p + ".norm"] = vec(dv)
        out[p + ".g"], out[p + ".o"] = mat(H * dv, width), mat(width, H * dv)
    if layer.get("mlp") is not None:
        f = layer["mlp"]["ff"]
        out[f"l{i}.norm2"] = vec(width)
        out[f"l{i}.mlp.up"], out[f"l{i}.mlp.down"] = mat(f, width), mat(width, f)
    return out


def random_weights(cfg, seed):
    """Weights of a size that keeps every mechanism in play: products of unit scale, decays
    spread between forgetting at once and hardly at all."""
    g = torch.Generator().manual_seed(seed)
    width = cfg["width"]
    w = {"embed": torch.randn(cfg["vocab"], width, generator=g, dtype=F64) / math.sqrt(width) * 2.0,
         "final.norm": 1.0 + 0.2 * torch.randn(width, generator=g, dtype=F64)}
    for i, layer in enumerate(cfg["layers"]):
        if layer.get("weights_of") is None:
            w.update(_layer_tensors(layer, i, width, g))
    return w
