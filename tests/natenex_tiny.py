"""Small Natenex configurations for the tests, each unlike the others in every size and constant,
and helpers to write them as model folders.

N1: all three mixers and a layer run twice: attention of 4 heads on 2 KV heads of 32 of which 16
    turn with slowed-down pairs, window 24 keeping the first 3, beside a recurrence of 48 channels
    in 3 blocks with 4 taps; a delta layer without feed-forward (keys of 16, values of 24, 3
    taps); latents of 24 and 40 for 3 heads of 16 + 8 with values of 20.
N2: latent attention first, values wider than keys; attention whose values are narrower than
    its keys, window 40 without kept positions, whole-head rotation; a delta layer with as
    many key heads as heads and 2 taps, run twice.
N3: no mask at all and no rotation (heads of 128: the kernels on the matrix cores), one block
    of gates, a convolution of one tap (no inputs to keep), another eps.
N4: nothing a multiple of 4 or 8: width 50, five heads of 20 with values of 12, window 7
    keeping 2, a recurrence of 30 channels in 5 blocks with 5 taps, latents of 22 and 14, one
    key head for three delta heads.
N5: factors of one everywhere (embedding, left and right), kept positions as many as the
    window, a window of one page, heads of 64 on one KV head.
D1, P1, L1: one mixer each, alone, without feed-forward.
N6, N7: sizes nearer to a real model's layers (heads of 64 and 128, latents of 160 and 448, delta
    heads of 64 x 96 and 128 x 128).
N8: the same delta layer three times, the first two running with the last one's tensors.
"""

import json
import math
import os

import torch

import plain_natenex as P


def attn(heads, kv, dim, vdim=None, rot=None, base=10000.0, scaling=None, window=0, keep=0, scale=None):
    a = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim or dim, "scale": scale or 1.3 * dim ** -0.5}
    if rot:
        a["rot"] = {"base": base, "dims": rot}
        if scaling:
            a["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    if window:
        a["mask"] = {"size": window, "keep_first": keep}
    return a


def parallel(left, width, blocks, conv, left_scale=1.25, right_scale=0.8, ff=None, weights_of=None):
    return _layer("parallel", {"left": left, "right": {"width": width, "blocks": blocks, "conv": conv},
                               "left_scale": left_scale, "right_scale": right_scale}, ff, weights_of)


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, base=10000.0, scale=None, ff=None, weights_of=None, scaling=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return _layer("latent_attention", {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank,
                                       "kv_rank": kv_rank, "scale": scale or (dim + rot_dim) ** -0.5, "rot": rot},
                  ff, weights_of)


def delta(heads, kv, dim, vdim, conv, ff=None, weights_of=None):
    return _layer("delta", {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}, ff, weights_of)


def _layer(kind, mixer, ff, weights_of):
    out = {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def _cfg(vocab, width, eps, scale, layers):
    return {"architecture": "Natenex", "vocab": vocab, "width": width, "embedding": {"scale": scale},
            "norm": {"eps": eps}, "layers": layers}


_A1 = attn(4, 2, 32, rot=16, base=5000.0, scaling=(4.0, 1.0, 3.0, 48), window=24, keep=3)
_A2 = attn(4, 1, 64, vdim=32, rot=64, base=300.0, window=40)
_A4 = attn(5, 5, 20, vdim=12, rot=10, base=77.0, scaling=(2.5, 2.0, 5.0, 30), window=7, keep=2)
_A5 = attn(4, 1, 64, rot=32, window=16, keep=16)

CONFIGS = {
    "N1": _cfg(90, 64, 1e-5, 2.5, [
        parallel(_A1, 48, 3, 4, ff=80),
        delta(4, 2, 16, 24, 3),
        latent(3, 16, 8, 20, 24, 40, base=2000.0, ff=96),
        parallel(_A1, 48, 3, 4, ff=80, weights_of=0)]),
    "N2": _cfg(128, 128, 1e-6, 0.7, [
        latent(4, 32, 16, 48, 64, 80, ff=72),
        parallel(_A2, 96, 2, 2, left_scale=0.6, right_scale=1.5),
        delta(2, 2, 64, 32, 2, ff=160),
        delta(2, 2, 64, 32, 2, ff=160, weights_of=2)]),
    "N3": _cfg(101, 72, 1e-4, 4.0, [
        parallel(attn(2, 2, 128), 72, 1, 1, left_scale=2.0, right_scale=0.5, ff=40),
        delta(3, 1, 128, 16, 1, ff=56)]),
    "N4": _cfg(61, 50, 1e-5, 1.7, [
        delta(3, 1, 12, 10, 5),
        parallel(_A4, 30, 5, 5, left_scale=0.9, right_scale=1.3, ff=34),
        latent(5, 6, 6, 14, 22, 14, base=50.0, ff=30)]),
    "N5": _cfg(77, 48, 1e-3, 1.0, [
        parallel(_A5, 64, 4, 3, left_scale=1.0, right_scale=1.0, ff=56),
        parallel(_A5, 64, 4, 3, left_scale=1.0, right_scale=1.0, ff=56, weights_of=0)]),
    "D1": _cfg(50, 32, 1e-5, 2.0, [delta(4, 2, 24, 40, 4)]),
    "P1": _cfg(50, 40, 1e-5, 2.0, [parallel(attn(2, 1, 48, vdim=16, rot=24, window=20, keep=5), 56, 7, 3)]),
    "L1": _cfg(50, 40, 1e-5, 2.0, [latent(2, 24, 16, 12, 20, 36)]),
}


def write_model(out_dir, cfg, seed, store="float32", weights=None):
    """A model folder written with the safetensors library."""
    from safetensors.torch import save_file
    w = weights if weights is not None else P.random_weights(cfg, seed)
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[store]
    os.makedirs(out_dir, exist_ok=True)
    save_file({k: v.to(dt).contiguous() for k, v in w.items()}, os.path.join(out_dir, "model.safetensors"))
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(cfg, f)
    return out_dir


def read_weights(model_dir, as_stored_in=None):
    """The folder's weights as float64 CPU tensors; with as_stored_in="bfloat16" what a bfloat16
    engine keeps in bfloat16 (the matrices of the products) is rounded first; everything that
    enters a recurrence or a norm stays in 32-bit."""
    from safetensors.torch import load_file
    kept_wide = (".conv", ".ra", ".ri", ".norm", ".lam", ".A_log", ".dt_bias", ".b")
    out = {}
    for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items():
        v = v.float()
        wide = v.dim() < 2 or (k.endswith(kept_wide) and not k.endswith(".mix.b"))
        if as_stored_in == "bfloat16" and not wide:
            v = v.to(torch.bfloat16).float()
        out[k] = v.double()
    return out


def tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


# Sizes nearer to a real model's layers (N6, N7): heads of 64 and 128 on the matrix cores' kernels,
# cached latent rows of several hundred elements, delta heads of 64 and 128.
CONFIGS["N6"] = _cfg(200, 192, 1e-6, 1.5, [
    delta(6, 3, 64, 96, 4, ff=128),
    parallel(attn(6, 2, 64, rot=32, base=30000.0, scaling=(6.0, 1.0, 4.0, 64), window=48, keep=4), 256, 8, 4, ff=160),
    latent(6, 64, 32, 64, 96, 160, base=3000.0, ff=128),
    parallel(attn(6, 2, 64, rot=32, base=30000.0, scaling=(6.0, 1.0, 4.0, 64), window=48, keep=4), 256, 8, 4, ff=160,
             weights_of=1)])
CONFIGS["N7"] = _cfg(160, 128, 1e-5, 0.5, [
    latent(3, 128, 64, 128, 72, 448, ff=96, scaling=(2.0, 1.0, 4.0, 40)),
    delta(2, 1, 128, 128, 4),
    parallel(attn(4, 4, 128, vdim=128, rot=128, window=32, keep=1), 128, 2, 2, left_scale=0.5, right_scale=2.0)])
# The same layer three times, the first of them running with the last one's tensors.
CONFIGS["N8"] = _cfg(64, 48, 1e-5, 1.0, [
    delta(2, 2, 16, 16, 2, ff=32, weights_of=2),
    delta(2, 2, 16, 16, 2, ff=32, weights_of=2),
    delta(2, 2, 16, 16, 2, ff=32)])


def aimed_attention(cfg, w, query_token, key_token, strength=30.0):
    """Changes ``w`` (weights of a model whose FIRST layer has windowed attention) so that, in
    layer 0, the query of ``query_token`` looks along the key of ``key_token`` wherever it stands:
    the two tokens get an embedding direction of their own each, which the query and key matrices
    turn into one and the same long vector in the part of every head that does not rotate.  The
    norm makes every query and key as long as any other, so the aimed score is about
    sqrt(dim) times a random one; the value of ``key_token`` is unlike any other."""
    m = cfg["layers"][0]["mixer"]["left"]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    rot = (m.get("rot") or {}).get("dims", 0)
    assert rot < d, "only the part of a head that does not rotate can be aimed"
    width = cfg["width"]
    g = torch.Generator().manual_seed(99)
    a, b = torch.zeros(width, dtype=torch.float64), torch.zeros(width, dtype=torch.float64)
    a[0], b[1] = 1.0, 1.0
    w["embed"][:, :2] = 0.0
    w["embed"][query_token, 0] = 1.0
    w["embed"][key_token, 1] = 1.0
    u = torch.randn(d - rot, generator=g, dtype=torch.float64)
    p = "l0.mix.left"
    for h in range(H):
        w[p + ".q"][h * d + rot:(h + 1) * d] += strength * torch.outer(u, a)
    for h in range(G):
        w[p + ".k"][h * d + rot:(h + 1) * d] += strength * torch.outer(u, b)
    w[p + ".v"] += 3.0 * torch.outer(torch.randn(w[p + ".v"].shape[0], generator=g, dtype=torch.float64), b)
    return w


def aimed_latent(cfg, w, query_token, key_token, strength=30.0, score=25.0):
    """The same for a model whose FIRST layer is latent attention: channel 0 of both latents is
    the aimed tokens' own, and the up-projections turn it into one vector in the unrotated
    part of every head, of a length that makes the aimed score ``score``."""
    m = cfg["layers"][0]["mixer"]
    H, d, dr, rank, q_rank = m["heads"], m["dim"], m["rot_dim"], m["kv_rank"], m["q_rank"]
    g = torch.Generator().manual_seed(98)
    w["embed"][:, :2] = 0.0
    w["embed"][query_token, 0] = 1.0
    w["embed"][key_token, 1] = 1.0
    p = "l0.mix"
    w[p + ".dq"][0] = 0.0
    w[p + ".dq"][0, 0] = strength
    w[p + ".dkv"][0] = 0.0
    w[p + ".dkv"][0, 1] = strength
    w[p + ".dq"][1:, 0] = 0.0
    w[p + ".dkv"][1:, 1] = 0.0
    u = torch.randn(d, generator=g, dtype=torch.float64)
    u = u / u.norm()
    # after the norms channel 0 holds about sqrt(q_rank) g_q[0] and sqrt(rank) g_c[0]
    amp = math.sqrt(score / (float(m["scale"]) * math.sqrt(q_rank * rank)
                             * abs(float(w[p + ".dq.norm"][0] * w[p + ".dkv.norm"][0]))))
    for h in range(H):
        w[p + ".uq"][h * (d + dr):h * (d + dr) + d, 0] = amp * u
        w[p + ".uq"][h * (d + dr) + d:(h + 1) * (d + dr), 0] = 0.0
        w[p + ".uk"][h * d:(h + 1) * d, 0] = amp * u
    w[p + ".uv"][:, 0] = 2.0 * torch.randn(w[p + ".uv"].shape[0], generator=g, dtype=torch.float64)
    return w
