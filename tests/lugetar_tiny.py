"""Small Lugetar configurations for the tests, each unlike the others in every size and constant,
and helpers to write them as model folders.

G1: both mixers and both feed-forwards: attention of 4 heads on 2 KV heads of 32 with a query
    temperature that steps every 20 positions; a parallel mixer whose left half has 4 heads on 2
    KV heads of 32 with values of 16, 16 elements that turn (slow pairs slowed down), chunks of 24,
    beside a delta rule of 4 heads on 2 key heads of 16 x 24 with 3 taps; 8 experts in 4 groups
    of which 2 are kept, 3 chosen, a shared expert.
G2: the parallel mixer first; values wider than keys on the left; as many key heads as heads;
    a convolution of 2 taps; no groups of experts, one chosen, no shared expert; a layer without
    feed-forward; residual factor and embedding scale of one.
G3: heads of 64 and 128 with values as wide (the kernels on the matrix cores), whole-head
    rotation without slowed pairs, chunks of 64 (whole pages), a convolution of one tap (no
    inputs to keep), all groups kept, every expert chosen.
G4: nothing a multiple of 4 or 8: width 50, five heads of 20 with values of 12, chunks of 7, one
    key head for three delta heads of 12 x 10 with 5 taps, 6 experts in 3 groups of 2 of which 1 is
    kept, ranks of 3 and 5, a temperature that steps at every position.
G5: attention layers with a chunked mask and a rotation of their own, a left half without either,
    a delta head of 128 x 128, experts in groups of one.
A1, P1: one mixer each, alone, without feed-forward.
"""

import json
import os

import torch

import plain_lugetar as P


def attn(heads, kv, dim, vdim=None, rot=None, base=10000.0, scaling=None, chunk=0, temp=None, scale=None):
    a = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim or dim, "scale": scale or 1.3 * dim ** -0.5}
    if rot:
        a["rot"] = {"base": base, "dims": rot}
        if scaling:
            a["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    if chunk:
        a["mask"] = {"size": chunk}
    if temp:
        a["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return a


def delta(heads, kv, dim, vdim, conv, a_rank=None, gate_rank=None):
    d = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}
    if a_rank:
        d["a_rank"] = a_rank
    if gate_rank:
        d["gate_rank"] = gate_rank
    return d


def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts, top, ff, groups=None, scale=None, shared=None):
    router = {"experts": experts, "top": top}
    if scale is not None:
        router["scale"] = scale
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def layer(kind, mixer, mlp=None):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def parallel(left, right, mlp=None):
    return layer("parallel", {"left": left, "right": right}, mlp)


def _cfg(vocab, width, eps, scale, mult, layers):
    return {"architecture": "Lugetar", "vocab": vocab, "width": width, "embedding": {"scale": scale},
            "norm": {"eps": eps}, "residual_mult": mult, "layers": layers}


_L1 = attn(4, 2, 32, vdim=16, rot=16, base=5000.0, scaling=(4.0, 1.0, 3.0, 48), chunk=24)

CONFIGS = {
    "G1": _cfg(90, 64, 1e-5, 2.5, 0.8, [
        layer("attention", attn(4, 2, 32, temp=(0.4, 20)), dense(80, 1.2)),
        parallel(_L1, delta(4, 2, 16, 24, 3), moe(8, 3, 24, groups=(4, 2), scale=1.7, shared=40)),
        layer("attention", attn(4, 2, 32, temp=(0.4, 20)), dense(80, 1.2)),
        parallel(_L1, delta(4, 2, 16, 24, 3), moe(8, 3, 24, groups=(4, 2), scale=1.7, shared=40))]),
    "G2": _cfg(128, 96, 1e-6, 1.0, 1.0, [
        parallel(attn(3, 3, 16, vdim=40, rot=8, base=300.0, chunk=40), delta(2, 2, 64, 32, 2), moe(5, 1, 56)),
        layer("attention", attn(6, 1, 16, vdim=8, temp=(0.25, 64))),
        parallel(attn(3, 3, 16, vdim=40, rot=8, base=300.0, chunk=40), delta(2, 2, 64, 32, 2), dense(72, 0.7))]),
    "G3": _cfg(101, 128, 1e-4, 4.0, 0.5, [
        layer("attention", attn(2, 1, 128, temp=(0.3, 50)), moe(4, 4, 32, groups=(2, 2), scale=0.6, shared=16)),
        parallel(attn(4, 2, 64, rot=64, base=20000.0, chunk=64), delta(3, 1, 128, 16, 1), dense(96, 2.0))]),
    "G4": _cfg(61, 50, 1e-5, 1.7, 1.3, [
        parallel(attn(5, 5, 20, vdim=12, rot=10, base=77.0, scaling=(2.5, 2.0, 5.0, 30), chunk=7),
                 delta(3, 1, 12, 10, 5, a_rank=3, gate_rank=5), moe(6, 2, 18, groups=(3, 1), scale=2.2, shared=10)),
        layer("attention", attn(5, 1, 10, vdim=14, temp=(0.5, 1)), dense(34, 0.9))]),
    "G5": _cfg(77, 64, 1e-3, 1.0, 0.9, [
        layer("attention", attn(2, 2, 32, rot=32, base=100.0, chunk=16, temp=(0.2, 7)), moe(6, 2, 16, groups=(6, 3))),
        parallel(attn(2, 1, 32), delta(1, 1, 128, 128, 4), dense(40, 5.0))]),
    "A1": _cfg(50, 32, 1e-5, 2.0, 0.65, [layer("attention", attn(4, 2, 24, vdim=40, temp=(0.3, 16)))]),
    "P1": _cfg(50, 40, 1e-5, 2.0, 0.75, [parallel(attn(2, 1, 48, vdim=16, rot=24, chunk=20), delta(4, 2, 24, 40, 4))]),
}

# Sizes nearer to a real model's layers: heads of 64 and 128 on the matrix cores' kernels, delta
# heads of 64 x 96 and 128 x 128, sixteen experts.
CONFIGS["G6"] = _cfg(200, 192, 1e-6, 1.5, 0.6, [
    layer("attention", attn(6, 2, 64, temp=(0.35, 100)), dense(160, 1.75)),
    parallel(attn(6, 2, 64, rot=32, base=30000.0, scaling=(6.0, 1.0, 4.0, 64), chunk=48), delta(6, 3, 64, 96, 4),
             moe(16, 4, 48, groups=(4, 3), scale=2.0, shared=64)),
    parallel(attn(4, 4, 128, rot=128, base=30000.0, chunk=80), delta(2, 1, 128, 128, 4), dense(128, 1.0))])


def without_choice(cfg):
    """The configuration with routers that choose every expert of every group: nothing then hangs
    on a close call between two scores, which rounding to bfloat16 can tip either way (and which
    the positions behind it then inherit through caches and states)."""
    import copy
    out = copy.deepcopy(cfg)
    for entry in out["layers"]:
        mlp = entry.get("mlp")
        if mlp and mlp["kind"] == "moe":
            mlp["router"]["top"] = mlp["router"]["experts"]
            if "groups" in mlp["router"]:
                mlp["router"]["groups"]["keep"] = mlp["router"]["groups"]["count"]
    return out


for _name in ("G1", "G2", "G3", "G4", "G5", "G6"):
    CONFIGS[_name + "n"] = without_choice(CONFIGS[_name])


def random_config(seed):
    """A configuration drawn from a seed: two to five layers in any order, every size and constant
    drawn anew (also the values that configurations written by hand tend to make equal or 1)."""
    import random
    r = random.Random(seed)
    pick = r.choice

    def attention(left):
        kv = pick([1, 2, 3, 4])
        heads = kv * pick([1, 2, 3])
        dim = pick([8, 12, 16, 24, 32, 40, 64, 128])
        a = attn(heads, kv, dim, vdim=pick([dim, dim, 8, 20, 48]), scale=r.uniform(0.6, 1.6) * dim ** -0.5)
        if r.random() < (0.8 if left else 0.3):
            dims = pick([d for d in (4, 8, dim // 2, dim) if d <= dim and d % 2 == 0])
            a["rot"] = {"base": pick([50.0, 1000.0, 500000.0]), "dims": dims}
            if r.random() < 0.6:
                low = pick([1.0, 2.0])
                a["rot"]["scaling"] = {"factor": pick([2.0, 8.0, 32.0]), "low": low, "high": low + pick([1.0, 3.0]),
                                       "original": pick([16, 64, 256])}
        if r.random() < (0.85 if left else 0.3):
            a["mask"] = {"size": pick([1, 5, 16, 23, 32, 50, 64, 100])}
        if r.random() < (0.3 if left else 0.85):
            a["q_temp"] = {"coef": r.uniform(0.05, 0.6), "every": pick([1, 3, 16, 64, 1000])}
        return a

    def feed_forward():
        kind = pick(["dense", "dense", "moe", "moe", None])
        if kind is None:
            return None
        if kind == "dense":
            return dense(pick([16, 40, 72, 130]), pick([0.5, 1.0, 3.0, 20.0]))
        count = pick([1, 2, 3, 4])
        experts = count * pick([1, 2, 3, 4])
        keep = r.randint(1, count)
        top = r.randint(1, experts // count * keep)
        return moe(experts, top, pick([8, 24, 50]), groups=(count, keep) if r.random() < 0.8 else None,
                   scale=pick([None, 1.0, 0.5, 3.0]), shared=pick([None, 16, 36]))

    layers = []
    for _ in range(r.randint(2, 5)):
        if r.random() < 0.5:
            layers.append(layer("attention", attention(False), feed_forward()))
        else:
            kv = pick([1, 2, 4])
            right = delta(kv * pick([1, 2, 3]), kv, pick([8, 16, 20, 32, 64]), pick([8, 16, 24, 64]), pick([1, 2, 3, 4, 6]))
            layers.append(parallel(attention(True), right, feed_forward()))
    cfg = _cfg(pick([40, 97, 256]), pick([24, 32, 50, 64, 96]), pick([1e-6, 1e-5, 1e-3]), pick([1.0, 3.0, 11.0]),
               pick([1.0, 0.4, 1.4]), layers)
    for entry in cfg["layers"]:          # a router without groups may choose among all its experts
        mlp = entry["mlp"]
        if mlp and mlp["kind"] == "moe" and "groups" not in mlp["router"]:
            mlp["router"]["top"] = r.randint(1, mlp["router"]["experts"])
    return cfg


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
    out = {}
    for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items():
        v = v.float()
        wide = v.dim() < 2 or k.endswith(".conv")
        if as_stored_in == "bfloat16" and not wide:
            v = v.to(torch.bfloat16).float()
        out[k] = v.double()
    return out


def tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def aimed_attention(cfg, w, layer_prefix, m, query_token, key_token, strength=30.0):
    """Changes ``w`` (weights of a model whose FIRST layer holds the attention ``m`` under
    ``layer_prefix``) so that there the query of ``query_token`` looks along the key of
    ``key_token`` wherever it stands: the two tokens get an embedding direction of their own each,
    which the query and key matrices turn into one and the same long vector in the part of every
    head that does not rotate.  The norms make every query and key as long as any other, so the
    aimed score is far above a random one; the value of ``key_token`` is unlike any other, and the
    layer's mixer weighs three times as much in the stream."""
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
    p = layer_prefix
    for h in range(H):
        w[p + ".q"][h * d + rot:(h + 1) * d] += strength * torch.outer(u, a)
    for h in range(G):
        w[p + ".k"][h * d + rot:(h + 1) * d] += strength * torch.outer(u, b)
    w[p + ".v"] += 3.0 * torch.outer(torch.randn(w[p + ".v"].shape[0], generator=g, dtype=torch.float64), b)
    # the mixer's output is normed, so a value's length does not show: the aimed half and this
    # layer's mixer are given more weight in the stream instead
    if p.endswith(".left"):
        w[p[:-5] + ".right.out"] *= 0.2
    w["l0.norm1b"] *= 3.0
    return w
