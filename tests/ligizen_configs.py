"""Tiny Ligizen configurations that differ in every size and option, and random weights for them.

The tensor list is written out here from the design (not asked of the package), so a part that expects another name
or shape fails to load.  Weights are drawn so that the mechanisms matter: matrices N(0, 1/in), norm weights around 1,
biases and sink values of a size that shows, experts' inputs large enough for the limits to bite now and then.
`sharpened` multiplies every mixer's `scale` so that a query singles out a few keys of what it sees, and a key that is
lost, read from a wrong page or one place outside a window or chunk changes the logits by far more than rounding."""
from __future__ import annotations

import copy
import json
import os
from typing import Dict

import torch


def rot(base, dims, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return r


def attn(heads, kv_heads, dim, vdim, scale, chunk, base=10000.0, turned=None, scaling=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": chunk},
         "rot": rot(base, dim if turned is None else turned, scaling)}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, window, base=10000.0):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                      "scale": scale, "mask": {"size": window}, "rot": rot(base, rot_dim)}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit, shared=None):
    f = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared is not None:
        f["shared"] = {"ff": shared[0], "limit": shared[1]}
    return f


def layer(mixer, mlp):
    return {**mixer, "mlp": mlp}


def model(vocab, width, layers, eps=1e-6, embed_scale=1.0, cap=30.0, side=None):
    cfg = {"architecture": "Ligizen", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "embedding": {"scale": embed_scale}, "logit_softcap": cap, "layers": layers}
    if side:
        cfg["token_side"] = {"dim": side}
    return cfg


# A: both mixers, grouped keys with values half as wide, part of a head turning with stretched frequencies (the three
# ranges of wavelengths all occur: base 50 over 8 features against an original length of 40), a reader whose chunks (40)
# are longer than its owner's (24: a page and a half), a window of 24, two experts a token of five with a shared expert,
# a layer without feed-forward, a token's own input of 6.
CFG_A = model(211, 48, [
    layer(latent(4, 8, 4, 8, 16, 12, 0.3, 24, base=1000.0), dense(40)),
    layer(attn(4, 2, 16, 8, 0.25, 24, base=50.0, turned=8, scaling=(4.0, 1.0, 4.0, 40)), moe(5, 2, 24, 1.2, shared=(32, 0.8))),
    layer(latent(2, 16, 8, 4, 8, 24, 0.2, 17, base=50000.0), moe(4, 1, 16, 2.5)),
    layer(attn(4, 2, 16, 8, 0.3, 40, base=50.0, turned=8, scaling=(4.0, 1.0, 4.0, 40), kv_from=1), None)],
    eps=1e-5, embed_scale=3.0, cap=8.0, side=6)
# B: every constant 1 and every size equal where the design lets them differ: as many key heads as query heads, values as
# wide as keys (64 and 48 + 16: the matrix cores in bfloat16), whole heads turning without stretching, chunks and a window
# of 1 (a token sees itself), a router that takes all its experts, no token input, a cap of 1.
CFG_B = model(97, 64, [
    layer(attn(2, 2, 64, 64, 0.125, 100, turned=64), moe(2, 2, 40, 7.0, shared=(40, 7.0))),
    layer(latent(2, 16, 16, 16, 16, 48, 0.2, 100, base=100.0), dense(72)),
    layer(attn(1, 1, 64, 64, 0.125, 1, turned=64), dense(24)),
    layer(latent(2, 16, 16, 16, 16, 48, 0.2, 1, base=100.0), None)],
    cap=1.0)
# C: sizes that fit no vector width: a width of 50, keys of 12 and values of 20, five heads, chunks of 17, three experts,
# feed-forwards of 30 and 22, a latent row of 14 + 6, a token input of 5.
CFG_C = model(101, 50, [
    layer(attn(5, 5, 12, 20, 0.4, 17, base=777.0, turned=6), moe(3, 2, 30, 1.0, shared=(22, 1.5))),
    layer(latent(3, 10, 6, 14, 10, 14, 0.3, 9, base=777.0), moe(3, 3, 30, 1.0)),
    layer(attn(5, 5, 12, 20, 0.4, 9, base=777.0, turned=6, kv_from=0), dense(30))],
    eps=1e-5, embed_scale=0.5, cap=3.0, side=5)
# D: the matrix cores' sizes with long sequences: keys of 128 and values of 64 over one key head for four query heads in
# chunks of 300 that two readers share, one with shorter chunks; a latent row of 96 + 32 under a window of 200 with eight
# heads; keys of 64 with values of 16.
CFG_D = model(150, 64, [
    layer(attn(4, 1, 128, 64, 0.09, 300, base=30000.0, turned=48, scaling=(8.0, 1.0, 4.0, 256)), dense(48)),
    layer(latent(8, 32, 32, 16, 24, 96, 0.12, 200, base=5000.0), moe(6, 2, 32, 1.3, shared=(16, 2.2))),
    layer(attn(4, 1, 128, 64, 0.09, 300, base=30000.0, turned=48, scaling=(8.0, 1.0, 4.0, 256), kv_from=0), None),
    layer(attn(2, 2, 64, 16, 0.15, 64, base=100.0), dense(48)),
    layer(attn(4, 1, 128, 64, 0.12, 33, base=30000.0, turned=48, scaling=(8.0, 1.0, 4.0, 256), kv_from=0), dense(48))],
    embed_scale=8.0, cap=12.0, side=8)
CONFIGS = {"A": CFG_A, "B": CFG_B, "C": CFG_C, "D": CFG_D}


def sharpened(cfg: dict, factor: float) -> dict:
    """The same model with every mixer's `scale` multiplied: its queries single out few of the keys they see."""
    out = copy.deepcopy(cfg)
    for L in out["layers"]:
        L["mixer"]["scale"] = L["mixer"]["scale"] * factor
    return out


def tensor_shapes(cfg: dict) -> Dict[str, tuple]:
    """Every tensor of a model, from the design."""
    W, V = cfg["width"], cfg["vocab"]
    side = cfg["token_side"]["dim"] if cfg.get("token_side") else 0
    out = {"embed": (V, W), "final.norm": (W,), "final.norm.b": (W,), "head": (V, W)}
    if side:
        out["side.embed"] = (V, side * len(cfg["layers"]))
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        out[p + "norm1"] = (W,)
        out[p + "norm1.b"] = (W,)
        H = m["heads"]
        if L["type"] == "attention":
            G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * d, W), p + "mix.q.b": (H * d,), p + "mix.g": (H, W), p + "mix.o": (W, H * dv)})
            if m.get("kv_from") is None:
                out.update({p + "mix.k": (G * d, W), p + "mix.k.b": (G * d,), p + "mix.v": (G * dv, W), p + "mix.v.b": (G * dv,)})
        else:
            d, r, dv, qr, kr = m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            out.update({p + "mix.dq": (qr, W), p + "mix.dq.norm": (qr,), p + "mix.uq": (H * (d + r), qr),
                        p + "mix.dkv": (kr + r, W), p + "mix.dkv.norm": (kr,), p + "mix.uk": (H * d, kr),
                        p + "mix.uv": (H * dv, kr), p + "mix.sink": (H,), p + "mix.g": (H, W), p + "mix.o": (W, H * dv)})
        if side:
            out.update({p + "side.gate": (side, W), p + "side.proj": (W, side), p + "side.norm": (W,)})
        f = L["mlp"]
        if f is None:
            continue
        if f["kind"] == "dense":
            out.update({p + "mlp.gate": (f["ff"], W), p + "mlp.up": (f["ff"], W), p + "mlp.down": (W, f["ff"])})
            continue
        out[p + "mlp.router"] = (f["router"]["experts"], W)
        for e in range(f["router"]["experts"]):
            q = f"{p}mlp.e{e}."
            out.update({q + "gate": (f["expert"]["ff"], W), q + "up": (f["expert"]["ff"], W), q + "down": (W, f["expert"]["ff"])})
        if f.get("shared"):
            q, ff = p + "mlp.shared.", f["shared"]["ff"]
            out.update({q + "gate": (ff, W), q + "up": (ff, W), q + "down": (W, ff), q + "sg": (1, W)})
    return out


def random_weights(cfg: dict, seed: int, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".", 1)[1] if name.startswith("l") and name[1].isdigit() else name
        if leaf in ("norm1", "mix.dq.norm", "mix.dkv.norm", "final.norm"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif leaf == "side.norm":
            t = 0.5 + 0.1 * torch.randn(shape, generator=g)
        elif leaf.endswith(".b"):
            t = 0.3 * torch.randn(shape, generator=g)
        elif leaf == "mix.sink":
            t = 1.0 + torch.randn(shape, generator=g)                       # (a denominator's term the size of a few keys')
        elif leaf == "mlp.router":
            t = 2.0 * torch.randn(shape, generator=g) / shape[-1] ** 0.5
        elif name in ("embed", "side.embed"):
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) / shape[-1] ** 0.5
            if leaf.endswith(("gate", "up")) and ("mlp.e" in leaf or "shared" in leaf):
                t = t * 1.5                                                  # so that the experts' limits bite now and then
        out[name] = t.to(dtype)
    return out


def write_model(folder: str, cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    from inferrs_amd.weights import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    weights = random_weights(cfg, seed)
    write_safetensors(os.path.join(folder, "model.safetensors"), weights)
    return weights


def random_tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
