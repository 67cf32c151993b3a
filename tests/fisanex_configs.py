"""Tiny Fisanex configurations that differ in every size and option, and random weights for them.

The tensor list is written out here from the design (not asked of the package), so a part that expects another name
or shape fails to load.  Weights are drawn so that the mechanisms matter: matrices N(0, 1/in), norm weights around 1,
router corrections large enough to change the choice against the scores alone; `sharpen` multiplies the weight of the
queries' norm (the norm takes any factor on the projection itself away) so that a query singles out a few keys of its
window, and a key that is lost, read from a wrong page or one place outside the window changes the logits by far more
than rounding."""
from __future__ import annotations

import json
import os
from typing import Dict

import torch


def attn(heads, kv_heads, dim, vdim, scale, window, base=10000.0, turned=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": window}}
    if turned is None or turned > 0:
        m["rot"] = {"base": base, "dims": dim if turned is None else turned}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, identity, top, ff, limit, shared=None):
    f = {"kind": "moe", "router": {"experts": experts, "identity": identity, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared is not None:
        f["shared"] = {"ff": shared[0], "limit": shared[1]}
    return f


def layer(mixer, mlp):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def model(vocab, width, layers, eps=1e-6, alpha=1.0, embed_scale=1.0, logit_scale=1.0):
    return {"architecture": "Fisanex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "postln_alpha": alpha,
            "embedding": {"scale": embed_scale}, "logit_scale": logit_scale, "layers": layers}


# A: grouped keys, values half as wide as keys, part of a head turning, a reader whose window (40) is wider than its
# owner's (24: a page and a half), experts with outputs that hand the input on and a shared expert; then values WIDER
# than keys over a single key head with whole heads turning, a router without such outputs and without a shared expert
# that takes one expert a token; a reader with a window of 5 and no feed-forward.
CFG_A = model(211, 48, [
    layer(attn(4, 2, 16, 8, 0.3, 24, base=1000.0, turned=8), dense(40)),
    layer(attn(4, 2, 16, 8, 0.25, 40, base=1000.0, turned=8, kv_from=0), moe(5, 2, 3, 24, 1.2, shared=(32, 0.8))),
    layer(attn(2, 1, 32, 48, 0.2, 17, base=50000.0), moe(4, 0, 1, 16, 2.5)),
    layer(attn(2, 1, 32, 48, 0.2, 5, base=50000.0, kv_from=2), None)],
    eps=1e-5, alpha=1.5, embed_scale=3.0, logit_scale=0.5)
# B: every constant 1 and every size equal where the design lets them differ: values as wide as keys (64: the
# matrix cores in bfloat16), as many key heads as query heads, no turning, a window of 100, a router that takes all of its
# outputs, no reader at all.
CFG_B = model(97, 64, [
    layer(attn(2, 2, 64, 64, 0.125, 100, turned=0), moe(2, 2, 4, 40, 7.0, shared=(40, 7.0))),
    layer(attn(2, 2, 64, 64, 0.125, 1, turned=0), dense(72))])
# C: sizes that fit no vector width: a width of 50, keys of 12 and values of 20, five heads, a window of 17, three
# experts and one output that hands on, feed-forwards of 30 and 22.
CFG_C = model(101, 50, [
    layer(attn(5, 5, 12, 20, 0.4, 17, base=777.0, turned=6), moe(3, 1, 2, 30, 1.0, shared=(22, 1.5))),
    layer(attn(5, 5, 12, 20, 0.4, 9, base=777.0, turned=6, kv_from=0), dense(30))],
    eps=1e-5, alpha=0.7, embed_scale=0.5, logit_scale=2.0)
# D: keys of 128 and values of 64 over one key head for four query heads (the matrix cores' kernels with values of a
# width of their own; long prompts, keys split between waves in decode steps), a window of 300 that two readers share, one
# of them further down with a narrower window; values of 16 beside keys of 64 in the last layer.
CFG_D = model(150, 64, [
    layer(attn(4, 1, 128, 64, 0.09, 300, base=30000.0, turned=48), dense(48)),
    layer(attn(2, 2, 64, 16, 0.15, 64, base=100.0), None),
    layer(attn(4, 1, 128, 64, 0.09, 300, base=30000.0, turned=48, kv_from=0), moe(6, 3, 2, 32, 1.3, shared=(16, 2.2))),
    layer(attn(4, 1, 128, 64, 0.12, 33, base=30000.0, turned=48, kv_from=0), dense(48))],
    alpha=2.5, embed_scale=8.0, logit_scale=0.3)
CONFIGS = {"A": CFG_A, "B": CFG_B, "C": CFG_C, "D": CFG_D}


def tensor_shapes(cfg: dict) -> Dict[str, tuple]:
    """Every tensor of a model, from the design."""
    W, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, W), "final.norm": (W,)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        out[p + "norm1"] = (W,)
        out.update({p + "mix.q": (H * d, W), p + "mix.q.norm": (d,), p + "mix.g": (H * dv, W), p + "mix.o": (W, H * dv)})
        if m.get("kv_from") is None:
            out.update({p + "mix.k": (G * d, W), p + "mix.k.norm": (d,), p + "mix.v": (G * dv, W)})
        f = L["mlp"]
        if f is None:
            continue
        out[p + "norm2"] = (W,)
        if f["kind"] == "dense":
            out.update({p + "mlp.gate": (f["ff"], W), p + "mlp.up": (f["ff"], W), p + "mlp.down": (W, f["ff"])})
            continue
        r = f["router"]
        out[p + "mlp.router"] = (r["experts"] + r["identity"], W)
        out[p + "mlp.correction"] = (r["experts"] + r["identity"],)
        for e in range(r["experts"]):
            q = f"{p}mlp.e{e}."
            out.update({q + "gate": (f["expert"]["ff"], W), q + "up": (f["expert"]["ff"], W), q + "down": (W, f["expert"]["ff"])})
        if f.get("shared"):
            q, ff = p + "mlp.shared.", f["shared"]["ff"]
            out.update({q + "gate": (ff, W), q + "up": (ff, W), q + "down": (W, ff)})
    return out


def random_weights(cfg: dict, seed: int, sharpen: float = 1.0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".", 1)[1] if name.startswith("l") and name[1].isdigit() else name
        if leaf in ("norm1", "norm2", "mix.k.norm") or name == "final.norm":
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif leaf == "mix.q.norm":
            t = (1.0 + 0.2 * torch.randn(shape, generator=g)) * sharpen
        elif leaf == "mlp.correction":
            t = 0.15 * torch.randn(shape, generator=g)                     # (scores are around 1 / outputs: this reorders them)
        elif leaf == "mlp.router":
            t = 2.0 * torch.randn(shape, generator=g) / shape[-1] ** 0.5
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) / shape[-1] ** 0.5
            if leaf.endswith(("gate", "up")) and "mlp.e" in leaf or "shared" in leaf:
                t = t * 1.5                                                  # so that the experts' clamps bite now and then
        out[name] = t.to(dtype)
    return out


def write_model(folder: str, cfg: dict, seed: int, sharpen: float = 1.0) -> Dict[str, torch.Tensor]:
    from inferrs_amd.weights import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    weights = random_weights(cfg, seed, sharpen)
    write_safetensors(os.path.join(folder, "model.safetensors"), weights)
    return weights


def random_tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
