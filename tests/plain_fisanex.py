"""A plain, slow implementation of the Fisanex decoder: whole sequences, no cache, no paging, no
batching, one function per mechanism, plain torch arithmetic on the CPU in one precision (float64
by default).  It shares no code with `inferrs_amd`: a model is a config dictionary (the keys of
config.json) and a dictionary of tensors by their names in the file.

The design in short.  The stream is normed AFTER every sum: x <- norm_a(alpha x + mixer(x)), then
x <- norm_b(alpha x + ff(x)), and both sub-layers read x as it stands.  The one mixer is a softmax attention over a
sliding window with grouped keys, values narrower or wider than keys, an RMS norm a head on queries and keys, a turn by
position of a head's first features, and a sigmoid gate on the joined heads in front of the output projection; a layer
may use the keys and values that an earlier layer cached instead of projecting its own.  The feed-forward is a gated
SiLU layer or routed experts: a softmax router over real and identity experts, a correction that counts in the
choice and not in the weights, clamped experts, and a shared expert beside them.  The embedding's rows are scaled on the
way in, the logits (a product with the same table, unscaled) on the way out.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

T = Dict[str, torch.Tensor]

EXPERT_SLOPE = 1.702          # the experts' activation is g * sigmoid(1.702 g)


# ---- small pieces ---------------------------------------------------------------------------

def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def rotate_halves(x: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [tokens, heads, dim]: the first `dims` features of every head turn, feature i with i + dims/2."""
    if dims == 0:
        return x
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    a = positions.to(x.dtype)[:, None, None] * f[None, None, :]
    c, s = torch.cos(a), torch.sin(a)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


# ---- the attention ----------------------------------------------------------------------------

def keys_and_values(h: torch.Tensor, w: T, p: str, m: dict, eps: float):
    """What a layer with projections of its own caches: keys after norm and turn [n, G, dim], values [n, G, vdim]."""
    n = h.shape[0]
    G, d, dv = int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    rot = m.get("rot") or {}
    k = (h @ w[p + "k"].T).view(n, G, d)
    k = rotate_halves(rms_norm(k, w[p + "k.norm"], eps), torch.arange(n), float(rot.get("base", 1.0)), int(rot.get("dims", 0)))
    return k, (h @ w[p + "v"].T).view(n, G, dv)


def windowed_attention(h: torch.Tensor, w: T, p: str, m: dict, eps: float, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """The mixer on input h with keys k and values v (its own, or an earlier layer's)."""
    n = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    mask = m.get("mask") or {}
    window = int(mask["size"]) if mask else n + 1              # no mask: every earlier key
    scale = float(m["scale"])
    rot = m.get("rot") or {}
    q = (h @ w[p + "q"].T).view(n, H, d)
    q = rotate_halves(rms_norm(q, w[p + "q.norm"], eps), torch.arange(n), float(rot.get("base", 1.0)), int(rot.get("dims", 0)))
    out = torch.zeros(n, H, dv, dtype=h.dtype)
    i = torch.arange(n)
    seen = (i[:, None] >= i[None, :]) & (i[:, None] - i[None, :] < window)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * scale
        s = s.masked_fill(~seen, float("-inf"))
        out[:, head] = torch.softmax(s, dim=-1) @ v[:, g]
    joined = out.reshape(n, H * dv) * torch.sigmoid(h @ w[p + "g"].T)
    return joined @ w[p + "o"].T


# ---- the feed-forwards --------------------------------------------------------------------------

def gated_ff(h: torch.Tensor, w: T, p: str) -> torch.Tensor:
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def clamped_expert(h: torch.Tensor, w: T, p: str, limit: float) -> torch.Tensor:
    g = (h @ w[p + "gate"].T).clamp(max=limit)
    u = (h @ w[p + "up"].T).clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(EXPERT_SLOPE * g) * (u + 1.0)) @ w[p + "down"].T


def route(h: torch.Tensor, w: T, p: str, top: int):
    """(chosen outputs of the router [n, top], their weights [n, top]): softmax over all outputs; the correction counts
    in the choice only."""
    s = torch.softmax(h @ w[p + "router"].T, dim=-1)
    chosen = torch.topk(s + w[p + "correction"], top, dim=-1).indices
    return chosen, torch.gather(s, 1, chosen)


def routed_ff(h: torch.Tensor, w: T, p: str, f: dict) -> torch.Tensor:
    r = f["router"]
    E, top = int(r["experts"]), int(r["top"])
    chosen, weight = route(h, w, p, top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(chosen[t, j])
            y = clamped_expert(h[t:t + 1], w, f"{p}e{e}.", float(f["expert"]["limit"]))[0] if e < E else h[t]
            out[t] += weight[t, j] * y                       # (an output past the real experts hands the input on)
    if f.get("shared"):
        out = out + clamped_expert(h, w, p + "shared.", float(f["shared"]["limit"]))
    return out


def feed_forward(h: torch.Tensor, w: T, p: str, f: dict) -> torch.Tensor:
    if f["kind"] == "dense":
        return gated_ff(h, w, p)
    if f["kind"] == "moe":
        return routed_ff(h, w, p, f)
    raise ValueError(f"feed-forward kind {f['kind']!r}")


# ---- the model ------------------------------------------------------------------------------------

def forward(cfg: dict, w: T, tokens: Sequence[int], dtype=torch.float64, layers_out: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits [tokens, vocab] of one sequence from position 0.  `layers_out` receives the stream after every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps, alpha = float(cfg["norm"]["eps"]), float(cfg["postln_alpha"])
    x = w["embed"][torch.tensor(list(tokens), dtype=torch.long)] * float(cfg["embedding"]["scale"])
    cached = {}
    for i, layer in enumerate(cfg["layers"]):
        if layer["type"] != "attention":
            raise ValueError(f"layer type {layer['type']!r}")
        p, m = f"l{i}.", layer["mixer"]
        if m.get("kv_from") is None:
            cached[i] = keys_and_values(x, w, p + "mix.", m, eps)
        k, v = cached[i if m.get("kv_from") is None else int(m["kv_from"])]
        x = rms_norm(alpha * x + windowed_attention(x, w, p + "mix.", m, eps, k, v), w[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            x = rms_norm(alpha * x + feed_forward(x, w, p + "mlp.", layer["mlp"]), w[p + "norm2"], eps)
        elif p + "norm2" in w:                  # (a file that holds a second norm for a layer without a feed-forward)
            x = rms_norm(alpha * x, w[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = rms_norm(x, w["final.norm"], eps)
    return (x @ w["embed"].T) * float(cfg["logit_scale"])
