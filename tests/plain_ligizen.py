"""A plain, slow implementation of the Ligizen decoder: whole sequences, no cache, no paging, no
batching, one function per mechanism, plain torch arithmetic on the CPU in one precision (float64
by default).  It shares no code with `inferrs_amd`: a model is a config dictionary (the keys of
config.json) and a dictionary of tensors by their names in the file.

The design in short.  A layer norms the stream once (a layer norm with weight and bias) and both of its sub-layers read
that: x <- x + mixer(h) + ff(h).  Behind the sum a small input of the token itself enters: a slice of a second
embedding table, gated by a projection of the stream, projected back, RMS-normed and added.  Two mixers.  "attention":
grouped keys, biases on q, k and v, a turn by position of a head's first features (halves paired) with frequencies
stretched the way Llama 3.1 stretches them, q and k brought to unit root mean square a head BEHIND the turn, a mask
of chunks (a query sees the keys of its own chunk up to itself), one sigmoid gate a head; a layer may read the keys and
values that an earlier layer cached.  "latent_attention": queries through a normed low-rank row, keys and values from
one normed low-rank row a token plus one turned key part that all heads share (neighbours paired), a sliding
window, a learned term a head in the softmax's denominator, one sigmoid gate a head.  The feed-forward is a gated SiLU
layer or routed experts: sigmoid scores, the best `top`, the score multiplying the expert's INPUT, clamped experts, and
a shared expert behind a sigmoid gate a token.  Logits through a matrix of their own, then capped by a tanh.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

T = Dict[str, torch.Tensor]

EXPERT_SLOPE = 1.702          # the experts' activation is g * sigmoid(1.702 g)


# ---- small pieces ---------------------------------------------------------------------------

def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    mu = x.mean(dim=-1, keepdim=True)
    var = ((x - mu) ** 2).mean(dim=-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def frequencies(rot: dict, dtype) -> torch.Tensor:
    """f_i = base^(-2i/dims), then stretched where `scaling` says so: wavelengths shorter than original/high stay, longer
    than original/low are divided by factor, between them a blend."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if sc:
        factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
        out = []
        for fi in f:
            wave = 2.0 * math.pi / fi
            if wave < orig / high:
                out.append(fi)
            elif wave > orig / low:
                out.append(fi / factor)
            else:
                s = (orig / wave - low) / (high - low)
                out.append((1.0 - s) * fi / factor + s * fi)
        f = out
    return torch.tensor(f, dtype=dtype)


def turn(x: torch.Tensor, positions: torch.Tensor, rot: dict, neighbours: bool) -> torch.Tensor:
    """x [tokens, heads, dim]: the first rot.dims features of every head turn; feature i with i + dims/2, or, with
    `neighbours`, 2i with 2i + 1."""
    dims = int(rot.get("dims", 0)) if rot else 0
    if dims == 0:
        return x
    half = dims // 2
    a = positions.to(x.dtype)[:, None, None] * frequencies(rot, x.dtype)[None, None, :]
    c, s = torch.cos(a), torch.sin(a)
    out = x.clone()
    if neighbours:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * c - v * s
        out[..., half:dims] = v * c + u * s
    return out


def softmax_rows(scores: torch.Tensor, seen: torch.Tensor, extra: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Softmax over the seen keys of every row; `extra` [rows]: one more term exp(extra) in the denominator."""
    s = scores.masked_fill(~seen, float("-inf"))
    m = s.max(dim=-1, keepdim=True).values
    if extra is not None:
        m = torch.maximum(m, extra[:, None])
    e = torch.exp(s - m)
    den = e.sum(dim=-1, keepdim=True)
    if extra is not None:
        den = den + torch.exp(extra[:, None] - m)
    return e / den


# ---- the mixers -------------------------------------------------------------------------------

def chunk_keys_values(h: torch.Tensor, w: T, p: str, m: dict, eps: float):
    """What an "attention" layer with projections of its own caches: keys after the turn and the unit norm [n, G, dim],
    values [n, G, vdim]."""
    n = h.shape[0]
    G, d, dv = int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(n, G, d)
    k = rms_norm(turn(k, torch.arange(n), m.get("rot"), False), None, eps)
    return k, (h @ w[p + "v"].T + w[p + "v.b"]).view(n, G, dv)


def chunk_attention(h: torch.Tensor, w: T, p: str, m: dict, eps: float, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    n = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    size = int(m["mask"]["size"])
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(n, H, d)
    q = rms_norm(turn(q, torch.arange(n), m.get("rot"), False), None, eps)
    i = torch.arange(n)
    seen = (i[:, None] >= i[None, :]) & ((i[:, None] // size) == (i[None, :] // size))
    gate = torch.sigmoid(h @ w[p + "g"].T)                     # [n, H]
    out = torch.zeros(n, H, dv, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * float(m["scale"])
        out[:, head] = (softmax_rows(s, seen) @ v[:, g]) * gate[:, head:head + 1]
    return out.reshape(n, H * dv) @ w[p + "o"].T


def latent_attention(h: torch.Tensor, w: T, p: str, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, d, r, dv, rank = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    window = int(m["mask"]["size"])
    pos = torch.arange(n)
    rot = dict(m["rot"])
    cq = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].T).view(n, H, d + r)
    q_plain, q_rot = q[..., :d], turn(q[..., d:], pos, rot, True)
    down = h @ w[p + "dkv"].T
    c = rms_norm(down[:, :rank], w[p + "dkv.norm"], eps)
    k_rot = turn(down[:, rank:].view(n, 1, r), pos, rot, True)[:, 0]
    k_plain = (c @ w[p + "uk"].T).view(n, H, d)
    v = (c @ w[p + "uv"].T).view(n, H, dv)
    seen = (pos[:, None] >= pos[None, :]) & (pos[:, None] - pos[None, :] < window)
    gate = torch.sigmoid(h @ w[p + "g"].T)
    out = torch.zeros(n, H, dv, dtype=h.dtype)
    for head in range(H):
        s = (q_plain[:, head] @ k_plain[:, head].T + q_rot[:, head] @ k_rot.T) * float(m["scale"])
        prob = softmax_rows(s, seen, w[p + "sink"][head].expand(n))
        out[:, head] = (prob @ v[:, head]) * gate[:, head:head + 1]
    return out.reshape(n, H * dv) @ w[p + "o"].T


# ---- the feed-forwards --------------------------------------------------------------------------

def gated_ff(h: torch.Tensor, w: T, p: str) -> torch.Tensor:
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def clamped_expert(h: torch.Tensor, w: T, p: str, limit: float) -> torch.Tensor:
    g = (h @ w[p + "gate"].T).clamp(max=limit)
    u = (h @ w[p + "up"].T).clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(EXPERT_SLOPE * g) * (u + 1.0)) @ w[p + "down"].T


def route(h: torch.Tensor, w: T, p: str, top: int):
    """(chosen experts [n, top], their weights [n, top]): the sigmoid of every logit, the largest `top`, as they are."""
    s = torch.sigmoid(h @ w[p + "router"].T)
    chosen = torch.topk(s, top, dim=-1).indices
    return chosen, torch.gather(s, 1, chosen)


def routed_ff(h: torch.Tensor, w: T, p: str, f: dict) -> torch.Tensor:
    top = int(f["router"]["top"])
    chosen, weight = route(h, w, p, top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(chosen[t, j])
            out[t] += clamped_expert(weight[t, j] * h[t:t + 1], w, f"{p}e{e}.", float(f["expert"]["limit"]))[0]
    if f.get("shared"):
        out = out + clamped_expert(h, w, p + "shared.", float(f["shared"]["limit"])) * torch.sigmoid(h @ w[p + "shared.sg"].T)
    return out


def feed_forward(h: torch.Tensor, w: T, p: str, f: dict) -> torch.Tensor:
    if f["kind"] == "dense":
        return gated_ff(h, w, p)
    if f["kind"] == "moe":
        return routed_ff(h, w, p, f)
    raise ValueError(f"feed-forward kind {f['kind']!r}")


def token_input(x: torch.Tensor, w: T, p: str, rows: torch.Tensor, eps: float) -> torch.Tensor:
    """What a token itself adds behind a layer: `rows` is the layer's slice of the second table for the tokens."""
    y = (gelu_tanh(x @ w[p + "gate"].T) * rows) @ w[p + "proj"].T
    return rms_norm(y, w[p + "norm"], eps)


# ---- the model ------------------------------------------------------------------------------------

def forward(cfg: dict, w: T, tokens: Sequence[int], dtype=torch.float64, layers_out: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits [tokens, vocab] of one sequence from position 0.  `layers_out` receives the stream after every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps = float(cfg["norm"]["eps"])
    ids = torch.tensor(list(tokens), dtype=torch.long)
    x = w["embed"][ids] * float(cfg["embedding"]["scale"])
    side = int(cfg["token_side"]["dim"]) if cfg.get("token_side") else 0
    cached = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps)
        if layer["type"] == "attention":
            if m.get("kv_from") is None:
                cached[i] = chunk_keys_values(h, w, p + "mix.", m, eps)
            k, v = cached[i if m.get("kv_from") is None else int(m["kv_from"])]
            y = chunk_attention(h, w, p + "mix.", m, eps, k, v)
        elif layer["type"] == "latent_attention":
            y = latent_attention(h, w, p + "mix.", m, eps)
        else:
            raise ValueError(f"layer type {layer['type']!r}")
        if layer.get("mlp") is not None:
            y = y + feed_forward(h, w, p + "mlp.", layer["mlp"])
        x = x + y
        if side:
            x = x + token_input(x, w, p + "side.", w["side.embed"][ids, i * side:(i + 1) * side], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    logits = x @ w["head"].T
    if cfg.get("logit_softcap") is None:            # (a model without a cap)
        return logits
    cap = float(cfg["logit_softcap"])
    return cap * torch.tanh(logits / cap)
