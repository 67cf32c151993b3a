"""Python face of the kernels for several residual streams, latent attention, the gated linear
recurrence and routed experts (`csrc/streams.hip`, `latent.hip`, `recurrence.hip`, `experts.hip`).
Shape checks on the host, then one C call a kernel; no other implementation stands behind them."""
from __future__ import annotations

import ctypes
import os
from typing import Optional, Tuple

import torch

from . import KernelError, _DT, _check, _dev, _dt, _f32, _i32, _p, _stream, library

MAX_STREAMS = 8
MAX_EXPERTS = 256
MAX_TOP = 16
ROW_TILE = 32                 # rows of a tile of the grouped products
LARGE_TILE = int(os.environ.get("INFERRS_AMD_EXPERT_TILE", "64"))     # rows of the matrix cores' large tile: 64 or 128
LARGE_TILE_FROM = 0.75        # rows an expert (on average), in large tiles, from which the experts' products take them
SCORE_FUNCTIONS = {"sigmoid": 0, "softmax": 1}


# ---- residual streams -----------------------------------------------------------------------

def streams_open(x: torch.Tensor, n_streams: int) -> torch.Tensor:
    """Rows [n, width] -> 32-bit streams [n, S, width], every stream a copy of the row."""
    _dev(x)
    n, width = x.shape
    out = torch.empty((n, n_streams, width), dtype=torch.float32, device=x.device)
    _check(library().ia_streams_open(_p(out), _p(x), n, n_streams, width, _dt(x), _stream()))
    return out


def streams_step(streams: torch.Tensor, *, y: Optional[torch.Tensor] = None, y_weights: Optional[torch.Tensor] = None,
                 scale: Optional[torch.Tensor] = None, mix: Optional[torch.Tensor] = None,
                 out: Optional[torch.Tensor] = None, read: Optional[torch.Tensor] = None,
                 norm_weight: Optional[torch.Tensor] = None, eps: float = 0.0,
                 h_dtype: Optional[torch.dtype] = None, rows: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """What stands between two sub-layers of a model with S residual streams.

    `y` [n, width] (or [n, K, width] with `y_weights` [n, K], added up in the order of K): the streams become
    x_t = sum_s mix[s, t] x_s + out[t] * scale * y, in place.  `h_dtype`: returns rmsnorm(sum_s read[s] x_s) *
    norm_weight in that precision (`read` None: every stream counts once; `rows`: only these rows, for a call
    without `y`)."""
    _dev(streams, y, y_weights, scale, mix, out, read, norm_weight, rows)
    for t, name in ((streams, "streams"), (y_weights, "y_weights"), (scale, "scale"), (mix, "mix"), (out, "out"),
                    (read, "read"), (norm_weight, "norm weight")):
        _f32(t, name)
    n, S, W = streams.shape
    K = 1
    if y is not None:
        if y_weights is not None:
            K = y_weights.shape[1]
            if tuple(y.shape) != (n, K, W) or tuple(y_weights.shape) != (n, K):
                raise KernelError(f"streams_step: y {tuple(y.shape)} and its weights {tuple(y_weights.shape)} do not fit [{n}, K, {W}]")
        elif tuple(y.shape) != (n, W):
            raise KernelError(f"streams_step: y {tuple(y.shape)} does not fit [{n}, {W}]")
        if mix is None or out is None or mix.numel() != S * S or out.numel() != S:
            raise KernelError(f"streams_step: an output to add needs mix [{S}, {S}] and out [{S}]")
        if rows is not None:
            raise KernelError("streams_step: a row list goes with a read only")
    if scale is not None and scale.numel() != W:
        raise KernelError(f"streams_step: scale has {scale.numel()} entries, the width is {W}")
    if read is not None and read.numel() != S:
        raise KernelError(f"streams_step: read has {read.numel()} entries for {S} streams")
    h = None
    n_out = n
    if rows is not None:
        _i32(rows, "rows")
        n_out = rows.numel()
    if h_dtype is not None:
        if norm_weight is not None and norm_weight.numel() != W:
            raise KernelError(f"streams_step: the norm weight has {norm_weight.numel()} entries, the width is {W}")
        h = torch.empty((n_out, W), dtype=h_dtype, device=streams.device)
    _check(library().ia_streams_step(
        _p(streams), _p(y), _p(y_weights), K, _p(scale), _p(mix), _p(out), _p(read), _p(norm_weight),
        ctypes.c_float(eps), _p(h), _p(rows), n_out, S, W, _dt(y) if y is not None else 0,
        _DT[h_dtype] if h_dtype is not None else 0, _stream()))
    return h


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """cap * tanh(logits / cap), in place (32-bit)."""
    _dev(logits); _f32(logits, "logits")
    _check(library().ia_softcap(_p(logits), logits.numel(), ctypes.c_float(cap), _stream()))
    return logits


# ---- latent attention -------------------------------------------------------------------------

def latent_prep(proj: torch.Tensor, *, heads: int, dim: int, rot_dim: int, rank: int, rotated: int, q_off: int,
                down_off: int, norm_weight: torch.Tensor, eps: float, cos: Optional[torch.Tensor],
                sin: Optional[torch.Tensor], magnitude: float, k_cache: Optional[torch.Tensor],
                v_cache: Optional[torch.Tensor], slots: Optional[torch.Tensor], page_size: int,
                interleaved: bool = False, q_rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """From the projections' rows to the attention's operands: the latent row is normed (32-bit) and written, with
    the rotated shared key part behind it, to the key cache as a row and to the value cache as a column; returns
    q [n, heads, rank + rot_dim] with the rotated parts in place at [rank:], the first `rank` features left for
    `head_product` to fill.  `interleaved`: of the rotated features 2i turns with 2i + 1 (else i with i + rotated / 2).
    `q_rows` [n, ...]: the queries' rows where they are no part of `proj` (a product of their own), q at `q_off` there."""
    _dev(proj, norm_weight, cos, sin, k_cache, v_cache, slots, q_rows)
    _f32(norm_weight, "norm weight"); _f32(cos, "cos"); _f32(sin, "sin")
    n, ld = proj.shape
    if q_rows is not None and (q_rows.dim() != 2 or q_rows.shape[0] != n or q_rows.dtype != proj.dtype or q_rows.stride(1) != 1):
        raise KernelError(f"latent_prep: the queries' rows {tuple(q_rows.shape)} {q_rows.dtype} do not fit {n} rows of {proj.dtype}")
    D = rank + rot_dim
    if norm_weight.numel() != rank:
        raise KernelError(f"latent_prep: the norm weight has {norm_weight.numel()} entries, the rank is {rank}")
    if rotated:
        if cos is None or sin is None or tuple(cos.shape) != (n, rotated // 2) or cos.shape != sin.shape:
            raise KernelError(f"latent_prep: rotary tables must be [{n}, {rotated // 2}]")
    if slots is not None:
        _i32(slots, "slots")
        if k_cache is None or v_cache is None or slots.numel() != n:
            raise KernelError("latent_prep: slots need a cache and one entry a token")
        if (tuple(k_cache.shape[1:]) != (1, page_size, D) or tuple(v_cache.shape[1:]) != (1, D, page_size)
                or k_cache.dtype != proj.dtype or v_cache.dtype != proj.dtype):
            raise KernelError(f"latent_prep: cache shapes {tuple(k_cache.shape)} / {tuple(v_cache.shape)} do not fit "
                              f"[pages, 1, {page_size}, {D}] / [pages, 1, {D}, {page_size}] {proj.dtype}")
    q = torch.empty((n, heads, D), dtype=proj.dtype, device=proj.device)
    _check(library().ia_latent_prep(
        _p(q), _p(k_cache if slots is not None else None), _p(v_cache if slots is not None else None), _p(proj),
        _p(norm_weight), _p(cos), _p(sin), _p(slots), n, heads, dim, rot_dim, rank, rotated, q_off, down_off, ld,
        page_size, ctypes.c_float(eps), ctypes.c_float(magnitude), int(bool(interleaved)), _p(q_rows),
        q_rows.stride(0) if q_rows is not None else 0, _dt(proj), _stream()))
    return q


def norm_slice(x: torch.Tensor, x_off: int, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """The RMS norm (32-bit statistics) of the columns x_off .. x_off + len(weight) of 2-D rows, as rows of their own."""
    _dev(x, weight); _f32(weight, "norm weight")
    cols = weight.numel()
    if x.dim() != 2 or x.stride(1) != 1 or x_off < 0 or x_off + cols > x.shape[1]:
        raise KernelError(f"norm_slice: {cols} columns at {x_off} do not fit rows {tuple(x.shape)}")
    out = torch.empty((x.shape[0], cols), dtype=x.dtype, device=x.device)
    _check(library().ia_norm_slice(_p(out), _p(x), x.stride(0), x_off, _p(weight), ctypes.c_float(eps), x.shape[0], cols, _dt(x),
                                   _stream()))
    return out


def head_product(x: torch.Tensor, w: torch.Tensor, *, x_off: int = 0, x_head: Optional[int] = None,
                 out: Optional[torch.Tensor] = None, o_off: int = 0, o_head: Optional[int] = None,
                 out_dtype: Optional[torch.dtype] = None, gate: Optional[torch.Tensor] = None,
                 g_off: int = 0, gate_per_head: bool = False) -> torch.Tensor:
    """A product with a matrix of its own for every head: w [H, n_out, k_in]; x is 2-D, head h of row t starts at
    x[t, x_off + h * x_head] (x_head default k_in); the result goes to out[t, o_off + h * o_head ...] (a new
    [n, H * n_out] tensor by default).  `gate` (2-D, head h at g_off + h * n_out): times its sigmoid; `gate_per_head`: one
    gate value a head, head h's at g_off + h."""
    _dev(x, w, out, gate)
    H, n_out, k_in = w.shape
    n, x_ld = x.shape
    x_head = k_in if x_head is None else x_head
    o_head = n_out if o_head is None else o_head
    if out is None:
        out = torch.empty((n, H * n_out), dtype=out_dtype or x.dtype, device=x.device)
    if out.dim() != 2 or out.shape[0] != n:
        raise KernelError(f"head_product: out {tuple(out.shape)} does not fit {n} rows")
    if gate is not None and (gate.dim() != 2 or gate.shape[0] != n or gate.dtype != x.dtype):
        raise KernelError("head_product: the gate must be 2-D rows of x's precision")
    _check(library().ia_head_product(
        _p(out), _p(x), _p(w), _p(gate), n, H, n_out, k_in, x_ld, x_off, x_head, out.shape[1], o_off, o_head,
        gate.shape[1] if gate is not None else 0, g_off, int(bool(gate_per_head)), _dt(x), _dt(w), _dt(out), _stream()))
    return out


# ---- gated linear recurrence ------------------------------------------------------------------

def conv_step(x: torch.Tensor, x_off: int, width: int, taps: torch.Tensor, bias: Optional[torch.Tensor],
              state: torch.Tensor, token_seq: torch.Tensor, cu_tokens: torch.Tensor,
              state_slots: torch.Tensor, rounded: bool = False):
    """The causal convolution a channel over the step's tokens: x[:, x_off : x_off + width] -> 32-bit u
    [n, width]; `taps` [k, width] (tap by tap, the last meets the current token); inputs before a request's portion
    come from rows 1.. of its state row ([slots, k, width]).
    `rounded`: returns (u, its bfloat16 copy)."""
    _dev(x, taps, bias, state, token_seq, cu_tokens, state_slots); _f32(state, "state")
    _i32(token_seq, "token_seq"); _i32(cu_tokens, "cu_tokens"); _i32(state_slots, "state_slots")
    n, k = x.shape[0], taps.shape[0]
    if (tuple(taps.shape) != (k, width) or taps.dtype != x.dtype or state.dim() != 3
            or tuple(state.shape[1:]) != (k, width) or (bias is not None and (bias.numel() != width or bias.dtype != x.dtype))):
        raise KernelError(f"conv_step: taps {tuple(taps.shape)} / state {tuple(state.shape)} do not fit width {width}")
    u = torch.empty((n, width), dtype=torch.float32, device=x.device)
    lo = torch.empty((n, width), dtype=torch.bfloat16, device=x.device) if rounded else None
    _check(library().ia_conv_step(_p(u), _p(lo), _p(x), _p(taps), _p(bias), _p(state), _p(token_seq), _p(cu_tokens),
                                  _p(state_slots), n, width, k, x.shape[1], x_off, _dt(x), _stream()))
    return (u, lo) if rounded else u


def rglru_scan(u: torch.Tensor, z: torch.Tensor, proj: torch.Tensor, *, branch_off: int, x_off: int,
               bias_r: torch.Tensor, bias_i: torch.Tensor, lam: torch.Tensor, state: torch.Tensor,
               cu_tokens: torch.Tensor, state_slots: torch.Tensor, block_width: int, decay: float,
               chunked: bool = False) -> torch.Tensor:
    """The recurrence over each request's tokens, from and into its state row; returns S_t * gelu_tanh(branch_t)
    in the precision of `proj` ([n, ...]: the gelu branch at `branch_off`, the convolution's input at `x_off`).
    z [n, 2 * width]: the gates' products before bias and sigmoid, block by block [recurrence gate | input gate].
    `chunked`: chunks of 64 tokens side by side and a short walk over the chunks (steps with long portions; the
    result differs from the token-by-token walk by rounding only)."""
    _dev(u, z, proj, bias_r, bias_i, lam, state, cu_tokens, state_slots)
    _f32(u, "u"); _f32(z, "z"); _f32(state, "state"); _i32(cu_tokens, "cu_tokens"); _i32(state_slots, "state_slots")
    n, width = u.shape
    k = state.shape[1]
    if tuple(z.shape) != (n, 2 * width) or proj.shape[0] != n or tuple(state.shape[1:]) != (k, width):
        raise KernelError("rglru_scan: u, z, the projections and the state do not fit each other")
    for t in (bias_r, bias_i, lam):
        if t.numel() != width or t.dtype != proj.dtype:
            raise KernelError("rglru_scan: biases and decay parameters are one entry a channel in the projections' precision")
    n_seqs = state_slots.numel()
    out = torch.empty((n, width), dtype=proj.dtype, device=proj.device)
    if chunked:
        lib = library()
        work = torch.empty((lib.ia_rglru_chunked_workspace(n, n_seqs, width),), dtype=torch.float32, device=proj.device)
        _check(lib.ia_rglru_scan_chunked(
            _p(out), _p(state), _p(work), _p(u), _p(z), _p(bias_r), _p(bias_i), _p(lam), _p(proj), _p(proj), _p(cu_tokens),
            _p(state_slots), n, n_seqs, width, block_width, k, ctypes.c_float(decay), proj.shape[1], branch_off,
            proj.shape[1], x_off, _dt(proj), _stream()))
        return out
    _check(library().ia_rglru_scan(
        _p(out), _p(state), _p(u), _p(z), _p(bias_r), _p(bias_i), _p(lam), _p(proj), _p(proj), _p(cu_tokens),
        _p(state_slots), n_seqs, width, block_width, k, ctypes.c_float(decay), proj.shape[1], branch_off,
        proj.shape[1], x_off, _dt(proj), _stream()))
    return out


# ---- routed experts -----------------------------------------------------------------------------

def route(h: torch.Tensor, router: torch.Tensor, top: int, scale: float, score: str = "sigmoid",
          renormalize: bool = False, choice_bias: Optional[torch.Tensor] = None, gates: int = 0):
    """Router logits in 32-bit (router [E, width] in the precision of h; every logit is a sum of 32-bit
    multiply-adds in an order that the width alone decides), the `top` experts by score for every row:
    (experts int32 [n, top] best first, weights float32 [n, top] = score * scale).  `choice_bias` [E] (32-bit):
    the choice goes by score + bias, the weights stay the scores.  `gates`: the last `gates` rows of `router` are no
    experts: they take no part in the choice, and the sigmoids of their logits (formed like the others, in 32-bit) come
    back as a third result, float32 [n, gates]."""
    _dev(h, router, choice_bias); _f32(choice_bias, "choice_bias")
    n, W = h.shape
    E = router.shape[0] - gates
    if gates < 0 or E < 1:
        raise KernelError(f"route: {gates} gate rows in a router of {router.shape[0]} rows")
    if choice_bias is not None and choice_bias.numel() != E:
        raise KernelError(f"route: {choice_bias.numel()} biases for {E} outputs of the router")
    if (router.shape[1] != W or router.dtype != h.dtype or not (1 <= top <= min(E, MAX_TOP)) or E + gates > MAX_EXPERTS
            or score not in SCORE_FUNCTIONS):
        raise KernelError(f"route: router {tuple(router.shape)} {router.dtype}, top {top}, score {score!r} (up to {MAX_EXPERTS} "
                          f"experts, top up to {MAX_TOP}, scores {sorted(SCORE_FUNCTIONS)})")
    sel = torch.empty((n, top), dtype=torch.int32, device=h.device)
    weight = torch.empty((n, top), dtype=torch.float32, device=h.device)
    gate_out = torch.empty((n, gates), dtype=torch.float32, device=h.device) if gates else None
    _check(library().ia_route(_p(sel), _p(weight), _p(h), _p(router), n, W, E, top, ctypes.c_float(scale),
                              SCORE_FUNCTIONS[score], int(renormalize), _p(choice_bias), gates, _p(gate_out), _dt(h), _stream()))
    return (sel, weight, gate_out) if gates else (sel, weight)


def tile_weights(w: torch.Tensor) -> torch.Tensor:
    """[..., features, k] -> [..., ceil(features / 64), ceil(k / 64), 64, 64], zero-padded: the layout that the routed
    experts' matrix-core products read (a tile of 64 features x 64 k values is 8 KB in one piece)."""
    *lead, f, k = w.shape
    fb, kc = -(-f // 64), -(-k // 64)
    padded = torch.zeros((*lead, fb * 64, kc * 64), dtype=w.dtype, device=w.device)
    padded[..., :f, :k] = w
    return padded.view(*lead, fb, 64, kc, 64).transpose(-3, -2).contiguous()


def experts_tiled_fits(dtype: torch.dtype, width: int, ff: int) -> bool:
    """Whether the routed experts run on the matrix cores over tiled weights."""
    return dtype == torch.bfloat16 and width % 8 == 0 and ff % 8 == 0


def experts_forward(h: torch.Tensor, sel: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor,
                    limit: float, alpha: float, ff: Optional[int] = None, in_weight: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The chosen experts of every row: w_gate_up [E, 2 ff, width] (gate rows, then up rows), w_down [E, width, ff],
    or both as tiles (`tile_weights` of [E, 2, ff, width] and of [E, width, ff]; then `ff` is given);
    act = g' * sigmoid(alpha g') * (u' + 1) with g' = min(g, limit), u' = clamp(u, -limit, limit).  Returns one
    32-bit output row a (row, k) pair, [n, top, width]; nothing is added up here.  A choice of E or beyond names no
    expert with weights: its row is left unwritten (whoever adds the rows up knows what stands for it).  `in_weight`
    [n, top] (32-bit): pair (row, k) runs its expert on in_weight[row, k] * h[row] (the factor meets the two products'
    32-bit sums ahead of the limits, which is the same number)."""
    _dev(h, sel, w_gate_up, w_down, in_weight); _i32(sel, "sel"); _f32(in_weight, "in_weight")
    if in_weight is not None and (tuple(in_weight.shape) != tuple(sel.shape) or not in_weight.is_contiguous()):
        raise KernelError(f"experts: input weights {tuple(in_weight.shape)} for choices {tuple(sel.shape)}")
    n, W = h.shape
    top = sel.shape[1]
    tiled = w_gate_up.dim() == 6
    E = w_gate_up.shape[0]
    if tiled:
        if (ff is None or not experts_tiled_fits(h.dtype, W, ff) or w_gate_up.dtype != h.dtype or w_down.dtype != h.dtype
                or tuple(w_gate_up.shape) != (E, 2, -(-ff // 64), -(-W // 64), 64, 64)
                or tuple(w_down.shape) != (E, -(-W // 64), -(-ff // 64), 64, 64)):
            raise KernelError(f"experts: tiled weights {tuple(w_gate_up.shape)} / {tuple(w_down.shape)} do not fit rows "
                              f"{tuple(h.shape)} {h.dtype} and {ff} features an expert")
    else:
        ff2, W2 = w_gate_up.shape[1:]
        ff = ff2 // 2
        if (W2 != W or ff2 != 2 * ff or tuple(w_down.shape) != (E, W, ff) or w_gate_up.dtype != h.dtype
                or w_down.dtype != h.dtype):
            raise KernelError(f"experts: weights {tuple(w_gate_up.shape)} / {tuple(w_down.shape)} do not fit rows {tuple(h.shape)}")
    if sel.shape[0] != n or E > MAX_EXPERTS:
        raise KernelError(f"experts: {tuple(sel.shape)} choices for {n} rows, {E} experts")
    pairs = n * top
    tiles = -(-pairs // ROW_TILE) + min(E, pairs)
    # many rows an expert: the matrix cores' large tiles (64 rows x 128 features)
    tile = LARGE_TILE if tiled and pairs >= LARGE_TILE_FROM * LARGE_TILE * E else ROW_TILE
    lib = library()
    plan = torch.empty((pairs + 3 * tiles + 1,), dtype=torch.int32, device=h.device)
    order, t_exp, t_first, t_rows, meta = (plan[:pairs], plan[pairs:pairs + tiles], plan[pairs + tiles:pairs + 2 * tiles],
                                           plan[pairs + 2 * tiles:pairs + 3 * tiles], plan[pairs + 3 * tiles:])
    _check(lib.ia_route_plan(_p(order), _p(t_exp), _p(t_first), _p(t_rows), _p(meta), _p(sel), pairs, E, tile, _stream()))
    act = torch.empty((pairs, ff), dtype=h.dtype, device=h.device)
    _check(lib.ia_experts_gate_up(_p(act), _p(h), _p(w_gate_up), _p(order), _p(t_exp), _p(t_first), _p(t_rows), _p(meta),
                                  pairs, E, top, W, ff, ctypes.c_float(limit), ctypes.c_float(alpha), tile, int(tiled),
                                  _p(in_weight), _dt(h), _stream()))
    y = torch.empty((n, top, W), dtype=torch.float32, device=h.device)
    _check(lib.ia_experts_down(_p(y), _p(act), _p(w_down), _p(order), _p(t_exp), _p(t_first), _p(t_rows), _p(meta), pairs,
                               E, W, ff, tile, int(tiled), _dt(h), _stream()))
    return y


# ---- a stream that is normed after every sum ------------------------------------------------------------------------

def postnorm_step(x: torch.Tensor, *, alpha: float = 1.0, y: Optional[torch.Tensor] = None, y2: Optional[torch.Tensor] = None,
                  routed: Optional[torch.Tensor] = None, routed_weights: Optional[torch.Tensor] = None,
                  sel: Optional[torch.Tensor] = None, real_experts: int = 0, weight: torch.Tensor, eps: float,
                  h_dtype: Optional[torch.dtype] = None, rows: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """What stands behind a sub-layer around a 32-bit stream x [n, width] that is normed after every sum (changed in place):

        x <- rmsnorm(alpha x + y + sum_k routed_weights[:, k] * routed[:, k] + y2) * weight

    and, with `h_dtype`, the new rows once more in that precision.  Every addend may be absent.  y and y2 may each be a
    product that is still split along its k (`Partials`, 32-bit [splits, n, width]): the kernel adds the splits up in
    their order, nothing is rounded in between.  `routed` [n, top, width]
    (32-bit): with `sel` [n, top], a pair whose entry is `real_experts` or more stands for the stream's own row (an expert
    that hands its input on).  `rows` (int32): only these rows are read, the stream is left as it is and the result has one
    row for each of them."""
    from . import Partials
    both = [t for t in (y, y2) if t is not None]
    if any(isinstance(t, Partials) for t in both) and any(not isinstance(t, Partials) and t.dtype != torch.float32 for t in both):
        y, y2 = (t.materialize() if isinstance(t, Partials) else t for t in (y, y2))    # (one precision for both)
    y_splits = y2_splits = 1
    if isinstance(y, Partials):
        y_splits, y = y.parts.shape[0], y.parts
    if isinstance(y2, Partials):
        y2_splits, y2 = y2.parts.shape[0], y2.parts
    _dev(x, y, y2, routed, routed_weights, sel, weight, rows)
    _f32(x, "the stream"); _f32(routed, "routed rows"); _f32(routed_weights, "routed weights"); _f32(weight, "norm weight")
    n, W = x.shape
    given = [t for t in (y, y2) if t is not None]
    for t, splits in ((y, y_splits), (y2, y2_splits)):
        if t is None:
            continue
        if (tuple(t.shape[-2:]) != (n, W) or t.dtype != given[0].dtype or not t.is_contiguous()
                or (t.dim() == 3 and (t.shape[0] != splits or t.dtype != torch.float32)) or t.dim() not in (2, 3)):
            raise KernelError(f"postnorm_step: an output {tuple(t.shape)} {t.dtype} does not fit the stream [{n}, {W}]")
    top = 0
    if routed is not None:
        top = routed.shape[1]
        if (routed.dim() != 3 or tuple(routed.shape) != (n, top, W) or routed_weights is None
                or tuple(routed_weights.shape) != (n, top) or top > MAX_TOP):
            raise KernelError(f"postnorm_step: routed rows {tuple(routed.shape)} and their weights do not fit [{n}, top <= {MAX_TOP}, {W}]")
        if sel is not None:
            _i32(sel, "sel")
            if tuple(sel.shape) != (n, top):
                raise KernelError(f"postnorm_step: choices {tuple(sel.shape)} do not fit [{n}, {top}]")
    if weight.numel() != W:
        raise KernelError(f"postnorm_step: the norm weight has {weight.numel()} entries, the stream is {W} wide")
    count = n
    if rows is not None:
        _i32(rows, "rows")
        count = rows.numel()
        if h_dtype is None or given or routed is not None:
            raise KernelError("postnorm_step: a row list goes with an output and nothing to add")
    h = torch.empty((count, W), dtype=h_dtype, device=x.device) if h_dtype is not None else None
    _check(library().ia_postnorm_step(
        _p(x), ctypes.c_float(alpha), _p(y), _p(y2), y_splits, y2_splits, _p(routed), _p(routed_weights), _p(sel), top,
        int(real_experts),
        _p(weight), ctypes.c_float(eps), _p(h), _p(rows), count, W, _dt(given[0]) if given else 0,
        _DT[h_dtype] if h_dtype is not None else 0, _stream()))
    return h


def embed_gather_scaled(table: torch.Tensor, ids: torch.Tensor, scale: float, rounded: bool = False):
    """table[ids] * scale as 32-bit rows; `rounded`: (rows, the same rows in the table's precision)."""
    _dev(table, ids); _i32(ids, "token ids")
    n, (vocab, hidden) = ids.numel(), table.shape
    out = torch.empty((n, hidden), dtype=torch.float32, device=table.device)
    lo = torch.empty((n, hidden), dtype=table.dtype, device=table.device) if rounded else None
    _check(library().ia_embed_gather_scaled(_p(out), _p(lo), _p(table), _p(ids), n, hidden, vocab, ctypes.c_float(scale),
                                            _dt(table), _stream()))
    return (out, lo) if rounded else out


def sigmoid_gate(a: torch.Tensor, g: torch.Tensor, g_off: int = 0, group: int = 1) -> torch.Tensor:
    """a[:, c] *= sigmoid(g[:, g_off + c // group]) in place; a [n, cols] contiguous, g 2-D rows of the same precision.
    `group`: neighbouring columns that share one gate value (a head's width: one value a head)."""
    _dev(a, g)
    n, cols = a.shape
    if (g.dim() != 2 or g.shape[0] != n or g.dtype != a.dtype or g_off < 0 or group < 1 or cols % group
            or g_off + cols // group > g.shape[1] or not a.is_contiguous()):
        raise KernelError(f"sigmoid_gate: a gate {tuple(g.shape)} {g.dtype} at {g_off} does not fit rows {tuple(a.shape)} {a.dtype}")
    _check(library().ia_sigmoid_gate(_p(a), _p(g), n, cols, g.stride(0), g_off, group, _dt(a), _stream()))
    return a


def clamped_gate_mul(gu: torch.Tensor, limit: float, slope: float) -> torch.Tensor:
    """Rows of [gate | up] -> g' * sigmoid(slope g') * (u' + 1) with g' = min(gate, limit), u' = clamp(up, -limit, limit)."""
    _dev(gu)
    n, two = gu.shape
    if two % 2 or not gu.is_contiguous():
        raise KernelError(f"clamped_gate_mul: rows {tuple(gu.shape)} are no [gate | up]")
    out = torch.empty((n, two // 2), dtype=gu.dtype, device=gu.device)
    _check(library().ia_clamped_gate_mul(_p(out), _p(gu), n, two // 2, ctypes.c_float(limit), ctypes.c_float(slope), _dt(gu),
                                         _stream()))
    return out


def scale_inplace(x: torch.Tensor, factor: float) -> torch.Tensor:
    """x *= factor (32-bit values)."""
    _dev(x); _f32(x, "x")
    _check(library().ia_scale(_p(x), ctypes.c_longlong(x.numel()), ctypes.c_float(factor), _stream()))
    return x


# ---- a stream whose sub-layers read one normed copy ---------------------------------------------------------------------

def parallel_step(x: torch.Tensor, *, y1=None, y2=None, y3=None, y3_scale: Optional[torch.Tensor] = None,
                  routed: Optional[torch.Tensor] = None, routed_weights: Optional[torch.Tensor] = None,
                  enter: Optional[torch.Tensor] = None, enter_weight: Optional[torch.Tensor] = None, enter_eps: float = 0.0,
                  x_dtype: Optional[torch.dtype] = None, norm_weight: Optional[torch.Tensor] = None,
                  norm_bias: Optional[torch.Tensor] = None, norm_eps: float = 0.0, center: bool = True,
                  h_dtype: Optional[torch.dtype] = None, rows: Optional[torch.Tensor] = None):
    """What stands between two layers around a 32-bit stream x [n, width] (changed in place) whose sub-layers all read
    one normed copy of it:

        x <- x + y1 + y2 + sum_k [routed_weights[:, k]] routed[:, k] + y3_scale[:, None] * y3
        x <- x + rmsnorm(enter) * enter_weight                       (`enter_eps` inside the root)
        h  = (x - mean) / sqrt(var + norm_eps) * norm_weight + norm_bias   (`center` False: an RMS norm; the bias may be None)

    Every line and every addend may be absent.  y1, y2, y3 may each be a product still split along its k (`Partials`).
    Returns (the new x once more in `x_dtype` or None, h in `h_dtype` or None).  `rows` (int32): only these rows go
    through the norm; nothing is added and the stream is left as it is."""
    from . import Partials
    ys = [y1, y2, y3]
    dense = [t for t in ys + [enter] if t is not None]
    if any(isinstance(t, Partials) for t in dense) and any(not isinstance(t, Partials) and t.dtype != torch.float32 for t in dense):
        ys = [t.materialize() if isinstance(t, Partials) else t for t in ys]       # (one precision for all)
    splits = [1, 1, 1]
    for i, t in enumerate(ys):
        if isinstance(t, Partials):
            splits[i], ys[i] = t.parts.shape[0], t.parts
    y1, y2, y3 = ys
    _dev(x, y1, y2, y3, y3_scale, routed, routed_weights, enter, enter_weight, norm_weight, norm_bias, rows)
    for t, name in ((x, "the stream"), (y3_scale, "y3_scale"), (routed, "routed rows"), (routed_weights, "routed weights"),
                    (enter_weight, "enter_weight"), (norm_weight, "norm weight"), (norm_bias, "norm bias")):
        _f32(t, name)
    n, W = x.shape
    given = [t for t in (y1, y2, y3, enter) if t is not None]
    for t, sp in ((y1, splits[0]), (y2, splits[1]), (y3, splits[2]), (enter, 1)):
        if t is None:
            continue
        if (tuple(t.shape[-2:]) != (n, W) or t.dtype != given[0].dtype or not t.is_contiguous() or t.dim() not in (2, 3)
                or (t.dim() == 3 and (t.shape[0] != sp or t.dtype != torch.float32))):
            raise KernelError(f"parallel_step: an output {tuple(t.shape)} {t.dtype} does not fit the stream [{n}, {W}]")
    top = 0
    if routed is not None:
        top = routed.shape[1]
        if (routed.dim() != 3 or tuple(routed.shape) != (n, top, W) or top > MAX_TOP or not routed.is_contiguous()
                or (routed_weights is not None and tuple(routed_weights.shape) != (n, top))):
            raise KernelError(f"parallel_step: routed rows {tuple(routed.shape)} do not fit [{n}, top <= {MAX_TOP}, {W}]")
    if y3_scale is not None and (y3 is None or y3_scale.numel() != n):
        raise KernelError("parallel_step: a factor a row goes with y3 and has one entry a row")
    if enter is not None and (enter_weight is None or enter_weight.numel() != W):
        raise KernelError("parallel_step: a row that enters comes with its norm's weight")
    for t in (norm_weight, norm_bias):
        if t is not None and t.numel() != W:
            raise KernelError(f"parallel_step: the norm has {t.numel()} entries, the stream is {W} wide")
    if h_dtype is not None and norm_weight is None:
        raise KernelError("parallel_step: normed rows come with the norm's weight")
    count = n
    if rows is not None:
        _i32(rows, "rows")
        count = rows.numel()
        if h_dtype is None or given or routed is not None or x_dtype is not None:
            raise KernelError("parallel_step: a row list goes with normed rows out and nothing to add")
    out_dtype = h_dtype if h_dtype is not None else x_dtype
    if h_dtype is not None and x_dtype is not None and h_dtype != x_dtype:
        raise KernelError("parallel_step: one precision for both outputs")
    xr = torch.empty((n, W), dtype=x_dtype, device=x.device) if x_dtype is not None else None
    h = torch.empty((count, W), dtype=h_dtype, device=x.device) if h_dtype is not None else None
    _check(library().ia_parallel_step(
        _p(x), _p(y1), _p(y2), _p(y3), splits[0], splits[1], splits[2], _p(y3_scale), _p(routed), _p(routed_weights), top,
        _p(enter), _p(enter_weight), ctypes.c_float(enter_eps), _p(xr), _p(norm_weight), _p(norm_bias),
        ctypes.c_float(norm_eps), int(bool(center)), _p(h), _p(rows), count, W, _dt(given[0]) if given else 0,
        _DT[out_dtype] if out_dtype is not None else 0, _stream()))
    return xr, h


def gate_rows(g: torch.Tensor, e: torch.Tensor, e_off: int, activation: str = "gelu_tanh") -> torch.Tensor:
    """act(g) * e[:, e_off : e_off + cols] for rows g [n, cols] (contiguous) and wider rows e of the same precision."""
    from . import activation_code
    _dev(g, e)
    n, cols = g.shape
    if (e.dim() != 2 or e.shape[0] != n or e.dtype != g.dtype or e_off < 0 or e_off + cols > e.shape[1] or e.stride(1) != 1
            or not g.is_contiguous()):
        raise KernelError(f"gate_rows: rows {tuple(e.shape)} {e.dtype} at {e_off} do not fit gates {tuple(g.shape)} {g.dtype}")
    out = torch.empty_like(g)
    _check(library().ia_gate_rows(_p(out), _p(g), _p(e), n, cols, e.stride(0), e_off, activation_code(activation), _dt(g),
                                  _stream()))
    return out
