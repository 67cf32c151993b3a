"""Ligizen on the GPU against the plain implementation (`plain_ligizen.py`, 64-bit).

Mechanisms alone, through the kernels' Python face: the kernel between two layers of a stream whose sub-layers read one
normed copy (every addend, routed rows with and without weights, a gated second output, products still split along their
k, the row that enters through its norm, the layer norm and the RMS norm at its end, the model's end), the small kernels
(a gate a head, the gated slice of a token's row), the latent attention's preparation with neighbours paired and queries
from a product of their own, the paged attention under a mask of chunks and with a learned term a head in the
denominator in every kernel that takes them (plain and matrix cores, keys split and not, prompts and single tokens) with
a key that stands out just inside an edge and a stronger one just outside it, the router with a gate row behind its
experts, the experts with the weight on their input.  Then whole models through the engine's step function under every
way of cutting the work (whole prompts, a prompt and then token by token, every token alone, portions down to two tokens,
up to four live requests mixed in a pool whose pages and slots are used again), in both precisions, with ordinary
weights and with sharpened queries.  Greedy generation runs through the engine's own entry point and scheduler, the
command line and the replay program.

Tolerances.  32-bit: 2e-5 of the largest logit against the 64-bit result, at every position; where the plain
implementation's own 32-bit arithmetic is further off than a third of that, three times what it is off.  bfloat16:
the measure is the distribution of the positions' errors against that of the plain implementation in bfloat16 arithmetic
(every operation rounded) on the same positions: the engine keeps more in 32-bit than that, so its median and its ninth
decile must not be larger (a tenth and a half of slack)."""
import copy
import io
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_ligizen as pl
import trace_modes as tm
from ligizen_configs import CONFIGS, random_tokens, sharpened, write_model

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = [1, 2, 3, 17, 64, 65, 130, 300, 700]
TOL_F32 = 2e-5
CASES = [("A", 1.0), ("B", 1.0), ("C", 1.0), ("D", 1.0), ("A", 6.0), ("C", 5.0), ("D", 4.0)]


def dev(t, dtype=None):
    return t.to(device="cuda", dtype=dtype or t.dtype).contiguous()


def assert_close(got, want, rel, what):
    err = float((got.double().cpu() - want).abs().max()) / max(float(want.abs().max()), 1e-9)
    assert err <= rel, f"{what}: {err:.3g} of the scale, allowed {rel:.3g}"


# ---- the kernel between two layers ---------------------------------------------------------------------

@pytest.mark.parametrize("W", [40, 33, 300, 5000])
@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
def test_step_between_layers(W, y_dtype):
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(W)
    n, top = 19, 3
    tol = dict(rtol=1e-5, atol=1e-5)
    lo = dict(rtol=1e-2, atol=2e-2) if y_dtype == torch.bfloat16 else tol
    x = torch.randn(n, W, generator=g) * 3 + 0.7
    y1, y2, y3, enter = (torch.randn(n, W, generator=g).to(y_dtype) for _ in range(4))
    routed = torch.randn(n, top, W, generator=g)
    rw, s3 = torch.rand(n, top, generator=g), torch.rand(n, generator=g)
    w, b, we = 1.0 + 0.1 * torch.randn(W, generator=g), 0.3 * torch.randn(W, generator=g), 0.5 + 0.1 * torch.randn(W, generator=g)
    # two dense outputs, then a layer norm of the sum
    xs = dev(x)
    xr, h = ops.parallel_step(xs, y1=dev(y1), y2=dev(y2), norm_weight=dev(w), norm_bias=dev(b), norm_eps=1e-5, h_dtype=y_dtype)
    want = x.double() + y1.double() + y2.double()
    assert xr is None
    np.testing.assert_allclose(xs.cpu().numpy(), want.numpy(), **tol)
    np.testing.assert_allclose(h.float().cpu().numpy(), pl.layer_norm(want, w.double(), b.double(), 1e-5).numpy(), **lo)
    # routed rows as they are, a second output behind a gate a row; the new rows once more in the products' precision
    xs = dev(x)
    xr, h = ops.parallel_step(xs, y1=dev(y1), routed=dev(routed), y3=dev(y3), y3_scale=dev(s3), x_dtype=y_dtype)
    want = x.double() + y1.double() + routed.double().sum(1) + s3.double()[:, None] * y3.double()
    assert h is None
    np.testing.assert_allclose(xs.cpu().numpy(), want.numpy(), **tol)
    np.testing.assert_allclose(xr.float().cpu().numpy(), want.numpy(), **lo)
    # routed rows with weights; an RMS norm at the end, without a bias
    xs = dev(x)
    _, h = ops.parallel_step(xs, routed=dev(routed), routed_weights=dev(rw), norm_weight=dev(w), norm_eps=1e-6, center=False,
                             h_dtype=torch.float32)
    want = x.double() + (rw.double()[:, :, None] * routed.double()).sum(1)
    np.testing.assert_allclose(h.cpu().numpy(), pl.rms_norm(want, w.double(), 1e-6).numpy(), **tol)
    # a row that enters through its norm, then the layer norm
    xs = dev(x)
    _, h = ops.parallel_step(xs, enter=dev(enter), enter_weight=dev(we), enter_eps=1e-5, norm_weight=dev(w), norm_bias=dev(b),
                             norm_eps=1e-5, h_dtype=torch.float32)
    want = x.double() + pl.rms_norm(enter.double(), we.double(), 1e-5)
    np.testing.assert_allclose(xs.cpu().numpy(), want.numpy(), **tol)
    np.testing.assert_allclose(h.cpu().numpy(), pl.layer_norm(want, w.double(), b.double(), 1e-5).numpy(), rtol=1e-4, atol=1e-4)
    # outputs that are products still split along their k: the kernel adds the splits up
    if y_dtype == torch.float32:
        parts, parts3 = (torch.randn(s, n, W, generator=g) for s in (3, 2))
        xs2 = dev(x)
        ops.parallel_step(xs2, y1=ops.Partials(dev(parts)), y3=ops.Partials(dev(parts3)), y3_scale=dev(s3), y2=dev(y2))
        want2 = x.double() + parts.double().sum(0) + y2.double() + s3.double()[:, None] * parts3.double().sum(0)
        np.testing.assert_allclose(xs2.cpu().numpy(), want2.numpy(), **tol)
    # the model's end: some rows through a norm, the stream left as it is; nothing at all: the norm alone
    before = xs.clone()
    pick = torch.tensor([5, 0, 18], dtype=torch.int32)
    _, tail = ops.parallel_step(xs, norm_weight=dev(w), norm_bias=dev(b), norm_eps=1e-6, h_dtype=torch.float32, rows=dev(pick))
    np.testing.assert_allclose(tail.cpu().numpy(), pl.layer_norm(want[pick.long()], w.double(), b.double(), 1e-6).numpy(), rtol=1e-4, atol=1e-4)
    assert torch.equal(xs, before)
    # a row of equal values has no deviations: the bias alone is left
    flat = dev(torch.full((2, W), 3.25))
    _, h = ops.parallel_step(flat, norm_weight=dev(w), norm_bias=dev(b), norm_eps=1e-5, h_dtype=torch.float32)
    np.testing.assert_allclose(h.cpu().numpy(), b.expand(2, W).numpy(), atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_small_kernels(dtype):
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(2)
    tol = dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(rtol=1e-5, atol=1e-6)
    # one gate value a head
    for heads, dv, ld, off in ((3, 8, 80, 40), (5, 3, 30, 17), (1, 16, 16, 15)):
        a, gate = torch.randn(11, heads * dv, generator=g).to(dtype), (3 * torch.randn(11, ld, generator=g)).to(dtype)
        got = ops.sigmoid_gate(dev(a.clone()), dev(gate), off, group=dv)
        want = a.double().view(11, heads, dv) * torch.sigmoid(gate.double()[:, off:off + heads])[:, :, None]
        np.testing.assert_allclose(got.float().cpu().numpy(), want.view(11, -1).numpy(), **tol)
    # the gated slice of a wider row
    for cols, ld, off in ((24, 96, 48), (5, 15, 10), (6, 6, 0)):
        gate, rows = (2 * torch.randn(13, cols, generator=g)).to(dtype), torch.randn(13, ld, generator=g).to(dtype)
        got = ops.gate_rows(dev(gate), dev(rows), off, "gelu_tanh")
        np.testing.assert_allclose(got.float().cpu().numpy(), (pl.gelu_tanh(gate.double()) * rows.double()[:, off:off + cols]).numpy(), **tol)
    # the RMS norm of a slice of wider rows
    for cols, ld, off in ((16, 40, 0), (10, 33, 7), (1024, 1300, 8)):
        rows, w = torch.randn(13, ld, generator=g).to(dtype), 1 + 0.2 * torch.randn(cols, generator=g)
        got = ops.norm_slice(dev(rows), off, dev(w), 1e-5)
        np.testing.assert_allclose(got.float().cpu().numpy(), pl.rms_norm(rows.double()[:, off:off + cols], w.double(), 1e-5).numpy(), **tol)
    # a product a head with one gate value a head behind it
    H, n_out, k_in = 3, 8, 16
    x, w = torch.randn(9, H * k_in, generator=g).to(dtype), (torch.randn(H, n_out, k_in, generator=g) / 4).to(dtype)
    gate = (2 * torch.randn(9, 10, generator=g)).to(dtype)
    got = ops.head_product(dev(x), dev(w), gate=dev(gate), g_off=4, gate_per_head=True)
    want = torch.einsum("thi,hji->thj", x.double().view(9, H, k_in), w.double()) * torch.sigmoid(gate.double()[:, 4:4 + H])[:, :, None]
    np.testing.assert_allclose(got.float().cpu().numpy(), want.reshape(9, -1).numpy(), **tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,d,r,rank,turned", [(4, 8, 4, 12, 4), (2, 16, 8, 24, 8), (3, 10, 6, 14, 4), (8, 32, 32, 96, 32)])
def test_latent_rows_with_neighbours_paired(H, d, r, rank, turned, dtype):
    """The latent row's norm, the turn of the shared key part and of the queries' turned parts (2i with 2i + 1), the cache
    writes; the queries from a product of their own."""
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(H * d + r)
    n, page, pages, D = 21, 8, 6, rank + r
    proj = torch.randn(n, 3 + D + H, generator=g).to(dtype)          # [3 unused | latent row, key part | a gate a head]
    q_rows = torch.randn(n, H * (d + r), generator=g).to(dtype)
    nw = 1 + 0.3 * torch.randn(rank, generator=g)
    positions = torch.randint(0, 500, (n,), generator=g)
    slots = torch.randperm(pages * page, generator=g)[:n].to(torch.int32)
    rot = {"base": 777.0, "dims": turned}
    ang = positions.double()[:, None] * pl.frequencies(rot, torch.float64)[None, :]
    kc, vc = dev(torch.zeros(pages, 1, page, D, dtype=dtype)), dev(torch.zeros(pages, 1, D, page, dtype=dtype))
    q = ops.latent_prep(dev(proj), heads=H, dim=d, rot_dim=r, rank=rank, rotated=turned, q_off=0, down_off=3, norm_weight=dev(nw),
                        eps=1e-5, cos=dev(torch.cos(ang).float()), sin=dev(torch.sin(ang).float()), magnitude=1.0, k_cache=kc,
                        v_cache=vc, slots=dev(slots), page_size=page, interleaved=True, q_rows=dev(q_rows))
    p64 = proj.double()
    want_row = torch.cat([pl.rms_norm(p64[:, 3:3 + rank], nw.double(), 1e-5),
                          pl.turn(p64[:, 3 + rank:3 + D].view(n, 1, r), positions, rot, True)[:, 0]], dim=1)
    want_q = pl.turn(q_rows.double().view(n, H, d + r)[..., d:], positions, rot, True)
    rel = 1e-2 if dtype == torch.bfloat16 else 1e-5
    assert_close(q[..., rank:], want_q, rel, "the queries' turned parts")
    assert_close(kc.cpu()[slots.long() // page, 0, slots.long() % page], want_row, rel, "cached rows")
    assert_close(vc.cpu()[slots.long() // page, 0, :, slots.long() % page], want_row, rel, "cached rows as columns")


# ---- the attention under a mask of chunks, with a learned term in the denominator ---------------------------

def first_seen(pos, window, chunk):
    lo = max(pos - window + 1, 0) if window else 0
    return max(lo, pos - pos % chunk) if chunk else lo


def attention_reference(q, kc, vc, positions, token_seq, table, window, chunk, scale, sinks):
    """Request by request on dense copies of its keys and values."""
    n, nq, d = q.shape
    nkv, page, dv = kc.shape[1], kc.shape[2], vc.shape[2]
    out = torch.zeros(n, nq, dv, dtype=torch.float64)
    for s in token_seq.unique().tolist():
        rows = (token_seq == s).nonzero().flatten()
        pos = positions[rows].long()
        length = int(pos.max()) + 1
        first = first_seen(int(pos.min()), window, chunk)
        pages = table[s, :-(-length // page)].long()
        k = kc[pages].double().permute(1, 0, 2, 3).reshape(nkv, -1, d)[:, :length].repeat_interleave(nq // nkv, 0)
        v = vc[pages].double().permute(1, 0, 3, 2).reshape(nkv, -1, dv)[:, :length].repeat_interleave(nq // nkv, 0)
        k[:, :first], v[:, :first] = 0.0, 0.0            # (what no query of the step sees may hold anything)
        sc = torch.einsum("thd,hjd->thj", q[rows].double(), k) * scale
        j = torch.arange(length)
        lows = torch.tensor([first_seen(int(p), window, chunk) for p in pos])
        seen = (j[None, :] <= pos[:, None]) & (j[None, :] >= lows[:, None])
        for h in range(nq):
            p = pl.softmax_rows(sc[:, h], seen, None if sinks is None else sinks[h].double().expand(len(rows)))
            out[rows, h] = p @ v[h]
    return out


def attention_case(dtype, nq, nkv, d, dv, page, lens, q_lens, window, chunk, seed):
    """Cached requests in shuffled pages; what lies beyond a request's length, and in pages that no query of the step sees,
    is NaN.  For every request's last query, head 0: the first key it sees points along the query, and the key one place
    further back, which it does not see, does so twice as strongly."""
    g = torch.Generator().manual_seed(seed)
    max_pages = max(-(-l // page) for l in lens)
    total = sum(-(-l // page) for l in lens) + 3
    perm = torch.randperm(total, generator=g).tolist()
    table = torch.zeros(len(lens), max_pages, dtype=torch.int32)
    for s, l in enumerate(lens):
        for j in range(-(-l // page)):
            table[s, j] = perm.pop()
    kc = torch.randn(total, nkv, page, d, generator=g).to(dtype)
    vc = torch.randn(total, nkv, dv, page, generator=g).to(dtype)
    positions = torch.tensor([p for l, ql in zip(lens, q_lens) for p in range(l - ql, l)], dtype=torch.int32)
    token_seq = torch.tensor([s for s, ql in enumerate(q_lens) for _ in range(ql)], dtype=torch.int32)
    q = torch.randn(len(positions), nq, d, generator=g).to(dtype)
    for s, (l, ql) in enumerate(zip(lens, q_lens)):
        last = q[token_seq == s][-1, 0].float()
        inside = first_seen(l - 1, window, chunk)
        kc[int(table[s, inside // page]), 0, inside % page] = (last * 3).to(dtype)
        if inside > 0:
            kc[int(table[s, (inside - 1) // page]), 0, (inside - 1) % page] = (last * 6).to(dtype)
        passed = (first_seen(l - ql, window, chunk) // page) * page
        for j in list(range(passed)) + list(range(l, -(-l // page) * page)):
            kc[int(table[s, j // page]), :, j % page] = float("nan")
            vc[int(table[s, j // page]), :, :, j % page] = float("nan")
    return q, kc, vc, positions, token_seq, table


SHAPES = [(4, 2, 16, 8), (5, 5, 12, 20), (4, 1, 128, 64), (2, 2, 64, 64), (8, 1, 128, 128), (3, 1, 48, 48), (4, 1, 160, 160)]
MASKS = [(0, 1), (0, 17), (0, 64), (0, 80), (0, 300), (0, 5000), (24, 0), (200, 0), (50, 64)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,d,dv", SHAPES)
@pytest.mark.parametrize("window,chunk", MASKS)
def test_attention_in_chunks_with_sinks(nq, nkv, d, dv, window, chunk, dtype):
    """Prompts, portions late in a context (one that begins in the middle of a chunk and crosses its end) and single tokens
    (one at a chunk's first place, one at its last) in one step, in every kernel that takes the sizes; with and without a
    learned term a head in the denominator."""
    from inferrs_amd import ops
    page = 16
    first_of_chunk = (chunk * 3 + 1) if 0 < chunk < 300 else 641
    lens, q_lens = [700, 333, 64, first_of_chunk, 1100, max(chunk * 2, 1) if chunk < 600 else 1000], [700, 40, 1, 1, 1, 1]
    g = torch.Generator().manual_seed(nq + chunk)
    q, kc, vc, positions, token_seq, table = attention_case(dtype, nq, nkv, d, dv, page, lens, q_lens, window, chunk,
                                                            seed=d + dv + window + chunk)
    rel = 2e-2 if dtype == torch.bfloat16 else 2e-5
    args = [dev(t) for t in (q, kc, vc, positions, token_seq, table)]
    cu = dev(torch.tensor([0] + list(np.cumsum(q_lens)), dtype=torch.int32))
    single = [s for s, ql in enumerate(q_lens) if ql == 1]
    rows = torch.tensor([int(np.cumsum(q_lens)[s]) - 1 for s in single])
    for sinks in (None, 1.5 * torch.randn(nq, generator=g) + 1.0):
        want = attention_reference(q, kc, vc, positions, token_seq, table, window, chunk, 0.2, sinks)
        kw = dict(window=window or None, mask_chunk=chunk or None, scale=0.2, sinks=None if sinks is None else dev(sinks))
        for split in (None, False):
            got = ops.attention_generic(*args, max_kv_len=max(lens), split=split, **kw)
            assert_close(got, want, rel, f"plain kernel, split {split}, sinks {sinks is not None}")
        if not ops.attention_mfma_fits(dtype, d, page, dv):
            continue
        for splits in (None, 1, 4):
            got = ops.attention_mfma(args[0], args[1], args[2], args[3], cu, args[5], max_q_len=max(q_lens), max_kv_len=max(lens),
                                     splits=splits, **kw)
            assert_close(got, want, rel, f"matrix cores, splits {splits}, sinks {sinks is not None}")
        # single tokens alone (the decode launch)
        got = ops.attention_mfma(dev(q[rows]), args[1], args[2], dev(positions[rows]), dev(torch.arange(len(single) + 1, dtype=torch.int32)),
                                 dev(table[single]), max_q_len=1, max_kv_len=max(lens), **kw)
        assert_close(got, want[rows], rel, f"matrix cores, single tokens, sinks {sinks is not None}")
    # the planted keys are what the test rests on: one place more of sight moves the last query's output
    if chunk and not window and chunk < 600:
        other = attention_reference(q, kc.nan_to_num(), vc.nan_to_num(), positions, token_seq, table, 0, chunk + 1, 0.2, None)
        clean = attention_reference(q, kc.nan_to_num(), vc.nan_to_num(), positions, token_seq, table, 0, chunk, 0.2, None)
        assert float((other - clean)[:, 0].abs().max()) > 0.05


# ---- the router with a gate row, the experts with the weight on their input --------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,top,W", [(5, 2, 48), (2, 2, 64), (3, 3, 50), (70, 6, 136), (4, 1, 40), (10, 1, 384)])
def test_router_with_a_gate_row(E, top, W, dtype):
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(E * W)
    for n in (1, 57, 200):
        h = torch.randn(n, W, generator=g).to(dtype)
        router = (2 * torch.randn(E + 1, W, generator=g) / W ** 0.5).to(dtype)
        router[E] *= 50.0                                      # (a gate row that would win every choice if it took part)
        sel, weight, gate = ops.route(dev(h), dev(router), top, 1.0, "sigmoid", False, None, gates=1)
        z = h.double() @ router.double().T
        s = torch.sigmoid(z[:, :E])
        order = torch.argsort(s, dim=-1, descending=True)
        ranked = torch.gather(s, 1, order)
        clear = ((ranked[:, :-1] - ranked[:, 1:])[:, :top].abs().min(dim=1).values > 1e-5) if E > 1 else torch.ones(n, dtype=torch.bool)
        assert clear.float().mean() > 0.8 and int(sel.max()) < E
        assert torch.equal(sel.cpu().long()[clear], order[clear, :top])
        np.testing.assert_allclose(weight.cpu()[clear].numpy(), ranked[:, :top][clear].numpy(), rtol=1e-4, atol=1e-6)
        np.testing.assert_allclose(gate.cpu().numpy()[:, 0], torch.sigmoid(z[:, E]).numpy(), rtol=1e-4, atol=1e-6)
        # the same choice and weights as without the row
        sel2, weight2 = ops.route(dev(h), dev(router[:E]), top, 1.0, "sigmoid", False, None)
        assert torch.equal(sel2, sel) and torch.equal(weight2, weight)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,top,W,ff", [(5, 2, 48, 24), (3, 3, 50, 30), (6, 2, 64, 32), (10, 1, 384, 48)])
def test_experts_with_the_weight_on_their_input(E, top, W, ff, dtype):
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(E + ff)
    for n in (1, 9, 150):
        h = (1.5 * torch.randn(n, W, generator=g)).to(dtype)
        sel = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(n)]).to(torch.int32)
        weight = torch.rand(n, top, generator=g)
        gu = (1.5 * torch.randn(E, 2 * ff, W, generator=g) / W ** 0.5).to(dtype)
        down = (torch.randn(E, W, ff, generator=g) / ff ** 0.5).to(dtype)
        tiled = ops.mix.experts_tiled_fits(dtype, W, ff)
        a, b = dev(gu), dev(down)
        if tiled:
            a, b = ops.mix.tile_weights(a.view(E, 2, ff, W)), ops.mix.tile_weights(b)
        y = ops.experts_forward(dev(h), dev(sel), a, b, 1.2, 1.702, ff=ff if tiled else None, in_weight=dev(weight)).cpu()
        apart = 0.0
        for t in range(n):
            for k in range(top):
                e = int(sel[t, k])
                w = {"gate": gu[e, :ff].double(), "up": gu[e, ff:].double(), "down": down[e].double()}
                want = pl.clamped_expert(weight[t, k].double() * h[t:t + 1].double(), w, "", 1.2)[0]
                assert_close(y[t, k], want, 2e-2 if dtype == torch.bfloat16 else 2e-5, f"n={n} pair ({t}, {k})")
                behind = weight[t, k].double() * pl.clamped_expert(h[t:t + 1].double(), w, "", 1.2)[0]
                apart = max(apart, float((want - behind).abs().max()) / float(want.abs().max()))
        assert apart > 0.05                                    # (the limits bite: a weight behind the expert is another number)


# ---- whole models under every cutting ---------------------------------------------------------------

_ROUNDED = {}
NOISE = {}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, sharpen in CASES:
        cfg = sharpened(CONFIGS[name], sharpen)
        folder = str(tmp_path_factory.mktemp(f"ligizen_{name}"))
        tensors = write_model(folder, cfg, seed=11)
        reqs = {f"r{i}": random_tokens(n, cfg["vocab"], 40 + i) for i, n in enumerate(LENGTHS)}
        ref64 = {r: pl.forward(cfg, tensors, t) for r, t in reqs.items()}
        ref = {r: v.numpy().astype(np.float32) for r, v in ref64.items()}
        scale = max(float(v.abs().max()) for v in ref64.values())
        # what rounding alone does at every position: the plain implementation in 32-bit against itself in 64-bit
        NOISE[(name, sharpen)] = {r: ((pl.forward(cfg, tensors, t, dtype=torch.float32).double() - ref64[r]).abs().max(1).values
                                      / scale).numpy() for r, t in reqs.items()}
        out[(name, sharpen)] = (folder, cfg, tensors, reqs, ref)
    return out


def errors(got, ref, reqs):
    scale = max(float(np.abs(v).max()) for v in ref.values())
    return {r: np.array([float(np.abs(got[r][p] - ref[r][p]).max()) / scale for p in range(len(t))]) for r, t in reqs.items()}


def rounded_errors(key, models):
    """request -> the errors of the plain implementation in bfloat16 arithmetic, position by position."""
    if key not in _ROUNDED:
        folder, cfg, tensors, reqs, ref = models[key]
        some = {r: t for r, t in reqs.items() if len(t) <= 300}
        rounded = {r: pl.forward(cfg, tensors, t, dtype=torch.bfloat16).float().numpy() for r, t in some.items()}
        _ROUNDED[key] = errors(rounded, ref, some)
    return _ROUNDED[key]


def worst(got, ref, reqs):
    scale = max(float(np.abs(v).max()) for v in ref.values())
    err, where = 0.0, None
    for r, toks in reqs.items():
        for p in range(len(toks)):
            e = float(np.abs(got[r][p] - ref[r][p]).max())
            if not e <= err:
                err, where = e, (r, p)
    return err / scale, where


def replay(folder, cfg, dtype, trace, out_dir, page=16, **kw):
    from inferrs_amd.engine import Engine, run_trace
    eng = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=-(-trace.max_tokens // page), max_seqs=4, **kw)
    run_trace(eng, trace.lines, out_dir, io.StringIO())
    eng.cache.check_invariants()
    assert not eng.cache.sequences and all(g.pool.num_free == g.pool.num_pages for g in eng.cache.groups)
    assert eng.cache.slots.num_free == eng.cache.slots.num_slots
    return trace.read(out_dir, cfg["vocab"])


def traces(reqs):
    short = {r: t for r, t in reqs.items() if len(t) <= 65}
    return {
        "whole": tm.whole(reqs),
        "tail32": tm.prefix_then_single(reqs, 32),
        "every token alone": tm.prefix_then_single(short, 10 ** 6),
        "a long tail": tm.prefix_then_single({r: t for r, t in reqs.items() if 130 <= len(t) <= 300}, 120),
        "portions": tm.portions(reqs, [7, 2, 16, 3, 2, 33, 5, 2, 64]),
        "portions of two and three": tm.portions(short, [2, 3]),
        "mixed": tm.mixed(reqs, seed=1),
        "mixed2": tm.mixed(dict(reversed(list(reqs.items()))), seed=2, max_live=3),
    }


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{c[0]}x{c[1]:g}")
def test_every_cutting_matches_plain(models, tmp_path, case, dtype):
    folder, cfg, tensors, reqs, ref = models[case]
    for mode, trace in traces(reqs).items():
        if mode.startswith("mixed"):
            assert trace.max_live >= 3 and trace.max_tokens < sum(tm.round_up(len(t), 64) for t in reqs.values())
        got = replay(folder, cfg, dtype, trace, str(tmp_path / f"{mode}_{dtype}"), page=16 if mode != "mixed2" else 32)
        part = {r: reqs[r] for r in got}
        if dtype == "float32":
            for r, e in errors(got, ref, part).items():
                allowed = np.maximum(TOL_F32, 3.0 * NOISE[case][r])
                assert (e <= allowed).all(), (f"{case} {dtype} {mode}: {float(e[np.argmax(e / allowed)]):.3g} of the scale at "
                                              f"({r}, {int(np.argmax(e / allowed))}), allowed {float(allowed[np.argmax(e / allowed)]):.3g}")
            continue
        plain = rounded_errors(case, models)
        common = [r for r in part if r in plain]
        mine = np.concatenate([errors(got, ref, part)[r] for r in common])
        theirs = np.concatenate([plain[r] for r in common])
        assert np.isfinite(np.concatenate(list(errors(got, ref, part).values()))).all(), f"{case} {mode}: not finite"
        for q, slack in ((0.5, 1.1), (0.9, 1.5)):
            a, b = float(np.quantile(mine, q)), float(np.quantile(theirs, q))
            assert a <= slack * b + 1e-3, f"{case} {dtype} {mode}: quantile {q} of the errors {a:.3g}, plain in bfloat16 {b:.3g}"


def test_the_models_rest_on_what_the_tests_are_for(models):
    """A chunk or a window that is one place off, in an owner or in a reader, a sink or a gate that is left out: each moves
    the logits by far more than any tolerance above."""
    folder, cfg, tensors, reqs, ref = models[("A", 6.0)]
    toks = reqs["r7"]
    scale = float(np.abs(ref["r7"]).max())

    def moved(other_cfg, other_w):
        return float(np.abs(pl.forward(other_cfg, other_w, toks).numpy() - ref["r7"]).max()) / scale

    for i in range(len(cfg["layers"])):
        for delta in (-1, 1):
            other = copy.deepcopy(cfg)
            other["layers"][i]["mixer"]["mask"]["size"] += delta
            assert moved(other, tensors) > 100 * TOL_F32, f"layer {i}, a mask of {delta:+d}"
    for name in ("l0.mix.sink", "l2.mix.sink", "l1.mix.g", "l1.mlp.shared.sg", "l3.side.proj", "l1.mix.k.b"):
        assert moved(cfg, dict(tensors, **{name: torch.zeros_like(tensors[name])})) > 100 * TOL_F32, name


@pytest.mark.parametrize("name", ["A", "C", "D"])
def test_greedy_generation_through_the_scheduler(models, name):
    from inferrs_amd.engine import Engine
    from inferrs_amd.sampling import SamplingParams
    folder, cfg, tensors, reqs, ref = models[(name, 1.0)]
    prompts = [random_tokens(n, cfg["vocab"], 900 + n) for n in (1, 5, 40, 90, 17, 64)]
    n_new = [12, 30, 7, 20, 25, 3]
    eng = Engine.from_folder(folder, dtype="float32", page_size=8, num_pages=40, max_seqs=4)
    outs = eng.generate(prompts, [SamplingParams.greedy(max_tokens=n, bypass_stop_tokens=True) for n in n_new],
                        max_batch_size=3, max_tokens_per_step=48, prefill_chunk=16)
    for prompt, n, out in zip(prompts, n_new, outs):
        toks = list(prompt)
        for _ in range(n):
            toks.append(int(pl.forward(cfg, tensors, toks)[-1].argmax()))
        assert out.error is None and out.tokens == toks[len(prompt):]
    eng.cache.check_invariants()
    assert not eng.cache.sequences and eng.cache.slots.num_free == eng.cache.slots.num_slots


def test_decode_steps_replayed_from_graphs(models):
    """Generation with the serving loop's graphs against the same engine without them.  32-bit: the same sums in the
    same order, so the same tokens.  bfloat16: a graph's step sees its context bucket's width and an eager step the
    longest request, so keys may be split between waves in another way; given tokens are fed and the logits compared."""
    from inferrs_amd.engine import Engine
    from inferrs_amd.engine.engine import Entry
    from inferrs_amd.sampling import SamplingParams
    folder, cfg, tensors, reqs, ref = models[("D", 1.0)]
    prompts = [random_tokens(n, cfg["vocab"], 700 + n) for n in (33, 5, 120)]
    outs = []
    for graphs in (False, True):
        eng = Engine.from_folder(folder, dtype="float32", page_size=16, num_pages=64, max_seqs=4, use_graphs=graphs)
        assert eng.use_graphs == graphs
        res = eng.generate(prompts, [SamplingParams.greedy(max_tokens=40, bypass_stop_tokens=True)] * 3, max_batch_size=3)
        assert all(o.error is None for o in res) and (eng.graph_replays > 20) == graphs
        outs.append([o.tokens for o in res])
    assert outs[0] == outs[1]
    toks = reqs["r7"]                                    # 300 tokens: 250 as a prompt, 50 fed one by one across the ends of the shorter chunks
    want = ref["r7"][249:]
    scale = float(np.abs(ref["r7"]).max())
    for graphs in (False, True):
        eng = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=64, max_seqs=4, use_graphs=graphs)
        rows = [eng.step([Entry("a", toks[:250], [249])])[0].clone()]
        rows += [eng.step([Entry("a", [t], [0])])[0].clone() for t in toks[250:]]
        assert (eng.graph_replays > 20) == graphs
        err = float(np.abs(torch.stack(rows).cpu().numpy() - want).max()) / scale
        assert err <= 3e-2, (graphs, err)


def test_random_weights_engine_steps():
    """The measurement script's way in: a configuration object and weights drawn on the device."""
    from inferrs_amd.config.ligizen import LigizenConfig
    from inferrs_amd.engine import Engine
    from inferrs_amd.engine.engine import Entry
    eng = Engine.from_random(LigizenConfig.from_dict(CONFIGS["A"]), seed=1, dtype="bfloat16", page_size=16, num_pages=16, max_seqs=2)
    logits = eng.step([Entry("a", random_tokens(33, 211, 1), [32]), Entry("b", [5], [0])])
    assert logits.shape == (2, 211) and bool(torch.isfinite(logits).all())


def test_command_line_run_and_bench(models):
    """The command line serves the design as it serves the others: greedy tokens are the plain implementation's, a drawn run
    and the timing command finish."""
    folder, cfg, tensors, reqs, ref = models[("A", 1.0)]
    prompt = random_tokens(9, cfg["vocab"], 3)
    toks = list(prompt)
    for _ in range(6):
        toks.append(int(pl.forward(cfg, tensors, toks)[-1].argmax()))
    exe = [sys.executable, os.path.join(ROOT, "bin", "inferrs-amd")]
    common = ["--block-size", "16", "--max-blocks", "32", "--max-batch-size", "2"]
    proc = subprocess.run(exe + ["run", folder, ",".join(map(str, prompt)), "--dtype", "f32", "--temperature", "0",
                                 "--repetition-penalty", "1.0", "--max-tokens", "6"] + common, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [int(t) for t in proc.stdout.split()] == toks[len(prompt):]
    proc = subprocess.run(exe + ["run", folder, ",".join(map(str, prompt)), "--dtype", "bf16", "--seed", "5", "--max-tokens", "12",
                                 "--ignore-eos"] + common, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    drawn = [int(t) for t in proc.stdout.split()]
    assert len(drawn) == 12 and all(0 <= t < cfg["vocab"] for t in drawn)
    proc = subprocess.run(exe + ["bench", folder, "--dtype", "bf16", "--prompt-len", "40", "--max-tokens", "8", "--runs", "2"] + common,
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    rec = json.loads(proc.stdout.strip().splitlines()[-1])
    assert rec["prefill_tok_s"] > 0 and rec["decode_tok_s"] > 0


def test_trace_runner_program(models, tmp_path):
    folder, cfg, tensors, reqs, ref = models[("C", 1.0)]
    some = {r: reqs[r] for r in ("r2", "r3", "r4")}
    trace = tm.mixed(some, seed=5, max_live=2)
    out_dir = str(tmp_path / "out")
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", out_dir,
                        "--max-tokens", str(trace.max_tokens)], input=trace.text(), capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(len(trace.lines))]
    err, where = worst(trace.read(out_dir, cfg["vocab"]), ref, some)
    assert err <= TOL_F32, (err, where)
