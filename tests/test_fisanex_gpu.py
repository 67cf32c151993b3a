"""Fisanex on the GPU against the plain implementation (`plain_fisanex.py`, 64-bit).

Mechanisms alone, through the kernels' Python face: the kernel behind a sub-layer of a stream that is normed after every
sum (a dense output, routed rows with pairs that stand for the stream's own row, a second output, the model's end), the
norm / rotation / cache write on rows of any layout (values of a width of their own, a gate in the rows, no keys at
all), the paged attention with values narrower and wider than keys in every kernel that takes them (plain and matrix
cores, keys split and not, prompts and single tokens) with a key that stands out just inside a window's edge and a
stronger one just outside it, the router with a correction in the choice and outputs that name no expert, the experts'
plan without those pairs, the small kernels (sigmoid gate, clamped gate, scaled embedding, a factor on the logits).
Then whole models through the engine's step function under every way of cutting the work (whole prompts, a prompt and
then token by token, every token alone, portions down to two tokens, up to four live requests mixed in a pool whose pages
and slots are used again), in both precisions, with ordinary weights and with sharpened queries.  Greedy generation runs
through the engine's own entry point and scheduler, the command line and the replay program.

Tolerances.  32-bit: 2e-5 of the largest logit against the 64-bit result, at every position; where the plain
implementation's own 32-bit arithmetic is further off than a third of that, three times what it is off.  bfloat16:
the measure is the distribution of the positions' errors against that of the plain implementation in bfloat16 arithmetic
(every operation rounded) on the same positions: the engine keeps more in 32-bit than that, so its median and its ninth
decile must not be larger (a tenth and a half of slack)."""
import copy
import io
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_fisanex as pf
import trace_modes as tm
from fisanex_configs import CONFIGS, random_tokens, write_model

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


# ---- the kernel behind a sub-layer ------------------------------------------------------------------

@pytest.mark.parametrize("W", [40, 33, 300, 5000])
@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
def test_step_behind_a_sublayer(W, y_dtype):
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(W)
    n, top, real = 19, 3, 4
    x = torch.randn(n, W, generator=g)
    y, y2 = (torch.randn(n, W, generator=g).to(y_dtype) for _ in range(2))
    routed = torch.randn(n, top, W, generator=g)
    rw = torch.rand(n, top, generator=g)
    sel = torch.randint(0, real + 2, (n, top), generator=g, dtype=torch.int32)
    routed[sel >= real] = float("nan")                     # (rows of pairs that name no expert are never written: never read)
    w = 1.0 + 0.1 * torch.randn(W, generator=g)
    # a dense output
    xs = dev(x)
    h = ops.postnorm_step(xs, alpha=1.7, y=dev(y), weight=dev(w), eps=1e-5, h_dtype=y_dtype)
    want = pf.rms_norm(1.7 * x.double() + y.double(), w.double(), 1e-5)
    np.testing.assert_allclose(xs.cpu().numpy(), want.numpy(), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(h.float().cpu().numpy(), want.numpy(), rtol=1e-2 if y_dtype == torch.bfloat16 else 1e-5, atol=1e-2 if y_dtype == torch.bfloat16 else 1e-5)
    # routed rows, some of them the stream's own row, and a second output beside them
    xs = dev(x)
    ops.postnorm_step(xs, alpha=0.6, routed=dev(routed), routed_weights=dev(rw), sel=dev(sel), real_experts=real, y2=dev(y2),
                      weight=dev(w), eps=1e-6)
    rows = torch.where((sel >= real)[:, :, None], x.double()[:, None, :], routed.double().nan_to_num())
    want = pf.rms_norm(0.6 * x.double() + (rw.double()[:, :, None] * rows).sum(1) + y2.double(), w.double(), 1e-6)
    np.testing.assert_allclose(xs.cpu().numpy(), want.numpy(), rtol=1e-5, atol=1e-5)
    # outputs that are products still split along their k: the kernel adds the splits up
    if y_dtype == torch.float32:
        parts, parts2 = (torch.randn(s, n, W, generator=g) for s in (3, 1))
        xs2 = dev(x)
        ops.postnorm_step(xs2, alpha=0.6, y=ops.Partials(dev(parts)), weight=dev(w), eps=1e-6)
        np.testing.assert_allclose(xs2.cpu().numpy(), pf.rms_norm(0.6 * x.double() + parts.double().sum(0), w.double(), 1e-6).numpy(),
                                   rtol=1e-5, atol=1e-5)
        xs2 = dev(x)
        ops.postnorm_step(xs2, alpha=0.6, routed=dev(routed), routed_weights=dev(rw), sel=dev(sel), real_experts=real,
                          y=ops.Partials(dev(parts2)), y2=ops.Partials(dev(parts)), weight=dev(w), eps=1e-6)
        want2 = pf.rms_norm(0.6 * x.double() + (rw.double()[:, :, None] * rows).sum(1) + parts.double().sum(0) + parts2.double().sum(0),
                            w.double(), 1e-6)
        np.testing.assert_allclose(xs2.cpu().numpy(), want2.numpy(), rtol=1e-5, atol=1e-5)
    # the model's end: some rows through a norm, the stream left as it is
    before = xs.clone()
    pick = torch.tensor([5, 0, 18], dtype=torch.int32)
    tail = ops.postnorm_step(xs, weight=dev(w), eps=1e-6, h_dtype=torch.float32, rows=dev(pick))
    np.testing.assert_allclose(tail.cpu().numpy(), pf.rms_norm(want[pick.long()], w.double(), 1e-6).numpy(), rtol=1e-5, atol=1e-5)
    assert torch.equal(xs, before)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_small_kernels(dtype):
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(2)
    tol = dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(rtol=1e-5, atol=1e-6)
    for cols, ld, off in ((24, 80, 40), (13, 30, 17)):
        a, gate = torch.randn(11, cols, generator=g).to(dtype), (3 * torch.randn(11, ld, generator=g)).to(dtype)
        got = ops.sigmoid_gate(dev(a.clone()), dev(gate), off)
        np.testing.assert_allclose(got.float().cpu().numpy(), (a.double() * torch.sigmoid(gate.double()[:, off:off + cols])).numpy(), **tol)
    for inter in (16, 7):
        gu = (2 * torch.randn(9, 2 * inter, generator=g)).to(dtype)
        got = ops.clamped_gate_mul(dev(gu), 1.1, 1.702)
        gg, uu = gu.double()[:, :inter].clamp(max=1.1), gu.double()[:, inter:].clamp(-1.1, 1.1)
        np.testing.assert_allclose(got.float().cpu().numpy(), (gg * torch.sigmoid(1.702 * gg) * (uu + 1)).numpy(), **tol)
    table = torch.randn(31, 20, generator=g).to(dtype)
    ids = torch.tensor([3, 30, 0, 3], dtype=torch.int32)
    rows, lo = ops.embed_gather_scaled(dev(table), dev(ids), 12.0, rounded=True)
    assert torch.equal(rows.cpu(), table.float()[ids.long()] * 12.0) and lo.dtype == dtype
    np.testing.assert_allclose(lo.float().cpu().numpy(), rows.cpu().numpy(), **tol)
    z = torch.randn(5, 7, generator=g)
    assert torch.equal(ops.scale_inplace(dev(z.clone()), 0.25).cpu(), z * 0.25)


# ---- norm, rotation and cache write on rows of any layout ----------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,dv,rot", [(4, 2, 16, 8, 8), (2, 1, 32, 48, 32), (5, 5, 12, 20, 6), (3, 1, 128, 64, 0)])
def test_rows_of_any_layout(H, G, d, dv, rot, dtype):
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(H * d)
    n, page, pages, extra = 21, 8, 6, 5
    width = extra + H * d + G * d + G * dv + H * dv
    q_off, k_off, v_off = extra, extra + H * d, extra + H * d + G * d
    proj = torch.randn(n, width, generator=g).to(dtype)
    qw, kw = 1 + 0.3 * torch.randn(d, generator=g), 1 + 0.3 * torch.randn(d, generator=g)
    positions = torch.randint(0, 500, (n,), generator=g)
    slots = torch.randperm(pages * page, generator=g)[:n].to(torch.int32)
    cos = sin = None
    if rot:
        f = torch.tensor([777.0 ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float64)
        ang = positions.double()[:, None] * f
        cos, sin = dev(torch.cos(ang).float()), dev(torch.sin(ang).float())
    kc, vc = torch.zeros(pages, G, page, d, dtype=dtype), torch.zeros(pages, G, dv, page, dtype=dtype)
    kc_d, vc_d = dev(kc), dev(vc)
    q = ops.qk_rope_kv_strided(dev(proj), H, G, d, dv, q_off=q_off, k_off=k_off, v_off=v_off, q_norm_w=dev(qw), k_norm_w=dev(kw),
                               eps=1e-5, add_one=False, cos=cos, sin=sin, rot=rot, interleaved=False, k_cache=kc_d, v_cache=vc_d,
                               slots=dev(slots), page_size=page)
    p64 = proj.double()
    want_q = pf.rotate_halves(pf.rms_norm(p64[:, q_off:k_off].view(n, H, d), qw.double(), 1e-5), positions, 777.0, rot)
    want_k = pf.rotate_halves(pf.rms_norm(p64[:, k_off:v_off].view(n, G, d), kw.double(), 1e-5), positions, 777.0, rot)
    want_v = p64[:, v_off:v_off + G * dv].view(n, G, dv)
    rel = 1e-2 if dtype == torch.bfloat16 else 1e-5
    assert_close(q, want_q, rel, "queries")
    got_k = kc_d.cpu()[slots.long() // page, :, slots.long() % page]
    got_v = vc_d.cpu()[slots.long() // page, :, :, slots.long() % page]
    assert_close(got_k, want_k, rel, "cached keys")
    assert_close(got_v, want_v, rel, "cached values")
    unused = torch.ones(pages * page, dtype=torch.bool)
    unused[slots.long()] = False
    assert not kc_d.cpu().view(pages, G, page, d).permute(0, 2, 1, 3).reshape(pages * page, -1)[unused].any()
    # a layer without keys of its own: the same queries, the cache left alone
    only_q = torch.cat([proj[:, :k_off], proj[:, v_off + G * dv:]], dim=1).contiguous()
    before = kc_d.clone()
    q2 = ops.qk_rope_kv_strided(dev(only_q), H, G, d, dv, q_off=q_off, k_off=None, v_off=None, q_norm_w=dev(qw), k_norm_w=None,
                                eps=1e-5, add_one=False, cos=cos, sin=sin, rot=rot, interleaved=False, k_cache=kc_d, v_cache=vc_d,
                                slots=dev(slots), page_size=page)
    assert torch.equal(q2, q) and torch.equal(kc_d, before)


# ---- the attention with values of a width of their own, at a window's edge ----------------------------------

def attention_reference(q, kc, vc, positions, token_seq, table, window, scale):
    """Request by request on dense copies of its keys and values."""
    n, nq, d = q.shape
    nkv, page, dv = kc.shape[1], kc.shape[2], vc.shape[2]
    out = torch.zeros(n, nq, dv, dtype=torch.float64)
    for s in token_seq.unique().tolist():
        rows = (token_seq == s).nonzero().flatten()
        pos = positions[rows].long()
        length = int(pos.max()) + 1
        first = max(int(pos.min()) - window + 1, 0) if window else 0
        pages = table[s, :-(-length // page)].long()
        k = kc[pages].double().permute(1, 0, 2, 3).reshape(nkv, -1, d)[:, :length].repeat_interleave(nq // nkv, 0)
        v = vc[pages].double().permute(1, 0, 3, 2).reshape(nkv, -1, dv)[:, :length].repeat_interleave(nq // nkv, 0)
        k[:, :first], v[:, :first] = 0.0, 0.0            # (pages that every window has passed may hold anything)
        sc = torch.einsum("thd,hjd->thj", q[rows].double(), k) * scale
        j = torch.arange(length)
        hidden = j[None, :] > pos[:, None]
        if window:
            hidden |= j[None, :] < (pos[:, None] - window + 1)
        p = torch.softmax(sc.masked_fill(hidden[:, None, :], float("-inf")), dim=-1)
        out[rows] = torch.einsum("thj,hjd->thd", p, v)
    return out


def attention_case(dtype, nq, nkv, d, dv, page, lens, q_lens, window, seed):
    """Cached requests in shuffled pages; what lies beyond a request's length, and in pages that every window of the step
    has passed, is NaN.  For every request's last query, head 0: the key just inside the window's edge points along the
    query, and the key one place further back, outside the window, does so twice as strongly."""
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
        inside = max(l - window, 0) if window else 0
        kc[int(table[s, inside // page]), 0, inside % page] = (last * 3).to(dtype)
        if window and inside > 0:
            kc[int(table[s, (inside - 1) // page]), 0, (inside - 1) % page] = (last * 6).to(dtype)
        passed = (max(l - ql - window + 1, 0) // page) * page if window else 0
        for j in list(range(passed)) + list(range(l, -(-l // page) * page)):
            kc[int(table[s, j // page]), :, j % page] = float("nan")
            vc[int(table[s, j // page]), :, :, j % page] = float("nan")
    return q, kc, vc, positions, token_seq, table


SHAPES = [(4, 2, 16, 8), (2, 1, 32, 48), (5, 5, 12, 20), (4, 1, 128, 64), (2, 2, 64, 16), (3, 1, 64, 256), (2, 2, 48, 48)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,d,dv", SHAPES)
@pytest.mark.parametrize("window", [0, 1, 17, 64, 300])
def test_attention_with_values_of_their_own_width(nq, nkv, d, dv, window, dtype):
    """Prompts, portions late in a context and single tokens in one step, in every kernel that takes the sizes."""
    from inferrs_amd import ops
    page = 16
    lens, q_lens = [700, 333, 64, 1, 1100], [700, 40, 1, 1, 1]
    q, kc, vc, positions, token_seq, table = attention_case(dtype, nq, nkv, d, dv, page, lens, q_lens, window, seed=d + dv + window)
    want = attention_reference(q, kc, vc, positions, token_seq, table, window, 0.2)
    rel = 2e-2 if dtype == torch.bfloat16 else 2e-5
    args = [dev(t) for t in (q, kc, vc, positions, token_seq, table)]
    for split in (None, False):
        got = ops.attention_generic(*args, window=window or None, scale=0.2, max_kv_len=max(lens), split=split)
        assert got.shape == (len(positions), nq, dv)
        assert_close(got, want, rel, f"plain kernel, split {split}")
    if not ops.attention_mfma_fits(dtype, d, page, dv):
        return
    cu = dev(torch.tensor([0] + list(np.cumsum(q_lens)), dtype=torch.int32))
    for splits in (None, 1, 4):
        got = ops.attention_mfma(args[0], args[1], args[2], args[3], cu, args[5], max_q_len=max(q_lens), max_kv_len=max(lens),
                                 window=window or None, scale=0.2, splits=splits)
        assert got.shape == (len(positions), nq, dv)
        assert_close(got, want, rel, f"matrix cores, splits {splits}")
    # single tokens alone (the decode launch)
    single = [s for s, ql in enumerate(q_lens) if ql == 1]
    rows = torch.tensor([int(np.cumsum(q_lens)[s]) - 1 for s in single])
    q1, pos1 = dev(q[rows]), dev(positions[rows])
    cu1 = dev(torch.arange(len(single) + 1, dtype=torch.int32))
    got = ops.attention_mfma(q1, args[1], args[2], pos1, cu1, dev(table[single]), max_q_len=1, max_kv_len=max(lens),
                             window=window or None, scale=0.2)
    assert_close(got, want[rows], rel, "matrix cores, single tokens")


# ---- the router and the experts' plan ----------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,identity,top,W", [(5, 2, 3, 48), (2, 2, 4, 64), (3, 1, 2, 50), (70, 9, 6, 136), (4, 0, 1, 40)])
def test_router_with_a_correction(E, identity, top, W, dtype):
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(E * W)
    n = 57
    h = torch.randn(n, W, generator=g).to(dtype)
    router = (2 * torch.randn(E + identity, W, generator=g) / W ** 0.5).to(dtype)
    corr = 0.15 * torch.randn(E + identity, generator=g)
    sel, weight = ops.route(dev(h), dev(router), top, 1.0, "softmax", False, dev(corr))
    s = torch.softmax(h.double() @ router.double().T, dim=-1)
    key = s + corr.double()
    order = torch.argsort(key, dim=-1, descending=True)
    # (a choice between two keys closer than rounding may go either way: such rows are left out)
    gap = torch.gather(key, 1, order)[:, :-1] - torch.gather(key, 1, order)[:, 1:] if E + identity > 1 else torch.ones(n, 1)
    clear = (gap[:, :top].abs().min(dim=1).values > 1e-5) if gap.shape[1] else torch.ones(n, dtype=torch.bool)
    assert clear.float().mean() > 0.8
    assert torch.equal(sel.cpu().long()[clear], order[clear, :top])
    np.testing.assert_allclose(weight.cpu().numpy()[clear], torch.gather(s, 1, order[:, :top]).numpy()[clear], rtol=1e-4, atol=1e-6)
    # the choice differs from the scores' own order somewhere: the correction counts
    assert not torch.equal(order[:, :top], torch.argsort(s, dim=-1, descending=True)[:, :top])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,top,W", [(36, 4, 256), (12, 2, 50), (70, 6, 136), (200, 3, 64)])
def test_router_does_not_depend_on_the_step(E, top, W, dtype):
    """A step of few tokens and one of many launch the router differently (more waves a token, fewer outputs a wave): a
    token's choice and weights are the same bits in both, wherever in a step the token stands."""
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(E + W)
    n = 1031
    h = dev(torch.randn(n, W, generator=g).to(dtype))
    router = dev((2 * torch.randn(E, W, generator=g) / W ** 0.5).to(dtype))
    corr = dev(0.15 * torch.randn(E, generator=g))
    sel, weight = ops.route(h, router, top, 1.0, "softmax", False, corr)
    for first, count in ((0, 1), (3, 8), (40, 64), (100, 65), (500, 300), (1000, 31), (n - 1, 1)):
        s2, w2 = ops.route(h[first:first + count].contiguous(), router, top, 1.0, "softmax", False, corr)
        assert torch.equal(s2, sel[first:first + count]) and torch.equal(w2, weight[first:first + count]), (first, count)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,identity,top,W,ff", [(5, 2, 3, 48, 24), (3, 1, 2, 50, 30), (6, 3, 2, 64, 32)])
def test_experts_leave_out_pairs_that_name_none(E, identity, top, W, ff, dtype):
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(E + ff)
    for n in (1, 9, 150):
        h = torch.randn(n, W, generator=g).to(dtype)
        sel = torch.stack([torch.randperm(E + identity, generator=g)[:top] for _ in range(n)]).to(torch.int32)
        gu = (1.5 * torch.randn(E, 2 * ff, W, generator=g) / W ** 0.5).to(dtype)
        down = (torch.randn(E, W, ff, generator=g) / ff ** 0.5).to(dtype)
        tiled = ops.mix.experts_tiled_fits(dtype, W, ff)
        a, b = dev(gu), dev(down)
        if tiled:
            a, b = ops.mix.tile_weights(a.view(E, 2, ff, W)), ops.mix.tile_weights(b)
        y = ops.experts_forward(dev(h), dev(sel), a, b, 1.2, 1.702, ff=ff if tiled else None).cpu()
        for t in range(n):
            for k in range(top):
                e = int(sel[t, k])
                if e >= E:
                    continue
                w = {"gate": gu[e, :ff], "up": gu[e, ff:], "down": down[e]}
                want = pf.clamped_expert(h[t:t + 1].double(), {k2: v.double() for k2, v in w.items()}, "", 1.2)[0]
                assert_close(y[t, k], want, 2e-2 if dtype == torch.bfloat16 else 2e-5, f"n={n} pair ({t}, {k})")


# ---- whole models under every cutting ---------------------------------------------------------------

_ROUNDED = {}
NOISE = {}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, sharpen in CASES:
        cfg = CONFIGS[name]
        folder = str(tmp_path_factory.mktemp(f"fisanex_{name}"))
        tensors = write_model(folder, cfg, seed=11, sharpen=sharpen)
        reqs = {f"r{i}": random_tokens(n, cfg["vocab"], 40 + i) for i, n in enumerate(LENGTHS)}
        ref64 = {r: pf.forward(cfg, tensors, t) for r, t in reqs.items()}
        ref = {r: v.numpy().astype(np.float32) for r, v in ref64.items()}
        scale = max(float(v.abs().max()) for v in ref64.values())
        # what rounding alone does at every position: the plain implementation in 32-bit against itself in 64-bit
        NOISE[(name, sharpen)] = {r: ((pf.forward(cfg, tensors, t, dtype=torch.float32).double() - ref64[r]).abs().max(1).values
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
        rounded = {r: pf.forward(cfg, tensors, t, dtype=torch.bfloat16).float().numpy() for r, t in some.items()}
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
    """A window that is one place off, in an owner or in a reader, moves the logits by far more than any tolerance above."""
    folder, cfg, tensors, reqs, ref = models[("A", 6.0)]
    toks = reqs["r7"]
    scale = float(np.abs(ref["r7"]).max())
    for i in range(len(cfg["layers"])):
        for delta in (-1, 1):
            other = copy.deepcopy(cfg)
            other["layers"][i]["mixer"]["mask"]["size"] += delta
            moved = float(np.abs(pf.forward(other, tensors, toks).numpy() - ref["r7"]).max()) / scale
            assert moved > 100 * TOL_F32, f"layer {i}, a window of {delta:+d}: {moved}"


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
            toks.append(int(pf.forward(cfg, tensors, toks)[-1].argmax()))
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
    toks = reqs["r6"]                                    # 130 tokens: 90 as a prompt, 40 fed one by one
    want = ref["r6"][89:]
    scale = float(np.abs(ref["r6"]).max())
    for graphs in (False, True):
        eng = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=64, max_seqs=4, use_graphs=graphs)
        rows = [eng.step([Entry("a", toks[:90], [89])])[0].clone()]
        rows += [eng.step([Entry("a", [t], [0])])[0].clone() for t in toks[90:]]
        assert (eng.graph_replays > 20) == graphs
        err = float(np.abs(torch.stack(rows).cpu().numpy() - want).max()) / scale
        assert err <= 3e-2, (graphs, err)


def test_a_second_norm_without_a_feed_forward(models, tmp_path):
    """A file that holds a second norm for a layer without a feed-forward: the scaled stream goes through it."""
    from inferrs_amd.engine import Engine
    from inferrs_amd.engine.engine import Entry
    from inferrs_amd.weights import write_safetensors
    folder, cfg, tensors, reqs, ref = models[("A", 1.0)]
    more = dict(tensors, **{"l3.norm2": (0.5 + torch.rand(cfg["width"])).to(torch.bfloat16)})
    new = str(tmp_path / "with_norm2")
    os.makedirs(new)
    with open(os.path.join(new, "config.json"), "w") as f:
        import json
        json.dump(cfg, f)
    write_safetensors(os.path.join(new, "model.safetensors"), more)
    toks = reqs["r5"]
    want = pf.forward(cfg, more, toks)
    assert float((want - torch.from_numpy(ref["r5"]).double()).abs().max()) > 1e-2
    eng = Engine.from_folder(new, dtype="float32", page_size=16, num_pages=8, max_seqs=2)
    got = eng.step([Entry("a", toks, list(range(len(toks))))]).double().cpu()
    assert float((got - want).abs().max()) <= TOL_F32 * float(want.abs().max())


def test_random_weights_engine_steps():
    """The measurement script's way in: a configuration object and weights drawn on the device."""
    from inferrs_amd.config.fisanex import FisanexConfig
    from inferrs_amd.engine import Engine
    from inferrs_amd.engine.engine import Entry
    eng = Engine.from_random(FisanexConfig.from_dict(CONFIGS["A"]), seed=1, dtype="bfloat16", page_size=16, num_pages=16, max_seqs=2)
    logits = eng.step([Entry("a", random_tokens(33, 211, 1), [32]), Entry("b", [5], [0])])
    assert logits.shape == (2, 211) and bool(torch.isfinite(logits).all())


def test_command_line_run_and_bench(models):
    """The command line serves the design as it serves the others: greedy tokens are the plain implementation's, a drawn run
    and the timing command finish."""
    import json
    folder, cfg, tensors, reqs, ref = models[("A", 1.0)]
    prompt = random_tokens(9, cfg["vocab"], 3)
    toks = list(prompt)
    for _ in range(6):
        toks.append(int(pf.forward(cfg, tensors, toks)[-1].argmax()))
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
