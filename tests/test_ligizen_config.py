"""Ligizen without a GPU: config.json -> the model as data (layers, run order, whose cache a layer reads, tensor names
and shapes, what each mixer keeps per request), the errors that name a key, the stretched frequencies, and the plain
implementation against itself (a prefix, what each mechanism is worth, the edges of chunks and windows)."""
import copy
import math

import numpy as np
import pytest
import torch

import plain_ligizen as pl
from ligizen_configs import CONFIGS, random_tokens, random_weights, sharpened, tensor_shapes

from inferrs_amd.cache import CacheManager
from inferrs_amd.config.base import ConfigError
from inferrs_amd.config.ligizen import LigizenConfig
from inferrs_amd.config.registry import resolve_architecture
from inferrs_amd.config.spec import PositionSpec
from inferrs_amd.parts.assemble import model_tensors
from inferrs_amd.parts.base import PagedKV, part_class
from inferrs_amd.parts.position import inverse_frequencies, llama3_scaling


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_tensor_names_and_shapes(name):
    cfg = CONFIGS[name]
    assert resolve_architecture(cfg) is LigizenConfig
    spec = LigizenConfig.from_dict(cfg).to_spec()
    expected, optional = model_tensors(spec)
    assert optional == {"head"}           # (a file without it would take its logits through the embedding's table)
    assert {k: tuple(v.shape) for k, v in expected.items()} == tensor_shapes(cfg)


def test_the_model_as_data():
    spec = LigizenConfig.from_dict(CONFIGS["A"]).to_spec()
    assert [(e.layer, e.cache_of) for e in spec.schedule] == [(0, None), (1, None), (2, None), (3, 1)]
    assert all(l.arrangement == "parallel" and len(l.norms) == 1 and l.norms[0].kind == "layernorm" for l in spec.layers)
    assert [l.residual.side.offset for l in spec.layers] == [0, 6, 12, 18] and spec.embedding.side_width == 24
    assert spec.embedding.scale == 3.0 and spec.embedding.wide and spec.head.cap == 8.0 and spec.head.name == "head"
    assert spec.final_norm.kind == "layernorm" and spec.layers[3].ffn is None
    m0, m1, m3 = spec.layers[0].mixer, spec.layers[1].mixer, spec.layers[3].mixer
    assert (m0.kind, m0.q_rank, m0.kv_rank, m0.window, m0.sink, m0.gate_per_head) == ("latent_attention", 16, 12, 24, True, True)
    assert m0.position.pairing == "interleaved" and m0.position.rot_dim == 4 and m0.position.scaling is None
    assert (m1.kind, m1.mask_chunk, m1.window, m1.qkv_bias, m1.qk_unit_norm, m1.gate_per_head) == ("attention", 24, None, True, True, True)
    assert m1.position.pairing == "half" and m1.position.scaling == ("llama3", 4.0, 1.0, 4.0, 40.0)
    assert m1.own_kv and not m3.own_kv and m3.mask_chunk == 40 and m3.scale == 0.3
    f1, f2 = spec.layers[1].ffn, spec.layers[2].ffn
    assert (f1.experts, f1.top, f1.score, f1.renormalize, f1.weight_on_input, f1.shared_gate) == (5, 2, "sigmoid", False, True, True)
    assert f1.shared.intermediate == 32 and f1.shared.limit == 0.8 and f2.shared is None and not f2.shared_gate
    none = LigizenConfig.from_dict(CONFIGS["B"]).to_spec()
    assert none.embedding.side_name is None and all(l.residual.side is None for l in none.layers)


def test_what_each_mixer_keeps():
    spec = LigizenConfig.from_dict(CONFIGS["A"]).to_spec()
    needs = [part_class("mixer", l.mixer).cache_need(l.mixer) for l in spec.layers]
    # a latent layer keeps one row a position under its window; chunks keep every position; a reader keeps nothing
    assert needs == [PagedKV(1, 16, 24), PagedKV(2, 16, None, v_head_dim=8), PagedKV(1, 32, 17), None]
    cm = CacheManager({i: n for i, n in enumerate(needs) if n is not None}, page_size=8, num_pages=40, max_seqs=2)
    cm.add_sequence("a")
    assert cm.reserve("a", 200)
    cm.commit("a", 200)
    by_window = {g.need.window: g for g in cm.groups}
    assert by_window[None].pool.num_free == 40 - 25 and by_window[17].pool.num_free > by_window[24].pool.num_free > 40 - 25
    cm.free_sequence("a")
    cm.check_invariants()
    assert all(g.pool.num_free == 40 for g in cm.groups)


@pytest.mark.parametrize("change, key", [
    (lambda c: c["layers"][2].__setitem__("type", "mamba2"), "layers[2].type"),
    (lambda c: c["layers"][3]["mixer"].__setitem__("kv_from", 3), "kv_from"),
    (lambda c: c["layers"][3]["mixer"].__setitem__("kv_from", 0), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].__setitem__("kv_from", 1), "kv_from"),
    (lambda c: c["layers"][3]["mixer"].__setitem__("vdim", 16), "vdim"),
    (lambda c: c["layers"][3]["mixer"]["rot"].__setitem__("base", 7.0), "rot"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "mixer.scale"),
    (lambda c: c["layers"][0]["mixer"].pop("q_rank"), "q_rank"),
    (lambda c: c["layers"][0]["mixer"].pop("mask"), "mask"),
    (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 7), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].pop("low"), "scaling.low"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("kv_heads", 3), "kv_heads"),
    (lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 9), "router.top"),
    (lambda c: c["layers"][1]["mlp"]["expert"].pop("limit"), "expert.limit"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "gelu"), "mlp.kind"),
    (lambda c: c["norm"].pop("eps"), "norm.eps"),
    (lambda c: c["token_side"].pop("dim"), "token_side.dim"),
    (lambda c: c["embedding"].pop("scale"), "embedding.scale"),
    (lambda c: c.pop("width"), "width"),
])
def test_errors_name_the_key(change, key):
    cfg = copy.deepcopy(CONFIGS["A"])
    change(cfg)
    with pytest.raises(ConfigError) as e:
        LigizenConfig.from_dict(cfg)
    assert key in str(e.value)


def test_stretched_frequencies():
    """The package's law against the plain implementation's, pair by pair, with all three ranges present."""
    for base, dims, sc in ((50.0, 8, (4.0, 1.0, 4.0, 40.0)), (30000.0, 48, (8.0, 1.0, 4.0, 256.0)), (10000.0, 64, (2.0, 0.5, 3.0, 1000.0))):
        mine = llama3_scaling(inverse_frequencies(base, dims), *sc)
        plain = pl.frequencies({"base": base, "dims": dims, "scaling": dict(zip(("factor", "low", "high", "original"), sc))}, torch.float64)
        assert np.allclose(mine, plain.numpy(), rtol=2e-6)
        bare = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
        ratio = plain.numpy() / bare
        kept, divided = np.isclose(ratio, 1.0), np.isclose(ratio, 1.0 / sc[0])
        assert kept.any() and divided.any() and (~kept & ~divided).any(), (base, dims)
        wave = 2 * math.pi / bare
        assert (kept == (wave < sc[3] / sc[2])).all() and (divided == (wave > sc[3] / sc[1])).all()
    from inferrs_amd.parts.position import Rotary
    assert PositionSpec("rope", 8, 8, 50.0, "half", ("llama3", 4.0, 1.0, 4.0, 40.0)) is not None
    assert Rotary(PositionSpec("rope", 8, 8, 50.0, "half", ("llama3", 4.0, 1.0, 4.0, 40.0)), {}, torch.float32, "cpu").magnitude == 1.0


def test_plain_against_itself():
    cfg = sharpened(CONFIGS["A"], 6.0)
    w = random_weights(cfg, 3)
    toks = random_tokens(70, cfg["vocab"], 1)
    whole = pl.forward(cfg, w, toks)
    scale = float(whole.abs().max())
    # causal: a prefix gives the same logits
    assert torch.allclose(pl.forward(cfg, w, toks[:23]), whole[:23], atol=1e-10)
    streams = []
    pl.forward(cfg, w, toks, layers_out=streams)
    assert len(streams) == 4

    def moved(other_cfg=None, other_w=None, rows=slice(None)):
        return float((pl.forward(other_cfg or cfg, other_w or w, toks) - whole)[rows].abs().max()) / scale

    # a chunk or a window one place longer or shorter shows; a chunk's edge moves where the FIRST token behind it stands
    for i in range(4):
        for delta in (-1, 1):
            c = copy.deepcopy(cfg)
            c["layers"][i]["mixer"]["mask"]["size"] += delta
            assert moved(c) > 1e-3, (i, delta)
    c = copy.deepcopy(cfg)
    c["layers"][1]["mixer"]["mask"]["size"] = 25                     # (tokens 0..23 see the same keys either way)
    assert moved(c, rows=slice(0, 24)) < 1e-12 < moved(c, rows=slice(24, 25))
    # keys of its own instead of the earlier layer's
    c = copy.deepcopy(cfg)
    c["layers"][3]["mixer"].pop("kv_from")
    w2 = dict(w, **{f"l3.mix.{n}": w[f"l1.mix.{n}"] for n in ("k", "k.b", "v", "v.b")})
    assert moved(c, w2) > 1e-3
    # every mechanism is worth something: the sink, the gates, the biases, the shared expert and its gate, the token's
    # input, the stretching, the norm's bias, the cap, the scale on the embedding
    zero = lambda n: {n: torch.zeros_like(w[n])}
    for n in ("l0.mix.sink", "l0.mix.g", "l1.mix.g", "l1.mix.q.b", "l1.mix.k.b", "l1.mix.v.b", "l1.mlp.shared.sg",
              "l1.mlp.shared.down", "l2.side.proj", "l0.norm1.b", "final.norm.b", "side.embed"):
        assert moved(other_w=dict(w, **zero(n))) > 1e-4, n
    c = copy.deepcopy(cfg)
    c["layers"][1]["mixer"]["rot"].pop("scaling")
    c["layers"][3]["mixer"]["rot"].pop("scaling")
    assert moved(c) > 1e-3
    assert moved(dict(cfg, logit_softcap=1000.0)) > 1e-3 and moved(dict(cfg, embedding={"scale": 1.0})) > 1e-3
    # the weight stands on the expert's input: behind it the result differs wherever a limit bites
    h = torch.randn(9, 48, dtype=torch.float64)
    wd = {k: v.double() for k, v in w.items()}
    chosen, weight = pl.route(h, wd, "l1.mlp.", 2)
    inside = pl.clamped_expert(weight[:1, :1] * h[:1], wd, f"l1.mlp.e{int(chosen[0, 0])}.", 1.2)
    outside = weight[:1, :1] * pl.clamped_expert(h[:1], wd, f"l1.mlp.e{int(chosen[0, 0])}.", 1.2)
    assert (inside - outside).abs().max() > 1e-3 and (weight <= 1).all() and (weight[:, 0] >= weight[:, 1]).all()
