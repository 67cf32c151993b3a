"""Fisanex without a GPU: config.json -> the model as data (layers, run order, whose cache a layer reads, tensor names
and shapes, what each mixer keeps per request), the errors that name a key, the cache manager's groups, and the plain
implementation against itself (a prefix, a window wider than the sequence, what each mechanism is worth)."""
import copy

import pytest
import torch

import plain_fisanex as pf
from fisanex_configs import CONFIGS, random_tokens, random_weights, tensor_shapes

from inferrs_amd.cache import CacheManager
from inferrs_amd.config.base import ConfigError
from inferrs_amd.config.fisanex import FisanexConfig
from inferrs_amd.config.registry import resolve_architecture
from inferrs_amd.parts.assemble import model_tensors
from inferrs_amd.parts.base import PagedKV, part_class


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_tensor_names_and_shapes(name):
    cfg = CONFIGS[name]
    assert resolve_architecture(cfg) is FisanexConfig
    spec = FisanexConfig.from_dict(cfg).to_spec()
    expected, optional = model_tensors(spec)
    # (a layer without a feed-forward may still carry a second norm in its file: the one optional tensor)
    assert optional == {f"l{i}.norm2" for i, L in enumerate(cfg["layers"]) if L["mlp"] is None}
    assert {k: tuple(v.shape) for k, v in expected.items() if k not in optional} == tensor_shapes(cfg)
    assert not optional - set(expected)


def test_whose_cache_a_layer_reads():
    spec = FisanexConfig.from_dict(CONFIGS["A"]).to_spec()
    assert [(e.layer, e.cache_of) for e in spec.schedule] == [(0, None), (1, 0), (2, None), (3, 2)]
    assert [len(l.norms) for l in spec.layers] == [2, 2, 2, 1]
    assert all(l.arrangement == "post_norm" and l.residual.alpha == 1.5 for l in spec.layers)
    spec = FisanexConfig.from_dict(CONFIGS["D"]).to_spec()
    assert [(e.layer, e.cache_of) for e in spec.schedule] == [(0, None), (1, None), (2, 0), (3, 0)]
    assert spec.embedding.scale == 8.0 and spec.embedding.wide and spec.head.scale == 0.3 and spec.head.name is None


def test_what_each_mixer_keeps():
    spec = FisanexConfig.from_dict(CONFIGS["A"]).to_spec()
    needs = [part_class("mixer", l.mixer).cache_need(l.mixer) for l in spec.layers]
    # the owner keeps what its widest reader sees (40 against its own 24); a reader keeps nothing
    assert needs == [PagedKV(2, 16, 40, v_head_dim=8), None, PagedKV(1, 32, 17, v_head_dim=48), None]
    m0, m1 = spec.layers[0].mixer, spec.layers[1].mixer
    assert m0.own_kv and m0.gate and m0.window == 24 and m0.reader_windows == (40,) and m0.position.rot_dim == 8
    assert not m1.own_kv and m1.window == 40 and m1.scale == 0.25 and m1.value_dim == 8
    f1, f2 = spec.layers[1].ffn, spec.layers[2].ffn
    assert (f1.experts, f1.identity, f1.top, f1.score, f1.correction, f1.renormalize) == (5, 2, 3, "softmax", True, False)
    assert f1.shared.intermediate == 32 and f1.shared.limit == 0.8 and f2.shared is None and f2.identity == 0
    same = FisanexConfig.from_dict(CONFIGS["B"]).to_spec().layers[0].mixer
    assert same.position.kind == "none" and part_class("mixer", same).cache_need(same) == PagedKV(2, 64, 100)
    d = FisanexConfig.from_dict(CONFIGS["D"]).to_spec().layers[0].mixer
    assert d.reader_windows == (300, 33) and d.kept_window == 300


def test_cache_groups():
    spec = FisanexConfig.from_dict(CONFIGS["D"]).to_spec()
    needs = {}
    for stop, e in enumerate(spec.schedule):
        if e.cache_of is None:
            m = spec.layers[e.layer].mixer
            needs[stop] = part_class("mixer", m).cache_need(m)
    cm = CacheManager(needs, page_size=8, num_pages=50, max_seqs=2)
    assert sorted(g.layers for g in cm.groups) == [[0], [1]]
    cm.add_sequence("a")
    assert cm.reserve("a", 390)
    cm.commit("a", 390)
    by_window = {g.need.window: g for g in cm.groups}
    # pages that a window has passed are back in the pool: the group of window 64 holds far fewer than that of 300
    assert by_window[64].pool.num_free > by_window[300].pool.num_free
    cm.free_sequence("a")
    cm.check_invariants()
    assert all(g.pool.num_free == 50 for g in cm.groups)


@pytest.mark.parametrize("change, key", [
    (lambda c: c["layers"][1].__setitem__("type", "mamba2"), "layers[1].type"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("kv_from", 1), "kv_from"),
    (lambda c: c["layers"][3]["mixer"].__setitem__("kv_from", 1), "kv_from"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("vdim", 16), "vdim"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "mixer.scale"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 7), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 3), "kv_heads"),
    (lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 9), "router.top"),
    (lambda c: c["layers"][1]["mlp"]["expert"].pop("limit"), "expert.limit"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "gelu"), "mlp.kind"),
    (lambda c: c["norm"].pop("eps"), "norm.eps"),
    (lambda c: c.pop("postln_alpha"), "postln_alpha"),
    (lambda c: c.pop("logit_scale"), "logit_scale"),
    (lambda c: c["embedding"].pop("scale"), "embedding.scale"),
    (lambda c: c.pop("width"), "width"),
])
def test_errors_name_the_key(change, key):
    cfg = copy.deepcopy(CONFIGS["A"])
    change(cfg)
    with pytest.raises(ConfigError) as e:
        FisanexConfig.from_dict(cfg)
    assert key in str(e.value)


def test_plain_against_itself():
    cfg = CONFIGS["A"]
    w = random_weights(cfg, 3, sharpen=4.0)
    toks = random_tokens(70, cfg["vocab"], 1)
    whole = pf.forward(cfg, w, toks)
    scale = float(whole.abs().max())
    # causal: a prefix gives the same logits
    assert torch.allclose(pf.forward(cfg, w, toks[:23]), whole[:23], atol=1e-10)
    streams = []
    pf.forward(cfg, w, toks, layers_out=streams)
    assert len(streams) == 4

    def moved(other_cfg=None, other_w=None):
        return float((pf.forward(other_cfg or cfg, other_w or w, toks) - whole).abs().max()) / scale

    # a window wider than the sequence is every earlier key; one place more or less shows
    for i in range(4):
        for delta in (-1, 1):
            c = copy.deepcopy(cfg)
            c["layers"][i]["mixer"]["mask"]["size"] += delta
            assert moved(c) > 1e-3, (i, delta)
    # keys of its own instead of the earlier layer's
    c = copy.deepcopy(cfg)
    c["layers"][1]["mixer"].pop("kv_from")
    w2 = dict(w, **{"l1.mix.k": w["l0.mix.k"], "l1.mix.v": w["l0.mix.v"], "l1.mix.k.norm": w["l0.mix.k.norm"]})
    assert moved(c, w2) > 1e-3
    # the correction in the choice, the outputs that hand the input on, the shared expert, the gate, the factors
    assert moved(other_w=dict(w, **{"l1.mlp.correction": torch.zeros_like(w["l1.mlp.correction"])})) > 1e-3
    c = copy.deepcopy(cfg)
    c["layers"][1]["mlp"]["router"].update(experts=7, identity=0)
    w2 = dict(w, **{f"l1.mlp.e{e}.{n}": torch.zeros_like(w[f"l1.mlp.e0.{n}"]) for e in (5, 6) for n in ("gate", "up", "down")})
    assert moved(c, w2) > 1e-3
    c = copy.deepcopy(cfg)
    c["layers"][1]["mlp"].pop("shared")
    assert moved(c) > 1e-3
    assert moved(other_w=dict(w, **{"l0.mix.g": torch.zeros_like(w["l0.mix.g"])})) > 1e-3
    for key, value in (("postln_alpha", 1.0), ("logit_scale", 1.0)):
        assert moved(dict(cfg, **{key: value})) > 1e-3
    assert moved(dict(cfg, embedding={"scale": 1.0})) > 1e-6          # (only eps sees a factor on what is normed next)
    # the weights are the scores, not renormalised: with every output taken they sum to one
    chosen, weight = pf.route(torch.randn(9, 64, dtype=torch.float64), {k: v.double() for k, v in random_weights(CONFIGS["B"], 1).items()},
                              "l0.mlp.", 4)
    assert torch.allclose(weight.sum(-1), torch.ones(9, dtype=torch.float64)) and sorted(chosen[0].tolist()) == [0, 1, 2, 3]
