"""Random Ligizen configurations through the engine against the plain implementation: both mixers in any order, layers
that read an earlier layer's keys and values (with chunks of their own), layers without feed-forward, query and key head
counts, key and value sizes in and out of those the matrix-core attention takes (16 to 256 in steps of 16, values of a
width of their own), latent rows whose width fits it or not, chunks and windows from 1 to longer than any request, whole
heads turning, parts of them or nothing, stretched frequencies or none, dense feed-forwards and routed experts with one
expert a token up to all of them, with and without a shared expert, with and without a token's own input, with and without
a cap on the logits, widths from odd ones to those whose products run on the kernels for many rows, vocabularies of any
size.  Every configuration runs whole prompts, a prompt and then token by token, and a mixed schedule (four live requests,
pages and slots used again) in 32-bit (2e-5 of the largest logit at every position, or three times what the plain
implementation's own 32-bit arithmetic is off there) and in bfloat16 (the distribution of the errors against the plain
implementation's in bfloat16 arithmetic, as in `test_ligizen_gpu.py`)."""
import io
import random

import numpy as np
import pytest
import torch

import plain_ligizen as pl
import trace_modes as tm
from ligizen_configs import attn, dense, latent, layer, model, moe, random_tokens, write_model

pytestmark = pytest.mark.gpu

LENGTHS = [1, 2, 19, 64, 150, 260]


def random_attention(rng: random.Random, sharp: float):
    kv = rng.choice([1, 1, 2, 3])
    dim = rng.choice([16, 32, 48, 64, 128]) if rng.random() < 0.6 else rng.choice([8, 12, 24, 40, 80, 96])
    # (of the pairs of widths that the matrix cores take, those that are built beside the package: another pair would be
    # compiled inside the test)
    from inferrs_amd.ops.build import ATTN_VALUE_PAIRS
    widths = [v for v in (8, 16, 20, 32, 48, 64, 256) if v % 16 or dim % 16 or (dim, v) in ATTN_VALUE_PAIRS]
    vdim = dim if rng.random() < 0.5 else rng.choice(widths)
    turned = rng.choice([dim, dim, dim // 2 // 2 * 2, 0])
    scaling = None
    if turned and rng.random() < 0.6:
        scaling = (rng.choice([2.0, 4.0, 8.0]), rng.choice([0.5, 1.0]), rng.choice([2.0, 4.0]), rng.choice([32, 64, 512]))
    return attn(kv * rng.choice([1, 2, 4, 6]), kv, dim, vdim, sharp * rng.choice([0.05, 0.125, 0.3]), rng.choice([1, 7, 16, 33, 64, 80, 100, 1000]),
                base=rng.choice([100.0, 10000.0, 500000.0]), turned=max(turned, 0), scaling=scaling)


def random_latent(rng: random.Random, sharp: float):
    rot_dim = rng.choice([4, 8, 16, 32])
    rank = rng.choice([12, 24, 48 - rot_dim, 64 - rot_dim, 128 - rot_dim, 96]) if rng.random() < 0.7 else rng.choice([10, 30, 50])
    return latent(rng.choice([1, 2, 3, 6, 8]), rng.choice([8, 10, 16, 32]), rot_dim, rng.choice([4, 8, 14, 16, 32]),
                  rng.choice([8, 16, 24, 40]), max(rank, 4), sharp * rng.choice([0.08, 0.125, 0.3]),
                  rng.choice([1, 7, 16, 33, 64, 80, 100, 1000]), base=rng.choice([100.0, 10000.0, 200000.0]))


def random_mlp(rng: random.Random, big: bool):
    r = rng.random()
    if r < 0.15:
        return None
    if r < 0.45:
        return dense(rng.choice([64, 128, 512]) if big else rng.choice([10, 16, 24, 40]))
    experts = rng.choice([1, 2, 3, 5, 8, 12, 40])
    top = rng.choice([1, 1, 2, min(experts, 4), experts if experts <= 8 else 3])
    shared = (rng.choice([8, 24, 40, 128]), rng.choice([0.8, 2.0, 7.0])) if rng.random() < 0.6 else None
    return moe(experts, min(top, experts), rng.choice([8, 16, 30, 64]), rng.choice([1.0, 1.5, 7.0]), shared=shared)


def random_config(rng: random.Random, sharp: float) -> dict:
    big = rng.random() < 0.35
    width = rng.choice([128, 256, 384]) if big else rng.choice([24, 33, 40, 50, 64, 72, 96])
    layers = []
    for i in range(rng.randint(1, 5)):
        owners = [j for j, L in enumerate(layers) if L["type"] == "attention" and L["mixer"].get("kv_from") is None]
        if owners and rng.random() < 0.35:
            j = rng.choice(owners)
            m = {"type": "attention", "mixer": dict(layers[j]["mixer"], kv_from=j, scale=sharp * rng.choice([0.1, 0.2]),
                                                    mask={"size": rng.choice([1, 5, 24, 64, 80, 300])})}
            m["mixer"]["heads"] = layers[j]["mixer"]["kv_heads"] * rng.choice([1, 2, 3])
        else:
            m = random_attention(rng, sharp) if rng.random() < 0.5 else random_latent(rng, sharp)
        layers.append(layer(m, random_mlp(rng, big)))
    return model(rng.choice([31, 64, 100, 257, 576]), width, layers, eps=rng.choice([1e-6, 1e-5]),
                 embed_scale=rng.choice([1.0, 3.0, 17.0]), cap=rng.choice([None, 5.0, 12.0, 30.0]),
                 side=rng.choice([None, 4, 6, 20]))


def run(folder, cfg, dtype, trace, out_dir):
    from inferrs_amd.engine import Engine, run_trace
    eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=-(-trace.max_tokens // 16), max_seqs=4)
    run_trace(eng, trace.lines, out_dir, io.StringIO())
    eng.cache.check_invariants()
    assert not eng.cache.sequences and eng.cache.slots.num_free == eng.cache.slots.num_slots
    return trace.read(out_dir, cfg["vocab"])


def errors(got, ref, reqs):
    scale = max(float(np.abs(v).max()) for v in ref.values())
    return np.concatenate([[float(np.abs(got[r][p] - ref[r][p]).max()) / scale for p in range(len(t))] for r, t in reqs.items()])


@pytest.mark.parametrize("seed", range(24))
def test_random_configuration(tmp_path, seed):
    rng = random.Random(9000 + seed)
    cfg = random_config(rng, rng.choice([1.0, 1.0, 4.0]))
    if cfg["logit_softcap"] is None:
        del cfg["logit_softcap"]
    tensors = write_model(str(tmp_path / "model"), cfg, seed=seed)
    folder = str(tmp_path / "model")
    reqs = {f"r{i}": random_tokens(n, cfg["vocab"], 70 + i) for i, n in enumerate(LENGTHS)}
    ref64 = {r: pl.forward(cfg, tensors, t) for r, t in reqs.items()}
    ref = {r: v.numpy().astype(np.float32) for r, v in ref64.items()}
    noise = errors({r: pl.forward(cfg, tensors, t, dtype=torch.float32).double().numpy() for r, t in reqs.items()},
                   {r: v.numpy() for r, v in ref64.items()}, reqs)
    rounded = {r: pl.forward(cfg, tensors, t, dtype=torch.bfloat16).float().numpy() for r, t in reqs.items()}
    theirs = errors(rounded, ref, reqs)
    for mode, trace in (("whole", tm.whole(reqs)), ("tail", tm.prefix_then_single(reqs, 40)), ("mixed", tm.mixed(reqs, seed=seed))):
        got = run(folder, cfg, "float32", trace, str(tmp_path / f"{mode}_f32"))
        err = errors(got, ref, reqs)
        assert (err <= np.maximum(2e-5, 3.0 * noise)).all(), \
            f"seed {seed} {mode} float32: {err.max():.3g} of the scale (the plain 32-bit arithmetic: {noise.max():.3g}); {cfg}"
        got = run(folder, cfg, "bfloat16", trace, str(tmp_path / f"{mode}_bf16"))
        mine = errors(got, ref, reqs)
        assert np.isfinite(mine).all(), f"seed {seed} {mode} bfloat16: not finite; {cfg}"
        for q, slack in ((0.5, 1.1), (0.9, 1.5)):
            a, b = float(np.quantile(mine, q)), float(np.quantile(theirs, q))
            assert a <= slack * b + 1e-3, f"seed {seed} {mode} bfloat16: quantile {q} of the errors {a:.3g}, plain in bfloat16 {b:.3g}; {cfg}"
