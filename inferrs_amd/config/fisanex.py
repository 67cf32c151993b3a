"""Configuration of the Fisanex decoder, read from its config.json.

config.json describes the model layer by layer:

    "architecture": "Fisanex", "vocab", "width", "norm": {"eps"}, "postln_alpha", "embedding": {"scale"}, "logit_scale",
    "layers": [{"type": "attention", "mixer": {...}, "mlp": {...} | null}, ...]

    mixer: heads, kv_heads, dim, vdim, scale, mask: {size}, rot: {base, dims}, and optionally kv_from: j (the layer has no
           keys and values of its own and reads those that layer j cached)
    mlp:   {"kind": "dense", "ff"}
           {"kind": "moe", "router": {experts, identity, top}, "expert": {ff, limit}, "shared": {ff, limit} | absent}

Every size and every constant that differs from model to model comes from there; what the design fixes (the norm after
every sum, the softmax router whose correction counts in the choice only and whose weights are not renormalised, the
experts' slope 1.702, the sigmoid gate on the joined heads, the logits through the embedding's own table) stands in
`to_spec`.  Tensor names: "embed", "final.norm", and for layer i "l<i>.norm1|norm2", "l<i>.mix.q|k|v|g|o|q.norm|k.norm",
"l<i>.mlp.gate|up|down" or "l<i>.mlp.router|correction|e<j>.gate|up|down|shared.gate|up|down".
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

from .base import ConfigError
from .buketar import _int, _num
from .spec import (AttentionSpec, ClampedMlpSpec, EmbeddingSpec, GatedMlpSpec, HeadSpec, LayerSpec, ModelSpec, NormSpec,
                   PositionSpec, PostNormSpec, RoutedExpertsSpec, ScheduleEntry)

DEFAULT_MAX_POSITION = 1 << 17
EXPERT_SLOPE = 1.702                # an expert's activation is g * sigmoid(1.702 g)

# the mixer's tensors as the attention part names them -> as the file names them
MIXER_NAMES = (("q_proj.weight", "q"), ("k_proj.weight", "k"), ("v_proj.weight", "v"), ("g_proj.weight", "g"),
               ("o_proj.weight", "o"), ("q_norm.weight", "q.norm"), ("k_norm.weight", "k.norm"))
DENSE_NAMES = (("gate_proj.weight", "gate"), ("up_proj.weight", "up"), ("down_proj.weight", "down"))


@dataclass(frozen=True)
class FisanexConfig:
    raw: Any                        # config.json as read (a dictionary), checked by `from_dict`

    architecture = "Fisanex"
    model_type = "fisanex"
    chat_template = None

    # ---- reading ----------------------------------------------------------------------------
    @classmethod
    def from_dict(cls, raw: Dict[str, Any], allow_ignored_keys: bool = False) -> "FisanexConfig":
        cfg = cls(copy.deepcopy(raw))
        cfg.to_spec()                # every key is read and checked there
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        out = copy.deepcopy(self.raw)
        out.setdefault("architecture", self.architecture)
        return out

    @property
    def vocab_size(self) -> int:
        return _int(self.raw, "vocab", "")

    @property
    def hidden_size(self) -> int:
        return _int(self.raw, "width", "")

    @property
    def eos_token_ids(self) -> Tuple[int, ...]:
        return ()

    # ---- the model as data --------------------------------------------------------------------
    def _sources(self) -> List[Optional[int]]:
        """For every layer the layer whose cache it reads (None: its own)."""
        layers = self.raw.get("layers") or []
        out: List[Optional[int]] = []
        for i, layer in enumerate(layers):
            m = layer.get("mixer") if isinstance(layer, dict) else None
            src = m.get("kv_from") if isinstance(m, dict) else None
            if src is not None:
                where = f"layers[{i}].mixer"
                src = _int(m, "kv_from", where, 0)
                if src >= i:
                    raise ConfigError(f"config.json: '{where}.kv_from' = {src} must name an earlier layer")
                if out[src] is not None:
                    raise ConfigError(f"config.json: '{where}.kv_from' = {src} names a layer that has no keys and values of its own")
            out.append(src)
        return out

    @staticmethod
    def _window(m: Dict[str, Any], where: str) -> Optional[int]:
        mask = m.get("mask") or {}
        return _int(mask, "size", where + ".mask") if mask else None

    def _mixer(self, i: int, layer: Dict[str, Any], hidden: int, eps: float, sources: List[Optional[int]]) -> AttentionSpec:
        where = f"layers[{i}].mixer"
        kind, m = layer.get("type"), layer.get("mixer")
        if kind != "attention":
            raise ConfigError(f"config.json: layers[{i}].type = {kind!r} is no mixer of this design (known: 'attention')")
        if not isinstance(m, dict):
            raise ConfigError(f"config.json: '{where}' must be an object")
        dim = _int(m, "dim", where)
        vdim = _int(m, "vdim", where) if m.get("vdim") is not None else dim
        heads, kv_heads = _int(m, "heads", where), _int(m, "kv_heads", where)
        if heads % kv_heads:
            raise ConfigError(f"config.json: '{where}.heads' = {heads} is no multiple of 'kv_heads' = {kv_heads}")
        rot = m.get("rot") or {}
        turned = _int(rot, "dims", where + ".rot", 0) if rot else 0
        if turned > dim or turned % 2:
            raise ConfigError(f"config.json: '{where}.rot.dims' = {turned} must be even and within dim {dim}")
        position = (PositionSpec("rope", head_dim=dim, rot_dim=turned, theta=_num(rot, "base", where + ".rot"), pairing="half")
                    if turned else PositionSpec("none"))
        layers = self.raw["layers"]
        if sources[i] is not None:
            owner = layers[sources[i]].get("mixer") or {}
            for key in ("kv_heads", "dim", "vdim"):
                if owner.get(key, dim if key == "vdim" else None) != m.get(key, dim if key == "vdim" else None):
                    raise ConfigError(f"config.json: '{where}.{key}' differs from layer {sources[i]}'s, whose keys and values it reads")
        readers = tuple(self._window(layers[j]["mixer"], f"layers[{j}].mixer") for j, src in enumerate(sources) if src == i)
        return AttentionSpec(hidden=hidden, n_heads=heads, n_kv_heads=kv_heads, head_dim=dim, position=position,
                             qk_norm=NormSpec(dim, eps), window=self._window(m, where), scale=_num(m, "scale", where),
                             names=MIXER_NAMES, v_head_dim=vdim, gate=True, own_kv=sources[i] is None,
                             reader_windows=readers)

    def _mlp(self, i: int, layer: Dict[str, Any], hidden: int):
        f = layer.get("mlp")
        if f is None:
            return None
        where = f"layers[{i}].mlp"
        if not isinstance(f, dict):
            raise ConfigError(f"config.json: '{where}' must be an object or null")
        if f.get("kind") == "dense":
            return GatedMlpSpec(hidden=hidden, intermediate=_int(f, "ff", where), activation="silu", names=DENSE_NAMES)
        if f.get("kind") == "moe":
            expert, router = f.get("expert"), f.get("router")
            if not isinstance(expert, dict) or not isinstance(router, dict):
                raise ConfigError(f"config.json: '{where}' needs the objects 'router' and 'expert'")
            experts, top = _int(router, "experts", where + ".router"), _int(router, "top", where + ".router")
            identity = _int(router, "identity", where + ".router", 0) if router.get("identity") is not None else 0
            if top > experts + identity:
                raise ConfigError(f"config.json: '{where}.router.top' = {top} exceeds the router's {experts + identity} outputs")
            shared = f.get("shared")
            if shared is not None and not isinstance(shared, dict):
                raise ConfigError(f"config.json: '{where}.shared' must be an object or null")
            return RoutedExpertsSpec(
                hidden=hidden, intermediate=_int(expert, "ff", where + ".expert"), experts=experts, top=top, scale=1.0,
                limit=_num(expert, "limit", where + ".expert"), alpha=EXPERT_SLOPE, score="softmax", renormalize=False,
                identity=identity, correction=True,
                shared=None if shared is None else ClampedMlpSpec(hidden, _int(shared, "ff", where + ".shared"),
                                                                   _num(shared, "limit", where + ".shared"), EXPERT_SLOPE))
        raise ConfigError(f"config.json: '{where}.kind' = {f.get('kind')!r} is no feed-forward of this design "
                          "(known: 'dense', 'moe')")

    def to_spec(self) -> ModelSpec:
        raw = self.raw
        if not isinstance(raw, dict):
            raise ConfigError("config.json must hold an object")
        vocab, hidden = self.vocab_size, self.hidden_size
        eps = _num(raw.get("norm"), "eps", "norm")
        alpha = _num(raw, "postln_alpha", "")
        embed_scale = _num(raw.get("embedding"), "scale", "embedding")
        logit_scale = _num(raw, "logit_scale", "")
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        for i, layer in enumerate(layers_raw):
            if not isinstance(layer, dict):
                raise ConfigError(f"config.json: layers[{i}] must be an object")
        sources = self._sources()
        norm = NormSpec(hidden, eps)
        layers = []
        for i, layer in enumerate(layers_raw):
            p = f"l{i}."
            ffn = self._mlp(i, layer, hidden)
            names = (p + "norm1",) + ((p + "norm2",) if ffn is not None else ())
            layers.append(LayerSpec(mixer=self._mixer(i, layer, hidden, eps, sources), ffn=ffn, norms=(norm,) * len(names),
                                    norm_names=names, mixer_prefix=p + "mix.", ffn_prefix=p + "mlp.",
                                    arrangement="post_norm",
                                    residual=PostNormSpec(alpha, bare_norm_name=None if ffn is not None else p + "norm2")))
        max_position = int(raw.get("max_position") or DEFAULT_MAX_POSITION)
        return ModelSpec(
            architecture=self.architecture, vocab_size=vocab, hidden=hidden, layers=tuple(layers),
            schedule=tuple(ScheduleEntry(i, cache_of=sources[i]) for i in range(len(layers))),
            final_norm=norm, final_norm_name="final.norm", embed_name="embed", head_name=None,
            max_position=max_position, head_required=False, eos_token_ids=(),
            embedding=EmbeddingSpec(vocab, hidden, "embed", scale=embed_scale, wide=True),
            head=HeadSpec(vocab, hidden, None, required=False, scale=logit_scale))
