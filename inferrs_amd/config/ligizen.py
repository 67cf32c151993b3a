"""Configuration of the Ligizen decoder, read from its config.json.

config.json describes the model layer by layer:

    "architecture": "Ligizen", "vocab", "width", "norm": {"eps"}, "embedding": {"scale"}, "logit_softcap",
    "token_side": {"dim"} | absent, "layers": [{"type", "mixer": {...}, "mlp": {...} | null}, ...]

    type "attention":        heads, kv_heads, dim, vdim, scale, mask: {size} (chunks), rot: {base, dims, scaling:
                             {factor, low, high, original} | absent}, and optionally kv_from: j (the layer has no keys and
                             values of its own and reads those that layer j cached)
    type "latent_attention": heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, mask: {size} (a window), rot: {base, dims}
    mlp:   {"kind": "dense", "ff"}
           {"kind": "moe", "router": {experts, top}, "expert": {ff, limit}, "shared": {ff, limit} | absent}

Every size and every constant that differs from model to model comes from there; what the design fixes stands in
`to_spec`: one layer norm (weight and bias) a layer whose output both sub-layers read, their outputs added together; the
token's own input behind the sum (GELU in its tanh form, an RMS norm with a weight); in "attention" biases on q, k and v,
halves paired in the turn, q and k at unit root mean square a head, chunks, one sigmoid gate a head; in
"latent_attention" neighbours paired in the turn, a window, a learned term a head in the softmax's denominator, one
sigmoid gate a head; a sigmoid router whose weights multiply the experts' inputs and are not renormalised, the experts'
slope 1.702, a shared expert behind a sigmoid gate a token; logits through a matrix of their own, capped by a tanh.
Tensor names: "embed", "side.embed", "final.norm", "final.norm.b", "head", and for layer i "l<i>.norm1", "l<i>.norm1.b",
"l<i>.mix.q|k|v (+ .b)|g|o" or "l<i>.mix.dq|dq.norm|uq|dkv|dkv.norm|uk|uv|sink|g|o", "l<i>.mlp.gate|up|down" or
"l<i>.mlp.router|e<j>.gate|up|down|shared.gate|up|down|sg", "l<i>.side.gate|proj|norm".
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

from .base import ConfigError
from .buketar import _int, _num
from .spec import (AttentionSpec, CappedHeadSpec, ClampedMlpSpec, EmbeddingSpec, GatedMlpSpec, LatentAttentionSpec,
                   LayerNormSpec, LayerSpec, ModelSpec, NormSpec, ParallelSpec, PositionSpec, RoutedExpertsSpec,
                   ScheduleEntry, TokenSideSpec)

DEFAULT_MAX_POSITION = 1 << 17
EXPERT_SLOPE = 1.702                # an expert's activation is g * sigmoid(1.702 g)

# the mixer's tensors as the attention part names them -> as the file names them
ATTENTION_NAMES = (("q_proj.weight", "q"), ("k_proj.weight", "k"), ("v_proj.weight", "v"), ("g_proj.weight", "g"),
                   ("o_proj.weight", "o"), ("q_proj.bias", "q.b"), ("k_proj.bias", "k.b"), ("v_proj.bias", "v.b"))
DENSE_NAMES = (("gate_proj.weight", "gate"), ("up_proj.weight", "up"), ("down_proj.weight", "down"))
MIXERS = ("attention", "latent_attention")


@dataclass(frozen=True)
class LigizenConfig:
    raw: Any                        # config.json as read (a dictionary), checked by `from_dict`

    architecture = "Ligizen"
    model_type = "ligizen"
    chat_template = None

    # ---- reading ----------------------------------------------------------------------------
    @classmethod
    def from_dict(cls, raw: Dict[str, Any], allow_ignored_keys: bool = False) -> "LigizenConfig":
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
                if layer.get("type") != "attention":
                    raise ConfigError(f"config.json: '{where}.kv_from' goes with the mixer 'attention'")
                src = _int(m, "kv_from", where, 0)
                if src >= i:
                    raise ConfigError(f"config.json: '{where}.kv_from' = {src} must name an earlier layer")
                if out[src] is not None or layers[src].get("type") != "attention":
                    raise ConfigError(f"config.json: '{where}.kv_from' = {src} names a layer that has no keys and values "
                                      "of this kind of its own")
            out.append(src)
        return out

    @staticmethod
    def _mask(m: Dict[str, Any], where: str) -> int:
        mask = m.get("mask")
        if not isinstance(mask, dict):
            raise ConfigError(f"config.json: '{where}.mask' must be an object with 'size'")
        return _int(mask, "size", where + ".mask")

    @staticmethod
    def _rotation(rot: Any, where: str, head_dim: int, pairing: str) -> PositionSpec:
        if not rot:
            return PositionSpec("none")
        if not isinstance(rot, dict):
            raise ConfigError(f"config.json: '{where}' must be an object")
        turned = _int(rot, "dims", where, 0)
        if turned == 0:
            return PositionSpec("none")
        if turned > head_dim or turned % 2:
            raise ConfigError(f"config.json: '{where}.dims' = {turned} must be even and within {head_dim}")
        scaling = None
        sc = rot.get("scaling")
        if sc is not None:
            if not isinstance(sc, dict):
                raise ConfigError(f"config.json: '{where}.scaling' must be an object or absent")
            w = where + ".scaling"
            scaling = ("llama3", _num(sc, "factor", w), _num(sc, "low", w), _num(sc, "high", w), _num(sc, "original", w))
            if not (scaling[1] > 0 and scaling[3] > scaling[2] and scaling[4] > 0):
                raise ConfigError(f"config.json: '{w}' needs factor > 0, high > low and original > 0")
        return PositionSpec("rope", head_dim=head_dim, rot_dim=turned, theta=_num(rot, "base", where), pairing=pairing,
                            scaling=scaling)

    def _attention(self, i: int, m: Dict[str, Any], hidden: int, eps: float, sources: List[Optional[int]]) -> AttentionSpec:
        where = f"layers[{i}].mixer"
        dim = _int(m, "dim", where)
        vdim = _int(m, "vdim", where) if m.get("vdim") is not None else dim
        heads, kv_heads = _int(m, "heads", where), _int(m, "kv_heads", where)
        if heads % kv_heads:
            raise ConfigError(f"config.json: '{where}.heads' = {heads} is no multiple of 'kv_heads' = {kv_heads}")
        layers = self.raw["layers"]
        if sources[i] is not None:
            owner = layers[sources[i]].get("mixer") or {}
            for key in ("kv_heads", "dim", "vdim", "rot"):
                if owner.get(key, dim if key == "vdim" else None) != m.get(key, dim if key == "vdim" else None):
                    raise ConfigError(f"config.json: '{where}.{key}' differs from layer {sources[i]}'s, whose keys and "
                                      "values it reads")
        return AttentionSpec(hidden=hidden, n_heads=heads, n_kv_heads=kv_heads, head_dim=dim,
                             position=self._rotation(m.get("rot"), where + ".rot", dim, "half"),
                             qk_norm=NormSpec(dim, eps), qk_unit_norm=True, scale=_num(m, "scale", where), qkv_bias=True,
                             names=ATTENTION_NAMES, v_head_dim=vdim, gate=True, gate_per_head=True,
                             own_kv=sources[i] is None, mask_chunk=self._mask(m, where))

    def _latent(self, i: int, m: Dict[str, Any], hidden: int, eps: float) -> LatentAttentionSpec:
        where = f"layers[{i}].mixer"
        rot_dim = _int(m, "rot_dim", where)
        position = self._rotation(m.get("rot"), where + ".rot", rot_dim, "interleaved")
        return LatentAttentionSpec(hidden=hidden, n_heads=_int(m, "heads", where), head_dim=_int(m, "dim", where),
                                   rot_dim=rot_dim, v_dim=_int(m, "vdim", where), kv_rank=_int(m, "kv_rank", where),
                                   position=position, scale=_num(m, "scale", where), norm_eps=eps, gate=True,
                                   window=self._mask(m, where), q_rank=_int(m, "q_rank", where), sink=True,
                                   gate_per_head=True)

    def _mixer(self, i: int, layer: Dict[str, Any], hidden: int, eps: float, sources: List[Optional[int]]):
        kind, m = layer.get("type"), layer.get("mixer")
        if kind not in MIXERS:
            raise ConfigError(f"config.json: layers[{i}].type = {kind!r} is no mixer of this design (known: {list(MIXERS)})")
        if not isinstance(m, dict):
            raise ConfigError(f"config.json: 'layers[{i}].mixer' must be an object")
        return self._attention(i, m, hidden, eps, sources) if kind == "attention" else self._latent(i, m, hidden, eps)

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
            if top > experts:
                raise ConfigError(f"config.json: '{where}.router.top' = {top} exceeds the router's {experts} experts")
            shared = f.get("shared")
            if shared is not None and not isinstance(shared, dict):
                raise ConfigError(f"config.json: '{where}.shared' must be an object or null")
            return RoutedExpertsSpec(
                hidden=hidden, intermediate=_int(expert, "ff", where + ".expert"), experts=experts, top=top, scale=1.0,
                limit=_num(expert, "limit", where + ".expert"), alpha=EXPERT_SLOPE, score="sigmoid", renormalize=False,
                weight_on_input=True, shared_gate=shared is not None,
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
        embed_scale = _num(raw.get("embedding"), "scale", "embedding")
        cap = _num(raw, "logit_softcap", "") if raw.get("logit_softcap") is not None else None
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        for i, layer in enumerate(layers_raw):
            if not isinstance(layer, dict):
                raise ConfigError(f"config.json: layers[{i}] must be an object")
        side = raw.get("token_side")
        if side is not None and not isinstance(side, dict):
            raise ConfigError("config.json: 'token_side' must be an object or absent")
        side_dim = _int(side, "dim", "token_side") if side is not None else 0
        sources = self._sources()
        norm = LayerNormSpec(hidden, eps)
        layers = []
        for i, layer in enumerate(layers_raw):
            p = f"l{i}."
            residual = ParallelSpec(side=TokenSideSpec(side_dim, i * side_dim, p + "side.", eps) if side_dim else None)
            layers.append(LayerSpec(mixer=self._mixer(i, layer, hidden, eps, sources), ffn=self._mlp(i, layer, hidden),
                                    norms=(norm,), norm_names=(p + "norm1",), mixer_prefix=p + "mix.",
                                    ffn_prefix=p + "mlp.", arrangement="parallel", residual=residual))
        max_position = int(raw.get("max_position") or DEFAULT_MAX_POSITION)
        return ModelSpec(
            architecture=self.architecture, vocab_size=vocab, hidden=hidden, layers=tuple(layers),
            schedule=tuple(ScheduleEntry(i, cache_of=sources[i]) for i in range(len(layers))),
            final_norm=norm, final_norm_name="final.norm", embed_name="embed", head_name="head",
            max_position=max_position, head_required=True, eos_token_ids=(),
            embedding=EmbeddingSpec(vocab, hidden, "embed", scale=embed_scale, wide=True,
                                    side_name="side.embed" if side_dim else None, side_width=side_dim * len(layers)),
            head=CappedHeadSpec(vocab, hidden, "head", cap=cap, required=True))
