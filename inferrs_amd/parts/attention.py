"""Grouped-query attention over the paged cache.

Order of operations as in the reference (`inferrs-models/src/models/qwen3.rs:105-195`):
q, k, v projections without bias; per-head RMS norm of q and k; rotation of q and k by
position; append of k and v to the cache; scores (q.k)/sqrt(d) against keys at positions
<= the query's (and inside the window, when one is set); softmax; weighted sum of values;
output projection.  q head h reads kv head h // (n_heads / n_kv_heads)
(`attention_utils.rs:38-49`).

Options of the spec beyond the reference's layer: biases, a window, a sink in the softmax (`sink`: the denominator
holds one more term, exp(0)), values that are the key projection's own rows, ahead of norm and rotation (`values_from_keys`: no
value projection is loaded; the key projection's rows stand twice in the fused product, so the kernels that take
[q | k | v] serve unchanged), and other names for the tensors in the file (`names`).  Further: values of a width of
their own (`v_head_dim`: the cache's value array, the heads' outputs and the output projection's input are that wide), a
sigmoid gate on the joined heads (`gate`: sigmoid(W_g h), one product with the projections), and a layer without keys and
values of its own (`own_kv` False: its stop of the schedule reads another stop's cache, after that layer's norm and
rotation, with its own queries, window and scale).  Such a layer's rows are [q | k | v | g], whatever of these it has, and
go through the kernels that take rows of any layout.  Further still: a mask of chunks instead of a window (`mask_chunk`:
a query sees the keys of its own chunk of that many positions, up to itself; every attention kernel takes it beside the
window), one gate value a head instead of one a feature (`gate_per_head`), and q and k at unit root mean square a head
without a learned weight (`qk_unit_norm`: the norm kernels run with a weight of ones; a turn by position keeps a head's
sum of squares, so it does not matter on which side of the turn the norm stands).
"""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.spec import AttentionSpec, SpecError
from ..weights.loader import TensorSpec
from .base import Mixer, PagedKV, part_class, register_mixer
from .linear import Linear


@register_mixer("attention")
class Attention(Mixer):
    graph_safe = True
    takes_normed_rows = True      # the q|k|v product norms the rows it is given as `ops.NormedRows`
    adds_to_stream = True         # the output projection adds itself to `ctx.stream` where it can

    @classmethod
    def tensors(cls, spec: AttentionSpec) -> Dict[str, TensorSpec]:
        named = dict(spec.names or ())
        t = cls._tensors(spec)
        if spec.values_from_keys:
            t = {k: v for k, v in t.items() if not k.startswith("v_proj.")}
        if not spec.own_kv:
            t = {k: v for k, v in t.items() if not k.startswith(("k_proj.", "v_proj.", "k_norm."))}
        return {named.get(k, k): v for k, v in t.items()}

    @classmethod
    def _tensors(cls, spec: AttentionSpec) -> Dict[str, TensorSpec]:
        q_out, kv_out = spec.n_heads * spec.head_dim, spec.n_kv_heads * spec.head_dim
        t = {
            "q_proj.weight": TensorSpec((q_out, spec.hidden)),
            "k_proj.weight": TensorSpec((kv_out, spec.hidden)),
            "v_proj.weight": TensorSpec((spec.n_kv_heads * spec.value_dim, spec.hidden)),
            "o_proj.weight": TensorSpec((spec.hidden, spec.n_heads * spec.value_dim)),
        }
        if spec.gate:
            t["g_proj.weight"] = TensorSpec((spec.n_heads * (1 if spec.gate_per_head else spec.value_dim), spec.hidden))
        if spec.qk_norm is not None and not spec.qk_unit_norm:
            t["q_norm.weight"] = TensorSpec((spec.head_dim,), "norm")
            t["k_norm.weight"] = TensorSpec((spec.head_dim,), "norm")
        if spec.qkv_bias:
            t["q_proj.bias"] = TensorSpec((q_out,))
            t["k_proj.bias"] = TensorSpec((kv_out,))
            t["v_proj.bias"] = TensorSpec((spec.n_kv_heads * spec.value_dim,))
        if spec.o_bias:
            t["o_proj.bias"] = TensorSpec((spec.hidden,))
        return t

    @classmethod
    def cache_need(cls, spec: AttentionSpec):
        if not spec.own_kv:
            return None
        return PagedKV(spec.n_kv_heads, spec.head_dim, spec.kept_window,
                       v_head_dim=spec.value_dim if spec.value_dim != spec.head_dim else None)

    def __init__(self, spec: AttentionSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        if spec.n_heads % spec.n_kv_heads:
            raise SpecError(f"attention: {spec.n_heads} heads are not a multiple of {spec.n_kv_heads} kv heads")
        # (the matrix-core kernels take head sizes in steps of 16 up to 256 in bfloat16; every other size, and the
        # 32-bit path, runs on the plain kernels, which take any size up to 512)
        if not (1 <= spec.head_dim <= 512):
            raise SpecError(f"attention: head_dim {spec.head_dim} is outside 1..512, the range of the attention kernels")
        rot = getattr(spec.position, "rot_dim", 0) if getattr(spec.position, "kind", "none") != "none" else 0
        if rot % 2 or rot > spec.head_dim:
            raise SpecError(f"attention: the rotated part of a head ({rot}) must be even and within head_dim {spec.head_dim}")
        if spec.window is not None and spec.window < 1:
            raise SpecError(f"attention: window {spec.window} must be >= 1")
        if spec.mask_chunk is not None and spec.mask_chunk < 1:
            raise SpecError(f"attention: mask_chunk {spec.mask_chunk} must be >= 1")
        if spec.qk_unit_norm and spec.qk_norm is None:
            raise SpecError("attention: qk_unit_norm takes size and eps from qk_norm")
        if spec.qk_norm is not None and spec.qk_norm.size != spec.head_dim:
            raise SpecError("attention: qk_norm must span head_dim")
        if not (1 <= spec.value_dim <= 512):
            raise SpecError(f"attention: v_head_dim {spec.value_dim} is outside 1..512, the range of the attention kernels")
        if spec.values_from_keys and (spec.value_dim != spec.head_dim or not spec.own_kv):
            raise SpecError("attention: values that are the keys have the keys' width and a key projection to come from")
        self.spec = spec
        named = dict(spec.names or ())
        tensors = {k: tensors[named.get(k, k)] for k in self._tensors(spec) if named.get(k, k) in tensors}
        # rows of the plain layout [q | k | v], heads of one width, go through the kernels made for it; everything else
        # (a gate in the rows, values of another width, no keys at all) through those that take any layout
        self.plain = (spec.own_kv and not spec.gate and spec.value_dim == spec.head_dim and not spec.mask_chunk
                      and not spec.qk_unit_norm)
        if not self.plain:
            self._init_general(spec, tensors, dtype, device)
            return
        if spec.values_from_keys:
            tensors["v_proj.weight"] = tensors["k_proj.weight"]
            if spec.qkv_bias:
                tensors["v_proj.bias"] = tensors["k_proj.bias"]
        self.qkv = Linear([tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]], dtype, device,
                          [tensors["q_proj.bias"], tensors["k_proj.bias"], tensors["v_proj.bias"]] if spec.qkv_bias else None)
        self.o = Linear([tensors["o_proj.weight"]], dtype, device, [tensors["o_proj.bias"]] if spec.o_bias else None)
        if spec.qk_norm is not None:
            self.q_norm_w = tensors["q_norm.weight"].to(device=device, dtype=torch.float32).contiguous()
            self.k_norm_w = tensors["k_norm.weight"].to(device=device, dtype=torch.float32).contiguous()
            self.norm_eps, self.norm_add_one = float(spec.qk_norm.eps), bool(spec.qk_norm.add_one)
        else:
            self.q_norm_w = self.k_norm_w = None
            self.norm_eps, self.norm_add_one = 0.0, False
        self.position = part_class("position", spec.position)(spec.position, {}, dtype, device)
        if getattr(self.position, "magnitude", 1.0) != 1.0:
            raise SpecError("attention: a rotation law that scales cos and sin is not taken by this mixer's kernels")

    def _init_general(self, spec: AttentionSpec, tensors, dtype, device):
        H, G, d, dv = spec.n_heads, spec.n_kv_heads, spec.head_dim, spec.value_dim
        stacked, at = [tensors["q_proj.weight"]], H * d
        biases = [tensors["q_proj.bias"]] if spec.qkv_bias else None
        self.q_off, self.k_off, self.v_off, self.g_off = 0, None, None, None
        if spec.own_kv:
            stacked += [tensors["k_proj.weight"], tensors["v_proj.weight"]]
            if spec.qkv_bias:
                biases += [tensors["k_proj.bias"], tensors["v_proj.bias"]]
            self.k_off, self.v_off, at = at, at + G * d, at + G * d + G * dv
        if spec.gate:
            g_w = tensors["g_proj.weight"]
            g_rows = H * (1 if spec.gate_per_head else dv)
            if g_rows % 8:                           # (rows of zeros keep the fused product's pitch a multiple of 16 bytes,
                pad = 8 - g_rows % 8                 # which the kernels that walk its rows in 16-byte pieces ask for)
                g_w = torch.cat([g_w, torch.zeros((pad, g_w.shape[1]), dtype=g_w.dtype, device=g_w.device)], dim=0)
                g_rows += pad
            stacked.append(g_w)
            if spec.qkv_bias:                        # (the gate has no bias: zeros keep the one fused product)
                biases.append(torch.zeros((g_rows,), dtype=tensors["q_proj.bias"].dtype))
            self.g_off, at = at, at + g_rows
        self.qkv = Linear(stacked, dtype, device, biases)
        self.o = Linear([tensors["o_proj.weight"]], dtype, device, [tensors["o_proj.bias"]] if spec.o_bias else None)
        self.q_norm_w = self.k_norm_w = None
        self.norm_eps, self.norm_add_one = 0.0, False
        if spec.qk_unit_norm:
            self.q_norm_w = self.k_norm_w = torch.ones((d,), dtype=torch.float32, device=device)
            self.norm_eps = float(spec.qk_norm.eps)
        elif spec.qk_norm is not None:
            self.q_norm_w = tensors["q_norm.weight"].to(device=device, dtype=torch.float32).contiguous()
            if spec.own_kv:
                self.k_norm_w = tensors["k_norm.weight"].to(device=device, dtype=torch.float32).contiguous()
            self.norm_eps, self.norm_add_one = float(spec.qk_norm.eps), bool(spec.qk_norm.add_one)
        self.position = part_class("position", spec.position)(spec.position, {}, dtype, device)
        if getattr(self.position, "magnitude", 1.0) != 1.0:
            raise SpecError("attention: a rotation law that scales cos and sin is not taken by this mixer's kernels")

    def _forward_general(self, ctx, h, cache):
        s = self.spec
        H, G, d, dv = s.n_heads, s.n_kv_heads, s.head_dim, s.value_dim
        group = ctx.groups[cache.group]
        if hasattr(h, "materialize"):
            h = h.materialize()
        proj = self.qkv(h)                                       # [n, q | k | v | g]
        table = ctx.position_table(self.position)
        cos, sin = table if table is not None else (None, None)
        writes = cache.writable and s.own_kv
        q = ops.qk_rope_kv_strided(
            proj, H, G, d, dv, q_off=self.q_off, k_off=self.k_off if writes else None, v_off=self.v_off,
            q_norm_w=self.q_norm_w, k_norm_w=self.k_norm_w, eps=self.norm_eps, add_one=self.norm_add_one, cos=cos, sin=sin,
            rot=self.position.rot_dim, interleaved=self.position.interleaved, k_cache=cache.k, v_cache=cache.v,
            slots=group.slots if writes else None, page_size=group.page_size)
        a = self._attend(ctx, q, cache, group)
        joined = a.view(a.shape[0], H * dv)
        if s.gate:
            ops.sigmoid_gate(joined, proj, self.g_off, group=dv if s.gate_per_head else 1)
        return self._project(ctx, joined)

    def _attend(self, ctx, q, cache, group):
        """The paged attention of the step's queries: the matrix cores where they take the sizes, else the plain kernel."""
        s = self.spec
        if ops.attention_mfma_fits(q.dtype, s.head_dim, group.page_size, s.value_dim):
            common = dict(window=s.window, scale=s.softmax_scale, sink=s.sink, mask_chunk=s.mask_chunk)
            if 0 < ctx.n_single < ctx.n_seqs:
                # single tokens (decode) and portions of prompts want different launches: the first
                # split their long key ranges between waves, the second have columns enough
                a = ops.attention_mfma(q, cache.k, cache.v, ctx.positions, ctx.cu_tokens, group.block_table,
                                       max_q_len=1, max_kv_len=ctx.max_kv_single, seqs=(0, ctx.n_single),
                                       tokens=(0, ctx.n_single), **common)
                ops.attention_mfma(q, cache.k, cache.v, ctx.positions, ctx.cu_tokens, group.block_table,
                                   max_q_len=ctx.max_q_len, max_kv_len=ctx.max_kv_multi,
                                   seqs=(ctx.n_single, ctx.n_seqs - ctx.n_single),
                                   tokens=(ctx.n_single, ctx.n_tokens - ctx.n_single), out=a, **common)
                return a
            return ops.attention_mfma(q, cache.k, cache.v, ctx.positions, ctx.cu_tokens, group.block_table,
                                      max_q_len=ctx.max_q_len, max_kv_len=ctx.max_kv_len, **common)
        return ops.attention_generic(q, cache.k, cache.v, ctx.positions, ctx.token_seq, group.block_table,
                                     window=s.window, scale=s.softmax_scale, max_kv_len=ctx.max_kv_len, sink=s.sink,
                                     mask_chunk=s.mask_chunk)

    def load_notes(self, page_size: int):
        """What the log should say once when a model with this part is set up: a decode step that cannot take the
        fused kernel still runs, three kernels where one would do."""
        dtype = self.qkv.weight.dtype
        if not self.plain:
            return []
        has_rotation = self.position.rot_dim > 0
        if dtype != torch.bfloat16 or ops.attention_decode_fused_fits(dtype, self.spec.head_dim, page_size,
                                                                      self.position.rot_dim, self.position.interleaved,
                                                                      has_rotation):
            return []
        s = self.spec
        return [f"attention with head size {s.head_dim}, page size {page_size}, rotation of {self.position.rot_dim} features "
                f"({'interleaved' if self.position.interleaved else 'halves'}): decode steps do not take the fused kernel "
                "(head sizes in steps of 64, page sizes in steps of 16, whole heads rotated in halves); norm and "
                "rotation, the cache write and the attention run as kernels of their own"]

    def _project(self, ctx, a: torch.Tensor):
        """The output projection: added to the step's stream by the product itself where that can be."""
        if getattr(ctx, "stream", None) is not None:
            norm = getattr(ctx, "stream_norm", None)
            added = ops.linear_add(a, self.o.weight, ctx.stream, norm, self.o.bias)
            if added is not None:
                return ops.Added(added[0], added[1], norm)
        if getattr(ctx, "partial_sums", False):
            split = ops.linear_partials(a, self.o.weight, self.o.bias)
            if split is not None:
                return split
        return self.o(a)

    def forward(self, ctx, h, cache):
        if not self.plain:
            return self._forward_general(ctx, h, cache)
        s = self.spec
        group = ctx.groups[cache.group]
        qkv = self.qkv(h)
        table = ctx.position_table(self.position)
        cos, sin = table if table is not None else (None, None)
        if ctx.max_q_len == 1 and ops.attention_decode_fused_fits(qkv.dtype, s.head_dim, group.page_size,
                                                                   self.position.rot_dim, self.position.interleaved,
                                                                   cos is not None):
            # decode steps: norm, rotation, cache write and attention in one kernel
            a = ops.attention_decode_fused(
                qkv, cache.k, cache.v, ctx.positions, ctx.cu_tokens, group.block_table, nq=s.n_heads,
                nkv=s.n_kv_heads, d=s.head_dim, slots=group.slots if cache.writable else None,
                q_norm_w=self.q_norm_w, k_norm_w=self.k_norm_w, eps=self.norm_eps, add_one=self.norm_add_one,
                cos=cos, sin=sin, max_kv_len=ctx.max_kv_len, window=s.window, scale=s.softmax_scale, sink=s.sink)
            return self._project(ctx, a.view(a.shape[0], s.n_heads * s.head_dim))
        q = ops.qk_rope_kv(
            qkv, s.n_heads, s.n_kv_heads, s.head_dim,
            q_norm_w=self.q_norm_w, k_norm_w=self.k_norm_w, eps=self.norm_eps, add_one=self.norm_add_one,
            cos=cos, sin=sin, rot=self.position.rot_dim, interleaved=self.position.interleaved,
            k_cache=cache.k, v_cache=cache.v, slots=group.slots if cache.writable else None,
            page_size=group.page_size)
        if ops.attention_mfma_fits(q.dtype, s.head_dim, group.page_size):
            common = dict(window=s.window, scale=s.softmax_scale, sink=s.sink)
            if 0 < ctx.n_single < ctx.n_seqs:
                # single tokens (decode) and portions of prompts want different launches: the first
                # split their long key ranges between waves, the second have columns enough
                a = ops.attention_mfma(q, cache.k, cache.v, ctx.positions, ctx.cu_tokens, group.block_table,
                                       max_q_len=1, max_kv_len=ctx.max_kv_single, seqs=(0, ctx.n_single),
                                       tokens=(0, ctx.n_single), **common)
                ops.attention_mfma(q, cache.k, cache.v, ctx.positions, ctx.cu_tokens, group.block_table,
                                   max_q_len=ctx.max_q_len, max_kv_len=ctx.max_kv_multi,
                                   seqs=(ctx.n_single, ctx.n_seqs - ctx.n_single),
                                   tokens=(ctx.n_single, ctx.n_tokens - ctx.n_single), out=a, **common)
            else:
                a = ops.attention_mfma(q, cache.k, cache.v, ctx.positions, ctx.cu_tokens, group.block_table,
                                       max_q_len=ctx.max_q_len, max_kv_len=ctx.max_kv_len, **common)
        else:
            a = ops.attention_generic(q, cache.k, cache.v, ctx.positions, ctx.token_seq, group.block_table,
                                      window=s.window, scale=s.softmax_scale, max_kv_len=ctx.max_kv_len, sink=s.sink)
        return self._project(ctx, a.view(a.shape[0], s.n_heads * s.head_dim))
