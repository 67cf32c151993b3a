"""Latent attention: keys and values of all heads are products of one low-rank row a token, so only that
row and one rotated key part shared by the heads are cached.

    q_h = [q_plain,h | q_rot,h] = W_q h;   [down | k_rot] = W_dkv h;   c = rmsnorm(down) * w
    score_h(i, j) = (q_plain,h(i) . W_uk,h c(j) + rot(q_rot,h(i)) . rot(k_rot(j))) * scale,  j <= i
    out = W_o ( concat_h (W_uv,h sum_j p_h(i, j) c(j))  *  sigmoid(W_g h) )

The heads' matrices are moved across the attention: the query becomes [W_uk,h^T q_plain,h | q_rot,h] and the
attention runs over the cached rows [c | k_rot] with ONE key/value head whose values are the key rows themselves,
which is the shape that the paged attention kernels of this package take (a group of `heads` query heads on one
key/value head).  Behind it W_uv,h turns a head's mixed latent row into its value.  The cache holds the row twice, as
the kernels want their operands: as a row among the keys and as a column among the values.

Options of the spec: the queries through a low-rank row of their own (`q_rank`: q = W_uq rmsnorm(W_dq h) * w; W_dq shares the
one product of everything that reads h, a norm of that slice and a second product follow), neighbours paired in the turn (the position's `pairing`), a window, a
learned term a head in the softmax's denominator (`sink`: the attention kernels take one value a query head), and one gate
value a head (`gate_per_head`).
"""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.spec import LatentAttentionSpec, SpecError
from ..weights.loader import TensorSpec
from .base import Mixer, PagedKV, part_class, register_mixer
from .linear import Linear, to_compute


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    graph_safe = True

    @classmethod
    def tensors(cls, spec: LatentAttentionSpec) -> Dict[str, TensorSpec]:
        H, d, r, dv, rank = spec.n_heads, spec.head_dim, spec.rot_dim, spec.v_dim, spec.kv_rank
        t = {"q": TensorSpec((H * (d + r), spec.hidden))}
        if spec.q_rank:
            t = {"dq": TensorSpec((spec.q_rank, spec.hidden)), "dq.norm": TensorSpec((spec.q_rank,), "norm"),
                 "uq": TensorSpec((H * (d + r), spec.q_rank))}
        t.update({
            "dkv": TensorSpec((rank + r, spec.hidden)),
            "dkv.norm": TensorSpec((rank,), "norm"),
            "uk": TensorSpec((H * d, rank)),
            "uv": TensorSpec((H * dv, rank)),
            "o": TensorSpec((spec.hidden, H * dv)),
        })
        if spec.sink:
            t["sink"] = TensorSpec((H,))
        if spec.gate:
            t["g"] = TensorSpec((H * (1 if spec.gate_per_head else dv), spec.hidden))
        return t

    @classmethod
    def cache_need(cls, spec: LatentAttentionSpec):
        return PagedKV(1, spec.kv_rank + spec.rot_dim, spec.window)

    def __init__(self, spec: LatentAttentionSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        D = spec.kv_rank + spec.rot_dim
        if not (1 <= D <= 512):
            raise SpecError(f"latent_attention: kv_rank + rot_dim = {D} is outside 1..512, the range of the attention kernels")
        self.spec = spec
        self.position = part_class("position", spec.position)(spec.position, {}, dtype, device)
        if self.position.rot_dim > spec.rot_dim:
            raise SpecError("latent_attention: the rotation turns at most rot_dim features")
        H, d, dv, rank = spec.n_heads, spec.head_dim, spec.v_dim, spec.kv_rank
        # one product for everything that reads h: [q, or the queries' low-rank row | latent row, key part | gate]
        first = tensors["dq"] if spec.q_rank else tensors["q"]
        self.proj = Linear([first, tensors["dkv"]] + ([tensors["g"]] if spec.gate else []), dtype, device)
        self.q_off = 0
        self.down_off = first.shape[0]
        self.g_off = self.down_off + D
        self.q_up = self.q_norm_w = None
        if spec.q_rank:
            self.q_up = Linear([tensors["uq"]], dtype, device)
            self.q_norm_w = tensors["dq.norm"].to(device=device, dtype=torch.float32).contiguous()
        self.sinks = tensors["sink"].to(device=device, dtype=torch.float32).contiguous() if spec.sink else None
        self.norm_w = tensors["dkv.norm"].to(device=device, dtype=torch.float32).contiguous()
        # W_uk,h^T as [H, rank, d]: the query side of the keys' up-projection; W_uv,h as [H, dv, rank]
        self.uk_t = to_compute(tensors["uk"], dtype, device).view(H, d, rank).transpose(1, 2).contiguous()
        self.uv = to_compute(tensors["uv"], dtype, device).view(H, dv, rank).contiguous()
        self.o = Linear([tensors["o"]], dtype, device)

    def forward(self, ctx, h, cache):
        s = self.spec
        H, d, r, dv, rank = s.n_heads, s.head_dim, s.rot_dim, s.v_dim, s.kv_rank
        D = rank + r
        group = ctx.groups[cache.group]
        proj = self.proj(h)                                      # [n, q (or its low-rank row) | down, k_rot | g]
        q_rows = None                                            # the queries' rows where a product of their own made them
        if self.q_up is not None:
            q_rows = self.q_up(ops.norm_slice(proj, 0, self.q_norm_w, s.norm_eps))
        table = ctx.position_table(self.position)
        cos, sin = table if table is not None else (None, None)
        q = ops.latent_prep(proj, heads=H, dim=d, rot_dim=r, rank=rank, rotated=self.position.rot_dim if cos is not None else 0,
                            interleaved=self.position.interleaved, q_rows=q_rows,
                            q_off=self.q_off, down_off=self.down_off, norm_weight=self.norm_w, eps=s.norm_eps,
                            cos=cos, sin=sin, magnitude=self.position.magnitude, k_cache=cache.k, v_cache=cache.v,
                            slots=group.slots if cache.writable else None, page_size=group.page_size)
        n = q.shape[0]
        # the plain query parts through W_uk^T, into the first `rank` features of every head's query
        ops.head_product(proj if q_rows is None else q_rows, self.uk_t, x_off=self.q_off, x_head=d + r,
                         out=q.view(n, H * D), o_head=D)
        if ops.attention_mfma_fits(q.dtype, D, group.page_size):
            common = dict(window=s.window, scale=s.scale, sinks=self.sinks)
            if 0 < ctx.n_single < ctx.n_seqs:
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
                                      window=s.window, scale=s.scale, max_kv_len=ctx.max_kv_len, sinks=self.sinks)
        # a [n, H, D]: its first `rank` features are the mixed latent rows; through W_uv, times the gate
        joined = ops.head_product(a.view(n, H * D), self.uv, x_head=D,
                                  gate=proj if s.gate else None, g_off=self.g_off, gate_per_head=s.gate_per_head)
        return self.o(joined)
