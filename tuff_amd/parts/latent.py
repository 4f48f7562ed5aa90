"""Latent attention mixer over the paged cache.

Keys and values are expansions of one narrow row a token: with h the mixer's input,
    [c_raw | k_r] = W_dkv h,   c = rmsnorm(c_raw) * w   (rank channels),   k_r rotated (rot channels, shared by all heads)
    head a:  key = [W_uk,a c | k_r],  value = W_uv,a c,  query = [q_plain,a | rotate(q_rot,a)] from W_q h
    score = (query . key) * scale, causal softmax, head output times sigmoid((W_g h)_a) (where there is a gate), W_o.
The cache keeps [c | k_r] and nothing else: rank + rot numbers a token, one "kv head" for all query
heads, the row's first `rank` channels serving as the value.  Where a row is narrow enough for the
matrix-core attention kernels (a multiple of 8, at most 256 channels) the rows are kept a second time with
a channel's positions contiguous within the page, which is how those kernels read values; wider rows are
kept once and go through the general kernel.  The expansions are never formed for the
cached tokens: the query is carried into the latent space, q' = [W_uk,a^T q_plain,a | q_rot,a], attention
runs over the cache rows as they lie, and W_uv,a is applied to the head's weighted sum of rows.
Both per-head products (ops.head_matmul) run on the matrix cores in bfloat16 where head sizes, rank and the projected
row are multiples of 8 (the weights are then also kept with a column's entries together), else in a scalar kernel.

Options: a sink per head (a name 'sink': a learned logit whose exponential counts once, unscaled, in the softmax's
denominator, with neither key nor value); no rotated part at all (rot_dim 0); a mixer without 'dkv' among its names
has no latent rows of its own: it reads the rows an earlier layer's mixer keeps (the model runs it on that layer's
cache entry, read only) with its own W_uk and W_uv, queries and everything else; exact_weights: the softmax weights
stay float32 where they meet the cached rows.

Rotation: neighbouring pairs (2i, 2i + 1) of the first `rot_dims` channels of the rotated part turn by
position * base^(-2i / rot_dims); the rest passes.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..csrc import ops
from .attention import PagedAttention
from .base import MIXERS, Mixer, PagedKV, Runtime, WeightDecl
from .linear import Linear


@MIXERS.register("latent_attention")
class LatentAttentionMixer(Mixer, PagedAttention):
    graph_safe = True
    records_portions = True
    accepts_pending_norm = True
    adds_once_through_linear = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, rank: int, *,
                 names: dict[str, str], norm_eps: float, scale: float, rot_base: float = 1.0, rot_dims: Optional[int] = None,
                 window: Optional[int] = None, exact_weights: bool = False):
        """names: checkpoint names of 'q' [H (dim + rot), d], 'dkv' [rank + rot, d], 'dkv.norm' [rank],
        'uk' [H dim, rank], 'uv' [H vdim, rank], 'o' [d, H vdim] and, for gated heads, 'g' [H, d]; with 'sink' [H]
        the heads have sinks.  Without 'dkv' (and 'dkv.norm') the mixer keeps no rows: it reads another run's entry.
        rot_dims: how many of the rot channels turn (default: all).
        exact_weights: the softmax weights keep float32's precision where they meet the cached rows, also with
        bfloat16 activations (the kernels that round them to bfloat16 for the matrix cores are not used)."""
        self.exact_weights = bool(exact_weights)
        self.d, self.H, self.dk, self.dr = int(hidden_size), int(num_heads), int(head_dim), int(rot_dim)
        self.dv, self.rank = int(value_dim), int(rank)
        self.lat = self.rank + self.dr
        self.rot_dims = self.dr if rot_dims is None else int(rot_dims)
        if self.rot_dims % 2 or not 0 <= self.rot_dims <= self.dr:
            raise ValueError(f"{self.rot_dims} rotated channels of {self.dr}: an even number within the rotated part is needed")
        if self.lat > ops.ATTN_GENERAL_MAX_DIM:
            raise ValueError(f"a latent row of {self.lat} channels is wider than the attention kernels take "
                             f"({ops.ATTN_GENERAL_MAX_DIM})")
        if max(self.dk, self.rank) > ops.HEAD_MATMUL_MAX_K:
            raise ValueError(f"head size {self.dk} / rank {self.rank} above {ops.HEAD_MATMUL_MAX_K}")
        self.eps, self.scale, self.rot_base = float(norm_eps), float(scale), float(rot_base)
        self.window = int(window) if window else None
        # what PagedAttention reads: every query head against the one row a position
        self.twice = self.lat % 8 == 0 and self.lat <= 256        # rows also kept the matrix cores' way
        self.Hkv, self.hd, self.vd = 1, self.lat, (self.lat if self.twice else self.rank)
        self.sinks = self.slopes = None
        self.names = dict(names)
        self.gated = "g" in self.names
        self.has_sink = "sink" in self.names
        self.own_rows = "dkv" in self.names
        if not self.own_rows and self.dr:
            raise ValueError("a latent mixer that reads another's rows has no rotated part (the shared key part is the writer's)")
        ins = [names["q"]] + ([names["dkv"]] if self.own_rows else []) + ([names["g"]] if self.gated else [])
        outs = [self.H * (self.dk + self.dr)] + ([self.lat] if self.own_rows else []) + ([self.H] if self.gated else [])
        self.proj = Linear(ins, self.d, outs)                       # one product: queries, latent, gates
        self.out = Linear(names["o"], self.H * self.dv, self.d)

    def weight_decls(self):
        n = self.names
        decls = self.proj.weight_decls() + self.out.weight_decls()
        if self.own_rows:
            decls.append(WeightDecl(n["dkv.norm"], (self.rank,), "norm"))
        decls += [WeightDecl(n["uk"], (self.H * self.dk, self.rank), "normal", role="projection"),
                  WeightDecl(n["uv"], (self.H * self.dv, self.rank), "normal", role="projection")]
        if self.has_sink:
            decls.append(WeightDecl(n["sink"], (self.H,), "normal"))
        return decls

    def kernel_modules(self):
        return ["latent", "attention"] + (["attention_mfma", "attention_prefill"] if self.twice else [])

    def cache_spec(self):
        if self.twice:
            return PagedKV(1, self.lat, self.window)
        return PagedKV(1, self.lat, self.window, value_dim=self.rank, values_in_keys=True)

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        self.proj.bind(weights, rt)
        self.out.bind(weights, rt)
        n = self.names
        self.norm_w = weights[n["dkv.norm"]] if self.own_rows else None
        if self.has_sink:
            self.sinks = weights[n["sink"]].float().contiguous()
        dt = rt.dtype
        # W_uk as stored is [H][dim][rank]: k runs over dim, n over rank.  W_uv [H][vdim][rank] is turned per head
        # to [H][rank][vdim], so that both per-head products read a weight row a step of the inner index.
        self.w_uk = weights[n["uk"]].to(dt).reshape(self.H, self.dk, self.rank).contiguous()
        self.w_uv = weights[n["uv"]].to(dt).reshape(self.H, self.dv, self.rank).transpose(1, 2).contiguous()
        # the matrix-core form of those products reads a column's weights together: [H][rank][dim] and [H][vdim][rank]
        self.w_uk_nk = self.w_uv_nk = None
        if ops.head_matmul_mfma_supported(dt, self.dk, self.proj.out_features, 0, self.dk + self.dr):
            self.w_uk_nk = self.w_uk.transpose(1, 2).contiguous()
        if ops.head_matmul_mfma_supported(dt, self.rank, self.H * self.vd, 0, self.vd):
            self.w_uv_nk = weights[n["uv"]].to(dt).reshape(self.H, self.dv, self.rank).contiguous()
        half = self.rot_dims // 2
        self.inv_freq = torch.tensor([self.rot_base ** (-2.0 * i / self.rot_dims) for i in range(half)],
                                     dtype=torch.float64).to(torch.float32).to(rt.device)

    def forward(self, h, ctx, cache, residual, write_cache: bool = True, next_norm=None) -> None:
        T = h.shape[0]
        H, dk, dr, dv, rank, lat = self.H, self.dk, self.dr, self.dv, self.rank, self.lat
        if write_cache and not self.own_rows:
            raise ValueError("a latent mixer without rows of its own runs on another run's cache entry, read only")
        proj = self.proj.forward(h)                                           # [T, H (dk + dr) + lat + H]
        q_width = H * (dk + dr)
        gate_col = q_width + (lat if self.own_rows else 0)
        q_lat = self.rt.empty(T, H * lat)
        o_lat = self.rt.empty(T, H * self.vd)         # (with the rows kept twice a head's sum is a whole row: its rotated part is not used)
        o = self.rt.empty(T, H * dv)
        # the queries' plain parts into the latent space: q'[t, a, :rank] = W_uk,a^T q_plain[t, a]
        ops.head_matmul(proj, self.w_uk, q_lat, H=H, x_head=dk + dr, y_head=lat, w_nk=self.w_uk_nk)

        def over_the_cache(ctx):
            g = ctx.groups[cache.group]
            if self.own_rows:                 # (a reader of another's rows has no rotated part: its queries are complete)
                ops.latent_post(proj, q_lat, cache.k, q_off=0, ckr_off=q_width, norm_w=self.norm_w, eps=self.eps,
                                inv_freq=self.inv_freq, rot_dims=self.rot_dims, positions=ctx.positions,
                                slot_mapping=g.slot_mapping if write_cache else None, H=H, dim=dk, rot=dr, rank=rank,
                                cache_t=cache.v if write_cache else None)
            self.attend(q_lat, o_lat, ctx, cache, g)

        ctx.run_eagerly(over_the_cache)
        # a head's value expansion of its weighted sum of latent rows, times its gate
        ops.head_matmul(o_lat, self.w_uv, o, H=H, x_head=self.vd, y_head=dv,
                        gate=proj if self.gated else None, gate_col=gate_col, w_nk=self.w_uv_nk)
        self.out.forward(o, accumulate_into=residual, next_norm=next_norm)
