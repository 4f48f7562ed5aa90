"""Grouped-query attention mixer over the paged cache.

q = W_q h, k = W_k h, v = W_v h; optional per-head RMSNorm of q and k with a shared [hd]
weight; optional position encoding; k (normed, encoded) and v (as projected) go to the cache
at the token's slot; every token attends to the cached keys of its request up to its own
position (within `window` if given); query head i reads kv head i // (H / Hkv); scores are
scaled by 1/sqrt(hd); o = W_o concat(heads).  Options: a per-head norm of q and k without a
weight (unit root mean square), and a distance penalty slope_h * (i - j) taken off the scaled
score of query i and key j, slope_h = 2^(-span (h + 1) / H).  Further options: biases on q, k, v; a
logarithmic distance penalty r1_h ln(1 + r2_h (i - j)) with learned r1, r2 per head; the heads' softmax
weights mixed by a learned [H, H] matrix, p'_h = sum_g talk[h, g] p_g, head h applying p'_h to the values of
its own kv head; a short causal convolution per channel on q, k and v right after the projection (its last
taps - 1 inputs are state of the request); a gate per head, sigmoid(W_g h)_h, on the head's output.
Reference: src/lfm25_engine.c:386-405, src/lfm25_gpu.cu:420-485, :506-558.
"""
from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch

from ..csrc import ops
from .base import MIXERS, FixedState, Mixer, PagedKV, PositionEncoding, Runtime, WeightDecl
from .linear import Linear


class PagedAttention:
    """Which attention kernels run over a paged cache, and their launch: shared by the mixers whose attention is
    softmax(q . k * scale [- slope (i - j)]) over a request's cached positions (all of them or a window), with
    grouped heads and optional sinks.  It reads the mixer's H, Hkv, hd, vd, window, scale, sinks, slopes and, where
    the mixer has them, log_distance ((r1, r2): the penalty r1_h ln(1 + r2_h (i - j))) and talk (a matrix that mixes
    the heads' softmax weights: o is then float32 [T, H * Hkv * vd], every head's weights on every kv head's values,
    from which ops.head_mix_gate forms the mixed heads)."""

    @staticmethod
    def _upload(array, device):
        """Through pinned memory, so that the host does not wait for the stream."""
        return torch.from_numpy(array).pin_memory().to(device, non_blocking=True)

    @classmethod
    def _blocks(cls, ctx, G, nb, device, skip_single: bool = False, longest_first: bool = False):
        key = ("query_blocks", G, nb, skip_single, longest_first)
        blocks = ctx.host.get(key)
        if blocks is None:
            q_len = ctx.host["q_len"]
            if skip_single:
                q_len = np.where(q_len == 1, 0, q_len)
            ctx_len = ctx.host["ctx_len"] if longest_first else None
            blocks = ctx.host[key] = cls._upload(ops.query_blocks(q_len, G, nb, ctx_len), device)
        return blocks

    @classmethod
    def _single_token_runs(cls, ctx, G, device):
        """Runs of neighbouring requests with one token each in a step that also holds portions:
        [(first token, tokens, block list, request records relative to the first token, longest
        context)], made once a step.  Only where a request's heads fit one block of 16 columns."""
        key = ("single_token_runs", G)
        runs = ctx.host.get(key)
        if runs is None:
            runs = []
            q_len, ctx_len = ctx.host["q_len"], ctx.host["ctx_len"]
            if G <= 16 and (q_len == 1).any():
                start = np.concatenate([[0], np.cumsum(q_len)[:-1]])
                single = np.concatenate([[False], q_len == 1, [False]])
                edges = np.flatnonzero(single[1:] != single[:-1])          # run r_lo .. r_hi - 1 for every pair
                for r_lo, r_hi in zip(edges[0::2], edges[1::2]):
                    tok_lo = int(start[r_lo])
                    info = np.stack([start - tok_lo, q_len, ctx_len - q_len, ctx_len], axis=1).astype(np.int32)
                    blocks = np.stack([np.arange(r_lo, r_hi), np.zeros(r_hi - r_lo, dtype=np.int64)], axis=1).astype(np.int32)
                    runs.append((tok_lo, int(r_hi - r_lo), cls._upload(blocks, device), cls._upload(info, device),
                                 int(ctx_len[r_lo:r_hi].max())))
            ctx.host[key] = runs
        return runs

    def _single_tokens_exact(self, dtype, ctx, page_size) -> bool:
        """A step of single tokens whose weights stay float32: the kernels that read a request's keys and values once
        for all heads, and mix and gate the heads themselves."""
        special = (getattr(self, "log_distance", None) is not None or getattr(self, "talk", None) is not None
                   or getattr(self, "exact_weights", False))
        return (special and ctx.max_q_len == 1
                and ops.attention_decode_exact_supported(dtype, self.H, self.hd, self.vd, page_size))

    def attend(self, q, o, ctx, cache, g, gates=None) -> None:
        G = self.H // self.Hkv
        log_distance, talk = getattr(self, "log_distance", None), getattr(self, "talk", None)
        exact = getattr(self, "exact_weights", False)
        if self._single_tokens_exact(q.dtype, ctx, cache.page_size):
            ops.attention_decode_exact(q, cache.k, cache.v, o, block_table=g.block_table, req_of_token=ctx.req_of_token,
                                       positions=ctx.positions, H=self.H, Hkv=self.Hkv, hd=self.hd, vd=self.vd,
                                       page_size=cache.page_size, max_ctx_len=ctx.max_ctx_len, window=self.window or 0,
                                       scale=self.scale, sinks=self.sinks, slopes=self.slopes, log_distance=log_distance,
                                       talk=talk, gates=gates)
            return
        if ((log_distance is not None or talk is not None or exact) and ctx.max_q_len > 1
                and ops.attention_prefill_wide_supported(q.dtype, self.hd, self.vd, cache.page_size)):
            # prompt portions in the step: the matrix-core kernel in its wide form (single tokens beside them are blocks
            # of one token's heads)
            nb = ops.attention_prefill_block_columns(max(self.hd, self.vd)) // 16
            ops.attention_prefill_wide(q, cache.k, cache.v, o, block_table=g.block_table,
                                       blocks=self._blocks(ctx, G, nb, q.device, longest_first=True), req_info=ctx.req_info,
                                       H=self.H, Hkv=self.Hkv, hd=self.hd, vd=self.vd, page_size=cache.page_size,
                                       max_ctx_len=ctx.max_ctx_len, window=self.window or 0, scale=self.scale, sinks=self.sinks,
                                       slopes=self.slopes, log_distance=log_distance, all_values=talk is not None)
            return
        if log_distance is not None or talk is not None or exact:
            ops.attention_general(q, cache.k, cache.v, o, block_table=g.block_table,
                                  req_of_token=ctx.req_of_token, positions=ctx.positions,
                                  H=self.H, Hkv=self.Hkv, hd=self.hd, page_size=cache.page_size,
                                  window=self.window or 0, scale=self.scale, vd=self.vd, sinks=self.sinks, slopes=self.slopes,
                                  log_distance=log_distance, all_values=talk is not None)
            return
        if self.vd == self.hd and ops.attention_mfma_supported(q.dtype, self.hd, cache.page_size):
            common = dict(block_table=g.block_table, req_info=ctx.req_info, H=self.H, Hkv=self.Hkv, hd=self.hd,
                          page_size=cache.page_size, max_ctx_len=ctx.max_ctx_len, window=self.window or 0,
                          scale=self.scale, sinks=self.sinks, slopes=self.slopes)
            if ctx.max_q_len > 1:
                # prompt portions in the step: blocks of columns walk over their keys through LDS.
                # Requests with a single token beside them (runs of neighbours in the step's order) go
                # the way of a step of single tokens: one workgroup walking all keys of such a request
                # would be the longest of the step.
                nb = ops.attention_prefill_block_columns(self.hd) // 16
                runs = self._single_token_runs(ctx, G, q.device)
                # (first: with key segments it writes every row of o, the single tokens' rows come after)
                ops.attention_prefill(q, cache.k, cache.v, o, blocks=self._blocks(ctx, G, nb, q.device, skip_single=bool(runs), longest_first=True),
                                      positions=ctx.positions, **common)
                for tok_lo, n, blocks, info, ctx_len in runs:
                    ops.attention_mfma(q[tok_lo:tok_lo + n], cache.k, cache.v, o[tok_lo:tok_lo + n], blocks=blocks, nb=1,
                                       positions=ctx.positions[tok_lo:tok_lo + n], **dict(common, req_info=info, max_ctx_len=ctx_len))
                return
            # single tokens: the keys of a request are split over many waves, then merged
            # (heads wider than 128 channels: one column block a wave, which leaves registers to load a step's keys ahead)
            nb = 1 if G <= 16 or self.hd > 128 else (2 if G <= 32 else 4)
            blocks = self._blocks(ctx, G, nb, q.device) if G > 16 * nb else None
            ops.attention_mfma(q, cache.k, cache.v, o, blocks=blocks, nb=nb, positions=ctx.positions, **common)
            return
        ops.attention_general(q, cache.k, cache.v, o, block_table=g.block_table,
                              req_of_token=ctx.req_of_token, positions=ctx.positions,
                              H=self.H, Hkv=self.Hkv, hd=self.hd, page_size=cache.page_size,
                              window=self.window or 0, scale=self.scale, vd=self.vd, sinks=self.sinks, slopes=self.slopes)


@MIXERS.register("attention")
class AttentionMixer(Mixer, PagedAttention):
    accepts_pending_norm = True
    adds_once_through_linear = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, *,
                 names: dict[str, str], qk_norm_eps: Optional[float] = None,
                 position: Optional[PositionEncoding] = None, window: Optional[int] = None,
                 scale: Optional[float] = None, aliases: Optional[dict[str, tuple]] = None,
                 value_dim: Optional[int] = None, slope_span: Optional[float] = None, conv_taps: Optional[int] = None,
                 exact_weights: bool = False):
        """names: checkpoint names of 'q', 'k', 'v', 'o' and, with qk_norm_eps, 'q_norm', 'k_norm' (without these
        two names the norm has no weight: q and k are divided by their root mean square over the head); with a
        'sink' among them the heads have sinks.  value_dim: width of a value head (default: head_dim).
        slope_span: heads have distance slopes 2^(-slope_span (h + 1) / H) (None: none).
        Further names switch further options on: 'q.b', 'k.b', 'v.b' biases of the projections; 'r1', 'r2' [H] the
        logarithmic distance penalty; 'talk' [H, H] the matrix that mixes the heads' softmax weights; 'g' [H, d] the
        gate per head; with conv_taps, 'q.conv', 'k.conv', 'v.conv' [channels, taps] the convolutions' taps (one tap: a
        factor per channel and no state).
        exact_weights: the softmax weights keep float32's precision where they meet the values, also with bfloat16
        activations (the kernels that round them to bfloat16 for the matrix cores are not used)."""
        self.exact_weights = bool(exact_weights)
        if num_heads % num_kv_heads:
            raise ValueError(f"heads {num_heads} must be a multiple of kv heads {num_kv_heads}")
        if head_dim > 256:
            raise ValueError(f"head size {head_dim} above 256 is not supported by the attention kernels")
        self.d, self.H, self.Hkv, self.hd = int(hidden_size), int(num_heads), int(num_kv_heads), int(head_dim)
        self.vd = self.hd if value_dim is None else int(value_dim)
        if self.vd > 256 or self.vd < 1:
            raise ValueError(f"value size {self.vd} is outside 1..256")
        if self.vd != self.hd and position is not None and position.rotary_tables() is None:
            raise ValueError("values of another width than keys go with a rotary encoding or none")
        self.has_sink = "sink" in names
        self.norm_has_weight = qk_norm_eps is not None and "q_norm" in names
        self.slope_span = None if slope_span is None else float(slope_span)
        self.slopes = None
        self.sinks = None
        self.eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.position, self.window = position, (int(window) if window else None)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.hd)
        self.names = dict(names)
        al = aliases or {}
        self.has_bias = "q.b" in names
        self.has_log_distance, self.has_talk = "r1" in names, "talk" in names
        self.K = 0 if conv_taps is None else int(conv_taps)              # 0: no convolution
        if conv_taps is not None and not 1 <= self.K <= ops.CONV_ACT_MAX_TAPS:
            raise ValueError(f"{self.K} convolution taps are outside 1..{ops.CONV_ACT_MAX_TAPS}")
        self.C = (self.H + self.Hkv) * self.hd + self.Hkv * self.vd            # channels of a token's q, k, v
        self.log_distance = self.talk = self.taps = None
        self.qkv = Linear([names["q"], names["k"], names["v"]], self.d,
                          [self.H * self.hd, self.Hkv * self.hd, self.Hkv * self.vd],
                          aliases=[al.get("q", ()), al.get("k", ()), al.get("v", ())],
                          bias=[names["q.b"], names["k.b"], names["v.b"]] if self.has_bias else None)
        self.gate = Linear(names["g"], self.d, self.H) if "g" in names else None
        self.out = Linear(names["o"], self.H * self.vd, self.d, aliases=[al.get("o", ())])
        self._al = al
        self.q_norm_w = self.k_norm_w = None

    @property
    def graph_safe(self):
        return self.position is None or self.position.graph_safe

    @property
    def records_portions(self):
        return self.graph_safe

    def weight_decls(self):
        decls = self.qkv.weight_decls() + self.out.weight_decls()
        if self.norm_has_weight:
            decls += [WeightDecl(self.names["q_norm"], (self.hd,), "norm", aliases=self._al.get("q_norm", ())),
                      WeightDecl(self.names["k_norm"], (self.hd,), "norm", aliases=self._al.get("k_norm", ()))]
        if self.position is not None:
            decls += self.position.weight_decls()
        if self.has_sink:
            decls.append(WeightDecl(self.names["sink"], (self.H,), "normal", aliases=self._al.get("sink", ())))
        if self.has_log_distance:
            decls += [WeightDecl(self.names["r1"], (self.H,), "norm"), WeightDecl(self.names["r2"], (self.H,), "norm")]
        if self.has_talk:
            decls.append(WeightDecl(self.names["talk"], (self.H, self.H), "identity"))
        if self.gate is not None:
            decls += self.gate.weight_decls()
        if self.K >= 1:
            decls += [WeightDecl(self.names[k + ".conv"], (n, self.K), "normal")
                      for k, n in (("q", self.H * self.hd), ("k", self.Hkv * self.hd), ("v", self.Hkv * self.vd))]
        return decls

    def kernel_modules(self):
        mods = ["rope_kv", "attention", "attention_mfma", "attention_prefill"]
        if self.K >= 1:
            mods.append("recurrent")
        if self.position is not None:
            mods += self.position.kernel_modules()
        return mods

    def token_inputs(self):
        return self.position.token_inputs() if self.position is not None else []

    def cache_spec(self):
        kv = PagedKV(self.Hkv, self.hd, self.window, value_dim=None if self.vd == self.hd else self.vd)
        # with a convolution: its last taps - 1 inputs, then the keys and values
        return (FixedState((self.K - 1, self.C)), kv) if self.K > 1 else kv

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        self.qkv.bind(weights, rt)
        self.out.bind(weights, rt)
        if self.norm_has_weight:
            self.q_norm_w = weights[self.names["q_norm"]]
            self.k_norm_w = weights[self.names["k_norm"]]
            if self.q_norm_w.dtype != self.k_norm_w.dtype:
                self.q_norm_w = self.q_norm_w.float()
                self.k_norm_w = self.k_norm_w.float()
        elif self.eps is not None:
            self.q_norm_w = self.k_norm_w = torch.ones(self.hd, dtype=torch.float32, device=rt.device)
        if self.slope_span is not None:
            # in float64, then rounded once
            self.slopes = torch.tensor([2.0 ** (-self.slope_span * (h + 1) / self.H) for h in range(self.H)],
                                       dtype=torch.float64).to(torch.float32).to(rt.device)
        if self.position is not None:
            self.position.bind(weights, rt)
        if self.has_sink:
            self.sinks = weights[self.names["sink"]].float().contiguous()
        f32 = lambda name: weights[self.names[name]].float().contiguous()
        if self.has_log_distance:
            self.log_distance = (f32("r1"), f32("r2"))
        if self.has_talk:
            self.talk = f32("talk")
        if self.gate is not None:
            self.gate.bind(weights, rt)
        if self.K >= 1:
            self.taps = torch.cat([f32("q.conv"), f32("k.conv"), f32("v.conv")]).contiguous()      # [C, K]

    def forward(self, h, ctx, cache, residual, write_cache: bool = True, next_norm=None) -> None:
        T = h.shape[0]
        H, Hkv, hd, vd = self.H, self.Hkv, self.hd, self.vd
        qkv = self.qkv.forward(h)
        # the gate's activation reads the product's float32 sums
        gates = self.gate.forward(h, out_dtype=torch.float32) if self.gate is not None else None
        if self.K >= 1:
            if not write_cache and self.K > 1:
                raise ValueError("a convolution's state has one owner: it cannot be read by another run")
            tail = None
            if self.K > 1:
                tail, cache = cache
            x, qkv = qkv, self.rt.empty(T, self.C)
            ops.conv_act(x, self.taps, None if tail is None else tail.state, qkv, req_of_token=ctx.req_of_token, q_start=ctx.q_start,
                         state_slot=ctx.state_slot, q_len=ctx.q_len, activation=None)
        q = self.rt.empty(T, H * hd) if vd == hd else None
        # (with mixed heads: every head's weights on every kv head's values, float32, for the kernel that mixes them)
        # (single tokens with float32 weights: the attention kernels mix and gate the heads themselves)
        finished = self._single_tokens_exact(qkv.dtype, ctx, cache.page_size)
        o = (self.rt.empty(T, H * vd) if self.talk is None or finished
             else torch.empty(T, H * Hkv * vd, dtype=torch.float32, device=qkv.device))
        norm = dict(eps=self.eps or 0.0, q_norm_w=self.q_norm_w, k_norm_w=self.k_norm_w)
        tables = self.position.rotary_tables() if self.position is not None else None
        fused = self.position is None or tables is not None
        # a position encoding of its own: norm, then its apply(), then the cache write
        k = None if fused else self.rt.empty(T, Hkv * hd)

        one_kernel = (fused and tables is not None and ctx.max_q_len == 1 and self.sinks is None and self.talk is None
                      and not self.exact_weights
                      and self.log_distance is None and ops.attention_decode_fused_supported(
            qkv.dtype, H, Hkv, hd, cache.page_size, tables[1], tables[2]))

        def over_the_cache(ctx):
            """What depends on where the step's tokens lie: positions, cache slots, block tables."""
            g = ctx.groups[cache.group]
            if vd != hd:
                # keys and values of different widths: the rows are cut out (normed, where there is a norm) and written
                if self.eps is not None or tables is not None:
                    qq, kk = self.rt.empty(T, H * hd), self.rt.empty(T, Hkv * hd)
                    rot = {} if tables is None else dict(inv_freq=tables[0], rotary_dim=tables[1], interleaved=tables[2])
                    ops.qkv_post(qkv, qq, H=H, Hkv=Hkv, hd=hd, positions=ctx.positions, k_out=kk, wide_rows=True, **norm, **rot)
                else:
                    qq, kk = qkv[:, :H * hd].contiguous(), qkv[:, H * hd:(H + Hkv) * hd].contiguous()
                if write_cache:
                    ops.kv_write(kk, qkv[:, (H + Hkv) * hd:].contiguous(),
                                 cache.k, cache.v, g.slot_mapping, Hkv=Hkv, hd=hd, vd=vd, page_size=cache.page_size)
                self.attend(qq, o, ctx, cache, g, gates)
                return
            if one_kernel:
                # single tokens, heads of 64: norm, rotation, cache write and attention in one kernel
                ops.attention_decode_fused(qkv, cache.k, cache.v, o, block_table=g.block_table, req_info=ctx.req_info,
                                           positions=ctx.positions, inv_freq=tables[0], H=H, Hkv=Hkv,
                                           page_size=cache.page_size, max_ctx_len=ctx.max_ctx_len,
                                           slot_mapping=g.slot_mapping if write_cache else None,
                                           q_norm_w=self.q_norm_w, k_norm_w=self.k_norm_w, eps=self.eps or 0.0,
                                           window=self.window or 0, scale=self.scale,
                                           angles=getattr(self.position, "angle_table", lambda: None)())
                return
            if fused:
                rot = {}
                if tables is not None:
                    rot = dict(inv_freq=tables[0], rotary_dim=tables[1], interleaved=tables[2],
                               angles=getattr(self.position, "angle_table", lambda: None)())
                wr = dict(k_cache=cache.k, v_cache=cache.v, slot_mapping=g.slot_mapping) if write_cache else {}
                ops.qkv_post(qkv, q, H=H, Hkv=Hkv, hd=hd, positions=ctx.positions, page_size=cache.page_size,
                             **norm, **rot, **wr)
            else:
                ops.qkv_post(qkv, q, H=H, Hkv=Hkv, hd=hd, positions=ctx.positions, k_out=k, **norm)
                self.position.apply_step(q, k, ctx)
                if write_cache:
                    v = qkv[:, (H + Hkv) * hd:].contiguous()
                    ops.kv_write(k, v, cache.k, cache.v, g.slot_mapping, Hkv=Hkv, hd=hd, page_size=cache.page_size)
            self.attend(q, o, ctx, cache, g, gates)

        ctx.run_eagerly(over_the_cache)
        heads = o             # (over_the_cache keeps `o` for its replays: the name is not bound anew)
        if not finished and (self.talk is not None or gates is not None):
            heads = self.rt.empty(T, H * vd)
            ops.head_mix_gate(o, heads, H=H, Hkv=Hkv, vd=vd, talk=self.talk, gates=gates)
        self.out.forward(heads, accumulate_into=residual, next_norm=next_norm)
