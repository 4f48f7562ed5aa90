"""Mixers that carry a matrix state per head from token to token instead of a growing cache.

WkvMixer (RWKV-style time mixing).  With h' the token before (zeros before the first), every one of
r, k, v, g, w reads its own blend  x_s = h + (h' - h) * mu_s.  r, k, v = W_r x_r, W_k x_k, W_v x_v in heads
of D channels, the output gate is silu(W_g x_g), and the decay per head and key channel is
w = exp(-exp(W_w2 tanh(W_w1 x_w) + w0)).  Per head, with the state S [D, D] (key channel, value channel):
    o_t = (S + diag(u) k_t v_t^T)^T r_t          (the bonus u counts for the current token only)
    S   <- diag(w_t) S + k_t v_t^T
Each head's o is divided by its root mean square, the heads side by side are multiplied by a weight and
by the gate, and W_o adds the result into the stream.  State per request: h of its last token and S.

GatedDeltaMixer (gated delta rule with a decay per key channel).  q, k = W_q h, W_k h in Hk heads of D
channels, v = W_v h in H heads of Dv; value head i reads q/k head i // (H / Hk).  q, k and v each pass a
short causal convolution per channel (the last tap is the current token's) and silu; q and k are then
unit vectors per head, q also times D^-1/2.  beta = sigmoid(W_b h) per head;
g = exp(-exp(A_log) * softplus(W_a2 (W_a1 h) + dt_bias)) per head and key channel.  Per head:
    S <- diag(g) S;   e = beta (v - S^T k);   S <- S + k e^T;   o = S^T q
(the read sees the current token's write).  Each head's o is divided by its root mean square over Dv,
multiplied by a weight [Dv] shared by the heads and by sigmoid(W_g2 (W_g1 h)); W_o adds the result into the
stream.  State per request: the last taps - 1 inputs of the convolutions and S.

With a name 'a' in place of 'a1', 'a2' the decay is one number per head, g = exp(-exp(A_log) * softplus(W_a h + dt_bias))
with W_a [H, d] and dt_bias [H]; with a name 'g' in place of 'g1', 'g2' the output gate's projection is one matrix
W_g [H*Dv, d]; gate_activation names the gate's function (sigmoid or silu).

Mamba2Mixer (the state-space recurrence of Mamba-2: a scalar decay per head).  One projection gives a token's
[z | x | B | C | dt]: z and x in H heads of P channels, B and C in G groups of N state channels (head h reads group
h // (H / G)), dt one number per head.  x, B and C together pass a short causal convolution per channel with a bias
(the last tap is the current token's) and silu.  dt = softplus(dt + dt_bias); per head, with the state S [N, P]:
    S <- exp(-exp(A_log) dt) S + dt B x^T;   y = S^T C + D x
(the read sees the current token's write).  y, the heads side by side, is multiplied by silu(z), then divided by its
root mean square in `norm_groups` equal parts, each on its own, times a weight; W_o adds the result into the stream.
State per request: the last taps - 1 inputs of the convolution and S.

ForgetGateMixer (a gated linear recurrence whose forget gate also sets what is written, as in HGRN2).
q = silu(W_q h) in H heads of D channels, v = W_v h in H heads of Dv; the forget gate per head and key channel is
f = lower + (1 - lower) sigmoid(W_f h + b) with a learned lower bound `lower` [H*D].  Per head:
    S <- diag(f) S + (1 - f) v^T;   o = S^T q
(there is no key: 1 - f stands in its place; the read sees the current token's write).  Each head's o is normed
over Dv (RMS norm with a weight [Dv] shared by the heads); W_o adds the result into the stream.  State per
request: S.

States, decays, write strengths and unit norms are float32 in every mode; the recurrences run token by
token in one order, so a position's result does not depend on how the sequence was cut into steps.
"""
from __future__ import annotations

import torch

from ..csrc import ops
from .base import MIXERS, FixedState, Mixer, Runtime, WeightDecl
from .linear import Linear


def _pad_rank(weights: dict, first: str, second: str) -> dict:
    """For a pair of projections through a narrow middle (x -> rank -> out) in bfloat16: a rank that is no
    multiple of 8 is filled up with zero rows of the first and zero columns of the second, the same function."""
    a, b = weights[first], weights[second]
    rank = a.shape[0]
    if rank % 8 == 0 or a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
        return weights
    pad = -rank % 8
    weights = dict(weights)
    weights[first] = torch.cat([a, a.new_zeros(pad, a.shape[1])])
    weights[second] = torch.cat([b, b.new_zeros(b.shape[0], pad)], dim=1).contiguous()
    return weights


class _LowRank:
    """y = W2 f(W1 x): two projections through a narrow middle, f the identity or tanh."""

    def __init__(self, names: tuple, d_in: int, rank: int, d_out: int, activation=None):
        self.names, self.d_in, self.rank, self.d_out, self.activation = names, d_in, rank, d_out, activation
        self._make(rank)

    def _make(self, rank: int) -> None:
        self.first = Linear(self.names[0], self.d_in, rank)
        self.second = Linear(self.names[1], rank, self.d_out)

    def weight_decls(self):
        return [WeightDecl(self.names[0], (self.rank, self.d_in), "normal", role="projection"),
                WeightDecl(self.names[1], (self.d_out, self.rank), "normal", role="projection")]

    def bind(self, weights, rt: Runtime) -> None:
        padded = _pad_rank(weights, *self.names)
        if padded is not weights:
            self._make(padded[self.names[0]].shape[0])
        self.first.bind(padded, rt)
        self.second.bind(padded, rt)

    def forward(self, x, out_dtype=None):
        if self.activation is None:
            mid = self.first.forward(x)
        else:
            # the activation reads the product's float32 sums; what the second product takes is rounded once
            raw = self.first.forward(x, out_dtype=torch.float32)
            mid = torch.empty(raw.shape, dtype=self.first.rt.dtype, device=raw.device)
            ops.act_rows(raw, mid, self.activation)
        return self.second.forward(mid, out_dtype=out_dtype)


@MIXERS.register("wkv")
class WkvMixer(Mixer):
    graph_safe = True
    records_portions = True
    adds_once_through_linear = True

    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, eps: float, *, names: dict[str, str]):
        """names: checkpoint names of 'mu.r', 'mu.k', 'mu.v', 'mu.g', 'mu.w' [d]; 'r', 'k', 'v', 'g' [H*D, d];
        'w1' [rank, d], 'w2' [H*D, rank], 'w0' [H*D]; 'u' [H, D]; 'norm' [H*D]; 'o' [d, H*D].  The rank is read
        from names['rank'] (an int)."""
        self.d, self.H, self.D, self.eps = int(hidden_size), int(num_heads), int(head_dim), float(eps)
        if self.D > ops.SCAN_MAX_DIM:
            raise ValueError(f"head size {self.D} above {ops.SCAN_MAX_DIM} is not supported by the recurrence kernels")
        self.names = dict(names)
        self.rank = int(self.names.pop("rank"))
        n, HD = self.names, self.H * self.D
        self.proj = {s: Linear(n[s], self.d, HD) for s in ("r", "k", "v", "g")}
        self.decay = _LowRank((n["w1"], n["w2"]), self.d, self.rank, HD, activation="tanh")
        self.out = Linear(n["o"], HD, self.d)

    def weight_decls(self):
        n, HD = self.names, self.H * self.D
        decls = [WeightDecl(n["mu." + s], (self.d,), "normal") for s in self.MIXES]
        for s in ("r", "k", "v", "g"):
            decls += self.proj[s].weight_decls()
        decls += self.decay.weight_decls()
        decls += [WeightDecl(n["w0"], (HD,), "normal"), WeightDecl(n["u"], (self.H, self.D), "normal"),
                  WeightDecl(n["norm"], (HD,), "norm")]
        return decls + self.out.weight_decls()

    def kernel_modules(self):
        return ["recurrent", "elementwise"]

    def cache_spec(self):
        return (FixedState((self.d,)), FixedState((self.H, self.D, self.D)))

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        n = self.names
        for lin in self.proj.values():
            lin.bind(weights, rt)
        self.decay.bind(weights, rt)
        self.out.bind(weights, rt)
        f32 = lambda name: weights[name].float().contiguous()
        self.mu = torch.stack([f32(n["mu." + s]) for s in self.MIXES]).contiguous()
        self.w0, self.u, self.norm_w = f32(n["w0"]), f32(n["u"]), f32(n["norm"])

    def forward(self, h, ctx, cache, residual, write_cache: bool = True, next_norm=None) -> None:
        if not write_cache:
            raise ValueError("a recurrent state has one owner: it cannot be read by another run")
        prev, S = cache
        T, HD = h.shape[0], self.H * self.D
        step = dict(q_start=ctx.q_start, state_slot=ctx.state_slot)
        mixes = self.rt.empty(len(self.MIXES), T, self.d)
        # (the kernel also leaves the state for the next step: each request's last row)
        ops.shift_mix(h, prev.state, self.mu, mixes, req_of_token=ctx.req_of_token, q_len=ctx.q_len, **step)
        r, k, v = (self.proj[s].forward(mixes[i]) for i, s in enumerate(("r", "k", "v")))
        g = self.proj["g"].forward(mixes[3], out_dtype=torch.float32)          # the gate's activation reads the sums as they are
        lw = self.decay.forward(mixes[4], out_dtype=torch.float32)
        o = torch.empty(T, HD, dtype=torch.float32, device=h.device)
        ops.wkv_scan(r, k, v, lw, self.w0, self.u, S.state, o, q_len=ctx.q_len, H=self.H, D=self.D, **step)
        y = self.rt.empty(T, HD)
        ops.head_norm_gate(o, self.norm_w, g, y, H=self.H, Dv=self.D, eps=self.eps, per_head_weight=True,
                           gate_activation="silu")
        self.out.forward(y, accumulate_into=residual, next_norm=next_norm)


@MIXERS.register("gated_delta")
class GatedDeltaMixer(Mixer):
    graph_safe = True
    records_portions = True
    adds_once_through_linear = True

    def __init__(self, hidden_size: int, num_heads: int, num_qk_heads: int, key_dim: int, value_dim: int,
                 conv_taps: int, eps: float, *, names: dict[str, str], gate_activation: str = "sigmoid"):
        """names: checkpoint names of 'q', 'k' [Hk*D, d], 'v' [H*Dv, d] and their taps 'q.conv', 'k.conv', 'v.conv'
        [channels, taps]; 'b' [H, d]; 'A_log' [H]; 'a1' [rank, d], 'a2' [H*D, rank], 'dt_bias' [H*D]; 'g1' [rank, d],
        'g2' [H*Dv, rank]; 'norm' [Dv]; 'o' [d, H*Dv]; and the ints 'a_rank', 'g_rank'.
        With 'a' [H, d] in place of 'a1', 'a2' (and no 'a_rank'): one decay per head, 'dt_bias' [H].  With 'g' [H*Dv, d]
        in place of 'g1', 'g2' (and no 'g_rank'): the gate's projection in one matrix.  A mixer with both runs q, k, v,
        g, b and a as one product whose float32 sums go on as they are.
        gate_activation: "sigmoid" or "silu", the function of the output gate."""
        if gate_activation not in ("sigmoid", "silu"):
            raise ValueError(f"unknown gate activation '{gate_activation}'")
        self.gate_activation = gate_activation
        self.d, self.H, self.Hk = int(hidden_size), int(num_heads), int(num_qk_heads)
        self.D, self.Dv, self.K, self.eps = int(key_dim), int(value_dim), int(conv_taps), float(eps)
        if self.H % self.Hk:
            raise ValueError(f"heads {self.H} must be a multiple of the q/k heads {self.Hk}")
        if self.D > ops.SCAN_MAX_DIM:
            raise ValueError(f"key size {self.D} above {ops.SCAN_MAX_DIM} is not supported by the recurrence kernels")
        if not 1 <= self.K <= ops.CONV_ACT_MAX_TAPS:
            raise ValueError(f"{self.K} convolution taps are outside 1..{ops.CONV_ACT_MAX_TAPS}")
        self.names = dict(names)
        n = self.names
        self.per_head_decay, self.full_gate = "a" in n, "g" in n
        self.Cq, self.Cv = self.Hk * self.D, self.H * self.Dv
        self.C = 2 * self.Cq + self.Cv
        self.one_product = self.per_head_decay and self.full_gate
        if self.one_product:
            self.qkv = Linear([n["q"], n["k"], n["v"], n["g"], n["b"], n["a"]], self.d,
                              [self.Cq, self.Cq, self.Cv, self.Cv, self.H, self.H])
            self.beta = self.decay = self.gate = None
        else:
            self.qkv = Linear([n["q"], n["k"], n["v"]], self.d, [self.Cq, self.Cq, self.Cv])
            self.beta = Linear(n["b"], self.d, self.H)
            self.decay = (Linear(n["a"], self.d, self.H) if self.per_head_decay
                          else _LowRank((n["a1"], n["a2"]), self.d, int(self.names.pop("a_rank")), self.H * self.D))
            self.gate = (Linear(n["g"], self.d, self.Cv) if self.full_gate
                         else _LowRank((n["g1"], n["g2"]), self.d, int(self.names.pop("g_rank")), self.Cv))
        self.out = Linear(n["o"], self.Cv, self.d)

    def weight_decls(self):
        n = self.names
        decls = self.qkv.weight_decls()
        for part in (self.beta, self.decay, self.gate):
            if part is not None:
                decls += part.weight_decls()
        return (decls
                + [WeightDecl(n["q.conv"], (self.Cq, self.K), "normal"), WeightDecl(n["k.conv"], (self.Cq, self.K), "normal"),
                   WeightDecl(n["v.conv"], (self.Cv, self.K), "normal"), WeightDecl(n["A_log"], (self.H,), "normal"),
                   WeightDecl(n["dt_bias"], (self.H if self.per_head_decay else self.H * self.D,), "normal"),
                   WeightDecl(n["norm"], (self.Dv,), "norm")]
                + self.out.weight_decls())

    def kernel_modules(self):
        return ["recurrent", "elementwise"]

    def cache_spec(self):
        S = FixedState((self.H, self.D, self.Dv))
        return (FixedState((self.K - 1, self.C)), S) if self.K > 1 else (S,)

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        n = self.names
        for part in (self.qkv, self.beta, self.decay, self.gate, self.out):
            if part is not None:
                part.bind(weights, rt)
        f32 = lambda name: weights[name].float().contiguous()
        self.taps = torch.cat([f32(n["q.conv"]), f32(n["k.conv"]), f32(n["v.conv"])]).contiguous()      # [C, K]
        self.A_log, self.dt_bias, self.norm_w = f32(n["A_log"]), f32(n["dt_bias"]), f32(n["norm"])

    def forward(self, h, ctx, cache, residual, write_cache: bool = True, next_norm=None) -> None:
        if not write_cache:
            raise ValueError("a recurrent state has one owner: it cannot be read by another run")
        tail, S = cache if self.K > 1 else (None, cache[0])
        T = h.shape[0]
        step = dict(q_start=ctx.q_start, state_slot=ctx.state_slot)
        if self.one_product:
            # one product; its float32 sums go on unrounded, as column ranges of the same rows
            x, gate, b, a = self.qkv.forward(h, out_dtype=torch.float32).split([self.C, self.Cv, self.H, self.H], dim=1)
        else:
            x = self.qkv.forward(h)
            b = self.beta.forward(h, out_dtype=torch.float32)
            a = self.decay.forward(h, out_dtype=torch.float32)
            gate = self.gate.forward(h, out_dtype=torch.float32)
        qkv = self.rt.empty(T, self.C)
        ops.conv_act(x, self.taps, None if tail is None else tail.state, qkv, req_of_token=ctx.req_of_token,
                     q_len=ctx.q_len, activation="silu", **step)
        q, k, v = qkv.split([self.Cq, self.Cq, self.Cv], dim=1)         # column ranges of the same rows, no copies
        o = torch.empty(T, self.Cv, dtype=torch.float32, device=h.device)
        ops.delta_scan(q, k, v, a, self.dt_bias, self.A_log, b, S.state, o, q_len=ctx.q_len, H=self.H, Hk=self.Hk,
                       D=self.D, Dv=self.Dv, per_head=self.per_head_decay, **step)
        y = self.rt.empty(T, self.Cv)
        ops.head_norm_gate(o, self.norm_w, gate, y, H=self.H, Dv=self.Dv, eps=self.eps, per_head_weight=False,
                           gate_activation=self.gate_activation)
        self.out.forward(y, accumulate_into=residual, next_norm=next_norm)


@MIXERS.register("mamba2")
class Mamba2Mixer(Mixer):
    graph_safe = True
    records_portions = True
    adds_once_through_linear = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, state_dim: int, groups: int, norm_groups: int,
                 conv_taps: int, eps: float, *, names: dict[str, str]):
        """names: checkpoint names of 'in' [2 H P + 2 G N + H, d] (rows z, x, B, C, dt), 'conv' [H P + 2 G N, taps] with
        its bias 'conv.b', 'dt_bias', 'A_log', 'D' [H], 'norm' [H P], 'o' [d, H P]."""
        self.d, self.H, self.P, self.N = int(hidden_size), int(num_heads), int(head_dim), int(state_dim)
        self.G, self.norm_groups, self.K, self.eps = int(groups), int(norm_groups), int(conv_taps), float(eps)
        if self.G < 1 or self.H % self.G:
            raise ValueError(f"heads {self.H} must be a multiple of the groups {self.G}")
        self.inner = self.H * self.P
        if self.norm_groups < 1 or self.inner % self.norm_groups:
            raise ValueError(f"{self.norm_groups} norm groups do not divide {self.inner} channels")
        if self.N > ops.SCAN_MAX_DIM:
            raise ValueError(f"state size {self.N} above {ops.SCAN_MAX_DIM} is not supported by the recurrence kernels")
        if not 1 <= self.K <= ops.CONV_ACT_MAX_TAPS:
            raise ValueError(f"{self.K} convolution taps are outside 1..{ops.CONV_ACT_MAX_TAPS}")
        self.names = dict(names)
        self.C = self.inner + 2 * self.G * self.N                        # channels that pass the convolution
        self.inp = Linear(self.names["in"], self.d, self.inner + self.C + self.H)
        self.out = Linear(self.names["o"], self.inner, self.d)

    def weight_decls(self):
        n = self.names
        return (self.inp.weight_decls()
                + [WeightDecl(n["conv"], (self.C, self.K), "normal"), WeightDecl(n["conv.b"], (self.C,), "normal"),
                   WeightDecl(n["dt_bias"], (self.H,), "normal"), WeightDecl(n["A_log"], (self.H,), "normal"),
                   WeightDecl(n["D"], (self.H,), "norm"), WeightDecl(n["norm"], (self.inner,), "norm")]
                + self.out.weight_decls())

    def kernel_modules(self):
        return ["recurrent", "elementwise"]

    def cache_spec(self):
        S = FixedState((self.H, self.N, self.P))
        return (FixedState((self.K - 1, self.C)), S) if self.K > 1 else (S,)

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        n = self.names
        self.inp.bind(weights, rt)
        self.out.bind(weights, rt)
        f32 = lambda name: weights[n[name]].float().contiguous()
        self.taps, self.conv_b = f32("conv"), f32("conv.b")
        self.dt_bias, self.A_log, self.D_skip, self.norm_w = f32("dt_bias"), f32("A_log"), f32("D"), f32("norm")

    def forward(self, h, ctx, cache, residual, write_cache: bool = True, next_norm=None) -> None:
        if not write_cache:
            raise ValueError("a recurrent state has one owner: it cannot be read by another run")
        tail, S = cache if self.K > 1 else (None, cache[0])
        T = h.shape[0]
        step = dict(q_start=ctx.q_start, state_slot=ctx.state_slot)
        # the product's float32 sums go on unrounded: the gate, the convolution's input and dt are column ranges of its rows
        z, raw, dt = self.inp.forward(h, out_dtype=torch.float32).split([self.inner, self.C, self.H], dim=1)
        xbc = self.rt.empty(T, self.C)
        ops.conv_act(raw, self.taps, None if tail is None else tail.state, xbc, req_of_token=ctx.req_of_token,
                     q_len=ctx.q_len, activation="silu", bias=self.conv_b, **step)
        o = torch.empty(T, self.inner, dtype=torch.float32, device=h.device)
        # a step with prompt portions (of 64 tokens and more in all): the recurrence in chunks on the matrix cores, where
        # its sizes fit; single tokens, short steps and float32 runs: token by token
        chunked = ctx.max_q_len > 1 and T >= ops.SSD_CHUNK and ops.ssd_chunked_supported(xbc.dtype, self.N, self.P)
        (ops.ssd_chunked if chunked else ops.ssd_scan)(xbc, dt, self.dt_bias, self.A_log, self.D_skip, S.state, o, q_len=ctx.q_len,
                                                       H=self.H, G=self.G, N=self.N, P=self.P, **step)
        y = self.rt.empty(T, self.inner)
        ops.head_norm_gate(o, self.norm_w, z, y, H=self.norm_groups, Dv=self.inner // self.norm_groups, eps=self.eps,
                           per_head_weight=True, gate_activation="silu", gate_first=True)
        self.out.forward(y, accumulate_into=residual, next_norm=next_norm)


@MIXERS.register("forget_gate")
class ForgetGateMixer(Mixer):
    graph_safe = True
    records_portions = True
    adds_once_through_linear = True

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, eps: float, *, names: dict[str, str]):
        """names: checkpoint names of 'q', 'f' [H*D, d], 'f.b', 'lower' [H*D], 'v' [H*Dv, d], 'norm' [Dv], 'o' [d, H*Dv]."""
        self.d, self.H, self.D, self.Dv, self.eps = int(hidden_size), int(num_heads), int(key_dim), int(value_dim), float(eps)
        if self.D > ops.SCAN_MAX_DIM:
            raise ValueError(f"key size {self.D} above {ops.SCAN_MAX_DIM} is not supported by the recurrence kernels")
        self.names = dict(names)
        n, HD = self.names, self.H * self.D
        # one product for q, the gate's logits and v; its float32 sums go into the recurrence's kernels as they are
        self.qfv = Linear([n["q"], n["f"], n["v"]], self.d, [HD, HD, self.H * self.Dv])
        self.out = Linear(n["o"], self.H * self.Dv, self.d)

    def weight_decls(self):
        n, HD = self.names, self.H * self.D
        return (self.qfv.weight_decls() + [WeightDecl(n["f.b"], (HD,), "normal"), WeightDecl(n["lower"], (HD,), "around:0.5"),
                                           WeightDecl(n["norm"], (self.Dv,), "norm")] + self.out.weight_decls())

    def kernel_modules(self):
        return ["recurrent", "elementwise"]

    def cache_spec(self):
        return FixedState((self.H, self.D, self.Dv))

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        n = self.names
        self.qfv.bind(weights, rt)
        self.out.bind(weights, rt)
        f32 = lambda name: weights[n[name]].float().contiguous()
        self.f_bias, self.lower, self.norm_w = f32("f.b"), f32("lower"), f32("norm")

    def forward(self, h, ctx, cache, residual, write_cache: bool = True, next_norm=None) -> None:
        if not write_cache:
            raise ValueError("a recurrent state has one owner: it cannot be read by another run")
        T = h.shape[0]
        x = self.qfv.forward(h, out_dtype=torch.float32)
        o = torch.empty(T, self.H * self.Dv, dtype=torch.float32, device=x.device)
        ops.forget_scan(x, self.f_bias, self.lower, cache.state, o, q_start=ctx.q_start, q_len=ctx.q_len,
                        state_slot=ctx.state_slot, H=self.H, D=self.D, Dv=self.Dv)
        y = self.rt.empty(T, self.H * self.Dv)
        ops.head_norm_gate(o, self.norm_w, None, y, H=self.H, Dv=self.Dv, eps=self.eps, per_head_weight=False,
                           gate_activation=None)
        self.out.forward(y, accumulate_into=residual, next_norm=next_norm)
